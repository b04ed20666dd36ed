// delta[h][t] = sum_d O[t,h,d] * dO[t,h,d]  (fp32, [Hq, T] contiguous): the softmax-backward row term.
#pragma once
#include "nsa_common.h"

// With stat != nullptr the (lse, delta) pair of every row is also stored token-major, stat[t][h][2] (what the dK/dV pass
// over query lists reads).
template <typename T, int D>
__global__ __launch_bounds__(256) void delta_kernel(const T* __restrict__ o, const T* __restrict__ dout, float* __restrict__ delta,
                                                    int total_len, int Hq, long long osn, long long osh, long long dsn, long long dsh,
                                                    const float* __restrict__ lse, float* __restrict__ stat) {
  using v8 = typename Elem<T>::v8;
  constexpr int LPR = D / 8;                       // lanes per row (16-byte pieces)
  constexpr int LPR2 = LPR <= 4 ? 4 : (LPR <= 8 ? 8 : 16);
  const int sub = threadIdx.x % LPR2;
  const long long row = (long long)blockIdx.x * (256 / LPR2) + threadIdx.x / LPR2;
  const bool live = row < (long long)total_len * Hq;
  float acc = 0.f;
  int t = 0, h = 0;
  if (live) {
    t = (int)(row / Hq); h = (int)(row % Hq);
    if (sub < LPR) {
      v8 a = ld16<v8>(o + (long long)t * osn + (long long)h * osh + 8 * sub);
      v8 b = ld16<v8>(dout + (long long)t * dsn + (long long)h * dsh + 8 * sub);
#pragma unroll
      for (int i = 0; i < 8; i++) acc += (float)a[i] * (float)b[i];
    }
  }
#pragma unroll
  for (int s = LPR2 / 2; s > 0; s >>= 1) acc += __shfl_xor(acc, s);
  if (live && sub == 0) {
    delta[(long long)h * total_len + t] = acc;
    if (stat) *reinterpret_cast<float2*>(stat + ((long long)t * Hq + h) * 2) = float2{lse[(long long)h * total_len + t], acc};
  }
}


template <typename T, int D>
static inline void launch_delta(const T* o, const T* dout, float* delta, int64_t total_len, int64_t Hq, long long osn, long long osh,
                                long long dsn, long long dsh, hipStream_t stream, const float* lse = nullptr, float* stat = nullptr) {
  constexpr int LPR = D / 8, LPR2 = LPR <= 4 ? 4 : (LPR <= 8 ? 8 : 16);
  const long long rows = (long long)total_len * Hq;
  delta_kernel<T, D><<<(unsigned)((rows + 256 / LPR2 - 1) / (256 / LPR2)), 256, 0, stream>>>(o, dout, delta, (int)total_len, (int)Hq, osn, osh, dsn, dsh, lse, stat);
}
