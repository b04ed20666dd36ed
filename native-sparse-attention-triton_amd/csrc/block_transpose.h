// Block-transposed copy of a varlen [T, H, D] tensor, used wherever an MFMA contracts over
// the key dimension (P*V in the forward, dS*K in the dQ pass): the matrix cores want the
// contracted index contiguous per lane, while K/V rows are contiguous in head_dim.
//
// Layout of the copy: XT[h][slot][d][32].  A slot is a run of 32 consecutive keys of one
// sequence; sequence b starts at slot ceil(cu[b]/32) + b, so slots never straddle sequences
// and no prefix sum is needed.  Inside a slot the 32 keys are stored in the order the
// 16x16x32 MFMA consumes them after two 16x16 score tiles: position 8*g + 4*n + r holds key
// 16*n + 4*g + r (g in 0..3, n in 0..1, r in 0..3).  Keys past the end of the sequence are
// stored as zeros.
#pragma once
#include "nsa_common.h"

__device__ __forceinline__ int seq_first_slot(const int32_t* __restrict__ cu, int b) { return (cu[b] + 31) / 32 + b; }

template <typename T, int D>
__global__ __launch_bounds__(256) void block_transpose_kernel(const T* __restrict__ x, T* __restrict__ xt,
                                                              const int32_t* __restrict__ cu, int batch,
                                                              long long stride_n, long long stride_h, int n_slots) {
  __shared__ T tile[32][D + 8];
  const int slot = blockIdx.x, h = blockIdx.y;
  // sequence whose slot range contains `slot`
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (seq_first_slot(cu, mid) <= slot) lo = mid; else hi = mid;
  }
  const int b = lo;
  const int s0 = cu[b], len = cu[b + 1] - s0;
  const int key0 = (slot - seq_first_slot(cu, b)) * 32;
  if (key0 >= len) return;  // slack slot between sequences: never read
  constexpr int PIECES = D / 8;
  for (int i = threadIdx.x; i < 32 * PIECES; i += 256) {
    int r = i / PIECES, c = (i % PIECES) * 8;
    uint4 val = {0u, 0u, 0u, 0u};
    if (key0 + r < len) val = *reinterpret_cast<const uint4*>(x + (long long)(s0 + key0 + r) * stride_n + (long long)h * stride_h + c);
    *reinterpret_cast<uint4*>(&tile[r][c]) = val;
  }
  __syncthreads();
  T* dst = xt + ((long long)h * n_slots + slot) * D * 32;
  for (int i = threadIdx.x; i < D * 4; i += 256) {
    int d = i >> 2, g = i & 3;
    T out[8];
#pragma unroll
    for (int n = 0; n < 2; n++)
#pragma unroll
      for (int r = 0; r < 4; r++) out[4 * n + r] = tile[16 * n + 4 * g + r][d];
    *reinterpret_cast<uint4*>(dst + d * 32 + 8 * g) = *reinterpret_cast<uint4*>(out);
  }
}

template <typename T, int D>
static inline void launch_block_transpose(const T* x, T* xt, const int32_t* cu, int64_t batch, int64_t stride_n,
                                          int64_t stride_h, int64_t n_slots, int64_t heads, hipStream_t stream) {
  dim3 grid((unsigned)n_slots, (unsigned)heads);
  block_transpose_kernel<T, D><<<grid, 256, 0, stream>>>(x, xt, cu, (int)batch, stride_n, stride_h, (int)n_slots);
}
