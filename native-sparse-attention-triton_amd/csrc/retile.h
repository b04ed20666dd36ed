// Fragment-major copies of a varlen [T, H, D] tensor (K or V) for the query-stationary kernels.
//
// A wavefront that feeds MFMA operands straight from global memory wants lane l to fetch the 16
// bytes that lane l holds in the operand.  In a row-major tensor consecutive lanes then touch
// different rows (different cache lines), and the L1 spends one cycle per 16 bytes.  These copies
// store every operand fragment as one contiguous KiB in lane order, so a fragment load is a single
// fully coalesced 1 KiB read (8 cache lines instead of 64 partial ones).
//
// Unit of storage: a "slot" = 32 consecutive keys of one sequence x D columns.  Sequence b starts
// at slot ceil(cu[b]/32) + b, so slots never straddle sequences and no prefix sum is needed
// (at most one slack slot per sequence).  Keys past the end of a sequence are stored as zeros.
//
//   ROWS layout (contraction over D, e.g. S^T = K Q^T, dP^T = V dO^T):
//     [h][slot][sub (2 x 16 keys)][kk (D/32)][lane (64)][8]
//     lane (li, lg) holds key 16*sub + li, columns 32*kk + 8*lg .. +7.
//   COLS layout (contraction over keys, e.g. O^T += V^T P^T):
//     [h][slot][dt (D/16)][lane (64)][8]
//     lane (li, lg) holds column 16*dt + li and the keys {4*lg + r, 16 + 4*lg + r : r < 4} - the
//     order in which a lane holds two 16x16 score tiles, so the score registers feed the next MFMA
//     without a shuffle.
#pragma once
#include "nsa_common.h"

enum { RETILE_ROWS = 0, RETILE_COLS = 1 };

__device__ __forceinline__ int seq_first_slot(const int32_t* __restrict__ cu, int b) { return (cu[b] + 31) / 32 + b; }

template <typename T, int D, int MODE>
__device__ __forceinline__ void retile_body(const T* __restrict__ x, T* __restrict__ out, const int32_t* __restrict__ cu, int batch,
                                            long long stride_n, long long stride_h, int n_slots, T (*tile)[lds_pitch(D)]) {
  const int slot = blockIdx.x, h = blockIdx.y;
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
    const int r = i / PIECES, c = (i % PIECES) * 8;
    uint4 val = {0u, 0u, 0u, 0u};
    if (key0 + r < len) val = *reinterpret_cast<const uint4*>(x + (long long)(s0 + key0 + r) * stride_n + (long long)h * stride_h + c);
    *reinterpret_cast<uint4*>(&tile[r][c]) = val;
  }
  __syncthreads();
  T* dst = out + ((long long)h * n_slots + slot) * 32 * D;
  // 32*D/8 = 4*D output pieces of 16 bytes, written in storage order (coalesced)
  for (int i = threadIdx.x; i < 4 * D; i += 256) {
    const int lane = i & 63, frag = i >> 6, li = lane & 15, lg = lane >> 4;
    if (MODE == RETILE_ROWS) {
      const int kk = frag % (D / 32), sub = frag / (D / 32);
      *reinterpret_cast<uint4*>(dst + (long long)i * 8) = *reinterpret_cast<const uint4*>(&tile[16 * sub + li][32 * kk + 8 * lg]);
    } else {
      const int dt = frag;
      T v[8];
#pragma unroll
      for (int n = 0; n < 2; n++)
#pragma unroll
        for (int r = 0; r < 4; r++) v[4 * n + r] = tile[16 * n + 4 * lg + r][16 * dt + li];
      *reinterpret_cast<uint4*>(dst + (long long)i * 8) = *reinterpret_cast<uint4*>(v);
    }
  }
}

template <typename T, int D, int MODE>
__global__ __launch_bounds__(256) void retile_kernel(const T* __restrict__ x, T* __restrict__ out, const int32_t* __restrict__ cu, int batch,
                                                     long long stride_n, long long stride_h, int n_slots) {
  __shared__ __attribute__((aligned(16))) T tile[32][lds_pitch(D)];
  retile_body<T, D, MODE>(x, out, cu, batch, stride_n, stride_h, n_slots, tile);
}

// two tensors of the same shape (K and V) in one launch: blockIdx.z picks the tensor and its layout
template <typename T, int D, int MODE0, int MODE1>
__global__ __launch_bounds__(256) void retile_pair_kernel(const T* __restrict__ x0, T* __restrict__ out0, long long sn0, long long sh0,
                                                          const T* __restrict__ x1, T* __restrict__ out1, long long sn1, long long sh1,
                                                          const int32_t* __restrict__ cu, int batch, int n_slots) {
  __shared__ __attribute__((aligned(16))) T tile[32][lds_pitch(D)];
  if (blockIdx.z == 0) retile_body<T, D, MODE0>(x0, out0, cu, batch, sn0, sh0, n_slots, tile);
  else retile_body<T, D, MODE1>(x1, out1, cu, batch, sn1, sh1, n_slots, tile);
}

template <typename T, int D, int MODE>
static inline void launch_retile(const T* x, T* out, const int32_t* cu, int64_t batch, int64_t stride_n, int64_t stride_h,
                                 int64_t n_slots, int64_t heads, hipStream_t stream) {
  dim3 grid((unsigned)n_slots, (unsigned)heads);
  retile_kernel<T, D, MODE><<<grid, 256, 0, stream>>>(x, out, cu, (int)batch, stride_n, stride_h, (int)n_slots);
}

template <typename T, int D, int MODE0, int MODE1>
static inline void launch_retile_pair(const T* x0, T* out0, int64_t sn0, int64_t sh0, const T* x1, T* out1, int64_t sn1, int64_t sh1,
                                      const int32_t* cu, int64_t batch, int64_t n_slots, int64_t heads, hipStream_t stream) {
  dim3 grid((unsigned)n_slots, (unsigned)heads, 2);
  retile_pair_kernel<T, D, MODE0, MODE1><<<grid, 256, 0, stream>>>(x0, out0, sn0, sh0, x1, out1, sn1, sh1, cu, (int)batch, (int)n_slots);
}

// bytes of one fragment-major copy
static inline size_t retile_bytes(int64_t total_len, int64_t batch, int64_t heads, int64_t head_dim) {
  return (size_t)heads * (size_t)nsa_chunk_slots(total_len, batch) * 32 * (size_t)head_dim * 2;
}
