// Shared device/host helpers for the gfx950 NSA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nsa_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define NSA_LOG2E 1.4426950408889634f
// floor of the running score maxima (raw q.k units): finite, so differences of maxima never form inf - inf
#define M_FLOOR (-1e30f)
// how far (in powers of two) a new maximum may exceed the reference maximum before online-softmax
// accumulators are rescaled
#define RESCALE_SLACK 8.f

// Element-type traits: 8-wide register fragments and the 16x16x32 / 32x32x16 MFMA for that type.
// Fragment layout (wave64): A is [16][32] with lane l holding row l%16, k = 8*(l/16)..+7;
// B is [32][16] with lane l holding column l%16, k = 8*(l/16)..+7; the 16x16 result has lane l
// holding column l%16, rows 4*(l/16)..+3.
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  using v8 = bf16x8;
  using v4 = bf16x4;
  static __device__ __forceinline__ f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<_Float16> {
  using v8 = f16x8;
  using v4 = f16x4;
  static __device__ __forceinline__ f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

template <typename V> __device__ __forceinline__ V ld16(const void* p) {
  static_assert(sizeof(V) == 16, "16-byte fragment");
  uint4 r = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(V, r);
}
template <typename V> __device__ __forceinline__ V zero16() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(V, z);
}
// the eight 2-byte floating-point elements of a fragment with their signs flipped
template <typename V> __device__ __forceinline__ V negated16(V v) {
  uint4 r = __builtin_bit_cast(uint4, v);
  r.x ^= 0x80008000u; r.y ^= 0x80008000u; r.z ^= 0x80008000u; r.w ^= 0x80008000u;
  return __builtin_bit_cast(V, r);
}
template <typename V> __device__ __forceinline__ void st16(void* p, V v) {
  *reinterpret_cast<uint4*>(p) = __builtin_bit_cast(uint4, v);
}
template <typename V> __device__ __forceinline__ void st8(void* p, V v) {
  static_assert(sizeof(V) == 8, "8-byte fragment");
  *reinterpret_cast<uint2*>(p) = __builtin_bit_cast(uint2, v);
}

// x rounded to the 2-byte element type T and widened again.  The compiler treats float -> T -> float as
// removable and then contracts the surrounding multiply/add into an FMA; kernels that must reproduce
// element-wise 16-bit tensor arithmetic (every product and sum rounded) pass the 16 bits through an opaque
// register move so that the rounding stays.
template <typename T> __device__ __forceinline__ float rounded(float x) {
  const T t = (T)x;
  unsigned bits = __builtin_bit_cast(unsigned short, t);
  asm volatile("" : "+v"(bits));
  return (float)__builtin_bit_cast(T, (unsigned short)bits);
}

// Row pitch (in 2-byte elements) of LDS tiles whose rows hold D elements.  Measured on gfx950: both the
// 16-byte row-fragment reads (16 lanes on 16 rows, same column) and the transposing 8-byte reads (4
// rows per 16 lanes) run at full rate exactly when the pitch in bytes is an odd multiple of 32; a pitch
// of D + 8 elements halves the rate of the former and costs 40% on the latter.
constexpr int lds_pitch(int d) { return d + 16; }

// Asynchronous copies from global memory straight into LDS (no registers in between): every lane
// supplies its own source address, the 64 lanes of a wave fill 64 consecutive 16-byte (4-byte) pieces
// starting at the wave-uniform LDS address.  Completion is counted by vmcnt like any other load.
typedef __attribute__((address_space(3))) void* nsa_lds_ptr;
__device__ __forceinline__ void dma16(const void* src, unsigned char* lds) { __builtin_amdgcn_global_load_lds(src, (nsa_lds_ptr)lds, 16, 0, 0); }
__device__ __forceinline__ void dma4(const void* src, unsigned char* lds) { __builtin_amdgcn_global_load_lds(src, (nsa_lds_ptr)lds, 4, 0, 0); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Reductions over the four lanes {l, l^16, l^32, l^48} that share one MFMA column, as VALU
// lane swaps (v_permlane32_swap / v_permlane16_swap) instead of LDS-crossbar shuffles. After a
// swap of x with itself the two results hold, for every lane, its own half and the partner's.
// The halves are copied into scalars before the float reinterpretation: reinterpreting a
// vector element in place reads element 0 for every index.
typedef unsigned nsa_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void lane_halves32(float x, float& a, float& b) {
  const unsigned u = __float_as_uint(x);
  const nsa_u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __uint_as_float(r0); b = __uint_as_float(r1);
}
__device__ __forceinline__ void lane_halves16(float x, float& a, float& b) {
  const unsigned u = __float_as_uint(x);
  const nsa_u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __uint_as_float(r0); b = __uint_as_float(r1);
}
__device__ __forceinline__ float column_max(float x) {
  float a, b;
  lane_halves32(x, a, b); x = fmaxf(a, b);
  lane_halves16(x, a, b); return fmaxf(a, b);
}
__device__ __forceinline__ float column_sum(float x) {
  float a, b;
  lane_halves32(x, a, b); x = a + b;
  lane_halves16(x, a, b); return a + b;
}

// Sums over the four lanes of a column for four values at once: on return the lanes of group g (lanes
// 16g..16g+15) hold the column sums of x_g.  Three swaps and three adds instead of four column_sum calls.
__device__ __forceinline__ float column_sum_scatter4(float x0, float x1, float x2, float x3) {
  const nsa_u32x2 p = __builtin_amdgcn_permlane32_swap(__float_as_uint(x0), __float_as_uint(x2), false, false);
  const nsa_u32x2 q = __builtin_amdgcn_permlane32_swap(__float_as_uint(x1), __float_as_uint(x3), false, false);
  const unsigned p0 = p[0], p1 = p[1], q0 = q[0], q1 = q[1];
  const float y02 = __uint_as_float(p0) + __uint_as_float(p1);  // lower half: x0 over both halves, upper half: x2
  const float y13 = __uint_as_float(q0) + __uint_as_float(q1);
  const nsa_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(y02), __float_as_uint(y13), false, false);
  const unsigned r0 = r[0], r1 = r[1];
  return __uint_as_float(r0) + __uint_as_float(r1);
}

// Value of another lane of the same 16-lane row by a DPP control word (0x110 + n: from n lanes below,
// 0x100 + n: from n lanes above, both 0 where that lane is outside the row; 0xB1 / 0x4E: partner in a
// pair / quad; 0x141 / 0x140: mirror within 8 / 16 lanes).
template <int CTRL> __device__ __forceinline__ float dpp_f32(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}

// Sum / maximum over the 64 lanes of a wave, returned to every lane, in a fixed order.
__device__ __forceinline__ float wave_sum_f32(float x) {
  x += dpp_f32<0xB1>(x); x += dpp_f32<0x4E>(x); x += dpp_f32<0x141>(x); x += dpp_f32<0x140>(x);
  return column_sum(x);
}
__device__ __forceinline__ float wave_max_f32(float x) {
  x = fmaxf(x, dpp_f32<0xB1>(x)); x = fmaxf(x, dpp_f32<0x4E>(x)); x = fmaxf(x, dpp_f32<0x141>(x)); x = fmaxf(x, dpp_f32<0x140>(x));
  return column_max(x);
}

// Wave-wide maximum of a signed 64-bit key, returned to every lane: four DPP steps inside each row of
// 16 lanes (pair, quad, half-row mirror, row mirror), then the two lane swaps across rows.
template <int CTRL> __device__ __forceinline__ long long dpp_exchange64(long long k) {
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(unsigned)(unsigned long long)k, CTRL, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(k >> 32), CTRL, 0xf, 0xf, false);
  return ((long long)hi << 32) | (unsigned)lo;
}
__device__ __forceinline__ long long wave_max_i64(long long k) {
  long long o;
  o = dpp_exchange64<0xB1>(k); k = o > k ? o : k;   // quad_perm [1,0,3,2]
  o = dpp_exchange64<0x4E>(k); k = o > k ? o : k;   // quad_perm [2,3,0,1]
  o = dpp_exchange64<0x141>(k); k = o > k ? o : k;  // row_half_mirror
  o = dpp_exchange64<0x140>(k); k = o > k ? o : k;  // row_mirror
  {
    const unsigned lo = (unsigned)(unsigned long long)k, hi = (unsigned)((unsigned long long)k >> 32);
    const nsa_u32x2 a = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
    const nsa_u32x2 b = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
    const unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
    const long long x = ((long long)(int)b0 << 32) | a0, y = ((long long)(int)b1 << 32) | a1;
    k = x > y ? x : y;
  }
  {
    const unsigned lo = (unsigned)(unsigned long long)k, hi = (unsigned)((unsigned long long)k >> 32);
    const nsa_u32x2 a = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
    const nsa_u32x2 b = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
    const unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
    const long long x = ((long long)(int)b0 << 32) | a0, y = ((long long)(int)b1 << 32) | a1;
    k = x > y ? x : y;
  }
  return k;
}
// Sort key of a (score, index) candidate: larger score first, smaller index on ties.  Scores here are
// non-negative (or +inf), whose bit patterns order like the numbers; negative markers sort below.
__device__ __forceinline__ long long candidate_key(float score, int index) {
  return ((long long)__float_as_int(score) << 32) | (unsigned)(0x7fffffff - index);
}
__device__ __forceinline__ int candidate_index(long long key) { return 0x7fffffff - (int)(unsigned)(unsigned long long)key; }

// out[0] = 0, out[b + 1] = sum over sequences <= b of ceil((cu[b + 1] - cu[b]) / unit): the prefix sum of the number
// of unit-sized blocks per sequence, by one workgroup of 256 threads (thread t owns a contiguous run of sequences,
// the 256 run totals are scanned in LDS).  Every thread of the workgroup must call it; ends with a barrier.
__device__ __forceinline__ void block_count_prefix_256(const int32_t* __restrict__ cu, int batch, int unit, int32_t* __restrict__ out) {
  __shared__ int run_total[256];
  const int tid = threadIdx.x, per = (batch + 255) / 256;
  const int b0 = min(batch, tid * per), b1 = min(batch, b0 + per);
  int sum = 0;
  for (int b = b0; b < b1; b++) sum += (cu[b + 1] - cu[b] + unit - 1) / unit;
  run_total[tid] = sum;
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const int v = tid >= d ? run_total[tid - d] : 0;
    __syncthreads();
    run_total[tid] += v;
    __syncthreads();
  }
  int acc = run_total[tid] - sum;
  if (tid == 0) out[0] = 0;
  for (int b = b0; b < b1; b++) {
    acc += (cu[b + 1] - cu[b] + unit - 1) / unit;
    out[b + 1] = acc;
  }
  __syncthreads();
}

// Index of the sequence that holds global token t: largest b with cu[b] <= t.
__device__ __forceinline__ int find_sequence(const int32_t* __restrict__ cu, int batch, int t) {
  int lo = 0, hi = batch;  // invariant: cu[lo] <= t < cu[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// A token's row of selected block ids is a set: an id listed twice counts once (in the forward, in dQ and in the
// reverse index alike).  The query-stationary kernels hold a stretch of 64 entries one per lane and visit the valid
// ones through a bit mask.  row_stretch loads the stretch that starts at entry e0 into my_blk and returns the mask of
// entries that are valid (0 <= id <= own block) and repeat no entry of an earlier stretch; repeats inside the stretch
// are dropped when the first of them is visited (row_visited).
__device__ __forceinline__ unsigned long long row_stretch(const int32_t* __restrict__ ip, long long isk, int topk, int e0, int lane, int own_block, int& my_blk) {
  my_blk = e0 + lane < topk ? ip[(long long)(e0 + lane) * isk] : -1;
  unsigned long long valid = __ballot(my_blk >= 0 && my_blk <= own_block);
  for (int p0 = 0; p0 < e0 && valid; p0 += 64) {   // rows of more than 64 entries only
    const int earlier = ip[(long long)(p0 + lane) * isk];
    for (int j = 0; j < 64; j++) {
      const int b = __builtin_amdgcn_readlane(earlier, j);
      if (b >= 0) valid &= ~__ballot(my_blk == b);
    }
  }
  return valid;
}
// mask of the entries still to visit once block blk has been taken
__device__ __forceinline__ unsigned long long row_visited(unsigned long long todo, int my_blk, int blk) { return todo & ~__ballot(my_blk == blk); }

// Spread consecutive logical work ids over the 8 XCDs in contiguous runs: hardware hands
// workgroup i to XCD i%8, so logical id = (i%8)*ceil(n/8) + i/8 keeps neighbours on one L2.
__device__ __forceinline__ long long xcd_remap(long long wg, long long n_wg) {
  long long per = (n_wg + 7) / 8;
  return (wg % 8) * per + wg / 8;
}

// How the two query-stationary kernels (one wave per (token, kv-head, head tile)) share their work items out over
// the 8 XCDs.  Hardware hands workgroup i to XCD i % 8; a stream = the tokens of one (kv-head, head tile), whose
// K/V should stay on as few L2s as possible.  When the streams divide the XCDs evenly and the batch is a single
// sequence, each stream is cut into 8 / streams contiguous parts of equal estimated cost, one per XCD: a
// token's cost grows with its position (its blocks are drawn from a longer prefix, of which the L2 holds a
// smaller share); measured on single sequences of 16K..64K tokens the cost per token is proportional to
// q0 + q, q = position / 64 and q0 = q0_l2_blocks x (the 64-key blocks of K and V that fit one XCD's 4 MiB L2), with
// q0_l2_blocks about 5.5 for the forward and 8 for the dQ pass (more work per block at the same traffic).  With
// equal token counts instead, the XCD holding the late half of a sequence ran 40 % longer than its partner.
// parts = 0: every XCD takes an equal share of all items in (stream, token) order.
struct XcdSchedule {
  int parts;        // XCDs per stream, or 0
  int wgs_per_xcd;  // workgroups (of 4 items) each XCD is given
  int bound[9];     // part j of a stream holds the 64-token runs [bound[j], bound[j + 1])
};
static inline XcdSchedule nsa_xcd_schedule(long long total_len, long long batch, int streams, int head_dim, double q0_l2_blocks) {
  XcdSchedule s;
  s.parts = 0; s.wgs_per_xcd = 0;
  for (int i = 0; i < 9; i++) s.bound[i] = 0;
  const long long runs = (total_len + 63) / 64;
  if (batch != 1 || streams <= 0 || streams > 8 || 8 % streams != 0 || runs < 64) return s;
  const int parts = 8 / streams;
  const double q0 = q0_l2_blocks * (4.0 * 1024 * 1024) / (64.0 * head_dim * 4), total = q0 * runs + 0.5 * runs * runs;
  s.parts = parts;
  s.bound[parts] = (int)runs;
  long long longest = 0;
  for (int j = 1; j <= parts; j++) {
    if (j < parts) {
      // C(q) = q0 q + q^2 / 2 = (j / parts) C(runs)
      const double target = total * j / parts;
      s.bound[j] = (int)(-q0 + __builtin_sqrt(q0 * q0 + 2.0 * target));
    }
    if (s.bound[j] - s.bound[j - 1] > longest) longest = s.bound[j] - s.bound[j - 1];
  }
  s.wgs_per_xcd = (int)(longest * 16);
  return s;
}

static inline int nsa_check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? NSA_OK : NSA_ERR_LAUNCH;
}

// Number of 32-key chunk slots in a block-transposed copy of a [T, H, D] tensor: every
// sequence starts on a fresh slot, so at most one slot of slack per sequence boundary.
static inline int64_t nsa_chunk_slots(int64_t total_len, int64_t batch) { return (total_len + 31) / 32 + batch + 1; }
