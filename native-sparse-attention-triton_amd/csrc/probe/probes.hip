// Memory-system and MFMA probes for the benchmark report (libnsa_probe.so; nothing in the operator library or the
// Python package uses them).  Each one isolates a rate that bounds one of the attention kernels:
//   nsa_probe_gather_blocks : the access pattern of the two query-stationary kernels without their arithmetic -
//                             one wave per (token, kv-head) fetches the 64-key blocks named by topk_idx from the
//                             fragment-major K / V copies, 32 KiB per block, and folds them into a checksum;
//   nsa_probe_gather_rows   : the access pattern of the dK/dV pass - 4 KiB rows at random offsets of a buffer;
//   nsa_probe_copy          : a plain copy (reference point for the FETCH_SIZE / WRITE_SIZE counters);
//   nsa_probe_mfma          : back-to-back independent MFMAs on registers (the matrix-core ceiling).
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, long long n) {
  // a workgroup moves 16 KiB per trip: four 16-byte pieces per thread, all loads before the stores
  for (long long i = (long long)blockIdx.x * 1024 + threadIdx.x; i < n; i += (long long)gridDim.x * 1024) {
    uint4 x[4];
#pragma unroll
    for (int u = 0; u < 4; u++) x[u] = i + 256 * u < n ? src[i + 256 * u] : uint4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < 4; u++) if (i + 256 * u < n) dst[i + 256 * u] = x[u];
  }
}

// kf / vf: [Hkv][n_slots][32 keys][D = 128] 2-byte elements, a 64-key block = 16 KiB of each; idx [Hkv][T][topk].
// fold > 0: block ids are taken modulo fold (a working set that stays in L2).  contiguous_split = 1: the first half
// of a head's tokens on one XCD, the second half on its partner (workgroup i runs on XCD i % 8).
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void probe_gather_blocks_kernel(
    const uint4* __restrict__ kf, const uint4* __restrict__ vf, const int32_t* __restrict__ idx, int T, int Hkv, int topk, int n_slots, int fold,
    uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long per = (gridDim.x + 7) / 8;
  const long long item = ((blockIdx.x % 8) * per + blockIdx.x / 8) * 4 + wave;
  if (item >= (long long)T * Hkv) return;
  const int t = (int)(item % T), h = (int)(item / T);
  const int32_t* ip = idx + ((long long)h * T + t) * topk;
  // a 32-key slot = 32 x 128 x 2 B = 512 uint4; a 64-key block = two slots = 16 fragments of 64 lanes x 16 B, in K and in V
  const uint4* kb = kf + (long long)h * n_slots * 512 + lane;
  const uint4* vb = vf + (long long)h * n_slots * 512 + lane;
  uint4 acc = {0u, 0u, 0u, 0u};
  const int my_blk = lane < topk ? ip[lane] : -1;
  unsigned long long todo = __ballot(my_blk >= 0);
  while (todo) {
    const int e = __builtin_ctzll(todo);
    todo &= todo - 1;
    int blk = __builtin_amdgcn_readlane(my_blk, e);
    if (fold > 0) blk %= fold;
    const uint4* kp = kb + (long long)(2 * blk) * 512;
    const uint4* vp = vb + (long long)(2 * blk) * 512;
    uint4 x[32];
#pragma unroll
    for (int f = 0; f < 16; f++) { x[f] = kp[f * 64]; x[16 + f] = vp[f * 64]; }
#pragma unroll
    for (int f = 0; f < 32; f++) { acc.x ^= x[f].x; acc.y ^= x[f].y; acc.z ^= x[f].z; acc.w ^= x[f].w; }
  }
  out[item * 64 + lane] = acc;
}

// every wave reads `reads` (a multiple of 8) rows of 4 KiB at pseudo-random row indices of buf, eight rows in flight
__global__ __launch_bounds__(256) void probe_gather_rows_kernel(const uint4* __restrict__ buf, long long n_rows, int reads, uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  unsigned long long state = 0x9E3779B97F4A7C15ull * (unsigned long long)(wave + 1);
  uint4 acc = {0u, 0u, 0u, 0u};
  for (int r = 0; r < reads; r += 8) {
    uint4 x[32];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      state = state * 6364136223846793005ull + 1442695040888963407ull;
      const long long row = (long long)((state >> 20) % (unsigned long long)n_rows);
      const uint4* p = buf + row * 256 + lane;
#pragma unroll
      for (int c = 0; c < 4; c++) x[4 * u + c] = p[c * 64];
    }
#pragma unroll
    for (int u = 0; u < 32; u++) { acc.x ^= x[u].x; acc.y ^= x[u].y; acc.z ^= x[u].z; acc.w ^= x[u].w; }
  }
  out[wave * 64 + lane] = acc;
}

template <int SHAPE>
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* __restrict__ out) {
  bf16x8 a, b;
  for (int i = 0; i < 8; i++) { a[i] = (__bf16)(threadIdx.x * 0.001f + i); b[i] = (__bf16)(1.f - threadIdx.x * 0.002f); }
  float sum = 0.f;
  if (SHAPE == 16) {
    f32x4 c[8];
    for (int j = 0; j < 8; j++) c[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int j = 0; j < 8; j++) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c[j], 0, 0, 0);
    }
    for (int j = 0; j < 8; j++) sum += c[j][0] + c[j][1] + c[j][2] + c[j][3];
  } else {
    f32x16 c[4];
    for (int j = 0; j < 4; j++) for (int r = 0; r < 16; r++) c[j][r] = 0.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int j = 0; j < 4; j++) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[j], 0, 0, 0);
    }
    for (int j = 0; j < 4; j++) for (int r = 0; r < 16; r++) sum += c[j][r];
  }
  out[(long long)blockIdx.x * 256 + threadIdx.x] = sum;
}

// Do the matrix pipe and the vector ALU of a SIMD work at the same time?  Per trip a wave issues 8 independent
// 16x16x32 MFMAs (MODE & 1) and 8 exp2 + 24 fused multiply-adds on 24 independent registers (MODE & 2), in source
// order MFMA, 4 vector operations (a multiply-add feeding an exp2, two more multiply-adds), MFMA, ...; MODE & 4 puts
// four more multiply-adds (same issue time) in the place of the exp2
// MODE & 16: the two kinds of work on different waves of a SIMD: workgroups of the first half of the grid issue only the MFMAs,
// those of the second half only the vector operations (with 512 workgroups each CU gets one of either kind)
template <int MODE>
__global__ __launch_bounds__(256) void probe_coexec_kernel(int iters, float* __restrict__ out) {
  bf16x8 a, b;
  for (int i = 0; i < 8; i++) { a[i] = (__bf16)(threadIdx.x * 0.001f + i); b[i] = (__bf16)(1.f - threadIdx.x * 0.002f); }
  f32x4 c[8];
  float x[32];
  for (int j = 0; j < 8; j++) c[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < 32; j++) x[j] = 0.001f * (float)(threadIdx.x + j);
  const float ka = 0.5f + 1e-6f * (float)threadIdx.x, kb = -0.25f;
  auto trips = [&](auto with_mfma, auto with_valu) {
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int j = 0; j < 8; j++) {
        if (decltype(with_mfma)::value) {
          if (MODE & 8) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c[j]) : "v"(a), "v"(b));   // accumulator in AGPRs
          else c[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c[j], 0, 0, 0);
        }
        if (decltype(with_valu)::value) {
          if (MODE & 4) { x[4 * j] = __builtin_fmaf(x[4 * j], ka, kb); x[4 * j + 3] = __builtin_fmaf(x[4 * j + 3], ka, kb); x[4 * j] = __builtin_fmaf(x[4 * j], kb, ka); x[4 * j + 3] = __builtin_fmaf(x[4 * j + 3], kb, ka); }
          else x[4 * j] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[4 * j], ka, kb));
          x[4 * j + 1] = __builtin_fmaf(x[4 * j + 1], ka, kb);
          x[4 * j + 2] = __builtin_fmaf(x[4 * j + 2], ka, kb);
        }
      }
    }
  };
  using yes = std::true_type;
  using no = std::false_type;
  if (MODE & 16) {
    if (blockIdx.x < gridDim.x / 2) trips(yes{}, no{}); else trips(no{}, yes{});
  } else {
    trips(std::integral_constant<bool, (MODE & 1) != 0>{}, std::integral_constant<bool, (MODE & 2) != 0>{});
  }
  float sum = 0.f;
  for (int j = 0; j < 8; j++) sum += c[j][0] + c[j][1] + c[j][2] + c[j][3];
  for (int j = 0; j < 32; j++) sum += x[j];
  out[(long long)blockIdx.x * 256 + threadIdx.x] = sum;
}

extern "C" int nsa_probe_coexec(int mode, int iters, int n_workgroups, float* out, void* stream) {
  if (mode == 1) probe_coexec_kernel<1><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 2) probe_coexec_kernel<2><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 3) probe_coexec_kernel<3><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 6) probe_coexec_kernel<6><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 11) probe_coexec_kernel<11><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 19) probe_coexec_kernel<19><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (mode == 7) probe_coexec_kernel<7><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else return -2;
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int nsa_probe_copy(const void* src, void* dst, long long bytes, void* stream) {
  probe_copy_kernel<<<16384, 256, 0, (hipStream_t)stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int nsa_probe_gather_blocks(const void* kf, const void* vf, const int32_t* idx, int total_len, int num_kv_heads, int topk,
                                       int n_slots, int fold, void* out, void* stream) {
  if (topk > 64) return -2;
  long long n_wg = ((long long)total_len * num_kv_heads + 3) / 4;
  n_wg = (n_wg + 7) / 8 * 8;
  probe_gather_blocks_kernel<<<(unsigned)n_wg, 256, 0, (hipStream_t)stream>>>((const uint4*)kf, (const uint4*)vf, idx, total_len, num_kv_heads,
                                                                               topk, n_slots, fold, (uint4*)out);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int nsa_probe_gather_rows(const void* buf, long long n_rows, int row_bytes, int reads_per_wave, int n_workgroups, void* out, void* stream) {
  if (row_bytes != 4096 || reads_per_wave % 8 != 0) return -2;
  probe_gather_rows_kernel<<<n_workgroups, 256, 0, (hipStream_t)stream>>>((const uint4*)buf, n_rows, reads_per_wave, (uint4*)out);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

// flops per launch = n_workgroups * 4 waves * iters * 8 (or 4) MFMAs * 16384 (or 32768) flops
extern "C" int nsa_probe_mfma(int shape, int iters, int n_workgroups, float* out, void* stream) {
  if (shape == 16) probe_mfma_kernel<16><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else if (shape == 32) probe_mfma_kernel<32><<<n_workgroups, 256, 0, (hipStream_t)stream>>>(iters, out);
  else return -2;
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

// ------------------------------------------------------------------------------------------
// nsa_probe_tile_gather: the block gather with sharing inside a tile of 24 consecutive tokens.  A workgroup of 8
// waves (3 tokens each) forms the ascending list of the distinct blocks its tokens selected, stages each block once
// in a ring of 4 LDS buffers (asynchronous global->LDS copies issued by whichever wave reaches a safe point
// first), and every wave reads the staged block once per token of its own that selected it.  No arithmetic:
// the time is what the memory system and the ring allow a forward kernel of this shape.
struct TileCtl { int pos[8]; int ready[4]; int next_issue; int n_list; int err; int wave_cnt[8]; };

__global__ __launch_bounds__(512) void probe_tile_gather_kernel(const uint4* __restrict__ kf, const uint4* __restrict__ vf, const int32_t* __restrict__ idx,
                                                                int T, int Hkv, int topk, int n_slots, int n_tiles, uint4* __restrict__ out,
                                                                int* __restrict__ err_out) {
  constexpr int NW = 8, TPW = 3, TT = NW * TPW, R = 4, NB_MAX = 2048, L_MAX = TT * 32;
  __shared__ __attribute__((aligned(1024))) uint4 ring[R][2048];   // 32 KiB per block: 16 K fragments then 16 V fragments of 64 x 16 B
  __shared__ unsigned bmask[NB_MAX];
  __shared__ unsigned short list_blk[L_MAX];
  __shared__ unsigned list_mask[L_MAX];
  __shared__ TileCtl ctl;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long long per = (gridDim.x + 7) / 8;
  const long long item = (blockIdx.x % 8) * per + blockIdx.x / 8;    // consecutive tiles of a head on one XCD
  if (item >= (long long)n_tiles * Hkv) return;
  const int h = (int)(item / n_tiles), tile = (int)(item % n_tiles);
  const int t0 = tile * TT, nt = min(TT, T - t0);
  const int nb = (t0 + nt - 1) / 64 + 1;
  for (int i = tid; i < nb; i += 512) bmask[i] = 0u;
  if (tid < NW) ctl.pos[tid] = 0;
  if (tid < R) ctl.ready[tid] = 0;
  if (tid == 0) { ctl.next_issue = 0; ctl.err = 0; }
  __syncthreads();
  for (int e = tid; e < TT * topk; e += 512) {
    const int tk = e / topk, k = e % topk;
    if (tk < nt) {
      const int blk = idx[((long long)h * T + t0 + tk) * topk + k];
      if (blk >= 0 && blk <= (t0 + tk) / 64) atomicOr(&bmask[blk], 1u << tk);
    }
  }
  __syncthreads();
  int base = 0;
  for (int c0 = 0; c0 < nb; c0 += 512) {
    const int blk = c0 + tid;
    const unsigned m = blk < nb ? bmask[blk] : 0u;
    const unsigned long long ball = __ballot(m != 0u);
    if (lane == 0) ctl.wave_cnt[wave] = __popcll(ball);
    __syncthreads();
    int off = base, total = 0;
    for (int w = 0; w < NW; w++) { const int c = ctl.wave_cnt[w]; if (w < wave) off += c; total += c; }
    off += __popcll(ball & ((1ull << lane) - 1ull));
    if (m != 0u) { list_blk[off] = (unsigned short)blk; list_mask[off] = m; }
    __syncthreads();
    base += total;
  }
  const int n_list = base;
  const uint4* kb = kf + (long long)h * n_slots * 512 + lane;
  const uint4* vb = vf + (long long)h * n_slots * 512 + lane;
  uint4 acc[TPW];
  for (int j = 0; j < TPW; j++) acc[j] = uint4{0u, 0u, 0u, 0u};
  int pending = -1;
  // publish a finished copy, then start the next one if its buffer is free and nobody else has claimed it
  auto produce = [&]() {
    if (pending >= 0) {
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the copy has landed in LDS
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0) __hip_atomic_store(&ctl.ready[pending % R], pending + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      pending = -1;
    }
    const int j = __hip_atomic_load(&ctl.next_issue, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (j >= n_list) return;
    int lo = 1 << 30;
    for (int w = 0; w < NW; w++) lo = min(lo, __hip_atomic_load(&ctl.pos[w], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
    if (lo + R <= j) return;          // some wave still needs the block that sits in this buffer
    int won = 0;
    if (lane == 0) {
      int expect = j;
      won = __hip_atomic_compare_exchange_strong(&ctl.next_issue, &expect, j + 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    won = __builtin_amdgcn_readfirstlane(won);
    if (!won) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int blk = list_blk[j];
    const uint4* kp = kb + (long long)(2 * blk) * 512;
    const uint4* vp = vb + (long long)(2 * blk) * 512;
    unsigned char* dst = (unsigned char*)&ring[j % R][0];
#pragma unroll
    for (int f = 0; f < 16; f++) {
      __builtin_amdgcn_global_load_lds(kp + f * 64, (__attribute__((address_space(3))) void*)(dst + f * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(vp + f * 64, (__attribute__((address_space(3))) void*)(dst + 16384 + f * 1024), 16, 0, 0);
    }
    pending = j;
  };
  for (int i = 0; i < n_list; i++) {
    const unsigned m = (list_mask[i] >> (TPW * wave)) & ((1u << TPW) - 1u);
    if (m != 0u) {
      int spins = 0;
      while (__hip_atomic_load(&ctl.ready[i % R], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != i + 1) {
        produce();
        __builtin_amdgcn_s_sleep(1);
        if (++spins > (1 << 22) || __hip_atomic_load(&ctl.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) {
          if (lane == 0) { __hip_atomic_store(&ctl.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); *err_out = 1; }
          i = n_list;   // give up: every wave leaves its loop
          break;
        }
      }
      if (i >= n_list) break;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      const uint4* src = &ring[i % R][lane];
#pragma unroll
      for (int j = 0; j < TPW; j++) {
        if (m & (1u << j)) {
          uint4 x[32];
#pragma unroll
          for (int f = 0; f < 32; f++) x[f] = src[f * 64];
#pragma unroll
          for (int f = 0; f < 32; f++) { acc[j].x ^= x[f].x; acc[j].y ^= x[f].y; acc[j].z ^= x[f].z; acc[j].w ^= x[f].w; }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0) __hip_atomic_store(&ctl.pos[wave], i + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    produce();
  }
  // a copy this wave started may still be in flight: let it land before the workgroup's LDS is given away
  __builtin_amdgcn_s_waitcnt(0x0F70);
  if (pending >= 0 && lane == 0) __hip_atomic_store(&ctl.ready[pending % R], pending + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  for (int j = 0; j < TPW; j++)
    if (wave * TPW + j < nt) out[((long long)h * T + t0 + wave * TPW + j) * 64 + lane] = acc[j];
}

extern "C" int nsa_probe_tile_gather(const void* kf, const void* vf, const int32_t* idx, int total_len, int num_kv_heads, int topk, int n_slots,
                                     void* out, int* err_out, void* stream) {
  if (topk > 32 || (total_len + 63) / 64 > 2048) return -2;
  const int n_tiles = (total_len + 23) / 24;
  long long n_wg = ((long long)n_tiles * num_kv_heads + 7) / 8 * 8;
  probe_tile_gather_kernel<<<(unsigned)n_wg, 512, 0, (hipStream_t)stream>>>((const uint4*)kf, (const uint4*)vf, idx, total_len, num_kv_heads, topk,
                                                                            n_slots, n_tiles, (uint4*)out, err_out);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
