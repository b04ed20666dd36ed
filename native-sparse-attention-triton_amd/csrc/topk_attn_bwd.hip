// Backward of block-sparse GQA attention (topk_sparse_attention): dQ, dK, dV.
//
// Passes, all on the caller's stream and out of the caller's workspace:
//   1. delta[h][t] = sum_d O*dO.
//   2. Reverse index "KV block -> queries that selected it": one (key = head*blocks + block,
//      value = token) pair per valid topk_idx entry, stable radix sort by key (tokens stay
//      ascending inside a block), segment offsets by binary search.  No host round trips.
//   3. dK/dV: a workgroup keeps one KV block's K and V rows in registers (each wave owns 16
//      keys) and streams the queries of that block two tokens at a time through LDS; per-chunk
//      fp32 partials are reduced in a fixed order, so the result is deterministic (no atomics).
//   4. dQ: one wavefront per (token, kv-head), same dataflow as the forward kernel, with a
//      block-transposed copy of K feeding dQ^T += K^T * dS^T.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "block_transpose.h"

// ------------------------------------------------------------------------------------------
// workspace carving (host and entry point must agree)
struct BwdLayout {
  size_t delta, cu_blk, keys_in, keys_out, vals_in, vals_out, seg_off, chunk_off, sort_tmp, kt, partial, total;
  size_t sort_tmp_bytes;
  int64_t max_blocks, n_pairs, max_items, n_slots;
};

static constexpr int CHUNK_TOKENS = 1024;  // queries per dK/dV work item

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

static BwdLayout bwd_layout(int64_t T, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t topk, int64_t bs) {
  BwdLayout L;
  L.max_blocks = T / bs + B;  // every sequence adds at most one ragged block
  L.n_pairs = Hkv * T * topk;
  const int64_t GT = (Hq / Hkv + 15) / 16;
  L.max_items = (L.n_pairs + CHUNK_TOKENS - 1) / CHUNK_TOKENS + Hkv * L.max_blocks;
  L.n_slots = nsa_chunk_slots(T, B);
  (void)GT;
  size_t tmp = 0;
  uint32_t* nk = nullptr;
  int32_t* nv = nullptr;
  (void)rocprim::radix_sort_pairs(nullptr, tmp, nk, nk, nv, nv, (size_t)L.n_pairs, 0u, 32u, (hipStream_t)0);
  L.sort_tmp_bytes = tmp;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align256(bytes); return o; };
  L.delta = take((size_t)Hq * T * 4);
  L.cu_blk = take((size_t)(B + 1) * 4);
  L.keys_in = take((size_t)L.n_pairs * 4);
  L.keys_out = take((size_t)L.n_pairs * 4);
  L.vals_in = take((size_t)L.n_pairs * 4);
  L.vals_out = take((size_t)L.n_pairs * 4);
  L.seg_off = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.chunk_off = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.sort_tmp = take(tmp);
  L.kt = take((size_t)Hkv * L.n_slots * D * 32 * 2);
  L.partial = take((size_t)L.max_items * bs * D * 4 * 2);
  L.total = off;
  return L;
}

// ------------------------------------------------------------------------------------------
// pass 1: delta
template <typename T, int D>
__global__ __launch_bounds__(256) void delta_kernel(const T* __restrict__ o, const T* __restrict__ dout, float* __restrict__ delta,
                                                    int total_len, int Hq, long long osn, long long osh, long long dsn, long long dsh) {
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
  if (live && sub == 0) delta[(long long)h * total_len + t] = acc;
}

// ------------------------------------------------------------------------------------------
// pass 2: reverse index
__global__ void seq_blocks_kernel(const int32_t* __restrict__ cu, int batch, int bs, int32_t* __restrict__ cu_blk) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int acc = 0;
    cu_blk[0] = 0;
    for (int b = 0; b < batch; b++) {
      acc += (cu[b + 1] - cu[b] + bs - 1) / bs;
      cu_blk[b + 1] = acc;
    }
  }
}

__global__ __launch_bounds__(256) void emit_pairs_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ cu,
                                                         const int32_t* __restrict__ cu_blk, int batch, int total_len, int Hkv,
                                                         int topk, int bs, int max_blocks, long long ish, long long isn,
                                                         long long isk, uint32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // (h, t, e), e fastest
  const long long n = (long long)Hkv * total_len * topk;
  if (i >= n) return;
  const int e = (int)(i % topk);
  const int t = (int)((i / topk) % total_len);
  const int h = (int)(i / ((long long)topk * total_len));
  const int b = find_sequence(cu, batch, t);
  const int qb = (t - cu[b]) / bs;
  const int blk = idx[(long long)h * ish + (long long)t * isn + (long long)e * isk];
  const bool ok = blk >= 0 && blk <= qb;
  keys[i] = ok ? (uint32_t)(h * max_blocks + cu_blk[b] + blk) : (uint32_t)(Hkv * max_blocks);
  vals[i] = t;
}

// seg_off[j] = first sorted position whose key >= j, j in [0, n_seg]; chunk counts alongside.
__global__ __launch_bounds__(256) void segment_offsets_kernel(const uint32_t* __restrict__ keys, long long n, int n_seg,
                                                              int32_t* __restrict__ seg_off) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j > n_seg) return;
  long long lo = 0, hi = n;  // first position with keys[pos] >= j
  while (lo < hi) {
    long long mid = (lo + hi) >> 1;
    if (keys[mid] < (uint32_t)j) lo = mid + 1; else hi = mid;
  }
  seg_off[j] = (int32_t)lo;
}

// chunk_off = exclusive scan of ceil(count/CHUNK_TOKENS) over segments (single workgroup).
__global__ __launch_bounds__(1024) void chunk_scan_kernel(const int32_t* __restrict__ seg_off, int n_seg, int32_t* __restrict__ chunk_off) {
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int per = (n_seg + 1023) / 1024;
  const int j0 = tid * per, j1 = min(n_seg, j0 + per);
  int s = 0;
  for (int j = j0; j < j1; j++) s += (seg_off[j + 1] - seg_off[j] + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
  part[tid] = s;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    int v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = part[tid] - s;
  for (int j = j0; j < j1; j++) {
    chunk_off[j] = run;
    run += (seg_off[j + 1] - seg_off[j] + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
  }
  if (tid == 1023) chunk_off[n_seg] = part[1023];
}

// ------------------------------------------------------------------------------------------
// pass 3: dK / dV
struct DkdvParams {
  const void* q; const void* k; const void* v; const void* dout; const float* lse; const float* delta;
  const int32_t* cu; const int32_t* cu_blk; const int32_t* seg_off; const int32_t* chunk_off; const int32_t* queries;
  float* partial;
  int total_len, batch, Hkv, G, GT, max_blocks, n_seg;
  long long qsn, qsh, ksn, ksh, vsn, vsh, dsn, dsh;
  float qk_scale, sm_scale;
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(BS >= 64 ? 256 : 128) void dkdv_kernel(DkdvParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, NDT = D / 16, NSUB = BS / 16;
  constexpr int NW = NSUB < 4 ? NSUB : 4;     // waves per workgroup
  constexpr int KT = NSUB / NW;               // 16-key tiles per wave
  constexpr int NT = NW * 64;
  constexpr int LD = D + 8;                   // padded LDS row (elements)
  __shared__ __attribute__((aligned(16))) T q_s[2][2][16][LD];
  __shared__ __attribute__((aligned(16))) T do_s[2][2][16][LD];
  __shared__ float lse_s[2][32], delta_s[2][32];
  __shared__ int pos_s[2][2];

  const int total_items = p.chunk_off[p.n_seg];
  const int item = blockIdx.x;
  if (item >= total_items) return;
  // segment (head, global block) that owns this work item
  int lo = 0, hi = p.n_seg;  // chunk_off[lo] <= item < chunk_off[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (p.chunk_off[mid] <= item) lo = mid; else hi = mid;
  }
  const int seg = lo;
  const int h = seg / p.max_blocks, gb = seg % p.max_blocks;
  const int b = find_sequence(p.cu_blk, p.batch, gb);
  const int s0 = p.cu[b], len = p.cu[b + 1] - s0;
  const int key0 = (gb - p.cu_blk[b]) * BS;
  const int first = p.seg_off[seg] + (item - p.chunk_off[seg]) * CHUNK_TOKENS;
  const int n_tok = min(CHUNK_TOKENS, p.seg_off[seg + 1] - first);
  const int n_rg = n_tok * p.GT;              // row groups (token, head tile) in this chunk
  const int n_step = (n_rg + 1) / 2;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;

  // stationary operands: this wave's keys of K and V, B-operand layout (column = key)
  v8 kf[KT][NK], vf[KT][NK];
#pragma unroll
  for (int j = 0; j < KT; j++) {
    int row = key0 + 16 * (wave * KT + j) + li;
    row = row < len ? row : len - 1;
    const T* kp = (const T*)p.k + (long long)(s0 + row) * p.ksn + (long long)h * p.ksh + 8 * lg;
    const T* vp = (const T*)p.v + (long long)(s0 + row) * p.vsn + (long long)h * p.vsh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) { kf[j][kk] = ld16<v8>(kp + 32 * kk); vf[j][kk] = ld16<v8>(vp + 32 * kk); }
  }
  f32x4 dk[KT][NDT], dv[KT][NDT];
#pragma unroll
  for (int j = 0; j < KT; j++)
#pragma unroll
    for (int i = 0; i < NDT; i++) { dk[j][i] = f32x4{0.f, 0.f, 0.f, 0.f}; dv[j][i] = f32x4{0.f, 0.f, 0.f, 0.f}; }

  // staging: 2 row groups x 16 heads x D elements for each of Q and dO = 2*2*16*D/8 16-byte pieces
  constexpr int PIECES = 2 * 2 * 16 * (D / 8);
  constexpr int PPT = (PIECES + NT - 1) / NT;
  uint4 stage[PPT];
  float st_lse = 0.f, st_delta = 0.f;
  int st_pos = 0;

  auto fetch = [&](int step) {
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = tid + u * NT;
      uint4 val = {0u, 0u, 0u, 0u};
      if (pc < PIECES) {
        const int c = pc % (D / 8), hd = (pc / (D / 8)) % 16, rg = (pc / (D / 8) / 16) % 2, which = pc / (D / 8) / 32;
        const int r = step * 2 + rg;
        if (r < n_rg) {
          const int t = p.queries[first + r / p.GT];
          const int hq = (r % p.GT) * 16 + hd;
          if (hq < p.G) {
            const T* src = which == 0 ? (const T*)p.q + (long long)t * p.qsn + (long long)(h * p.G + hq) * p.qsh
                                      : (const T*)p.dout + (long long)t * p.dsn + (long long)(h * p.G + hq) * p.dsh;
            val = *reinterpret_cast<const uint4*>(src + 8 * c);
          }
        }
      }
      stage[u] = val;
    }
    if (tid < 32) {
      const int rg = tid >> 4, hd = tid & 15;
      const int r = step * 2 + rg;
      st_lse = INFINITY; st_delta = 0.f; st_pos = -1;
      if (r < n_rg) {
        const int t = p.queries[first + r / p.GT];
        const int hq = (r % p.GT) * 16 + hd;
        st_pos = t - s0;
        if (hq < p.G) {
          st_lse = p.lse[(long long)(h * p.G + hq) * p.total_len + t];
          st_delta = p.delta[(long long)(h * p.G + hq) * p.total_len + t];
        }
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = tid + u * NT;
      if (pc < PIECES) {
        const int c = pc % (D / 8), hd = (pc / (D / 8)) % 16, rg = (pc / (D / 8) / 16) % 2, which = pc / (D / 8) / 32;
        T* dst = which == 0 ? &q_s[buf][rg][hd][8 * c] : &do_s[buf][rg][hd][8 * c];
        *reinterpret_cast<uint4*>(dst) = stage[u];
      }
    }
    if (tid < 32) {
      lse_s[buf][tid] = st_lse;
      delta_s[buf][tid] = st_delta;
      if ((tid & 15) == 0) pos_s[buf][tid >> 4] = st_pos;
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  for (int step = 0; step < n_step; step++) {
    const int buf = step & 1;
    if (step + 1 < n_step) fetch(step + 1);

    // S = Q K^T and dP = dO V^T for this wave's keys; lane holds column key=li, rows 4*lg+r of each token
    v8 pf[KT], dsf[KT];
#pragma unroll
    for (int j = 0; j < KT; j++) {
      const int key = key0 + 16 * (wave * KT + j) + li;
#pragma unroll
      for (int tk = 0; tk < 2; tk++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          v8 qa = ld16<v8>(&q_s[buf][tk][li][32 * kk + 8 * lg]);
          v8 da = ld16<v8>(&do_s[buf][tk][li][32 * kk + 8 * lg]);
          s = E::mfma16(qa, kf[j][kk], s);
          dp = E::mfma16(da, vf[j][kk], dp);
        }
        const int pos = pos_s[buf][tk];
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float l2 = lse_s[buf][tk * 16 + 4 * lg + r];
          const float dl = delta_s[buf][tk * 16 + 4 * lg + r];
          const float pr = key <= pos ? fast_exp2(s[r] * p.qk_scale - l2) : 0.f;
          pf[j][tk * 4 + r] = (T)pr;
          dsf[j][tk * 4 + r] = (T)(pr * (dp[r] - dl) * p.sm_scale);
        }
      }
    }
    // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key]
    // transposed fragments come from LDS: lane j of a 16-lane group addresses the 4-element
    // chunk (row 4*lg + j/4, columns 16*dt + 4*(j%4)) and receives column li of those 4 rows.
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 qt, dot;
#pragma unroll
      for (int tk = 0; tk < 2; tk++) {
        const T* qa = &q_s[buf][tk][4 * lg + (li >> 2)][16 * dt + 4 * (li & 3)];
        const T* da = &do_s[buf][tk][4 * lg + (li >> 2)][16 * dt + 4 * (li & 3)];
        s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(qa));
        s16x4 c = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(da));
#pragma unroll
        for (int r = 0; r < 4; r++) { qt[tk * 4 + r] = a[r]; dot[tk * 4 + r] = c[r]; }
      }
      const v8 qtf = __builtin_bit_cast(v8, qt), dotf = __builtin_bit_cast(v8, dot);
#pragma unroll
      for (int j = 0; j < KT; j++) {
        dv[j][dt] = E::mfma16(dotf, pf[j], dv[j][dt]);
        dk[j][dt] = E::mfma16(qtf, dsf[j], dk[j][dt]);
      }
    }
    if (step + 1 < n_step) stash(buf ^ 1);
    __syncthreads();
  }
  // partial[item][0 = dK, 1 = dV][key][d], fp32
  float* out = p.partial + (long long)item * 2 * BS * D;
#pragma unroll
  for (int j = 0; j < KT; j++) {
    const int kl = 16 * (wave * KT + j) + li;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      *reinterpret_cast<f32x4*>(out + (long long)kl * D + 16 * dt + 4 * lg) = dk[j][dt];
      *reinterpret_cast<f32x4*>(out + (long long)(BS + kl) * D + 16 * dt + 4 * lg) = dv[j][dt];
    }
  }
}

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) void dkdv_reduce_kernel(const float* __restrict__ partial, const int32_t* __restrict__ chunk_off,
                                                          const int32_t* __restrict__ cu, const int32_t* __restrict__ cu_blk,
                                                          int batch, int max_blocks, T* __restrict__ dk, T* __restrict__ dv,
                                                          long long dksn, long long dksh, long long dvsn, long long dvsh) {
  const int seg = blockIdx.x;
  const int h = seg / max_blocks, gb = seg % max_blocks;
  if (gb >= cu_blk[batch]) return;
  const int b = find_sequence(cu_blk, batch, gb);
  const int s0 = cu[b], len = cu[b + 1] - s0;
  const int key0 = (gb - cu_blk[b]) * BS;
  const int c0 = chunk_off[seg], c1 = chunk_off[seg + 1];
  for (int i = threadIdx.x; i < 2 * BS * (D / 4); i += 256) {
    const int which = i / (BS * (D / 4)), key = (i / (D / 4)) % BS, d4 = i % (D / 4);
    if (key0 + key >= len) continue;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int c = c0; c < c1; c++) acc += *reinterpret_cast<const f32x4*>(partial + ((long long)c * 2 + which) * BS * D + (long long)key * D + 4 * d4);
    typename Elem<T>::v4 o;
#pragma unroll
    for (int r = 0; r < 4; r++) o[r] = (T)acc[r];
    T* dst = which == 0 ? dk + (long long)(s0 + key0 + key) * dksn + (long long)h * dksh : dv + (long long)(s0 + key0 + key) * dvsn + (long long)h * dvsh;
    st8(dst + 4 * d4, o);
  }
}

// ------------------------------------------------------------------------------------------
// pass 4: dQ
struct DqParams {
  const void* q; const void* k; const void* v; const void* kt; const void* dout; const float* lse; const float* delta;
  const int32_t* idx; const int32_t* cu; void* dq;
  int total_len, batch, Hkv, G, GT, topk, n_slots;
  long long n_items;
  long long qsn, qsh, ksn, ksh, vsn, vsh, dsn, dsh, ish, isn, isk, dqsn, dqsh;
  float qk_scale, sm_scale;
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) void dq_kernel(DqParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, NSUB = BS / 16, NCH = BS / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const long long item = xcd_remap(blockIdx.x, gridDim.x) * 4 + wave;
  if (item >= p.n_items) return;
  const int t = (int)(item % p.total_len);
  const int gt = (int)((item / p.total_len) % p.GT);
  const int h = (int)(item / ((long long)p.total_len * p.GT));
  const int b = find_sequence(p.cu, p.batch, t);
  const int s0 = p.cu[b], len = p.cu[b + 1] - s0;
  const int pos = t - s0, qb = pos / BS;
  const int slot0 = seq_first_slot(p.cu, b);
  const int hq = gt * 16 + li;
  const bool has_head = hq < p.G;
  const int hh = h * p.G + (has_head ? hq : 0);
  const T* qp = (const T*)p.q + (long long)t * p.qsn + (long long)hh * p.qsh + 8 * lg;
  const T* dp_ = (const T*)p.dout + (long long)t * p.dsn + (long long)hh * p.dsh + 8 * lg;
  v8 qf[NK], dof[NK];
#pragma unroll
  for (int kk = 0; kk < NK; kk++) {
    qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
    dof[kk] = has_head ? ld16<v8>(dp_ + 32 * kk) : zero16<v8>();
  }
  const float l2 = has_head ? p.lse[(long long)hh * p.total_len + t] : INFINITY;
  const float dl = has_head ? p.delta[(long long)hh * p.total_len + t] : 0.f;
  f32x4 acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* ip = p.idx + (long long)h * p.ish + (long long)t * p.isn;
  const T* kbase = (const T*)p.k + (long long)s0 * p.ksn + (long long)h * p.ksh + 8 * lg;
  const T* vbase = (const T*)p.v + (long long)s0 * p.vsn + (long long)h * p.vsh + 8 * lg;
  const T* ktbase = (const T*)p.kt + ((long long)h * p.n_slots + slot0) * D * 32 + li * 32 + 8 * lg;
  for (int e = 0; e < p.topk; e++) {
    const int blk = ip[(long long)e * p.isk];
    if (blk < 0 || blk > qb) continue;
    const int key0 = blk * BS;
    f32x4 ds[NSUB];
#pragma unroll
    for (int nt = 0; nt < NSUB; nt++) {
      f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
      if (key0 + 16 * nt <= pos) {
        int row = key0 + 16 * nt + li;
        row = row < len ? row : len - 1;
        const T* kp = kbase + (long long)row * p.ksn;
        const T* vp = vbase + (long long)row * p.vsn;
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          s = E::mfma16(ld16<v8>(kp + 32 * kk), qf[kk], s);
          dp = E::mfma16(ld16<v8>(vp + 32 * kk), dof[kk], dp);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int key = key0 + 16 * nt + 4 * lg + r;
        const float pr = key <= pos ? fast_exp2(s[r] * p.qk_scale - l2) : 0.f;
        ds[nt][r] = pr * (dp[r] - dl) * p.sm_scale;
      }
    }
#pragma unroll
    for (int c = 0; c < NCH; c++) {
      if (key0 + 32 * c > pos) break;
      v8 dsf;
#pragma unroll
      for (int r = 0; r < 4; r++) { dsf[r] = (T)ds[2 * c][r]; dsf[4 + r] = (T)ds[2 * c + 1][r]; }
      const T* ktp = ktbase + (long long)((key0 >> 5) + c) * D * 32;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) acc[dt] = E::mfma16(ld16<v8>(ktp + dt * 16 * 32), dsf, acc[dt]);
    }
  }
  if (has_head) {
    T* op = (T*)p.dq + (long long)t * p.dqsn + (long long)hh * p.dqsh + 4 * lg;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      v4 out;
#pragma unroll
      for (int r = 0; r < 4; r++) out[r] = (T)acc[dt][r];
      st8(op + 16 * dt, out);
    }
  }
}

// ------------------------------------------------------------------------------------------
struct BwdArgs {
  const void *q, *k, *v, *o, *dout; const float* lse; const int32_t* idx; const int32_t* cu; void *dq, *dk, *dv;
  int64_t T, B, Hq, Hkv, D, topk, bs;
  int64_t qsn, qsh, ksn, ksh, vsn, vsh, osn, osh, dsn, dsh, ish, isn, isk, dqsn, dqsh, dksn, dksh, dvsn, dvsh;
  float sm_scale; char* ws; hipStream_t stream; int phases;
  int32_t* out_seg_off; int32_t* out_queries;  // optional copies of the reverse index (tests)
};

static int build_reverse_index(const BwdArgs& a, const BwdLayout& L) {
  char* ws = a.ws;
  int32_t* cu_blk = (int32_t*)(ws + L.cu_blk);
  uint32_t* keys_in = (uint32_t*)(ws + L.keys_in);
  uint32_t* keys_out = (uint32_t*)(ws + L.keys_out);
  int32_t* vals_in = (int32_t*)(ws + L.vals_in);
  int32_t* vals_out = (int32_t*)(ws + L.vals_out);
  int32_t* seg_off = (int32_t*)(ws + L.seg_off);
  int32_t* chunk_off = (int32_t*)(ws + L.chunk_off);
  const int n_seg = (int)(a.Hkv * L.max_blocks);
  seq_blocks_kernel<<<1, 64, 0, a.stream>>>(a.cu, (int)a.B, (int)a.bs, cu_blk);
  emit_pairs_kernel<<<(unsigned)((L.n_pairs + 255) / 256), 256, 0, a.stream>>>(
      a.idx, a.cu, cu_blk, (int)a.B, (int)a.T, (int)a.Hkv, (int)a.topk, (int)a.bs, (int)L.max_blocks, a.ish, a.isn, a.isk, keys_in, vals_in);
  unsigned bits = 1;
  while ((1ull << bits) <= (unsigned long long)n_seg) bits++;
  size_t tmp = L.sort_tmp_bytes;
  if (rocprim::radix_sort_pairs(ws + L.sort_tmp, tmp, keys_in, keys_out, vals_in, vals_out, (size_t)L.n_pairs, 0u, bits, a.stream) != hipSuccess)
    return NSA_ERR_LAUNCH;
  segment_offsets_kernel<<<(n_seg + 1 + 255) / 256, 256, 0, a.stream>>>(keys_out, L.n_pairs, n_seg, seg_off);
  chunk_scan_kernel<<<1, 1024, 0, a.stream>>>(seg_off, n_seg, chunk_off);
  return nsa_check_launch();
}

template <typename T, int D, int BS>
static int run_bwd(const BwdArgs& a) {
  const BwdLayout L = bwd_layout(a.T, a.B, a.Hq, a.Hkv, a.D, a.topk, a.bs);
  char* ws = a.ws;
  float* delta = (float*)(ws + L.delta);
  const int G = (int)(a.Hq / a.Hkv), GT = (G + 15) / 16;
  const int n_seg = (int)(a.Hkv * L.max_blocks);
  if (a.phases & NSA_BWD_PHASE_PREP) {
    constexpr int LPR = D / 8, LPR2 = LPR <= 4 ? 4 : (LPR <= 8 ? 8 : 16);
    const long long rows = (long long)a.T * a.Hq;
    delta_kernel<T, D><<<(unsigned)((rows + 256 / LPR2 - 1) / (256 / LPR2)), 256, 0, a.stream>>>(
        (const T*)a.o, (const T*)a.dout, delta, (int)a.T, (int)a.Hq, a.osn, a.osh, a.dsn, a.dsh);
  }
  if (a.phases & NSA_BWD_PHASE_PREP) {
    int rc = build_reverse_index(a, L);
    if (rc != NSA_OK) return rc;
  }
  if (a.out_seg_off) {
    (void)hipMemcpyAsync(a.out_seg_off, ws + L.seg_off, (size_t)(n_seg + 1) * 4, hipMemcpyDeviceToDevice, a.stream);
    (void)hipMemcpyAsync(a.out_queries, ws + L.vals_out, (size_t)L.n_pairs * 4, hipMemcpyDeviceToDevice, a.stream);
  }
  if (a.phases & NSA_BWD_PHASE_DKDV) {
    DkdvParams p;
    p.q = a.q; p.k = a.k; p.v = a.v; p.dout = a.dout; p.lse = a.lse; p.delta = delta; p.cu = a.cu;
    p.cu_blk = (const int32_t*)(ws + L.cu_blk); p.seg_off = (const int32_t*)(ws + L.seg_off);
    p.chunk_off = (const int32_t*)(ws + L.chunk_off); p.queries = (const int32_t*)(ws + L.vals_out);
    p.partial = (float*)(ws + L.partial);
    p.total_len = (int)a.T; p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.max_blocks = (int)L.max_blocks; p.n_seg = n_seg;
    p.qsn = a.qsn; p.qsh = a.qsh; p.ksn = a.ksn; p.ksh = a.ksh; p.vsn = a.vsn; p.vsh = a.vsh; p.dsn = a.dsn; p.dsh = a.dsh;
    p.qk_scale = a.sm_scale * NSA_LOG2E; p.sm_scale = a.sm_scale;
    constexpr int NT = (BS / 16 < 4 ? BS / 16 : 4) * 64;
    dkdv_kernel<T, D, BS><<<(unsigned)L.max_items, NT, 0, a.stream>>>(p);
    dkdv_reduce_kernel<T, D, BS><<<(unsigned)n_seg, 256, 0, a.stream>>>(
        p.partial, p.chunk_off, a.cu, p.cu_blk, (int)a.B, (int)L.max_blocks, (T*)a.dk, (T*)a.dv, a.dksn, a.dksh, a.dvsn, a.dvsh);
  }
  if (a.phases & NSA_BWD_PHASE_DQ) {
    T* kt = (T*)(ws + L.kt);
    launch_block_transpose<T, D>((const T*)a.k, kt, a.cu, a.B, a.ksn, a.ksh, L.n_slots, a.Hkv, a.stream);
    DqParams p;
    p.q = a.q; p.k = a.k; p.v = a.v; p.kt = kt; p.dout = a.dout; p.lse = a.lse; p.delta = delta; p.idx = a.idx; p.cu = a.cu; p.dq = a.dq;
    p.total_len = (int)a.T; p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.topk = (int)a.topk; p.n_slots = (int)L.n_slots;
    p.n_items = (long long)a.T * GT * a.Hkv;
    p.qsn = a.qsn; p.qsh = a.qsh; p.ksn = a.ksn; p.ksh = a.ksh; p.vsn = a.vsn; p.vsh = a.vsh; p.dsn = a.dsn; p.dsh = a.dsh;
    p.ish = a.ish; p.isn = a.isn; p.isk = a.isk; p.dqsn = a.dqsn; p.dqsh = a.dqsh;
    p.qk_scale = a.sm_scale * NSA_LOG2E; p.sm_scale = a.sm_scale;
    long long n_wg = ((p.n_items + 3) / 4 + 7) / 8 * 8;
    dq_kernel<T, D, BS><<<(unsigned)n_wg, 256, 0, a.stream>>>(p);
  }
  return nsa_check_launch();
}

template <typename T, int D>
static int bwd_bs(const BwdArgs& a) {
  switch (a.bs) {
    case 32: return run_bwd<T, D, 32>(a);
    case 64: return run_bwd<T, D, 64>(a);
    case 128: return run_bwd<T, D, 128>(a);
    case 256: return run_bwd<T, D, 256>(a);
  }
  return NSA_ERR_UNSUPPORTED;
}
template <typename T>
static int bwd_d(const BwdArgs& a) {
  switch (a.D) {
    case 32: return bwd_bs<T, 32>(a);
    case 64: return bwd_bs<T, 64>(a);
    case 96: return bwd_bs<T, 96>(a);
    case 128: return bwd_bs<T, 128>(a);
  }
  return NSA_ERR_UNSUPPORTED;
}

extern "C" size_t nsa_topk_attn_bwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                                    int64_t head_dim, int64_t topk, int64_t block_size) {
  return bwd_layout(total_len, batch, num_q_heads, num_kv_heads, head_dim, topk, block_size).total;
}

extern "C" int64_t nsa_topk_reverse_index_segments(int64_t total_len, int64_t batch, int64_t num_kv_heads, int64_t block_size) {
  return num_kv_heads * (total_len / block_size + batch);
}

extern "C" int nsa_topk_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                                 const int32_t* topk_idx, const int32_t* cu_seqlens, void* dq, void* dk, void* dv,
                                 int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                 int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale, int dtype,
                                 void* workspace, size_t workspace_bytes, int32_t* out_segment_offsets, int32_t* out_queries,
                                 int phases, void* stream) {
  if (!q || !k || !v || !o || !dout || !lse || !topk_idx || !cu_seqlens || !dq || !dk || !dv || !strides || !workspace) return NSA_ERR_BAD_ARG;
  if (total_len <= 0 || batch <= 0 || num_kv_heads <= 0 || topk <= 0 || num_q_heads % num_kv_heads != 0) return NSA_ERR_BAD_ARG;
  if ((out_segment_offsets == nullptr) != (out_queries == nullptr)) return NSA_ERR_BAD_ARG;
  if (num_kv_heads * total_len * topk >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
  for (int i = 0; i < 10; i++) if (strides[i] % 8 != 0) return NSA_ERR_UNSUPPORTED;       // 16-byte loads
  for (int i = 13; i < 19; i++) if (strides[i] % 4 != 0) return NSA_ERR_UNSUPPORTED;      // 8-byte stores
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)dout) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) % 8 != 0 || (uintptr_t)workspace % 256 != 0) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_topk_attn_bwd_workspace_bytes(total_len, batch, num_q_heads, num_kv_heads, head_dim, topk, block_size)) return NSA_ERR_WORKSPACE;
  BwdArgs a;
  a.q = q; a.k = k; a.v = v; a.o = o; a.dout = dout; a.lse = lse; a.idx = topk_idx; a.cu = cu_seqlens; a.dq = dq; a.dk = dk; a.dv = dv;
  a.T = total_len; a.B = batch; a.Hq = num_q_heads; a.Hkv = num_kv_heads; a.D = head_dim; a.topk = topk; a.bs = block_size;
  a.qsn = strides[0]; a.qsh = strides[1]; a.ksn = strides[2]; a.ksh = strides[3]; a.vsn = strides[4]; a.vsh = strides[5];
  a.osn = strides[6]; a.osh = strides[7]; a.dsn = strides[8]; a.dsh = strides[9];
  a.ish = strides[10]; a.isn = strides[11]; a.isk = strides[12];
  a.dqsn = strides[13]; a.dqsh = strides[14]; a.dksn = strides[15]; a.dksh = strides[16]; a.dvsn = strides[17]; a.dvsh = strides[18];
  a.sm_scale = sm_scale; a.ws = (char*)workspace; a.stream = (hipStream_t)stream;
  a.out_seg_off = out_segment_offsets; a.out_queries = out_queries; a.phases = phases;
  if (dtype == NSA_BF16) return bwd_d<__bf16>(a);
  if (dtype == NSA_FP16) return bwd_d<_Float16>(a);
  return NSA_ERR_UNSUPPORTED;
}
