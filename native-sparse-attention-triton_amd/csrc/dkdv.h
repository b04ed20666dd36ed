// dK/dV pass shared by the block-sparse and the compressed attention backward.
//
// A workgroup keeps one block of BS keys (K and V rows) in registers, each wave 16*KT of them as
// MFMA B operands, and streams query rows through double-buffered LDS two (token, head-tile) row
// groups at a time.  P and dS leave the score MFMA already in B-operand layout; the transposed
// Q and dO fragments are read from LDS with ds_read_b64_tr_b16.  Work items are (segment,
// chunk of CHUNK_TOKENS queries); each writes an fp32 partial, a second kernel adds the chunks of
// a segment in order, so no atomics are needed and results are reproducible.
//   RANGE = false: the queries of a segment come from a sorted list (reverse index of topk_idx),
//                  key j is visible to a query at position pos iff j <= pos.
//   RANGE = true : the queries are the contiguous range [seg_off[s], seg_off[s+1]) of global token
//                  ids, keys are compressed tokens: visible iff j*st + ks - 1 <= pos.
#pragma once
#include "nsa_common.h"

static constexpr int CHUNK_TOKENS = 1024;  // queries per dK/dV work item

// Waves per dK/dV workgroup; each wave owns bs / (16 * waves) key tiles.  Every wave reads all
// staged query rows from LDS, so fewer waves would mean fewer LDS reads per token, but two waves
// of 32 keys need > 256 registers each (one wave per SIMD) and measured 17% slower than four.
constexpr int dkdv_waves(int bs) { return bs >= 64 ? 4 : bs / 16; }

// chunk_off = exclusive scan of ceil((seg_end - seg_begin)/CHUNK_TOKENS) over segments (single workgroup).
static __global__ __launch_bounds__(1024) void chunk_scan_kernel(const int32_t* __restrict__ seg_begin, const int32_t* __restrict__ seg_end, int n_seg,
                                                          int32_t* __restrict__ chunk_off) {
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int per = (n_seg + 1023) / 1024;
  const int j0 = tid * per, j1 = min(n_seg, j0 + per);
  int s = 0;
  for (int j = j0; j < j1; j++) s += (seg_end[j] - seg_begin[j] + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
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
    run += (seg_end[j] - seg_begin[j] + CHUNK_TOKENS - 1) / CHUNK_TOKENS;
  }
  if (tid == 1023) chunk_off[n_seg] = part[1023];
}

struct DkdvParams {
  const void* q; const void* k; const void* v; const void* dout; const float* lse; const float* delta;
  const int32_t* cu; const int32_t* cu_k; const int32_t* cu_blk; const int32_t* seg_begin; const int32_t* seg_end; const int32_t* chunk_off; const int32_t* queries;
  float* partial;
  int total_len, batch, Hkv, G, GT, max_blocks, n_seg, ks, st;
  int window;  // range mode: -1 compressed keys (key c seen from position c*st + ks - 1 on), >= 0 ordinary keys seen by [key, key + window], -2 every key seen by every position
  long long ksn, ksh, vsn, vsh;
  int qsn, qsh, dsn, dsh;  // element strides of q / dO (checked on the host to fit 31 bits)
  float qk_scale, sm_scale;
};

// GT1: the GQA group has at most 16 query heads (one head tile), which removes every run-time division
template <typename T, int D, int BS, bool RANGE, bool GT1>
__global__ __launch_bounds__(64 * dkdv_waves(BS), BS <= 64 ? 2 : 1) void dkdv_kernel(DkdvParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, NDT = D / 16, NSUB = BS / 16;
  constexpr int NW = dkdv_waves(BS);          // waves per workgroup
  constexpr int KT = NSUB / NW;               // 16-key tiles per wave
  constexpr int NT = NW * 64;
  constexpr int LD = lds_pitch(D);                   // padded LDS row (elements)
  __shared__ __attribute__((aligned(16))) T q_s[2][2][16][LD];
  __shared__ __attribute__((aligned(16))) T do_s[2][2][16][LD];
  __shared__ __attribute__((aligned(16))) float lse_s[2][32], delta_s[2][32];
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
  const int s0 = p.cu[b];                                  // first query token of the sequence
  const int k0 = p.cu_k[b], len = p.cu_k[b + 1] - k0;      // its keys
  const int key0 = (gb - p.cu_blk[b]) * BS;
  const int first = p.seg_begin[seg] + (item - p.chunk_off[seg]) * CHUNK_TOKENS;
  const int n_tok = min(CHUNK_TOKENS, p.seg_end[seg] - first);
  const int GT = GT1 ? 1 : p.GT;
  const int n_rg = n_tok * GT;                // row groups (token, head tile) in this chunk
  const int n_step = (n_rg + 1) / 2;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;

  // stationary operands: this wave's keys of K and V, B-operand layout (column = key)
  v8 kf[KT][NK], vf[KT][NK];
#pragma unroll
  for (int j = 0; j < KT; j++) {
    int row = key0 + 16 * (wave * KT + j) + li;
    row = row < len ? row : len - 1;
    const T* kp = (const T*)p.k + (long long)(k0 + row) * p.ksn + (long long)h * p.ksh + 8 * lg;
    const T* vp = (const T*)p.v + (long long)(k0 + row) * p.vsn + (long long)h * p.vsh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) { kf[j][kk] = ld16<v8>(kp + 32 * kk); vf[j][kk] = ld16<v8>(vp + 32 * kk); }
  }
  f32x4 dk[KT][NDT], dv[KT][NDT];
#pragma unroll
  for (int j = 0; j < KT; j++)
#pragma unroll
    for (int i = 0; i < NDT; i++) { dk[j][i] = f32x4{0.f, 0.f, 0.f, 0.f}; dv[j][i] = f32x4{0.f, 0.f, 0.f, 0.f}; }

  // staging: 2 row groups x 16 heads x D elements of Q and of dO per step, as 16-byte pieces.
  // Q and dO are handled by separate, fully unrolled loops: selecting the tensor at run time makes
  // the compiler fetch base pointers from a table and serialises the prefetch behind those loads.
  constexpr int PIECES = 2 * 16 * (D / 8);       // per tensor
  constexpr int PPT = (PIECES + NT - 1) / NT;
  // token ids of this chunk, read once (list mode); every later global load then has a single
  // level of dependence and can be issued two steps ahead
  __shared__ int tok_s[CHUNK_TOKENS];
  for (int i = tid; i < n_tok; i += NT) tok_s[i] = RANGE ? first + i : p.queries[first + i];
  __syncthreads();
  // fetch() is branch-free: loads are always issued (from a clamped, valid address) and the
  // validity mask is applied when the registers are written to LDS.  Conditional loads make the
  // compiler wait for every outstanding load at each join, which defeats the prefetch.
  struct Stage { uint4 qd[PPT]; uint4 dd[PPT]; float lse, delta; int pos; unsigned ok; };
  Stage stg[2];
  const T* const qbase = (const T*)p.q + (long long)h * p.G * p.qsh;
  const T* const dbase = (const T*)p.dout + (long long)h * p.G * p.dsh;
  const float* const lbase = p.lse + (long long)h * p.G * p.total_len;
  const float* const ebase = p.delta + (long long)h * p.G * p.total_len;

  auto fetch = [&](int step, Stage& sg) {
    unsigned ok = 0;
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = min(tid + u * NT, PIECES - 1);
      const int c = pc % (D / 8), hd = (pc / (D / 8)) % 16, rg = pc / (D / 8) / 16;
      const int r = step * 2 + rg;
      const int rc = min(r, n_rg - 1);
      const int t = tok_s[GT1 ? rc : rc / GT];
      const int hq = (GT1 ? 0 : (rc % GT) * 16) + hd;
      const int hc = min(hq, p.G - 1);
      sg.qd[u] = *reinterpret_cast<const uint4*>(qbase + (long long)t * p.qsn + (long long)hc * p.qsh + 8 * c);
      sg.dd[u] = *reinterpret_cast<const uint4*>(dbase + (long long)t * p.dsn + (long long)hc * p.dsh + 8 * c);
      ok |= (unsigned)(r < n_rg && hq < p.G) << u;
    }
    {
      const int rg = (tid >> 4) & 1, hd = tid & 15;
      const int r = step * 2 + rg;
      const int rc = min(r, n_rg - 1);
      const int t = tok_s[GT1 ? rc : rc / GT];
      const int hq = (GT1 ? 0 : (rc % GT) * 16) + hd;
      const int hc = min(hq, p.G - 1);
      sg.lse = lbase[(long long)hc * p.total_len + t];
      sg.delta = ebase[(long long)hc * p.total_len + t];
      sg.pos = r < n_rg ? t - s0 : -1;
      ok |= (unsigned)(r < n_rg && hq < p.G) << 31;
    }
    sg.ok = ok;
  };
  auto stash = [&](int buf, const Stage& sg) {
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = tid + u * NT;
      if (pc < PIECES) {
        const int c = pc % (D / 8), hd = (pc / (D / 8)) % 16, rg = pc / (D / 8) / 16;
        const unsigned m = 0u - ((sg.ok >> u) & 1u);  // all ones when the piece exists
        uint4 a = sg.qd[u], b2 = sg.dd[u];
        a.x &= m; a.y &= m; a.z &= m; a.w &= m;
        b2.x &= m; b2.y &= m; b2.z &= m; b2.w &= m;
        *reinterpret_cast<uint4*>(&q_s[buf][rg][hd][8 * c]) = a;
        *reinterpret_cast<uint4*>(&do_s[buf][rg][hd][8 * c]) = b2;
      }
    }
    if (tid < 32) {
      const bool ok = sg.ok >> 31;
      lse_s[buf][tid] = ok ? sg.lse : INFINITY;   // +inf -> probability 0 for rows that do not exist
      delta_s[buf][tid] = ok ? sg.delta : 0.f;
      if ((tid & 15) == 0) pos_s[buf][tid >> 4] = sg.pos;
    }
  };

  // one step of the pipeline with compile-time buffer / register-set roles (no run-time choice of
  // the register set, which would force copies that wait for the loads in flight)
  auto compute = [&](const int buf) {
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
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&lse_s[buf][tk * 16 + 4 * lg]);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(&delta_s[buf][tk * 16 + 4 * lg]);
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float l2 = l4[r];
          const float dl = d4[r];
          const bool vis = RANGE ? (key < len && (p.window == -2 || (key * p.st + p.ks - 1 <= pos && (p.window < 0 || key >= pos - p.window)))) : key <= pos;
          const float pr = fast_exp2(vis ? s[r] * p.qk_scale - l2 : -INFINITY);  // select, not a branch
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
  };
  auto pipeline_step = [&](int step, const int buf, Stage& refill, const Stage& ready) {
    // `refill` was written to LDS one step ago: reuse it for step + 2 (clamped: the tail re-loads the last step)
    fetch(min(step + 2, n_step - 1), refill);
    compute(buf);
    if (step + 1 < n_step) stash(buf ^ 1, ready);
    __syncthreads();
  };
  fetch(0, stg[0]);
  stash(0, stg[0]);
  fetch(min(1, n_step - 1), stg[1]);
  __syncthreads();
  for (int step = 0; step < n_step; step += 2) {
    pipeline_step(step, 0, stg[0], stg[1]);
    if (step + 1 < n_step) pipeline_step(step + 1, 1, stg[1], stg[0]);
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
  // blockIdx.y splits the 2*BS*D/4 output pieces of a segment so that short segments still fill the chip
  for (int i = blockIdx.y * 256 + threadIdx.x; i < 2 * BS * (D / 4); i += 256 * gridDim.y) {
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

