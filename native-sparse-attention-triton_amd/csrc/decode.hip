// Single-query (decode) attention over KV-cache slabs [B, max_len, Hkv, D]:
//   dense      - the first seqlens[b] rows (sliding-window ring, plain KV cache)
//   top-k      - the 64-token-aligned blocks named by topk_idx[h, b, :]
//   compressed - dense over the compressed slab, then per-key probabilities summed over the GQA
//                group -> overlap-weighted block scores -> forced init/local blocks -> top-k ids
// All three share one split-K body: a wave takes a chunk of up to 64 keys of one (sequence, kv-head) with the
// (up to 16) query heads of the group as MFMA columns and writes a partial (max, sum, O) triple to the
// workspace; a second kernel merges the partials.  The work is a few MiB per step, so the aim is few launches,
// few dependent round trips to memory and no barriers, not MFMA rate.  For a whole decode step the
// selected-block and the sliding-window branch share one partial launch, and one launch does both merges and
// the gated sum with the compressed branch; the compressed branch's merge runs inside its block-selection kernel.
#include "nsa_common.h"
#include <mutex>
#include <type_traits>

struct DecodeParams {
  const void* q; const void* k; const void* v; const int32_t* lens; const int32_t* idx;
  float* pm; float* pl; float* po;
  int B, Hkv, G, GT, n_chunks, topk, bs, slab_len;
  long long qsb, qsh, ksb, ksn, ksh, vsb, vsn, vsh, ish, isb, isk;
  float qk_scale;
};

// MODE 0: dense prefix, MODE 1: top-k blocks.  A wave owns one chunk of up to 64 keys and writes its own
// partial: nothing is exchanged between the waves of a workgroup, so the kernel has no barrier.  The V rows
// of the chunk are copied straight from global memory into a wave-private LDS tile (no registers, no
// ds_write) while the scores are formed; rows are 256 bytes, unpadded, with the 16-byte pieces of row r
// rotated by 2r positions so that the transposing reads hit every bank once.
template <int D> struct DecodeTile {
  static constexpr int CP = D > 64 ? 16 : (D > 32 ? 8 : 4);   // 16-byte pieces per staged row
  static constexpr int BYTES = 64 * CP * 16;                  // one wave's V tile
};

template <typename T, int D, int MODE>
__device__ __forceinline__ void decode_partial_body(const DecodeParams& p, int block_x, unsigned char* vs_all) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, NDT = D / 16;
  constexpr int CP = DecodeTile<D>::CP;
  constexpr int RPI = 64 / CP;                         // rows per 1 KiB wave-copy
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), li = lane & 15, lg = lane >> 4;
  const int chunk = block_x * 4 + wave, h = blockIdx.y / p.GT, gt = blockIdx.y % p.GT, b = blockIdx.z;
  if (chunk >= p.n_chunks) return;
  const int len = min(p.lens[b], p.slab_len);  // never read past the slab
  int k0, kend;  // keys [k0, kend) of this chunk are visible
  if (MODE == 0) {
    k0 = chunk * 64;
    kend = min(len, k0 + 64);
  } else {
    const int cpb = p.bs >= 64 ? p.bs / 64 : 1;
    const int e = chunk / cpb, sub = chunk % cpb;
    const int blk = p.idx[(long long)h * p.ish + (long long)b * p.isb + (long long)e * p.isk];
    const bool ok = blk >= 0 && len > 0 && blk <= (len - 1) / p.bs;
    k0 = ok ? blk * p.bs + 64 * sub : 0;
    kend = ok ? min(len, min(k0 + 64, (blk + 1) * p.bs)) : 0;
  }
  const long long slot = (((long long)b * p.Hkv + h) * p.GT + gt) * p.n_chunks + chunk;
  float* pm = p.pm + slot * 16;
  float* pl = p.pl + slot * 16;
  float* po = p.po + slot * 16 * D;
  if (kend <= k0) {  // nothing visible: neutral partial
    if (lane < 16) { pm[lane] = -INFINITY; pl[lane] = 0.f; }
    for (int i = lane; i < 16 * D; i += 64) po[i] = 0.f;
    return;
  }
  // V rows -> LDS, started first.  Rows past kend are copied from row k0 (slab rows past the length may hold
  // anything, and 0 * NaN would poison the sum); their probabilities are exactly 0.
  unsigned char* vs = vs_all + wave * DecodeTile<D>::BYTES;
#pragma unroll
  for (int i = 0; i < 64 / RPI; i++) {
    const int row = i * RPI + lane / CP;
    const int c = ((lane % CP) - 2 * row) & (CP - 1);
    const int cc = c < D / 8 ? c : D / 8 - 1;
    const int key = k0 + row < kend ? k0 + row : k0;
    dma16((const T*)p.v + (long long)b * p.vsb + (long long)key * p.vsn + (long long)h * p.vsh + 8 * cc, vs + i * 1024);
  }
  const int hq = gt * 16 + li;
  const bool has_head = hq < p.G;
  const T* qp = (const T*)p.q + (long long)b * p.qsb + (long long)(h * p.G + (has_head ? hq : 0)) * p.qsh + 8 * lg;
  v8 qf[NK], kf[4][NK];
#pragma unroll
  for (int kk = 0; kk < NK; kk++) qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int key = k0 + 16 * nt + li;
    const T* kp = (const T*)p.k + (long long)b * p.ksb + (long long)(key < kend ? key : k0) * p.ksn + (long long)h * p.ksh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) kf[nt][kk] = ld16<v8>(kp + 32 * kk);
  }
  f32x4 s[4];
  float mw = -INFINITY;
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < NK; kk++) c = E::mfma16(kf[nt][kk], qf[kk], c);
#pragma unroll
    for (int r = 0; r < 4; r++) {
      c[r] = (k0 + 16 * nt + 4 * lg + r) < kend ? c[r] * p.qk_scale : -INFINITY;
      mw = fmaxf(mw, c[r]);
    }
    s[nt] = c;
  }
  mw = column_max(mw);   // key k0 is visible, so the maximum is finite
  float lw = 0.f;
  v8 pf[2];
#pragma unroll
  for (int nt = 0; nt < 4; nt++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float x = fast_exp2(s[nt][r] - mw);
      lw += x;
      pf[nt >> 1][(nt & 1) * 4 + r] = (T)x;
    }
  lw = column_sum(lw);
  // O^T[d][head] = V^T[d][key] P^T[key][head]; the transposing read hands lane (li, lg) column li of rows
  // 4*lg..+3 of a 16-key tile
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  f32x4 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; dt++) {
    acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 2; c++) {
      s16x4 x[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const int row = 32 * c + 16 * u + 4 * lg + (li >> 2);
        const int at = (row * CP + ((2 * dt + ((li >> 1) & 1) + 2 * row) & (CP - 1))) * 16 + (li & 1) * 8;
        x[u] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vs + at));
      }
      const s16x8 z = {x[0][0], x[0][1], x[0][2], x[0][3], x[1][0], x[1][1], x[1][2], x[1][3]};
      acc[dt] = E::mfma16(__builtin_bit_cast(v8, z), pf[c], acc[dt]);
    }
  }
  if (lg == 0) { pm[li] = mw; pl[li] = lw; }
#pragma unroll
  for (int dt = 0; dt < NDT; dt++) *reinterpret_cast<f32x4*>(po + li * D + 16 * dt + 4 * lg) = acc[dt];
}

template <typename T, int D, int MODE>
__global__ __launch_bounds__(256) void decode_partial_kernel(DecodeParams p) {
  __shared__ __attribute__((aligned(256))) unsigned char v_s[4 * DecodeTile<D>::BYTES];
  decode_partial_body<T, D, MODE>(p, blockIdx.x, v_s);
}

// the partials of the selected-block branch (first blocks_a workgroups in x) and of a dense branch in one launch
template <typename T, int D>
__global__ __launch_bounds__(256) void decode_partial_pair_kernel(DecodeParams pa, DecodeParams pb, int blocks_a) {
  __shared__ __attribute__((aligned(256))) unsigned char v_s[4 * DecodeTile<D>::BYTES];
  if ((int)blockIdx.x < blocks_a) decode_partial_body<T, D, 1>(pa, blockIdx.x, v_s);
  else decode_partial_body<T, D, 0>(pb, blockIdx.x - blocks_a, v_s);
}

struct MergeScratch { float red_m[2], red_l[2]; float w_s[256]; };

// Merged output column d = tid of one (sequence, query head): sum_c w_c O_c[d] / sum_c w_c l_c; m_out / l_out
// receive the maximum and the sum.  Called by all threads of the workgroup (blockDim = 64 or 128).
template <int D>
__device__ __forceinline__ float decode_merge_body(const DecodeParams& p, int hq_all, int b, MergeScratch& sh, float& m_out, float& l_out) {
  constexpr int WCAP = 256;  // chunk weights kept in LDS at a time
  const int tid = threadIdx.x, nt = blockDim.x, wave = tid >> 6, nw = nt >> 6;
  const int h = hq_all / p.G, hq = hq_all % p.G, gt = hq / 16, col = hq % 16;
  const long long base = (((long long)b * p.Hkv + h) * p.GT + gt) * p.n_chunks;
  float m = -INFINITY;
  for (int c = tid; c < p.n_chunks; c += nt) m = fmaxf(m, p.pm[(base + c) * 16 + col]);
  m = wave_max_f32(m);
  if ((tid & 63) == 0) sh.red_m[wave] = m;
  __syncthreads();
  m = nw == 2 ? fmaxf(sh.red_m[0], sh.red_m[1]) : sh.red_m[0];
  float l = 0.f, acc = 0.f;  // acc: this thread's output column d = tid (nt >= D is guaranteed by the launch)
  for (int c0 = 0; c0 < p.n_chunks; c0 += WCAP) {
    const int n = min(WCAP, p.n_chunks - c0);
    if (c0 > 0) __syncthreads();   // the previous batch of weights has been used
    for (int c = tid; c < n; c += nt) {
      const float mc = p.pm[(base + c0 + c) * 16 + col];
      const float w = mc != -INFINITY ? fast_exp2(mc - m) : 0.f;
      sh.w_s[c] = w;
      l += w * p.pl[(base + c0 + c) * 16 + col];
    }
    __syncthreads();
    if (tid < D) {
#pragma unroll 8
      for (int c = 0; c < n; c++) acc += p.po[((base + c0 + c) * 16 + col) * D + tid] * sh.w_s[c];
    }
  }
  l = wave_sum_f32(l);
  if ((tid & 63) == 0) sh.red_l[wave] = l;
  __syncthreads();
  l = nw == 2 ? sh.red_l[0] + sh.red_l[1] : sh.red_l[0];
  m_out = m; l_out = l;
  return l > 0.f ? acc / l : 0.f;
}

// merge the chunk partials of one (sequence, query head); optionally keep the base-2 LSE.  The chunk maxima and
// sums are read by different threads (independent loads, not a serial chain) and reduced inside each wave by
// lane exchanges; two barriers per call instead of a barrier tree.  The per-chunk weights go through LDS.
template <typename T, int D>
__global__ void decode_merge_kernel(DecodeParams p, T* __restrict__ o, long long osb, long long osh, float* __restrict__ lse) {
  __shared__ MergeScratch sh;
  const int hq_all = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  float m, l;
  const float val = decode_merge_body<D>(p, hq_all, b, sh, m, l);
  if (tid < D) o[(long long)b * osb + (long long)hq_all * osh + tid] = (T)val;
  if (lse && tid == 0) lse[(long long)b * p.Hkv * p.G + hq_all] = l > 0.f ? m + fast_log2(l) : INFINITY;
}

// Merges of the selected-block branch (pa) and of the sliding-window branch (pb), and the gated sum with the
// compressed branch, out = g0 * cmp + g1 * sel + g2 * win, every product and partial sum rounded to the element
// type in that order (the arithmetic of the tensor expression); the two branch outputs are stored as well.
struct GateParams {
  const void* cmp; const void* gate; void* out; void* o_a; void* o_b;
  long long csb, csh, gsb, gsh, gsk, osb, osh, asb, ash, bsb, bsh;
};
template <typename T, int D>
__global__ void decode_merge_pair_gate_kernel(DecodeParams pa, DecodeParams pb, GateParams g) {
  __shared__ MergeScratch sh;
  const int hq_all = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  float m, l;
  const float va = decode_merge_body<D>(pa, hq_all, b, sh, m, l);
  __syncthreads();   // the scratch is reused
  const float vb = decode_merge_body<D>(pb, hq_all, b, sh, m, l);
  if (tid < D) {
    const T ta = (T)va, tb = (T)vb;
    ((T*)g.o_a)[(long long)b * g.asb + (long long)hq_all * g.ash + tid] = ta;
    ((T*)g.o_b)[(long long)b * g.bsb + (long long)hq_all * g.bsh + tid] = tb;
    const T* gp = (const T*)g.gate + (long long)b * g.gsb + (long long)hq_all * g.gsh;
    const float g0 = (float)gp[0], g1 = (float)gp[g.gsk], g2 = (float)gp[2 * g.gsk];
    const float c = (float)((const T*)g.cmp)[(long long)b * g.csb + (long long)hq_all * g.csh + tid];
    const float x = rounded<T>(g0 * c), y = rounded<T>(g1 * (float)ta), z = rounded<T>(g2 * (float)tb);
    ((T*)g.out)[(long long)b * g.osb + (long long)hq_all * g.osh + tid] = (T)(rounded<T>(x + y) + z);
  }
}

// ------------------------------------------------------------------------------------------
// compressed decode: probabilities -> block scores -> top-k ids
struct ScoreParams {
  const void* q; const void* k; const float* lse; const int32_t* seqlens; const int32_t* clens; float* score; int32_t* out_idx;
  int B, Hkv, G, GT, slab_len, ks, st, bs, init_blocks, local_blocks, k_out, max_blocks, full_blocks;
  long long qsb, qsh, ksb, ksn, ksh, osh, osb, osk;
  float qk_scale;
  // merge of the attention partials, done here when selection follows (one launch less, and the LSE never
  // leaves the chip): partials as in DecodeParams, o = attention output [B, Hq, D]
  const float* pm; const float* pl; const float* po; int n_chunks; void* o; long long oob, ooh;
};

static constexpr int MAX_SCORE_BLOCKS = 8192, MAX_SCORE_GROUP = 128;

// One workgroup of SEL_NT threads per (kv-head, sequence): the work is a chain of short dependent phases, so
// the aim is few round trips to memory and few barriers, not throughput.
static constexpr int SEL_NT = 1024, SEL_NW = SEL_NT / 64, SEL_LDS_SCORES = 8192, SEL_REG_BLOCKS = 16;

template <typename T, int D>
__global__ __launch_bounds__(SEL_NT) void decode_score_select_kernel(ScoreParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32;
  __shared__ float bscore[MAX_SCORE_BLOCKS];
  __shared__ int picked[64];
  __shared__ long long wave_best[2][SEL_NW];
  const int h = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), li = lane & 15, lg = lane >> 4;
  const int lc = min(p.clens[b], p.slab_len);
  const int qb = (p.seqlens[b] - 1) / p.bs;
  // per-key scores stay in LDS when they fit (a round trip to memory less), else in the workspace
  __shared__ float score_s[SEL_LDS_SCORES];
  __shared__ float lse_s[MAX_SCORE_GROUP];
  float* score = lc <= SEL_LDS_SCORES ? score_s : p.score + ((long long)b * p.Hkv + h) * p.slab_len;
  // phase 0: merge the chunk partials of this kv-head's query heads, one wave per head: the lanes share out
  // the chunks for the maximum and the sum, then each lane owns output columns lane, lane + 64
  for (int hq = wave; hq < p.G; hq += SEL_NW) {
    const int col = hq % 16;
    const long long base = (((long long)b * p.Hkv + h) * p.GT + hq / 16) * p.n_chunks;
    float m = -INFINITY;
    for (int c = lane; c < p.n_chunks; c += 64) m = fmaxf(m, p.pm[(base + c) * 16 + col]);
    m = wave_max_f32(m);
    float l = 0.f;
    for (int c = lane; c < p.n_chunks; c += 64) {
      const float mc = p.pm[(base + c) * 16 + col];
      if (mc != -INFINITY) l += fast_exp2(mc - m) * p.pl[(base + c) * 16 + col];
    }
    l = wave_sum_f32(l);
    float acc[(D + 63) / 64];
#pragma unroll
    for (int u = 0; u < (D + 63) / 64; u++) acc[u] = 0.f;
#pragma unroll 4
    for (int c = 0; c < p.n_chunks; c++) {
      const float mc = p.pm[(base + c) * 16 + col];
      const float w = mc != -INFINITY ? fast_exp2(mc - m) : 0.f;
#pragma unroll
      for (int u = 0; u < (D + 63) / 64; u++)
        if (lane + 64 * u < D) acc[u] += p.po[((base + c) * 16 + col) * D + lane + 64 * u] * w;
    }
    T* orow = (T*)p.o + (long long)b * p.oob + (long long)(h * p.G + hq) * p.ooh;
#pragma unroll
    for (int u = 0; u < (D + 63) / 64; u++)
      if (lane + 64 * u < D) orow[lane + 64 * u] = (T)(l > 0.f ? acc[u] / l : 0.f);
    if (lane == 0) lse_s[hq] = l > 0.f ? m + fast_log2(l) : INFINITY;
  }
  __syncthreads();
  // phase A: score[c] = sum over the group's heads of exp2(s*scale - lse); a wave takes two 16-key tiles per
  // trip and issues the K loads of both before it uses either
  for (int sub0 = 2 * wave; sub0 * 16 < lc; sub0 += 2 * SEL_NW) {
    v8 kf[2][NK];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int key = (sub0 + u) * 16 + li;
      const int row = key < lc ? key : 0;
      const T* kp = (const T*)p.k + (long long)b * p.ksb + (long long)row * p.ksn + (long long)h * p.ksh + 8 * lg;
#pragma unroll
      for (int kk = 0; kk < NK; kk++) kf[u][kk] = ld16<v8>(kp + 32 * kk);
    }
    f32x4 tot[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int gt = 0; gt < p.GT; gt++) {
      const int hq = gt * 16 + li;
      const bool has_head = hq < p.G;
      const T* qp = (const T*)p.q + (long long)b * p.qsb + (long long)(h * p.G + (has_head ? hq : 0)) * p.qsh + 8 * lg;
      const float l2 = has_head ? lse_s[hq] : INFINITY;
      v8 qf[NK];
#pragma unroll
      for (int kk = 0; kk < NK; kk++) qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
#pragma unroll
      for (int u = 0; u < 2; u++) {
        f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) sc = E::mfma16(kf[u][kk], qf[kk], sc);
#pragma unroll
        for (int r = 0; r < 4; r++) {
          float x = ((sub0 + u) * 16 + 4 * lg + r) < lc ? fast_exp2(sc[r] * p.qk_scale - l2) : 0.f;
          // sum over the 16 heads (the lanes of a row), in a fixed order
          x += dpp_f32<0xB1>(x); x += dpp_f32<0x4E>(x); x += dpp_f32<0x141>(x); x += dpp_f32<0x140>(x);
          tot[u][r] += x;
        }
      }
    }
    if (li == 0) {
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int r = 0; r < 4; r++) if ((sub0 + u) * 16 + 4 * lg + r < lc) score[(sub0 + u) * 16 + 4 * lg + r] = tot[u][r];
    }
  }
  __syncthreads();
  // phase B: block scores
  const int a = p.ks / p.st, rr = p.bs / p.st, pad = a - 1;
  for (int blk = tid; blk < p.max_blocks; blk += SEL_NT) {
    float v = 0.f;
    if (blk < p.full_blocks) {
      for (int o = 0; o < a + rr - 1; o++) {
        const int c = blk * rr + o - pad;
        const int w = min(min(o, a + rr - 2 - o), min(a - 1, rr - 1)) + 1;
        if (c >= 0 && c < lc) v += (float)w * score[c];
      }
    }
    if (v != v) v = 0.f;
    if (blk < p.init_blocks || (blk <= qb && blk > qb - p.local_blocks)) v = INFINITY;
    bscore[blk] = v;
  }
  // phase C: k_out rounds of (largest value, smallest index).
  if (p.max_blocks <= 64 * SEL_REG_BLOCKS) {
    // up to 1024 blocks: one wave keeps every candidate in registers (lane l owns blocks l, l + 64, ...), so a
    // round is that wave's lane exchanges and nothing else - no LDS traffic, no barrier; the ids then leave
    // in ascending order straight from the registers (ballot + prefix count per 64 blocks)
    __syncthreads();
    if (wave != 0) return;
    int32_t* out = p.out_idx + (long long)h * p.osh + (long long)b * p.osb;
    auto pick = [&](auto nreg_c) __attribute__((always_inline)) {
      constexpr int NREG = decltype(nreg_c)::value;
      float cand[NREG];
#pragma unroll
      for (int i = 0; i < NREG; i++) cand[i] = lane + 64 * i < p.max_blocks ? bscore[lane + 64 * i] : -3.f;
      float bv = -1.f;
      int bi = 0x7fffffff;
#pragma unroll
      for (int i = 0; i < NREG; i++)
        if (cand[i] > bv) { bv = cand[i]; bi = lane + 64 * i; }
      for (int round = 0; round < p.k_out; round++) {
        const int win = candidate_index(wave_max_i64(candidate_key(bv, bi)));
        if (bi == win) {
          bv = -1.f; bi = 0x7fffffff;
#pragma unroll
          for (int i = 0; i < NREG; i++) {
            if (lane + 64 * i == win) cand[i] = -2.f;
            if (cand[i] > bv) { bv = cand[i]; bi = lane + 64 * i; }
          }
        }
      }
      // winners beyond the query's own block (possible only when fewer than k_out blocks are causal) sort
      // last and are written as -1
      int base = 0;
#pragma unroll
      for (int i = 0; i < NREG; i++) {
        const int blk = lane + 64 * i;
        const bool taken = cand[i] == -2.f && blk <= qb;
        const unsigned long long mask = __ballot(taken);
        if (taken) out[(long long)(base + __popcll(mask & ((1ull << lane) - 1ull))) * p.osk] = blk;
        base += __popcll(mask);
      }
      for (int i = base + lane; i < p.k_out; i += 64) out[(long long)i * p.osk] = -1;
    };
    if (p.max_blocks <= 128) pick(std::integral_constant<int, 2>{});
    else if (p.max_blocks <= 256) pick(std::integral_constant<int, 4>{});
    else pick(std::integral_constant<int, SEL_REG_BLOCKS>{});
    return;
  } else {
    // A thread only ever reads the entries it wrote in phase B (blk = tid mod SEL_NT), and it is the owner
    // that retires a winner, so no barrier is needed around bscore; the wave maxima alternate between two
    // LDS rows, which leaves one barrier per round.
    for (int round = 0; round < p.k_out; round++) {
      float bv = -1.f;
      int bi = 0x7fffffff;
      for (int blk = tid; blk < p.max_blocks; blk += SEL_NT) {
        const float v = bscore[blk];
        if (v > bv) { bv = v; bi = blk; }
      }
      const long long mine = wave_max_i64(candidate_key(bv, bi));
      if (lane == 0) wave_best[round & 1][wave] = mine;
      __syncthreads();
      long long m = wave_best[round & 1][0];
      for (int w = 1; w < SEL_NW; w++) { const long long o = wave_best[round & 1][w]; m = o > m ? o : m; }
      const int win = candidate_index(m);
      if (tid == 0) picked[round] = win;
      if ((win % SEL_NT) == tid) bscore[win] = -2.f;
    }
  }
  // ascending order, ids beyond the query's block become -1 at the tail
  if (tid == 0) {
    int32_t* out = p.out_idx + (long long)h * p.osh + (long long)b * p.osb;
    for (int i = 1; i < p.k_out; i++) {  // insertion sort of <= 64 ids
      int x = picked[i], j = i - 1;
      while (j >= 0 && picked[j] > x) { picked[j + 1] = picked[j]; j--; }
      picked[j + 1] = x;
    }
    for (int i = 0; i < p.k_out; i++) out[(long long)i * p.osk] = picked[i] > qb ? -1 : picked[i];
  }
}

// ------------------------------------------------------------------------------------------
static inline int chunks_for(int mode, int64_t slab_len, int64_t topk, int64_t bs) {
  return mode == 0 ? (int)((slab_len + 63) / 64) : (int)(topk * (bs >= 64 ? bs / 64 : 1));
}

static size_t decode_partial_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int n_chunks) {
  const int64_t GT = (Hq / Hkv + 15) / 16;
  return (size_t)(B * Hkv * GT * n_chunks) * 16 * (size_t)(D + 2) * 4;
}

template <typename T, int D>
static int run_decode(int mode, DecodeParams& p, void* o, long long osb, long long osh, float* lse, char* ws, hipStream_t s) {
  const size_t n = (size_t)p.B * p.Hkv * p.GT * p.n_chunks * 16;
  p.pm = (float*)ws; p.pl = p.pm + n; p.po = p.pl + n;
  dim3 grid((unsigned)((p.n_chunks + 3) / 4), (unsigned)(p.Hkv * p.GT), (unsigned)p.B);
  if (mode == 0) decode_partial_kernel<T, D, 0><<<grid, 256, 0, s>>>(p);
  else decode_partial_kernel<T, D, 1><<<grid, 256, 0, s>>>(p);
  decode_merge_kernel<T, D><<<dim3((unsigned)(p.Hkv * p.G), (unsigned)p.B), D <= 64 ? 64 : 128, 0, s>>>(p, (T*)o, osb, osh, lse);
  return nsa_check_launch();
}

#define DECODE_DISPATCH(CALL)                                                   \
  switch (head_dim) {                                                           \
    case 32: return dtype == NSA_BF16 ? CALL(__bf16, 32) : CALL(_Float16, 32);  \
    case 64: return dtype == NSA_BF16 ? CALL(__bf16, 64) : CALL(_Float16, 64);  \
    case 96: return dtype == NSA_BF16 ? CALL(__bf16, 96) : CALL(_Float16, 96);  \
    case 128: return dtype == NSA_BF16 ? CALL(__bf16, 128) : CALL(_Float16, 128); \
  }                                                                             \
  return NSA_ERR_UNSUPPORTED;

static int fill_decode(DecodeParams& p, const void* q, const void* k, const void* v, const int32_t* lens, int64_t B, int64_t Hq,
                       int64_t Hkv, int64_t slab_len, const int64_t* st, float sm_scale) {
  if (!q || !k || !v || !lens || !st || B <= 0 || Hkv <= 0 || Hq % Hkv != 0 || slab_len <= 0) return NSA_ERR_BAD_ARG;
  for (int i = 0; i < 8; i++) if (st[i] % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  p.q = q; p.k = k; p.v = v; p.lens = lens; p.idx = nullptr; p.B = (int)B; p.Hkv = (int)Hkv; p.G = (int)(Hq / Hkv);
  p.GT = (p.G + 15) / 16; p.slab_len = (int)slab_len; p.topk = 0; p.bs = 64;
  p.qsb = st[0]; p.qsh = st[1]; p.ksb = st[2]; p.ksn = st[3]; p.ksh = st[4]; p.vsb = st[5]; p.vsn = st[6]; p.vsh = st[7];
  p.ish = p.isb = p.isk = 0; p.qk_scale = sm_scale * NSA_LOG2E;
  return NSA_OK;
}

extern "C" size_t nsa_dense_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len) {
  return decode_partial_bytes(batch, num_q_heads, num_kv_heads, head_dim, chunks_for(0, slab_len, 0, 64));
}

extern "C" int nsa_dense_decode(const void* q, const void* k, const void* v, const int32_t* seqlens, void* o, int64_t batch,
                                int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len,
                                const int64_t* strides, float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  DecodeParams p;
  int rc = fill_decode(p, q, k, v, seqlens, batch, num_q_heads, num_kv_heads, slab_len, strides, sm_scale);
  if (rc != NSA_OK) return rc;
  if (!o || !workspace) return NSA_ERR_BAD_ARG;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_dense_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, slab_len)) return NSA_ERR_WORKSPACE;
  p.n_chunks = chunks_for(0, slab_len, 0, 64);
  const long long osb = strides[8], osh = strides[9];
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) run_decode<T, D>(0, p, o, osb, osh, nullptr, (char*)workspace, s)
  DECODE_DISPATCH(CALL)
#undef CALL
}

extern "C" size_t nsa_topk_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                                  int64_t topk, int64_t block_size) {
  return decode_partial_bytes(batch, num_q_heads, num_kv_heads, head_dim, chunks_for(1, 0, topk, block_size));
}

extern "C" int nsa_topk_decode(const void* q, const void* k, const void* v, const int32_t* topk_idx, const int32_t* seqlens, void* o,
                               int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len,
                               int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale, int dtype,
                               void* workspace, size_t workspace_bytes, void* stream) {
  DecodeParams p;
  int rc = fill_decode(p, q, k, v, seqlens, batch, num_q_heads, num_kv_heads, slab_len, strides, sm_scale);
  if (rc != NSA_OK) return rc;
  if (!o || !workspace || !topk_idx || topk <= 0) return NSA_ERR_BAD_ARG;
  if (block_size != 32 && block_size != 64 && block_size != 128 && block_size != 256) return NSA_ERR_UNSUPPORTED;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_topk_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, topk, block_size)) return NSA_ERR_WORKSPACE;
  p.idx = topk_idx; p.topk = (int)topk; p.bs = (int)block_size;
  p.ish = strides[10]; p.isb = strides[11]; p.isk = strides[12];
  p.n_chunks = chunks_for(1, 0, topk, block_size);
  const long long osb = strides[8], osh = strides[9];
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) run_decode<T, D>(1, p, o, osb, osh, nullptr, (char*)workspace, s)
  DECODE_DISPATCH(CALL)
#undef CALL
}

// ------------------------------------------------------------------------------------------
// nsa_topk_decode for callers that cannot allocate: the split-K partials live in a file-scope device array
// instead of a caller workspace.  Every GPU the library runs on holds its own copy of the array until the
// process ends; its device address is looked up once per device (the array's name in host code is only a
// handle for that lookup, never an address a kernel may be given).
static constexpr size_t STATIC_SCRATCH_BYTES = NSA_TOPK_DECODE_STATIC_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
static constexpr int STATIC_MAX_DEVICES = 64;
static void* scratch_addr[STATIC_MAX_DEVICES];   // per device, filled on the first call with that device current
static std::mutex scratch_mutex;

static int static_scratch(void** out, hipStream_t stream) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return NSA_ERR_LAUNCH;
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (!scratch_addr[dev]) {
    // the address lookup is not a stream operation: made while the caller's stream records a graph it would fail
    // or break the recording, so that case is refused with a code of its own before anything is attempted
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) return NSA_ERR_LAUNCH;
    if (capturing != hipStreamCaptureStatusNone) return NSA_ERR_NOT_READY;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return NSA_ERR_LAUNCH;
    scratch_addr[dev] = ptr;
  }
  *out = scratch_addr[dev];
  return NSA_OK;
}

extern "C" int nsa_topk_decode_static(const void* q, const void* k, const void* v, const int32_t* topk_idx, const int32_t* seqlens,
                                      void* o, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                      int64_t slab_len, int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale,
                                      int dtype, void* stream) {
  if (batch <= 0 || num_kv_heads <= 0 || num_q_heads <= 0 || num_q_heads % num_kv_heads != 0 || topk <= 0) return NSA_ERR_BAD_ARG;
  if (block_size != 32 && block_size != 64 && block_size != 128 && block_size != 256) return NSA_ERR_UNSUPPORTED;
  // sizes whose partials do not fit the array are refused before anything is looked up or launched
  if (nsa_topk_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, topk, block_size) > STATIC_SCRATCH_BYTES)
    return NSA_ERR_WORKSPACE;
  void* ws = nullptr;
  const int rc = static_scratch(&ws, (hipStream_t)stream);
  if (rc != NSA_OK) return rc;
  // the partial kernel writes every (m, l, O) slot the merge kernel reads, so nothing left behind by an
  // earlier call needs clearing
  return nsa_topk_decode(q, k, v, topk_idx, seqlens, o, batch, num_q_heads, num_kv_heads, head_dim, slab_len, topk, block_size,
                         strides, sm_scale, dtype, ws, STATIC_SCRATCH_BYTES, stream);
}

static size_t cmp_decode_partial(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t slab_len) {
  return (decode_partial_bytes(B, Hq, Hkv, D, chunks_for(0, slab_len, 0, 64)) + 255) & ~(size_t)255;
}

extern "C" size_t nsa_cmp_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len) {
  return cmp_decode_partial(batch, num_q_heads, num_kv_heads, head_dim, slab_len) + (size_t)batch * num_q_heads * 4 + 256 +
         (size_t)batch * num_kv_heads * slab_len * 4;
}

template <typename T, int D>
static int run_cmp_decode(DecodeParams& p, ScoreParams& sp, void* o, long long osb, long long osh, char* ws, size_t part_bytes, hipStream_t s) {
  float* lse = (float*)(ws + part_bytes);
  float* score = (float*)(ws + part_bytes + (((size_t)p.B * p.Hkv * p.G * 4 + 255) & ~(size_t)255));
  if (!sp.out_idx) return run_decode<T, D>(0, p, o, osb, osh, lse, ws, s);
  // with selection: partials, then one kernel that merges them, scores the blocks and picks
  const size_t n = (size_t)p.B * p.Hkv * p.GT * p.n_chunks * 16;
  p.pm = (float*)ws; p.pl = p.pm + n; p.po = p.pl + n;
  decode_partial_kernel<T, D, 0><<<dim3((unsigned)((p.n_chunks + 3) / 4), (unsigned)(p.Hkv * p.GT), (unsigned)p.B), 256, 0, s>>>(p);
  sp.lse = lse; sp.score = score;
  sp.pm = p.pm; sp.pl = p.pl; sp.po = p.po; sp.n_chunks = p.n_chunks; sp.o = o; sp.oob = osb; sp.ooh = osh;
  decode_score_select_kernel<T, D><<<dim3((unsigned)p.Hkv, (unsigned)p.B), SEL_NT, 0, s>>>(sp);
  return nsa_check_launch();
}

extern "C" int nsa_cmp_decode(const void* q, const void* k, const void* v, const int32_t* seqlens, const int32_t* compress_seqlens,
                              void* o, int32_t* out_topk_idx, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                              int64_t head_dim, int64_t slab_len, int64_t kernel_size, int64_t kernel_stride, int64_t block_size,
                              int64_t k_out, int64_t max_seqlen, int64_t init_blocks, int64_t local_blocks, const int64_t* strides,
                              float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  DecodeParams p;
  int rc = fill_decode(p, q, k, v, compress_seqlens, batch, num_q_heads, num_kv_heads, slab_len, strides, sm_scale);
  if (rc != NSA_OK) return rc;
  if (!o || !workspace || !seqlens) return NSA_ERR_BAD_ARG;
  if (kernel_stride <= 0 || kernel_size % kernel_stride != 0 || block_size % kernel_size != 0) return NSA_ERR_BAD_ARG;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_cmp_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, slab_len)) return NSA_ERR_WORKSPACE;
  const int64_t max_blocks = (max_seqlen + block_size - 1) / block_size;
  if (out_topk_idx && (k_out <= 0 || k_out > 64 || k_out > max_blocks || max_blocks > MAX_SCORE_BLOCKS || p.G > MAX_SCORE_GROUP)) return NSA_ERR_UNSUPPORTED;
  p.n_chunks = chunks_for(0, slab_len, 0, 64);
  ScoreParams sp;
  sp.q = q; sp.k = k; sp.seqlens = seqlens; sp.clens = compress_seqlens; sp.out_idx = out_topk_idx;
  sp.B = p.B; sp.Hkv = p.Hkv; sp.G = p.G; sp.GT = p.GT; sp.slab_len = p.slab_len; sp.ks = (int)kernel_size; sp.st = (int)kernel_stride;
  sp.bs = (int)block_size; sp.init_blocks = (int)init_blocks; sp.local_blocks = (int)local_blocks; sp.k_out = (int)k_out;
  sp.max_blocks = (int)max_blocks; sp.full_blocks = (int)(max_seqlen / block_size);
  sp.qsb = p.qsb; sp.qsh = p.qsh; sp.ksb = p.ksb; sp.ksn = p.ksn; sp.ksh = p.ksh;
  sp.osh = strides[10]; sp.osb = strides[11]; sp.osk = strides[12]; sp.qk_scale = p.qk_scale;
  const long long osb = strides[8], osh = strides[9];
  const size_t part = cmp_decode_partial(batch, num_q_heads, num_kv_heads, head_dim, slab_len);
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) run_cmp_decode<T, D>(p, sp, o, osb, osh, (char*)workspace, part, s)
  DECODE_DISPATCH(CALL)
#undef CALL
}

// ------------------------------------------------------------------------------------------
// selected-block branch + sliding-window branch + gate in two launches
extern "C" size_t nsa_decode_branches_gate_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                                           int64_t window_rows, int64_t topk, int64_t block_size) {
  const size_t a = (decode_partial_bytes(batch, num_q_heads, num_kv_heads, head_dim, chunks_for(1, 0, topk, block_size)) + 255) & ~(size_t)255;
  return a + decode_partial_bytes(batch, num_q_heads, num_kv_heads, head_dim, chunks_for(0, window_rows, 0, 64));
}

template <typename T, int D>
static int run_branches_gate(DecodeParams& pa, DecodeParams& pb, const GateParams& g, char* ws, size_t bytes_a, hipStream_t s) {
  const size_t na = (size_t)pa.B * pa.Hkv * pa.GT * pa.n_chunks * 16, nb = (size_t)pb.B * pb.Hkv * pb.GT * pb.n_chunks * 16;
  pa.pm = (float*)ws; pa.pl = pa.pm + na; pa.po = pa.pl + na;
  pb.pm = (float*)(ws + bytes_a); pb.pl = pb.pm + nb; pb.po = pb.pl + nb;
  const int blocks_a = (pa.n_chunks + 3) / 4, blocks_b = (pb.n_chunks + 3) / 4;
  decode_partial_pair_kernel<T, D><<<dim3((unsigned)(blocks_a + blocks_b), (unsigned)(pa.Hkv * pa.GT), (unsigned)pa.B), 256, 0, s>>>(pa, pb, blocks_a);
  decode_merge_pair_gate_kernel<T, D><<<dim3((unsigned)(pa.Hkv * pa.G), (unsigned)pa.B), D <= 64 ? 64 : 128, 0, s>>>(pa, pb, g);
  return nsa_check_launch();
}

extern "C" int nsa_decode_branches_gate(const void* q, const void* sparse_k, const void* sparse_v, const int32_t* sparse_len,
                                        const int32_t* topk_idx, const void* window_k, const void* window_v, const int32_t* window_len,
                                        const void* cmp_out, const void* gate, void* out, void* o_topk, void* o_window, int64_t batch,
                                        int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t sparse_rows,
                                        int64_t window_rows, int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale,
                                        int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (!strides) return NSA_ERR_BAD_ARG;
  const int64_t sa[8] = {strides[0], strides[1], strides[2], strides[3], strides[4], strides[5], strides[6], strides[7]};
  const int64_t sb[8] = {strides[0], strides[1], strides[11], strides[12], strides[13], strides[14], strides[15], strides[16]};
  DecodeParams pa, pb;
  int rc = fill_decode(pa, q, sparse_k, sparse_v, sparse_len, batch, num_q_heads, num_kv_heads, sparse_rows, sa, sm_scale);
  if (rc != NSA_OK) return rc;
  rc = fill_decode(pb, q, window_k, window_v, window_len, batch, num_q_heads, num_kv_heads, window_rows, sb, sm_scale);
  if (rc != NSA_OK) return rc;
  if (!topk_idx || !cmp_out || !gate || !out || !o_topk || !o_window || !workspace || topk <= 0) return NSA_ERR_BAD_ARG;
  if (block_size != 32 && block_size != 64 && block_size != 128 && block_size != 256) return NSA_ERR_UNSUPPORTED;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_decode_branches_gate_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, window_rows, topk, block_size))
    return NSA_ERR_WORKSPACE;
  pa.idx = topk_idx; pa.topk = (int)topk; pa.bs = (int)block_size;
  pa.ish = strides[8]; pa.isb = strides[9]; pa.isk = strides[10];
  pa.n_chunks = chunks_for(1, 0, topk, block_size);
  pb.n_chunks = chunks_for(0, window_rows, 0, 64);
  GateParams g;
  g.cmp = cmp_out; g.gate = gate; g.out = out; g.o_a = o_topk; g.o_b = o_window;
  g.csb = strides[17]; g.csh = strides[18]; g.gsb = strides[19]; g.gsh = strides[20]; g.gsk = strides[21];
  g.osb = strides[22]; g.osh = strides[23]; g.asb = strides[24]; g.ash = strides[25]; g.bsb = strides[26]; g.bsh = strides[27];
  const size_t bytes_a = (decode_partial_bytes(batch, num_q_heads, num_kv_heads, head_dim, pa.n_chunks) + 255) & ~(size_t)255;
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) run_branches_gate<T, D>(pa, pb, g, (char*)workspace, bytes_a, s)
  DECODE_DISPATCH(CALL)
#undef CALL
}
