// Attention of queries over compressed keys/values (compressed_attention), forward, block
// selection and backward.
//
// Tiling: a workgroup owns 16 (forward, selection) or 8 (dQ) consecutive query tokens of one
// sequence and one kv-head, each wave 2 or 4 tokens x the <=16 query heads of the GQA group;
// compressed K/V chunks of 32 keys are staged once per workgroup in double-buffered LDS and
// shared by those tokens, which see almost the same causal range (key c is visible to position i iff c*stride + kernel - 1 <= i).
// Scores are produced transposed (S^T = K Q^T) so that one lane holds one head and P^T / dS^T
// feed the next MFMA directly; V^T and K^T fragments are read from the row-major LDS tiles with
// ds_read_b64_tr_b16.
//
// Selection (replaces the dense [Hkv, T, Tc] score tensor + transform + torch.topk of the
// reference): per token the probabilities are recomputed chunk by chunk from the final LSE,
// summed over the group's heads, folded into block scores with the overlap weights, then the k
// best blocks are extracted by repeated wave-wide arg-max and written in ascending order.
#include <type_traits>
#include "delta.h"
#include "dkdv.h"

struct CmpParams {
  const void* q; const void* k; const void* v; const void* dout; void* o; void* dq; float* lse; const float* delta;
  float* delta_out;  // backward dQ: when set, delta = rowsum(o * dout) is formed there (from the dO rows it holds) and stored here
  float* stat_out;   // backward dQ: (lse, delta) of every row, token-major [total_q][Hkv * G][2], for the dK/dV pass
  const int32_t* cu_q; const int32_t* cu_k;
  int total_q, batch, Hkv, G, GT, ks, st;
  int window;  // -1: compressed keys (rule above); >= 0: ordinary keys, position i sees j in [i - window, i]; -2: ordinary keys, all visible
  long long qsn, qsh, ksn, ksh, vsn, vsh, osn, osh, dsn, dsh, dqsn, dqsh;
  float qk_scale, sm_scale;
};

__device__ __forceinline__ int first_tile(const int32_t* __restrict__ cu, int b) { return (cu[b] + 15) / 16 + b; }
static inline int64_t n_tile_slots(int64_t total_q, int64_t batch) { return (total_q + 15) / 16 + batch + 1; }

struct TileInfo { int b, s0q, lq, k0, lk, i0; };
__device__ __forceinline__ bool locate_tile(const int32_t* cu_q, const int32_t* cu_k, int batch, int slot, TileInfo& ti) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (first_tile(cu_q, mid) <= slot) lo = mid; else hi = mid;
  }
  ti.b = lo;
  ti.s0q = cu_q[lo]; ti.lq = cu_q[lo + 1] - ti.s0q;
  ti.k0 = cu_k[lo]; ti.lk = cu_k[lo + 1] - ti.k0;
  ti.i0 = (slot - first_tile(cu_q, lo)) * 16;
  return ti.i0 < ti.lq;
}
// number of compressed keys visible to position pos
__device__ __forceinline__ int visible_keys(int pos, int lq, int lk, int ks, int st) {
  if (pos >= lq || pos < ks - 1) return 0;
  const int n = (pos - ks + 1) / st + 1;
  return n < lk ? n : lk;
}

// half-open range [lo, hi) of keys visible to position pos
__device__ __forceinline__ void visible_range(int pos, int lq, int lk, int ks, int st, int window, int& lo, int& hi) {
  if (window == -2) {
    lo = 0;
    hi = pos < lq ? lk : 0;
  } else if (window < 0) {
    lo = 0;
    hi = visible_keys(pos, lq, lk, ks, st);
  } else {
    hi = pos < lq ? min(pos + 1, lk) : 0;
    lo = hi > 0 ? max(0, pos - window) : 0;
  }
}

// stage rows [32*chunk, +32) of one or two [*, H, D] tensors into LDS tiles (zeros past lk).  The two
// tensors are handled by separate unrolled loops (no run-time choice of the base pointer).
template <typename T, int D, int NTENS, int NT = 256>
struct Stager {
  static constexpr int PIECES = 32 * (D / 8);  // per tensor
  static constexpr int PPT = (PIECES + NT - 1) / NT;
  uint4 ra[PPT], rb[PPT];
  unsigned ok;
  // branch-free: always load (from a clamped row), mask when writing to LDS
  __device__ __forceinline__ void fetch(const T* a, long long asn, const T* b2, long long bsn, int chunk, int lk, int tid) {
    ok = 0;
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = min(tid + u * NT, PIECES - 1);
      const int c = pc % (D / 8), r = pc / (D / 8);
      const int key = chunk * 32 + r;
      const int kc = min(key, lk - 1);
      ra[u] = *reinterpret_cast<const uint4*>(a + (long long)kc * asn + 8 * c);
      if (NTENS == 2) rb[u] = *reinterpret_cast<const uint4*>(b2 + (long long)kc * bsn + 8 * c);
      ok |= (unsigned)(key < lk) << u;
    }
  }
  __device__ __forceinline__ void stash(T (*ta)[lds_pitch(D)], T (*tb)[lds_pitch(D)], int tid) {
#pragma unroll
    for (int u = 0; u < PPT; u++) {
      const int pc = tid + u * NT;
      if (pc < PIECES) {
        const int c = pc % (D / 8), r = pc / (D / 8);
        const unsigned m = 0u - ((ok >> u) & 1u);  // all ones when the row exists
        uint4 x = ra[u];
        x.x &= m; x.y &= m; x.z &= m; x.w &= m;
        *reinterpret_cast<uint4*>(&ta[r][8 * c]) = x;
        if (NTENS == 2) {
          uint4 y = rb[u];
          y.x &= m; y.y &= m; y.z &= m; y.w &= m;
          *reinterpret_cast<uint4*>(&tb[r][8 * c]) = y;
        }
      }
    }
  }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
// fragment of X^T for 16 columns starting at d0 over the 32 staged rows, in the k-order of the
// packed score registers: slots 0..3 = rows 4*lg+r of the first 16, slots 4..7 = same of the second 16
template <typename T, int LD>
__device__ __forceinline__ typename Elem<T>::v8 tr_frag(const T (*tile)[LD], int d0, int li, int lg) {
  const T* a0 = &tile[4 * lg + (li >> 2)][d0 + 4 * (li & 3)];
  const T* a1 = &tile[16 + 4 * lg + (li >> 2)][d0 + 4 * (li & 3)];
  s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
  s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a1));
  s16x8 z = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
  return __builtin_bit_cast(typename Elem<T>::v8, z);
}

// ------------------------------------------------------------------------------------------
// tokens per wave of the forward kernel: two keeps a wave within 256 registers, so two waves share a
// SIMD and one wave's softmax arithmetic overlaps the other's MFMAs
constexpr int FWD_TPW = 2;
template <typename T, int D>
__global__ __launch_bounds__(64 * (16 / FWD_TPW)) void cmp_fwd_kernel(CmpParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, LD = lds_pitch(D), TPW = FWD_TPW, NT = 64 * (16 / TPW);
  __shared__ __attribute__((aligned(16))) T k_s[2][32][LD];
  __shared__ __attribute__((aligned(16))) T v_s[2][32][LD];
  TileInfo ti;
  if (!locate_tile(p.cu_q, p.cu_k, p.batch, blockIdx.x, ti)) return;
  const int h = blockIdx.y / p.GT, gt = blockIdx.y % p.GT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
  const int hq = gt * 16 + li;
  const bool has_head = hq < p.G;
  const int hh = h * p.G + (has_head ? hq : 0);
  v8 qf[TPW][NK];
  int lo[TPW], hi[TPW];
  int wave_lo = 1 << 30, wave_hi = 0, wave_lo_max = 0, wave_hi_min = 1 << 30;
#pragma unroll
  for (int j = 0; j < TPW; j++) {
    const int pos = ti.i0 + TPW * wave + j;
    visible_range(pos, ti.lq, ti.lk, p.ks, p.st, p.window, lo[j], hi[j]);
    wave_hi = max(wave_hi, hi[j]);
    wave_hi_min = min(wave_hi_min, hi[j]);
    wave_lo_max = max(wave_lo_max, lo[j]);
    if (hi[j] > 0) wave_lo = min(wave_lo, lo[j]);
    const bool live = has_head && pos < ti.lq;
    const T* qp = (const T*)p.q + (long long)(ti.s0q + (pos < ti.lq ? pos : 0)) * p.qsn + (long long)hh * p.qsh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) qf[j][kk] = live ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
    // running maxima are taken on unscaled scores: a negative scale is applied as -q and |scale|
    if (p.qk_scale < 0.f) {
#pragma unroll
      for (int kk = 0; kk < NK; kk++) qf[j][kk] = negated16(qf[j][kk]);
    }
  }
  const float qs = fabsf(p.qk_scale);
  int tile_lo, tile_hi, unused;
  visible_range(min(ti.i0 + 15, ti.lq - 1), ti.lq, ti.lk, p.ks, p.st, p.window, unused, tile_hi);
  visible_range(ti.i0, ti.lq, ti.lk, p.ks, p.st, p.window, tile_lo, unused);
  const int ch0 = tile_lo / 32;                 // the first token of the tile reaches furthest back
  const int n_chunks = (tile_hi + 31) / 32;
  f32x4 acc[TPW][NDT];
  float m[TPW], l[TPW];
#pragma unroll
  for (int j = 0; j < TPW; j++) {
    m[j] = M_FLOOR; l[j] = 0.f;
#pragma unroll
    for (int i = 0; i < NDT; i++) acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const T* kb = (const T*)p.k + (long long)ti.k0 * p.ksn + (long long)h * p.ksh;
  const T* vb = (const T*)p.v + (long long)ti.k0 * p.vsn + (long long)h * p.vsh;
  // Software pipeline over the 32-key chunks.  Iteration ch holds, in one basic block, the MFMAs of
  // P(ch-1) V(ch-1) and of S(ch+1) = K(ch+1) Q^T together with the softmax arithmetic of S(ch): the
  // matrix pipe and the vector ALU work on different chunks, so neither waits for the other.  K and V
  // tiles therefore live in LDS for different spans: iteration ch reads K(ch+1) and V(ch-1) and
  // writes K(ch+2) and V(ch) (fetched into registers one iteration earlier) into the other parity.
  Stager<T, D, 1, NT> sk, sv;
  auto qk = [&](const int buf, f32x4 (&s)[TPW][2]) {
#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
      v8 kf[NK];
#pragma unroll
      for (int kk = 0; kk < NK; kk++) kf[kk] = ld16<v8>(&k_s[buf][16 * sub + li][32 * kk + 8 * lg]);
#pragma unroll
      for (int j = 0; j < TPW; j++) {
        f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) c = E::mfma16(kf[kk], qf[j][kk], c);
        s[j][sub] = c;
      }
    }
  };
  auto pv = [&](const int buf, const v8 (&pf)[TPW]) {
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      const v8 vt = tr_frag<T, LD>(v_s[buf], 16 * dt, li, lg);
#pragma unroll
      for (int j = 0; j < TPW; j++) acc[j][dt] = E::mfma16(vt, pf[j], acc[j][dt]);
    }
  };
  // Running maxima are kept in raw score units with a finite floor, so a token that sees nothing yet
  // needs no special case: exp2(-inf - finite) is 0 and the floor minus itself gives alpha 1.
  float alpha[TPW];
  auto softmax = [&](auto masked, const int ch, f32x4 (&s)[TPW][2], v8 (&pf)[TPW]) {
#pragma unroll
    for (int j = 0; j < TPW; j++) {
      float mloc = M_FLOOR;
#pragma unroll
      for (int sub = 0; sub < 2; sub++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          if (decltype(masked)::value) {
            const int c = 32 * ch + 16 * sub + 4 * lg + r;
            if (!(c >= lo[j] && c < hi[j])) s[j][sub][r] = -INFINITY;
          }
          mloc = fmaxf(mloc, s[j][sub][r]);
        }
      mloc = column_max(mloc);
      // the reference maximum only moves when a chunk beats it by more than RESCALE_SLACK in the exponent:
      // until then probabilities are formed against the old reference (at most 2^RESCALE_SLACK: exact in
      // the fp32 sums, within range of bf16/fp16) and alpha stays exactly 1, so the rescale below is skipped
      const float m_new = (mloc - m[j]) * qs > RESCALE_SLACK ? mloc : m[j];
      alpha[j] = fast_exp2((m[j] - m_new) * qs);
      const float mb = m_new * qs;
      m[j] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int sub = 0; sub < 2; sub++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float x = fast_exp2(__builtin_fmaf(s[j][sub][r], qs, -mb));
          psum += x;
          pf[j][4 * sub + r] = (T)x;
        }
      l[j] = l[j] * alpha[j] + psum;
    }
  };
  if (n_chunks > ch0) {
    const int last = n_chunks - 1;
    f32x4 s_cur[TPW][2], s_nxt[TPW][2];
    v8 pf[TPW];
#pragma unroll
    for (int j = 0; j < TPW; j++) pf[j] = zero16<v8>();
    // P = 0 meets the not yet written V tile of the other parity in the first iteration: clear it
    for (int i = tid; i < 32 * LD / 8; i += NT) reinterpret_cast<uint4*>(&v_s[(ch0 + 1) & 1][0][0])[i] = uint4{0u, 0u, 0u, 0u};
    sk.fetch(kb, p.ksn, kb, p.ksn, ch0, ti.lk, tid);
    sk.stash(k_s[ch0 & 1], k_s[ch0 & 1], tid);
    sk.fetch(kb, p.ksn, kb, p.ksn, min(ch0 + 1, last), ti.lk, tid);
    sk.stash(k_s[(ch0 + 1) & 1], k_s[(ch0 + 1) & 1], tid);
    sk.fetch(kb, p.ksn, kb, p.ksn, min(ch0 + 2, last), ti.lk, tid);
    sv.fetch(vb, p.vsn, vb, p.vsn, ch0, ti.lk, tid);
    __syncthreads();
    qk(ch0 & 1, s_cur);
    __syncthreads();
    for (int ch = ch0; ch < n_chunks; ch++) {
      const int par = ch & 1;
      sk.stash(k_s[par], k_s[par], tid);
      sv.stash(v_s[par], v_s[par], tid);
      sk.fetch(kb, p.ksn, kb, p.ksn, min(ch + 3, last), ti.lk, tid);
      sv.fetch(vb, p.vsn, vb, p.vsn, min(ch + 1, last), ti.lk, tid);
      // chunks every token of the wave sees completely (all but the one or two at the causal edge) take
      // the path without per-element visibility tests
      if (32 * ch >= wave_lo_max && 32 * ch + 32 <= wave_hi_min) {
        pv(par ^ 1, pf);
        qk(par ^ 1, s_nxt);
        softmax(std::false_type{}, ch, s_cur, pf);
      } else {
        pv(par ^ 1, pf);
        qk(par ^ 1, s_nxt);
        softmax(std::true_type{}, ch, s_cur, pf);
      }
      // the running maximum settles after the first chunks: skip the multiplies when no lane rescales
#pragma unroll
      for (int j = 0; j < TPW; j++)
        if (__ballot(alpha[j] != 1.f)) {
#pragma unroll
          for (int i = 0; i < NDT; i++) acc[j][i] *= alpha[j];
        }
#pragma unroll
      for (int j = 0; j < TPW; j++)
#pragma unroll
        for (int sub = 0; sub < 2; sub++) s_cur[j][sub] = s_nxt[j][sub];
      __syncthreads();
    }
    pv(last & 1, pf);
  }
#pragma unroll
  for (int j = 0; j < TPW; j++) {
    const int pos = ti.i0 + TPW * wave + j;
    float lt = l[j];
    lt = column_sum(lt);
    if (pos < ti.lq && has_head) {
      const float inv = lt > 0.f ? 1.f / lt : 0.f;
      T* op = (T*)p.o + (long long)(ti.s0q + pos) * p.osn + (long long)hh * p.osh + 4 * lg;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        v4 out;
#pragma unroll
        for (int r = 0; r < 4; r++) out[r] = (T)(acc[j][dt][r] * inv);
        st8(op + 16 * dt, out);
      }
      if (lg == 0) p.lse[(long long)hh * p.total_q + ti.s0q + pos] = lt > 0.f ? m[j] * qs + fast_log2(lt) : -INFINITY;
    }
  }
}

// ------------------------------------------------------------------------------------------
template <typename T, int D>
__global__ __launch_bounds__(256) void cmp_dq_kernel(CmpParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, LD = lds_pitch(D), TPW = 2;  // tokens per wave: 8-token tiles inside the 16-token slot
  __shared__ __attribute__((aligned(16))) T k_s[2][32][LD];
  __shared__ __attribute__((aligned(16))) T v_s[2][32][LD];
  TileInfo ti;
  if (!locate_tile(p.cu_q, p.cu_k, p.batch, blockIdx.x >> 1, ti)) return;
  ti.i0 += 8 * (blockIdx.x & 1);
  if (ti.i0 >= ti.lq) return;
  const int h = blockIdx.y / p.GT, gt = blockIdx.y % p.GT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
  const int hq = gt * 16 + li;
  const bool has_head = hq < p.G;
  const int hh = h * p.G + (has_head ? hq : 0);
  v8 qf[TPW][NK], dof[TPW][NK];
  int lo[TPW], hi[TPW];
  float l2[TPW], dl[TPW];
  int wave_lo = 1 << 30, wave_hi = 0;
#pragma unroll
  for (int j = 0; j < TPW; j++) {
    const int pos = ti.i0 + TPW * wave + j;
    visible_range(pos, ti.lq, ti.lk, p.ks, p.st, p.window, lo[j], hi[j]);
    wave_hi = max(wave_hi, hi[j]);
    if (hi[j] > 0) wave_lo = min(wave_lo, lo[j]);
    const bool live = has_head && pos < ti.lq;
    const long long t = ti.s0q + (pos < ti.lq ? pos : 0);
    const T* qp = (const T*)p.q + t * p.qsn + (long long)hh * p.qsh + 8 * lg;
    const T* dp = (const T*)p.dout + t * p.dsn + (long long)hh * p.dsh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) {
      qf[j][kk] = live ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
      dof[j][kk] = live ? ld16<v8>(dp + 32 * kk) : zero16<v8>();
    }
    l2[j] = live ? p.lse[(long long)hh * p.total_q + t] : INFINITY;
    if (p.delta_out) {
      const T* op = (const T*)p.o + t * p.osn + (long long)hh * p.osh + 8 * lg;
      float part = 0.f;
#pragma unroll
      for (int kk = 0; kk < NK; kk++) {
        const v8 of = live ? ld16<v8>(op + 32 * kk) : zero16<v8>();
#pragma unroll
        for (int e = 0; e < 8; e++) part = __builtin_fmaf((float)of[e], (float)dof[j][kk][e], part);
      }
      dl[j] = column_sum(part);
      if (live && lg == 0) p.delta_out[(long long)hh * p.total_q + t] = dl[j];
    } else {
      dl[j] = live ? p.delta[(long long)hh * p.total_q + t] : 0.f;
    }
    if (p.stat_out && live && lg == 0) *reinterpret_cast<float2*>(p.stat_out + (t * p.Hkv * p.G + hh) * 2) = float2{l2[j], dl[j]};
  }
  int tile_lo, tile_hi, unused;
  visible_range(min(ti.i0 + 7, ti.lq - 1), ti.lq, ti.lk, p.ks, p.st, p.window, unused, tile_hi);
  visible_range(ti.i0, ti.lq, ti.lk, p.ks, p.st, p.window, tile_lo, unused);
  const int ch0 = tile_lo / 32;                 // the first token of the tile reaches furthest back
  const int n_chunks = (tile_hi + 31) / 32;
  f32x4 acc[TPW][NDT];
#pragma unroll
  for (int j = 0; j < TPW; j++)
#pragma unroll
    for (int i = 0; i < NDT; i++) acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const T* kb = (const T*)p.k + (long long)ti.k0 * p.ksn + (long long)h * p.ksh;
  const T* vb = (const T*)p.v + (long long)ti.k0 * p.vsn + (long long)h * p.vsh;
  // two register stages with fixed roles (the loop is unrolled by two): chunk ch+2 is requested while
  // chunk ch is being consumed, so a full chunk of compute hides each load
  Stager<T, D, 2> stg0, stg1;
  if (n_chunks > ch0) {
    stg0.fetch(kb, p.ksn, vb, p.vsn, ch0, ti.lk, tid);
    stg0.stash(k_s[0], v_s[0], tid);
    stg1.fetch(kb, p.ksn, vb, p.vsn, min(ch0 + 1, n_chunks - 1), ti.lk, tid);
  }
  __syncthreads();
  auto compute = [&](const int ch, const int buf) {
    if (32 * ch < wave_hi && 32 * ch + 32 > wave_lo) {
      v8 dsf[TPW];
#pragma unroll
      for (int sub = 0; sub < 2; sub++) {
        v8 kf[NK], vf[NK];
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          kf[kk] = ld16<v8>(&k_s[buf][16 * sub + li][32 * kk + 8 * lg]);
          vf[kk] = ld16<v8>(&v_s[buf][16 * sub + li][32 * kk + 8 * lg]);
        }
#pragma unroll
        for (int j = 0; j < TPW; j++) {
          f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kk = 0; kk < NK; kk++) {
            s = E::mfma16(kf[kk], qf[j][kk], s);
            dp = E::mfma16(vf[kk], dof[j][kk], dp);
          }
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int c = 32 * ch + 16 * sub + 4 * lg + r;
            const float pr = (c >= lo[j] && c < hi[j]) ? fast_exp2(s[r] * p.qk_scale - l2[j]) : 0.f;
            dsf[j][4 * sub + r] = (T)(pr * (dp[r] - dl[j]) * p.sm_scale);
          }
        }
      }
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        const v8 kt = tr_frag<T, LD>(k_s[buf], 16 * dt, li, lg);
#pragma unroll
        for (int j = 0; j < TPW; j++) acc[j][dt] = E::mfma16(kt, dsf[j], acc[j][dt]);
      }
    }
  };
  for (int ch = ch0; ch < n_chunks; ch += 2) {
    stg0.fetch(kb, p.ksn, vb, p.vsn, min(ch + 2, n_chunks - 1), ti.lk, tid);
    compute(ch, 0);
    if (ch + 1 < n_chunks) stg1.stash(k_s[1], v_s[1], tid);
    __syncthreads();
    if (ch + 1 < n_chunks) {
      stg1.fetch(kb, p.ksn, vb, p.vsn, min(ch + 3, n_chunks - 1), ti.lk, tid);
      compute(ch + 1, 1);
      if (ch + 2 < n_chunks) stg0.stash(k_s[0], v_s[0], tid);
      __syncthreads();
    }
  }
#pragma unroll
  for (int j = 0; j < TPW; j++) {
    const int pos = ti.i0 + TPW * wave + j;
    if (pos < ti.lq && has_head) {
      T* op = (T*)p.dq + (long long)(ti.s0q + pos) * p.dqsn + (long long)hh * p.dqsh + 4 * lg;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        v4 out;
#pragma unroll
        for (int r = 0; r < 4; r++) out[r] = (T)acc[j][dt][r];
        st8(op + 16 * dt, out);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// block selection
struct SelParams {
  const void* q; const void* k; const float* lse; const int32_t* cu_q; const int32_t* cu_k; int32_t* out;
  int total_q, batch, Hkv, G, GT, ks, st, bs, init_blocks, local_blocks, k_out, nb_cap, full_blocks;
  int nb_lo, nb_row;  // this launch takes the tiles that need nb_lo < blocks <= nb_row score entries per token; nb_row is the row pitch
  long long qsn, qsh, ksn, ksh, osh, osn, osk;
  float qk_scale;
};

constexpr int SEL_LOCAL = 16;  // candidates a lane keeps in registers during selection (64 * SEL_LOCAL blocks)

// sum over the A keys that end at each lane's key: lanes below in this row, then the tail of the previous 16 keys
template <int U, int A> __device__ __forceinline__ float window_sum(float xs, float xprev) {
  if constexpr (U >= A) return 0.f;
  else return dpp_f32<0x110 + U>(xs) + dpp_f32<0x100 + 16 - U>(xprev) + window_sum<U + 1, A>(xs, xprev);
}

// A, RR: keys per kernel window and per selection block when they are the compile-time pair handled
// with DPP lane moves (A = 0: any power-of-two pair, through run-time lane shuffles).
template <typename T, int D, int A, int RR>
__global__ __launch_bounds__(256) void cmp_select_kernel(SelParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, LD = lds_pitch(D);
  __shared__ __attribute__((aligned(16))) T k_s[2][32][LD];
  extern __shared__ float dyn[];
  float* bs_s = dyn;                           // [16][nb_row] block scores of the tile's tokens
  TileInfo ti;
  if (!locate_tile(p.cu_q, p.cu_k, p.batch, blockIdx.x, ti)) return;
  const int tile_last = min(ti.i0 + 15, ti.lq - 1);
  {  // tiles are shared out over launches by the number of blocks their last token can choose from
    const int need = min(tile_last / p.bs + 1, p.nb_cap);
    if (need <= p.nb_lo || need > p.nb_row) return;
  }
  const int h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), li = lane & 15, lg = lane >> 4;
  const int a = A ? A : p.ks / p.st, rr = A ? RR : p.bs / p.st;  // keys per kernel window and per selection block
  for (int i = tid; i < 16 * p.nb_row; i += 256) bs_s[i] = 0.f;
  int lim[4];
  int wave_lim = 0, wave_lim_min = 1 << 30;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    lim[j] = visible_keys(ti.i0 + 4 * wave + j, ti.lq, ti.lk, p.ks, p.st);
    wave_lim = max(wave_lim, lim[j]);
    wave_lim_min = min(wave_lim_min, lim[j]);
  }
  const int n_chunks = (visible_keys(tile_last, ti.lq, ti.lk, p.ks, p.st) + 31) / 32;
  const T* kb = (const T*)p.k + (long long)ti.k0 * p.ksn + (long long)h * p.ksh;
  Stager<T, D, 1> stg;
  __syncthreads();
  for (int gt = 0; gt < p.GT; gt++) {
    v8 qf[4][NK];
    float l2[4][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int pos = ti.i0 + 4 * wave + j;
      const long long t = ti.s0q + (pos < ti.lq ? pos : 0);
      const int hq = gt * 16 + li;
      const bool live = hq < p.G && pos < ti.lq;
      const T* qp = (const T*)p.q + t * p.qsn + (long long)(h * p.G + (hq < p.G ? hq : 0)) * p.qsh + 8 * lg;
#pragma unroll
      for (int kk = 0; kk < NK; kk++) qf[j][kk] = live ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int hr = gt * 16 + 4 * lg + r;
        l2[j][r] = (hr < p.G && pos < ti.lq) ? p.lse[(long long)(h * p.G + hr) * p.total_q + t] : INFINITY;
      }
    }
    float xprev = 0.f;  // scores of the 16 keys before the current ones (none before key 0)
    if (n_chunks > 0) {
      stg.fetch(kb, p.ksn, kb, p.ksn, 0, ti.lk, tid);
      stg.stash(k_s[0], k_s[0], tid);
    }
    __syncthreads();
    for (int ch = 0; ch < n_chunks; ch++) {
      const int buf = ch & 1;
      if (ch + 1 < n_chunks) stg.fetch(kb, p.ksn, kb, p.ksn, ch + 1, ti.lk, tid);
      if (32 * ch < wave_lim) {
        // all 8 score tiles of the chunk first (independent MFMA chains), then the exponentials in bulk
        f32x4 s[2][4];
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
          v8 kf[NK];
#pragma unroll
          for (int kk = 0; kk < NK; kk++) kf[kk] = ld16<v8>(&k_s[buf][16 * sub + li][32 * kk + 8 * lg]);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < NK; kk++) c = E::mfma16(qf[j][kk], kf[kk], c);  // rows = heads 4*lg+r
            s[sub][j] = c;
          }
        }
        const bool edge = 32 * ch + 32 > wave_lim_min;  // some token of the wave does not see the whole chunk
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
          const int c = 32 * ch + 16 * sub + li;  // this lane's key (column)
          float x[4];
#pragma unroll
          for (int j = 0; j < 4; j++) {
            x[j] = 0.f;
#pragma unroll
            for (int r = 0; r < 4; r++) x[j] += fast_exp2(__builtin_fmaf(s[sub][j][r], p.qk_scale, -l2[j][r]));
            if (edge) x[j] = c < lim[j] ? x[j] : 0.f;
          }
          const float xs = column_sum_scatter4(x[0], x[1], x[2], x[3]);  // lane group lg: token lg, summed over all heads
          // Overlap weights = box(a) convolved with box(rr): first the sum over the a keys that end at
          // each key (reaching into the previous 16 keys, kept in xprev), then the sum over the rr keys
          // of a block, both as lane exchanges inside the 16 lanes of a token.
          float z = xs;
          if constexpr (A != 0) {
            z += window_sum<1, A>(xs, xprev);
            if constexpr (RR >= 2) z += dpp_f32<0xB1>(z);
            if constexpr (RR >= 4) z += dpp_f32<0x4E>(z);
            if constexpr (RR >= 8) z += dpp_f32<0x141>(z);
            if constexpr (RR >= 16) z += dpp_f32<0x140>(z);
          } else {
            for (int u = 1; u < a; u++) {
              const float same = __shfl(xs, lane - u), before = __shfl(xprev, lane + 16 - u);
              z += li >= u ? same : before;
            }
            for (int mk = 1; mk < rr && mk < 16; mk <<= 1) z += __shfl_xor(z, mk);
          }
          xprev = xs;
          const int blk = c / rr;
          if ((li & (min(rr, 16) - 1)) == 0 && blk < p.full_blocks && blk < p.nb_row)
            // LDS add without return: nothing waits for it.  Row 4 * wave + lg belongs to this wave alone and an
            // instruction holds at most one lane per (row, block), so all additions to one address come from one
            // wave in program order (head tiles, then chunks): the sum, and with it the selection, is the same
            // on every run
            atomicAdd(&bs_s[(4 * wave + lg) * p.nb_row + blk], z);
        }
      }
      if (ch + 1 < n_chunks) stg.stash(k_s[buf ^ 1], k_s[buf ^ 1], tid);
      __syncthreads();
    }
  }
  // forced blocks, then k best per token (value descending, index ascending), written ascending
  for (int j = 0; j < 4; j++) {
    const int pos = ti.i0 + 4 * wave + j;
    if (pos >= ti.lq) continue;  // wave-uniform
    float* row = bs_s + (4 * wave + j) * p.nb_row;
    const int qb = pos / p.bs;
    const int nb = min(qb + 1, p.nb_row);
    for (int blk = lane; blk < nb; blk += 64)
      if (blk < p.init_blocks || blk > qb - p.local_blocks) row[blk] = INFINITY;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int n_pick = min(p.k_out, nb);
    int32_t* out = p.out + (long long)h * p.osh + (long long)(ti.s0q + pos) * p.osn;
    if (n_pick == nb) {  // everything causal is selected
      for (int i = lane; i < p.k_out; i += 64) out[(long long)i * p.osk] = i < nb ? i : -1;
      continue;
    }
    // Every lane owns the blocks lane, lane + 64, ... and remembers the best of them; a round is one
    // wave-wide maximum over those, after which only the owner of the winner updates its best.
    if (nb <= 64 * SEL_LOCAL) {
      // the lane's candidates fit in registers: no LDS traffic inside the rounds
      float cand[SEL_LOCAL];
#pragma unroll
      for (int i = 0; i < SEL_LOCAL; i++) cand[i] = lane + 64 * i < nb ? row[lane + 64 * i] : -3.f;
      float bv = -1.f;
      int bi = 0x7fffffff;
#pragma unroll
      for (int i = 0; i < SEL_LOCAL; i++)
        if (cand[i] > bv) { bv = cand[i]; bi = lane + 64 * i; }
      for (int round = 0; round < n_pick; round++) {
        const int win = candidate_index(wave_max_i64(candidate_key(bv, bi)));
        if (bi == win) {
          row[win] = -2.f;  // taken
          bv = -1.f; bi = 0x7fffffff;
#pragma unroll
          for (int i = 0; i < SEL_LOCAL; i++) {
            if (lane + 64 * i == win) cand[i] = -2.f;
            if (cand[i] > bv) { bv = cand[i]; bi = lane + 64 * i; }
          }
        }
      }
    } else {
      float bv;
      int bi;
      auto rescan = [&]() {
        bv = -1.f; bi = 0x7fffffff;
        for (int blk = lane; blk < nb; blk += 64) {
          const float v = row[blk];
          if (v > bv) { bv = v; bi = blk; }
        }
      };
      rescan();
      for (int round = 0; round < n_pick; round++) {
        const int win = candidate_index(wave_max_i64(candidate_key(bv, bi)));
        if (bi == win) {
          row[win] = -2.f;  // taken
          rescan();
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int base = 0;
    for (int blk0 = 0; blk0 < nb; blk0 += 64) {
      const int blk = blk0 + lane;
      const bool taken = blk < nb && row[blk] == -2.f;
      const unsigned long long mask = __ballot(taken);
      const int before = __popcll(mask & ((1ull << lane) - 1ull));
      if (taken) out[(long long)(base + before) * p.osk] = blk;
      base += __popcll(mask);
    }
    for (int i = n_pick + lane; i < p.k_out; i += 64) out[(long long)i * p.osk] = -1;
  }
}

// ------------------------------------------------------------------------------------------
// work items of the dK/dV pass over query ranges (dkdv.h, RANGE = true)
// chunk_off = exclusive scan of range_chunks over segments (single workgroup).
static __global__ __launch_bounds__(1024) void chunk_scan_kernel(const int32_t* __restrict__ seg_begin, const int32_t* __restrict__ seg_end, int n_seg,
                                                          int32_t* __restrict__ chunk_off, int chunk) {
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int per = (n_seg + 1023) / 1024;
  const int j0 = tid * per, j1 = min(n_seg, j0 + per);
  int s = 0;
  for (int j = j0; j < j1; j++) s += range_chunks(seg_begin[j], seg_end[j], chunk);
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
    run += range_chunks(seg_begin[j], seg_end[j], chunk);
  }
  if (tid == 1023) chunk_off[n_seg] = part[1023];
}

// Launch order of the range-mode work items: by (kv-head, token window), i.e. all key blocks that stream the same
// `chunk` tokens of Q and dO next to each other.  Together with the contiguous run of the order that each XCD
// takes (workgroup i runs on XCD i % 8), the workgroups resident on an XCD then read the same rows at about the
// same time and all but the first find them in its L2; in segment order every work item fetched its rows
// over the fabric (measured at 65 536 tokens, 32q/2kv heads: 33 GiB of fetches for 1 GiB of Q and dO).
// Counting sort in one workgroup; the place of an item inside its window is whatever the LDS atomics hand out:
// it decides when an item runs, not what it computes.  More windows than ORDER_BUCKETS: launch order = item order.
constexpr int ORDER_BUCKETS = 8192;
static __global__ __launch_bounds__(1024) void item_order_kernel(const int32_t* __restrict__ seg_begin, const int32_t* __restrict__ chunk_off, int n_seg,
                                                            int max_blocks, int chunk, int n_win, int32_t* __restrict__ order) {
  __shared__ int cnt[ORDER_BUCKETS];
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int total = chunk_off[n_seg];
  const int n_bucket = (n_seg / max_blocks) * n_win;
  if (n_bucket > ORDER_BUCKETS) {
    for (int i = tid; i < total; i += 1024) order[i] = i;
    return;
  }
  auto bucket_of = [&](int item) {
    int lo = 0, hi = n_seg;  // chunk_off[lo] <= item < chunk_off[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (chunk_off[mid] <= item) lo = mid; else hi = mid;
    }
    return (lo / max_blocks) * n_win + seg_begin[lo] / chunk + (item - chunk_off[lo]);
  };
  for (int i = tid; i < n_bucket; i += 1024) cnt[i] = 0;
  __syncthreads();
  for (int i = tid; i < total; i += 1024) atomicAdd(&cnt[bucket_of(i)], 1);
  __syncthreads();
  const int per = (n_bucket + 1023) / 1024;
  const int j0 = min(n_bucket, tid * per), j1 = min(n_bucket, j0 + per);
  int s = 0;
  for (int j = j0; j < j1; j++) s += cnt[j];
  part[tid] = s;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = part[tid] - s;
  for (int j = j0; j < j1; j++) {
    const int c = cnt[j];
    cnt[j] = run;  // becomes the bucket's write cursor
    run += c;
  }
  __syncthreads();
  for (int i = tid; i < total; i += 1024) order[atomicAdd(&cnt[bucket_of(i)], 1)] = i;
}

// ------------------------------------------------------------------------------------------
// dK/dV segments: blocks of 64 compressed keys per (head, sequence); their queries are the
// contiguous range from the first position that sees the block's first key to the sequence end
__global__ __launch_bounds__(256) void cmp_segments_kernel(const int32_t* __restrict__ cu_q, const int32_t* __restrict__ cu_k, int batch, int Hkv, int ks, int st,
                                                            int window, int max_blocks, int32_t* __restrict__ cu_blk, int32_t* __restrict__ seg_begin, int32_t* __restrict__ seg_end) {
  // one workgroup: the prefix sum of the 64-key blocks per sequence first (kept in LDS as well, for the
  // searches below), then the Hkv * max_blocks segments are filled by all threads
  extern __shared__ int32_t blk_s[];  // [batch + 1]
  block_count_prefix_256(cu_k, batch, 64, cu_blk);
  for (int b = threadIdx.x; b <= batch; b += 256) blk_s[b] = cu_blk[b];
  __syncthreads();
  const int n_blk = blk_s[batch];
  for (int i = threadIdx.x; i < Hkv * max_blocks; i += 256) {
    const int g = i % max_blocks;
    int lo = 0, hi = 0;
    if (g < n_blk) {
      const int b = find_sequence(blk_s, batch, g);
      const int lq = cu_q[b + 1] - cu_q[b];
      const int first_pos = window == -2 ? 0 : (g - blk_s[b]) * 64 * st + ks - 1;
      lo = cu_q[b] + min(first_pos, lq);
      // window mode (ordinary keys): the block's last key 64*g' + 63 is seen up to position 64*g' + 63 + window
      hi = cu_q[b] + (window < 0 ? lq : (int)min((long long)lq, (long long)(g - blk_s[b]) * 64 + 64 + window));  // -1, -2: to the end
    }
    seg_begin[i] = lo; seg_end[i] = hi;
  }
}

struct CmpBwdLayout { size_t delta, stat, cu_blk, seg_begin, seg_end, chunk_off, order, partial, total; int64_t max_blocks, max_items; int chunk; };
static CmpBwdLayout cmp_bwd_layout(int64_t Tq, int64_t Tk, int64_t B, int64_t Hq, int64_t Hkv, int64_t D) {
  CmpBwdLayout L;
  L.max_blocks = Tk / 64 + B;
  // queries per work item from a bound on the (query, key block) pairs (a causal range covers about half of Tq);
  // every block's range is at most Tq tokens: ceil(Tq/chunk)+1 items per segment is a safe bound
  L.chunk = dkdv_chunk_tokens(Hkv * L.max_blocks * Tq / 2, MAX_CHUNK_TOKENS);
  L.max_items = Hkv * L.max_blocks * ((Tq + L.chunk - 1) / L.chunk + 1);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) & ~(size_t)255; return o; };
  L.delta = take((size_t)Hq * Tq * 4);
  L.stat = take((size_t)Hq * Tq * 8);
  L.cu_blk = take((size_t)(B + 1) * 4);
  L.seg_begin = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.seg_end = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.chunk_off = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.order = take((size_t)L.max_items * 4);
  L.partial = take((size_t)L.max_items * 64 * D * 4 * 2);
  L.total = off;
  return L;
}

// ------------------------------------------------------------------------------------------
struct CmpArgs {
  CmpParams p; SelParams sp; const void* o_in; void* dk; void* dv; long long dksn, dksh, dvsn, dvsh;
  int64_t Tq, Tk, B, Hq, Hkv; char* ws; hipStream_t stream; int what;  // 0 fwd, 1 select, 2 bwd
};

template <typename T, int D>
static int run_cmp(CmpArgs& a) {
  const int64_t slots = n_tile_slots(a.Tq, a.B);
  if (a.what == 0) {
    cmp_fwd_kernel<T, D><<<dim3((unsigned)slots, (unsigned)(a.Hkv * a.p.GT)), 64 * (16 / FWD_TPW), 0, a.stream>>>(a.p);
  } else if (a.what == 1) {
    // kernel 32 / stride 16 / block 64 (the published configuration) gets the compile-time fold
    const bool usual = a.sp.ks == 2 * a.sp.st && a.sp.bs == 4 * a.sp.st;
    const void* fn = usual ? (const void*)cmp_select_kernel<T, D, 2, 4> : (const void*)cmp_select_kernel<T, D, 0, 0>;
    // A workgroup's LDS is the K staging tiles plus 64 bytes per block a token of the tile can choose from.
    // One launch sized for the longest sequence would leave a single workgroup per CU from ~1000 blocks
    // on, so tiles are grouped by need: up to three launches, with row pitches for which three, two and
    // one workgroup fit a CU's 160 KiB (workgroups of the other groups return at once).
    const int tiles_bytes = 2 * 32 * lds_pitch(D) * (int)sizeof(T);
    const int fits[3] = {(53760 - tiles_bytes) / 64, (80640 - tiles_bytes) / 64, 1 << 30};
    int lo = 0;
    for (int c = 0; c < 3 && lo < a.sp.nb_cap; c++) {
      const int hi = a.sp.nb_cap < fits[c] ? a.sp.nb_cap : fits[c];
      a.sp.nb_lo = lo; a.sp.nb_row = hi;
      const size_t dyn = (size_t)16 * hi * 4;
      if (dyn > 64 * 1024) {
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess) return NSA_ERR_UNSUPPORTED;
      }
      if (usual) cmp_select_kernel<T, D, 2, 4><<<dim3((unsigned)slots, (unsigned)a.Hkv), 256, dyn, a.stream>>>(a.sp);
      else cmp_select_kernel<T, D, 0, 0><<<dim3((unsigned)slots, (unsigned)a.Hkv), 256, dyn, a.stream>>>(a.sp);
      lo = hi;
    }
  } else {
    const CmpBwdLayout L = cmp_bwd_layout(a.Tq, a.Tk, a.B, a.Hq, a.Hkv, D);
    float* delta = (float*)(a.ws + L.delta);
    int32_t* cu_blk = (int32_t*)(a.ws + L.cu_blk);
    int32_t* seg_begin = (int32_t*)(a.ws + L.seg_begin);
    int32_t* seg_end = (int32_t*)(a.ws + L.seg_end);
    int32_t* chunk_off = (int32_t*)(a.ws + L.chunk_off);
    const int n_seg = (int)(a.Hkv * L.max_blocks);
    // dQ first: it forms delta = rowsum(O * dO) from the dO rows it holds and leaves it behind for the dK/dV pass
    a.p.o = const_cast<void*>(a.o_in); a.p.delta = nullptr; a.p.delta_out = delta; a.p.stat_out = (float*)(a.ws + L.stat);
    cmp_dq_kernel<T, D><<<dim3((unsigned)(2 * slots), (unsigned)(a.Hkv * a.p.GT)), 256, 0, a.stream>>>(a.p);
    cmp_segments_kernel<<<1, 256, (size_t)(a.B + 1) * 4, a.stream>>>(a.p.cu_q, a.p.cu_k, (int)a.B, (int)a.Hkv, a.p.ks, a.p.st, a.p.window, (int)L.max_blocks, cu_blk, seg_begin, seg_end);
    chunk_scan_kernel<<<1, 1024, 0, a.stream>>>(seg_begin, seg_end, n_seg, chunk_off, L.chunk);
    int32_t* order = (int32_t*)(a.ws + L.order);
    item_order_kernel<<<1, 1024, 0, a.stream>>>(seg_begin, chunk_off, n_seg, (int)L.max_blocks, L.chunk, (int)(a.Tq / L.chunk + 1), order);
    DkdvParams d;
    d.order = order;
    d.q = a.p.q; d.k = a.p.k; d.v = a.p.v; d.dout = a.p.dout; d.stat = (const float*)(a.ws + L.stat); d.cu = a.p.cu_q; d.cu_k = a.p.cu_k;
    d.cu_blk = cu_blk; d.seg_begin = seg_begin; d.seg_end = seg_end; d.chunk_off = chunk_off; d.queries = nullptr;
    d.partial = (float*)(a.ws + L.partial);
    d.batch = (int)a.B; d.Hkv = (int)a.Hkv; d.G = a.p.G; d.GT = a.p.GT; d.max_blocks = (int)L.max_blocks;
    d.n_seg = n_seg; d.ks = a.p.ks; d.st = a.p.st; d.window = a.p.window; d.chunk = L.chunk;
    d.qsn = (int)a.p.qsn; d.qsh = (int)a.p.qsh; d.ksn = a.p.ksn; d.ksh = a.p.ksh; d.vsn = a.p.vsn; d.vsh = a.p.vsh; d.dsn = (int)a.p.dsn; d.dsh = (int)a.p.dsh;
    d.qk_scale = a.p.qk_scale; d.sm_scale = a.p.sm_scale;
    if (a.p.GT == 1) dkdv_kernel<T, D, 64, true, true><<<(unsigned)L.max_items + 7, 64 * dkdv_waves(64), 0, a.stream>>>(d);
    else dkdv_kernel<T, D, 64, true, false><<<(unsigned)L.max_items + 7, 64 * dkdv_waves(64), 0, a.stream>>>(d);
    dkdv_reduce_kernel<T, D, 64><<<dim3((unsigned)n_seg, 8), 256, 0, a.stream>>>(d.partial, chunk_off, a.p.cu_k, cu_blk, (int)a.B, (int)L.max_blocks,
                                                                       (T*)a.dk, (T*)a.dv, a.dksn, a.dksh, a.dvsn, a.dvsh);
  }
  return nsa_check_launch();
}

static int cmp_dispatch(CmpArgs& a, int64_t head_dim, int dtype) {
#define CALL(T, D) run_cmp<T, D>(a)
  switch (head_dim) {
    case 32: return dtype == NSA_BF16 ? CALL(__bf16, 32) : CALL(_Float16, 32);
    case 64: return dtype == NSA_BF16 ? CALL(__bf16, 64) : CALL(_Float16, 64);
    case 96: return dtype == NSA_BF16 ? CALL(__bf16, 96) : CALL(_Float16, 96);
    case 128: return dtype == NSA_BF16 ? CALL(__bf16, 128) : CALL(_Float16, 128);
  }
#undef CALL
  return NSA_ERR_UNSUPPORTED;
}

static int cmp_common(CmpArgs& a, const void* q, const void* k, const void* v, const int32_t* cu_q, const int32_t* cu_k, int64_t Tq,
                      int64_t Tk, int64_t B, int64_t Hq, int64_t Hkv, int64_t ks, int64_t st, const int64_t* strides, float sm_scale,
                      int dtype, void* stream) {
  if (!q || !k || !cu_q || !cu_k || !strides || Tq <= 0 || Tk < 0 || B <= 0 || Hkv <= 0 || Hq % Hkv != 0 || ks <= 0 || st <= 0) return NSA_ERR_BAD_ARG;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (!(sm_scale == sm_scale) || sm_scale - sm_scale != 0.f) return NSA_ERR_BAD_ARG;  // NaN or infinite scale
  for (int i = 0; i < 6; i++) if (strides[i] % 8 != 0 || strides[i] >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  CmpParams& p = a.p;
  p.q = q; p.k = k; p.v = v; p.cu_q = cu_q; p.cu_k = cu_k; p.total_q = (int)Tq; p.batch = (int)B; p.Hkv = (int)Hkv;
  p.G = (int)(Hq / Hkv); p.GT = (p.G + 15) / 16; p.ks = (int)ks; p.st = (int)st;
  p.qsn = strides[0]; p.qsh = strides[1]; p.ksn = strides[2]; p.ksh = strides[3]; p.vsn = strides[4]; p.vsh = strides[5];
  // forward: a zero scale is applied as the smallest positive one (masked scores are -inf there, and 0 * inf has no value)
  p.qk_scale = (sm_scale == 0.f ? 1.17549435e-38f : sm_scale) * NSA_LOG2E; p.sm_scale = sm_scale; p.window = -1;
  p.dout = nullptr; p.o = nullptr; p.dq = nullptr; p.lse = nullptr; p.delta = nullptr; p.delta_out = nullptr; p.stat_out = nullptr;
  a.Tq = Tq; a.Tk = Tk; a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.stream = (hipStream_t)stream; a.ws = nullptr;
  return NSA_OK;
}

extern "C" int nsa_cmp_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens_q,
                                const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                                int64_t num_kv_heads, int64_t head_dim, int64_t kernel_size, int64_t kernel_stride,
                                const int64_t* strides, float sm_scale, int dtype, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens_q, cu_seqlens_k, total_q, total_k, batch, num_q_heads, num_kv_heads, kernel_size, kernel_stride, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !lse || strides[6] % 4 != 0 || strides[7] % 4 != 0 || (uintptr_t)o % 8 != 0) return NSA_ERR_BAD_ARG;
  a.p.o = o; a.p.lse = lse; a.p.osn = strides[6]; a.p.osh = strides[7];
  a.what = 0;
  return cmp_dispatch(a, head_dim, dtype);
}

extern "C" int nsa_cmp_attn_select(const void* q, const void* k, const float* lse, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   int32_t* out_topk_idx, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                                   int64_t num_kv_heads, int64_t head_dim, int64_t kernel_size, int64_t kernel_stride,
                                   int64_t block_size, int64_t k_out, int64_t max_seqlen_q, int64_t init_blocks, int64_t local_blocks,
                                   const int64_t* strides, float sm_scale, int dtype, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, k, cu_seqlens_q, cu_seqlens_k, total_q, total_k, batch, num_q_heads, num_kv_heads, kernel_size, kernel_stride, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!lse || !out_topk_idx || k_out <= 0 || max_seqlen_q <= 0) return NSA_ERR_BAD_ARG;
  if (kernel_size % kernel_stride != 0 || block_size % kernel_size != 0) return NSA_ERR_BAD_ARG;
  const int64_t rr = block_size / kernel_stride, pad = kernel_size / kernel_stride - 1;
  // the lane-exchange fold of key scores into block scores needs a power-of-two block and a window of at most 16 keys
  if ((rr & (rr - 1)) != 0 || pad > 15) return NSA_ERR_UNSUPPORTED;
  const int64_t nb = (max_seqlen_q + block_size - 1) / block_size;
  if (k_out > nb) return NSA_ERR_BAD_ARG;
  if ((size_t)16 * nb * 4 > 140 * 1024) return NSA_ERR_UNSUPPORTED;  // block scores of a 16-token tile must fit LDS
  SelParams& s = a.sp;
  s.q = q; s.k = k; s.lse = lse; s.cu_q = cu_seqlens_q; s.cu_k = cu_seqlens_k; s.out = out_topk_idx;
  s.total_q = (int)total_q; s.batch = (int)batch; s.Hkv = (int)num_kv_heads; s.G = a.p.G; s.GT = a.p.GT; s.ks = (int)kernel_size;
  s.st = (int)kernel_stride; s.bs = (int)block_size; s.init_blocks = (int)init_blocks; s.local_blocks = (int)local_blocks;
  s.k_out = (int)k_out; s.nb_cap = (int)nb; s.full_blocks = (int)(max_seqlen_q / block_size);
  s.qsn = strides[0]; s.qsh = strides[1]; s.ksn = strides[2]; s.ksh = strides[3]; s.osh = strides[6]; s.osn = strides[7]; s.osk = strides[8];
  s.qk_scale = sm_scale * NSA_LOG2E;
  a.what = 1;
  return cmp_dispatch(a, head_dim, dtype);
}

extern "C" size_t nsa_cmp_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                                   int64_t head_dim) {
  return cmp_bwd_layout(total_q, total_k, batch, num_q_heads, num_kv_heads, head_dim).total;
}

extern "C" int nsa_cmp_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq,
                                void* dk, void* dv, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int64_t total_q,
                                int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                int64_t kernel_size, int64_t kernel_stride, const int64_t* strides, float sm_scale, int dtype,
                                void* workspace, size_t workspace_bytes, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens_q, cu_seqlens_k, total_q, total_k, batch, num_q_heads, num_kv_heads, kernel_size, kernel_stride, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !dout || !lse || !dq || !dk || !dv || !workspace) return NSA_ERR_BAD_ARG;
  for (int i = 6; i < 10; i++) if (strides[i] % 8 != 0 || strides[i] >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
  for (int i = 10; i < 16; i++) if (strides[i] % 4 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)o | (uintptr_t)dout) % 16 != 0 || ((uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) % 8 != 0 || (uintptr_t)workspace % 256 != 0) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_cmp_attn_bwd_workspace_bytes(total_q, total_k, batch, num_q_heads, num_kv_heads, head_dim)) return NSA_ERR_WORKSPACE;
  a.o_in = o; a.p.dout = dout; a.p.lse = (float*)lse; a.p.dq = dq; a.dk = dk; a.dv = dv;
  a.p.osn = strides[6]; a.p.osh = strides[7]; a.p.dsn = strides[8]; a.p.dsh = strides[9];
  if (!dkdv_strides_fit(a.p.qsn, a.p.qsh, a.p.dsn, a.p.dsh, a.p.G, head_dim)) return NSA_ERR_UNSUPPORTED;
  a.p.dqsn = strides[10]; a.p.dqsh = strides[11]; a.dksn = strides[12]; a.dksh = strides[13]; a.dvsn = strides[14]; a.dvsh = strides[15];
  a.ws = (char*)workspace;
  a.what = 2;
  return cmp_dispatch(a, head_dim, dtype);
}

// Causal sliding-window (or, with a window >= the longest sequence, plain causal) varlen attention:
// the same tile kernels with the visibility rule "j in [i - window, i]".
extern "C" int nsa_window_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens,
                                   int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                   int64_t window_size, const int64_t* strides, float sm_scale, int dtype, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens, cu_seqlens, total_len, total_len, batch, num_q_heads, num_kv_heads, 1, 1, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !lse || window_size < 0 || strides[6] % 4 != 0 || strides[7] % 4 != 0 || (uintptr_t)o % 8 != 0) return NSA_ERR_BAD_ARG;
  a.p.o = o; a.p.lse = lse; a.p.osn = strides[6]; a.p.osh = strides[7];
  a.p.window = (int)(window_size > (1 << 30) ? (1 << 30) : window_size);
  a.what = 0;
  return cmp_dispatch(a, head_dim, dtype);
}

extern "C" size_t nsa_window_attn_bwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim) {
  return cmp_bwd_layout(total_len, total_len, batch, num_q_heads, num_kv_heads, head_dim).total;
}

extern "C" int nsa_window_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq,
                                   void* dk, void* dv, const int32_t* cu_seqlens, int64_t total_len, int64_t batch, int64_t num_q_heads,
                                   int64_t num_kv_heads, int64_t head_dim, int64_t window_size, const int64_t* strides, float sm_scale,
                                   int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens, cu_seqlens, total_len, total_len, batch, num_q_heads, num_kv_heads, 1, 1, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !dout || !lse || !dq || !dk || !dv || !workspace || window_size < 0) return NSA_ERR_BAD_ARG;
  for (int i = 6; i < 10; i++) if (strides[i] % 8 != 0 || strides[i] >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
  for (int i = 10; i < 16; i++) if (strides[i] % 4 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)o | (uintptr_t)dout) % 16 != 0 || ((uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) % 8 != 0 || (uintptr_t)workspace % 256 != 0) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_window_attn_bwd_workspace_bytes(total_len, batch, num_q_heads, num_kv_heads, head_dim)) return NSA_ERR_WORKSPACE;
  a.o_in = o; a.p.dout = dout; a.p.lse = (float*)lse; a.p.dq = dq; a.dk = dk; a.dv = dv;
  a.p.osn = strides[6]; a.p.osh = strides[7]; a.p.dsn = strides[8]; a.p.dsh = strides[9];
  if (!dkdv_strides_fit(a.p.qsn, a.p.qsh, a.p.dsn, a.p.dsh, a.p.G, head_dim)) return NSA_ERR_UNSUPPORTED;
  a.p.dqsn = strides[10]; a.p.dqsh = strides[11]; a.dksn = strides[12]; a.dksh = strides[13]; a.dvsn = strides[14]; a.dvsh = strides[15];
  a.p.window = (int)(window_size > (1 << 30) ? (1 << 30) : window_size);
  a.ws = (char*)workspace;
  a.what = 2;
  return cmp_dispatch(a, head_dim, dtype);
}

// Dense varlen attention with separate query / key lengths per sequence (causal: query i sees keys j <= i, counted
// from the start of both; otherwise every key): the same tile kernels once more.
extern "C" size_t nsa_flash_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                                     int64_t head_dim) {
  return cmp_bwd_layout(total_q, total_k, batch, num_q_heads, num_kv_heads, head_dim).total;
}

extern "C" int nsa_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens_q,
                                  const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int causal, const int64_t* strides, float sm_scale, int dtype,
                                  void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens_q, cu_seqlens_k, total_q, total_k, batch, num_q_heads, num_kv_heads, 1, 1, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !lse || strides[6] % 4 != 0 || strides[7] % 4 != 0 || (uintptr_t)o % 8 != 0) return NSA_ERR_BAD_ARG;
  a.p.o = o; a.p.lse = lse; a.p.osn = strides[6]; a.p.osh = strides[7];
  a.p.window = causal ? (1 << 30) : -2;
  a.what = 0;
  return cmp_dispatch(a, head_dim, dtype);
}

extern "C" int nsa_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq,
                                  void* dk, void* dv, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int64_t total_q,
                                  int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int causal,
                                  const int64_t* strides, float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  CmpArgs a;
  int rc = cmp_common(a, q, k, v, cu_seqlens_q, cu_seqlens_k, total_q, total_k, batch, num_q_heads, num_kv_heads, 1, 1, strides, sm_scale, dtype, stream);
  if (rc != NSA_OK) return rc;
  if (!v || !o || !dout || !lse || !dq || !dk || !dv || !workspace) return NSA_ERR_BAD_ARG;
  for (int i = 6; i < 10; i++) if (strides[i] % 8 != 0 || strides[i] >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
  for (int i = 10; i < 16; i++) if (strides[i] % 4 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)o | (uintptr_t)dout) % 16 != 0 || ((uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) % 8 != 0 || (uintptr_t)workspace % 256 != 0) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_flash_attn_bwd_workspace_bytes(total_q, total_k, batch, num_q_heads, num_kv_heads, head_dim)) return NSA_ERR_WORKSPACE;
  a.o_in = o; a.p.dout = dout; a.p.lse = (float*)lse; a.p.dq = dq; a.dk = dk; a.dv = dv;
  a.p.osn = strides[6]; a.p.osh = strides[7]; a.p.dsn = strides[8]; a.p.dsh = strides[9];
  if (!dkdv_strides_fit(a.p.qsn, a.p.qsh, a.p.dsn, a.p.dsh, a.p.G, head_dim)) return NSA_ERR_UNSUPPORTED;
  a.p.dqsn = strides[10]; a.p.dqsh = strides[11]; a.dksn = strides[12]; a.dksh = strides[13]; a.dvsn = strides[14]; a.dvsh = strides[15];
  a.p.window = causal ? (1 << 30) : -2;
  a.ws = (char*)workspace;
  a.what = 2;
  return cmp_dispatch(a, head_dim, dtype);
}
