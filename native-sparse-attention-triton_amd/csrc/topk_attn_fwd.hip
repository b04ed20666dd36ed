// Forward of block-sparse GQA attention (topk_sparse_attention).
//
// One wavefront owns one (token, kv-head) pair and the up-to-16 query heads of that GQA
// group.  Scores are produced transposed, S^T[key][head] = K * Q^T, so that each lane ends
// up holding values of a single head: the row maximum and sum become per-lane scalars plus
// two cross-lane steps, and P^T is already in the B-operand layout of the next MFMA,
// O^T[d][head] += V^T[d][key] * P^T[key][head].  K and V are read from fragment-major copies
// (retile.h): every operand fragment is one coalesced 1 KiB load.  Nothing is staged in LDS:
// with one token per wave every K/V element feeds exactly one MFMA, so there is no reuse for
// LDS to exploit.
#include "retile.h"
#include "pace.h"

struct TopkFwdParams {
  const void* q; const void* kf; const void* vf; const int32_t* idx; void* o; float* lse; const int32_t* cu;
  int total_len, batch, Hkv, G, GT, topk, n_slots;
  long long n_items;
  XcdSchedule sched;
  long long qsn, qsh, ish, isn, isk, osn, osh;
  float qk_scale;  // sm_scale * log2(e)
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void topk_fwd_kernel(TopkFwdParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16;
  // the wave index is made a scalar so that everything derived from it (token, sequence, block ids,
  // fragment addresses) is computed once per wave on the scalar unit
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lg = lane >> 4;
  int t, gt, h;
  if (p.sched.parts) {
    const int xcd = blockIdx.x & 7, stream = xcd / p.sched.parts, part = xcd % p.sched.parts;
    t = p.sched.bound[part] * 64 + (blockIdx.x >> 3) * 4 + wave;
    if (t >= min(p.sched.bound[part + 1] * 64, p.total_len)) return;
    h = stream / p.GT; gt = stream % p.GT;
  } else {
    const long long item = xcd_remap(blockIdx.x, gridDim.x) * 4 + wave;
    if (item >= p.n_items) return;
    t = (int)(item % p.total_len);
    gt = (int)((item / p.total_len) % p.GT);
    h = (int)(item / ((long long)p.total_len * p.GT));
  }
  const int b = find_sequence(p.cu, p.batch, t);
  const int s0 = p.cu[b], len = p.cu[b + 1] - s0;
  const int pos = t - s0, qb = pos / BS;
  const int slot0 = seq_first_slot(p.cu, b);

  const int hq = gt * 16 + li;
  const bool has_head = hq < p.G;
  const T* qp = (const T*)p.q + (long long)t * p.qsn + (long long)(h * p.G + (has_head ? hq : 0)) * p.qsh + 8 * lg;
  v8 qf[NK];
#pragma unroll
  for (int kk = 0; kk < NK; kk++) qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
  // Running maxima are taken on unscaled scores, which is only right for a positive scale: with a negative one the
  // kernel works on -q and |scale| (the same products; a zero scale needs nothing: every probability is then 1).
  const float qs = fabsf(p.qk_scale);
  if (p.qk_scale < 0.f) {
#pragma unroll
    for (int kk = 0; kk < NK; kk++) qf[kk] = negated16(qf[kk]);
  }

  f32x4 acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = M_FLOOR, lsum = 0.f;

  const int32_t* ip = p.idx + (long long)h * p.ish + (long long)t * p.isn;
  const T* kbase = (const T*)p.kf + ((long long)h * p.n_slots + slot0) * 32 * D;  // wave-uniform; lanes add lane * 8
  const T* vbase = (const T*)p.vf + ((long long)h * p.n_slots + slot0) * 32 * D;
  const unsigned lane8 = lane * 8u;

  const int last_slot = (len - 1) >> 5;  // last slot of this sequence that exists in the copies
  // the row of block ids is read once, 64 entries at a time (lane e holds entry e); the valid
  // ones are then visited through a wave-uniform bit mask, so no load sits between two blocks
  for (int e0 = 0; e0 < p.topk; e0 += 64) {
  int my_blk;
  unsigned long long todo = row_stretch(ip, p.isk, p.topk, e0, lane, qb, my_blk);
  while (todo) {
    const int blk = __builtin_amdgcn_readlane(my_blk, __builtin_ctzll(todo));
    todo = row_visited(todo, my_blk, blk);
    // a block is walked in slices of up to 64 keys: all 2*NS*NK + NC*NDT fragment loads of a slice
    // are issued back to back (no branches in between) so that ~32 KiB per wave are in flight
#pragma unroll
    for (int sl = 0; sl < (BS + 63) / 64; sl++) {
      const int key0 = blk * BS + 64 * sl;
      if (key0 > pos) break;
      constexpr int NS = BS >= 64 ? 4 : BS / 16, NC = NS / 2;
      v8 kfr[NS][NK], vfr[NC][NDT];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        // sub-tiles wholly in the future are masked below; clamp them onto storage that exists
        const int st = min((key0 >> 4) + nt, 2 * last_slot + 1);
#pragma unroll
        for (int kk = 0; kk < NK; kk++) kfr[nt][kk] = ld16<v8>(kbase + (long long)(st * NK + kk) * 512 + lane8);
      }
#pragma unroll
      for (int c = 0; c < NC; c++) {
        const int slot = min((key0 >> 5) + c, last_slot);
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) vfr[c][dt] = ld16<v8>(vbase + (long long)slot * D * 32 + dt * 512 + lane8);
      }
      f32x4 s[NS];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) c = E::mfma16(kfr[nt][kk], qf[kk], c);
        s[nt] = c;
      }
      // only the slice that holds the query's own position needs the causal test
      if (key0 + 16 * NS - 1 > pos) {
#pragma unroll
        for (int nt = 0; nt < NS; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (key0 + 16 * nt + 4 * lg + r > pos) s[nt][r] = -INFINITY;
      }
      float mloc = M_FLOOR;
#pragma unroll
      for (int nt = 0; nt < NS; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++) mloc = fmaxf(mloc, s[nt][r]);
      mloc = column_max(mloc);
      // The reference maximum m (raw q.k units) only moves when a slice beats it by more than
      // RESCALE_SLACK in the exponent: until then probabilities are formed against the old reference
      // (at most 2^RESCALE_SLACK, exact in fp32 sums and within range of bf16/fp16), and the
      // accumulator rescale, a multiply per accumulator register, is skipped.
      const bool moved = (mloc - m) * qs > RESCALE_SLACK;
      if (__ballot(moved)) {
        const float m_new = moved ? mloc : m;
        const float alpha = fast_exp2((m - m_new) * qs);
        m = m_new;
        lsum *= alpha;
#pragma unroll
        for (int i = 0; i < NDT; i++) acc[i] *= alpha;
      }
      const float mb = m * qs;
      float psum = 0.f;
#pragma unroll
      for (int nt = 0; nt < NS; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float x = fast_exp2(__builtin_fmaf(s[nt][r], qs, -mb));
          s[nt][r] = x;
          psum += x;
        }
      lsum += psum;
#pragma unroll
      for (int c = 0; c < NC; c++) {
        v8 pf;  // probabilities of masked keys are exactly 0, the clamped V data they meet is finite
#pragma unroll
        for (int r = 0; r < 4; r++) {
          pf[r] = (T)s[2 * c][r];
          pf[4 + r] = (T)s[2 * c + 1][r];
        }
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) acc[dt] = E::mfma16(vfr[c][dt], pf, acc[dt]);
      }
    }
  }
  }
  lsum = column_sum(lsum);
  const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
  if (has_head) {
    T* op = (T*)p.o + (long long)t * p.osn + (long long)(h * p.G + hq) * p.osh + 4 * lg;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      v4 out;
#pragma unroll
      for (int r = 0; r < 4; r++) out[r] = (T)(acc[dt][r] * inv);
      st8(op + 16 * dt, out);
    }
    if (lg == 0) p.lse[(long long)(h * p.G + hq) * p.total_len + t] = lsum > 0.f ? m * qs + fast_log2(lsum) : -INFINITY;
  }
}


// ------------------------------------------------------------------------------------------
// Long sequences: the same dataflow in persistent waves whose key positions are paced (pace.h).  A wave owns TPW
// consecutive tokens of a sweep and visits the union of their selected blocks in ascending key order; the per-token
// state (Q fragments, output accumulators, running maximum and sum) stays in registers for the whole sweep.  Only
// TPW = 1 is launched: with two tokens per wave (a block that both select is fetched once, half as many sweeps
// stream the prefix) the state no longer fits 256 registers beside the 128 of a block in flight, and the spills cost
// more than the sharing saves (forward at 32 K / 64 K / 128 K tokens: 2.84 / 6.14 / 14.9 ms against 2.75 / 5.74 / 13.9).
// Also measured and dropped: the same kernel with a wave's fetches software-pipelined over its blocks (the next slice's
// K fragments requested right after the score MFMAs, its V fragments after the P V MFMAs, into the registers just
// consumed): 2.60 against 2.59 ms at 32 K tokens, 5.77 / 5.76 at 64 K - the launch is bound by what the L2 hands to the
// L1s (63 GiB per launch at 64 B per clock and compute unit would take 1.75 ms), not by a wave's own exposed latency.
template <typename T, int D> struct FwdToken : SweepToken {
  typename Elem<T>::v8 qf[D / 32];
  f32x4 acc[D / 16];
  float m, lsum;
  int last_slot;
  const T* kbase; const T* vbase;
};
// what a token brings with it: fetched one sweep ahead, so that the loads are long back when its turn comes
template <typename T, int D> struct FwdAhead {
  typename Elem<T>::v8 qf[D / 32];
  int my_blk;
  int t, pos, qb, last_slot;
  const T* kbase; const T* vbase; const int32_t* ip;
};

// One block for the tokens of `who` (all of one sequence): the K/V fragments of a slice are fetched once and serve
// every token of the set.  after_loads() runs once, after the fragment loads of the block's first slice have been issued.
template <typename T, int D, int BS, int TPW, typename F>
__device__ __forceinline__ void fwd_visit_block(FwdToken<T, D> (&tok)[TPW], unsigned who, int blk, float qs, unsigned lane8, int lg, F after_loads) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, NDT = D / 16;
  int first = 0, pos_max = -1;
#pragma unroll
  for (int i = TPW - 1; i >= 0; i--)
    if (who >> i & 1) { first = i; pos_max = max(pos_max, tok[i].pos); }
  const T* kbase = tok[0].kbase; const T* vbase = tok[0].vbase;
  int last_slot = tok[0].last_slot;
#pragma unroll
  for (int i = 1; i < TPW; i++)
    if (first == i) { kbase = tok[i].kbase; vbase = tok[i].vbase; last_slot = tok[i].last_slot; }
#pragma unroll
  for (int sl = 0; sl < (BS + 63) / 64; sl++) {
    const int key0 = blk * BS + 64 * sl;
    if (key0 > pos_max) break;
    constexpr int NS = BS >= 64 ? 4 : BS / 16, NC = NS / 2;
    v8 kfr[NS][NK], vfr[NC][NDT];
#pragma unroll
    for (int nt = 0; nt < NS; nt++) {
      const int st = min((key0 >> 4) + nt, 2 * last_slot + 1);   // sub-tiles wholly in the future: clamp onto storage that exists
#pragma unroll
      for (int kk = 0; kk < NK; kk++) kfr[nt][kk] = ld16<v8>(kbase + (long long)(st * NK + kk) * 512 + lane8);
    }
#pragma unroll
    for (int c = 0; c < NC; c++) {
      const int slot = min((key0 >> 5) + c, last_slot);
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) vfr[c][dt] = ld16<v8>(vbase + (long long)slot * D * 32 + dt * 512 + lane8);
    }
    if (sl == 0) after_loads();
#pragma unroll
    for (int i = 0; i < TPW; i++) {
      FwdToken<T, D>& k = tok[i];
      if (!(who >> i & 1) || key0 > k.pos) continue;
      f32x4 s[NS];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) c = E::mfma16(kfr[nt][kk], k.qf[kk], c);
        s[nt] = c;
      }
      // only the slice that holds the query's own position needs the causal test
      if (key0 + 16 * NS - 1 > k.pos) {
#pragma unroll
        for (int nt = 0; nt < NS; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (key0 + 16 * nt + 4 * lg + r > k.pos) s[nt][r] = -INFINITY;
      }
      float mloc = M_FLOOR;
#pragma unroll
      for (int nt = 0; nt < NS; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++) mloc = fmaxf(mloc, s[nt][r]);
      mloc = column_max(mloc);
      const bool moved = (mloc - k.m) * qs > RESCALE_SLACK;
      if (__ballot(moved)) {
        const float m_new = moved ? mloc : k.m;
        const float alpha = fast_exp2((k.m - m_new) * qs);
        k.m = m_new;
        k.lsum *= alpha;
#pragma unroll
        for (int d = 0; d < NDT; d++) k.acc[d] *= alpha;
      }
      const float mb = k.m * qs;
      float psum = 0.f;
#pragma unroll
      for (int nt = 0; nt < NS; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float x = fast_exp2(__builtin_fmaf(s[nt][r], qs, -mb));
          s[nt][r] = x;
          psum += x;
        }
      k.lsum += psum;
#pragma unroll
      for (int c = 0; c < NC; c++) {
        v8 pf;  // probabilities of masked keys are exactly 0, the clamped V data they meet is finite
#pragma unroll
        for (int r = 0; r < 4; r++) {
          pf[r] = (T)s[2 * c][r];
          pf[4 + r] = (T)s[2 * c + 1][r];
        }
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) k.acc[dt] = E::mfma16(vfr[c][dt], pf, k.acc[dt]);
      }
    }
  }
}

template <typename T, int D, int BS, int TPW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void topk_fwd_sweep_kernel(TopkFwdParams p, PaceParams pp, int32_t* __restrict__ table) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lg = lane >> 4;
  const int slot = (blockIdx.x >> 3) * 4 + wave;
  const unsigned lane8 = lane * 8u;
  const float qs = fabsf(p.qk_scale);
  using Tok = FwdToken<T, D>;
  using Ahead = FwdAhead<T, D>;
  auto fetch = [&](int sw, Ahead (&f)[TPW], int& reach) {
    const SweepPlace sp = sweep_place(pp, sw, p.cu, p.batch, p.total_len);
    reach = sp.reach;
    const int h = sp.stream / p.GT, hq = (sp.stream % p.GT) * 16 + li;
    const bool has_head = hq < p.G;
#pragma unroll
    for (int i = 0; i < TPW; i++) {
      Ahead& k = f[i];
      const int t = sp.base + slot * TPW + i;
      k.t = t <= sp.t_last ? t : -1;
      k.my_blk = -1;
      if (k.t < 0) continue;
      const int b = find_sequence(p.cu, p.batch, t);
      const int s0 = p.cu[b], len = p.cu[b + 1] - s0;
      k.pos = t - s0; k.qb = k.pos / BS; k.last_slot = (len - 1) >> 5;
      const int slot0 = seq_first_slot(p.cu, b);
      k.kbase = (const T*)p.kf + ((long long)h * p.n_slots + slot0) * 32 * D;
      k.vbase = (const T*)p.vf + ((long long)h * p.n_slots + slot0) * 32 * D;
      k.ip = p.idx + (long long)h * p.ish + (long long)t * p.isn;
      const T* qp = (const T*)p.q + (long long)t * p.qsn + (long long)(h * p.G + (has_head ? hq : 0)) * p.qsh + 8 * lg;
#pragma unroll
      for (int kk = 0; kk < NK; kk++) k.qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
      k.my_blk = lane < p.topk ? k.ip[(long long)lane * p.isk] : -1;
    }
  };
  auto adopt = [&](Tok& k, const Ahead& f, int) {
    k.t = f.t; k.pos = f.pos; k.qb = f.qb; k.last_slot = f.last_slot; k.kbase = f.kbase; k.vbase = f.vbase; k.ip = f.ip;
    k.my_blk = f.my_blk; k.e0 = 0; k.m = M_FLOOR; k.lsum = 0.f;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) k.qf[kk] = p.qk_scale < 0.f ? negated16(f.qf[kk]) : f.qf[kk];
#pragma unroll
    for (int d = 0; d < NDT; d++) k.acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    k.todo = k.t >= 0 ? __ballot(k.my_blk >= 0 && k.my_blk <= k.qb) : 0ull;
  };
  auto visit = [&](Tok (&tok)[TPW], unsigned who, int blk, auto after_loads) { fwd_visit_block<T, D, BS, TPW>(tok, who, blk, qs, lane8, lg, after_loads); };
  auto finish = [&](Tok& k, int, int sw) {
    const int stream = sw / pp.sweeps_per_stream;
    const int h = stream / p.GT, hq = (stream % p.GT) * 16 + li;
    const float lsum = column_sum(k.lsum);
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
    if (hq < p.G) {
      T* op = (T*)p.o + (long long)k.t * p.osn + (long long)(h * p.G + hq) * p.osh + 4 * lg;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        v4 out;
#pragma unroll
        for (int r = 0; r < 4; r++) out[r] = (T)(k.acc[dt][r] * inv);
        st8(op + 16 * dt, out);
      }
      if (lg == 0) p.lse[(long long)(h * p.G + hq) * p.total_len + k.t] = lsum > 0.f ? k.m * qs + fast_log2(lsum) : -INFINITY;
    }
  };
  run_paced_sweeps<BS, TPW, TPW == 1, Tok, Ahead>(pp, table, p.topk, p.isk, lane, slot, fetch, adopt, visit, finish);
}

// everything one forward call needs on the host side
struct FwdCall {
  TopkFwdParams p;
  PaceParams pace;   // pace.slots == 0: the plain kernel
  int tokens_per_wave, fixed_units;
  const void* k; const void* v;
  long long ksn, ksh, vsn, vsh;
  int phases;
  hipStream_t stream;
};

template <typename T, int D, int BS>
static int launch_fwd(const FwdCall& c) {
  const TopkFwdParams& p = c.p;
  if (c.phases & NSA_FWD_PHASE_TRANSPOSE) {
    launch_retile_pair<T, D, RETILE_ROWS, RETILE_COLS>((const T*)c.k, (T*)p.kf, c.ksn, c.ksh, (const T*)c.v, (T*)p.vf, c.vsn, c.vsh, p.cu, p.batch, p.n_slots, p.Hkv, c.stream);
  }
  if ((c.phases & NSA_FWD_PHASE_ATTEND) && c.pace.slots) {
    launch_pace_prepare(c.pace, p.cu, p.batch, p.total_len, p.GT * p.Hkv, c.fixed_units, c.stream);
    const unsigned n_wg = (unsigned)(2 * c.pace.slots);   // 8 XCDs x slots / 4 workgroups
    topk_fwd_sweep_kernel<T, D, BS, 1><<<n_wg, 256, 0, c.stream>>>(p, c.pace, c.pace.table);
  } else if (c.phases & NSA_FWD_PHASE_ATTEND) {
    long long n_wg = (p.n_items + 3) / 4;
    n_wg = (n_wg + 7) / 8 * 8;
    if (p.sched.parts) n_wg = 8ll * p.sched.wgs_per_xcd;
    topk_fwd_kernel<T, D, BS><<<dim3((unsigned)n_wg), 256, 0, c.stream>>>(p);
  }
  return nsa_check_launch();
}

template <typename T, int D>
static int dispatch_bs(int bs, const FwdCall& c) {
  switch (bs) {
    case 32: return launch_fwd<T, D, 32>(c);
    case 64: return launch_fwd<T, D, 64>(c);
    case 128: return launch_fwd<T, D, 128>(c);
    case 256: return launch_fwd<T, D, 256>(c);
  }
  return NSA_ERR_UNSUPPORTED;
}

template <typename T>
static int dispatch_d(int d, int bs, const FwdCall& c) {
  switch (d) {
    case 32: return dispatch_bs<T, 32>(bs, c);
    case 64: return dispatch_bs<T, 64>(bs, c);
    case 96: return dispatch_bs<T, 96>(bs, c);
    case 128: return dispatch_bs<T, 128>(bs, c);
  }
  return NSA_ERR_UNSUPPORTED;
}

extern "C" size_t nsa_topk_attn_fwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_kv_heads, int64_t head_dim) {
  return 2 * retile_bytes(total_len, batch, num_kv_heads, head_dim) + pace_table_bytes();  // K and V copies, pacing table
}

extern "C" int nsa_topk_attn_fwd(const void* q, const void* k, const void* v, const int32_t* topk_idx, void* o, float* lse,
                                 const int32_t* cu_seqlens, int64_t total_len, int64_t batch, int64_t num_q_heads,
                                 int64_t num_kv_heads, int64_t head_dim, int64_t topk, int64_t block_size,
                                 int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                                 int64_t v_stride_n, int64_t v_stride_h, int64_t idx_stride_h, int64_t idx_stride_n,
                                 int64_t idx_stride_k, int64_t o_stride_n, int64_t o_stride_h, float sm_scale, int dtype,
                                 void* workspace, size_t workspace_bytes, int phases, void* stream) {
  if (!q || !k || !v || !topk_idx || !o || !lse || !cu_seqlens || !workspace) return NSA_ERR_BAD_ARG;
  if (total_len <= 0 || batch <= 0 || num_kv_heads <= 0 || topk <= 0 || num_q_heads % num_kv_heads != 0) return NSA_ERR_BAD_ARG;
  if (total_len >= (1ll << 31)) return NSA_ERR_BAD_ARG;
  if (!(sm_scale == sm_scale) || sm_scale - sm_scale != 0.f) return NSA_ERR_BAD_ARG;  // NaN or infinite scale
  // 16-byte fragment loads need 8-element alignment of every row start
  if ((q_stride_n | q_stride_h | k_stride_n | k_stride_h | v_stride_n | v_stride_h) % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if ((o_stride_n | o_stride_h) % 4 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)workspace) % 16 != 0 || (uintptr_t)o % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if (workspace_bytes < nsa_topk_attn_fwd_workspace_bytes(total_len, batch, num_kv_heads, head_dim)) return NSA_ERR_WORKSPACE;
  FwdCall c;
  TopkFwdParams& p = c.p;
  const size_t copy_bytes = retile_bytes(total_len, batch, num_kv_heads, head_dim);
  p.q = q; p.kf = workspace; p.vf = (char*)workspace + copy_bytes; p.idx = topk_idx; p.o = o; p.lse = lse; p.cu = cu_seqlens;
  p.total_len = (int)total_len; p.batch = (int)batch; p.Hkv = (int)num_kv_heads; p.G = (int)(num_q_heads / num_kv_heads);
  p.GT = (p.G + 15) / 16; p.topk = (int)topk; p.n_slots = (int)nsa_chunk_slots(total_len, batch);
  p.n_items = (long long)total_len * p.GT * p.Hkv;
  p.sched = nsa_xcd_schedule(total_len, batch, p.GT * p.Hkv, (int)head_dim, 5.5);
  p.qsn = q_stride_n; p.qsh = q_stride_h;
  p.ish = idx_stride_h; p.isn = idx_stride_n; p.isk = idx_stride_k; p.osn = o_stride_n; p.osh = o_stride_h;
  // a zero scale is applied as the smallest positive one: finite scores then still give probability 1, masked
  // (-inf) scores still probability 0 (with an exact zero they would give 0 * inf)
  p.qk_scale = (sm_scale == 0.f ? 1.17549435e-38f : sm_scale) * NSA_LOG2E;
  c.k = k; c.v = v; c.ksn = k_stride_n; c.ksh = k_stride_h; c.vsn = v_stride_n; c.vsh = v_stride_h; c.phases = phases;
  c.stream = (hipStream_t)stream;
  c.pace.slots = 0; c.pace.table = (int32_t*)((char*)workspace + 2 * copy_bytes); c.tokens_per_wave = 1;
  // fixed part of a sweep's cost in the XCD schedule, in 64-key positions: fitted to the per-XCD times of paced
  // launches at 32 K .. 128 K tokens (1300 balances 32 K, 2500 the longer ones)
  c.fixed_units = 2000;
  const bool paced = (phases & NSA_FWD_SCHEDULE_PACED) || (!(phases & NSA_FWD_SCHEDULE_PLAIN) && pace_pays(total_len, (int)head_dim, (int)topk));
  if (paced) pace_fill_params(c.pace, total_len, pace_slots(), c.tokens_per_wave, pace_window_units((int)head_dim));
  if (dtype == NSA_BF16) return dispatch_d<__bf16>((int)head_dim, (int)block_size, c);
  if (dtype == NSA_FP16) return dispatch_d<_Float16>((int)head_dim, (int)block_size, c);
  return NSA_ERR_UNSUPPORTED;
}

extern "C" int nsa_version(void) { return 100; }
