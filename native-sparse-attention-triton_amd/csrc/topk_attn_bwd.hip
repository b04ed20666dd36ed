// Backward of block-sparse GQA attention (topk_sparse_attention): dQ, dK, dV.
//
// Passes, all on the caller's stream and out of the caller's workspace (run in the order 1, 3, 2: the dQ
// pass leaves delta behind for the dK/dV pass):
//   1. Reverse index "KV block -> queries that selected it": one (key = head*blocks + block,
//      value = token) pair per valid topk_idx entry, stable radix sort by key (tokens stay
//      ascending inside a block), segment offsets by binary search.  No host round trips.
//   2. dK/dV: a workgroup keeps one KV block's K and V rows in registers (each wave owns 16
//      keys) and streams the queries of that block two tokens at a time through LDS; per-chunk
//      fp32 partials are reduced in a fixed order, so the result is deterministic (no atomics).
//   3. dQ: one wavefront per (token, kv-head), same dataflow as the forward kernel; the K rows are
//      written through to wave-private LDS and read back transposed for dQ^T += K^T * dS^T.  It
//      also forms delta[h][t] = sum_d O*dO from the dO rows it holds (a delta pass of its own
//      runs only when the index phase is requested alone).
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "retile.h"
#include "delta.h"
#include "dkdv.h"

// ------------------------------------------------------------------------------------------
// workspace carving (host and entry point must agree)
struct BwdLayout {
  size_t delta, cu_blk, keys_in, keys_out, vals_in, vals_out, seg_off, chunk_off, sort_tmp, kf, vf, partial, total;
  size_t sort_tmp_bytes;
  int64_t max_blocks, n_pairs, max_items, n_slots;
};

static constexpr int LIST_CHUNK = 768;

// Key block of the dK/dV pass.  Blocks of 256 keys are handled as four 64-key blocks (one reverse-index entry per
// query and 64-key piece at or before the query's position): the 256-key variant of the kernel needs more registers
// than a wave has (it spilled inside its loop and took 9 ms where the 64-key variant takes 3).
constexpr int dkdv_block(int bs) { return bs >= 256 ? 64 : bs; }  // queries per dK/dV work item in big launches

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

static BwdLayout bwd_layout(int64_t T, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t topk, int64_t bs) {
  BwdLayout L;
  const int64_t ebs = dkdv_block((int)bs);
  L.max_blocks = T / ebs + B;  // every sequence adds at most one ragged block
  L.n_pairs = Hkv * T * topk * (bs / ebs);
  const int chunk = dkdv_chunk_tokens(L.n_pairs, LIST_CHUNK);
  L.max_items = (L.n_pairs + chunk - 1) / chunk + Hkv * L.max_blocks;
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
  L.n_slots = nsa_chunk_slots(T, B);
  L.kf = take(retile_bytes(T, B, Hkv, D));   // row-fragment copies of K and V for the dQ pass
  L.vf = take(retile_bytes(T, B, Hkv, D));
  L.partial = take((size_t)L.max_items * ebs * D * 4 * 2);
  L.total = off;
  return L;
}

// ------------------------------------------------------------------------------------------
// pass 2: reverse index
__global__ __launch_bounds__(256) void seq_blocks_kernel(const int32_t* __restrict__ cu, int batch, int bs, int32_t* __restrict__ cu_blk) {
  block_count_prefix_256(cu, batch, bs, cu_blk);
}

__global__ __launch_bounds__(256) void emit_pairs_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ cu,
                                                         const int32_t* __restrict__ cu_blk, int batch, int total_len, int Hkv,
                                                         int topk, int bs, int ebs, int max_blocks, long long ish, long long isn,
                                                         long long isk, uint32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  // one thread per (head, token, entry, piece of ebs keys inside the selected block); bs == ebs: one piece
  const int sub = bs / ebs;
  const long long n = (long long)Hkv * total_len * topk * sub;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int s = (int)(i % sub);
  const int e = (int)((i / sub) % topk);
  const int t = (int)((i / ((long long)sub * topk)) % total_len);
  const int h = (int)(i / ((long long)sub * topk * total_len));
  const int b = find_sequence(cu, batch, t);
  const int pos = t - cu[b];
  const int blk = idx[(long long)h * ish + (long long)t * isn + (long long)e * isk];
  const int piece = blk * sub + s;
  const bool ok = blk >= 0 && blk <= pos / bs && piece * ebs <= pos;  // pieces wholly after the query hold nothing it sees
  keys[i] = ok ? (uint32_t)(h * max_blocks + cu_blk[b] + piece) : (uint32_t)(Hkv * max_blocks);
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

// ------------------------------------------------------------------------------------------
// pass 4: dQ
struct DqParams {
  const void* q; const void* kf; const void* vf; const void* dout; const float* lse;
  const void* o;   // forward output: when given, delta = rowsum(O * dO) is formed here and stored for the dK/dV pass
  float* delta;    // read when o is null
  const int32_t* idx; const int32_t* cu; void* dq;
  int total_len, batch, Hkv, G, GT, topk, n_slots;
  long long n_items;
  long long qsn, qsh, dsn, dsh, osn, osh, ish, isn, isk, dqsn, dqsh;
  float qk_scale, sm_scale;
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) void dq_kernel(DqParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, NCH = BS / 32, LD = lds_pitch(D);
  // K and V come from their fragment-major copies (one coalesced 1 KiB load per operand fragment).
  // Wave-private staging of one 64-key slice of K: the fragments arrive in A-operand layout for
  // S^T = K Q^T, are written through to LDS as rows, and come back transposed (K^T fragments)
  // for dQ^T += K^T dS^T - K is fetched once per (token, block) instead of twice
  __shared__ __attribute__((aligned(16))) T k_s[4][64][LD];
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  // scalar wave index: token, sequence, block ids and fragment addresses are then computed once per wave
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
  float dl;
  if (p.o) {
    // the wave holds this token's dO rows already: one more row of loads gives delta without a pass of its own
    const T* op_ = (const T*)p.o + (long long)t * p.osn + (long long)hh * p.osh + 8 * lg;
    float part = 0.f;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) {
      const v8 of = has_head ? ld16<v8>(op_ + 32 * kk) : zero16<v8>();
#pragma unroll
      for (int e = 0; e < 8; e++) part = __builtin_fmaf((float)of[e], (float)dof[kk][e], part);
    }
    dl = column_sum(part);
    if (has_head && lg == 0) p.delta[(long long)hh * p.total_len + t] = dl;
  } else {
    dl = has_head ? p.delta[(long long)hh * p.total_len + t] : 0.f;
  }
  f32x4 acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* ip = p.idx + (long long)h * p.ish + (long long)t * p.isn;
  const T* kbase = (const T*)p.kf + ((long long)h * p.n_slots + slot0) * 32 * D;  // wave-uniform; lanes add lane * 8
  const T* vbase = (const T*)p.vf + ((long long)h * p.n_slots + slot0) * 32 * D;
  const unsigned lane8 = lane * 8u;
  const float dls = dl * p.sm_scale;
  T (*ks)[LD] = k_s[wave];
  const int last_slot = (len - 1) >> 5;
  // block ids are read once (lane e holds entry e) and visited through a wave-uniform bit mask
  for (int e0 = 0; e0 < p.topk; e0 += 64) {
  const int my_e = e0 + lane;
  const int my_blk = my_e < p.topk ? ip[(long long)my_e * p.isk] : -1;
  unsigned long long todo = __ballot(my_blk >= 0 && my_blk <= qb);
  while (todo) {
    const int e = __builtin_ctzll(todo);
    todo &= todo - 1;
    const int blk = __builtin_amdgcn_readlane(my_blk, e);
    // 64 keys at a time (larger blocks are walked in 64-key slices); all fragment loads of a slice
    // are issued back to back before any of them is consumed
#pragma unroll
    for (int half = 0; half < (BS + 63) / 64; half++) {
      const int key0 = blk * BS + 64 * half;
      if (key0 > pos) break;
      constexpr int NS = BS >= 64 ? 4 : BS / 16;  // 16-key sub-tiles in this slice
      v8 kfr[NS][NK], vfr[NS][NK];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        const int st = min((key0 >> 4) + nt, 2 * last_slot + 1);  // future sub-tiles: clamp onto existing storage
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          kfr[nt][kk] = ld16<v8>(kbase + (long long)(st * NK + kk) * 512 + lane8);
          vfr[nt][kk] = ld16<v8>(vbase + (long long)(st * NK + kk) * 512 + lane8);
        }
      }
      f32x4 ds[NS];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          st16(&ks[16 * nt + li][32 * kk + 8 * lg], kfr[nt][kk]);
          s = E::mfma16(kfr[nt][kk], qf[kk], s);
          dp = E::mfma16(vfr[nt][kk], dof[kk], dp);
        }
#pragma unroll
        for (int r = 0; r < 4; r++)
          ds[nt][r] = fast_exp2(__builtin_fmaf(s[r], p.qk_scale, -l2)) * __builtin_fmaf(dp[r], p.sm_scale, -dls);
      }
      // only the slice that holds the query's own position needs the causal test
      if (key0 + 16 * NS - 1 > pos) {
#pragma unroll
        for (int nt = 0; nt < NS; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (key0 + 16 * nt + 4 * lg + r > pos) ds[nt][r] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < (NS + 1) / 2; c++) {
        v8 dsf;  // dS of masked keys is exactly 0; the (clamped, finite) K rows it meets do not matter
#pragma unroll
        for (int r = 0; r < 4; r++) {
          dsf[r] = (T)ds[2 * c][r];
          dsf[4 + r] = (T)(2 * c + 1 < NS ? ds[(2 * c + 1) % NS][r] : 0.f);
        }
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) {
          const T* a0 = &ks[32 * c + 4 * lg + (li >> 2)][16 * dt + 4 * (li & 3)];
          const T* a1 = &ks[32 * c + 16 + 4 * lg + (li >> 2)][16 * dt + 4 * (li & 3)];
          s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
          s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a1));
          s16x8 z = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
          acc[dt] = E::mfma16(__builtin_bit_cast(v8, z), dsf, acc[dt]);
        }
      }
    }
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
  seq_blocks_kernel<<<1, 256, 0, a.stream>>>(a.cu, (int)a.B, dkdv_block((int)a.bs), cu_blk);
  emit_pairs_kernel<<<(unsigned)((L.n_pairs + 255) / 256), 256, 0, a.stream>>>(
      a.idx, a.cu, cu_blk, (int)a.B, (int)a.T, (int)a.Hkv, (int)a.topk, (int)a.bs, dkdv_block((int)a.bs), (int)L.max_blocks, a.ish, a.isn, a.isk,
      keys_in, vals_in);
  unsigned bits = 1;
  while ((1ull << bits) <= (unsigned long long)n_seg) bits++;
  size_t tmp = L.sort_tmp_bytes;
  if (rocprim::radix_sort_pairs(ws + L.sort_tmp, tmp, keys_in, keys_out, vals_in, vals_out, (size_t)L.n_pairs, 0u, bits, a.stream) != hipSuccess)
    return NSA_ERR_LAUNCH;
  segment_offsets_kernel<<<(n_seg + 1 + 255) / 256, 256, 0, a.stream>>>(keys_out, L.n_pairs, n_seg, seg_off);
  chunk_scan_kernel<<<1, 1024, 0, a.stream>>>(seg_off, seg_off + 1, n_seg, chunk_off, dkdv_chunk_tokens(L.n_pairs, LIST_CHUNK));
  return nsa_check_launch();
}

template <typename T, int D, int BS>
static int run_bwd(const BwdArgs& a) {
  const BwdLayout L = bwd_layout(a.T, a.B, a.Hq, a.Hkv, a.D, a.topk, a.bs);
  char* ws = a.ws;
  float* delta = (float*)(ws + L.delta);
  const int G = (int)(a.Hq / a.Hkv), GT = (G + 15) / 16;
  const int n_seg = (int)(a.Hkv * L.max_blocks);
  // delta = rowsum(O * dO): formed inside the dQ pass when that pass runs in the same call (it holds the dO
  // rows anyway), by a pass of its own when only the preparation is asked for
  const bool fused_delta = (a.phases & NSA_BWD_PHASE_PREP) && (a.phases & NSA_BWD_PHASE_DQ);
  if ((a.phases & NSA_BWD_PHASE_PREP) && !fused_delta)
    launch_delta<T, D>((const T*)a.o, (const T*)a.dout, delta, a.T, a.Hq, a.osn, a.osh, a.dsn, a.dsh, a.stream);
  if (a.phases & NSA_BWD_PHASE_PREP) {
    int rc = build_reverse_index(a, L);
    if (rc != NSA_OK) return rc;
  }
  if (a.out_seg_off) {
    (void)hipMemcpyAsync(a.out_seg_off, ws + L.seg_off, (size_t)(n_seg + 1) * 4, hipMemcpyDeviceToDevice, a.stream);
    (void)hipMemcpyAsync(a.out_queries, ws + L.vals_out, (size_t)L.n_pairs * 4, hipMemcpyDeviceToDevice, a.stream);
  }
  // dQ first: it leaves delta behind for the dK/dV pass
  if (a.phases & NSA_BWD_PHASE_DQ) {
    DqParams p;
    T* kf = (T*)(ws + L.kf);
    T* vf = (T*)(ws + L.vf);
    launch_retile<T, D, RETILE_ROWS>((const T*)a.k, kf, a.cu, a.B, a.ksn, a.ksh, L.n_slots, a.Hkv, a.stream);
    launch_retile<T, D, RETILE_ROWS>((const T*)a.v, vf, a.cu, a.B, a.vsn, a.vsh, L.n_slots, a.Hkv, a.stream);
    p.q = a.q; p.kf = kf; p.vf = vf; p.dout = a.dout; p.lse = a.lse; p.o = fused_delta ? a.o : nullptr; p.delta = delta; p.idx = a.idx; p.cu = a.cu; p.dq = a.dq;
    p.total_len = (int)a.T; p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.topk = (int)a.topk; p.n_slots = (int)L.n_slots;
    p.n_items = (long long)a.T * GT * a.Hkv;
    p.qsn = a.qsn; p.qsh = a.qsh; p.dsn = a.dsn; p.dsh = a.dsh; p.osn = a.osn; p.osh = a.osh;
    p.ish = a.ish; p.isn = a.isn; p.isk = a.isk; p.dqsn = a.dqsn; p.dqsh = a.dqsh;
    p.qk_scale = a.sm_scale * NSA_LOG2E; p.sm_scale = a.sm_scale;
    long long n_wg = ((p.n_items + 3) / 4 + 7) / 8 * 8;
    dq_kernel<T, D, BS><<<(unsigned)n_wg, 256, 0, a.stream>>>(p);
  }
  if (a.phases & NSA_BWD_PHASE_DKDV) {
    DkdvParams p;
    p.q = a.q; p.k = a.k; p.v = a.v; p.dout = a.dout; p.lse = a.lse; p.delta = delta; p.cu = a.cu;
    p.cu_blk = (const int32_t*)(ws + L.cu_blk); p.seg_begin = (const int32_t*)(ws + L.seg_off); p.seg_end = p.seg_begin + 1;
    p.chunk_off = (const int32_t*)(ws + L.chunk_off); p.queries = (const int32_t*)(ws + L.vals_out);
    p.partial = (float*)(ws + L.partial);
    p.total_len = (int)a.T; p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.max_blocks = (int)L.max_blocks; p.n_seg = n_seg;
    p.qsn = (int)a.qsn; p.qsh = (int)a.qsh; p.ksn = a.ksn; p.ksh = a.ksh; p.vsn = a.vsn; p.vsh = a.vsh; p.dsn = (int)a.dsn; p.dsh = (int)a.dsh;
    p.qk_scale = a.sm_scale * NSA_LOG2E; p.sm_scale = a.sm_scale; p.cu_k = a.cu; p.ks = 1; p.st = 1; p.window = -1;
    p.chunk = dkdv_chunk_tokens(L.n_pairs, LIST_CHUNK);
    constexpr int EBS = dkdv_block(BS), NT = 64 * dkdv_waves(EBS);
    if (GT == 1) dkdv_kernel<T, D, EBS, false, true><<<(unsigned)L.max_items, NT, 0, a.stream>>>(p);
    else dkdv_kernel<T, D, EBS, false, false><<<(unsigned)L.max_items, NT, 0, a.stream>>>(p);
    dkdv_reduce_kernel<T, D, EBS><<<dim3((unsigned)n_seg, 8), 256, 0, a.stream>>>(
        p.partial, p.chunk_off, a.cu, p.cu_blk, (int)a.B, (int)L.max_blocks, (T*)a.dk, (T*)a.dv, a.dksn, a.dksh, a.dvsn, a.dvsh);
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
  return num_kv_heads * (total_len / dkdv_block((int)block_size) + batch);
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
  for (int i = 0; i < 10; i++) if (strides[i] % 8 != 0 || strides[i] >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;  // 16-byte loads, 31-bit strides
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
  if (!dkdv_strides_fit(a.qsn, a.qsh, a.dsn, a.dsh, num_q_heads / num_kv_heads, head_dim)) return NSA_ERR_UNSUPPORTED;
  a.sm_scale = sm_scale; a.ws = (char*)workspace; a.stream = (hipStream_t)stream;
  a.out_seg_off = out_segment_offsets; a.out_queries = out_queries; a.phases = phases;
  if (dtype == NSA_BF16) return bwd_d<__bf16>(a);
  if (dtype == NSA_FP16) return bwd_d<_Float16>(a);
  return NSA_ERR_UNSUPPORTED;
}
