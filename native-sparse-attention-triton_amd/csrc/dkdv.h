// dK/dV pass shared by the block-sparse and the compressed attention backward.
//
// A workgroup keeps one block of BS keys (K and V rows) in registers, each wave 16*KT of them as
// MFMA B operands, and streams query rows two (token, head-tile) row groups at a time through three
// LDS buffers that asynchronous global-to-LDS copies fill two steps ahead.  P and dS leave the score MFMA already in B-operand layout; the transposed
// Q and dO fragments are read from LDS with ds_read_b64_tr_b16.  Work items are (segment,
// chunk of up to MAX_CHUNK_TOKENS queries); each writes an fp32 partial, a second kernel adds the chunks of
// a segment in order, so no atomics are needed and results are reproducible.
//   RANGE = false: the queries of a segment come from a sorted list (reverse index of topk_idx),
//                  key j is visible to a query at position pos iff j <= pos.
//   RANGE = true : the queries are the contiguous range [seg_begin[s], seg_end[s]) of global token ids;
//                  DkdvParams::window says which keys a position sees (compressed keys, a sliding
//                  window of ordinary keys, or all of them).
#pragma once
#include "nsa_common.h"

// Most queries per dK/dV work item.  The token list of an item lives in LDS next to the three staging
// buffers; with 960 entries a d = 128 workgroup needs 53760 bytes, the most for which three workgroups
// share a CU's 160 KiB (with 1024 entries only two were resident and the pass ran 8 % slower).
static constexpr int MAX_CHUNK_TOKENS = 960;

// Queries per work item, from the number of (query, key block) pairs of the launch: long items amortise the
// loading of K/V and the partial they write, but a launch needs a few thousand items to fill 256 CUs three
// workgroups deep and to even out the one segment every token selects (its chunks are the longest items); a small
// launch lasts as long as its longest item (two queries per step, about 1.3 us a step).
// `longest` is the size used by big launches (measured best: 768 for query lists, 960 for query ranges); the
// smaller sizes are the measured best of 64..768 at 2048..16384 tokens with 8 and 16 blocks per token
// (2048 tokens, 8 blocks: backward 0.30 -> 0.26 ms against one size of 256 below 256 Ki pairs).
static inline int dkdv_chunk_tokens(long long pairs, int longest) {
  if (pairs >= 2048ll * 1024) return longest < MAX_CHUNK_TOKENS ? longest : MAX_CHUNK_TOKENS;
  if (pairs >= 256ll * 1024) return 384;
  if (pairs >= 96ll * 1024) return 192;
  return 128;
}

// Waves per dK/dV workgroup; each wave owns bs / (16 * waves) key tiles.  Every wave reads all staged
// query rows from LDS, so fewer waves would mean fewer LDS reads per token, but 32 keys per wave need 192
// registers for the stationary operands and the accumulators alone: at two waves per SIMD that spills,
// and at one wave per SIMD (with the score and the dK/dV MFMAs of neighbouring steps interleaved by
// hand) the single wave's instruction issue became the limit - both measured slower than one tile per
// wave at three waves per SIMD.
constexpr int dkdv_waves(int bs) { return bs >= 256 ? 8 : (bs >= 64 ? 4 : bs / 16); }

// Range mode cuts a segment's queries at the multiples of `chunk` in global token ids, so that the work items of
// different segments that cover the same tokens cover exactly the same tokens (see item_order_kernel).
__device__ __forceinline__ int range_chunks(int begin, int end, int chunk) { return end > begin ? (end + chunk - 1) / chunk - begin / chunk : 0; }

struct DkdvParams {
  const void* q; const void* k; const void* v; const void* dout;
  // (lse, delta) pairs per token, [tokens][Hkv * G][2], left behind by the dQ pass (or the stand-alone delta pass).  In [head][token]
  // arrays the 16 heads of a token lie in 32 different cache lines: with the scattered tokens of a query list 39 % of the pass's
  // L2 requests went there; here they share one line.
  const float* stat;
  const int32_t* cu; const int32_t* cu_k; const int32_t* cu_blk; const int32_t* seg_begin; const int32_t* seg_end; const int32_t* chunk_off; const int32_t* queries;
  const int32_t* order;  // range mode: launch order of the work items (item_order_kernel), or null
  float* partial;
  int batch, Hkv, G, GT, max_blocks, n_seg, ks, st;
  int chunk;   // queries per work item (dkdv_chunk_tokens)
  int window;  // range mode: -1 compressed keys (key c seen from position c*st + ks - 1 on), >= 0 ordinary keys seen by [key, key + window], -2 every key seen by every position
  long long ksn, ksh, vsn, vsh;
  int qsn, qsh, dsn, dsh;  // element strides of q / dO (dkdv_strides_fit() on the host)
  float qk_scale, sm_scale;
};

// Workgroup barrier that lets the n youngest vector-memory operations of each wave stay in flight: waits
// for all LDS traffic and for all but n loads, then meets.  (__syncthreads() would wait for every
// outstanding copy into LDS, including the ones meant to land during the next step.)
template <int N> __device__ __forceinline__ void barrier_keeping_loads() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));  // vmcnt(N), lgkmcnt(0), expcnt untouched
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Token and head strides of q / dO are carried as 32-bit numbers: they, and the offset of the last head of
// a group, must fit 31 bits.
static inline bool dkdv_strides_fit(long long qsn, long long qsh, long long dsn, long long dsh, long long G, long long D) {
  const long long lim = 0x7fffffffLL;
  return qsn >= 0 && dsn >= 0 && qsh >= 0 && dsh >= 0 && qsn <= lim && dsn <= lim && G * qsh + D <= lim && G * dsh + D <= lim;
}

// GT1: the GQA group has at most 16 query heads (one head tile), which removes every run-time division.
// The workgroups-per-CU hint is the largest for which the variant compiles without register spills.
template <typename T, int D, int BS, bool RANGE, bool GT1>
__global__ __launch_bounds__(64 * dkdv_waves(BS), BS == 64 ? (GT1 ? 3 : 2) : (BS < 64 ? (D >= 96 ? 3 : 2) : 1)) void dkdv_kernel(DkdvParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  constexpr int NK = D / 32, NDT = D / 16, NSUB = BS / 16;
  constexpr int NW = dkdv_waves(BS);          // waves per workgroup
  constexpr int KT = NSUB / NW;               // 16-key tiles per wave
  constexpr int NT = NW * 64;
  // Staged rows (2 row groups x 16 heads of Q, the same of dO) are CP 16-byte pieces long and not padded:
  // the copy engine writes whole 1 KiB stretches.  Piece c of row r sits at position (c + 2r) mod CP
  // instead, which for CP = 16 gives every access the bank (address mod 256) it would have with a row
  // pitch of 288 bytes: 16-byte row-fragment reads and the transposing 8-byte reads run at full rate.
  constexpr int CP = D > 64 ? 16 : (D > 32 ? 8 : 4);
  constexpr int TENSOR_BYTES = 32 * CP * 16;
  constexpr int BUF_BYTES = 2 * TENSOR_BYTES + 256;   // Q rows | dO rows | 32 lse | 32 delta
  // three buffers in rotation, each its own array so that the compiler can tell a copy in flight into
  // one of them from reads of another
  __shared__ __attribute__((aligned(256))) unsigned char buf0[BUF_BYTES], buf1[BUF_BYTES], buf2[BUF_BYTES];

  const int total_items = p.chunk_off[p.n_seg];
  int item = blockIdx.x;
  if (RANGE && p.order) {
    const int per = (total_items + 7) / 8;          // XCD x takes the run [x * per, (x + 1) * per) of the order
    item = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per || item >= total_items) return;
    item = p.order[item];
  }
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
  int first, n_tok;
  if (RANGE) {  // pieces between multiples of the chunk size in global token ids
    const int c = p.seg_begin[seg] / p.chunk + (item - p.chunk_off[seg]);
    first = max(p.seg_begin[seg], c * p.chunk);
    n_tok = min(p.seg_end[seg], (c + 1) * p.chunk) - first;
  } else {
    first = p.seg_begin[seg] + (item - p.chunk_off[seg]) * p.chunk;
    n_tok = min(p.chunk, p.seg_end[seg] - first);
  }
  const int GT = GT1 ? 1 : p.GT;
  const int n_rg = n_tok * GT;                // row groups (token, head tile) in this chunk
  const int n_step = (n_rg + 1) / 2;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  // token ids of this chunk, read once (list mode): the source addresses of a step then need no
  // global load of their own
  __shared__ int tok_s[MAX_CHUNK_TOKENS];
  for (int i = tid; i < n_tok; i += NT) tok_s[i] = RANGE ? first + i : p.queries[first + i];
  __syncthreads();

  const T* const qbase = (const T*)p.q + (long long)h * p.G * p.qsh;
  const T* const dbase = (const T*)p.dout + (long long)h * p.G * p.dsh;

  constexpr int NI = CP / 2;                 // 1 KiB wave-copies per tensor per step
  constexpr int LPW = (NI + NW - 1) / NW;    // of which one wave issues at most this many
  constexpr int RPI = 64 / CP;               // rows per wave-copy
  // copies per wave and step that every wave issues at least: waiting until no more than these are
  // outstanding means that everything issued one step earlier has arrived
  constexpr int KEEP = 2 * (NI / NW) + 1;
  // Starts the copies of one step into `buf`.  Rows past the end of the chunk and heads past the group
  // are read from clamped (valid) addresses; compute() gives them probability 0 by its own test.
  auto issue = [&](int step, unsigned char* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < LPW; u++) {
      const int i = wave + NW * u;
      if (NI % NW != 0 && i >= NI) break;
      const int row = i * RPI + lane / CP;
      const int c = ((lane % CP) - 2 * row) & (CP - 1);
      const int cc = c < D / 8 ? c : D / 8 - 1;   // D = 96: four positions per row hold nothing
      const int rg = row >> 4, hd = row & 15;
      const int r = min(step * 2 + rg, n_rg - 1);
      const int t = tok_s[GT1 ? r : r / GT];
      const int hq = min((GT1 ? 0 : (r % GT) * 16) + hd, p.G - 1);
      dma16(qbase + (long long)t * p.qsn + (long long)hq * p.qsh + 8 * cc, buf + i * 1024);
      dma16(dbase + (long long)t * p.dsn + (long long)hq * p.dsh + 8 * cc, buf + TENSOR_BYTES + i * 1024);
    }
    {  // lanes 0..31: lse of the 32 rows, lanes 32..63: their delta (every wave writes the same 256 bytes:
       // no wave-dependent branch, and the same number of copies in flight for all of them)
      const int rg = (lane >> 4) & 1, hd = lane & 15;
      const int r = min(step * 2 + rg, n_rg - 1);
      const int t = tok_s[GT1 ? r : r / GT];
      const int hq = min((GT1 ? 0 : (r % GT) * 16) + hd, p.G - 1);
      dma4(p.stat + (((long long)t * p.Hkv + h) * p.G + hq) * 2 + (lane >> 5), buf + 2 * TENSOR_BYTES);
    }
  };

  auto compute = [&](int step, const unsigned char* buf) __attribute__((always_inline)) {
    // position of the two tokens of this step and how many of their 16 rows are real heads
    int pos[2], nh[2];
#pragma unroll
    for (int tk = 0; tk < 2; tk++) {
      const int r = step * 2 + tk, rc = min(r, n_rg - 1);
      pos[tk] = tok_s[GT1 ? rc : rc / GT] - s0;
      nh[tk] = r < n_rg ? min(16, p.G - (GT1 ? 0 : (rc % GT) * 16)) : 0;
    }
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
          const int at = ((tk * 16 + li) * CP + ((4 * kk + lg + 2 * li) & (CP - 1))) * 16;
          v8 qa = ld16<v8>(buf + at);
          v8 da = ld16<v8>(buf + TENSOR_BYTES + at);
          s = E::mfma16(qa, kf[j][kk], s);
          dp = E::mfma16(da, vf[j][kk], dp);
        }
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(buf + 2 * TENSOR_BYTES + (tk * 16 + 4 * lg) * 4);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(buf + 2 * TENSOR_BYTES + 128 + (tk * 16 + 4 * lg) * 4);
        const bool seen = RANGE ? (key < len && (p.window == -2 || (key * p.st + p.ks - 1 <= pos[tk] && (p.window < 0 || key >= pos[tk] - p.window))))
                                : key <= pos[tk];
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const bool vis = seen && 4 * lg + r < nh[tk];
          const float pr = fast_exp2(vis ? s[r] * p.qk_scale - l4[r] : -INFINITY);  // select, not a branch
          pf[j][tk * 4 + r] = (T)pr;
          dsf[j][tk * 4 + r] = (T)(pr * (dp[r] - d4[r]) * p.sm_scale);
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
        const int row = tk * 16 + 4 * lg + (li >> 2);
        const int at = (row * CP + ((2 * dt + ((li >> 1) & 1) + 2 * row) & (CP - 1))) * 16 + (li & 1) * 8;
        s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(buf + at));
        s16x4 c = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(buf + TENSOR_BYTES + at));
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
  // one step: start the copies for two steps ahead into the buffer that was read one step ago, work on
  // the current buffer, then wait for the copies started one step ago (the next buffer) and meet
  auto pipeline_step = [&](int step, const unsigned char* cur, unsigned char* refill) __attribute__((always_inline)) {
    issue(step + 2, refill);   // steps past the end copy the last row again, harmlessly
    compute(step, cur);
    barrier_keeping_loads<KEEP>();
  };
  issue(0, buf0);
  issue(1, buf1);
  barrier_keeping_loads<KEEP>();
  // three steps per trip so that the buffer roles are compile-time; a trip may run up to two steps past
  // the end, which see no rows (nh = 0) and add nothing
  for (int step = 0; step < n_step; step += 3) {
    pipeline_step(step, buf0, buf2);
    pipeline_step(step + 1, buf1, buf0);
    pipeline_step(step + 2, buf2, buf1);
  }
  // copies still in flight target LDS that the next workgroup on this CU may own: let them land first
  __builtin_amdgcn_s_waitcnt(0x0F70);
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

