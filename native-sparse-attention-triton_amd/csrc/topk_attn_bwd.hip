// Backward of block-sparse GQA attention (topk_sparse_attention): dQ, dK, dV.
//
// Passes, all on the caller's stream and out of the caller's workspace (run in the order 1, 3, 2: the dQ
// pass leaves delta behind for the dK/dV pass):
//   1. Reverse index "KV block -> queries that selected it" as a stable counting sort of the valid
//      topk_idx entries by (head, block), tokens ascending inside a block: per-tile block counts,
//      prefix sums over tiles and over blocks, then a scatter that ranks the tokens of a 64-token
//      group by bit masks.  Integer work only, no atomics whose order matters, no host round
//      trips, no memsets: the whole backward can be recorded into a HIP graph.
//   2. dK/dV: a workgroup keeps one KV block's K and V rows in registers (each wave owns 16
//      keys) and streams the queries of that block two tokens at a time through LDS; per-chunk
//      fp32 partials are reduced in a fixed order, so the result is deterministic (no atomics).
//   3. dQ: one wavefront per (token, kv-head), same dataflow as the forward kernel; the K rows are
//      written through to wave-private LDS and read back transposed for dQ^T += K^T * dS^T.  It
//      also forms delta[h][t] = sum_d O*dO from the dO rows it holds (a delta pass of its own
//      runs only when the index phase is requested alone).
#include <cstring>

#include "retile.h"
#include "pace.h"
#include "delta.h"
#include "dkdv.h"

// ------------------------------------------------------------------------------------------
// workspace carving (host and entry point must agree)
struct BwdLayout {
  size_t delta, stat, cu_blk, hist, queries, seg_off, chunk_off, kf, vf, pace, partial, total;
  int64_t max_blocks, n_pairs, max_items, n_slots;
  int tile_tokens, n_tiles;
};

static constexpr int LIST_CHUNK = 768;

// Key block of the dK/dV pass.  Blocks of 256 keys are handled as four 64-key blocks (one reverse-index entry per
// query and 64-key piece at or before the query's position): the 256-key variant of the kernel needs more registers
// than a wave has (it spilled inside its loop and took 9 ms where the 64-key variant takes 3).
constexpr int dkdv_block(int bs) { return bs >= 256 ? 64 : bs; }  // queries per dK/dV work item in big launches

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// The counting sort walks the tokens in at most RI_MAX_TILES tiles (one wave each, 64 tokens at a time), keeps the
// counters of RI_CAP blocks in LDS at a time (more blocks: more sweeps over the tile) and loads RI_ROW ids of a token at once.
static constexpr int RI_MAX_TILES = 512, RI_CAP = 2048, RI_WAVES = 2, RI_ROW = 16;

static BwdLayout bwd_layout(int64_t T, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t topk, int64_t bs) {
  BwdLayout L;
  const int64_t ebs = dkdv_block((int)bs);
  L.max_blocks = T / ebs + B;  // every sequence adds at most one ragged block
  L.n_pairs = Hkv * T * topk * (bs / ebs);
  const int chunk = dkdv_chunk_tokens(L.n_pairs, LIST_CHUNK);
  L.max_items = (L.n_pairs + chunk - 1) / chunk + Hkv * L.max_blocks;
  L.tile_tokens = (int)(((T + RI_MAX_TILES - 1) / RI_MAX_TILES + 63) / 64 * 64);
  L.n_tiles = (int)((T + L.tile_tokens - 1) / L.tile_tokens);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align256(bytes); return o; };
  L.delta = take((size_t)Hq * T * 4);
  L.stat = take((size_t)Hq * T * 8);   // (lse, delta) per token and head, token-major
  L.cu_blk = take((size_t)(B + 1) * 4);
  L.hist = take((size_t)Hkv * L.n_tiles * L.max_blocks * 4);   // [head][tile][block] counts, then their prefix over tiles
  L.queries = take((size_t)L.n_pairs * 4);
  L.seg_off = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.chunk_off = take((size_t)(Hkv * L.max_blocks + 1) * 4);
  L.n_slots = nsa_chunk_slots(T, B);
  L.kf = take(retile_bytes(T, B, Hkv, D));   // row-fragment copies of K and V for the dQ pass
  L.vf = take(retile_bytes(T, B, Hkv, D));
  L.pace = take(pace_table_bytes());
  L.partial = take((size_t)L.max_items * ebs * D * 4 * 2);
  L.total = off;
  return L;
}

// ------------------------------------------------------------------------------------------
// pass 2: reverse index
__global__ __launch_bounds__(256) void seq_blocks_kernel(const int32_t* __restrict__ cu, int batch, int bs, int32_t* __restrict__ cu_blk) {
  block_count_prefix_256(cu, batch, bs, cu_blk);
}

struct RiParams {
  const int32_t* idx; const int32_t* cu; const int32_t* cu_blk;
  int batch, total_len, Hkv, topk, bs, ebs, max_blocks, tile_tokens, n_tiles;
  long long ish, isn, isk;
  int32_t* hist;            // [Hkv][n_tiles][max_blocks]: counts (written by the counting pass), then exclusive prefix over tiles
  const int32_t* seg_off;   // scatter pass: first slot of every (head, block) segment
  int32_t* queries;         // scatter pass: token ids, segment by segment, ascending inside a segment
};

// One wave per (head, tile of consecutive tokens), 64 tokens (one per lane) at a time.  Entry (token, e) is valid iff
// 0 <= blk <= own block (and, for 256-key blocks split in four, the piece starts at or before the token).  The rank of
// a token among the tokens of its group that selected the same block comes from a 64-bit mask per block (bit = lane),
// built with LDS or-operations whose order cannot matter; the blocks' running counts within the tile sit next to the
// masks.  SCATTER = false: writes the tile's count of every block.  SCATTER = true: writes every token to
// seg_off[segment] + (entries of earlier tiles) + (entries of earlier groups of this tile) + rank.
// A block listed twice by one token is counted and stored once.  SUB: pieces per selected block (1, or 4 for
// 256-key blocks).  Everything a wave waits for from global memory is asked for in batches (the ids of 16
// entries, then the offsets of all their segments): with one load per entry the kernel was a chain of a
// few hundred dependent round trips.
template <bool SCATTER, int SUB>
__global__ __launch_bounds__(64 * RI_WAVES) void reverse_index_kernel(RiParams p) {
  __shared__ unsigned long long mask_s[RI_WAVES][RI_CAP];
  __shared__ int cnt_s[RI_WAVES][RI_CAP];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tile = blockIdx.x * RI_WAVES + wave, h = blockIdx.y;
  if (tile >= p.n_tiles) return;   // waves never meet at a workgroup barrier
  unsigned long long* mask = mask_s[wave];
  int* cnt = cnt_s[wave];
  constexpr int NE = RI_ROW * SUB;
  const int t_begin = tile * p.tile_tokens, t_end = min(p.total_len, t_begin + p.tile_tokens);
  int32_t* hist = p.hist + ((long long)h * p.n_tiles + tile) * p.max_blocks;
  const int32_t* seg_off = SCATTER ? p.seg_off + (long long)h * p.max_blocks : nullptr;
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // sequence of the tile's first token, found once; lanes beyond its end search on their own
  const int b_first = find_sequence(p.cu, p.batch, t_begin);
  const int end_first = p.cu[b_first + 1];
  for (int r0 = 0; r0 < p.max_blocks; r0 += RI_CAP) {
    const int n_here = min(RI_CAP, p.max_blocks - r0);
    for (int i = lane; i < n_here; i += 64) { mask[i] = 0ull; cnt[i] = 0; }
    wave_sync();
    for (int t0 = t_begin; t0 < t_end; t0 += 64) {
      const int t = t0 + lane;
      const bool live = t < t_end;
      const int tt = live ? t : t_begin;
      const int b = tt < end_first ? b_first : find_sequence(p.cu, p.batch, tt);
      const int pos = tt - p.cu[b], first_blk = p.cu_blk[b] - r0, own = pos / p.bs;
      const int32_t* ip = p.idx + (long long)h * p.ish + (long long)tt * p.isn;
      // local block (relative to r0) of every (entry, piece) of a stretch of RI_ROW entries, -1 where it names
      // nothing this token sees or lies outside the sweep
      auto stretch = [&](int e0, int (&lb)[NE]) {
        int row[RI_ROW];
#pragma unroll
        for (int j = 0; j < RI_ROW; j++) row[j] = e0 + j < p.topk ? ip[(long long)(e0 + j) * p.isk] : -1;
#pragma unroll
        for (int j = 0; j < RI_ROW; j++)
#pragma unroll
          for (int s2 = 0; s2 < SUB; s2++) {
            const int blk = row[j], piece = blk * SUB + s2;
            const bool ok = live && blk >= 0 && blk <= own && piece * p.ebs <= pos;
            const int x = first_blk + piece;
            lb[j * SUB + s2] = ok && x >= 0 && x < RI_CAP ? x : -1;
          }
      };
      // Three passes over the token's entries (mark, store, count), each complete before the next starts: the
      // rank of a token must count every lower lane that names the block, at whatever entry position.
      for (int e0 = 0; e0 < p.topk; e0 += RI_ROW) {
        int lb[NE];
        stretch(e0, lb);
#pragma unroll
        for (int i = 0; i < NE; i++)
          if (lb[i] >= 0) atomicOr(&mask[lb[i]], 1ull << lane);
      }
      wave_sync();
      if (SCATTER) {
        for (int e0 = 0; e0 < p.topk; e0 += RI_ROW) {
          int lb[NE], base[NE];
          stretch(e0, lb);
#pragma unroll
          for (int i = 0; i < NE; i++) {   // all offsets first (independent loads), then the stores
            const int g = r0 + (lb[i] >= 0 ? lb[i] : 0);
            base[i] = seg_off[g] + hist[g];
          }
#pragma unroll
          for (int i = 0; i < NE; i++)
            if (lb[i] >= 0) p.queries[base[i] + cnt[lb[i]] + __popcll(mask[lb[i]] & ((1ull << lane) - 1ull))] = t;
        }
        wave_sync();
      }
      // the lowest lane of every mask adds the group's entries to the block's count and clears the mask
      for (int e0 = 0; e0 < p.topk; e0 += RI_ROW) {
        int lb[NE];
        stretch(e0, lb);
#pragma unroll
        for (int i = 0; i < NE; i++) {
          if (lb[i] < 0) continue;
          const unsigned long long m = mask[lb[i]];
          if (m != 0ull && __builtin_ctzll(m) == lane) { cnt[lb[i]] += __popcll(m); mask[lb[i]] = 0ull; }
        }
      }
      wave_sync();
    }
    if (!SCATTER)
      for (int i = lane; i < n_here; i += 64) hist[r0 + i] = cnt[i];
    wave_sync();
  }
}

// hist[h][tile][blk] -> exclusive prefix over the tiles; total[h * max_blocks + blk] = the sum.  A workgroup owns 64
// segments (lanes, coalesced) and splits the tiles over its 16 waves: partial sums, then the prefixes.
__global__ __launch_bounds__(1024) void tile_prefix_kernel(int32_t* __restrict__ hist, int32_t* __restrict__ total, int Hkv, int n_tiles, int max_blocks) {
  constexpr int NW = 16;
  __shared__ int part[NW][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seg = blockIdx.x * 64 + lane, n_seg = Hkv * max_blocks;
  const bool live = seg < n_seg;
  const int h = live ? seg / max_blocks : 0, blk = live ? seg % max_blocks : 0;
  int32_t* col = hist + (long long)h * n_tiles * max_blocks + blk;
  const int per = (n_tiles + NW - 1) / NW, c0 = min(n_tiles, wave * per), c1 = min(n_tiles, c0 + per);
  int sum = 0;
  if (live) {
#pragma unroll 8
    for (int c = c0; c < c1; c++) sum += col[(long long)c * max_blocks];
  }
  part[wave][lane] = sum;
  __syncthreads();
  int run = 0;
  for (int w = 0; w < wave; w++) run += part[w][lane];
  if (live) {
#pragma unroll 8
    for (int c = c0; c < c1; c++) {
      const int v = col[(long long)c * max_blocks];
      col[(long long)c * max_blocks] = run;
      run += v;
    }
    if (wave == NW - 1) total[seg] = run;
  }
}

// seg_off = exclusive scan of total over the segments (seg_off[n_seg] = number of valid entries) and chunk_off =
// exclusive scan of ceil(total / chunk): one workgroup, thread t owns a run of consecutive segments.  total may
// alias chunk_off (every thread reads its run before anything is written).
__global__ __launch_bounds__(1024) void segment_scan_kernel(const int32_t* total, int n_seg, int chunk, int32_t* __restrict__ seg_off,
                                                            int32_t* chunk_off) {
  __shared__ int part_a[1024], part_b[1024];
  const int tid = threadIdx.x, per = (n_seg + 1023) / 1024;
  const int j0 = min(n_seg, tid * per), j1 = min(n_seg, j0 + per);
  int a = 0, b = 0;
  for (int j = j0; j < j1; j++) { const int c = total[j]; a += c; b += (c + chunk - 1) / chunk; }
  part_a[tid] = a; part_b[tid] = b;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int va = tid >= d ? part_a[tid - d] : 0, vb = tid >= d ? part_b[tid - d] : 0;
    __syncthreads();
    part_a[tid] += va; part_b[tid] += vb;
    __syncthreads();
  }
  int ra = part_a[tid] - a, rb = part_b[tid] - b;
  // the counts of this thread's run are read again here: nobody has written them yet (other threads write only
  // their own runs of chunk_off, and seg_off is a different array)
  for (int j = j0; j < j1; j++) {
    const int c = total[j];
    seg_off[j] = ra; chunk_off[j] = rb;
    ra += c; rb += (c + chunk - 1) / chunk;
  }
  __syncthreads();
  if (tid == 1023) { seg_off[n_seg] = part_a[1023]; chunk_off[n_seg] = part_b[1023]; }
}

// ------------------------------------------------------------------------------------------
// pass 4: dQ
struct DqParams {
  const void* q; const void* kf; const void* vf; const void* dout; const float* lse;
  const void* o;   // forward output: when given, delta = rowsum(O * dO) is formed here and stored for the dK/dV pass
  float* delta;    // read when o is null
  float* stat;     // (lse, delta) of every row, [total_len][Hq][2]: written for the dK/dV pass
  const int32_t* idx; const int32_t* cu; void* dq;
  int total_len, batch, Hkv, G, GT, topk, n_slots;
  long long n_items;
  XcdSchedule sched;
  long long qsn, qsh, dsn, dsh, osn, osh, ish, isn, isk, dqsn, dqsh;
  float qk_scale, sm_scale;
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) void dq_kernel(DqParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, LD = lds_pitch(D);
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
  if (has_head && lg == 0) *reinterpret_cast<float2*>(p.stat + ((long long)t * p.Hkv * p.G + hh) * 2) = float2{l2, dl};
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
  int my_blk;
  unsigned long long todo = row_stretch(ip, p.isk, p.topk, e0, lane, qb, my_blk);
  while (todo) {
    const int blk = __builtin_amdgcn_readlane(my_blk, __builtin_ctzll(todo));
    todo = row_visited(todo, my_blk, blk);
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

// Long sequences: the dQ dataflow in persistent waves with paced key positions (pace.h), one token per wave.
template <typename T, int D> struct DqToken : SweepToken {
  typename Elem<T>::v8 qf[D / 32], dof[D / 32];
  f32x4 acc[D / 16];
  float l2, dls;
  int last_slot;
  const T* kbase; const T* vbase;
};

template <typename T, int D, int BS>
__global__ __launch_bounds__(256) void dq_sweep_kernel(DqParams p, PaceParams pp, int32_t* __restrict__ table) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16, LD = lds_pitch(D);
  __shared__ __attribute__((aligned(16))) T k_s[4][64][LD];
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, lg = lane >> 4;
  const int slot = (blockIdx.x >> 3) * 4 + wave;
  const unsigned lane8 = lane * 8u;
  T (*ks)[LD] = k_s[wave];
  using Tok = DqToken<T, D>;
  auto fetch = [&](int sw, Tok (&f)[1], int& reach) {
    const SweepPlace sp = sweep_place(pp, sw, p.cu, p.batch, p.total_len);
    reach = sp.reach;
    const int h = sp.stream / p.GT, hq = (sp.stream % p.GT) * 16 + li;
    const bool has_head = hq < p.G;
    Tok& k = f[0];
    const int t = sp.base + slot;
    k.t = t <= sp.t_last ? t : -1;
    k.my_blk = -1; k.todo = 0ull; k.e0 = 0;
#pragma unroll
    for (int i = 0; i < NDT; i++) k.acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (k.t < 0) return;
    const int b = find_sequence(p.cu, p.batch, t);
    const int s0 = p.cu[b], len = p.cu[b + 1] - s0;
    k.pos = t - s0; k.qb = k.pos / BS; k.last_slot = (len - 1) >> 5;
    const int slot0 = seq_first_slot(p.cu, b);
    k.kbase = (const T*)p.kf + ((long long)h * p.n_slots + slot0) * 32 * D;
    k.vbase = (const T*)p.vf + ((long long)h * p.n_slots + slot0) * 32 * D;
    k.ip = p.idx + (long long)h * p.ish + (long long)t * p.isn;
    const int hh = h * p.G + (has_head ? hq : 0);
    const T* qp = (const T*)p.q + (long long)t * p.qsn + (long long)hh * p.qsh + 8 * lg;
    const T* dp_ = (const T*)p.dout + (long long)t * p.dsn + (long long)hh * p.dsh + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) {
      k.qf[kk] = has_head ? ld16<v8>(qp + 32 * kk) : zero16<v8>();
      k.dof[kk] = has_head ? ld16<v8>(dp_ + 32 * kk) : zero16<v8>();
    }
    k.my_blk = lane < p.topk ? k.ip[(long long)lane * p.isk] : -1;
    k.l2 = has_head ? p.lse[(long long)hh * p.total_len + t] : INFINITY;
    float dl;
    if (p.o) {
      const T* op_ = (const T*)p.o + (long long)t * p.osn + (long long)hh * p.osh + 8 * lg;
      float part = 0.f;
#pragma unroll
      for (int kk = 0; kk < NK; kk++) {
        const v8 of = has_head ? ld16<v8>(op_ + 32 * kk) : zero16<v8>();
#pragma unroll
        for (int e = 0; e < 8; e++) part = __builtin_fmaf((float)of[e], (float)k.dof[kk][e], part);
      }
      dl = column_sum(part);
      if (has_head && lg == 0) p.delta[(long long)hh * p.total_len + t] = dl;
    } else {
      dl = has_head ? p.delta[(long long)hh * p.total_len + t] : 0.f;
    }
    if (has_head && lg == 0) *reinterpret_cast<float2*>(p.stat + ((long long)t * p.Hkv * p.G + hh) * 2) = float2{k.l2, dl};
    k.dls = dl * p.sm_scale;
    k.todo = __ballot(k.my_blk >= 0 && k.my_blk <= k.qb);
  };
  auto adopt = [&](Tok& k, const Tok& f, int) { k = f; };
  auto visit = [&](Tok (&tok)[1], unsigned, int blk, auto after_loads) {
    Tok& k = tok[0];
#pragma unroll
    for (int half = 0; half < (BS + 63) / 64; half++) {
      const int key0 = blk * BS + 64 * half;
      if (key0 > k.pos) break;
      constexpr int NS = BS >= 64 ? 4 : BS / 16;
      v8 kfr[NS][NK], vfr[NS][NK];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        const int st = min((key0 >> 4) + nt, 2 * k.last_slot + 1);
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          kfr[nt][kk] = ld16<v8>(k.kbase + (long long)(st * NK + kk) * 512 + lane8);
          vfr[nt][kk] = ld16<v8>(k.vbase + (long long)(st * NK + kk) * 512 + lane8);
        }
      }
      if (half == 0) after_loads();
      f32x4 ds[NS];
#pragma unroll
      for (int nt = 0; nt < NS; nt++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; kk++) {
          st16(&ks[16 * nt + li][32 * kk + 8 * lg], kfr[nt][kk]);
          s = E::mfma16(kfr[nt][kk], k.qf[kk], s);
          dp = E::mfma16(vfr[nt][kk], k.dof[kk], dp);
        }
#pragma unroll
        for (int r = 0; r < 4; r++)
          ds[nt][r] = fast_exp2(__builtin_fmaf(s[r], p.qk_scale, -k.l2)) * __builtin_fmaf(dp[r], p.sm_scale, -k.dls);
      }
      if (key0 + 16 * NS - 1 > k.pos) {
#pragma unroll
        for (int nt = 0; nt < NS; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (key0 + 16 * nt + 4 * lg + r > k.pos) ds[nt][r] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < (NS + 1) / 2; c++) {
        v8 dsf;
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
          k.acc[dt] = E::mfma16(__builtin_bit_cast(v8, z), dsf, k.acc[dt]);
        }
      }
    }
  };
  auto finish = [&](Tok& k, int, int sw) {
    const int stream = sw / pp.sweeps_per_stream;
    const int h = stream / p.GT, hq = (stream % p.GT) * 16 + li;
    if (hq < p.G) {
      T* op = (T*)p.dq + (long long)k.t * p.dqsn + (long long)(h * p.G + hq) * p.dqsh + 4 * lg;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        v4 out;
#pragma unroll
        for (int r = 0; r < 4; r++) out[r] = (T)k.acc[dt][r];
        st8(op + 16 * dt, out);
      }
    }
  };
  run_paced_sweeps<BS, 1, false, Tok, Tok>(pp, table, p.topk, p.isk, lane, slot, fetch, adopt, visit, finish);
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
  int32_t* seg_off = (int32_t*)(ws + L.seg_off);
  int32_t* chunk_off = (int32_t*)(ws + L.chunk_off);
  const int n_seg = (int)(a.Hkv * L.max_blocks);
  RiParams p;
  p.idx = a.idx; p.cu = a.cu; p.cu_blk = cu_blk; p.batch = (int)a.B; p.total_len = (int)a.T; p.Hkv = (int)a.Hkv; p.topk = (int)a.topk;
  p.bs = (int)a.bs; p.ebs = dkdv_block((int)a.bs); p.max_blocks = (int)L.max_blocks; p.tile_tokens = L.tile_tokens; p.n_tiles = L.n_tiles;
  p.ish = a.ish; p.isn = a.isn; p.isk = a.isk; p.hist = (int32_t*)(ws + L.hist); p.seg_off = seg_off; p.queries = (int32_t*)(ws + L.queries);
  const dim3 grid((unsigned)((L.n_tiles + RI_WAVES - 1) / RI_WAVES), (unsigned)a.Hkv);
  seq_blocks_kernel<<<1, 256, 0, a.stream>>>(a.cu, (int)a.B, p.ebs, cu_blk);
  if (p.bs == p.ebs) reverse_index_kernel<false, 1><<<grid, 64 * RI_WAVES, 0, a.stream>>>(p);
  else reverse_index_kernel<false, 4><<<grid, 64 * RI_WAVES, 0, a.stream>>>(p);
  // the per-segment totals live in chunk_off until the scan replaces them
  tile_prefix_kernel<<<(n_seg + 63) / 64, 1024, 0, a.stream>>>(p.hist, chunk_off, (int)a.Hkv, L.n_tiles, (int)L.max_blocks);
  segment_scan_kernel<<<1, 1024, 0, a.stream>>>(chunk_off, n_seg, dkdv_chunk_tokens(L.n_pairs, LIST_CHUNK), seg_off, chunk_off);
  if (p.bs == p.ebs) reverse_index_kernel<true, 1><<<grid, 64 * RI_WAVES, 0, a.stream>>>(p);
  else reverse_index_kernel<true, 4><<<grid, 64 * RI_WAVES, 0, a.stream>>>(p);
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
    launch_delta<T, D>((const T*)a.o, (const T*)a.dout, delta, a.T, a.Hq, a.osn, a.osh, a.dsn, a.dsh, a.stream, a.lse, (float*)(ws + L.stat));
  if (a.phases & NSA_BWD_PHASE_PREP) {
    int rc = build_reverse_index(a, L);
    if (rc != NSA_OK) return rc;
  }
  if (a.out_seg_off) {
    (void)hipMemcpyAsync(a.out_seg_off, ws + L.seg_off, (size_t)(n_seg + 1) * 4, hipMemcpyDeviceToDevice, a.stream);
    (void)hipMemcpyAsync(a.out_queries, ws + L.queries, (size_t)L.n_pairs * 4, hipMemcpyDeviceToDevice, a.stream);
  }
  // dQ first: it leaves delta behind for the dK/dV pass
  if (a.phases & NSA_BWD_PHASE_DQ) {
    DqParams p;
    T* kf = (T*)(ws + L.kf);
    T* vf = (T*)(ws + L.vf);
    launch_retile_pair<T, D, RETILE_ROWS, RETILE_ROWS>((const T*)a.k, kf, a.ksn, a.ksh, (const T*)a.v, vf, a.vsn, a.vsh, a.cu, a.B, L.n_slots, a.Hkv, a.stream);
    p.q = a.q; p.kf = kf; p.vf = vf; p.dout = a.dout; p.lse = a.lse; p.o = fused_delta ? a.o : nullptr; p.delta = delta; p.stat = (float*)(ws + L.stat); p.idx = a.idx; p.cu = a.cu; p.dq = a.dq;
    p.total_len = (int)a.T; p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.topk = (int)a.topk; p.n_slots = (int)L.n_slots;
    p.n_items = (long long)a.T * GT * a.Hkv;
    p.qsn = a.qsn; p.qsh = a.qsh; p.dsn = a.dsn; p.dsh = a.dsh; p.osn = a.osn; p.osh = a.osh;
    p.ish = a.ish; p.isn = a.isn; p.isk = a.isk; p.dqsn = a.dqsn; p.dqsh = a.dqsh;
    p.qk_scale = a.sm_scale * NSA_LOG2E; p.sm_scale = a.sm_scale;
    p.sched = nsa_xcd_schedule(a.T, a.B, GT * (int)a.Hkv, (int)a.D, 8.0);
    const bool paced = (a.phases & NSA_BWD_SCHEDULE_PACED) || (!(a.phases & NSA_BWD_SCHEDULE_PLAIN) && pace_pays(a.T, (int)a.D, (int)a.topk));
    if (paced) {
      PaceParams pace;
      pace.table = (int32_t*)(ws + L.pace);
      pace_fill_params(pace, a.T, pace_slots(), 1, pace_window_units((int)a.D));
      launch_pace_prepare(pace, a.cu, (int)a.B, (int)a.T, GT * (int)a.Hkv, 2000, a.stream);
      dq_sweep_kernel<T, D, BS><<<(unsigned)(2 * pace.slots), 256, 0, a.stream>>>(p, pace, pace.table);
    } else {
    long long n_wg = ((p.n_items + 3) / 4 + 7) / 8 * 8;
    if (p.sched.parts) n_wg = 8ll * p.sched.wgs_per_xcd;
    dq_kernel<T, D, BS><<<(unsigned)n_wg, 256, 0, a.stream>>>(p);
    }
  }
  if (a.phases & NSA_BWD_PHASE_DKDV) {
    DkdvParams p;
    p.order = nullptr;
    p.q = a.q; p.k = a.k; p.v = a.v; p.dout = a.dout; p.stat = (const float*)(ws + L.stat); p.cu = a.cu;
    p.cu_blk = (const int32_t*)(ws + L.cu_blk); p.seg_begin = (const int32_t*)(ws + L.seg_off); p.seg_end = p.seg_begin + 1;
    p.chunk_off = (const int32_t*)(ws + L.chunk_off); p.queries = (const int32_t*)(ws + L.queries);
    p.partial = (float*)(ws + L.partial);
    p.batch = (int)a.B; p.Hkv = (int)a.Hkv; p.G = G; p.GT = GT; p.max_blocks = (int)L.max_blocks; p.n_seg = n_seg;
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
  // 31-bit positions in the reverse index (256-key blocks are listed as four 64-key pieces)
  if (num_kv_heads * total_len * topk * (block_size / dkdv_block((int)block_size)) >= (1ll << 31)) return NSA_ERR_UNSUPPORTED;
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
