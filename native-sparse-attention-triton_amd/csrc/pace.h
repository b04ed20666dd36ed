// Key-position pacing for the query-stationary kernels on long sequences.
//
// A wave of these kernels owns a token and walks the blocks that token selected in ascending key order, fetching
// 32 KiB of K and V per 64-key block.  Left alone, the few hundred waves resident on one XCD are at unrelated key
// positions, so their combined working set is the whole K/V of a kv-head (16 MiB at 32 K tokens of 128 columns)
// against 4 MiB of L2: most fetches of late tokens go over the fabric.  Here the waves of an XCD are persistent,
// take their tokens in "sweeps" (one token, or a pair, per resident wave, consecutive tokens of one kv-head) and
// keep within a window of key positions of each other: every wave publishes the position of its next block in a
// per-XCD table and does not start a block that lies more than `window` 64-key units ahead of the table's minimum.
// The XCD's L2 then has to hold the window only, and every K/V line crosses the fabric about once per sweep.
//
// The pacing is advisory: results do not depend on it.  A wave that has polled `spin_limit` times in one wait stops
// pacing for the rest of its life, so every wave ends whatever the other waves do (also when fewer workgroups are
// resident than the launch assumed); a table entry of a wave that has not started or has finished is INT_MAX; a wave
// that does not run on the XCD its row stands for does not pace at all.
#pragma once
#include "nsa_common.h"

#define NSA_PACE_IDLE 0x7fffffff
#define NSA_PACE_MAX_SLOTS 512   // waves per XCD the table has room for

struct PaceParams {
  int32_t* table;        // [8][NSA_PACE_MAX_SLOTS] int32, then first_sweep[9]: both written by pace_prepare_kernel.  The kernels
                         // take it as an argument of its own (__restrict__): the polls and publishes are atomics, and an
                         // atomic through a pointer held in a parameter struct makes every array the structs point to a
                         // possible target, after which none of their uniform loads stays a scalar load
  int slots;             // waves per XCD of this launch (multiple of 4, <= NSA_PACE_MAX_SLOTS)
  int window;            // 64-key units a wave may be ahead of the slowest one
  int spin_limit;        // polls after which a wave gives up pacing
  int tokens_per_sweep;  // slots x tokens per wave
  int sweeps_per_stream; // ceil(total_len / tokens_per_sweep)
};
// XCD x runs the sweeps [first_sweep[x], first_sweep[x + 1]) of the (stream, token) order
__device__ __host__ __forceinline__ const int32_t* pace_first_sweep(const int32_t* table) { return table + 8 * NSA_PACE_MAX_SLOTS; }

static inline size_t pace_table_bytes() { return (size_t)(8 * NSA_PACE_MAX_SLOTS + 16) * 4; }

// One workgroup: fills the table with NSA_PACE_IDLE and cuts the sweeps of all streams into eight runs of equal
// estimated cost.  A sweep costs (its tokens) x (fixed_units + position of its last token in 64-key units): a fixed
// part for the blocks every token visits, and a part that grows with the length of the prefix the sweep streams
// through the L2 once.  Every stream has the same sweeps, so the cut is found on one stream's cost curve.
static __global__ __launch_bounds__(1024) void pace_prepare_kernel(int32_t* __restrict__ table, const int32_t* __restrict__ cu, int batch,
                                                            int total_len, int tokens_per_sweep, int sweeps_per_stream, int streams,
                                                            int fixed_units) {
  __shared__ long long part[1024];
  const int tid = threadIdx.x;
  for (int i = tid; i < 8 * NSA_PACE_MAX_SLOTS; i += 1024) table[i] = NSA_PACE_IDLE;
  auto sweep_cost = [&](int k) -> long long {
    const int first = k * tokens_per_sweep, last = min(first + tokens_per_sweep, total_len) - 1;
    const int b = find_sequence(cu, batch, last);
    return (long long)(last - first + 1) * (fixed_units + (last - cu[b]) / 64);
  };
  const int per = (sweeps_per_stream + 1023) / 1024;
  const int k0 = min(sweeps_per_stream, tid * per), k1 = min(sweeps_per_stream, k0 + per);
  long long sum = 0;
  for (int k = k0; k < k1; k++) sum += sweep_cost(k);
  part[tid] = sum;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const long long v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  const long long stream_cost = part[1023], before = part[tid] - sum;
  int32_t* first_sweep = table + 8 * NSA_PACE_MAX_SLOTS;
  if (tid == 0) { first_sweep[0] = 0; first_sweep[8] = sweeps_per_stream * streams; }
  for (int x = 1; x < 8; x++) {
    // the sweep that holds cost x/8 of all streams' total
    const long long target = stream_cost * streams * x / 8;
    const int stream = min((int)(stream_cost > 0 ? target / stream_cost : 0), streams - 1);
    const long long within = target - stream * stream_cost;
    if (within >= before && (within < before + sum || (tid == 1023 && within >= before + sum))) {
      long long run = before;
      int k = k0;
      while (k < k1 && run + sweep_cost(k) <= within) { run += sweep_cost(k); k++; }
      first_sweep[x] = stream * sweeps_per_stream + k;
    }
  }
}

// Which launches are paced, and how.  Measured on single sequences of 64 q / 4 kv heads, 128 columns (forward, ms,
// plain -> paced): top-16 at 16 K tokens 1.31 -> 1.45, 32 K 2.9 -> 2.65, 64 K 9.1 -> 5.7, 128 K 23.7 -> 13.6; top-8 at
// 16 K 0.78 -> 0.78, 32 K 1.63 -> 1.58, 64 K 4.1 -> 3.6, 128 K 10.2 -> 9.1; top-4 (one random block per token) 32 K
// 0.89 -> 1.02, 64 K 1.9 -> 2.4.  The dQ pass: top-16 at 32 K 3.1 -> 3.0, 64 K 9.2 -> 6.5; top-8 unchanged.  Pacing
// pays once the K/V of a kv-head is several times the 4 MiB of an L2 and a token fetches enough blocks that miss it.
// Window: best at 160..240 positions of 32 KiB (K and V rows of 64 keys); below, waves wait for each other (a wave's
// next block is on average a topk-th of its prefix away), above, the L2 loses the window.
static inline bool pace_pays(long long total_len, int head_dim, int topk) { return topk >= 8 && total_len * head_dim * 4 >= (12ll << 20); }
static inline int pace_window_units(int head_dim) { return (int)((25ll << 18) / (64 * head_dim * 4)); }  // 6.25 MiB
static inline int pace_slots() {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  int slots = cus / 8 * 8;   // 8 waves on each of an XCD's compute units
  if (slots < 8) slots = 8;
  return slots > NSA_PACE_MAX_SLOTS ? NSA_PACE_MAX_SLOTS : slots;
}

static inline void pace_fill_params(PaceParams& pp, long long total_len, int slots, int tokens_per_wave, int window_units) {
  pp.slots = slots;
  pp.window = window_units;
  pp.spin_limit = 3000;   // about 3 ms
  pp.tokens_per_sweep = slots * tokens_per_wave;
  pp.sweeps_per_stream = (int)((total_len + pp.tokens_per_sweep - 1) / pp.tokens_per_sweep);
}

static inline void launch_pace_prepare(const PaceParams& pp, const int32_t* cu, int batch, int total_len, int streams, int fixed_units,
                                       hipStream_t stream) {
  pace_prepare_kernel<<<1, 1024, 0, stream>>>(pp.table, cu, batch, total_len, pp.tokens_per_sweep, pp.sweeps_per_stream, streams, fixed_units);
}

struct Pacer {
  int32_t* row;
  int slots, window, spin_limit, me, lane, frontier;

  __device__ __forceinline__ void init(const PaceParams& pp, int32_t* table, int xcd, int slot, int lane_) {
    row = table + xcd * NSA_PACE_MAX_SLOTS;
    slots = pp.slots; window = pp.window; spin_limit = pp.spin_limit; me = slot; lane = lane_; frontier = 0;
    // The table of a row only works as a meeting point if the row's workgroups share one L2, i.e. if workgroup i runs on
    // XCD i % 8 (what the hardware's round-robin dispatch gives: measured, all 2048 waves of a launch).  A wave that finds
    // itself elsewhere does not pace: it would wait on entries it cannot see change.  (A register read, nothing more: an
    // atomic on the table here made the compiler give up scalar loads in the whole kernel, 2.58 -> 2.75 ms.)
    const int my_xcc = __builtin_amdgcn_s_getreg(20 /* HW_REG_XCC_ID */ | (0 << 6) | ((4 - 1) << 11));
    if (my_xcc != xcd) window = NSA_PACE_IDLE;
  }
  // position (in the XCD's running count of 64-key units) of the block this wave turns to next
  __device__ __forceinline__ void publish(int position) {
    // the table of an XCD is written and read through that XCD's L2 only: a store that the L1 writes through ...
    if (lane == 0) __hip_atomic_store(row + me, position, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  // returns once `position` lies within the window of the slowest wave (or pacing has been given up)
  __device__ __forceinline__ void wait(int position) {
    if (position - frontier < window) return;
    for (int spin = 0; spin < spin_limit; spin++) {
      int m = NSA_PACE_IDLE;
      // ... and reads that no L1 can serve: atomic or-with-zero, carried out in the L2 (plain loads marked for
      // workgroup scope were served from stale L1 lines, agent-scope loads and stores cross the fabric)
      for (int i = lane; i < slots; i += 64) m = min(m, __hip_atomic_fetch_or(row + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) m = min(m, __shfl_xor(m, d));
      frontier = __builtin_amdgcn_readfirstlane(m);
      if (position - frontier < window) return;
      __builtin_amdgcn_s_sleep(16);
    }
    window = NSA_PACE_IDLE;  // gave up: never wait again
    frontier = 0;
  }
};

// What the sweep driver needs to know of a token: its row of block ids and the entries not visited yet.  A kernel's
// token state derives from this.
struct SweepToken {
  int my_blk;                 // lane e: entry e0 + e of the token's row of block ids
  unsigned long long todo;    // valid entries of my_blk not visited yet
  int t, pos, qb, e0;         // t < 0: no token; pos: position in the sequence; qb: the token's own block
  const int32_t* ip;          // the token's row of block ids
};

// The persistent loop of a paced kernel.  Every wave of XCD `blockIdx.x & 7` runs that XCD's sweeps in order; in a
// sweep it owns TPW consecutive tokens and visits the union of their valid blocks in ascending order.
//   fetch(sw, ahead, reach)  loads what the tokens of sweep sw bring with them (AHEAD: one sweep early) and returns
//                            the number of 64-key positions the sweep can reach;
//   adopt(tok, ahead, i)     makes token i current (accumulators zeroed, todo set);
//   visit(tok, who, blk, f)  block blk for the tokens in the bit set who; calls f() once the block's loads are issued;
//   finish(tok, i, sw)       writes the token's results.
template <int BS, int TPW, bool AHEAD, typename Tok, typename Ahead, typename Fetch, typename Adopt, typename Visit, typename Finish>
__device__ __forceinline__ void run_paced_sweeps(const PaceParams& pp, int32_t* table, int topk, long long isk, int lane, int slot,
                                                 Fetch fetch, Adopt adopt, Visit visit, Finish finish) {
  const int xcd = blockIdx.x & 7;
  Pacer pc;
  pc.init(pp, table, xcd, slot, lane);
  const int32_t* first_sweep = pace_first_sweep(table);
  const int sw_begin = first_sweep[xcd], sw_end = first_sweep[xcd + 1];
  Ahead ahead[TPW];
  int reach_ahead = 0;
  if (AHEAD && sw_begin < sw_end) fetch(sw_begin, ahead, reach_ahead);
  int origin = 0;  // running count of 64-key units over the sweeps of this XCD
  for (int sw = sw_begin; sw < sw_end; sw++) {
    if (!AHEAD) fetch(sw, ahead, reach_ahead);
    const int reach = reach_ahead;
    Tok tok[TPW];
#pragma unroll
    for (int i = 0; i < TPW; i++) adopt(tok[i], ahead[i], i);
    if (AHEAD && sw + 1 < sw_end) fetch(sw + 1, ahead, reach_ahead);
    // the lowest block any of the wave's tokens has left, and the tokens (bit i: token i) of one sequence that are
    // at it: they are served by one fetch of the block
    auto next_pick = [&](unsigned& who, int& blk) {
      who = 0u; blk = 0x7fffffff;
      int at[TPW];
#pragma unroll
      for (int i = 0; i < TPW; i++) {
        SweepToken& k = tok[i];
        at[i] = 0x7fffffff;
        if (k.t < 0) continue;
        while (!k.todo && k.e0 + 64 < topk) {   // rows longer than 64 entries: next stretch
          k.e0 += 64;
          k.todo = row_stretch(k.ip, isk, topk, k.e0, lane, k.qb, k.my_blk);
        }
        if (k.todo) at[i] = __builtin_amdgcn_readlane(k.my_blk, __builtin_ctzll(k.todo));
        blk = min(blk, at[i]);
      }
      if (blk == 0x7fffffff) return;
      int seq_start = 0;
#pragma unroll
      for (int i = 0; i < TPW; i++) {
        if (at[i] != blk) continue;
        if (!who) seq_start = tok[i].t - tok[i].pos;
        if (tok[i].t - tok[i].pos == seq_start) who |= 1u << i;
      }
    };
    unsigned who;
    int blk;
    next_pick(who, blk);
    int position = who ? origin + ((blk * BS) >> 6) : origin + reach;
    pc.publish(position);
    while (who) {
      pc.wait(position);
#pragma unroll
      for (int i = 0; i < TPW; i++)
        if (who >> i & 1) tok[i].todo = row_visited(tok[i].todo, tok[i].my_blk, blk);
      unsigned who_next;
      int blk_next;
      next_pick(who_next, blk_next);
      position = who_next ? origin + ((blk_next * BS) >> 6) : origin + reach;
      // once this block's loads are on their way the wave no longer needs the L2 to hold its lines
      visit(tok, who, blk, [&] { pc.publish(position); });
      who = who_next; blk = blk_next;
    }
    origin += reach;
#pragma unroll
    for (int i = 0; i < TPW; i++)
      if (tok[i].t >= 0) finish(tok[i], i, sw);
  }
  pc.publish(NSA_PACE_IDLE);
}

// Tokens of sweep sw owned by the wave in `slot`, and the sweep's reach; shared by the kernels' fetch steps.
struct SweepPlace { int stream, base, t_last, reach; };
__device__ __forceinline__ SweepPlace sweep_place(const PaceParams& pp, int sw, const int32_t* __restrict__ cu, int batch, int total_len) {
  SweepPlace s;
  s.stream = sw / pp.sweeps_per_stream;
  s.base = (sw % pp.sweeps_per_stream) * pp.tokens_per_sweep;
  s.t_last = min(s.base + pp.tokens_per_sweep, total_len) - 1;
  // key positions the sweep can reach: those of its last token, or of the sequence that ends inside it
  const int b_lo = find_sequence(cu, batch, s.base), b_hi = find_sequence(cu, batch, s.t_last);
  s.reach = max(max(min(cu[b_lo + 1] - 1, s.t_last) - cu[b_lo], s.t_last - cu[b_hi]) / 64 + 1, 4);
  return s;
}
