/*
 * C ABI of libnsa_hip.so - hand-written gfx950 (MI355X) kernels for the Native Sparse
 * Attention operator path.  Every entry point replaces one Triton launch site (or one
 * torch-op chain) of the reference's native_sparse_attention/ops package; the citation
 * on each declaration names that site.
 *
 * Conventions
 *  - All pointers are device pointers owned by the caller.  The library never allocates,
 *    frees, retains or synchronises; work is enqueued on `stream` (a hipStream_t).
 *  - dtype: NSA_BF16 or NSA_FP16 for q/k/v/x/w/o tensors; accumulation is fp32.
 *  - Strides are in elements; the innermost (head_dim) stride must be 1.
 *  - Varlen tensors are [total_len, heads, head_dim]; cu_seqlens is int32 [batch+1].
 *  - sm_scale may be any finite number (NSA_ERR_BAD_ARG for NaN or infinity).
 *  - Return value: NSA_OK (0) or a negative NSA_ERR_* code; nothing is launched on error.
 *  - Re-entrant: no global state (one exception, stated there: nsa_topk_decode_static).
 */
#ifndef NSA_HIP_H
#define NSA_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NSA_OK 0
#define NSA_ERR_BAD_ARG (-1)      /* null pointer, negative size, inconsistent shapes   */
#define NSA_ERR_UNSUPPORTED (-2)  /* head_dim / block_size / dtype outside the built set */
#define NSA_ERR_WORKSPACE (-3)    /* workspace_bytes smaller than nsa_*_workspace_bytes  */
#define NSA_ERR_LAUNCH (-4)       /* hipGetLastError() after the launch was not success  */
#define NSA_ERR_NOT_READY (-5)    /* nsa_topk_decode_static: first call on this device made while the stream records a graph */

#define NSA_BF16 0
#define NSA_FP16 1

/* Library version (major*10000 + minor*100 + patch). */
int nsa_version(void);

/* ---- topk_sparse_attention -------------------------------------------------------------
 * Forward: replaces forward_kernel launched from _topk_sparse_attention_fwd
 * (native_sparse_attention/ops/triton/topk_sparse_attention.py:828-909).
 *   q,o [T,Hq,D]; k,v [T,Hkv,D]; topk_idx int32 [Hkv,T,topk] (entries <0 or beyond the
 *   query's own block are skipped; the ids of a row are a set: a block listed twice is attended
 *   to once, here and in every pass of the backward); lse fp32 [Hq,T] in base-2 units (contiguous).
 * workspace holds fragment-major copies of K and V (2x their size) and a 16 KiB pacing table:
 * nsa_topk_attn_fwd_workspace_bytes().
 * phases: NSA_FWD_PHASE_ALL, or a subset when the caller re-uses the workspace of a previous
 * call with the same K and V (profiling a single kernel).
 * Schedule: when topk >= 8 and the K/V rows of one kv-head reach 12 MiB (24 K tokens of 128 columns) the attend pass runs
 * as persistent waves whose key positions are kept within a window of each other, so that an XCD's L2 serves
 * most of the block fetches; below that, one wave per token in launch order.  Both give bit-identical
 * results.  Or-ing NSA_FWD_SCHEDULE_PLAIN or NSA_FWD_SCHEDULE_PACED into phases forces one of them.
 */
#define NSA_FWD_PHASE_TRANSPOSE 1
#define NSA_FWD_PHASE_ATTEND 2
#define NSA_FWD_PHASE_ALL 3
#define NSA_FWD_SCHEDULE_PLAIN 8
#define NSA_FWD_SCHEDULE_PACED 16
size_t nsa_topk_attn_fwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_kv_heads, int64_t head_dim);
int nsa_topk_attn_fwd(const void* q, const void* k, const void* v, const int32_t* topk_idx, void* o, float* lse,
                      const int32_t* cu_seqlens, int64_t total_len, int64_t batch, int64_t num_q_heads,
                      int64_t num_kv_heads, int64_t head_dim, int64_t topk, int64_t block_size, int64_t q_stride_n,
                      int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n,
                      int64_t v_stride_h, int64_t idx_stride_h, int64_t idx_stride_n, int64_t idx_stride_k,
                      int64_t o_stride_n, int64_t o_stride_h, float sm_scale, int dtype, void* workspace,
                      size_t workspace_bytes, int phases, void* stream);

/* Backward: replaces backward_sum_o_do, count_query + reorder_topk_idx (with their host
 * synchronisations and argsort), backward_dkdv and backward_dq launched from
 * _topk_sparse_attention_bwd (native_sparse_attention/ops/triton/topk_sparse_attention.py:912-1109).
 *   o,dout,dq [T,Hq,D]; dk,dv [T,Hkv,D]; lse as produced by nsa_topk_attn_fwd.
 *   strides: HOST array of 19 element strides in the order
 *     q(n,h) k(n,h) v(n,h) o(n,h) dout(n,h) idx(h,n,k) dq(n,h) dk(n,h) dv(n,h).
 *   out_segment_offsets / out_queries: optional (both or neither) device buffers that
 *   receive the "KV block -> queries" reverse index built on the way:
 *     segments = nsa_topk_reverse_index_segments(); segment s = kv_head*(T/block+batch) + global block;
 *     out_segment_offsets int32 [segments+1]; out_queries int32 [Hkv*T*topk], the tokens of
 *     segment s are out_queries[off[s] : off[s+1]], ascending.  For block_size 256 the index (and the
 *     dK/dV pass) works on the four 64-key pieces of every block: read `block` as 64 above, out_queries
 *     then holds up to 4*Hkv*T*topk entries, and a query appears under the pieces at or before its position.
 * dK/dV are reduced in a fixed order (no atomics): results are run-to-run deterministic.
 * phases: NSA_BWD_PHASE_ALL, or a subset to re-run single passes on a workspace that an
 * earlier call with identical arguments has already filled (PREP = delta, the (lse, delta) pairs laid out
 * per token for the dK/dV pass, and the reverse index).
 * When PREP and DQ run in the same call, delta = rowsum(o * dout) is formed inside the dQ pass
 * (which runs before dK/dV) instead of by a pass of its own (another summation order: the stored values agree to
 * fp32 rounding).
 * Token strides of q and dout, and group_size * their head strides + D, must fit 31 bits.
 * The dQ pass has the two schedules of the forward (same rule, same bit-identical results);
 * NSA_BWD_SCHEDULE_PLAIN / NSA_BWD_SCHEDULE_PACED or-ed into phases force one of them.
 */
#define NSA_BWD_PHASE_PREP 1
#define NSA_BWD_PHASE_DKDV 2
#define NSA_BWD_PHASE_DQ 4
#define NSA_BWD_PHASE_ALL 7
#define NSA_BWD_SCHEDULE_PLAIN 8
#define NSA_BWD_SCHEDULE_PACED 16
size_t nsa_topk_attn_bwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                         int64_t head_dim, int64_t topk, int64_t block_size);
int64_t nsa_topk_reverse_index_segments(int64_t total_len, int64_t batch, int64_t num_kv_heads, int64_t block_size);
int nsa_topk_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                      const int32_t* topk_idx, const int32_t* cu_seqlens, void* dq, void* dk, void* dv, int64_t total_len,
                      int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t topk,
                      int64_t block_size, const int64_t* strides, float sm_scale, int dtype, void* workspace,
                      size_t workspace_bytes, int32_t* out_segment_offsets, int32_t* out_queries, int phases,
                      void* stream);

/* ---- weightedpool_compress / avgpool_compress ---------------------------------------------
 * Forward: replaces sliding_pool_fwd_kernel (native_sparse_attention/ops/triton/weighted_pool.py:24-85,
 * launched at :218-236).  x [total_x,H,D]; w [H,kernel_size] in the dtype of x, or NULL for the
 * average; y [total_y,H,D]; y_cu_seqlens int32 [batch+1] as computed by get_compressed_seqlens
 * (ops/triton/utils.py:25-37).  The positional-embedding bias stays in the caller as in the reference.
 */
int nsa_pool_fwd(const void* x, const void* w, void* y, const int32_t* cu_seqlens, const int32_t* y_cu_seqlens,
                 int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim, int64_t kernel_size,
                 int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h, int64_t y_stride_n, int64_t y_stride_h,
                 int64_t w_stride_h, int dtype, void* stream);
/* The same with the reference's bias step folded in: replaces the `y + bias.unsqueeze(0)` that follows the launch
 * (weighted_pool.py:326-329 for the weighted pool, :361 for the average).  bias [H, D] in the dtype of x (NULL: none),
 * e.g. einsum(pe, w) or mean(pe): the pooled value is rounded to the element type, then the sum, as the tensor
 * expression does, so the result is bit-identical to nsa_pool_fwd followed by the addition.
 */
int nsa_pool_fwd_bias(const void* x, const void* w, const void* bias, void* y, const int32_t* cu_seqlens,
                      const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                      int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                      int64_t y_stride_n, int64_t y_stride_h, int64_t w_stride_h, int64_t bias_stride_h, int dtype,
                      void* stream);
/* Backward: replaces sliding_pool_dxdw_kernel (:89-179, launched at :262-292) and the dw.sum(1)
 * that follows (:297).  dx is a gather over the windows covering each token (no atomics);
 * dw (NULL iff w is NULL) is reduced over fp32 per-tile partials held in the workspace.
 */
size_t nsa_pool_bwd_workspace_bytes(int64_t total_y, int64_t num_heads, int64_t kernel_size);
int nsa_pool_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, const int32_t* cu_seqlens,
                 const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                 int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                 int64_t dy_stride_n, int64_t dy_stride_h, int64_t dx_stride_n, int64_t dx_stride_h, int64_t w_stride_h,
                 int64_t dw_stride_h, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- linear_compress ----------------------------------------------------------------------------
 * Forward: replaces linear_compress_fwd_kernel (native_sparse_attention/ops/triton/linear_compress.py:27-136,
 * launched at :379-410).  x [total_x,H,D]; w [H, kernel_size*D, D] contiguous; y [total_y,H,D].
 * The forward adds the shares of its waves in LDS and needs no workspace: the size query returns 0 and the
 * workspace arguments are ignored (both stay so that existing callers keep working).
 */
size_t nsa_linear_compress_fwd_workspace_bytes(int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim, int64_t kernel_size);
int nsa_linear_compress_fwd(const void* x, const void* w, void* y, const int32_t* cu_seqlens, const int32_t* y_cu_seqlens,
                            int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim,
                            int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                            int64_t y_stride_n, int64_t y_stride_h, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream);
/* The same with the reference's bias step folded in: replaces the `y + bias.unsqueeze(0)` after the launch
 * (linear_compress.py:520-524).  bias [H, D] in the dtype of x (NULL: none), i.e. pe[h].flatten() @ w[h]; rounded as
 * the tensor expression rounds (product first, then the sum).  Needs no workspace.
 */
int nsa_linear_compress_fwd_bias(const void* x, const void* w, const void* bias, void* y, const int32_t* cu_seqlens,
                                 const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch,
                                 int64_t num_heads, int64_t head_dim, int64_t kernel_size, int64_t kernel_stride,
                                 int64_t x_stride_n, int64_t x_stride_h, int64_t y_stride_n, int64_t y_stride_h,
                                 int64_t bias_stride_h, int dtype, void* stream);
/* Backward: replaces linear_compress_bwd_kernel and its fp32 atomic adds (:140-306, launched at
 * :449-480).  dx [total_x,H,D]; dw [H, kernel_size*D, D] contiguous, both in the dtype of x.
 * Gather formulation, no atomics: reproducible.
 */
int nsa_linear_compress_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, const int32_t* cu_seqlens,
                            const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                            int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                            int64_t dy_stride_n, int64_t dy_stride_h, int64_t dx_stride_n, int64_t dx_stride_h, int dtype,
                            void* stream);

/* ---- compressed_attention --------------------------------------------------------------------
 * Forward: replaces forward_kernel launched from _compressed_attention_fwd
 * (native_sparse_attention/ops/triton/compressed_attention.py:538-640).  q,o [Tq,Hq,D];
 * k,v [Tk,Hkv,D] compressed keys/values; query position i of a sequence sees its compressed key c
 * iff c*kernel_stride + kernel_size - 1 <= i; rows that see nothing get o = 0, lse = -inf.
 * lse fp32 [Hq,Tq] base-2.  strides (HOST int64[8]): q(n,h) k(n,h) v(n,h) o(n,h).
 */
int nsa_cmp_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens_q,
                     const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                     int64_t num_kv_heads, int64_t head_dim, int64_t kernel_size, int64_t kernel_stride,
                     const int64_t* strides, float sm_scale, int dtype, void* stream);
/* Block selection: replaces score_kernel + _transform_score_kernel + torch.topk/sort/mask
 * (:852-1179 and :1263-1292; the dense [Hkv,Tq,Tk] score tensor is never materialised).
 * out_topk_idx int32 [Hkv,Tq,k_out], k_out <= ceil(max_seqlen_q/block_size): ids of the k_out
 * best-scoring blocks per (kv head, token) in ascending order, -1 padded; init_blocks first and
 * local_blocks last causal blocks are always selected.  strides (HOST int64[9]):
 * q(n,h) k(n,h) 0 0 idx(h,n,k).
 */
int nsa_cmp_attn_select(const void* q, const void* k, const float* lse, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                        int32_t* out_topk_idx, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                        int64_t num_kv_heads, int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t block_size,
                        int64_t k_out, int64_t max_seqlen_q, int64_t init_blocks, int64_t local_blocks, const int64_t* strides,
                        float sm_scale, int dtype, void* stream);
/* Backward: replaces backward_sum_o_do, backward_dkdv (+ the .sum(0) over bf16 per-head partials)
 * and backward_dq launched from _compressed_attention_bwd (:643-780).
 * strides (HOST int64[16]): q k v o dout dq dk dv, (n,h) each.
 */
size_t nsa_cmp_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                        int64_t head_dim);
int nsa_cmp_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq, void* dk,
                     void* dv, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k,
                     int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t kernel_size,
                     int64_t kernel_stride, const int64_t* strides, float sm_scale, int dtype, void* workspace,
                     size_t workspace_bytes, void* stream);

/* ---- sliding-window attention ----------------------------------------------------------------
 * Stands in for flash_attn_varlen_func(..., causal=True, window_size=(window_size, -1)) as called from
 * native_sparse_attention/infer/inference_func.py:180-190 (prefill) and
 * native_sparse_attention/module/native_sparse_attention.py:213-223 (training; a third-party kernel
 * in the reference): position i attends to keys j of its sequence with i - window_size <= j <= i.
 * Forward strides (HOST int64[8]): q(n,h) k(n,h) v(n,h) o(n,h); lse fp32 [Hq,T] base-2.
 * Backward strides (HOST int64[16]): q k v o dout dq dk dv, (n,h) each; workspace 256-byte aligned.
 */
int nsa_window_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens,
                        int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                        int64_t window_size, const int64_t* strides, float sm_scale, int dtype, void* stream);
size_t nsa_window_attn_bwd_workspace_bytes(int64_t total_len, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim);
int nsa_window_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq, void* dk,
                        void* dv, const int32_t* cu_seqlens, int64_t total_len, int64_t batch, int64_t num_q_heads,
                        int64_t num_kv_heads, int64_t head_dim, int64_t window_size, const int64_t* strides, float sm_scale,
                        int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- dense varlen attention ------------------------------------------------------------------
 * Replaces _flash_attention_fwd / _flash_attention_bwd behind flash_attention_varlen
 * (native_sparse_attention/ops/triton/flash_attention.py:560-935): q [total_q, Hq, D], k/v [total_k, Hkv, D],
 * separate cu_seqlens for queries and keys; causal != 0: query i of a sequence sees keys j <= i of the same
 * sequence (both counted from their start, :117-131), otherwise every key.  lse fp32 [Hq, total_q], base 2.
 * Strides as for the sliding-window entry points (HOST int64[8] forward, int64[16] backward).
 */
int nsa_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* cu_seqlens_q,
                       const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads,
                       int64_t num_kv_heads, int64_t head_dim, int causal, const int64_t* strides, float sm_scale, int dtype,
                       void* stream);
size_t nsa_flash_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                          int64_t head_dim);
int nsa_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse, void* dq, void* dk,
                       void* dv, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int64_t total_q, int64_t total_k,
                       int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int causal, const int64_t* strides,
                       float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- compressed sequence lengths ---------------------------------------------------------------
 * get_compressed_seqlens of native_sparse_attention/ops/triton/utils.py:25-37 in one launch:
 * y_seqlens[b] = floor((len_b - kernel_size) / kernel_stride) + 1, or 0 when len_b < kernel_size; y_cu_seqlens =
 * its cumulative sum with a leading 0 (int32 [batch] and [batch + 1], device).
 */
int nsa_compressed_seqlens(const int32_t* cu_seqlens, int64_t batch, int64_t kernel_size, int64_t kernel_stride,
                           int32_t* y_seqlens, int32_t* y_cu_seqlens, void* stream);

/* ---- rotary position embedding ---------------------------------------------------------------
 * Replaces RotaryEmbedding.forward of native_sparse_attention/module/rope.py:199-209 (cos/sin tables
 * :120-152, per-sequence positions :154-197): x, out [n_rows, H, D] (strides in elements, multiples of 8),
 * inv_freq fp32 [D/2] on the device.  step == 0: row n is token (n - cu_seqlens[b]) of sequence b and is
 * rotated for position (n - cu_seqlens[b]) * stride.  step > 0 (decode): n_rows == batch, row b is rotated
 * for position (cu_seqlens[b+1] - cu_seqlens[b] + step - 1) * stride.  step < 0: cu_seqlens is instead an
 * int32 [n_rows] array of position indices on the device (row n is rotated for position index * stride; batch is
 * ignored), which lets a decode step take positions from the cache lengths without a host read.  inverse != 0
 * applies the transposed rotation (the gradient of the forward call).
 */
int nsa_rope(const void* x, void* out, const float* inv_freq, const int32_t* cu_seqlens, int64_t n_rows, int64_t batch,
             int64_t num_heads, int64_t head_dim, int64_t x_stride_n, int64_t x_stride_h, int64_t o_stride_n, int64_t o_stride_h,
             int64_t step, int64_t stride, float attention_scaling, int inverse, int dtype, void* stream);

/* ---- KV-cache slabs ----------------------------------------------------------------------------
 * Device-side counterparts of NSACache.prepare_compress / update_kv
 * (native_sparse_attention/module/kv_cache.py:233-302, 340-449) and of its slab fill kernel (:453-555).
 * A slab is a contiguous [2 (key, value), max_batch, rows, Hkv, D] array of 2-byte elements with an int32
 * length per sequence; lengths are read and written on the device only.  Token tensors are [n, Hkv, D]
 * with element strides (n, h), multiples of 8, D contiguous.
 *
 * nsa_cache_fill (prefill): for every sequence b, rows row_begin[b] .. row_end[b]-1 of key/value (cu_src gives
 *   the sequence of every source row) go to slab[:, b, 0..]; slab_len[b] = row_end[b] - row_begin[b].
 * nsa_cache_stage_token (decode, before compression): a staging window that holds kernel_size rows is shifted
 *   left by kernel_stride, then the new token [batch, Hkv, D] is appended and stage_len incremented.
 * nsa_cache_commit_token (decode, after compression and rotary embedding): tokens[6] = HOST array of device
 *   pointers {compressed k, v, full-length k, v, sliding k, v}, strides = HOST int64[12] (n, h) for each; the
 *   compressed pair is appended where stage_len[b] == kernel_size, the full-length pair is appended, the
 *   sliding pair is written at row sliding_len[b] % window_size; the three lengths are incremented.
 */
int nsa_cache_fill(const void* key, const void* value, const int32_t* cu_src, const int32_t* row_begin, const int32_t* row_end,
                   void* slab, int32_t* slab_len, int64_t total_rows, int64_t batch, int64_t num_kv_heads, int64_t head_dim,
                   int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h, int64_t max_batch,
                   int64_t slab_rows, void* stream);
int nsa_cache_stage_token(const void* key, const void* value, void* stage_slab, int32_t* stage_len, int64_t batch,
                          int64_t num_kv_heads, int64_t head_dim, int64_t k_stride_b, int64_t k_stride_h, int64_t v_stride_b,
                          int64_t v_stride_h, int64_t max_batch, int64_t kernel_size, int64_t kernel_stride, void* stream);
/* Plain KV cache (KVCache.update_kv of module/kv_cache.py:56-122): the new token of sequence b goes to row
 * slab_len[b] of slab[:, b], slab_len[b] += 1 (nothing is written once a sequence fills its rows). */
int nsa_cache_append_token(const void* key, const void* value, void* slab, int32_t* slab_len, int64_t batch, int64_t num_kv_heads,
                           int64_t head_dim, int64_t k_stride_b, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_h,
                           int64_t max_batch, int64_t slab_rows, void* stream);
int nsa_cache_commit_token(const void* const* tokens, const int64_t* strides, const int32_t* stage_len, void* compress_slab,
                           int32_t* compress_len, void* sparse_slab, int32_t* sparse_len, void* sliding_slab, int32_t* sliding_len,
                           int64_t batch, int64_t num_kv_heads, int64_t head_dim, int64_t max_batch, int64_t kernel_size,
                           int64_t compress_rows, int64_t sparse_rows, int64_t window_size, void* stream);

/* One decode step's work ahead of its attention branches in a single launch, for caches whose compression is
 * a (weighted) average pool: nsa_cache_stage_token, the pooling of a completed window
 * (ops/triton/weighted_pool.py:182-279 on the staging slab, as compress_infer of infer/inference_func.py:27-75
 * calls it), the three rotations of infer/nsa_inference.py:96-112 with positions sparse_len[b] (query, key) and
 * compress_len[b] * kernel_stride (compressed key), and nsa_cache_commit_token.  q [batch,Hq,D], k, v
 * [batch,Hkv,D]; q_out receives the rotated query.  pool_weight_k / pool_weight_v: contiguous [Hkv,kernel_size]
 * or NULL for the plain average; bias_k: optional contiguous [Hkv,D] added to the pooled key (the intra-block
 * position term).  strides: HOST int64[8] = q(b,h) k(b,h) v(b,h) q_out(b,h).  Cache contents, lengths and the
 * rotated query equal those of the separate entry points bit for bit.
 */
int nsa_decode_prepare(const void* q, const void* k, const void* v, void* q_out, const void* pool_weight_k,
                       const void* pool_weight_v, const void* bias_k, const float* inv_freq, float attention_scaling,
                       void* stage_slab, int32_t* stage_len, void* compress_slab, int32_t* compress_len, void* sparse_slab,
                       int32_t* sparse_len, void* sliding_slab, int32_t* sliding_len, int64_t batch, int64_t num_q_heads,
                       int64_t num_kv_heads, int64_t head_dim, const int64_t* strides, int64_t max_batch, int64_t kernel_size,
                       int64_t kernel_stride, int64_t compress_rows, int64_t sparse_rows, int64_t window_size, int dtype,
                       void* stream);

/* The selected-block branch, the sliding-window branch and the gated sum of a decode step in two launches
 * (one for the partials of both branches, one for both merges and the gate) instead of five: the calls of
 * topk_sparse_attention_infer and sliding_window_attention_infer (infer/inference_func.py:140-202) and the gate
 * expression of infer/nsa_inference.py:146-150.  Arguments as for nsa_topk_decode / nsa_dense_decode /
 * nsa_gate_combine; cmp_out is the compressed branch's output [batch,Hq,D]; o_topk / o_window receive the two
 * branch outputs, out the gated sum.  strides: HOST int64[28] =
 *   q(b,h) sparse_k(b,n,h) sparse_v(b,n,h) idx(h,b,k) window_k(b,n,h) window_v(b,n,h) cmp_out(b,h) gate(b,h,k)
 *   out(b,h) o_topk(b,h) o_window(b,h).
 * Every result equals that of the separate entry points bit for bit.
 */
size_t nsa_decode_branches_gate_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                                int64_t window_rows, int64_t topk, int64_t block_size);
int nsa_decode_branches_gate(const void* q, const void* sparse_k, const void* sparse_v, const int32_t* sparse_len,
                             const int32_t* topk_idx, const void* window_k, const void* window_v, const int32_t* window_len,
                             const void* cmp_out, const void* gate, void* out, void* o_topk, void* o_window, int64_t batch,
                             int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t sparse_rows,
                             int64_t window_rows, int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale,
                             int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- gated sum of the three branches -----------------------------------------------------------
 * out[n, h, :] = gate[n, h, 0] * branch0 + gate[n, h, 1] * branch1 + gate[n, h, 2] * branch2, rounded step by
 * step like the tensor expression of native_sparse_attention/infer/nsa_inference.py:146-150.
 * strides (HOST int64[11]): gate (n, h, k), branch0 (n, h), branch1 (n, h), branch2 (n, h), out (n, h).
 */
int nsa_gate_combine(const void* gate, const void* branch0, const void* branch1, const void* branch2, void* out, int64_t n_rows,
                     int64_t num_q_heads, int64_t head_dim, const int64_t* strides, int dtype, void* stream);

/* Backward of the gated sum as autograd derives it from native_sparse_attention/module/native_sparse_attention.py:228-232:
 * dbranch_i = gate[..., i] * dout, dgate[n, h, i] = sum over head_dim of dout * branch_i (products rounded to the
 * element type, fp32 sum).  dgate [n_rows, Hq, 3] and the three dbranch [n_rows, Hq, D] are written densely.
 * strides (HOST int64[11]): gate (n, h, k), branch0 (n, h), branch1 (n, h), branch2 (n, h), dout (n, h).
 */
int nsa_gate_combine_bwd(const void* gate, const void* branch0, const void* branch1, const void* branch2, const void* dout,
                         void* dgate, void* dbranch0, void* dbranch1, void* dbranch2, int64_t n_rows, int64_t num_q_heads,
                         int64_t head_dim, const int64_t* strides, int dtype, void* stream);

/* ---- decode (one query per sequence over KV-cache slabs [B, slab_len, Hkv, D]) ---------------
 * strides: HOST int64 array: q(b,h) k(b,n,h) v(b,n,h) o(b,h) [+ idx(h,b,k) for the entry points
 * that read or write topk ids] = 10 or 13 values.  q/k/v strides must be multiples of 8.
 *
 * nsa_dense_decode replaces decode_kernel (native_sparse_attention/ops/triton/flash_attention_decode.py:23-139,
 * launched at :186-216): attention over the first seqlens[b] rows of the slab.
 */
size_t nsa_dense_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len);
int nsa_dense_decode(const void* q, const void* k, const void* v, const int32_t* seqlens, void* o, int64_t batch,
                     int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len, const int64_t* strides,
                     float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream);
/* nsa_topk_decode replaces forward_kernel (native_sparse_attention/ops/triton/topk_sparse_attention_decode.py:23-148,
 * launched at :199-236): topk_idx int32 [Hkv,B,topk]; ids < 0 or beyond block (seqlens[b]-1)/block_size
 * are skipped; keys >= seqlens[b] are masked.
 */
size_t nsa_topk_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t topk,
                                       int64_t block_size);
int nsa_topk_decode(const void* q, const void* k, const void* v, const int32_t* topk_idx, const int32_t* seqlens, void* o,
                    int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len, int64_t topk,
                    int64_t block_size, const int64_t* strides, float sm_scale, int dtype, void* workspace,
                    size_t workspace_bytes, void* stream);
/* nsa_topk_decode_static: nsa_topk_decode for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * arguments and results as nsa_topk_decode, without the workspace: the split-K partials live in a device array
 * of NSA_TOPK_DECODE_STATIC_MAX_BYTES that the library holds on every GPU it runs on until the process ends
 * (this entry point is the library's one piece of global state).  Returns NSA_ERR_WORKSPACE, and launches
 * nothing, when nsa_topk_decode_workspace_bytes(...) of the call exceeds that size.  All calls on one GPU share
 * the array: calls that may overlap on one GPU (different streams, different threads) race and must be
 * serialised by the caller.  Nothing is allocated, freed or cleared; the first call on a device looks the
 * array's address up (make that call outside a graph capture).
 */
#define NSA_TOPK_DECODE_STATIC_MAX_BYTES (4u << 20)
int nsa_topk_decode_static(const void* q, const void* k, const void* v, const int32_t* topk_idx, const int32_t* seqlens, void* o,
                           int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len,
                           int64_t topk, int64_t block_size, const int64_t* strides, float sm_scale, int dtype, void* stream);
/* nsa_cmp_decode replaces the torch-op chain of compressed_attention_decode
 * (native_sparse_attention/ops/torch/compressed_attention_decode.py:65-153, with transform_score :21-62):
 * attention over the first compress_seqlens[b] rows of the compressed slab, then (if out_topk_idx is
 * not NULL) block scores and the k_out best block ids per (kv head, sequence), ascending, ids beyond
 * block (seqlens[b]-1)/block_size replaced by -1.  max_seqlen = max(seqlens) (host value, fixes the
 * number of blocks); k_out <= min(64, ceil(max_seqlen/block_size)).
 */
size_t nsa_cmp_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t slab_len);
int nsa_cmp_decode(const void* q, const void* k, const void* v, const int32_t* seqlens, const int32_t* compress_seqlens, void* o,
                   int32_t* out_topk_idx, int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                   int64_t slab_len, int64_t kernel_size, int64_t kernel_stride, int64_t block_size, int64_t k_out,
                   int64_t max_seqlen, int64_t init_blocks, int64_t local_blocks, const int64_t* strides, float sm_scale,
                   int dtype, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NSA_HIP_H */
