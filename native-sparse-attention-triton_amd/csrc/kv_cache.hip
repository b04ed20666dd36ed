// KV-cache slab maintenance for NSA inference, entirely stream-ordered: no length is read back by the host.
//
// A slab is a contiguous [2 (key, value), max_batch, rows, Hkv, D] array of 2-byte elements with an int32
// length per sequence.  Three kernels cover the update rules:
//   fill    (prefill)  slab[:, b, 0 : end[b]-begin[b]] = key/value[begin[b] : end[b]], len[b] = end[b]-begin[b]
//   stage   (decode, before compression)  a full staging window is shifted left by kernel_stride, then the
//           new token is appended
//   commit  (decode, after compression and rotary embedding)  the candidate compressed token is appended for
//           sequences whose staging window is full, the new token is appended to the full-length slab and
//           written into the sliding ring at len % window
// All of it is byte movement, bound by HBM (a few KiB per sequence and step).
#include "nsa_common.h"

typedef unsigned short u16;

__device__ __forceinline__ void copy_row(u16* __restrict__ dst, const u16* __restrict__ src, long long src_hs, int H, int D, int tid, int nt) {
  // dst is [H, D] contiguous, src has head stride src_hs; 16-byte pieces
  const int per = D / 8;
  for (int i = tid; i < H * per; i += nt) {
    const int h = i / per, c = i % per;
    *reinterpret_cast<uint4*>(dst + (long long)h * D + 8 * c) = *reinterpret_cast<const uint4*>(src + (long long)h * src_hs + 8 * c);
  }
}

struct FillParams {
  const u16* key; const u16* value; const int32_t* cu_src; const int32_t* begin; const int32_t* end; u16* slab; int32_t* len;
  int total_rows, batch, H, D, max_batch, rows;
  long long ksn, ksh, vsn, vsh;
};

__global__ __launch_bounds__(128) void cache_fill_kernel(FillParams p) {
  const int t = blockIdx.x, tid = threadIdx.x;
  if (t == 0)
    for (int b = tid; b < p.batch; b += 128) p.len[b] = max(p.end[b] - p.begin[b], 0);
  if (t >= p.total_rows) return;
  const int b = find_sequence(p.cu_src, p.batch, t);
  const int r = t - p.begin[b];
  if (t < p.begin[b] || t >= p.end[b] || r >= p.rows) return;
  const long long row = ((long long)b * p.rows + r) * p.H * p.D;
  const long long kv = (long long)p.max_batch * p.rows * p.H * p.D;
  copy_row(p.slab + row, p.key + (long long)t * p.ksn, p.ksh, p.H, p.D, tid, 128);
  copy_row(p.slab + kv + row, p.value + (long long)t * p.vsn, p.vsh, p.H, p.D, tid, 128);
}

struct StageParams {
  const u16* key; const u16* value; u16* slab; int32_t* len;
  int H, D, max_batch, ks, st;
  long long ksn, ksh, vsn, vsh;
};

__global__ __launch_bounds__(256) void cache_stage_kernel(StageParams p) {
  const int b = blockIdx.x, tid = threadIdx.x;
  const long long HD = (long long)p.H * p.D;
  const long long kv = (long long)p.max_batch * p.ks * HD;
  u16* base = p.slab + (long long)b * p.ks * HD;
  int n = p.len[b];
  __syncthreads();  // every wave holds the old length before thread 0 stores the new one
  if (n == p.ks) {
    // rows [st, ks) move to [0, ks - st), st rows at a time: a group's source rows are the next group's
    // destination, so every group is read completely before the next one is written
    const int per = (int)(p.st * HD / 8);  // 16-byte pieces of one group of st rows
    for (int g = 0; (g + 1) * p.st < p.ks; g++) {
      for (int which = 0; which < 2; which++) {
        u16* s = base + which * kv;
        for (int i = tid; i < per; i += 256)
          *reinterpret_cast<uint4*>(s + (long long)g * p.st * HD + 8ll * i) = *reinterpret_cast<const uint4*>(s + (long long)(g + 1) * p.st * HD + 8ll * i);
      }
      __syncthreads();
    }
    n -= p.st;
  }
  copy_row(base + (long long)n * HD, p.key + (long long)b * p.ksn, p.ksh, p.H, p.D, tid, 256);
  copy_row(base + kv + (long long)n * HD, p.value + (long long)b * p.vsn, p.vsh, p.H, p.D, tid, 256);
  if (tid == 0) p.len[b] = n + 1;
}

struct CommitParams {
  const u16* src[6];  // compressed k, v; full-length k, v; sliding k, v: [batch, H, D] each
  long long sn[6], sh[6];
  const int32_t* stage_len;
  u16* cmp_slab; int32_t* cmp_len; u16* full_slab; int32_t* full_len; u16* ring_slab; int32_t* ring_len;
  int H, D, max_batch, ks, cmp_rows, full_rows, window;
};

__global__ __launch_bounds__(256) void cache_commit_kernel(CommitParams p) {
  const int b = blockIdx.x, tid = threadIdx.x;
  const long long HD = (long long)p.H * p.D;
  const int nc = p.cmp_len[b], nf = p.full_len[b], nr = p.ring_len[b];
  const bool new_cmp = p.stage_len[b] == p.ks && nc < p.cmp_rows;
  __syncthreads();  // every wave holds the old lengths before thread 0 stores the new ones
  if (new_cmp) {
    const long long row = ((long long)b * p.cmp_rows + nc) * HD, kv = (long long)p.max_batch * p.cmp_rows * HD;
    copy_row(p.cmp_slab + row, p.src[0] + (long long)b * p.sn[0], p.sh[0], p.H, p.D, tid, 256);
    copy_row(p.cmp_slab + kv + row, p.src[1] + (long long)b * p.sn[1], p.sh[1], p.H, p.D, tid, 256);
  }
  if (nf < p.full_rows) {
    const long long row = ((long long)b * p.full_rows + nf) * HD, kv = (long long)p.max_batch * p.full_rows * HD;
    copy_row(p.full_slab + row, p.src[2] + (long long)b * p.sn[2], p.sh[2], p.H, p.D, tid, 256);
    copy_row(p.full_slab + kv + row, p.src[3] + (long long)b * p.sn[3], p.sh[3], p.H, p.D, tid, 256);
  }
  {
    const long long row = ((long long)b * p.window + nr % p.window) * HD, kv = (long long)p.max_batch * p.window * HD;
    copy_row(p.ring_slab + row, p.src[4] + (long long)b * p.sn[4], p.sh[4], p.H, p.D, tid, 256);
    copy_row(p.ring_slab + kv + row, p.src[5] + (long long)b * p.sn[5], p.sh[5], p.H, p.D, tid, 256);
  }
  if (tid == 0) {
    if (new_cmp) p.cmp_len[b] = nc + 1;
    if (nf < p.full_rows) p.full_len[b] = nf + 1;
    p.ring_len[b] = nr + 1;
  }
}

struct AppendParams {
  const u16* key; const u16* value; u16* slab; int32_t* len;
  int H, D, max_batch, rows;
  long long ksn, ksh, vsn, vsh;
};

// plain KV cache: the new token of every sequence goes to row len[b], len[b] += 1
__global__ __launch_bounds__(256) void cache_append_kernel(AppendParams p) {
  const int b = blockIdx.x, tid = threadIdx.x;
  const long long HD = (long long)p.H * p.D;
  const int n = p.len[b];
  __syncthreads();  // every wave holds the old length before thread 0 stores the new one
  if (n >= p.rows) return;
  const long long row = ((long long)b * p.rows + n) * HD, kv = (long long)p.max_batch * p.rows * HD;
  copy_row(p.slab + row, p.key + (long long)b * p.ksn, p.ksh, p.H, p.D, tid, 256);
  copy_row(p.slab + kv + row, p.value + (long long)b * p.vsn, p.vsh, p.H, p.D, tid, 256);
  if (tid == 0) p.len[b] = n + 1;
}

static bool rows_ok(const void* ptr, int64_t sn, int64_t sh) { return ptr && (uintptr_t)ptr % 16 == 0 && sn % 8 == 0 && sh % 8 == 0; }

extern "C" int nsa_cache_fill(const void* key, const void* value, const int32_t* cu_src, const int32_t* row_begin, const int32_t* row_end,
                              void* slab, int32_t* slab_len, int64_t total_rows, int64_t batch, int64_t num_kv_heads, int64_t head_dim,
                              int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h, int64_t max_batch,
                              int64_t slab_rows, void* stream) {
  if (!cu_src || !row_begin || !row_end || !slab || !slab_len) return NSA_ERR_BAD_ARG;
  if (total_rows < 0 || total_rows >= (1ll << 31) || batch <= 0 || batch > max_batch || num_kv_heads <= 0 || head_dim <= 0 || slab_rows <= 0) return NSA_ERR_BAD_ARG;
  if (head_dim % 8 != 0 || (uintptr_t)slab % 16 != 0) return NSA_ERR_UNSUPPORTED;
  if (total_rows > 0 && (!rows_ok(key, k_stride_n, k_stride_h) || !rows_ok(value, v_stride_n, v_stride_h))) return NSA_ERR_UNSUPPORTED;
  FillParams p;
  p.key = (const u16*)key; p.value = (const u16*)value; p.cu_src = cu_src; p.begin = row_begin; p.end = row_end; p.slab = (u16*)slab; p.len = slab_len;
  p.total_rows = (int)total_rows; p.batch = (int)batch; p.H = (int)num_kv_heads; p.D = (int)head_dim; p.max_batch = (int)max_batch; p.rows = (int)slab_rows;
  p.ksn = k_stride_n; p.ksh = k_stride_h; p.vsn = v_stride_n; p.vsh = v_stride_h;
  cache_fill_kernel<<<(unsigned)(total_rows > 0 ? total_rows : 1), 128, 0, (hipStream_t)stream>>>(p);
  return nsa_check_launch();
}

extern "C" int nsa_cache_stage_token(const void* key, const void* value, void* stage_slab, int32_t* stage_len, int64_t batch,
                                     int64_t num_kv_heads, int64_t head_dim, int64_t k_stride_b, int64_t k_stride_h, int64_t v_stride_b,
                                     int64_t v_stride_h, int64_t max_batch, int64_t kernel_size, int64_t kernel_stride, void* stream) {
  if (!stage_slab || !stage_len || batch <= 0 || batch > max_batch || num_kv_heads <= 0 || kernel_size <= 0 || kernel_stride <= 0) return NSA_ERR_BAD_ARG;
  if (kernel_size % kernel_stride != 0) return NSA_ERR_BAD_ARG;
  if (head_dim % 8 != 0 || (uintptr_t)stage_slab % 16 != 0 || !rows_ok(key, k_stride_b, k_stride_h) || !rows_ok(value, v_stride_b, v_stride_h)) return NSA_ERR_UNSUPPORTED;
  StageParams p;
  p.key = (const u16*)key; p.value = (const u16*)value; p.slab = (u16*)stage_slab; p.len = stage_len;
  p.H = (int)num_kv_heads; p.D = (int)head_dim; p.max_batch = (int)max_batch; p.ks = (int)kernel_size; p.st = (int)kernel_stride;
  p.ksn = k_stride_b; p.ksh = k_stride_h; p.vsn = v_stride_b; p.vsh = v_stride_h;
  cache_stage_kernel<<<(unsigned)batch, 256, 0, (hipStream_t)stream>>>(p);
  return nsa_check_launch();
}

extern "C" int nsa_cache_commit_token(const void* const* tokens, const int64_t* strides, const int32_t* stage_len, void* compress_slab,
                                      int32_t* compress_len, void* sparse_slab, int32_t* sparse_len, void* sliding_slab,
                                      int32_t* sliding_len, int64_t batch, int64_t num_kv_heads, int64_t head_dim, int64_t max_batch,
                                      int64_t kernel_size, int64_t compress_rows, int64_t sparse_rows, int64_t window_size, void* stream) {
  if (!tokens || !strides || !stage_len || !compress_slab || !compress_len || !sparse_slab || !sparse_len || !sliding_slab || !sliding_len) return NSA_ERR_BAD_ARG;
  if (batch <= 0 || batch > max_batch || num_kv_heads <= 0 || compress_rows <= 0 || sparse_rows <= 0 || window_size <= 0) return NSA_ERR_BAD_ARG;
  if (head_dim % 8 != 0 || ((uintptr_t)compress_slab | (uintptr_t)sparse_slab | (uintptr_t)sliding_slab) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  CommitParams p;
  for (int i = 0; i < 6; i++) {
    if (!rows_ok(tokens[i], strides[2 * i], strides[2 * i + 1])) return NSA_ERR_UNSUPPORTED;
    p.src[i] = (const u16*)tokens[i]; p.sn[i] = strides[2 * i]; p.sh[i] = strides[2 * i + 1];
  }
  p.stage_len = stage_len; p.cmp_slab = (u16*)compress_slab; p.cmp_len = compress_len; p.full_slab = (u16*)sparse_slab; p.full_len = sparse_len;
  p.ring_slab = (u16*)sliding_slab; p.ring_len = sliding_len;
  p.H = (int)num_kv_heads; p.D = (int)head_dim; p.max_batch = (int)max_batch; p.ks = (int)kernel_size; p.cmp_rows = (int)compress_rows;
  p.full_rows = (int)sparse_rows; p.window = (int)window_size;
  cache_commit_kernel<<<(unsigned)batch, 256, 0, (hipStream_t)stream>>>(p);
  return nsa_check_launch();
}

extern "C" int nsa_cache_append_token(const void* key, const void* value, void* slab, int32_t* slab_len, int64_t batch, int64_t num_kv_heads,
                                      int64_t head_dim, int64_t k_stride_b, int64_t k_stride_h, int64_t v_stride_b, int64_t v_stride_h,
                                      int64_t max_batch, int64_t slab_rows, void* stream) {
  if (!slab || !slab_len || batch <= 0 || batch > max_batch || num_kv_heads <= 0 || slab_rows <= 0) return NSA_ERR_BAD_ARG;
  if (head_dim % 8 != 0 || (uintptr_t)slab % 16 != 0 || !rows_ok(key, k_stride_b, k_stride_h) || !rows_ok(value, v_stride_b, v_stride_h)) return NSA_ERR_UNSUPPORTED;
  AppendParams p;
  p.key = (const u16*)key; p.value = (const u16*)value; p.slab = (u16*)slab; p.len = slab_len;
  p.H = (int)num_kv_heads; p.D = (int)head_dim; p.max_batch = (int)max_batch; p.rows = (int)slab_rows;
  p.ksn = k_stride_b; p.ksh = k_stride_h; p.vsn = v_stride_b; p.vsh = v_stride_h;
  cache_append_kernel<<<(unsigned)batch, 256, 0, (hipStream_t)stream>>>(p);
  return nsa_check_launch();
}
