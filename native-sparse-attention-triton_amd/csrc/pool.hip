// Sliding-window weighted / average pooling of K or V along the sequence (compression), forward
// and backward.  Bandwidth-bound: every thread moves 16-byte pieces, accumulation in fp32.
//   y[n,h,:]  = sum_k w[h,k] * x[s0 + n*stride + k, h, :]          (w == nullptr: w = 1/kernel)
//   dx[t,h,:] = sum over the <= kernel/stride windows that cover t of w[h, i - n*stride] * dy[n,h,:]
//   dw[h,k]   = sum_n sum_d dy[n,h,d] * x[s0 + n*stride + k, h, d]  (two-stage, fixed order)
// The backward is a gather (no atomics), so results are deterministic.
#include "nsa_common.h"

struct PoolParams {
  const void* x; const void* w; const void* y; const int32_t* cu; const int32_t* ycu;
  int total_x, total_y, batch, H, ks, st;
  long long xsn, xsh, ysn, ysh, wsh;
  const void* bias; long long bsh;   // optional [H, D] row added to every output row (null: none)
};

// out = y + bias as 16-bit tensor arithmetic does it: the pooled value is rounded to the element type first, the sum again
template <typename T, typename V8>
__device__ __forceinline__ V8 pooled_row_piece(const float (&acc)[8], const void* bias, long long bsh, int h, int c) {
  V8 out;
  if (bias) {
    const V8 b = ld16<V8>((const T*)bias + (long long)h * bsh + 8 * c);
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = (T)(rounded<T>(acc[j]) + (float)b[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = (T)acc[j];
  }
  return out;
}

template <typename T, int D>
__global__ __launch_bounds__(256) void pool_fwd_kernel(PoolParams p, T* __restrict__ y) {
  using v8 = typename Elem<T>::v8;
  constexpr int C = D / 8;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // (n, h, c), c fastest
  if (i >= (long long)p.total_y * p.H * C) return;
  const int c = (int)(i % C), h = (int)((i / C) % p.H), n = (int)(i / ((long long)C * p.H));
  const int b = find_sequence(p.ycu, p.batch, n);
  const int row0 = p.cu[b] + (n - p.ycu[b]) * p.st;
  const T* xp = (const T*)p.x + (long long)row0 * p.xsn + (long long)h * p.xsh + 8 * c;
  const T* wp = p.w ? (const T*)p.w + (long long)h * p.wsh : nullptr;
  const float wavg = 1.f / (float)p.ks;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  // eight rows per trip, their loads issued together: a decode step pools a single window per sequence and is
  // then bound by the round trips of this loop, not by bandwidth
  int k = 0;
  for (; k + 8 <= p.ks; k += 8) {
    v8 xv[8];
    float wk[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      xv[u] = ld16<v8>(xp + (long long)(k + u) * p.xsn);
      wk[u] = wp ? (float)wp[k + u] : wavg;
    }
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(wk[u], (float)xv[u][j], acc[j]);
  }
  for (; k < p.ks; k++) {
    const v8 xv = ld16<v8>(xp + (long long)k * p.xsn);
    const float wk = wp ? (float)wp[k] : wavg;
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(wk, (float)xv[j], acc[j]);
  }
  const v8 out = pooled_row_piece<T, v8>(acc, p.bias, p.bsh, h, c);
  st16(y + (long long)n * p.ysn + (long long)h * p.ysh + 8 * c, out);
}

// Forward for launches large enough to be bound by bandwidth: the window of an output piece is split over SPLIT
// threads of 16 rows each, whose 16 loads are all issued before the first is used (one round trip per thread
// instead of kernel_size / 8 in a row, and SPLIT times as many threads in flight); the partial sums meet in LDS and
// are added in window order.  Threads of a wave hold consecutive pieces of the same rows (coalesced).
template <typename T, int D, int SPLIT>
__global__ __launch_bounds__(256) void pool_fwd_split_kernel(PoolParams p, T* __restrict__ y) {
  using v8 = typename Elem<T>::v8;
  constexpr int C = D / 8, PPW = 256 / SPLIT;   // output pieces per workgroup
  __shared__ float part[SPLIT > 1 ? SPLIT - 1 : 1][PPW][8];
  const int sub = threadIdx.x / PPW, pl = threadIdx.x % PPW;
  const long long i = (long long)blockIdx.x * PPW + pl;   // (n, h, c), c fastest
  const bool live = i < (long long)p.total_y * p.H * C;
  const int c = (int)(i % C), h = (int)((i / C) % p.H), n = live ? (int)(i / ((long long)C * p.H)) : 0;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (live) {
    const int b = find_sequence(p.ycu, p.batch, n);
    const int row0 = p.cu[b] + (n - p.ycu[b]) * p.st + 16 * sub;
    const T* xp = (const T*)p.x + (long long)row0 * p.xsn + (long long)h * p.xsh + 8 * c;
    v8 xv[16];
#pragma unroll
    for (int u = 0; u < 16; u++) xv[u] = ld16<v8>(xp + (long long)u * p.xsn);
    float wk[16];
    if (p.w) {
      const T* wp = (const T*)p.w + (long long)h * p.wsh + 16 * sub;
#pragma unroll
      for (int u = 0; u < 16; u++) wk[u] = (float)wp[u];
    } else {
#pragma unroll
      for (int u = 0; u < 16; u++) wk[u] = 1.f / (float)p.ks;
    }
#pragma unroll
    for (int u = 0; u < 16; u++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(wk[u], (float)xv[u][j], acc[j]);
  }
  if (SPLIT > 1) {
    if (sub > 0) {
#pragma unroll
      for (int j = 0; j < 8; j++) part[sub - 1][pl][j] = acc[j];
    }
    __syncthreads();
    if (sub > 0) return;
#pragma unroll
    for (int s2 = 1; s2 < SPLIT; s2++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] += part[s2 - 1][pl][j];
  }
  if (!live) return;
  const v8 out = pooled_row_piece<T, v8>(acc, p.bias, p.bsh, h, c);
  st16(y + (long long)n * p.ysn + (long long)h * p.ysh + 8 * c, out);
}

template <typename T, int D>
__global__ __launch_bounds__(256) void pool_dx_kernel(PoolParams p, const T* __restrict__ dy, long long dysn, long long dysh,
                                                      T* __restrict__ dx, long long dxsn, long long dxsh) {
  using v8 = typename Elem<T>::v8;
  constexpr int C = D / 8;
  // a workgroup owns 256 / C consecutive tokens of one head; the sequence of its first token is found once (scalar),
  // a thread whose token lies beyond that sequence's end searches on its own
  constexpr int TPB = 256 / C;
  const int c = threadIdx.x % C, t = blockIdx.x * TPB + threadIdx.x / C, h = blockIdx.y;
  if (threadIdx.x / C >= TPB || t >= p.total_x) return;
  int b = find_sequence(p.cu, p.batch, blockIdx.x * TPB);
  if (t >= p.cu[b + 1]) b = find_sequence(p.cu, p.batch, t);
  const int pos = t - p.cu[b];
  const int ylen = p.ycu[b + 1] - p.ycu[b];
  // windows n with n * st <= pos <= n * st + ks - 1; a power-of-two stride divides by a shift
  const int sh = (p.st & (p.st - 1)) == 0 ? __builtin_ctz(p.st) : -1;
  int n_lo = pos - p.ks + 1;
  n_lo = n_lo <= 0 ? 0 : (sh >= 0 ? (n_lo + p.st - 1) >> sh : (n_lo + p.st - 1) / p.st);
  int n_hi = sh >= 0 ? pos >> sh : pos / p.st;
  n_hi = n_hi < ylen - 1 ? n_hi : ylen - 1;
  const T* wp = p.w ? (const T*)p.w + (long long)h * p.wsh : nullptr;
  const float wavg = 1.f / (float)p.ks;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int n = n_lo; n <= n_hi; n++) {
    const v8 g = ld16<v8>(dy + (long long)(p.ycu[b] + n) * dysn + (long long)h * dysh + 8 * c);
    const float wk = wp ? (float)wp[pos - n * p.st] : wavg;
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] += wk * (float)g[j];
  }
  v8 out;
#pragma unroll
  for (int j = 0; j < 8; j++) out[j] = (T)acc[j];
  st16(dx + (long long)t * dxsn + (long long)h * dxsh + 8 * c, out);
}

// partial[h][tile][k]: one workgroup per (tile of DW_TILE output tokens, head)
static constexpr int DW_TILE = 16;  // windows per workgroup of the dW pass: short tiles so that a few thousand windows still fill the chip
template <typename T, int D>
__global__ __launch_bounds__(256) void pool_dw_partial_kernel(PoolParams p, const T* __restrict__ dy, long long dysn, long long dysh,
                                                              float* __restrict__ partial, int n_tiles) {
  using v8 = typename Elem<T>::v8;
  constexpr int C = D / 8;            // threads per token
  constexpr int TPW = 256 / C;        // tokens in flight per pass
  __shared__ float red[4 * 16];
  const int tile = blockIdx.x, h = blockIdx.y;
  const int c = threadIdx.x % C, tl = threadIdx.x / C;
  const int n0 = tile * DW_TILE, n1 = min(p.total_y, n0 + DW_TILE);
  for (int k0 = 0; k0 < p.ks; k0 += 16) {
    float acc[16];
#pragma unroll
    for (int k = 0; k < 16; k++) acc[k] = 0.f;
    for (int n = n0 + tl; tl < TPW && n < n1; n += TPW) {  // threads beyond the last whole token idle
      const int b = find_sequence(p.ycu, p.batch, n);
      const int row0 = p.cu[b] + (n - p.ycu[b]) * p.st;
      const v8 g = ld16<v8>(dy + (long long)n * dysn + (long long)h * dysh + 8 * c);
      const T* xp = (const T*)p.x + (long long)row0 * p.xsn + (long long)h * p.xsh + 8 * c;
#pragma unroll
      for (int k = 0; k < 16; k++) {
        if (k0 + k < p.ks) {
          const v8 xv = ld16<v8>(xp + (long long)(k0 + k) * p.xsn);
#pragma unroll
          for (int j = 0; j < 8; j++) acc[k] += (float)g[j] * (float)xv[j];
        }
      }
    }
    // sum over the workgroup: lanes of a wave by lane exchanges, then the four waves through LDS
    // (fixed order, so the result does not depend on scheduling)
#pragma unroll
    for (int k = 0; k < 16; k++) {
      const float v = wave_sum_f32(acc[k]);
      if ((threadIdx.x & 63) == 0) red[(threadIdx.x >> 6) * 16 + k] = v;
    }
    __syncthreads();
    if (threadIdx.x < 16 && k0 + threadIdx.x < p.ks)
      partial[((long long)h * n_tiles + tile) * p.ks + k0 + threadIdx.x] =
          ((red[threadIdx.x] + red[16 + threadIdx.x]) + red[32 + threadIdx.x]) + red[48 + threadIdx.x];
    __syncthreads();
  }
}

// dw[h][k] = sum over the tiles' partials: one wave per (h, k); lane l adds tiles l, l + 64, ... in order, then
// the lanes meet in a fixed-order wave sum (reproducible whatever the number of tiles).
template <typename T>
__global__ __launch_bounds__(64) void pool_dw_final_kernel(const float* __restrict__ partial, int n_tiles, int H, int ks, T* __restrict__ dw, long long dwsh) {
  const int i = blockIdx.x;  // (h, k)
  const int h = i / ks, k = i % ks;
  float acc = 0.f;
  for (int t = threadIdx.x; t < n_tiles; t += 64) acc += partial[((long long)h * n_tiles + t) * ks + k];
  acc = wave_sum_f32(acc);
  if (threadIdx.x == 0) dw[(long long)h * dwsh + k] = (T)acc;
}

template <typename T, int D>
static int pool_fwd_t(const PoolParams& p, void* y, hipStream_t s) {
  const long long n = (long long)p.total_y * p.H * (D / 8);
  if (n <= 0) return NSA_OK;
  // big launches: one round of loads per thread; small ones (a decode step pools one window per sequence) keep the
  // plain kernel, whose summation order the single-launch decode preparation reproduces bit for bit
  const bool big = n >= 32768;
  if (big && p.ks == 16) pool_fwd_split_kernel<T, D, 1><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p, (T*)y);
  else if (big && p.ks == 32) pool_fwd_split_kernel<T, D, 2><<<(unsigned)((n + 127) / 128), 256, 0, s>>>(p, (T*)y);
  else if (big && p.ks == 64) pool_fwd_split_kernel<T, D, 4><<<(unsigned)((n + 63) / 64), 256, 0, s>>>(p, (T*)y);
  else if (big && p.ks == 128) pool_fwd_split_kernel<T, D, 8><<<(unsigned)((n + 31) / 32), 256, 0, s>>>(p, (T*)y);
  else pool_fwd_kernel<T, D><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p, (T*)y);
  return nsa_check_launch();
}
template <typename T, int D>
static int pool_bwd_t(const PoolParams& p, const void* dy, long long dysn, long long dysh, void* dx, long long dxsn, long long dxsh,
                      void* dw, long long dwsh, float* partial, hipStream_t s) {
  constexpr int TPB = 256 / (D / 8);
  pool_dx_kernel<T, D><<<dim3((unsigned)((p.total_x + TPB - 1) / TPB), (unsigned)p.H), 256, 0, s>>>(p, (const T*)dy, dysn, dysh, (T*)dx, dxsn, dxsh);
  if (dw) {
    const int n_tiles = (p.total_y + DW_TILE - 1) / DW_TILE;
    if (n_tiles > 0) pool_dw_partial_kernel<T, D><<<dim3((unsigned)n_tiles, (unsigned)p.H), 256, 0, s>>>(p, (const T*)dy, dysn, dysh, partial, n_tiles);
    pool_dw_final_kernel<T><<<p.H * p.ks, 64, 0, s>>>(partial, n_tiles, p.H, p.ks, (T*)dw, dwsh);
  }
  return nsa_check_launch();
}

#define POOL_DISPATCH(CALL)                                                     \
  switch (head_dim) {                                                           \
    case 32: return dtype == NSA_BF16 ? CALL(__bf16, 32) : CALL(_Float16, 32);  \
    case 64: return dtype == NSA_BF16 ? CALL(__bf16, 64) : CALL(_Float16, 64);  \
    case 96: return dtype == NSA_BF16 ? CALL(__bf16, 96) : CALL(_Float16, 96);  \
    case 128: return dtype == NSA_BF16 ? CALL(__bf16, 128) : CALL(_Float16, 128); \
    case 192: return dtype == NSA_BF16 ? CALL(__bf16, 192) : CALL(_Float16, 192); \
    case 256: return dtype == NSA_BF16 ? CALL(__bf16, 256) : CALL(_Float16, 256); \
  }                                                                             \
  return NSA_ERR_UNSUPPORTED;

static int fill_params(PoolParams& p, const void* x, const void* w, const int32_t* cu, const int32_t* ycu, int64_t total_x,
                       int64_t total_y, int64_t batch, int64_t H, int64_t ks, int64_t st, int64_t xsn, int64_t xsh, int64_t wsh) {
  if (!x || !cu || !ycu || total_x <= 0 || total_y < 0 || batch <= 0 || H <= 0 || ks <= 0 || st <= 0) return NSA_ERR_BAD_ARG;
  if ((xsn | xsh) % 8 != 0 || (uintptr_t)x % 16 != 0) return NSA_ERR_UNSUPPORTED;
  p.x = x; p.w = w; p.cu = cu; p.ycu = ycu; p.total_x = (int)total_x; p.total_y = (int)total_y; p.batch = (int)batch;
  p.H = (int)H; p.ks = (int)ks; p.st = (int)st; p.xsn = xsn; p.xsh = xsh; p.wsh = wsh; p.y = nullptr; p.ysn = p.ysh = 0;
  p.bias = nullptr; p.bsh = 0;
  return NSA_OK;
}

extern "C" int nsa_pool_fwd_bias(const void* x, const void* w, const void* bias, void* y, const int32_t* cu_seqlens, const int32_t* y_cu_seqlens,
                                 int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim,
                                 int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                                 int64_t y_stride_n, int64_t y_stride_h, int64_t w_stride_h, int64_t bias_stride_h, int dtype, void* stream) {
  PoolParams p;
  int rc = fill_params(p, x, w, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, kernel_size, kernel_stride, x_stride_n, x_stride_h, w_stride_h);
  if (rc != NSA_OK) return rc;
  if (total_y > 0 && (!y || (y_stride_n | y_stride_h) % 8 != 0 || (uintptr_t)y % 16 != 0)) return NSA_ERR_UNSUPPORTED;
  if (bias && (bias_stride_h % 8 != 0 || (uintptr_t)bias % 16 != 0)) return NSA_ERR_UNSUPPORTED;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  p.ysn = y_stride_n; p.ysh = y_stride_h; p.bias = bias; p.bsh = bias_stride_h;
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) pool_fwd_t<T, D>(p, y, s)
  POOL_DISPATCH(CALL)
#undef CALL
}

extern "C" int nsa_pool_fwd(const void* x, const void* w, void* y, const int32_t* cu_seqlens, const int32_t* y_cu_seqlens,
                            int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim,
                            int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                            int64_t y_stride_n, int64_t y_stride_h, int64_t w_stride_h, int dtype, void* stream) {
  return nsa_pool_fwd_bias(x, w, nullptr, y, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, head_dim, kernel_size,
                           kernel_stride, x_stride_n, x_stride_h, y_stride_n, y_stride_h, w_stride_h, 0, dtype, stream);
}

extern "C" size_t nsa_pool_bwd_workspace_bytes(int64_t total_y, int64_t num_heads, int64_t kernel_size) {
  return (size_t)num_heads * (size_t)((total_y + DW_TILE - 1) / DW_TILE + 1) * (size_t)kernel_size * 4;
}

extern "C" int nsa_pool_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, const int32_t* cu_seqlens,
                            const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                            int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                            int64_t dy_stride_n, int64_t dy_stride_h, int64_t dx_stride_n, int64_t dx_stride_h,
                            int64_t w_stride_h, int64_t dw_stride_h, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  PoolParams p;
  int rc = fill_params(p, x, w, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, kernel_size, kernel_stride, x_stride_n, x_stride_h, w_stride_h);
  if (rc != NSA_OK) return rc;
  if (!dx || (total_y > 0 && !dy) || ((w == nullptr) != (dw == nullptr))) return NSA_ERR_BAD_ARG;
  if ((dy_stride_n | dy_stride_h | dx_stride_n | dx_stride_h) % 8 != 0 || ((uintptr_t)dy | (uintptr_t)dx) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  if (dw && (!workspace || workspace_bytes < nsa_pool_bwd_workspace_bytes(total_y, num_heads, kernel_size))) return NSA_ERR_WORKSPACE;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
#define CALL(T, D) pool_bwd_t<T, D>(p, dy, dy_stride_n, dy_stride_h, dx, dx_stride_n, dx_stride_h, dw, dw_stride_h, (float*)workspace, s)
  POOL_DISPATCH(CALL)
#undef CALL
}

// y_len[b] = floor((len_b - ks) / st) + 1 (0 when len_b < ks) and its cumulative sum, in one launch
// (native_sparse_attention/ops/triton/utils.py:25-37 of the reference spends a dozen tensor-op launches on it).
__global__ __launch_bounds__(256) void compressed_seqlens_kernel(const int32_t* __restrict__ cu, int batch, int ks, int st,
                                                                 int32_t* __restrict__ y_len, int32_t* __restrict__ y_cu) {
  __shared__ int part[256];
  const int tid = threadIdx.x;
  // thread t owns sequences [t*per, (t+1)*per)
  const int per = (batch + 255) / 256;
  int sum = 0;
  for (int b = tid * per; b < min(batch, (tid + 1) * per); b++) {
    const int len = cu[b + 1] - cu[b];
    const int n = len < ks ? 0 : (len - ks) / st + 1;
    y_len[b] = n;
    sum += n;
  }
  part[tid] = sum;
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const int v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = part[tid] - sum;  // exclusive prefix of this thread's sequences
  if (tid == 0) y_cu[0] = 0;
  for (int b = tid * per; b < min(batch, (tid + 1) * per); b++) {
    const int len = cu[b + 1] - cu[b];
    run += len < ks ? 0 : (len - ks) / st + 1;
    y_cu[b + 1] = run;
  }
}

extern "C" int nsa_compressed_seqlens(const int32_t* cu_seqlens, int64_t batch, int64_t kernel_size, int64_t kernel_stride,
                                      int32_t* y_seqlens, int32_t* y_cu_seqlens, void* stream) {
  if (!cu_seqlens || !y_seqlens || !y_cu_seqlens || batch <= 0 || kernel_size <= 0 || kernel_stride <= 0 || batch >= (1ll << 31)) return NSA_ERR_BAD_ARG;
  compressed_seqlens_kernel<<<1, 256, 0, (hipStream_t)stream>>>(cu_seqlens, (int)batch, (int)kernel_size, (int)kernel_stride, y_seqlens, y_cu_seqlens);
  return nsa_check_launch();
}
