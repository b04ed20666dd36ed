// linear_compress: per-head sliding-window linear projection of K or V,
//   y[n,h,:] = concat_k( x[s0 + n*stride + k, h, :] ) @ W[h]          W[h]: [kernel*D, D]
// as strided-window GEMMs on the matrix cores, without materialising the unfolded windows.
//   forward : Y^T[e][n]  = sum_{k,d} W[(k,d)][e] * Xwin[n][(k,d)]   W pieces transposed in registers, no LDS staging
//   dX      : tokens grouped by phase (pos mod stride) share the same slices of W:
//             dX^T[d][m] = sum_{j,e} W[(phase + j*stride, d)][e] * dY[m - j][e]   all operands straight from global
//   dW      : dW^T[e][(k,d)] = sum_n dY[n][e] * x[row(n)+k][d]      both tiles through LDS, read transposed
// Every output element is produced by exactly one lane in a fixed order: no atomics, reproducible.
#include "nsa_common.h"

struct LinParams {
  const void* x; const void* w; const void* dy; void* y; void* dx; void* dw;
  const int32_t* cu; const int32_t* ycu;
  int total_x, total_y, batch, H, ks, st;
  long long xsn, xsh, ysn, ysh, dysn, dysh, dxsn, dxsh;  // w, dw: [H, ks*D, D] contiguous
  const void* bias; long long bsh;   // forward: optional [H, D] row added to every output row (null: none)
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
template <typename T, int LD>
__device__ __forceinline__ typename Elem<T>::v8 lds_tr_frag(const T (*tile)[LD], int c0, int li, int lg) {
  const T* a0 = &tile[4 * lg + (li >> 2)][c0 + 4 * (li & 3)];
  const T* a1 = &tile[16 + 4 * lg + (li >> 2)][c0 + 4 * (li & 3)];
  s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
  s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a1));
  s16x8 z = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
  return __builtin_bit_cast(typename Elem<T>::v8, z);
}
// 8 elements of a row in the slot order of lds_tr_frag: columns c0+4*lg..+3 and c0+16+4*lg..+3
template <typename T>
__device__ __forceinline__ typename Elem<T>::v8 row_frag(const T* row, int c0, int lg, bool live) {
  uint2 a = {0u, 0u}, b = {0u, 0u};
  if (live) {
    a = *reinterpret_cast<const uint2*>(row + c0 + 4 * lg);
    b = *reinterpret_cast<const uint2*>(row + c0 + 16 + 4 * lg);
  }
  uint4 r = {a.x, a.y, b.x, b.y};
  return __builtin_bit_cast(typename Elem<T>::v8, r);
}

__device__ __forceinline__ int first_slot_of(const int32_t* __restrict__ cu, int b, int unit) { return (cu[b] + unit - 1) / unit + b; }
__device__ __forceinline__ int slot_sequence(const int32_t* __restrict__ cu, int batch, int slot, int unit) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (first_slot_of(cu, mid, unit) <= slot) lo = mid; else hi = mid;
  }
  return lo;
}

// ------------------------------------------------------------------------------------------
// Forward.  A workgroup = 16*NT output rows of one head; its 8 waves split the window positions and add their
// fp32 sums through LDS in a fixed order.  Nothing is staged: per 32 contraction rows (a "chunk") a lane loads
// an 8 x (D/16) piece of W, rows d = 32q + 8*lg + 0..7, columns e = (D/16)*li + 0..D/16-1 (a wave reads 4 whole rows per
// load), and transposes it in its own registers with byte permutes into D/16 operand fragments: fragment j holds
// W[d.., (D/16)*li + j].  MFMA j therefore produces the output columns e = (D/16)*m + j, m the row index of its A
// operand, and a lane ends up with D/4 consecutive columns of one output row.  All loads of several chunks are in
// flight at once and there is no barrier before the final sum.
template <typename T, int D, int NT>
__global__ __launch_bounds__(512) void lin_fwd_kernel(LinParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NJ = D / 16, NW = D / 32, ROWS = 16 * NT, LP = D + 4;
  constexpr int GC0 = (NT == 1 ? 16 : NT == 2 ? 12 : 8) / NW, GC = GC0 < 1 ? 1 : GC0 > 8 ? 8 : GC0;   // chunks loaded together: at most 128 registers of W
  constexpr int VW = NW % 4 == 0 ? 4 : NW % 2 == 0 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) float part[4][ROWS][LP];
  const int h = blockIdx.y;
  const int b = slot_sequence(p.ycu, p.batch, blockIdx.x, ROWS);
  const int ylen = p.ycu[b + 1] - p.ycu[b];
  const int n0 = (blockIdx.x - first_slot_of(p.ycu, b, ROWS)) * ROWS;
  if (n0 >= ylen) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
  const T* xrow[NT];
  bool live[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int n = n0 + 16 * t + li;
    live[t] = n < ylen;
    xrow[t] = (const T*)p.x + (long long)(p.cu[b] + (live[t] ? n : 0) * p.st) * p.xsn + (long long)h * p.xsh + 8 * lg;
  }
  const T* wl = (const T*)p.w + (long long)h * p.ks * D * D + (long long)(8 * lg) * D + NJ * li;
  f32x4 acc[NT][NJ];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // this wave's window positions, as chunks of 32 rows of W[h]
  const int per = (p.ks + 7) / 8;
  const int q0 = min(p.ks, wave * per) * NW, q1 = min(p.ks, (wave + 1) * per) * NW;
  for (int g = q0; g < q1; g += GC) {
    uint32_t wr[GC][8][NW];
    v8 xf[GC][NT];
#pragma unroll
    for (int u = 0; u < GC; u++) {
      const int q = min(g + u, q1 - 1);   // a short last group loads its last chunk again and does not use it
      const T* wq = wl + (long long)q * 32 * D;
#pragma unroll
      for (int r = 0; r < 8; r++)
#pragma unroll
        for (int w0 = 0; w0 < NW; w0 += VW) {
          if constexpr (VW == 4) {
            const uint4 t4 = *reinterpret_cast<const uint4*>(wq + r * D + 2 * w0);
            wr[u][r][w0] = t4.x; wr[u][r][w0 + 1] = t4.y; wr[u][r][w0 + 2] = t4.z; wr[u][r][w0 + 3] = t4.w;
          } else if constexpr (VW == 2) {
            const uint2 t2 = *reinterpret_cast<const uint2*>(wq + r * D + 2 * w0);
            wr[u][r][w0] = t2.x; wr[u][r][w0 + 1] = t2.y;
          } else {
            wr[u][r][w0] = *reinterpret_cast<const uint32_t*>(wq + r * D + 2 * w0);
          }
        }
      const int k = q / NW, c = q % NW;
#pragma unroll
      for (int t = 0; t < NT; t++) xf[u][t] = live[t] ? ld16<v8>(xrow[t] + (long long)k * p.xsn + 32 * c) : zero16<v8>();
    }
#pragma unroll
    for (int u = 0; u < GC; u++) {
      if (g + u < q1) {
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          // 16-bit column j of the lane's 8 x NJ piece: element r comes from row r
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          uint4 f;
          f.x = __builtin_amdgcn_perm(wr[u][1][j >> 1], wr[u][0][j >> 1], sel);
          f.y = __builtin_amdgcn_perm(wr[u][3][j >> 1], wr[u][2][j >> 1], sel);
          f.z = __builtin_amdgcn_perm(wr[u][5][j >> 1], wr[u][4][j >> 1], sel);
          f.w = __builtin_amdgcn_perm(wr[u][7][j >> 1], wr[u][6][j >> 1], sel);
          const v8 wf = __builtin_bit_cast(v8, f);
#pragma unroll
          for (int t = 0; t < NT; t++) acc[t][j] = E::mfma16(wf, xf[u][t], acc[t][j]);
        }
      }
    }
  }
  // acc[t][j][r] = y[n0 + 16t + li][NJ * (4*lg + r) + j]: the lane's D/4 columns start at D/4 * lg, in (r, j) order.
  // Waves 4..7 hand their sums to waves 0..3, those hand theirs to all threads: ((w0 + w4) + (w1 + w5)) + ((w2 + w6) + (w3 + w7)).
  auto stash = [&](int slot) {
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
      for (int i = 0; i < 4 * NJ; i += 4) {
        f32x4 o;
#pragma unroll
        for (int z = 0; z < 4; z++) o[z] = acc[t][(i + z) % NJ][(i + z) / NJ];
        *reinterpret_cast<f32x4*>(&part[slot][16 * t + li][4 * NJ * lg + i]) = o;
      }
  };
  if (wave >= 4) stash(wave - 4);
  __syncthreads();
  if (wave < 4) {
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
      for (int i = 0; i < 4 * NJ; i += 4) {
        const f32x4 o = *reinterpret_cast<const f32x4*>(&part[wave][16 * t + li][4 * NJ * lg + i]);
#pragma unroll
        for (int z = 0; z < 4; z++) acc[t][(i + z) % NJ][(i + z) / NJ] += o[z];
      }
  }
  __syncthreads();
  if (wave < 4) stash(wave);
  __syncthreads();
  for (int i = tid; i < ROWS * (D / 4); i += 512) {
    const int row = i / (D / 4), c4 = 4 * (i % (D / 4));
    if (n0 + row >= ylen) continue;
    const f32x4 s = (*reinterpret_cast<const f32x4*>(&part[0][row][c4]) + *reinterpret_cast<const f32x4*>(&part[1][row][c4])) +
                    (*reinterpret_cast<const f32x4*>(&part[2][row][c4]) + *reinterpret_cast<const f32x4*>(&part[3][row][c4]));
    v4 o;
    if (p.bias) {   // y + bias as 16-bit tensor arithmetic does it: the product is rounded first, the sum again
      const v4 bv = *reinterpret_cast<const v4*>((const T*)p.bias + (long long)h * p.bsh + c4);
#pragma unroll
      for (int z = 0; z < 4; z++) o[z] = (T)(rounded<T>(s[z]) + (float)bv[z]);
    } else {
#pragma unroll
      for (int z = 0; z < 4; z++) o[z] = (T)s[z];
    }
    st8((T*)p.y + (long long)(p.ycu[b] + n0 + row) * p.ysn + (long long)h * p.ysh + c4, o);
  }
}

// ------------------------------------------------------------------------------------------
template <typename T, int D>
__global__ __launch_bounds__(256) void lin_dx_kernel(LinParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NK = D / 32, NDT = D / 16;
  const int h = blockIdx.z, phase = blockIdx.y;
  const int unit = 64 * p.st;
  const int b = slot_sequence(p.cu, p.batch, blockIdx.x, unit);
  const int len = p.cu[b + 1] - p.cu[b], ylen = p.ycu[b + 1] - p.ycu[b];
  const int m0 = (blockIdx.x - first_slot_of(p.cu, b, unit)) * 64;
  if (m0 * p.st >= len) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, lg = lane >> 4;
  const int m = m0 + 16 * wave + li;
  const int pos = phase + m * p.st;
  const T* wh = (const T*)p.w + (long long)h * p.ks * D * D;
  f32x4 acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int taps = p.ks / p.st;
  for (int j = 0; j < taps; j++) {
    const int n = m - j;
    const bool ok = n >= 0 && n < ylen;
    const T* dyrow = (const T*)p.dy + (long long)(p.ycu[b] + (ok ? n : 0)) * p.dysn + (long long)h * p.dysh + 8 * lg;
    const T* wk = wh + (long long)(phase + j * p.st) * D * D + 8 * lg;
#pragma unroll
    for (int kk = 0; kk < NK; kk++) {
      const v8 g = ok ? ld16<v8>(dyrow + 32 * kk) : zero16<v8>();
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) acc[dt] = E::mfma16(ld16<v8>(wk + (long long)(16 * dt + li) * D + 32 * kk), g, acc[dt]);
    }
  }
  if (pos < len) {
    T* op = (T*)p.dx + (long long)(p.cu[b] + pos) * p.dxsn + (long long)h * p.dxsh + 4 * lg;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++) {
      v4 o;
#pragma unroll
      for (int r = 0; r < 4; r++) o[r] = (T)acc[dt][r];
      st8(op + 16 * dt, o);
    }
  }
}

// ------------------------------------------------------------------------------------------
// one workgroup per (tap k, head): dW[h][(k, d)][e] for all d, e; wave w owns d in [D/4*w, +D/4)
template <typename T, int D>
__global__ __launch_bounds__(256) void lin_dw_kernel(LinParams p) {
  using E = Elem<T>;
  using v8 = typename E::v8;
  using v4 = typename E::v4;
  constexpr int NET = D / 16, LD = lds_pitch(D);
  constexpr int DTW = (D / 16 + 3) / 4;  // d tiles per wave
  __shared__ __attribute__((aligned(16))) T x_s[2][32][LD];
  __shared__ __attribute__((aligned(16))) T g_s[2][32][LD];
  const int k = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
  f32x4 acc[DTW][NET];
#pragma unroll
  for (int a = 0; a < DTW; a++)
#pragma unroll
    for (int i = 0; i < NET; i++) acc[a][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int PIECES1 = 32 * (D / 8), PPT1 = (PIECES1 + 255) / 256;  // per tensor
  uint4 rx[PPT1], rg[PPT1];
  auto fetch = [&](int chunk) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < PPT1; u++) {
      const int pc = tid + u * 256;
      const int c = pc % (D / 8), r = pc / (D / 8);
      const int n = chunk * 32 + r;
      uint4 vx = {0u, 0u, 0u, 0u}, vg = {0u, 0u, 0u, 0u};
      if (pc < PIECES1 && n < p.total_y) {
        const int b = find_sequence(p.ycu, p.batch, n);
        const long long row = p.cu[b] + (long long)(n - p.ycu[b]) * p.st + k;
        vx = *reinterpret_cast<const uint4*>((const T*)p.x + row * p.xsn + (long long)h * p.xsh + 8 * c);
        vg = *reinterpret_cast<const uint4*>((const T*)p.dy + (long long)n * p.dysn + (long long)h * p.dysh + 8 * c);
      }
      rx[u] = vx;
      rg[u] = vg;
    }
  };
  auto stash = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < PPT1; u++) {
      const int pc = tid + u * 256;
      if (pc < PIECES1) {
        const int c = pc % (D / 8), r = pc / (D / 8);
        *reinterpret_cast<uint4*>(&x_s[buf][r][8 * c]) = rx[u];
        *reinterpret_cast<uint4*>(&g_s[buf][r][8 * c]) = rg[u];
      }
    }
  };
  const int n_chunks = (p.total_y + 31) / 32;
  if (n_chunks > 0) { fetch(0); stash(0); }
  __syncthreads();
  for (int ch = 0; ch < n_chunks; ch++) {
    const int buf = ch & 1;
    if (ch + 1 < n_chunks) fetch(ch + 1);
#pragma unroll
    for (int a = 0; a < DTW; a++) {
      const int dt = wave * DTW + a;
      if (16 * dt < D) {
        const v8 xf = lds_tr_frag<T, LD>(x_s[buf], 16 * dt, li, lg);  // columns: d = 16*dt + li
#pragma unroll
        for (int et = 0; et < NET; et++) acc[a][et] = E::mfma16(lds_tr_frag<T, LD>(g_s[buf], 16 * et, li, lg), xf, acc[a][et]);
      }
    }
    if (ch + 1 < n_chunks) stash(buf ^ 1);
    __syncthreads();
  }
  T* dwh = (T*)p.dw + ((long long)h * p.ks + k) * D * D;
#pragma unroll
  for (int a = 0; a < DTW; a++) {
    const int dt = wave * DTW + a;
    if (16 * dt < D) {
#pragma unroll
      for (int et = 0; et < NET; et++) {
        v4 o;
#pragma unroll
        for (int r = 0; r < 4; r++) o[r] = (T)acc[a][et][r];
        st8(dwh + (long long)(16 * dt + li) * D + 16 * et + 4 * lg, o);  // row d, columns e..e+3
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
template <typename T, int D>
static int lin_run(const LinParams& p, int what, hipStream_t s) {
  if (what == 0) {
    // Rows per workgroup: W[h] passes through the workgroup's CU once per workgroup, so more rows mean fewer reads
    // of W, as long as at least 128 workgroups remain.  Measured, kernel 32 stride 16, 4 heads, d=128, inputs cached:
    // 1021 output rows 18.9 / 23.5 / 30.3 us at 16 / 32 / 64 rows (from memory, between other kernels: 33.7 / 25.5 / 34.2),
    // 4093 output rows 61.7 / 47.9 / 37.2 us.
    if (p.total_y > 0) {
      const auto wgs = [&](int rows) { return (p.total_y / rows + p.batch + 1) * (int64_t)p.H; };
      if constexpr (D <= 128) {
        if (wgs(64) >= 128) {
          lin_fwd_kernel<T, D, 4><<<dim3((unsigned)(wgs(64) / p.H), (unsigned)p.H), 512, 0, s>>>(p);
          return nsa_check_launch();
        }
        if (wgs(32) >= 128) {
          lin_fwd_kernel<T, D, 2><<<dim3((unsigned)(wgs(32) / p.H), (unsigned)p.H), 512, 0, s>>>(p);
          return nsa_check_launch();
        }
      }
      lin_fwd_kernel<T, D, 1><<<dim3((unsigned)(wgs(16) / p.H), (unsigned)p.H), 512, 0, s>>>(p);
    }
  } else {
    const int64_t unit = 64 * (int64_t)p.st;
    const int64_t slots = p.total_x / unit + p.batch + 1;
    lin_dx_kernel<T, D><<<dim3((unsigned)slots, (unsigned)p.st, (unsigned)p.H), 256, 0, s>>>(p);
    lin_dw_kernel<T, D><<<dim3((unsigned)p.ks, (unsigned)p.H), 256, 0, s>>>(p);
  }
  return nsa_check_launch();
}

static int lin_dispatch(const LinParams& p, int what, int64_t head_dim, int dtype, hipStream_t s) {
#define CALL(T, D) lin_run<T, D>(p, what, s)
  switch (head_dim) {
    case 32: return dtype == NSA_BF16 ? CALL(__bf16, 32) : CALL(_Float16, 32);
    case 64: return dtype == NSA_BF16 ? CALL(__bf16, 64) : CALL(_Float16, 64);
    case 96: return dtype == NSA_BF16 ? CALL(__bf16, 96) : CALL(_Float16, 96);
    case 128: return dtype == NSA_BF16 ? CALL(__bf16, 128) : CALL(_Float16, 128);
    case 192: return dtype == NSA_BF16 ? CALL(__bf16, 192) : CALL(_Float16, 192);
  }
#undef CALL
  return NSA_ERR_UNSUPPORTED;
}

static int lin_fill(LinParams& p, const void* x, const void* w, const int32_t* cu, const int32_t* ycu, int64_t total_x, int64_t total_y,
                    int64_t batch, int64_t H, int64_t ks, int64_t st, int64_t xsn, int64_t xsh, int dtype) {
  if (!x || !w || !cu || !ycu || total_x <= 0 || total_y < 0 || batch <= 0 || H <= 0 || ks <= 0 || st <= 0 || ks % st != 0) return NSA_ERR_BAD_ARG;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if ((xsn | xsh) % 8 != 0 || ((uintptr_t)x | (uintptr_t)w) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  p.x = x; p.w = w; p.cu = cu; p.ycu = ycu; p.total_x = (int)total_x; p.total_y = (int)total_y; p.batch = (int)batch; p.H = (int)H;
  p.ks = (int)ks; p.st = (int)st; p.xsn = xsn; p.xsh = xsh;
  p.bias = nullptr; p.bsh = 0;
  p.dy = nullptr; p.y = nullptr; p.dx = nullptr; p.dw = nullptr; p.ysn = p.ysh = p.dysn = p.dysh = p.dxsn = p.dxsh = 0;
  return NSA_OK;
}

// The forward keeps its partial sums in LDS: no workspace.  The query stays so that callers written against a
// library that needed one keep working.
extern "C" size_t nsa_linear_compress_fwd_workspace_bytes(int64_t, int64_t, int64_t, int64_t, int64_t) { return 0; }

extern "C" int nsa_linear_compress_fwd_bias(const void* x, const void* w, const void* bias, void* y, const int32_t* cu_seqlens,
                                            const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                                            int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n,
                                            int64_t x_stride_h, int64_t y_stride_n, int64_t y_stride_h, int64_t bias_stride_h, int dtype,
                                            void* stream) {
  LinParams p;
  int rc = lin_fill(p, x, w, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, kernel_size, kernel_stride, x_stride_n, x_stride_h, dtype);
  if (rc != NSA_OK) return rc;
  if (total_y > 0 && (!y || (y_stride_n | y_stride_h) % 4 != 0 || (uintptr_t)y % 8 != 0)) return NSA_ERR_UNSUPPORTED;
  if (bias && (bias_stride_h % 4 != 0 || (uintptr_t)bias % 8 != 0)) return NSA_ERR_UNSUPPORTED;
  p.y = y; p.ysn = y_stride_n; p.ysh = y_stride_h; p.bias = bias; p.bsh = bias_stride_h;
  return lin_dispatch(p, 0, head_dim, dtype, (hipStream_t)stream);
}

extern "C" int nsa_linear_compress_fwd(const void* x, const void* w, void* y, const int32_t* cu_seqlens, const int32_t* y_cu_seqlens,
                                       int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads, int64_t head_dim,
                                       int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n, int64_t x_stride_h,
                                       int64_t y_stride_n, int64_t y_stride_h, int dtype, void* workspace, size_t workspace_bytes,
                                       void* stream) {
  (void)workspace; (void)workspace_bytes;
  return nsa_linear_compress_fwd_bias(x, w, nullptr, y, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, head_dim, kernel_size,
                                      kernel_stride, x_stride_n, x_stride_h, y_stride_n, y_stride_h, 0, dtype, stream);
}

extern "C" int nsa_linear_compress_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, const int32_t* cu_seqlens,
                                       const int32_t* y_cu_seqlens, int64_t total_x, int64_t total_y, int64_t batch, int64_t num_heads,
                                       int64_t head_dim, int64_t kernel_size, int64_t kernel_stride, int64_t x_stride_n,
                                       int64_t x_stride_h, int64_t dy_stride_n, int64_t dy_stride_h, int64_t dx_stride_n,
                                       int64_t dx_stride_h, int dtype, void* stream) {
  LinParams p;
  int rc = lin_fill(p, x, w, cu_seqlens, y_cu_seqlens, total_x, total_y, batch, num_heads, kernel_size, kernel_stride, x_stride_n, x_stride_h, dtype);
  if (rc != NSA_OK) return rc;
  if (!dx || !dw || (total_y > 0 && !dy)) return NSA_ERR_BAD_ARG;
  if ((dy_stride_n | dy_stride_h) % 8 != 0 || (dx_stride_n | dx_stride_h) % 4 != 0) return NSA_ERR_UNSUPPORTED;
  if ((uintptr_t)dy % 16 != 0 || ((uintptr_t)dx | (uintptr_t)dw) % 8 != 0) return NSA_ERR_UNSUPPORTED;
  p.dy = dy; p.dx = dx; p.dw = dw; p.dysn = dy_stride_n; p.dysh = dy_stride_h; p.dxsn = dx_stride_n; p.dxsh = dx_stride_h;
  return lin_dispatch(p, 1, head_dim, dtype, (hipStream_t)stream);
}
