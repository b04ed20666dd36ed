// Gated sum of the three attention branches, out[n, h, :] = g[n, h, 0] * a + g[n, h, 1] * b + g[n, h, 2] * c,
// in one pass (four tensor reads/writes instead of the fifteen of five element-wise launches).  Products and
// partial sums are rounded to the element type in the order of the expression above, so the result is
// bit-identical to evaluating it with element-wise tensor arithmetic.  HBM-bound.
#include "nsa_common.h"

struct CombineParams {
  const void* gate; const void* br[3]; void* out;
  long long n_rows; int H;
  long long gsn, gsh, gsk, bsn[3], bsh[3], osn, osh;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void gate_combine_kernel(CombineParams p) {
  using v8 = typename Elem<T>::v8;
  constexpr int PER = D / 8;
  const long long total = p.n_rows * p.H * PER;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    const int c = (int)(i % PER);
    const int h = (int)((i / PER) % p.H);
    const long long n = i / ((long long)PER * p.H);
    const T* g = (const T*)p.gate + n * p.gsn + (long long)h * p.gsh;
    const float g0 = (float)g[0], g1 = (float)g[p.gsk], g2 = (float)g[2 * p.gsk];
    const v8 a = ld16<v8>((const T*)p.br[0] + n * p.bsn[0] + (long long)h * p.bsh[0] + 8 * c);
    const v8 b = ld16<v8>((const T*)p.br[1] + n * p.bsn[1] + (long long)h * p.bsh[1] + 8 * c);
    const v8 d = ld16<v8>((const T*)p.br[2] + n * p.bsn[2] + (long long)h * p.bsh[2] + 8 * c);
    v8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float x = rounded<T>(g0 * (float)a[e]), y = rounded<T>(g1 * (float)b[e]), z = rounded<T>(g2 * (float)d[e]);
      o[e] = (T)(rounded<T>(x + y) + z);
    }
    st16((T*)p.out + n * p.osn + (long long)h * p.osh + 8 * c, o);
  }
}

// Backward of the gated sum: d branch_i = g_i * dO (one rounding, as the element-wise product), and
// d g_i = sum over head_dim of dO * branch_i, each product rounded to the element type before the fp32 sum as
// element-wise arithmetic followed by a reduction would.  A row (token, head) is handled by head_dim / 8
// neighbouring threads; their three partial sums meet in LDS.  HBM-bound: 4 reads + 3 writes of [N, H, D].
struct CombineBwdParams {
  const void* gate; const void* br[3]; const void* dout; void* dbr[3]; void* dgate;
  long long n_rows; int H;
  long long gsn, gsh, gsk, bsn[3], bsh[3], dsn, dsh;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void gate_combine_bwd_kernel(CombineBwdParams p) {
  using v8 = typename Elem<T>::v8;
  constexpr int PER = D / 8, ROWS = 256 / PER;  // rows per workgroup pass (threads past ROWS * PER idle)
  __shared__ float part[3][256];
  const int tid = threadIdx.x, c = tid % PER, rl = tid / PER;
  const long long n_hrows = p.n_rows * p.H;
  for (long long r0 = (long long)blockIdx.x * ROWS; r0 < n_hrows; r0 += (long long)gridDim.x * ROWS) {
    const long long r = r0 + rl;
    const bool live = rl < ROWS && r < n_hrows;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
    if (live) {
      const long long n = r / p.H;
      const int h = (int)(r % p.H);
      const T* g = (const T*)p.gate + n * p.gsn + (long long)h * p.gsh;
      const float g0 = (float)g[0], g1 = (float)g[p.gsk], g2 = (float)g[2 * p.gsk];
      const v8 go = ld16<v8>((const T*)p.dout + n * p.dsn + (long long)h * p.dsh + 8 * c);
      const v8 a = ld16<v8>((const T*)p.br[0] + n * p.bsn[0] + (long long)h * p.bsh[0] + 8 * c);
      const v8 b = ld16<v8>((const T*)p.br[1] + n * p.bsn[1] + (long long)h * p.bsh[1] + 8 * c);
      const v8 d = ld16<v8>((const T*)p.br[2] + n * p.bsn[2] + (long long)h * p.bsh[2] + 8 * c);
      v8 da, db, dd;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float x = (float)go[e];
        da[e] = (T)(g0 * x); db[e] = (T)(g1 * x); dd[e] = (T)(g2 * x);
        s0 += rounded<T>(x * (float)a[e]); s1 += rounded<T>(x * (float)b[e]); s2 += rounded<T>(x * (float)d[e]);
      }
      const long long off = (r * PER + c) * 8;  // gradients are written densely, [N, H, D]
      st16((T*)p.dbr[0] + off, da); st16((T*)p.dbr[1] + off, db); st16((T*)p.dbr[2] + off, dd);
    }
    part[0][tid] = s0; part[1][tid] = s1; part[2][tid] = s2;
    __syncthreads();
    if (live && c < 3) {
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < PER; j++) t += part[c][rl * PER + j];
      ((T*)p.dgate)[r * 3 + c] = (T)t;
    }
    __syncthreads();
  }
}

template <typename T>
static int combine_bwd_dispatch(const CombineBwdParams& p, int d, hipStream_t s) {
  const long long rows = p.n_rows * p.H;
  const int per = d / 8, rpw = 256 / per;
  const long long wgs = (rows + rpw - 1) / rpw;
  const unsigned grid = (unsigned)(wgs < 65536 ? wgs : 65536);
  switch (d) {
    case 32: gate_combine_bwd_kernel<T, 32><<<grid, 256, 0, s>>>(p); break;
    case 64: gate_combine_bwd_kernel<T, 64><<<grid, 256, 0, s>>>(p); break;
    case 96: gate_combine_bwd_kernel<T, 96><<<grid, 256, 0, s>>>(p); break;
    case 128: gate_combine_bwd_kernel<T, 128><<<grid, 256, 0, s>>>(p); break;
    default: return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch();
}

template <typename T>
static int combine_dispatch(const CombineParams& p, int d, hipStream_t s) {
  const long long pieces = p.n_rows * p.H * (d / 8);
  const unsigned grid = (unsigned)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
  switch (d) {
    case 32: gate_combine_kernel<T, 32><<<grid, 256, 0, s>>>(p); break;
    case 64: gate_combine_kernel<T, 64><<<grid, 256, 0, s>>>(p); break;
    case 96: gate_combine_kernel<T, 96><<<grid, 256, 0, s>>>(p); break;
    case 128: gate_combine_kernel<T, 128><<<grid, 256, 0, s>>>(p); break;
    default: return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch();
}

extern "C" int nsa_gate_combine(const void* gate, const void* branch0, const void* branch1, const void* branch2, void* out,
                                int64_t n_rows, int64_t num_q_heads, int64_t head_dim, const int64_t* strides, int dtype, void* stream) {
  if (n_rows < 0 || num_q_heads <= 0) return NSA_ERR_BAD_ARG;
  if (n_rows == 0) return NSA_OK;  // nothing to do (the pointers of empty tensors may be null)
  if (!gate || !branch0 || !branch1 || !branch2 || !out || !strides) return NSA_ERR_BAD_ARG;
  CombineParams p;
  p.gate = gate; p.br[0] = branch0; p.br[1] = branch1; p.br[2] = branch2; p.out = out;
  p.n_rows = n_rows; p.H = (int)num_q_heads;
  p.gsn = strides[0]; p.gsh = strides[1]; p.gsk = strides[2];
  for (int i = 0; i < 3; i++) { p.bsn[i] = strides[3 + 2 * i]; p.bsh[i] = strides[4 + 2 * i]; }
  p.osn = strides[9]; p.osh = strides[10];
  for (int i = 3; i < 11; i++) if (strides[i] % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)branch0 | (uintptr_t)branch1 | (uintptr_t)branch2 | (uintptr_t)out) % 16 != 0) return NSA_ERR_UNSUPPORTED;
  if (dtype == NSA_BF16) return combine_dispatch<__bf16>(p, (int)head_dim, (hipStream_t)stream);
  if (dtype == NSA_FP16) return combine_dispatch<_Float16>(p, (int)head_dim, (hipStream_t)stream);
  return NSA_ERR_UNSUPPORTED;
}

extern "C" int nsa_gate_combine_bwd(const void* gate, const void* branch0, const void* branch1, const void* branch2, const void* dout,
                                    void* dgate, void* dbranch0, void* dbranch1, void* dbranch2, int64_t n_rows, int64_t num_q_heads,
                                    int64_t head_dim, const int64_t* strides, int dtype, void* stream) {
  if (n_rows < 0 || num_q_heads <= 0) return NSA_ERR_BAD_ARG;
  if (n_rows == 0) return NSA_OK;
  if (!gate || !branch0 || !branch1 || !branch2 || !dout || !dgate || !dbranch0 || !dbranch1 || !dbranch2 || !strides) return NSA_ERR_BAD_ARG;
  CombineBwdParams p;
  p.gate = gate; p.br[0] = branch0; p.br[1] = branch1; p.br[2] = branch2; p.dout = dout;
  p.dbr[0] = dbranch0; p.dbr[1] = dbranch1; p.dbr[2] = dbranch2; p.dgate = dgate;
  p.n_rows = n_rows; p.H = (int)num_q_heads;
  p.gsn = strides[0]; p.gsh = strides[1]; p.gsk = strides[2];
  for (int i = 0; i < 3; i++) { p.bsn[i] = strides[3 + 2 * i]; p.bsh[i] = strides[4 + 2 * i]; }
  p.dsn = strides[9]; p.dsh = strides[10];
  for (int i = 3; i < 11; i++) if (strides[i] % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)branch0 | (uintptr_t)branch1 | (uintptr_t)branch2 | (uintptr_t)dout | (uintptr_t)dbranch0 | (uintptr_t)dbranch1 |
       (uintptr_t)dbranch2) % 16 != 0)
    return NSA_ERR_UNSUPPORTED;
  if (dtype == NSA_BF16) return combine_bwd_dispatch<__bf16>(p, (int)head_dim, (hipStream_t)stream);
  if (dtype == NSA_FP16) return combine_bwd_dispatch<_Float16>(p, (int)head_dim, (hipStream_t)stream);
  return NSA_ERR_UNSUPPORTED;
}
