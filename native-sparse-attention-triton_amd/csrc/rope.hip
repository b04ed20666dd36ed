// Rotary position embedding over varlen rows, x [N, H, D] -> out [N, H, D]:
//   out[..., :D/2] = x1 * cos - x2 * sin,  out[..., D/2:] = x2 * cos + x1 * sin,  angle = position * inv_freq[i].
// One workgroup per row: the first D/2 threads evaluate cos/sin of the row's position once (fp32, full
// range reduction: angles reach 1e5 rad), every head then reuses them from LDS.  cos/sin and each product
// are rounded to the element type before the next operation, as element-wise bf16/fp16 tensor arithmetic
// does, so results match a framework-level x * cos + rotate_half(x) * sin.  HBM-bound: one read and one
// write of x.
#include "nsa_common.h"

struct RopeParams {
  const void* x; void* out; const float* inv_freq; const int32_t* cu;
  int n_rows, batch, H, step, stride;
  long long xsn, xsh, osn, osh;
  float scaling;
  int inverse;
};

// V: elements per load/store piece (8 when half a row is a multiple of 8 elements, else 4); any head_dim that is a
// multiple of 8 up to 2 * ROPE_MAX_HALF runs.
constexpr int ROPE_MAX_HALF = 128;
template <typename T, int V>
__global__ __launch_bounds__(256) void rope_kernel(RopeParams p, int D) {
  typedef T vec __attribute__((ext_vector_type(V)));
  const int HALF = D / 2, VEC = HALF / V;  // V-element pieces per half row
  __shared__ float cos_s[ROPE_MAX_HALF], sin_s[ROPE_MAX_HALF];
  const int n = blockIdx.x;
  int pos;
  if (p.step < 0) {   // the caller supplies one position index per row
    pos = p.cu[n] * p.stride;
  } else if (p.step == 0) {  // prefill: row n is token n - cu[b] of its sequence
    const int b = find_sequence(p.cu, p.batch, n);
    pos = (n - p.cu[b]) * p.stride;
  } else {            // decode: one row per sequence, `step` tokens after its prompt
    pos = (p.cu[n + 1] - p.cu[n] + p.step - 1) * p.stride;
  }
  if (threadIdx.x < HALF) {
    const float ang = (float)pos * p.inv_freq[threadIdx.x];
    const float c = rounded<T>(cosf(ang) * p.scaling), s = rounded<T>(sinf(ang) * p.scaling);
    cos_s[threadIdx.x] = c;
    sin_s[threadIdx.x] = p.inverse ? -s : s;
  }
  __syncthreads();
  const T* xr = (const T*)p.x + (long long)n * p.xsn;
  T* orow = (T*)p.out + (long long)n * p.osn;
  for (int i = threadIdx.x; i < p.H * VEC; i += 256) {
    const int h = i / VEC, c8 = (i % VEC) * V;
    const vec x1 = *reinterpret_cast<const vec*>(xr + (long long)h * p.xsh + c8), x2 = *reinterpret_cast<const vec*>(xr + (long long)h * p.xsh + HALF + c8);
    vec o1, o2;
#pragma unroll
    for (int e = 0; e < V; e++) {
      const float c = cos_s[c8 + e], s = sin_s[c8 + e];
      const float a1 = (float)x1[e], a2 = (float)x2[e];
      o1[e] = (T)(rounded<T>(a1 * c) - rounded<T>(a2 * s));
      o2[e] = (T)(rounded<T>(a2 * c) + rounded<T>(a1 * s));
    }
    *reinterpret_cast<vec*>(orow + (long long)h * p.osh + c8) = o1;
    *reinterpret_cast<vec*>(orow + (long long)h * p.osh + HALF + c8) = o2;
  }
}

template <typename T>
static int rope_dispatch(const RopeParams& p, int d, hipStream_t s) {
  if (d <= 0 || d % 8 != 0 || d > 2 * ROPE_MAX_HALF) return NSA_ERR_UNSUPPORTED;
  if (d % 16 == 0) rope_kernel<T, 8><<<p.n_rows, 256, 0, s>>>(p, d);
  else rope_kernel<T, 4><<<p.n_rows, 256, 0, s>>>(p, d);
  return nsa_check_launch();
}

extern "C" int nsa_rope(const void* x, void* out, const float* inv_freq, const int32_t* cu_seqlens, int64_t n_rows, int64_t batch,
                        int64_t num_heads, int64_t head_dim, int64_t x_stride_n, int64_t x_stride_h, int64_t o_stride_n,
                        int64_t o_stride_h, int64_t step, int64_t stride, float attention_scaling, int inverse, int dtype,
                        void* stream) {
  if (!x || !out || !inv_freq || !cu_seqlens) return NSA_ERR_BAD_ARG;
  if (n_rows < 0 || batch <= 0 || num_heads <= 0 || stride <= 0 || n_rows >= (1ll << 31)) return NSA_ERR_BAD_ARG;
  if (step > 0 && n_rows != batch) return NSA_ERR_BAD_ARG;
  // 16-byte pieces (8-byte ones when half a row is an odd multiple of 4 elements)
  const int64_t piece = head_dim % 16 == 0 ? 8 : 4;
  if ((x_stride_n | x_stride_h | o_stride_n | o_stride_h) % piece != 0 || ((uintptr_t)x | (uintptr_t)out) % (2 * piece) != 0) return NSA_ERR_UNSUPPORTED;
  if (n_rows == 0) return NSA_OK;
  RopeParams p;
  p.x = x; p.out = out; p.inv_freq = inv_freq; p.cu = cu_seqlens;
  p.n_rows = (int)n_rows; p.batch = (int)batch; p.H = (int)num_heads; p.step = (int)step; p.stride = (int)stride;
  p.xsn = x_stride_n; p.xsh = x_stride_h; p.osn = o_stride_n; p.osh = o_stride_h;
  p.scaling = attention_scaling; p.inverse = inverse;
  if (dtype == NSA_BF16) return rope_dispatch<__bf16>(p, (int)head_dim, (hipStream_t)stream);
  if (dtype == NSA_FP16) return rope_dispatch<_Float16>(p, (int)head_dim, (hipStream_t)stream);
  return NSA_ERR_UNSUPPORTED;
}
