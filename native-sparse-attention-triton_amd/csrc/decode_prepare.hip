// Everything a decode step does before its three attention branches, in one launch: the new token's K/V go to
// the staging window, a window that has become complete is pooled into one compressed K/V token, query, key
// and compressed key are rotated (positions = cache lengths, read here), and the three slabs and four length
// vectors are updated.  Run as separate operators this is eight launches of a few microseconds each, every
// one of them latency-bound on a few KiB per sequence; the arithmetic (pooling in fp32 in window order, the
// rotary products rounded to the element type one by one, the bias added in the element type) is kept
// identical, so the cache contents and the rotated query match the separate operators bit for bit.
// One workgroup per sequence.
#include "nsa_common.h"

typedef unsigned short u16;

struct PrepParams {
  const void* q; const void* k; const void* v; void* q_out;
  const void* wk; const void* wv; const void* bias_k; const float* inv_freq;
  u16* stage_slab; int32_t* stage_len; u16* cmp_slab; int32_t* cmp_len; u16* full_slab; int32_t* full_len; u16* ring_slab; int32_t* ring_len;
  int Hq, H, max_batch, ks, st, cmp_rows, full_rows, window;
  long long qsb, qsh, ksb, ksh, vsb, vsh, osb, osh;
  float scaling;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void decode_prepare_kernel(PrepParams p) {
  using v8 = typename Elem<T>::v8;
  constexpr int HALF = D / 2, VEC = HALF / 8, C = D / 8;
  __shared__ float cos_s[2][HALF], sin_s[2][HALF];
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn[];
  T* ck_s = reinterpret_cast<T*>(dyn);   // [H][D]: pooled key of the completed window, before its rotation
  const int b = blockIdx.x, tid = threadIdx.x;
  const long long HD = (long long)p.H * D;
  int n = p.stage_len[b];
  const int nc = p.cmp_len[b], nf = p.full_len[b], nr = p.ring_len[b];
  // cos / sin of the two positions: row 0 for the query and the key (position = tokens already cached), row 1
  // for the compressed key (compressed tokens already cached, kernel_stride apart)
  for (int i = tid; i < 2 * HALF; i += 256) {
    const int which = i / HALF, j = i % HALF;
    const int pos = which ? nc * p.st : nf;
    const float ang = (float)pos * p.inv_freq[j];
    cos_s[which][j] = rounded<T>(cosf(ang) * p.scaling);
    sin_s[which][j] = rounded<T>(sinf(ang) * p.scaling);
  }
  __syncthreads();  // every wave holds the old lengths before anything is stored
  // ---- staging window: when full, rows [st, ks) move to [0, ks - st), st rows at a time (a group's source rows
  // are the next group's destination, so every group is read completely before the next one is written)
  const long long stage_kv = (long long)p.max_batch * p.ks * HD;
  u16* stage = p.stage_slab + (long long)b * p.ks * HD;
  if (n == p.ks) {
    const int per = (int)(p.st * HD / 8);  // 16-byte pieces of one group of st rows
    for (int g = 0; (g + 1) * p.st < p.ks; g++) {
      for (int which = 0; which < 2; which++) {
        u16* s = stage + which * stage_kv;
        for (int i = tid; i < per; i += 256)
          *reinterpret_cast<uint4*>(s + (long long)g * p.st * HD + 8ll * i) = *reinterpret_cast<const uint4*>(s + (long long)(g + 1) * p.st * HD + 8ll * i);
      }
      __syncthreads();
    }
    n -= p.st;
  }
  const T* kin = (const T*)p.k + (long long)b * p.ksb;
  const T* vin = (const T*)p.v + (long long)b * p.vsb;
  for (int i = tid; i < p.H * C; i += 256) {
    const int h = i / C, c = i % C;
    *reinterpret_cast<uint4*>(stage + (long long)n * HD + (long long)h * D + 8 * c) = *reinterpret_cast<const uint4*>(kin + (long long)h * p.ksh + 8 * c);
    *reinterpret_cast<uint4*>(stage + stage_kv + (long long)n * HD + (long long)h * D + 8 * c) = *reinterpret_cast<const uint4*>(vin + (long long)h * p.vsh + 8 * c);
  }
  const int n_new = n + 1;
  const bool new_cmp = n_new == p.ks && nc < p.cmp_rows;
  __threadfence_block();
  __syncthreads();  // the window, new row included, is visible to the whole workgroup
  // ---- a completed window becomes one compressed token: y = sum_k w[h, k] * row k, fp32 in window order
  const long long cmp_kv = (long long)p.max_batch * p.cmp_rows * HD;
  u16* cmp_row = p.cmp_slab + ((long long)b * p.cmp_rows + nc) * HD;
  if (new_cmp) {
    const float wavg = 1.f / (float)p.ks;
    for (int i = tid; i < 2 * p.H * C; i += 256) {
      const int which = i / (p.H * C), h = (i / C) % p.H, c = i % C;
      const T* wp = (const T*)(which ? p.wv : p.wk);
      const u16* xp = stage + which * stage_kv + (long long)h * D + 8 * c;
      float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      for (int k = 0; k < p.ks; k++) {
        const v8 xv = ld16<v8>(xp + (long long)k * HD);
        const float wk = wp ? (float)wp[(long long)h * p.ks + k] : wavg;
#pragma unroll
        for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(wk, (float)xv[j], acc[j]);
      }
      v8 out;
      if (which == 0) {
        const T* bp = p.bias_k ? (const T*)p.bias_k + (long long)h * D + 8 * c : nullptr;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          float y = rounded<T>(acc[j]);
          if (bp) y = rounded<T>(y + (float)bp[j]);
          out[j] = (T)y;
        }
        st16(ck_s + h * D + 8 * c, out);
      } else {
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = (T)acc[j];
        st16(cmp_row + cmp_kv + (long long)h * D + 8 * c, out);
      }
    }
  }
  __syncthreads();
  // ---- rotations.  Items: query heads, then key heads, then (if a window completed) compressed key heads; the
  // rotated key goes to the full-length slab and to the sliding ring, the value rows are copied alongside
  const long long full_kv = (long long)p.max_batch * p.full_rows * HD, ring_kv = (long long)p.max_batch * p.window * HD;
  u16* full_row = p.full_slab + ((long long)b * p.full_rows + nf) * HD;
  u16* ring_row = p.ring_slab + ((long long)b * p.window + nr % p.window) * HD;
  const bool room = nf < p.full_rows;
  const int n_items = (p.Hq + p.H + (new_cmp ? p.H : 0)) * VEC;
  for (int i = tid; i < n_items; i += 256) {
    const int hh = i / VEC, c8 = (i % VEC) * 8;
    const int kind = hh < p.Hq ? 0 : (hh < p.Hq + p.H ? 1 : 2);
    const int h = kind == 0 ? hh : (kind == 1 ? hh - p.Hq : hh - p.Hq - p.H);
    const T* src = kind == 0 ? (const T*)p.q + (long long)b * p.qsb + (long long)h * p.qsh
                 : kind == 1 ? kin + (long long)h * p.ksh : ck_s + h * D;
    const int tab = kind == 2;
    const v8 x1 = ld16<v8>(src + c8), x2 = ld16<v8>(src + HALF + c8);
    v8 o1, o2;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float c = cos_s[tab][c8 + e], s = sin_s[tab][c8 + e];
      const float a1 = (float)x1[e], a2 = (float)x2[e];
      o1[e] = (T)(rounded<T>(a1 * c) - rounded<T>(a2 * s));
      o2[e] = (T)(rounded<T>(a2 * c) + rounded<T>(a1 * s));
    }
    if (kind == 0) {
      T* dst = (T*)p.q_out + (long long)b * p.osb + (long long)h * p.osh;
      st16(dst + c8, o1); st16(dst + HALF + c8, o2);
    } else if (kind == 1) {
      if (room) { st16(full_row + (long long)h * D + c8, o1); st16(full_row + (long long)h * D + HALF + c8, o2); }
      st16(ring_row + (long long)h * D + c8, o1); st16(ring_row + (long long)h * D + HALF + c8, o2);
    } else {
      st16(cmp_row + (long long)h * D + c8, o1); st16(cmp_row + (long long)h * D + HALF + c8, o2);
    }
  }
  for (int i = tid; i < p.H * C; i += 256) {
    const int h = i / C, c = i % C;
    const uint4 val = *reinterpret_cast<const uint4*>(vin + (long long)h * p.vsh + 8 * c);
    if (room) *reinterpret_cast<uint4*>(full_row + full_kv + (long long)h * D + 8 * c) = val;
    *reinterpret_cast<uint4*>(ring_row + ring_kv + (long long)h * D + 8 * c) = val;
  }
  if (tid == 0) {
    p.stage_len[b] = n_new;
    if (new_cmp) p.cmp_len[b] = nc + 1;
    if (room) p.full_len[b] = nf + 1;
    p.ring_len[b] = nr + 1;
  }
}

template <typename T>
static int prepare_dispatch(const PrepParams& p, int batch, int d, hipStream_t s) {
  const size_t dyn = (size_t)p.H * d * sizeof(T);
  switch (d) {
    case 32: decode_prepare_kernel<T, 32><<<batch, 256, dyn, s>>>(p); break;
    case 64: decode_prepare_kernel<T, 64><<<batch, 256, dyn, s>>>(p); break;
    case 96: decode_prepare_kernel<T, 96><<<batch, 256, dyn, s>>>(p); break;
    case 128: decode_prepare_kernel<T, 128><<<batch, 256, dyn, s>>>(p); break;
    default: return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch();
}

extern "C" int nsa_decode_prepare(const void* q, const void* k, const void* v, void* q_out, const void* pool_weight_k,
                                  const void* pool_weight_v, const void* bias_k, const float* inv_freq, float attention_scaling,
                                  void* stage_slab, int32_t* stage_len, void* compress_slab, int32_t* compress_len, void* sparse_slab,
                                  int32_t* sparse_len, void* sliding_slab, int32_t* sliding_len, int64_t batch, int64_t num_q_heads,
                                  int64_t num_kv_heads, int64_t head_dim, const int64_t* strides, int64_t max_batch, int64_t kernel_size,
                                  int64_t kernel_stride, int64_t compress_rows, int64_t sparse_rows, int64_t window_size, int dtype,
                                  void* stream) {
  if (!q || !k || !v || !q_out || !inv_freq || !strides || !stage_slab || !stage_len || !compress_slab || !compress_len || !sparse_slab ||
      !sparse_len || !sliding_slab || !sliding_len)
    return NSA_ERR_BAD_ARG;
  if (batch <= 0 || batch > max_batch || num_q_heads <= 0 || num_kv_heads <= 0 || kernel_size <= 0 || kernel_stride <= 0 ||
      kernel_size % kernel_stride != 0 || compress_rows <= 0 || sparse_rows <= 0 || window_size <= 0)
    return NSA_ERR_BAD_ARG;
  if (dtype != NSA_BF16 && dtype != NSA_FP16) return NSA_ERR_UNSUPPORTED;
  if (num_kv_heads * head_dim * 2 > 48 * 1024) return NSA_ERR_UNSUPPORTED;   // pooled key staged in LDS
  for (int i = 0; i < 8; i++) if (strides[i] % 8 != 0) return NSA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)q_out | (uintptr_t)stage_slab | (uintptr_t)compress_slab |
       (uintptr_t)sparse_slab | (uintptr_t)sliding_slab | (uintptr_t)bias_k) % 16 != 0)
    return NSA_ERR_UNSUPPORTED;
  PrepParams p;
  p.q = q; p.k = k; p.v = v; p.q_out = q_out; p.wk = pool_weight_k; p.wv = pool_weight_v; p.bias_k = bias_k; p.inv_freq = inv_freq;
  p.stage_slab = (u16*)stage_slab; p.stage_len = stage_len; p.cmp_slab = (u16*)compress_slab; p.cmp_len = compress_len;
  p.full_slab = (u16*)sparse_slab; p.full_len = sparse_len; p.ring_slab = (u16*)sliding_slab; p.ring_len = sliding_len;
  p.Hq = (int)num_q_heads; p.H = (int)num_kv_heads; p.max_batch = (int)max_batch; p.ks = (int)kernel_size; p.st = (int)kernel_stride;
  p.cmp_rows = (int)compress_rows; p.full_rows = (int)sparse_rows; p.window = (int)window_size;
  p.qsb = strides[0]; p.qsh = strides[1]; p.ksb = strides[2]; p.ksh = strides[3]; p.vsb = strides[4]; p.vsh = strides[5];
  p.osb = strides[6]; p.osh = strides[7];
  p.scaling = attention_scaling;
  if (dtype == NSA_BF16) return prepare_dispatch<__bf16>(p, (int)batch, (int)head_dim, (hipStream_t)stream);
  return prepare_dispatch<_Float16>(p, (int)batch, (int)head_dim, (hipStream_t)stream);
}
