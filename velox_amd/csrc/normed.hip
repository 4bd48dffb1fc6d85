// Kernels of decoders whose sub-layers read the residual stream itself and whose attention norms its queries and keys:
//
//   add_sinusoid:   hidden[t, 2i] += sin(p_t f_i), hidden[t, 2i + 1] += cos(p_t f_i)   (an absolute position encoding)
//   add_cast:       residual += delta; out = residual in the run dtype
//   norm_add:       residual += mult * y * rsqrt(mean(y^2) + eps) * w; out = residual in the run dtype   (the norm on a
//                   sub-layer's OUTPUT, float32 throughout, one rounding for the copy)
//   qk_norm_write:  RMS norm of the queries and of the keys (over the whole projection or per head), the query
//                   temperature, the blend of the values with an earlier layer's, queries written at the kernels' head
//                   size, keys and values into the paged cache (zeros in the padding channels)
#include "common.h"

// ---------------------------------------------------------------------------------------------
// The angle is worked out in float64 and brought into [-pi, pi] there, so that its error does not grow with the
// position; sine and cosine are then float32's.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) add_sinusoid_kernel(float* __restrict__ hidden, const int* __restrict__ positions, const double* __restrict__ freq,
                                                           int width) {
  const int t = blockIdx.x;
  const double p = (double)positions[t];
  float* row = hidden + (size_t)t * width;
  const int pairs = (width + 1) / 2;
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    double a = p * freq[i];
    a -= 6.283185307179586476925 * rint(a * 0.159154943091895335769);
    const float r = (float)a;
    row[2 * i] += sinf(r);
    if (2 * i + 1 < width) row[2 * i + 1] += cosf(r);
  }
}

extern "C" int velox_add_sinusoid(float* hidden, const int* positions, const double* freq, int tokens, int width, hipStream_t stream) {
  if (tokens <= 0) return 0;
  add_sinusoid_kernel<<<tokens, 256, 0, stream>>>(hidden, positions, freq, width);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
template <typename TD, typename TO>
__global__ void __launch_bounds__(256) add_cast_kernel(float* __restrict__ residual, const TD* __restrict__ delta, TO* __restrict__ out, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    float r = residual[i];
    if (delta) {
      r += to_f32(delta[i]);
      residual[i] = r;
    }
    if (out) out[i] = from_f32<TO>(r);
  }
}

// delta: nullptr or [T, H] of delta_dtype; out: nullptr (float32 run: the residual is its own copy) or bfloat16 [T, H]
extern "C" int velox_add_cast(float* residual, const void* delta, int delta_dtype, void* out_bf16, long long total, hipStream_t stream) {
  if (total <= 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  if (delta_dtype == VELOX_BF16)
    add_cast_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>(residual, (const bf16_t*)delta, (bf16_t*)out_bf16, (size_t)total);
  else
    add_cast_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>(residual, (const float*)delta, (bf16_t*)out_bf16, (size_t)total);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// norm_add: one workgroup per row.  y may come as `partials` stacked float32 tensors (partial sums of a split product),
// added first to last.  The row is held in registers between the two passes when it fits (CHUNKS x 256 elements).
// ---------------------------------------------------------------------------------------------
template <typename TD, int CHUNKS>
__global__ void __launch_bounds__(256) norm_add_kernel(float* __restrict__ residual, const TD* __restrict__ y, const float* __restrict__ weight,
                                                       bf16_t* __restrict__ out, int hidden, float eps, float mult, int partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const TD* src = y + row * hidden;
  float* res = residual + row * hidden;
  float held[CHUNKS > 0 ? CHUNKS : 1];
  float sumsq = 0.f;
  if constexpr (CHUNKS > 0) {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int i = threadIdx.x + 256 * c;
      float v = 0.f;
      if (i < hidden)
        for (int p = 0; p < partials; ++p) v += to_f32(src[p * partial_stride + i]);
      held[c] = v;
      sumsq += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += 256) {
      float v = 0.f;
      for (int p = 0; p < partials; ++p) v += to_f32(src[p * partial_stride + i]);
      sumsq += v * v;
    }
  }
  const float total = block_sum(sumsq, scratch);
  const float inv = 1.f / sqrtf(total / (float)hidden + eps);
  if constexpr (CHUNKS > 0) {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int i = threadIdx.x + 256 * c;
      if (i < hidden) {
        const float r = res[i] + mult * (held[c] * inv * weight[i]);
        res[i] = r;
        if (out) out[row * hidden + i] = from_f32<bf16_t>(r);
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += 256) {
      float v = 0.f;
      for (int p = 0; p < partials; ++p) v += to_f32(src[p * partial_stride + i]);
      const float r = res[i] + mult * (v * inv * weight[i]);
      res[i] = r;
      if (out) out[row * hidden + i] = from_f32<bf16_t>(r);
    }
  }
}

// The same with the row in registers as 4-element pieces: 8- or 16-byte accesses, up to 4 pieces per thread.  Needs
// hidden % 4 == 0, hidden <= 16 * threads and 16-byte aligned rows (the caller checks).
template <typename T> struct Piece4;
template <> struct Piece4<float> {
  float4_t v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
};
template <> struct Piece4<bf16_t> {
  short4_t v;
  __device__ __forceinline__ float get(int i) const { return __uint_as_float(((uint32_t)(uint16_t)v[i]) << 16); }
};

template <typename TD>
__global__ void norm_add_vec_kernel(float* __restrict__ residual, const TD* __restrict__ y, const float* __restrict__ weight, bf16_t* __restrict__ out,
                                    int hidden, float eps, float mult, int partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const TD* src = y + row * hidden;
  float* res = residual + row * hidden;
  float4_t held[4], old[4], w[4];
  float sumsq = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int at = (threadIdx.x + c * blockDim.x) * 4;
    held[c] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (at < hidden) {
      for (int p = 0; p < partials; ++p) {
        const Piece4<TD> q = *reinterpret_cast<const Piece4<TD>*>(src + p * partial_stride + at);
#pragma unroll
        for (int j = 0; j < 4; ++j) held[c][j] += q.get(j);
      }
      old[c] = *reinterpret_cast<const float4_t*>(res + at);  // (asked for before the reduction: its wait hides behind it)
      w[c] = *reinterpret_cast<const float4_t*>(weight + at);
#pragma unroll
      for (int j = 0; j < 4; ++j) sumsq += held[c][j] * held[c][j];
    }
  }
  const float total = block_sum(sumsq, scratch);
  const float inv = 1.f / sqrtf(total / (float)hidden + eps);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int at = (threadIdx.x + c * blockDim.x) * 4;
    if (at < hidden) {
      float4_t r;
      short4_t o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        r[j] = old[c][j] + mult * (held[c][j] * inv * w[c][j]);
        o[j] = bf16_bits(r[j]);
      }
      *reinterpret_cast<float4_t*>(res + at) = r;
      if (out) *reinterpret_cast<short4_t*>(out + row * hidden + at) = o;
    }
  }
}

template <typename TD>
static void norm_add_launch(float* residual, const void* y, const float* weight, void* out, int tokens, int hidden, float eps, float mult, int partials,
                            long long partial_stride, hipStream_t stream) {
  const TD* src = (const TD*)y;
  bf16_t* copy = (bf16_t*)out;
  // few rows: more threads each with less to do (the kernel is then a chain of waits); many rows: 256 threads a row
  const int threads = hidden <= 1024 ? 256 : (tokens <= 64 || hidden > 4096 ? (hidden > 8192 ? 1024 : 512) : 256);
  const bool aligned = (((uintptr_t)residual | (uintptr_t)y | (uintptr_t)weight | (uintptr_t)out) & 15) == 0 && (partial_stride % 4 == 0);
  if (aligned && hidden % 4 == 0 && hidden <= 16 * threads) {
    norm_add_vec_kernel<TD><<<tokens, threads, 0, stream>>>(residual, src, weight, copy, hidden, eps, mult, partials, (size_t)partial_stride);
    return;
  }
  if (hidden <= 1024) norm_add_kernel<TD, 4><<<tokens, 256, 0, stream>>>(residual, src, weight, copy, hidden, eps, mult, partials, (size_t)partial_stride);
  else if (hidden <= 4096) norm_add_kernel<TD, 16><<<tokens, 256, 0, stream>>>(residual, src, weight, copy, hidden, eps, mult, partials, (size_t)partial_stride);
  else norm_add_kernel<TD, 0><<<tokens, 256, 0, stream>>>(residual, src, weight, copy, hidden, eps, mult, partials, (size_t)partial_stride);
}

extern "C" int velox_norm_add(float* residual, const void* y, int y_dtype, const float* weight, void* out_bf16, int tokens, int hidden, float eps, float mult,
                              int partials, long long partial_stride, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (hidden < 1 || partials < 1 || (partials > 1 && y_dtype != VELOX_F32)) return -1;
  if (y_dtype == VELOX_BF16) norm_add_launch<bf16_t>(residual, y, weight, out_bf16, tokens, hidden, eps, mult, partials, partial_stride, stream);
  else norm_add_launch<float>(residual, y, weight, out_bf16, tokens, hidden, eps, mult, partials, partial_stride, stream);
  VELOX_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// qk_norm_write: one workgroup of four waves per token.  A row of `qkv` holds `heads` queries and `kv_heads` keys of `dim`
// channels and `kv_heads` values of `vdim`.  With `whole` the queries (and the keys) are normed over all their heads at
// once with weights of that size, else head by head with one weight of `dim` entries.  Heads are handed to the waves in
// turn; a head's sum of squares is one wave's reduction, in a fixed order.  Everything between the load and the store is
// float32; the stores round once.
//   q_out [T, heads * D]; k_cache [pages, kv_heads, page, D]; v_cache [pages, kv_heads, D, page]; channels from dim (vdim)
//   to D are written as zeros.  first: an earlier layer's values of the same tokens, rows `first_stride` apart, a
//   token's at `first_offset`; lambda: their weight, one float32 on the device.
// ---------------------------------------------------------------------------------------------
struct QkNormArgs {
  const void* qkv;
  int qkv_stride;
  void* q_out;
  const float* q_weight;
  const float* k_weight;
  const int* positions;
  const void* first;
  int first_stride, first_offset;
  const float* lambda;
  const int* slot_mapping;
  void* k_cache;
  void* v_cache;
  int heads, kv_heads, dim, vdim, D, page_shift, whole, write_kv, temp_every;
  float eps, temp_coef;
};

template <typename T>
__global__ void __launch_bounds__(256) qk_norm_write_kernel(const QkNormArgs a) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = (const T*)a.qkv + (size_t)t * a.qkv_stride;
  const int q_size = a.heads * a.dim, k_size = a.kv_heads * a.dim;
  float inv_q = 0.f, inv_k = 0.f;
  if (a.whole) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < q_size; i += blockDim.x) { const float v = to_f32(row[i]); sq += v * v; }
    for (int i = threadIdx.x; i < k_size; i += blockDim.x) { const float v = to_f32(row[q_size + i]); sk += v * v; }
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    inv_q = 1.f / sqrtf(sq / (float)q_size + a.eps);
    inv_k = 1.f / sqrtf(sk / (float)k_size + a.eps);
  }
  float temp = 1.f;
  if (a.temp_every > 0) temp = 1.f + a.temp_coef * logf((float)((a.positions[t] + 1) / a.temp_every + 1));
  const int page_size = 1 << a.page_shift;
  int page = 0, offset = 0;
  if (a.write_kv) {
    const int slot = a.slot_mapping[t];
    page = slot >> a.page_shift;
    offset = slot & (page_size - 1);
  }
  const int D = a.D;
  // queries and keys: head `h` of heads + kv_heads
  for (int h = wave; h < a.heads + (a.write_kv ? a.kv_heads : 0); h += 4) {
    const bool is_q = h < a.heads;
    const int g = is_q ? h : h - a.heads;
    const T* src = row + (is_q ? h * a.dim : q_size + g * a.dim);
    float inv = is_q ? inv_q : inv_k;
    if (!a.whole) {
      float s = 0.f;
      for (int c = lane; c < a.dim; c += 64) { const float v = to_f32(src[c]); s += v * v; }
      s = wave_sum(s);
      inv = 1.f / sqrtf(s / (float)a.dim + a.eps);
    }
    const float* w = (is_q ? a.q_weight : a.k_weight) + (a.whole ? g * a.dim : 0);
    const float factor = is_q ? temp : 1.f;
    T* dst = is_q ? (T*)a.q_out + ((size_t)t * a.heads + h) * D
                  : (T*)a.k_cache + (((size_t)page * a.kv_heads + g) * page_size + offset) * D;
    for (int c = lane; c < D; c += 64) dst[c] = c < a.dim ? from_f32<T>(to_f32(src[c]) * inv * w[c] * factor) : from_f32<T>(0.f);
  }
  if (!a.write_kv) return;
  // values, transposed inside the page
  const float lam = a.first ? *a.lambda : 0.f;
  const T* first = a.first ? (const T*)a.first + (size_t)t * a.first_stride + a.first_offset : nullptr;
  const T* values = row + q_size + k_size;
  for (int i = threadIdx.x; i < a.kv_heads * D; i += blockDim.x) {
    const int g = i / D, c = i % D;
    float v = 0.f;
    if (c < a.vdim) {
      v = to_f32(values[g * a.vdim + c]);
      if (first) v = (1.f - lam) * v + lam * to_f32(first[g * a.vdim + c]);
    }
    ((T*)a.v_cache)[(((size_t)page * a.kv_heads + g) * D + c) * page_size + offset] = from_f32<T>(v);
  }
}

// bfloat16 rows whose heads are whole 16-byte pieces (dim, vdim and D multiples of 8, at most QK_MAX_UNITS pieces of
// queries and keys per thread): a thread holds pieces of 8 channels.  The sums of squares are built in a fixed order:
// a piece's eight squares, the pieces of a head in order, the heads in order.
#define QK_MAX_UNITS 4
typedef __bf16 qk_bf16x8_t __attribute__((ext_vector_type(8)));

__global__ void __launch_bounds__(256) qk_norm_write_vec_kernel(const QkNormArgs a) {
  extern __shared__ float lds[];  // piece sums [q_units + k_units], head sums [heads + kv_heads]
  const int t = blockIdx.x;
  const bf16_t* row = (const bf16_t*)a.qkv + (size_t)t * a.qkv_stride;
  const int per_head = a.dim / 8;                       // pieces of a query or key head
  const int q_units = a.heads * per_head, k_units = a.kv_heads * per_head;
  const int units = q_units + (a.write_kv ? k_units : 0);
  float* piece_sum = lds;
  float* head_sum = lds + q_units + k_units;
  qk_bf16x8_t held[QK_MAX_UNITS];
#pragma unroll
  for (int c = 0; c < QK_MAX_UNITS; ++c) {
    const int u = threadIdx.x + 256 * c;
    if (u < units) {
      held[c] = *reinterpret_cast<const qk_bf16x8_t*>(row + 8 * u);  // (queries, then keys: one run of the row)
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float v = (float)held[c][j]; s += v * v; }
      piece_sum[u] = s;
    }
  }
  float temp = 1.f;
  if (a.temp_every > 0) temp = 1.f + a.temp_coef * logf((float)((a.positions[t] + 1) / a.temp_every + 1));
  const int page_size = 1 << a.page_shift;
  int page = 0, offset = 0;
  if (a.write_kv) {
    const int slot = a.slot_mapping[t];
    page = slot >> a.page_shift;
    offset = slot & (page_size - 1);
  }
  __syncthreads();
  const int all_heads = a.heads + (a.write_kv ? a.kv_heads : 0);
  for (int h = threadIdx.x; h < all_heads; h += 256) {
    float s = 0.f;
    for (int p = 0; p < per_head; ++p) s += piece_sum[h * per_head + p];
    head_sum[h] = s;
  }
  __syncthreads();
  float inv_q = 0.f, inv_k = 0.f;
  if (a.whole) {
    float sq = 0.f, sk = 0.f;
    for (int h = 0; h < a.heads; ++h) sq += head_sum[h];
    if (a.write_kv)
      for (int h = 0; h < a.kv_heads; ++h) sk += head_sum[a.heads + h];
    inv_q = 1.f / sqrtf(sq / (float)(a.heads * a.dim) + a.eps);
    inv_k = 1.f / sqrtf(sk / (float)(a.kv_heads * a.dim) + a.eps);
  }
  const int D = a.D;
#pragma unroll
  for (int c = 0; c < QK_MAX_UNITS; ++c) {
    const int u = threadIdx.x + 256 * c;
    if (u >= units) continue;
    const int h = u / per_head, c0 = (u % per_head) * 8;  // head (queries, then keys) and first channel
    const bool is_q = h < a.heads;
    const int g = is_q ? h : h - a.heads;
    const float inv = a.whole ? (is_q ? inv_q : inv_k) : 1.f / sqrtf(head_sum[h] / (float)a.dim + a.eps);
    const float* w = (is_q ? a.q_weight : a.k_weight) + (a.whole ? g * a.dim : 0) + c0;
    const float factor = is_q ? temp : 1.f;
    qk_bf16x8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (bf16_t)((float)held[c][j] * inv * w[j] * factor);
    bf16_t* dst = is_q ? (bf16_t*)a.q_out + ((size_t)t * a.heads + h) * D
                       : (bf16_t*)a.k_cache + (((size_t)page * a.kv_heads + g) * page_size + offset) * D;
    *reinterpret_cast<qk_bf16x8_t*>(dst + c0) = o;
  }
  // padding channels of queries and keys
  const int pad = (D - a.dim) / 8;
  for (int i = threadIdx.x; i < all_heads * pad; i += 256) {
    const int h = i / pad, c0 = a.dim + (i % pad) * 8;
    const bool is_q = h < a.heads;
    bf16_t* dst = is_q ? (bf16_t*)a.q_out + ((size_t)t * a.heads + h) * D
                       : (bf16_t*)a.k_cache + (((size_t)page * a.kv_heads + (h - a.heads)) * page_size + offset) * D;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    *reinterpret_cast<float4_t*>(dst + c0) = zero;
  }
  if (!a.write_kv) return;
  // values: pieces of 8 channels, each channel to its own row of the transposed page
  const float lam = a.first ? *a.lambda : 0.f;
  const bf16_t* first = a.first ? (const bf16_t*)a.first + (size_t)t * a.first_stride + a.first_offset : nullptr;
  const bf16_t* values = row + (size_t)(a.heads + a.kv_heads) * a.dim;
  const int v_per_head = D / 8, v_real = a.vdim / 8;
  for (int i = threadIdx.x; i < a.kv_heads * v_per_head; i += 256) {
    const int g = i / v_per_head, p = i % v_per_head;
    qk_bf16x8_t v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
    if (p < v_real) {
      v = *reinterpret_cast<const qk_bf16x8_t*>(values + g * a.vdim + 8 * p);
      if (first) {
        const qk_bf16x8_t f = *reinterpret_cast<const qk_bf16x8_t*>(first + g * a.vdim + 8 * p);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (bf16_t)((1.f - lam) * (float)v[j] + lam * (float)f[j]);
      }
    }
    bf16_t* dst = (bf16_t*)a.v_cache + (((size_t)page * a.kv_heads + g) * D + 8 * p) * page_size + offset;
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[(size_t)j * page_size] = v[j];
  }
}

extern "C" int velox_qk_norm_write(const void* qkv, int qkv_stride, void* q_out, const float* q_weight, const float* k_weight, const int* positions,
                                   const void* first, int first_stride, int first_offset, const float* lambda, const int* slot_mapping, void* k_cache,
                                   void* v_cache, int tokens, int heads, int kv_heads, int dim, int vdim, int D, int page_shift, int whole, int write_kv,
                                   float eps, float temp_coef, int temp_every, int dtype, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || dim < 1 || vdim < 1 || D < dim || D < vdim || page_shift < 0 || (first != nullptr && lambda == nullptr)) return -1;
  QkNormArgs a;
  a.qkv = qkv; a.qkv_stride = qkv_stride; a.q_out = q_out; a.q_weight = q_weight; a.k_weight = k_weight; a.positions = positions;
  a.first = first; a.first_stride = first_stride; a.first_offset = first_offset; a.lambda = lambda; a.slot_mapping = slot_mapping;
  a.k_cache = k_cache; a.v_cache = v_cache; a.heads = heads; a.kv_heads = kv_heads; a.dim = dim; a.vdim = vdim; a.D = D;
  a.page_shift = page_shift; a.whole = whole; a.write_kv = write_kv; a.temp_every = temp_every; a.eps = eps; a.temp_coef = temp_coef;
  const int q_units = heads * dim / 8, k_units = kv_heads * dim / 8;
  const bool pieces = dim % 8 == 0 && vdim % 8 == 0 && D % 8 == 0 && qkv_stride % 8 == 0 && first_stride % 8 == 0 && first_offset % 8 == 0 &&
                      q_units + k_units <= 256 * QK_MAX_UNITS &&
                      (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)first) & 15) == 0;
  if (dtype == VELOX_BF16 && pieces) {
    const size_t shared = (size_t)(q_units + k_units + heads + kv_heads) * sizeof(float);
    qk_norm_write_vec_kernel<<<tokens, 256, shared, stream>>>(a);
  } else if (dtype == VELOX_BF16) qk_norm_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>(a);
  else qk_norm_write_kernel<float><<<tokens, 256, 0, stream>>>(a);
  VELOX_RETURN_LAUNCH_STATUS();
}
