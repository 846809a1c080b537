// What stands between an attention layer's stacked projection and its attention when queries
// and keys are normed head by head, and the gates that multiply a sublayer's inner rows.
//
//   head_norm_rope_kv_write
//       per token: every query head and key head divided by its own root mean square over the
//       head (times a weight shared by the heads; no weight: no norm), then the rotation of the
//       first rotary_dim dims (dim j with j + rotary_dim/2, or 2j with 2j+1), queries in place,
//       keys and values into their page slots.  Statistics and rotation are float32 (statistics
//       64-bit in the 32-bit engine).  A wave takes a head.
//   gated_mul
//       out[t, i] = act(a[t, i]) * b[t, i] for act = silu, the tanh form of gelu, or the logistic
//       function; a and b are column ranges of rows that may be strided.
#include "common.h"

#include <math.h>

namespace {

template <typename T>
struct Wide {
  using type = float;
};
template <>
struct Wide<float> {
  using type = double;
};

template <typename A>
__device__ __forceinline__ A wave_sum_wide(A v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, float eps, int q_heads, int kv_heads, int head_dim, int rotary_dim, int interleaved,
    int page_size, int v_transposed, int v_dim) {
  using A = typename Wide<T>::type;
  const int t = blockIdx.x;
  const int lane = threadIdx.x % MI_WAVE;
  const int wave = blockIdx.y * (blockDim.x / MI_WAVE) + threadIdx.x / MI_WAVE;
  const int waves = gridDim.y * (blockDim.x / MI_WAVE);
  const int half = rotary_dim / 2;
  T* row = qkv + (int64_t)t * row_stride;
  const float* c = cos_t + (int64_t)t * half;
  const float* s = sin_t + (int64_t)t * half;
  const bool writes = kv_heads > 0 && slot_mapping != nullptr;
  const int slot = writes ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

  for (int item = wave; item < q_heads + kv_heads; item += waves) {
    const bool is_key = item >= q_heads;
    if (is_key && slot < 0) continue;
    const int h = is_key ? item - q_heads : item;
    const T* src = row + (int64_t)item * head_dim;  // (key heads follow the query heads, all head_dim wide)
    T* dst = is_key ? k_pages + (((int64_t)page * kv_heads + h) * page_size + off) * head_dim : row + (int64_t)h * head_dim;
    const float* w = is_key ? k_weight : q_weight;
    A factor = 1;
    if (w != nullptr) {
      A ss = 0;
      for (int d = lane; d < head_dim; d += MI_WAVE) {
        const A x = (A)to_f32(src[d]);
        ss += x * x;
      }
      ss = wave_sum_wide<A>(ss);
      if constexpr (sizeof(A) == 8) factor = 1.0 / sqrt(ss / (double)head_dim + (double)eps);
      else factor = 1.0f / sqrtf(ss / (float)head_dim + eps);
    }
    auto normed = [&](int d) -> float { return (float)((A)to_f32(src[d]) * factor * (A)(w ? w[d] : 1.f)); };
    for (int j = lane; j < half; j += MI_WAVE) {
      const int i0 = interleaved ? 2 * j : j;
      const int i1 = interleaved ? 2 * j + 1 : j + half;
      const float x0 = normed(i0), x1 = normed(i1);
      dst[i0] = from_f32<T>(x0 * c[j] - x1 * s[j]);
      dst[i1] = from_f32<T>(x1 * c[j] + x0 * s[j]);
    }
    for (int d = rotary_dim + lane; d < head_dim; d += MI_WAVE) dst[d] = from_f32<T>(normed(d));
  }
  if (slot < 0) return;
  const T* v_row = row + (int64_t)(q_heads + kv_heads) * head_dim;
  for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < kv_heads * v_dim; e += gridDim.y * blockDim.x) {
    const int h = e / v_dim, d = e % v_dim;
    const int64_t chunk = ((int64_t)page * kv_heads + h) * page_size * v_dim;
    const int64_t at = v_transposed ? chunk + (int64_t)d * page_size + off : chunk + (int64_t)off * v_dim + d;
    v_pages[at] = v_row[e];
  }
}

enum { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_LOGISTIC = 2 };

template <typename T>
__device__ __forceinline__ float act_times(int act, float a, float b) {
  if constexpr (sizeof(T) == 4) {
    const double z = (double)a;
    double f;
    if (act == ACT_SILU) f = z / (1.0 + exp(-z));
    else if (act == ACT_GELU_TANH) f = 0.5 * z * (1.0 + tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)));
    else f = 1.0 / (1.0 + exp(-z));
    return (float)(f * (double)b);
  } else {
    float f;
    if (act == ACT_SILU) f = a / (1.f + expf(-a));
    else if (act == ACT_GELU_TANH) f = 0.5f * a * (1.f + tanhf(0.7978845608028654f * (a + 0.044715f * a * a * a)));
    else f = 1.f / (1.f + expf(-a));
    return f * b;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_mul_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b,
                                                        int64_t b_stride, T* __restrict__ out, int64_t out_stride, int width,
                                                        int act) {
  const int t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  out[(int64_t)t * out_stride + i] =
      from_f32<T>(act_times<T>(act, to_f32(a[(int64_t)t * a_stride + i]), to_f32(b[(int64_t)t * b_stride + i])));
}

// four columns a thread: 8- or 16-byte loads and stores
template <typename T>
__global__ __launch_bounds__(256) void gated_mul_vec4_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b,
                                                             int64_t b_stride, T* __restrict__ out, int64_t out_stride,
                                                             int width, int act) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (i >= width) return;
  struct alignas(4 * sizeof(T)) Four {
    T v[4];
  };
  const Four av = *reinterpret_cast<const Four*>(a + (int64_t)t * a_stride + i);
  const Four bv = *reinterpret_cast<const Four*>(b + (int64_t)t * b_stride + i);
  Four ov;
#pragma unroll
  for (int k = 0; k < 4; ++k) ov.v[k] = from_f32<T>(act_times<T>(act, to_f32(av.v[k]), to_f32(bv.v[k])));
  *reinterpret_cast<Four*>(out + (int64_t)t * out_stride + i) = ov;
}

}  // namespace

// qkv rows: [q heads | k heads | v heads], q and k heads head_dim wide, v heads v_head_dim wide.
// q_weight, k_weight: float32 [head_dim] or null (that side is not normed).
extern "C" int mi_head_norm_rope_kv_write(int dtype, void* qkv, int64_t row_stride, const float* cos_t, const float* sin_t,
                                          const int* slot_mapping, void* k_pages, void* v_pages, const float* q_weight,
                                          const float* k_weight, float eps, int num_tokens, int q_heads, int kv_heads,
                                          int head_dim, int rotary_dim, int interleaved, int page_size, int num_pages,
                                          int v_transposed, int v_head_dim, hipStream_t stream) {
  if (v_head_dim <= 0) v_head_dim = head_dim;
  MI_REQUIRE(num_tokens >= 0 && q_heads >= 0 && kv_heads >= 0 && head_dim > 0,
             "head_norm_rope_kv_write: bad sizes tokens=%d q_heads=%d kv_heads=%d head_dim=%d", num_tokens, q_heads, kv_heads,
             head_dim);
  MI_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "head_norm_rope_kv_write: rotary_dim=%d must be even and at most head_dim=%d", rotary_dim, head_dim);
  MI_REQUIRE(row_stride >= (int64_t)(q_heads + kv_heads) * head_dim + (int64_t)kv_heads * v_head_dim,
             "head_norm_rope_kv_write: row stride %lld is shorter than the q, k and v heads", (long long)row_stride);
  MI_REQUIRE(kv_heads == 0 || slot_mapping == nullptr || (page_size > 0 && num_pages > 0 && k_pages && v_pages),
             "head_norm_rope_kv_write: pages are needed to write keys and values");
  MI_REQUIRE(rotary_dim == 0 || (cos_t && sin_t), "head_norm_rope_kv_write: a rotation needs its tables");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "head_norm_rope_kv_write: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int items = q_heads + kv_heads;
  const int blocks_y = min((num_tokens >= 512) ? 2 : 16, max(1, ceil_div(items, 4)));
  dim3 grid(num_tokens, blocks_y);
  if (dtype == MI_F32)
    head_norm_rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, row_stride, cos_t, sin_t, slot_mapping,
                                                                    (float*)k_pages, (float*)v_pages, q_weight, k_weight, eps,
                                                                    q_heads, kv_heads, head_dim, rotary_dim, interleaved,
                                                                    page_size, v_transposed, v_head_dim);
  else
    head_norm_rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)qkv, row_stride, cos_t, sin_t, slot_mapping,
                                                                     (bf16_t*)k_pages, (bf16_t*)v_pages, q_weight, k_weight,
                                                                     eps, q_heads, kv_heads, head_dim, rotary_dim, interleaved,
                                                                     page_size, v_transposed, v_head_dim);
  MI_CHECK_LAUNCH("head_norm_rope_kv_write");
  return MI_OK;
}

// act: 0 silu, 1 gelu (tanh form), 2 logistic.  a, b, out: [tokens, width] column ranges (row strides).
extern "C" int mi_gated_mul(int dtype, int act, const void* a, int64_t a_stride, const void* b, int64_t b_stride, void* out,
                            int64_t out_stride, int num_tokens, int width, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0, "gated_mul: bad sizes tokens=%d width=%d", num_tokens, width);
  MI_REQUIRE(act >= 0 && act <= 2, "gated_mul: activation %d (0 silu, 1 gelu_tanh, 2 logistic)", act);
  MI_REQUIRE(a_stride >= width && b_stride >= width && out_stride >= width, "gated_mul: row strides shorter than a row");
  MI_REQUIRE(ceil_div(width, 256) <= 65535, "gated_mul: width %d is too large", width);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "gated_mul: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const size_t elem = dtype == MI_F32 ? 4 : 2;
  const bool vec = width % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0 && out_stride % 4 == 0 &&
                   ((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) % (4 * elem) == 0;
  dim3 grid(num_tokens, ceil_div(width, vec ? 1024 : 256));
  if (dtype == MI_F32) {
    if (vec) gated_mul_vec4_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, a_stride, (const float*)b, b_stride, (float*)out, out_stride, width, act);
    else gated_mul_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, a_stride, (const float*)b, b_stride, (float*)out, out_stride, width, act);
  } else {
    if (vec) gated_mul_vec4_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)b, b_stride, (bf16_t*)out, out_stride, width, act);
    else gated_mul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)b, b_stride, (bf16_t*)out, out_stride, width, act);
  }
  MI_CHECK_LAUNCH("gated_mul");
  return MI_OK;
}
