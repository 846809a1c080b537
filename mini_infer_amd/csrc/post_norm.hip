// Row kernels of a stack whose norms stand BEHIND the residual sum (post-norm), and of an
// embedding with a second table indexed by a hash of a token and the token before it.
//
//   embed_pair_hash   stream[t] = table[id_t] + pairs[row_t],
//                     row_t = (prev_t * mul_prev + id_t * mul_cur) mod buckets, and `buckets` (the
//                     table's last row) for a sequence's first token.  The token before a step's
//                     first one is read from the request's state row, and the step's last token
//                     is left there.
//   scale_add_norm    x[t] <- rms_norm(alpha * x[t] + scale[c] * y[t, c]) * factor[c]  in place on the
//                     float32 stream, with the new row's copy in the element type for the products
//                     that read it next; without y and for a list of rows: the norm alone (how
//                     such a stack ends).
//   norm_rows         out[t] = rms_norm(in[t, 0..width)) * weight: a norm inside a mixer, on the
//                     first columns of a wider row.
//
// Sums and statistics are float32 for bfloat16 rows and 64-bit for float32 rows (rounded once).
#include "common.h"

#include <math.h>

namespace {

template <typename T>
struct WideOf {
  using type = float;
};
template <>
struct WideOf<float> {
  using type = double;
};

__device__ __forceinline__ float lane_add(float v, int off) { return v + __shfl_xor(v, off, MI_WAVE); }
__device__ __forceinline__ double lane_add(double v, int off) { return v + __shfl_xor(v, off, MI_WAVE); }

// sum over a block in a fixed order: lanes by butterfly, waves one after another
template <typename A>
__device__ __forceinline__ A block_add(A v, A* scratch) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v = lane_add(v, off);
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  A total = 0;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float inv_root_of(float mean_sq, float eps) { return 1.0f / sqrtf(mean_sq + eps); }
__device__ __forceinline__ double inv_root_of(double mean_sq, double eps) { return 1.0 / sqrt(mean_sq + eps); }

inline bool is_aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }
inline int threads_for(int rows, int items) { return (rows < 256 && items > 1024) ? 1024 : 256; }

// ---------------------------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(256) void embed_pair_hash_kernel(
    const T* __restrict__ table, const T* __restrict__ pairs, const int* __restrict__ ids,
    const int* __restrict__ positions, const int* __restrict__ token_request, const int* __restrict__ cu_seqlens,
    const int* __restrict__ state_slots, int* __restrict__ last_token, int64_t last_stride, int num_slots,
    float* __restrict__ out, T* __restrict__ cast, int hidden, int vocab, int buckets, int mul_prev, int mul_cur) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const int req = token_request[t];
  const int first = cu_seqlens[req];
  int prev = 0;
  if (t > first) {
    prev = ids[t - 1];
  } else {
    // the step's first token of its request: the token before it is what the last step left,
    // and what this step will leave is written by this same block (read first, then written)
    int slot = state_slots[req];
    if (slot < 0 || slot >= num_slots) slot = num_slots;  // nobody's row
    int* kept = last_token + (int64_t)slot * last_stride;
    prev = kept[0];
    __syncthreads();
    const int last = cu_seqlens[req + 1] - 1;
    if (threadIdx.x == 0 && last >= first) kept[0] = ids[last];
  }
  int64_t row = buckets;
  if (positions[t] > 0) row = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
  if (row < 0) row += buckets;
  const bool known = id >= 0 && id < vocab;
  const T* a = table + (int64_t)(known ? id : 0) * hidden;
  const T* b = pairs + row * hidden;
  float* o = out + (int64_t)t * hidden;
  for (int c = threadIdx.x * VEC; c < hidden; c += blockDim.x * VEC) {
    float x[VEC], y[VEC];
    mi_load_cols<T, VEC>(a + c, x);
    mi_load_cols<T, VEC>(b + c, y);
#pragma unroll
    for (int j = 0; j < VEC; ++j) x[j] = known ? x[j] + y[j] : 0.f;
    mi_store_cols<float, VEC>(o + c, x);
    if (cast != nullptr) mi_store_cols<T, VEC>(cast + (int64_t)t * hidden + c, x);
  }
}

// ---------------------------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(1024) void scale_add_norm_kernel(
    float* __restrict__ stream, const T* __restrict__ y, int64_t y_stride, const float* __restrict__ scale,
    const float* __restrict__ factor, const int* __restrict__ rows, T* __restrict__ cast, int hidden, float alpha,
    float eps) {
  using A = typename WideOf<T>::type;
  __shared__ A scratch[16];
  const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  float* x = stream + (int64_t)t * hidden;
  const T* add = y != nullptr ? y + (int64_t)t * y_stride : nullptr;
  // a row is at most a few thousand columns: the sums of a thread's columns stay in registers
  // between the two passes where they fit (4 turns), and are made again where they do not
  constexpr int KEPT = 4;
  A kept[KEPT][VEC];
  A squares = 0;
  int turn = 0;
  for (int c = threadIdx.x * VEC; c < hidden; c += blockDim.x * VEC, ++turn) {
    float v[VEC], u[VEC], s[VEC];
    mi_load_cols<float, VEC>(x + c, v);
    if (add != nullptr) {
      mi_load_cols<T, VEC>(add + c, u);
      if (scale != nullptr) mi_load_cols<float, VEC>(scale + c, s);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      A sum = (A)v[j];
      if (add != nullptr) sum = (A)alpha * (A)v[j] + (scale != nullptr ? (A)s[j] * (A)u[j] : (A)u[j]);
      if (turn < KEPT) kept[turn][j] = sum;
      squares += sum * sum;
    }
  }
  const A inv = inv_root_of(block_add<A>(squares, scratch) / (A)hidden, (A)eps);
  T* narrow = cast != nullptr ? cast + (int64_t)blockIdx.x * hidden : nullptr;
  turn = 0;
  for (int c = threadIdx.x * VEC; c < hidden; c += blockDim.x * VEC, ++turn) {
    float f[VEC], r[VEC];
    mi_load_cols<float, VEC>(factor + c, f);
    if (turn < KEPT) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) r[j] = (float)((kept[turn][j] * inv) * (A)f[j]);
    } else {
      float v[VEC], u[VEC], s[VEC];
      mi_load_cols<float, VEC>(x + c, v);
      if (add != nullptr) {
        mi_load_cols<T, VEC>(add + c, u);
        if (scale != nullptr) mi_load_cols<float, VEC>(scale + c, s);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        A sum = (A)v[j];
        if (add != nullptr) sum = (A)alpha * (A)v[j] + (scale != nullptr ? (A)s[j] * (A)u[j] : (A)u[j]);
        r[j] = (float)((sum * inv) * (A)f[j]);
      }
    }
    if (rows == nullptr) mi_store_cols<float, VEC>(x + c, r);
    if (narrow != nullptr) mi_store_cols<T, VEC>(narrow + c, r);
  }
}

// ---------------------------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void norm_rows_kernel(const T* __restrict__ in, int64_t in_stride,
                                                        const float* __restrict__ weight, T* __restrict__ out,
                                                        int64_t out_stride, int width, float eps) {
  using A = typename WideOf<T>::type;
  __shared__ A scratch[16];
  const T* x = in + (int64_t)blockIdx.x * in_stride;
  A squares = 0;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const A v = (A)to_f32(x[c]);
    squares += v * v;
  }
  const A inv = inv_root_of(block_add<A>(squares, scratch) / (A)width, (A)eps);
  T* o = out + (int64_t)blockIdx.x * out_stride;
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    o[c] = from_f32<T>((float)(((A)to_f32(x[c]) * inv) * (A)weight[c]));
}

}  // namespace

extern "C" int mi_embed_pair_hash(int dtype, const void* table, const void* pairs, const int* ids, const int* positions,
                                  const int* token_request, const int* cu_seqlens, const int* state_slots,
                                  int* last_token, int64_t last_stride, int num_slots, float* out, void* cast,
                                  int num_tokens, int hidden, int vocab, int buckets, int mul_prev, int mul_cur,
                                  hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0 && buckets > 0, "embed_pair_hash: bad sizes tokens=%d hidden=%d vocab=%d buckets=%d",
             num_tokens, hidden, vocab, buckets);
  MI_REQUIRE(last_token != nullptr && last_stride > 0 && num_slots > 0, "embed_pair_hash: the requests' state rows are missing");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "embed_pair_hash: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const bool vec = hidden % 4 == 0 && is_aligned16(table) && is_aligned16(pairs) && is_aligned16(out) && is_aligned16(cast);
#define MI_PAIR(T, VEC)                                                                                              \
  embed_pair_hash_kernel<T, VEC><<<num_tokens, 256, 0, stream>>>((const T*)table, (const T*)pairs, ids, positions,   \
                                                                 token_request, cu_seqlens, state_slots, last_token, \
                                                                 last_stride, num_slots, out, (T*)cast, hidden,      \
                                                                 vocab, buckets, mul_prev, mul_cur)
  if (dtype == MI_F32) {
    if (vec) MI_PAIR(float, 4);
    else MI_PAIR(float, 1);
  } else {
    if (vec) MI_PAIR(bf16_t, 4);
    else MI_PAIR(bf16_t, 1);
  }
#undef MI_PAIR
  MI_CHECK_LAUNCH("embed_pair_hash");
  return MI_OK;
}

// `y` (and `scale`) may be null: the norm alone.  `rows` (may be null) lists the rows to norm: the
// stream is then left as it is and `cast` [num_rows, hidden] gets the normed rows in list order.
extern "C" int mi_scale_add_norm(int dtype, float* stream_rows, const void* y, int64_t y_stride, const float* scale,
                                 const float* factor, const int* rows, void* cast, int num_rows, int hidden,
                                 float alpha, float eps, hipStream_t stream) {
  MI_REQUIRE(num_rows >= 0 && hidden > 0 && (y == nullptr || y_stride >= hidden), "scale_add_norm: bad sizes rows=%d hidden=%d stride=%lld",
             num_rows, hidden, (long long)y_stride);
  MI_REQUIRE(factor != nullptr && stream_rows != nullptr, "scale_add_norm: the stream and the norm's factors are needed");
  MI_REQUIRE(rows == nullptr || cast != nullptr, "scale_add_norm: rows picked from the stream need a place to go");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "scale_add_norm: unknown dtype %d", dtype);
  if (num_rows == 0) return MI_OK;
  const bool vec = hidden % 4 == 0 && y_stride % 4 == 0 && is_aligned16(stream_rows) && is_aligned16(y) && is_aligned16(scale) &&
                   is_aligned16(factor) && is_aligned16(cast);
  const int threads = threads_for(num_rows, vec ? hidden / 4 : hidden);
#define MI_POST(T, VEC)                                                                                            \
  scale_add_norm_kernel<T, VEC><<<num_rows, threads, 0, stream>>>(stream_rows, (const T*)y, y_stride, scale, factor, \
                                                                  rows, (T*)cast, hidden, alpha, eps)
  if (dtype == MI_F32) {
    if (vec) MI_POST(float, 4);
    else MI_POST(float, 1);
  } else {
    if (vec) MI_POST(bf16_t, 4);
    else MI_POST(bf16_t, 1);
  }
#undef MI_POST
  MI_CHECK_LAUNCH("scale_add_norm");
  return MI_OK;
}

extern "C" int mi_norm_rows(int dtype, const void* in, int64_t in_stride, const float* weight, void* out,
                            int64_t out_stride, int num_rows, int width, float eps, hipStream_t stream) {
  MI_REQUIRE(num_rows >= 0 && width > 0 && in_stride >= width && out_stride >= width, "norm_rows: bad sizes rows=%d width=%d", num_rows, width);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "norm_rows: unknown dtype %d", dtype);
  if (num_rows == 0) return MI_OK;
  if (dtype == MI_F32)
    norm_rows_kernel<float><<<num_rows, 256, 0, stream>>>((const float*)in, in_stride, weight, (float*)out, out_stride, width, eps);
  else
    norm_rows_kernel<bf16_t><<<num_rows, 256, 0, stream>>>((const bf16_t*)in, in_stride, weight, (bf16_t*)out, out_stride, width, eps);
  MI_CHECK_LAUNCH("norm_rows");
  return MI_OK;
}
