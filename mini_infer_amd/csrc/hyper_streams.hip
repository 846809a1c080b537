// A residual stream kept as several copies that sublayers read from and write to through
// small learned vectors and a matrix ("hyper-connections").
//
//   streams            float32 [tokens, S, hidden]: the S copies of a token lie side by side.
//   embed_norm_streams x = table[id];  every copy = x / sqrt(mean(x^2) + eps) * weight.
//   streams_update_norm
//       the write of a finished sublayer and the read of the next one in one launch:
//         y      = scale_a * a + scale_b * b                       (either may be absent)
//         x_t   <- sum_s mix[s][t] * x_s + out[t] * y              (all copies at once, from the old ones)
//         u      = sum_t read[t] * x_t                             (read absent: the plain sum)
//         result = u / sqrt(mean(u^2) + eps) * weight              (in the element type)
//       Without mix/out nothing is written (the first sublayer of a model); without a weight
//       nothing is read.  With a row list only those rows are handled, their new copies are
//       not stored (the final norm, at the rows whose logits are asked for).
//
// All of it is float32 arithmetic on float32 copies; in the 32-bit engine sums are carried in
// 64-bit and rounded once.  `weight` is float32 and holds the factor itself (a weight stored
// around zero has had its one added by the caller).
#include "common.h"

#include <math.h>

#define HYPER_MAX_STREAMS 8

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
__device__ __forceinline__ A block_sum_wide(A v, A* scratch) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  A total = 0;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

template <typename T>
__global__ __launch_bounds__(1024) void embed_norm_streams_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                                                 const float* __restrict__ weight, float* __restrict__ streams,
                                                                 int hidden, int vocab, int n_streams, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (int64_t)id * hidden;
  A ss = 0;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const A x = (A)to_f32(row[c]);
    ss += x * x;
  }
  ss = block_sum_wide<A>(ss, scratch);
  A r;
  if constexpr (sizeof(T) == 4) r = 1.0 / sqrt(ss / (double)hidden + (double)eps);
  else r = 1.0f / sqrtf(ss / (float)hidden + eps);
  float* dst = streams + (int64_t)t * n_streams * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float v = (float)((A)to_f32(row[c]) * r * (A)weight[c]);
    for (int s = 0; s < n_streams; ++s) dst[(int64_t)s * hidden + c] = v;
  }
}

// S copies (a template argument: the small matrix lives in registers and its loops unroll), V
// columns a thread at once.  A block takes a row; its threads are as many as the row has groups
// of V columns, up to 1,024, so a step of few rows is a few loads deep.
template <typename T, int S, int V>
__global__ __launch_bounds__(1024) void streams_update_norm_kernel(
    const T* __restrict__ ya, int64_t a_stride, const T* __restrict__ yb, int64_t b_stride, float scale_a, float scale_b,
    const float* __restrict__ mix, const float* __restrict__ outv, const float* __restrict__ readv,
    const float* __restrict__ weight, float* __restrict__ streams, T* __restrict__ out, const int* __restrict__ rows,
    int hidden, float eps) {
  using A = typename Wide<T>::type;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  float* u_lds = reinterpret_cast<float*>(lds_bytes);  // [hidden]: what the norm reads
  __shared__ A scratch[16];
  const bool writes = mix != nullptr;
  float m[S][S], ov[S], rv[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    ov[s] = writes ? outv[s] : 0.f;
    rv[s] = readv ? readv[s] : 1.f;
#pragma unroll
    for (int to = 0; to < S; ++to) m[s][to] = writes ? mix[s * S + to] : 0.f;
  }
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = streams + (int64_t)t * S * hidden;
  const bool store = writes && rows == nullptr;
  A ss = 0;
  for (int c = threadIdx.x * V; c < hidden; c += blockDim.x * V) {
    float old[S][V];
#pragma unroll
    for (int s = 0; s < S; ++s) mi_load_cols<float, V>(x + (int64_t)s * hidden + c, old[s]);
    float uf[V];
    if (writes) {
      float a[V], b[V];
#pragma unroll
      for (int j = 0; j < V; ++j) a[j] = b[j] = 0.f;
      if (ya) mi_load_cols<T, V>(ya + (int64_t)t * a_stride + c, a);
      if (yb) mi_load_cols<T, V>(yb + (int64_t)t * b_stride + c, b);
      A u[V];
#pragma unroll
      for (int j = 0; j < V; ++j) u[j] = 0;
#pragma unroll
      for (int to = 0; to < S; ++to) {
        float now[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
          A y = 0;
          if (ya) y = (A)scale_a * (A)a[j];
          if (yb) y += (A)scale_b * (A)b[j];
          A v = (A)ov[to] * y;
#pragma unroll
          for (int s = 0; s < S; ++s) v += (A)m[s][to] * (A)old[s][j];
          now[j] = (float)v;
          u[j] += (A)rv[to] * (A)now[j];
        }
        if (store) mi_store_cols<float, V>(x + (int64_t)to * hidden + c, now);
      }
#pragma unroll
      for (int j = 0; j < V; ++j) uf[j] = (float)u[j];
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        A u = 0;
#pragma unroll
        for (int s = 0; s < S; ++s) u += (A)rv[s] * (A)old[s][j];
        uf[j] = (float)u;
      }
    }
    mi_store_cols<float, V>(u_lds + c, uf);
#pragma unroll
    for (int j = 0; j < V; ++j) ss += (A)uf[j] * (A)uf[j];
  }
  if (weight == nullptr) return;
  ss = block_sum_wide<A>(ss, scratch);
  A r;
  if constexpr (sizeof(T) == 4) r = 1.0 / sqrt(ss / (double)hidden + (double)eps);
  else r = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* o = out + (int64_t)blockIdx.x * hidden;
  for (int c = threadIdx.x * V; c < hidden; c += blockDim.x * V) {
    float uf[V], w[V], res[V];
    mi_load_cols<float, V>(u_lds + c, uf);
    mi_load_cols<float, V>(weight + c, w);
#pragma unroll
    for (int j = 0; j < V; ++j) res[j] = (float)((A)uf[j] * r * (A)w[j]);
    mi_store_cols<T, V>(o + c, res);
  }
}

template <typename T, int S>
void launch_streams(const void* ya, int64_t a_stride, const void* yb, int64_t b_stride, float scale_a, float scale_b,
                    const float* mix, const float* outv, const float* readv, const float* weight, float* streams, void* out,
                    const int* rows, int n_out, int hidden, float eps, hipStream_t stream) {
  const size_t lds = (size_t)hidden * sizeof(float);
  auto aligned = [](const void* p, size_t to) { return ((uintptr_t)p % to) == 0; };
  const bool wide = hidden % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0 && aligned(ya, 4 * sizeof(T)) &&
                    aligned(yb, 4 * sizeof(T)) && aligned(out, 4 * sizeof(T)) && aligned(streams, 16) && aligned(weight, 16);
  if (wide) {
    const int threads = min(1024, ceil_div(hidden / 4, MI_WAVE) * MI_WAVE);
    streams_update_norm_kernel<T, S, 4><<<n_out, threads, lds, stream>>>((const T*)ya, a_stride, (const T*)yb, b_stride, scale_a,
                                                                         scale_b, mix, outv, readv, weight, streams, (T*)out, rows,
                                                                         hidden, eps);
  } else {
    const int threads = min(1024, ceil_div(hidden, MI_WAVE) * MI_WAVE);
    streams_update_norm_kernel<T, S, 1><<<n_out, threads, lds, stream>>>((const T*)ya, a_stride, (const T*)yb, b_stride, scale_a,
                                                                         scale_b, mix, outv, readv, weight, streams, (T*)out, rows,
                                                                         hidden, eps);
  }
}

template <typename T>
void launch_streams_of(int n_streams, const void* ya, int64_t a_stride, const void* yb, int64_t b_stride, float scale_a,
                       float scale_b, const float* mix, const float* outv, const float* readv, const float* weight,
                       float* streams, void* out, const int* rows, int n_out, int hidden, float eps, hipStream_t stream) {
#define MI_STREAMS(N)                                                                                                         \
  case N:                                                                                                                     \
    launch_streams<T, N>(ya, a_stride, yb, b_stride, scale_a, scale_b, mix, outv, readv, weight, streams, out, rows, n_out,  \
                         hidden, eps, stream);                                                                                \
    break
  switch (n_streams) {
    MI_STREAMS(1);
    MI_STREAMS(2);
    MI_STREAMS(3);
    MI_STREAMS(4);
    MI_STREAMS(5);
    MI_STREAMS(6);
    MI_STREAMS(7);
    MI_STREAMS(8);
  }
#undef MI_STREAMS
}

}  // namespace

extern "C" int mi_embed_norm_streams(int dtype, const void* table, const int* ids, const float* weight, float* streams,
                                     int num_tokens, int hidden, int vocab, int n_streams, float eps, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0, "embed_norm_streams: bad sizes tokens=%d hidden=%d vocab=%d", num_tokens,
             hidden, vocab);
  MI_REQUIRE(n_streams >= 1 && n_streams <= HYPER_MAX_STREAMS, "embed_norm_streams: streams=%d must be 1..%d", n_streams,
             HYPER_MAX_STREAMS);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "embed_norm_streams: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int threads = min(1024, ceil_div(hidden, MI_WAVE) * MI_WAVE);
  if (dtype == MI_F32)
    embed_norm_streams_kernel<float><<<num_tokens, threads, 0, stream>>>((const float*)table, ids, weight, streams, hidden, vocab,
                                                                     n_streams, eps);
  else
    embed_norm_streams_kernel<bf16_t><<<num_tokens, threads, 0, stream>>>((const bf16_t*)table, ids, weight, streams, hidden, vocab,
                                                                      n_streams, eps);
  MI_CHECK_LAUNCH("embed_norm_streams");
  return MI_OK;
}

// ya, yb: [tokens, hidden] in the element type (row strides; either may be null); mix float32 [S][S]
// indexed [from][to], outv [S] (both null: nothing is written); readv [S] or null (the plain sum);
// weight float32 [hidden] or null (nothing is read); out [n_out, hidden]; rows int32 [n_out] or null.
extern "C" int mi_streams_update_norm(int dtype, const void* ya, int64_t a_stride, const void* yb, int64_t b_stride,
                                      float scale_a, float scale_b, const float* mix, const float* outv, const float* readv,
                                      const float* weight, float* streams, void* out, const int* rows, int n_out, int hidden,
                                      int n_streams, float eps, hipStream_t stream) {
  MI_REQUIRE(n_out >= 0 && hidden > 0, "streams_update_norm: bad sizes rows=%d hidden=%d", n_out, hidden);
  MI_REQUIRE(n_streams >= 1 && n_streams <= HYPER_MAX_STREAMS, "streams_update_norm: streams=%d must be 1..%d", n_streams,
             HYPER_MAX_STREAMS);
  MI_REQUIRE((mix == nullptr) == (outv == nullptr), "streams_update_norm: a write needs both its matrix and its vector");
  MI_REQUIRE(mix != nullptr || (ya == nullptr && yb == nullptr), "streams_update_norm: a sublayer's output without a write");
  MI_REQUIRE(weight == nullptr || out != nullptr, "streams_update_norm: a norm needs somewhere to put its rows");
  MI_REQUIRE(weight != nullptr || rows == nullptr, "streams_update_norm: a row list only goes with a norm");
  MI_REQUIRE((int64_t)hidden * 4 <= 60 * 1024, "streams_update_norm: hidden=%d does not fit the block's scratch", hidden);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "streams_update_norm: unknown dtype %d", dtype);
  if (n_out == 0) return MI_OK;
  if (dtype == MI_F32)
    launch_streams_of<float>(n_streams, ya, a_stride, yb, b_stride, scale_a, scale_b, mix, outv, readv, weight, streams, out, rows,
                             n_out, hidden, eps, stream);
  else
    launch_streams_of<bf16_t>(n_streams, ya, a_stride, yb, b_stride, scale_a, scale_b, mix, outv, readv, weight, streams, out,
                              rows, n_out, hidden, eps, stream);
  MI_CHECK_LAUNCH("streams_update_norm");
  return MI_OK;
}
