// A feed-forward of routed experts: every token goes through `top` of the experts, chosen by a
// router, and the results are added with the router's weights.
//
//   route_top_k         per token: logits z = R x (R float32, sums float32; 64-bit in the 32-bit
//                       engine), scores s = softmax(z) over all router outputs, choice = s +
//                       correction, the `top` largest choices (the lower index wins a tie); leaves
//                       the chosen indices and their weights s * route_scale (not renormalized),
//                       and, where a gate row is given, logistic(gate . x) for a shared expert.
//   expert_gate_up      few rows: for every (token, chosen expert) pair the expert's stacked
//                       gate|up product and silu(gate) * up, the weights read by expert index.
//   expert_down_combine few rows: y[t] = sum_k w[t, k] * (W_down[e_k] act[t, k])  (+ shared_gate[t] *
//                       shared[t]); a chosen index past the real experts is an identity expert,
//                       whose output is the token's input row itself.
//   expert_combine      many rows: the same sum over rows of expert outputs that were made expert
//                       by expert (sorted by expert; `where` maps a pair to its sorted row).
//
// Expert weights are stacked: gate|up [experts, 2 * ff, width] (an expert's gate rows, then its up
// rows), down [experts, width, ff].
#include "common.h"

#include <math.h>

namespace {

template <typename T>
struct SumOf {
  using type = float;
};
template <>
struct SumOf<float> {
  using type = double;
};

__device__ __forceinline__ float lanes_total(float v) { return wave_sum(v); }
__device__ __forceinline__ double lanes_total(double v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

__device__ __forceinline__ float exp_of(float z) { return expf(z); }
__device__ __forceinline__ double exp_of(double z) { return exp(z); }

#define MI_ROUTER_MAX_OUTPUTS 1024

// R tokens a block: their rows wait in LDS while every wave walks router rows (16 bytes a lane, each
// router row read once for all R tokens), then thread r ranks token r's outputs.
template <typename T, int R>
__global__ __launch_bounds__(1024) void route_top_k_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ router, const float* __restrict__ correction,
    const float* __restrict__ gate_row, int* __restrict__ chosen, float* __restrict__ weights,
    float* __restrict__ shared_gate, int num_tokens, int width, int outputs, int top, float route_scale) {
  using A = typename SumOf<T>::type;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  A* z = reinterpret_cast<A*>(lds_bytes);                         // [R][outputs + 1]
  T* rows = reinterpret_cast<T*>(z + (size_t)R * (outputs + 1));  // [R][width]
  const int t0 = blockIdx.x * R;
  for (int i = threadIdx.x; i < R * width; i += blockDim.x) {
    const int r = i / width, c = i % width;
    rows[i] = (t0 + r < num_tokens) ? x[(int64_t)(t0 + r) * x_stride + c] : from_f32<T>(0.f);
  }
  __syncthreads();
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE, waves = blockDim.x / MI_WAVE;
  const int total = outputs + (gate_row != nullptr ? 1 : 0);
  const bool vec = width % 4 == 0 && ((uintptr_t)router % 16) == 0 && (gate_row == nullptr || ((uintptr_t)gate_row % 16) == 0);
  for (int e = wave; e < total; e += waves) {
    const float* w = e < outputs ? router + (int64_t)e * width : gate_row;
    A sum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) sum[r] = 0;
    if (vec) {
#pragma unroll 4
      for (int c = lane * 4; c < width; c += MI_WAVE * 4) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + c);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const T* xr = rows + (size_t)r * width + c;
          sum[r] += (A)w4.x * (A)to_f32(xr[0]) + (A)w4.y * (A)to_f32(xr[1]) + (A)w4.z * (A)to_f32(xr[2]) + (A)w4.w * (A)to_f32(xr[3]);
        }
      }
    } else {
      for (int c = lane; c < width; c += MI_WAVE) {
        const A wc = (A)w[c];
#pragma unroll
        for (int r = 0; r < R; ++r) sum[r] += wc * (A)to_f32(rows[(size_t)r * width + c]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const A all = lanes_total(sum[r]);
      if (lane == 0) z[r * (outputs + 1) + e] = all;
    }
  }
  __syncthreads();
  const int r = threadIdx.x, t = t0 + r;
  if (r >= R || t >= num_tokens) return;
  A* mine = z + r * (outputs + 1);
  if (gate_row != nullptr) shared_gate[t] = (float)((A)1 / ((A)1 + exp_of(-mine[outputs])));
  A most = mine[0];
  for (int e = 1; e < outputs; ++e) most = mine[e] > most ? mine[e] : most;
  A sum = 0;
  for (int e = 0; e < outputs; ++e) {
    mine[e] = exp_of(mine[e] - most);
    sum += mine[e];
  }
  const A inv = (A)1 / sum;
  // the choice is made on score + correction, the weight is the score alone
  for (int k = 0; k < top; ++k) {
    int best = -1;
    A best_choice = 0;
    for (int e = 0; e < outputs; ++e) {
      if (mine[e] < (A)0) continue;  // taken already
      const A choice = mine[e] * inv + (correction != nullptr ? (A)correction[e] : (A)0);
      if (best < 0 || choice > best_choice) best = e, best_choice = choice;
    }
    chosen[(int64_t)t * top + k] = best;
    weights[(int64_t)t * top + k] = (float)(mine[best] * inv * (A)route_scale);
    mine[best] = (A)-1;
  }
}

// a wave's dot product of a weight row with a vector kept in LDS in the element type
template <typename T, typename A>
__device__ __forceinline__ A dot_lds(const T* __restrict__ w, const T* __restrict__ v, int n, int lane) {
  A sum = 0;
  if (n % 8 == 0 && ((uintptr_t)w % 16) == 0) {
    constexpr int V = 16 / sizeof(T);
    for (int c = lane * V; c < n; c += MI_WAVE * V) {
      alignas(16) T a[V];
      *reinterpret_cast<uint4*>(a) = *reinterpret_cast<const uint4*>(w + c);
#pragma unroll
      for (int j = 0; j < V; ++j) sum += (A)to_f32(a[j]) * (A)to_f32(v[c + j]);
    }
  } else {
    for (int c = lane; c < n; c += MI_WAVE) sum += (A)to_f32(w[c]) * (A)to_f32(v[c]);
  }
  return lanes_total(sum);
}

#define MI_EXPERT_FEATURES 16  // features (or columns) a block of four waves makes

template <typename T>
__global__ __launch_bounds__(256) void expert_gate_up_kernel(
    const T* __restrict__ x, int64_t x_stride, const T* __restrict__ gate_up, const int* __restrict__ chosen,
    T* __restrict__ act, int width, int ff, int experts, int top) {
  using A = typename SumOf<T>::type;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  T* row = reinterpret_cast<T*>(lds_bytes);
  const int pair = blockIdx.x;
  const int e = chosen[pair];
  if (e < 0 || e >= experts) return;  // an identity expert: nothing to make (the whole block leaves)
  const T* src = x + (int64_t)(pair / top) * x_stride;
  for (int c = threadIdx.x; c < width; c += blockDim.x) row[c] = src[c];
  __syncthreads();
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE, waves = blockDim.x / MI_WAVE;
  const T* w = gate_up + (int64_t)e * 2 * ff * width;
  const int first = blockIdx.y * MI_EXPERT_FEATURES;
  for (int f = first + wave; f < min(first + MI_EXPERT_FEATURES, ff); f += waves) {
    const A g = dot_lds<T, A>(w + (int64_t)f * width, row, width, lane);
    const A u = dot_lds<T, A>(w + (int64_t)(ff + f) * width, row, width, lane);
    if (lane == 0) {
      // the two products as the element type holds them, then silu(g) * u
      const A gr = (A)to_f32(from_f32<T>((float)g)), ur = (A)to_f32(from_f32<T>((float)u));
      act[(int64_t)pair * ff + f] = from_f32<T>((float)(gr / ((A)1 + exp_of(-gr)) * ur));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void expert_down_combine_kernel(
    const T* __restrict__ act, const T* __restrict__ down, const int* __restrict__ chosen, const float* __restrict__ weights,
    const T* __restrict__ x, int64_t x_stride, const T* __restrict__ shared, int64_t shared_stride,
    const float* __restrict__ shared_gate, T* __restrict__ out, int width, int ff, int experts, int top) {
  using A = typename SumOf<T>::type;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  T* rows = reinterpret_cast<T*>(lds_bytes);  // [top][ff]
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < top * ff; i += blockDim.x) {
    const int e = chosen[(int64_t)t * top + i / ff];
    rows[i] = (e >= 0 && e < experts) ? act[(int64_t)t * top * ff + i] : from_f32<T>(0.f);
  }
  __syncthreads();
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE, waves = blockDim.x / MI_WAVE;
  const int first = blockIdx.y * MI_EXPERT_FEATURES;
  for (int c = first + wave; c < min(first + MI_EXPERT_FEATURES, width); c += waves) {
    A sum = 0;
    for (int k = 0; k < top; ++k) {
      const int e = chosen[(int64_t)t * top + k];
      const A weight = (A)weights[(int64_t)t * top + k];
      if (e >= experts) {
        sum += weight * (A)to_f32(x[(int64_t)t * x_stride + c]);
      } else if (e >= 0) {
        const A y = dot_lds<T, A>(down + ((int64_t)e * width + c) * ff, rows + (int64_t)k * ff, ff, lane);
        sum += weight * (A)to_f32(from_f32<T>((float)y));
      }
    }
    if (shared != nullptr) sum += (A)shared_gate[t] * (A)to_f32(shared[(int64_t)t * shared_stride + c]);
    if (lane == 0) out[(int64_t)t * width + c] = from_f32<T>((float)sum);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void expert_combine_kernel(
    const T* __restrict__ made, const int* __restrict__ where, const int* __restrict__ chosen,
    const float* __restrict__ weights, const T* __restrict__ x, int64_t x_stride, const T* __restrict__ shared,
    int64_t shared_stride, const float* __restrict__ shared_gate, T* __restrict__ out, int width, int experts, int top) {
  using A = typename SumOf<T>::type;
  const int t = blockIdx.x;
  for (int c = threadIdx.x * VEC; c < width; c += blockDim.x * VEC) {
    A sum[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) sum[j] = 0;
    for (int k = 0; k < top; ++k) {
      const int64_t pair = (int64_t)t * top + k;
      const int e = chosen[pair];
      if (e < 0) continue;
      const T* src = e >= experts ? x + (int64_t)t * x_stride : made + (int64_t)(where != nullptr ? where[pair] : pair) * width;
      float v[VEC];
      mi_load_cols<T, VEC>(src + c, v);
      const A weight = (A)weights[pair];
#pragma unroll
      for (int j = 0; j < VEC; ++j) sum[j] += weight * (A)v[j];
    }
    float r[VEC];
    if (shared != nullptr) {
      mi_load_cols<T, VEC>(shared + (int64_t)t * shared_stride + c, r);
      const A g = (A)shared_gate[t];
#pragma unroll
      for (int j = 0; j < VEC; ++j) sum[j] += g * (A)r[j];
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) r[j] = (float)sum[j];
    mi_store_cols<T, VEC>(out + (int64_t)t * width + c, r);
  }
}

inline bool is_aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

}  // namespace

extern "C" int mi_route_top_k(int dtype, const void* x, int64_t x_stride, const float* router, const float* correction,
                              const float* gate_row, int* chosen, float* weights, float* shared_gate, int num_tokens,
                              int width, int outputs, int top, float route_scale, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && x_stride >= width, "route_top_k: bad sizes tokens=%d width=%d", num_tokens, width);
  MI_REQUIRE(outputs > 0 && outputs <= MI_ROUTER_MAX_OUTPUTS && top > 0 && top <= outputs,
             "route_top_k: %d router outputs (at most %d) of which %d are chosen", outputs, MI_ROUTER_MAX_OUTPUTS, top);
  MI_REQUIRE(gate_row == nullptr || shared_gate != nullptr, "route_top_k: a gate row needs a place for the gates");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "route_top_k: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  // as many tokens a block as fit its staging (rows in the element type, sums beside them), at most 4
  const size_t elem = dtype == MI_F32 ? 4 : 2, acc = dtype == MI_F32 ? 8 : 4;
  auto lds_for = [&](int r) { return (size_t)r * (outputs + 1) * acc + (size_t)r * width * elem; };
  const int per_block = lds_for(4) <= 64 * 1024 ? 4 : (lds_for(2) <= 64 * 1024 ? 2 : 1);
  MI_REQUIRE(lds_for(per_block) <= 64 * 1024, "route_top_k: rows of %d do not fit the block's staging", width);
  const int threads = num_tokens <= 64 ? 1024 : 256;
  const int blocks = ceil_div(num_tokens, per_block);
#define MI_ROUTE(T, R)                                                                                               \
  route_top_k_kernel<T, R><<<blocks, threads, lds_for(R), stream>>>((const T*)x, x_stride, router, correction, gate_row, \
                                                                    chosen, weights, shared_gate, num_tokens, width,    \
                                                                    outputs, top, route_scale)
  if (dtype == MI_F32) {
    if (per_block == 4) MI_ROUTE(float, 4);
    else if (per_block == 2) MI_ROUTE(float, 2);
    else MI_ROUTE(float, 1);
  } else {
    if (per_block == 4) MI_ROUTE(bf16_t, 4);
    else if (per_block == 2) MI_ROUTE(bf16_t, 2);
    else MI_ROUTE(bf16_t, 1);
  }
#undef MI_ROUTE
  MI_CHECK_LAUNCH("route_top_k");
  return MI_OK;
}

// act: [num_tokens * top, ff]; rows of pairs whose expert is an identity expert are not written.
extern "C" int mi_expert_gate_up(int dtype, const void* x, int64_t x_stride, const void* gate_up, const int* chosen,
                                 void* act, int num_tokens, int width, int ff, int experts, int top, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && ff > 0 && experts > 0 && top > 0 && x_stride >= width,
             "expert_gate_up: bad sizes tokens=%d width=%d ff=%d experts=%d top=%d", num_tokens, width, ff, experts, top);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "expert_gate_up: unknown dtype %d", dtype);
  const size_t lds = (size_t)width * (dtype == MI_F32 ? 4 : 2);
  MI_REQUIRE(lds <= 64 * 1024, "expert_gate_up: rows of %d do not fit the block's staging", width);
  MI_REQUIRE((int64_t)num_tokens * top <= 0x7fffffff / 2 && ceil_div(ff, MI_EXPERT_FEATURES) <= 65535, "expert_gate_up: too many pairs or features");
  if (num_tokens == 0) return MI_OK;
  dim3 grid(num_tokens * top, ceil_div(ff, MI_EXPERT_FEATURES));
  if (dtype == MI_F32)
    expert_gate_up_kernel<float><<<grid, 256, lds, stream>>>((const float*)x, x_stride, (const float*)gate_up, chosen,
                                                             (float*)act, width, ff, experts, top);
  else
    expert_gate_up_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)x, x_stride, (const bf16_t*)gate_up, chosen,
                                                              (bf16_t*)act, width, ff, experts, top);
  MI_CHECK_LAUNCH("expert_gate_up");
  return MI_OK;
}

extern "C" int mi_expert_down_combine(int dtype, const void* act, const void* down, const int* chosen, const float* weights,
                                      const void* x, int64_t x_stride, const void* shared, int64_t shared_stride,
                                      const float* shared_gate, void* out, int num_tokens, int width, int ff, int experts,
                                      int top, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && ff > 0 && experts > 0 && top > 0 && x_stride >= width,
             "expert_down_combine: bad sizes tokens=%d width=%d ff=%d experts=%d top=%d", num_tokens, width, ff, experts, top);
  MI_REQUIRE(shared == nullptr || (shared_gate != nullptr && shared_stride >= width), "expert_down_combine: a shared expert's rows come with their gates");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "expert_down_combine: unknown dtype %d", dtype);
  const size_t lds = (size_t)top * ff * (dtype == MI_F32 ? 4 : 2);
  MI_REQUIRE(lds <= 64 * 1024, "expert_down_combine: %d rows of %d do not fit the block's staging", top, ff);
  MI_REQUIRE(ceil_div(width, MI_EXPERT_FEATURES) <= 65535, "expert_down_combine: too many columns");
  if (num_tokens == 0) return MI_OK;
  dim3 grid(num_tokens, ceil_div(width, MI_EXPERT_FEATURES));
  if (dtype == MI_F32)
    expert_down_combine_kernel<float><<<grid, 256, lds, stream>>>(
        (const float*)act, (const float*)down, chosen, weights, (const float*)x, x_stride, (const float*)shared, shared_stride,
        shared_gate, (float*)out, width, ff, experts, top);
  else
    expert_down_combine_kernel<bf16_t><<<grid, 256, lds, stream>>>(
        (const bf16_t*)act, (const bf16_t*)down, chosen, weights, (const bf16_t*)x, x_stride, (const bf16_t*)shared,
        shared_stride, shared_gate, (bf16_t*)out, width, ff, experts, top);
  MI_CHECK_LAUNCH("expert_down_combine");
  return MI_OK;
}

// made: rows of expert outputs [*, width]; pair (t, k) finds its row at where[t * top + k] (or at
// t * top + k itself with where = null).
extern "C" int mi_expert_combine(int dtype, const void* made, const int* where, const int* chosen, const float* weights,
                                 const void* x, int64_t x_stride, const void* shared, int64_t shared_stride,
                                 const float* shared_gate, void* out, int num_tokens, int width, int experts, int top,
                                 hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && experts > 0 && top > 0 && x_stride >= width,
             "expert_combine: bad sizes tokens=%d width=%d experts=%d top=%d", num_tokens, width, experts, top);
  MI_REQUIRE(shared == nullptr || (shared_gate != nullptr && shared_stride >= width), "expert_combine: a shared expert's rows come with their gates");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "expert_combine: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const bool vec = width % 4 == 0 && x_stride % 4 == 0 && shared_stride % 4 == 0 && is_aligned16(made) && is_aligned16(x) &&
                   is_aligned16(shared) && is_aligned16(out);
#define MI_COMBINE(T, VEC)                                                                                              \
  expert_combine_kernel<T, VEC><<<num_tokens, 256, 0, stream>>>((const T*)made, where, chosen, weights, (const T*)x,    \
                                                                x_stride, (const T*)shared, shared_stride, shared_gate, \
                                                                (T*)out, width, experts, top)
  if (dtype == MI_F32) {
    if (vec) MI_COMBINE(float, 4);
    else MI_COMBINE(float, 1);
  } else {
    if (vec) MI_COMBINE(bf16_t, 4);
    else MI_COMBINE(bf16_t, 1);
  }
#undef MI_COMBINE
  MI_CHECK_LAUNCH("expert_combine");
  return MI_OK;
}
