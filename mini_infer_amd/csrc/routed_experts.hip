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
  constexpr int V = 16 / sizeof(T);
  const size_t rows_at = (size_t)R * (outputs + 1) * sizeof(A);
  if (width % V == 0 && x_stride % V == 0 && ((uintptr_t)x % 16) == 0 && rows_at % 16 == 0) {  // 16 bytes a thread
    for (int i = threadIdx.x * V; i < R * width; i += blockDim.x * V) {
      const int r = i / width, c = i % width;
      uint4 got = make_uint4(0, 0, 0, 0);
      if (t0 + r < num_tokens) got = *reinterpret_cast<const uint4*>(x + (int64_t)(t0 + r) * x_stride + c);
      *reinterpret_cast<uint4*>(rows + i) = got;
    }
  } else {
    for (int i = threadIdx.x; i < R * width; i += blockDim.x) {
      const int r = i / width, c = i % width;
      rows[i] = (t0 + r < num_tokens) ? x[(int64_t)(t0 + r) * x_stride + c] : from_f32<T>(0.f);
    }
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

// ---------------------------------------------------------------------------------------------
// Expert by expert, for steps of few rows that the host knows nothing about (recorded steps):
//   expert_sort      one block: the (token, choice) pairs counted per chosen expert and listed expert
//                    by expert (`listed` [pairs], `first` [experts + 1]; identity experts are left out).
//   expert_rows      a block owns one expert and a tile of FT of its output features, and walks the
//                    expert's listed pairs R rows at a time: the rows wait in LDS, every wave streams
//                    its features' weight rows once for all R rows (16 bytes a lane) and keeps
//                    R sums a weight row.  GATED: features come in pairs (gate row f, up row
//                    ff + f) and silu(gate) * up is what is written; else the plain product.
// So an expert's weights are read once per R of its rows, whatever the number of pairs.
// ---------------------------------------------------------------------------------------------

#define MI_SORT_MAX_EXPERTS 1024

__global__ __launch_bounds__(256) void expert_sort_kernel(const int* __restrict__ chosen, int* __restrict__ listed,
                                                          int* __restrict__ first, int pairs, int experts) {
  __shared__ int count[MI_SORT_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e <= experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      const int n = count[e];
      first[e] = at;
      count[e] = at;  // where the expert's next pair goes
      at += n;
    }
    first[experts] = at;
  }
  __syncthreads();
  // (pairs of one expert in any order: each pair's result is its own)
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < experts) listed[atomicAdd(&count[e], 1)] = p;
  }
}

template <typename T, int R, bool GATED>
__global__ __launch_bounds__(256) void expert_rows_kernel(
    const T* __restrict__ src, int64_t src_stride, int src_div, const T* __restrict__ weight, int64_t expert_stride,
    const int* __restrict__ listed, const int* __restrict__ first, T* __restrict__ out, int64_t out_stride, int k_dim,
    int features) {
  using A = typename SumOf<T>::type;
  constexpr int FW = 4;             // features a wave
  constexpr int WR = GATED ? 2 : 1;  // weight rows a feature
  constexpr int V = 16 / sizeof(T);
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  T* rows = reinterpret_cast<T*>(lds_bytes);  // [R][k_dim]
  const int e = blockIdx.y;  // (feature tiles run fastest: a chosen expert's blocks follow one another and spread over all XCDs)
  const int begin = first[e], end = first[e + 1];
  if (begin >= end) return;  // nobody chose this expert (the whole block leaves)
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int f0 = (blockIdx.x * (blockDim.x / MI_WAVE) + wave) * FW;
  const T* w = weight + (int64_t)e * expert_stride;
  for (int chunk = begin; chunk < end; chunk += R) {
    const int n = min(R, end - chunk);
    __syncthreads();
    for (int i = threadIdx.x * V; i < R * k_dim; i += blockDim.x * V) {
      const int r = i / k_dim, c = i % k_dim;  // (V divides k_dim)
      uint4 got = make_uint4(0, 0, 0, 0);
      if (r < n) got = *reinterpret_cast<const uint4*>(src + (int64_t)(listed[chunk + r] / src_div) * src_stride + c);
      *reinterpret_cast<uint4*>(rows + i) = got;
    }
    __syncthreads();
    if (f0 >= features) continue;  // (a wave past the last feature still helps to stage rows)
    A sum[FW][WR][R];
#pragma unroll
    for (int f = 0; f < FW; ++f)
#pragma unroll
      for (int g = 0; g < WR; ++g)
#pragma unroll
        for (int r = 0; r < R; ++r) sum[f][g][r] = 0;
    for (int c = lane * V; c < k_dim; c += MI_WAVE * V) {
      alignas(16) T wv[FW][WR][V];
#pragma unroll
      for (int f = 0; f < FW; ++f)
#pragma unroll
        for (int g = 0; g < WR; ++g) {
          const int row = min(f0 + f, features - 1) + g * features;  // (past the end: the last feature again, not written)
          // (the weights are read once: non-temporal, whole 16-byte pieces)
          *reinterpret_cast<int32x4_t*>(wv[f][g]) =
              __builtin_nontemporal_load(reinterpret_cast<const int32x4_t*>(w + (int64_t)row * k_dim + c));
        }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        alignas(16) T xv[V];
        *reinterpret_cast<uint4*>(xv) = *reinterpret_cast<const uint4*>(rows + (size_t)r * k_dim + c);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const A xj = (A)to_f32(xv[j]);
#pragma unroll
          for (int f = 0; f < FW; ++f)
#pragma unroll
            for (int g = 0; g < WR; ++g) sum[f][g][r] += (A)to_f32(wv[f][g][j]) * xj;
        }
      }
    }
#pragma unroll
    for (int f = 0; f < FW; ++f)
#pragma unroll
      for (int r = 0; r < R; ++r) {
        A a = lanes_total(sum[f][0][r]);
        A b = GATED ? lanes_total(sum[f][WR - 1][r]) : (A)0;
        if (lane == 0 && r < n && f0 + f < features) {
          T* o = out + (int64_t)listed[chunk + r] * out_stride + f0 + f;
          if constexpr (GATED) {
            // the two products as the element type holds them, then silu(gate) * up
            const A gr = (A)to_f32(from_f32<T>((float)a)), ur = (A)to_f32(from_f32<T>((float)b));
            *o = from_f32<T>((float)(gr / ((A)1 + exp_of(-gr)) * ur));
          } else {
            *o = from_f32<T>((float)a);
          }
        }
      }
  }
}

// The same for bfloat16 on the matrix cores (MFMA 16x16x32): a block owns one expert and 16 of its
// output features and takes the expert's listed pairs 16 rows at a time.  Its four waves share K (wave w
// takes the w-th quarter of the steps of 32 elements); per step a lane reads 16 bytes of weight row `lane % 16` and
// 16 bytes of pair `lane % 16`'s input row (both at elements 32 * step + 8 * (lane / 16)), which are the
// two operands as they are, so nothing is staged; rows past the expert's last pair read nothing.  The
// waves' sums meet in LDS in wave order, and lane (quad, col) of wave 0 writes features 4 * quad .. + 3 of
// pair col.  Needs K a multiple of 32.
typedef float f32x4_e __attribute__((ext_vector_type(4)));

template <bool GATED>
__global__ __launch_bounds__(256) void expert_rows_mfma_kernel(
    const bf16_t* __restrict__ src, int64_t src_stride, int src_div, const bf16_t* __restrict__ weight,
    int64_t expert_stride, const int* __restrict__ listed, const int* __restrict__ first, bf16_t* __restrict__ out,
    int64_t out_stride, int k_dim, int features) {
  __shared__ f32x4_e meet[GATED ? 2 : 1][3][MI_WAVE];
  const int e = blockIdx.y;  // (feature tiles run fastest: a chosen expert's blocks follow one another and spread over all XCDs)
  const int begin = first[e], end = first[e + 1];
  if (begin >= end) return;  // nobody chose this expert (the whole block leaves)
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16, quad = lane / 16;
  const int f0 = blockIdx.x * 16;
  const int my_feature = min(f0 + col, features - 1);  // (past the end: the last feature again, not written)
  const bf16_t* w_gate = weight + (int64_t)e * expert_stride + (int64_t)my_feature * k_dim + quad * 8;
  const bf16_t* w_up = w_gate + (int64_t)features * k_dim;
  const int steps = k_dim / 32;
  for (int chunk = begin; chunk < end; chunk += 16) {
    const int n = min(16, end - chunk);
    const int pair = col < n ? listed[chunk + col] : -1;
    // (lanes past the expert's last pair read the chunk's first row and count it as nothing)
    const bf16_t* x_row = src + (int64_t)((pair >= 0 ? pair : listed[chunk]) / src_div) * src_stride + quad * 8;
    f32x4_e acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    const bf16x8_t nothing = {};
    // a wave's quarter of K in one stretch (its consecutive loads then use whole cache lines), four
    // steps' loads asked for before the first of them is used
    const int lo = steps * wave / 4, hi = steps * (wave + 1) / 4;
    int step = lo;
    for (; step + 4 <= hi; step += 4) {
      bf16x8_t a_g[4], a_u[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a_g[i] = *reinterpret_cast<const bf16x8_t*>(w_gate + (step + i) * 32);
        if constexpr (GATED) a_u[i] = *reinterpret_cast<const bf16x8_t*>(w_up + (step + i) * 32);
        b[i] = *reinterpret_cast<const bf16x8_t*>(x_row + (step + i) * 32);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bf16x8_t seen = pair >= 0 ? b[i] : nothing;
        acc_g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_g[i], seen, acc_g, 0, 0, 0);
        if constexpr (GATED) acc_u = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_u[i], seen, acc_u, 0, 0, 0);
      }
    }
    for (; step < hi; ++step) {
      const bf16x8_t a_g = *reinterpret_cast<const bf16x8_t*>(w_gate + step * 32);
      const bf16x8_t got = *reinterpret_cast<const bf16x8_t*>(x_row + step * 32);
      const bf16x8_t seen = pair >= 0 ? got : nothing;
      acc_g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_g, seen, acc_g, 0, 0, 0);
      if constexpr (GATED) {
        const bf16x8_t a_u = *reinterpret_cast<const bf16x8_t*>(w_up + step * 32);
        acc_u = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_u, seen, acc_u, 0, 0, 0);
      }
    }
    __syncthreads();  // (the last chunk's sums have been read)
    if (wave > 0) {
      meet[0][wave - 1][lane] = acc_g;
      if constexpr (GATED) meet[1][wave - 1][lane] = acc_u;
    }
    __syncthreads();
    if (wave == 0 && pair >= 0) {
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        acc_g += meet[0][w][lane];
        if constexpr (GATED) acc_u += meet[1][w][lane];
      }
      bf16_t* o = out + (int64_t)pair * out_stride;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int f = f0 + 4 * quad + r;
        if (f >= features) continue;
        if constexpr (GATED) {
          // the two products as bfloat16 holds them, then silu(gate) * up
          const float g = to_f32(from_f32<bf16_t>(acc_g[r])), u = to_f32(from_f32<bf16_t>(acc_u[r]));
          o[f] = from_f32<bf16_t>(g / (1.f + expf(-g)) * u);
        } else {
          o[f] = from_f32<bf16_t>(acc_g[r]);
        }
      }
    }
  }
}

// Many rows an expert (a prompt): a block owns one expert and 64 of its output features, a wave 16 of
// them over all of K, and the expert's listed pairs are taken 64 rows a pass: per step of 32 elements a wave
// reads its 16 weight rows once (16 bytes a lane) and the four row tiles' input rows (the same for the
// block's four waves, so three of four reads hit the cache), and makes 4 (gated: 8) MFMA 16x16x32.  An
// expert's weights are read once per 64 of its rows and its rows once per 64 of its features.
template <bool GATED>
__global__ __launch_bounds__(256) void expert_tiles_mfma_kernel(
    const bf16_t* __restrict__ src, int64_t src_stride, int src_div, const bf16_t* __restrict__ weight,
    int64_t expert_stride, const int* __restrict__ listed, const int* __restrict__ first, bf16_t* __restrict__ out,
    int64_t out_stride, int k_dim, int features) {
  constexpr int RT = 4;  // row tiles of 16
  const int e = blockIdx.y;
  const int begin = first[e], end = first[e + 1];
  if (begin >= end) return;
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16, quad = lane / 16;
  const int f0 = blockIdx.x * 64 + wave * 16;
  if (f0 >= features) return;  // (no barrier below: a wave past the last feature may leave)
  const int my_feature = min(f0 + col, features - 1);
  const bf16_t* w_gate = weight + (int64_t)e * expert_stride + (int64_t)my_feature * k_dim + quad * 8;
  const bf16_t* w_up = w_gate + (int64_t)features * k_dim;
  const int steps = k_dim / 32;
  const bf16x8_t nothing = {};
  for (int chunk = begin; chunk < end; chunk += 16 * RT) {
    const int n = min(16 * RT, end - chunk);
    int pair[RT];
    const bf16_t* x_row[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      pair[t] = 16 * t + col < n ? listed[chunk + 16 * t + col] : -1;
      x_row[t] = src + (int64_t)((pair[t] >= 0 ? pair[t] : listed[chunk]) / src_div) * src_stride + quad * 8;
    }
    f32x4_e acc_g[RT], acc_u[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) acc_g[t] = acc_u[t] = f32x4_e{0.f, 0.f, 0.f, 0.f};
    auto one_step = [&](int step) {
      const bf16x8_t a_g = *reinterpret_cast<const bf16x8_t*>(w_gate + step * 32);
      bf16x8_t a_u = nothing;
      if constexpr (GATED) a_u = *reinterpret_cast<const bf16x8_t*>(w_up + step * 32);
      bf16x8_t b[RT];
#pragma unroll
      for (int t = 0; t < RT; ++t) b[t] = *reinterpret_cast<const bf16x8_t*>(x_row[t] + step * 32);
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        if (16 * t >= n) continue;  // (a tile without rows: the same for the whole block)
        const bf16x8_t seen = pair[t] >= 0 ? b[t] : nothing;
        acc_g[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_g, seen, acc_g[t], 0, 0, 0);
        if constexpr (GATED) acc_u[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_u, seen, acc_u[t], 0, 0, 0);
      }
    };
    int step = 0;
    for (; step + 2 <= steps; step += 2) {
      one_step(step);
      one_step(step + 1);
    }
    for (; step < steps; ++step) one_step(step);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (pair[t] < 0) continue;
      bf16_t* o = out + (int64_t)pair[t] * out_stride;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int f = f0 + 4 * quad + r;
        if (f >= features) continue;
        if constexpr (GATED) {
          const float g = to_f32(from_f32<bf16_t>(acc_g[t][r])), u = to_f32(from_f32<bf16_t>(acc_u[t][r]));
          o[f] = from_f32<bf16_t>(g / (1.f + expf(-g)) * u);
        } else {
          o[f] = from_f32<bf16_t>(acc_g[t][r]);
        }
      }
    }
  }
}

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

extern "C" int mi_expert_sort(const int* chosen, int* listed, int* first, int pairs, int experts, hipStream_t stream) {
  MI_REQUIRE(pairs >= 0 && experts > 0 && experts <= MI_SORT_MAX_EXPERTS, "expert_sort: %d pairs over %d experts (at most %d)", pairs,
             experts, MI_SORT_MAX_EXPERTS);
  expert_sort_kernel<<<1, 256, 0, stream>>>(chosen, listed, first, pairs, experts);
  MI_CHECK_LAUNCH("expert_sort");
  return MI_OK;
}

// Rows a block keeps in LDS at a time for rows of k_dim elements (0: such rows do not fit).
extern "C" int mi_expert_rows_at_once(int dtype, int k_dim) {
  const size_t row = (size_t)k_dim * (dtype == MI_F32 ? 4 : 2);
  if (dtype != MI_F32 && 8 * row <= 64 * 1024) return 8;
  if (4 * row <= 64 * 1024) return 4;
  if (2 * row <= 64 * 1024) return 2;
  return 0;
}

// gated = 1: weight [experts, 2 * features, k_dim], out[pair, f] = silu(gate_f . row) * (up_f . row) with the row of
// pair p at src[p / src_div]; gated = 0: weight [experts, features, k_dim], out[pair, f] = w_f . src[p / src_div].
// many_rows = 1 (bfloat16 with k_dim a multiple of 32 only): blocks of 64 features that take 64 rows a pass.
extern "C" int mi_expert_rows(int dtype, int gated, const void* src, int64_t src_stride, int src_div, const void* weight,
                              const int* listed, const int* first, void* out, int64_t out_stride, int experts, int k_dim,
                              int features, int many_rows, hipStream_t stream) {
  MI_REQUIRE(experts > 0 && experts <= 65535 && k_dim > 0 && features > 0 && src_div > 0 && src_stride >= k_dim && out_stride >= features,
             "expert_rows: bad sizes experts=%d k=%d features=%d", experts, k_dim, features);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "expert_rows: unknown dtype %d", dtype);
  const int elem = dtype == MI_F32 ? 4 : 2, step = 16 / elem;
  MI_REQUIRE(k_dim % step == 0 && src_stride % step == 0 && is_aligned16(src) && is_aligned16(weight),
             "expert_rows: rows of %d elements are not read 16 bytes at a time", k_dim);
  const int64_t expert_stride = (int64_t)(gated ? 2 : 1) * features * k_dim;
  dim3 grid(ceil_div(features, 16), experts);
  if (dtype == MI_BF16 && k_dim % 32 == 0 && many_rows) {
    dim3 tiles(ceil_div(features, 64), experts);
    if (gated)
      expert_tiles_mfma_kernel<true><<<tiles, 256, 0, stream>>>((const bf16_t*)src, src_stride, src_div, (const bf16_t*)weight,
                                                                expert_stride, listed, first, (bf16_t*)out, out_stride, k_dim, features);
    else
      expert_tiles_mfma_kernel<false><<<tiles, 256, 0, stream>>>((const bf16_t*)src, src_stride, src_div, (const bf16_t*)weight,
                                                                 expert_stride, listed, first, (bf16_t*)out, out_stride, k_dim, features);
    MI_CHECK_LAUNCH("expert_tiles_mfma");
    return MI_OK;
  }
  if (dtype == MI_BF16 && k_dim % 32 == 0) {  // the matrix cores
    if (gated)
      expert_rows_mfma_kernel<true><<<grid, 256, 0, stream>>>((const bf16_t*)src, src_stride, src_div, (const bf16_t*)weight,
                                                              expert_stride, listed, first, (bf16_t*)out, out_stride, k_dim, features);
    else
      expert_rows_mfma_kernel<false><<<grid, 256, 0, stream>>>((const bf16_t*)src, src_stride, src_div, (const bf16_t*)weight,
                                                               expert_stride, listed, first, (bf16_t*)out, out_stride, k_dim, features);
    MI_CHECK_LAUNCH("expert_rows_mfma");
    return MI_OK;
  }
  const int at_once = mi_expert_rows_at_once(dtype, k_dim);
  MI_REQUIRE(at_once > 0, "expert_rows: rows of %d do not fit the block's staging", k_dim);
  const size_t lds = (size_t)at_once * k_dim * elem;
#define MI_ROWS(T, R)                                                                                                     \
  do {                                                                                                                    \
    if (gated)                                                                                                            \
      expert_rows_kernel<T, R, true><<<grid, 256, lds, stream>>>((const T*)src, src_stride, src_div, (const T*)weight,    \
                                                                 expert_stride, listed, first, (T*)out, out_stride, k_dim, \
                                                                 features);                                                \
    else                                                                                                                  \
      expert_rows_kernel<T, R, false><<<grid, 256, lds, stream>>>((const T*)src, src_stride, src_div, (const T*)weight,   \
                                                                  expert_stride, listed, first, (T*)out, out_stride, k_dim, \
                                                                  features);                                               \
  } while (0)
  if (dtype == MI_F32) {
    if (at_once == 4) MI_ROWS(float, 4);
    else MI_ROWS(float, 2);
  } else {
    if (at_once == 8) MI_ROWS(bf16_t, 8);
    else if (at_once == 4) MI_ROWS(bf16_t, 4);
    else MI_ROWS(bf16_t, 2);
  }
#undef MI_ROWS
  MI_CHECK_LAUNCH("expert_rows");
  return MI_OK;
}
