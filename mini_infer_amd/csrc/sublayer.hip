// Kernels around sublayers that add their own normed output to the residual stream, and the
// mixers and activations that go with them:
//   embed_sinusoid      table row * scale + interleaved sin/cos of the position -> float32 stream
//   norm_scale_add      stream += y * rsqrt(mean(y^2) + eps) * gain * scale[c]   (norm on a sublayer's OUTPUT)
//   cast_rows           the stream in the compute dtype, for the products that read it
//   gated_scan          minGRU: a gated recurrence whose gates read the current token only
//   qk_norm_kv_write    RMS norm of q and of k over the WHOLE projection; normed k -> key pages,
//                       k as projected -> value pages (values that are the keys)
//   poly_norm           a N(z) + b N(z^2) + c N(z^3) + e over a token's feed-forward values
//   gated_table_rows    gelu_tanh(gate) * (a slice of a per-token table row)
// Storage is float32 or bfloat16.  Statistics, gates, the recurrent state and the stream are
// float32 with bfloat16 elements; with float32 elements (the 32-bit path) they are evaluated
// in 64-bit and rounded once, as in the other per-token kernels.
#include "common.h"

#include <math.h>

typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));

// four consecutive elements at once (8- and 16-byte accesses; the caller checks alignment)
__device__ __forceinline__ void load4(const float* p, float v[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float v[4]) {
  const bf16x4_t x = *reinterpret_cast<const bf16x4_t*>(p);
  v[0] = (float)x[0]; v[1] = (float)x[1]; v[2] = (float)x[2]; v[3] = (float)x[3];
}
__device__ __forceinline__ void store4(float* p, const float v[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float v[4]) {
  bf16x4_t x;
  x[0] = (bf16_t)v[0]; x[1] = (bf16_t)v[1]; x[2] = (bf16_t)v[2]; x[3] = (bf16_t)v[3];
  *reinterpret_cast<bf16x4_t*>(p) = x;
}
static inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }
// Row kernels run one block a row: few rows (decode) get wide blocks so that a row is one or two
// trips a thread, many rows (prompts) narrow ones so that several rows share a CU.
static inline int row_block(int rows, int items) { return (rows < 256 && items > 1024) ? 1024 : 256; }

template <typename T>
struct Wide {
  using type = float;
};
template <>
struct Wide<float> {
  using type = double;
};

__device__ __forceinline__ float lane_xor(float v, int off) { return __shfl_xor(v, off, MI_WAVE); }
__device__ __forceinline__ double lane_xor(double v, int off) { return __shfl_xor(v, off, MI_WAVE); }

// Sum over the block in a fixed order; `scratch` holds one value per wave.  All threads get it.
template <typename A>
__device__ __forceinline__ A block_total(A v, A* scratch) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += lane_xor(v, off);
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  A total = 0;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float inv_root(float mean_sq, float eps) { return 1.0f / sqrtf(mean_sq + eps); }
__device__ __forceinline__ double inv_root(double mean_sq, double eps) { return 1.0 / sqrt(mean_sq + eps); }
__device__ __forceinline__ float logistic(float z) { return mi_logistic(z); }
__device__ __forceinline__ double logistic(double z) { return 1.0 / (1.0 + exp(-z)); }
// keep * s + add in one rounding, spelled out: left to the compiler, two kernels that step the
// same recurrence contracted it differently and their states differed in the last bit
__device__ __forceinline__ float fused_step(float keep, float s, float add) { return __builtin_fmaf(keep, s, add); }
__device__ __forceinline__ double fused_step(double keep, double s, double add) { return __builtin_fma(keep, s, add); }
__device__ __forceinline__ float tanh_of(float z) { return tanhf(z); }
__device__ __forceinline__ double tanh_of(double z) { return tanh(z); }

// ---------------------------------------------------------------------------
// embedding with a scale and an added sinusoid: column 2i gets sin(p * f_i), column 2i+1
// cos(p * f_i); `freq` [ceil(hidden/2)] holds f_i in 64-bit (made on the host).  bfloat16
// tables take the angle in float32; the 32-bit path takes it in 64-bit.
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void embed_sinusoid_kernel(
    const T* __restrict__ table, const int* __restrict__ ids, const int* __restrict__ positions,
    const double* __restrict__ freq, float* __restrict__ residual, T* __restrict__ cast, int hidden, float scale) {
  using A = typename Wide<T>::type;
  const int t = blockIdx.x;
  // a thread takes a pair of columns (2j, 2j + 1): one angle, its sine and its cosine from one
  // range reduction; the blocks along y share a token's pairs
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  const int i = 2 * j;
  if (i >= hidden) return;
  const A angle = (A)positions[t] * (A)freq[j];
  A wave[2];
  if constexpr (sizeof(T) == 4) {
    wave[0] = sin(angle);
    wave[1] = cos(angle);
  } else {
    sincosf(angle, &wave[0], &wave[1]);
  }
  const T* row = table + (int64_t)ids[t] * hidden;
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    if (i + k >= hidden) break;  // (an odd width ends on a sine)
    const float v = (float)((A)to_f32(row[i + k]) * (A)scale + wave[k]);
    residual[(int64_t)t * hidden + i + k] = v;
    if (cast != nullptr) cast[(int64_t)t * hidden + i + k] = from_f32<T>(v);
  }
}

extern "C" int mi_embed_sinusoid(int dtype, const void* table, const int* ids, const int* positions,
                                 const double* freq, float* residual, void* cast, int num_tokens, int hidden,
                                 int vocab, float scale, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0, "embed_sinusoid: bad sizes tokens=%d hidden=%d vocab=%d",
             num_tokens, hidden, vocab);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "embed_sinusoid: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  MI_REQUIRE(ceil_div(hidden, 512) <= 65535, "embed_sinusoid: hidden=%d is too wide for one launch", hidden);
  const dim3 grid(num_tokens, ceil_div(ceil_div(hidden, 2), 256));
  if (dtype == MI_F32) {
    embed_sinusoid_kernel<float><<<grid, 256, 0, stream>>>((const float*)table, ids, positions, freq, residual,
                                                                 (float*)cast, hidden, scale);
  } else {
    embed_sinusoid_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)table, ids, positions, freq,
                                                                  residual, (bf16_t*)cast, hidden, scale);
  }
  MI_CHECK_LAUNCH("embed_sinusoid");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// The norm on a sublayer's output with the add folded in:
//   residual[t, c] += y[t, c] * rsqrt(mean_c(y[t]^2) + eps) * gain * scale[c]
// `gain` is one number or absent, `scale` one number per column or absent (both float32).
// With `cast`, the new residual row is also written in the element type, which is what the
// next sublayer's products read.  One block a row.
// ---------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(1024) void norm_scale_add_kernel(
    const T* __restrict__ y, int64_t y_stride, float* __restrict__ residual, const float* __restrict__ gain,
    const float* __restrict__ scale, T* __restrict__ cast, int hidden, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x;
  const T* row = y + (int64_t)t * y_stride;
  A squares = 0;
  for (int i = threadIdx.x * VEC; i < hidden; i += blockDim.x * VEC) {
    float v[VEC];
    if constexpr (VEC == 4) load4(row + i, v);
    else v[0] = to_f32(row[i]);
#pragma unroll
    for (int k = 0; k < VEC; ++k) squares += (A)v[k] * (A)v[k];
  }
  const A inv = inv_root(block_total<A>(squares, scratch) / (A)hidden, (A)eps);
  const A g = gain != nullptr ? (A)gain[0] : (A)1;
  float* res = residual + (int64_t)t * hidden;
  for (int i = threadIdx.x * VEC; i < hidden; i += blockDim.x * VEC) {
    float v[VEC], r[VEC], sc[VEC];
    if constexpr (VEC == 4) {
      load4(row + i, v);
      load4(res + i, r);
      if (scale != nullptr) load4(scale + i, sc);
    } else {
      v[0] = to_f32(row[i]);
      r[0] = res[i];
      if (scale != nullptr) sc[0] = scale[i];
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      A add = ((A)v[k] * inv) * g;
      if (scale != nullptr) add *= (A)sc[k];
      r[k] = (float)((A)r[k] + add);
    }
    if constexpr (VEC == 4) {
      store4(res + i, r);
      if (cast != nullptr) store4(cast + (int64_t)t * hidden + i, r);
    } else {
      res[i] = r[0];
      if (cast != nullptr) cast[(int64_t)t * hidden + i] = from_f32<T>(r[0]);
    }
  }
}

template <typename T>
static int norm_scale_add_launch(const void* y, int64_t y_stride, float* residual, const float* gain, const float* scale,
                                 void* cast, int num_tokens, int hidden, float eps, hipStream_t stream) {
  const bool vec = hidden % 4 == 0 && y_stride % 4 == 0 && aligned16(y) && aligned16(residual) && aligned16(scale) &&
                   aligned16(cast) && (sizeof(T) == 4 || y_stride % 8 == 0);
  const int threads = row_block(num_tokens, vec ? hidden / 4 : hidden);
  if (vec) {
    norm_scale_add_kernel<T, 4><<<num_tokens, threads, 0, stream>>>((const T*)y, y_stride, residual, gain, scale, (T*)cast,
                                                                hidden, eps);
  } else {
    norm_scale_add_kernel<T, 1><<<num_tokens, threads, 0, stream>>>((const T*)y, y_stride, residual, gain, scale, (T*)cast,
                                                                hidden, eps);
  }
  MI_CHECK_LAUNCH("norm_scale_add");
  return MI_OK;
}

extern "C" int mi_norm_scale_add(int dtype, const void* y, int64_t y_stride, float* residual, const float* gain,
                                 const float* scale, void* cast, int num_tokens, int hidden, float eps,
                                 hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && hidden > 0 && y_stride >= hidden, "norm_scale_add: bad sizes tokens=%d hidden=%d stride=%lld",
             num_tokens, hidden, (long long)y_stride);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "norm_scale_add: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  if (dtype == MI_F32) return norm_scale_add_launch<float>(y, y_stride, residual, gain, scale, cast, num_tokens, hidden, eps, stream);
  return norm_scale_add_launch<bf16_t>(y, y_stride, residual, gain, scale, cast, num_tokens, hidden, eps, stream);
}

// ---------------------------------------------------------------------------
// The float32 stream in bfloat16.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ in, bf16_t* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (bf16_t)in[i];
}

extern "C" int mi_cast_rows(const float* in, void* out, int64_t n, hipStream_t stream) {
  MI_REQUIRE(n >= 0, "cast_rows: bad size %lld", (long long)n);
  if (n == 0) return MI_OK;
  cast_rows_kernel<<<(unsigned)ceil_div64(n, 256), 256, 0, stream>>>(in, (bf16_t*)out, n);
  MI_CHECK_LAUNCH("cast_rows");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// minGRU.  Row t of `zxg` holds the three projections of the token [z | x | g], `width` each.
//   z = sigmoid(z_in + bz)          u = x_in + bx
//   cand = u + 1/2 (u >= 0), sigmoid(u) (u < 0)
//   S = (1 - z) * S + z * cand      out = S * silu(g)
// S is one float32 row per state slot; request b's row is state[slots[b]] (a slot outside
// 0..num_slots-1, the -1 of a padding row, means the spare row at index num_slots).  Request
// b owns rows cu[b]..cu[b+1]-1; a request without rows is left alone.
//
// Sequential form: one thread per (request, column) walks the request's rows.
// ---------------------------------------------------------------------------

template <typename A>
__device__ __forceinline__ void gru_gates(A z_in, A u, A& keep, A& add) {
  const A z = logistic(z_in);
  const A cand = u >= (A)0 ? u + (A)0.5 : logistic(u);
  keep = (A)1 - z;
  add = z * cand;
}

// VEC consecutive columns of a row, as float
template <typename T, int VEC>
__device__ __forceinline__ void load_cols(const T* p, float v[VEC]) {
  if constexpr (VEC == 4) load4(p, v);
  else v[0] = to_f32(p[0]);
}
template <typename T, int VEC>
__device__ __forceinline__ void store_cols(T* p, const float v[VEC]) {
  if constexpr (VEC == 4) store4(p, v);
  else p[0] = from_f32<T>(v[0]);
}

// One step of the recurrence for a thread's VEC columns of row `in`; with `out`, the gated
// output of the row is written.
template <typename T, int VEC, bool SUMMARY, typename A>
__device__ __forceinline__ void gru_row(const T* __restrict__ in, int width, int c, const A* bias_z, const A* bias_x,
                                        A* s, A* p, T* __restrict__ out) {
  float z_in[VEC], u[VEC], g[VEC], y[VEC];
  load_cols<T, VEC>(in + c, z_in);
  load_cols<T, VEC>(in + width + c, u);
  if constexpr (!SUMMARY) load_cols<T, VEC>(in + 2 * (int64_t)width + c, g);
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    A keep, add;
    gru_gates<A>((A)z_in[k] + bias_z[k], (A)u[k] + bias_x[k], keep, add);
    s[k] = fused_step(keep, s[k], add);
    if constexpr (SUMMARY) p[k] *= keep;
    else y[k] = (float)(s[k] * ((A)g[k] * logistic((A)g[k])));
  }
  if constexpr (!SUMMARY) store_cols<T, VEC>(out + c, y);
}

template <typename T, int VEC>
__global__ __launch_bounds__(64) void gated_scan_kernel(
    const T* __restrict__ zxg, int64_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
    float* __restrict__ state, int64_t state_stride, const int* __restrict__ cu, const int* __restrict__ slots,
    T* __restrict__ out, int64_t out_stride, int width, int num_slots) {
  using A = typename Wide<T>::type;
  const int b = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (c >= width) return;
  const int first = cu[b], last = cu[b + 1];
  if (last <= first) return;
  const int slot = slots[b];
  float* mine = state + ((slot < 0 || slot >= num_slots) ? num_slots : slot) * state_stride + c;
  A s[VEC], bias_z[VEC], bias_x[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    s[k] = (A)mine[k];
    bias_z[k] = (A)bz[c + k];
    bias_x[k] = (A)bx[c + k];
  }
#pragma unroll 4
  for (int t = first; t < last; ++t)
    gru_row<T, VEC, false, A>(zxg + (int64_t)t * in_stride, width, c, bias_z, bias_x, s, nullptr, out + (int64_t)t * out_stride);
#pragma unroll
  for (int k = 0; k < VEC; ++k) mine[k] = (float)s[k];
}

// Chunked form for long portions: the recurrence S' = keep * S + add is linear in S, so a
// chunk of rows acts on its incoming state as S_out = P * S_in + Q with P the product of its
// keeps and Q its result from a zero state.  Pass 1 computes (P, Q) of every chunk, pass 2
// walks each request's chunks in order and leaves every chunk's incoming state, pass 3 redoes
// every chunk from its incoming state and writes the outputs.  Chunks are cut per request
// at multiples of `chunk` rows from the request's first row of the step.
template <typename T, int VEC>
__global__ __launch_bounds__(64) void gated_scan_summaries_kernel(
    const T* __restrict__ zxg, int64_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
    const int* __restrict__ cu, float* __restrict__ summaries, int width, int chunk, int chunks_per_request) {
  using A = typename Wide<T>::type;
  const int b = blockIdx.z, k = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (c >= width) return;
  const int first = cu[b] + k * chunk, last = min(cu[b + 1], first + chunk);
  if (last <= first) return;
  A p[VEC], q[VEC], bias_z[VEC], bias_x[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    p[j] = 1;
    q[j] = 0;
    bias_z[j] = (A)bz[c + j];
    bias_x[j] = (A)bx[c + j];
  }
#pragma unroll 8
  for (int t = first; t < last; ++t)
    gru_row<T, VEC, true, A>(zxg + (int64_t)t * in_stride, width, c, bias_z, bias_x, q, p, nullptr);
  float* at = summaries + (((int64_t)b * chunks_per_request + k) * 2) * width;
  float pf[VEC], qf[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    pf[j] = (float)p[j];
    qf[j] = (float)q[j];
  }
  store_cols<float, VEC>(at + c, pf);
  store_cols<float, VEC>(at + width + c, qf);
}

// Pass 2: every chunk's (P, Q) is replaced by its incoming state (in Q's place); the request's
// state row receives the state after its last row.
__global__ __launch_bounds__(64) void gated_scan_carry_kernel(
    float* __restrict__ summaries, float* __restrict__ state, int64_t state_stride, const int* __restrict__ cu,
    const int* __restrict__ slots, int width, int chunk, int chunks_per_request, int num_slots) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int rows = cu[b + 1] - cu[b];
  if (rows <= 0) return;
  const int slot = slots[b];
  float* mine = state + ((slot < 0 || slot >= num_slots) ? num_slots : slot) * state_stride + c;
  const int chunks = (rows + chunk - 1) / chunk;
  float s = *mine;
#pragma unroll 8
  for (int k = 0; k < chunks; ++k) {
    float* at = summaries + (((int64_t)b * chunks_per_request + k) * 2) * width;
    const float p = at[c], q = at[width + c];
    at[width + c] = s;
    s = p * s + q;
  }
  *mine = s;
}

template <typename T, int VEC>
__global__ __launch_bounds__(64) void gated_scan_outputs_kernel(
    const T* __restrict__ zxg, int64_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
    const int* __restrict__ cu, const float* __restrict__ summaries, T* __restrict__ out, int64_t out_stride,
    int width, int chunk, int chunks_per_request) {
  using A = typename Wide<T>::type;
  const int b = blockIdx.z, k = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (c >= width) return;
  const int first = cu[b] + k * chunk, last = min(cu[b + 1], first + chunk);
  if (last <= first) return;
  A s[VEC], bias_z[VEC], bias_x[VEC];
  float incoming[VEC];
  load_cols<float, VEC>(summaries + (((int64_t)b * chunks_per_request + k) * 2 + 1) * width + c, incoming);
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    s[j] = (A)incoming[j];
    bias_z[j] = (A)bz[c + j];
    bias_x[j] = (A)bx[c + j];
  }
#pragma unroll 8
  for (int t = first; t < last; ++t)
    gru_row<T, VEC, false, A>(zxg + (int64_t)t * in_stride, width, c, bias_z, bias_x, s, nullptr, out + (int64_t)t * out_stride);
}

// The chunked form's passes 1 and 3 as tiles: a block of 256 threads owns 64 columns of one
// chunk (ROWS rows).  All threads load the chunk's [z | x | g] in whole 128-byte pieces and
// evaluate the gates of their elements at once (the exponentials are the arithmetic of this
// kernel); keep and add go to LDS, where one wave, a lane a column, walks the rows; then all
// threads multiply the states with silu(g), which they kept in registers, and store.  There is
// no launch between the two passes: a block of pass 3 composes the (P, Q) of the chunks before
// its own by itself (at most a few dozen steps on values that lie in the L2).  A thread
// that walked a column of a chunk by itself had at most 24 loads of 8 bytes in flight and
// the kernel ran at 0.7-1.2 TB/s.
constexpr int TILE_COLS = 64;
constexpr int TILE_PAD = 4;

template <typename T, int ROWS, bool SUMMARY>
__global__ __launch_bounds__(256) void gated_scan_tile_kernel(
    const T* __restrict__ zxg, int64_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
    const int* __restrict__ cu, float* __restrict__ summaries, T* __restrict__ out, int64_t out_stride, int width,
    int chunks_per_request, float* __restrict__ state, int64_t state_stride, const int* __restrict__ slots,
    int num_slots) {
  using A = typename Wide<T>::type;
  constexpr int PER_THREAD = ROWS / 16;  // rows of a thread: r0, r0 + 16, ...
  __shared__ A keep_s[ROWS][TILE_COLS + TILE_PAD];
  __shared__ A add_s[ROWS][TILE_COLS + TILE_PAD];
  const int b = blockIdx.z, k = blockIdx.y;
  const int c0 = blockIdx.x * TILE_COLS;
  const int first = cu[b] + k * ROWS;
  const int rows = min(cu[b + 1], first + ROWS) - first;
  if (rows <= 0) return;
  const int cg = (threadIdx.x % 16) * 4, r0 = threadIdx.x / 16;
  const int c = c0 + cg;
  const bool mine = c < width;
  float act[PER_THREAD][4];
  if (mine) {
    float bias_z[4], bias_x[4];
    load4(bz + c, bias_z);
    load4(bx + c, bias_x);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int r = r0 + 16 * i;
      if (r >= rows) break;
      const T* in = zxg + (int64_t)(first + r) * in_stride;
      float z_in[4], u[4], g[4];
      load4(in + c, z_in);
      load4(in + width + c, u);
      if constexpr (!SUMMARY) load4(in + 2 * (int64_t)width + c, g);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        A keep, add;
        gru_gates<A>((A)z_in[j] + (A)bias_z[j], (A)u[j] + (A)bias_x[j], keep, add);
        keep_s[r][cg + j] = keep;
        add_s[r][cg + j] = add;
        if constexpr (!SUMMARY) act[i][j] = (float)((A)g[j] * logistic((A)g[j]));
      }
    }
  }
  __syncthreads();
  // summaries of request b: entries 0..chunks-1 hold (P, Q) of its chunks, entry `chunks_per_request`
  // holds the state the request came with (copied by pass 1, so that no block of pass 3, where
  // the last chunk's block writes the new state, reads a state row)
  float* mine_s = summaries + ((int64_t)b * (chunks_per_request + 1) * 2) * width;
  if (threadIdx.x < TILE_COLS && c0 + (int)threadIdx.x < width) {
    const int col = threadIdx.x;
    const int slot = slots[b];
    float* row = state + ((slot < 0 || slot >= num_slots) ? num_slots : slot) * state_stride + c0 + col;
    if constexpr (SUMMARY) {
      A p = 1, q = 0;
#pragma unroll 8
      for (int r = 0; r < rows; ++r) {
        const A keep = keep_s[r][col];
        p *= keep;
        q = fused_step(keep, q, add_s[r][col]);
      }
      float* at = mine_s + (int64_t)k * 2 * width;
      at[c0 + col] = (float)p;
      at[width + c0 + col] = (float)q;
      if (k == 0) mine_s[(int64_t)chunks_per_request * 2 * width + c0 + col] = *row;
    } else {
      A s = (A)mine_s[(int64_t)chunks_per_request * 2 * width + c0 + col];
#pragma unroll 8
      for (int j = 0; j < k; ++j) {  // through the chunks before this one
        const float* at = mine_s + (int64_t)j * 2 * width;
        s = (A)at[c0 + col] * s + (A)at[width + c0 + col];
      }
#pragma unroll 8
      for (int r = 0; r < rows; ++r) {
        s = fused_step(keep_s[r][col], s, add_s[r][col]);
        add_s[r][col] = s;
      }
      if (first + rows == cu[b + 1]) *row = (float)s;  // the request's last chunk of this step
    }
  }
  if constexpr (!SUMMARY) {
    __syncthreads();
    if (!mine) return;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int r = r0 + 16 * i;
      if (r >= rows) break;
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = (float)(add_s[r][cg + j] * (A)act[i][j]);
      store4(out + (int64_t)(first + r) * out_stride + c, y);
    }
  }
}

template <typename T>
constexpr int tile_rows() {
  return sizeof(T) == 4 ? 32 : 64;  // (keep and add of a tile in 64-bit fill the LDS a block may have at 32 rows)
}

template <typename T>
static int gated_scan_tiles_launch(const void* zxg, int64_t in_stride, const float* bz, const float* bx, float* state,
                                   int64_t state_stride, const int* cu, const int* slots, void* out, int64_t out_stride,
                                   int num_requests, int width, int num_slots, int chunks_per_request, float* summaries,
                                   hipStream_t stream) {
  constexpr int ROWS = tile_rows<T>();
  dim3 grid(ceil_div(width, TILE_COLS), chunks_per_request, num_requests);
  gated_scan_tile_kernel<T, ROWS, true><<<grid, 256, 0, stream>>>((const T*)zxg, in_stride, bz, bx, cu, summaries, nullptr,
                                                                  0, width, chunks_per_request, state, state_stride, slots,
                                                                  num_slots);
  MI_CHECK_LAUNCH("gated_scan (tile summaries)");
  gated_scan_tile_kernel<T, ROWS, false><<<grid, 256, 0, stream>>>((const T*)zxg, in_stride, bz, bx, cu, summaries, (T*)out,
                                                                   out_stride, width, chunks_per_request, state,
                                                                   state_stride, slots, num_slots);
  MI_CHECK_LAUNCH("gated_scan (tile outputs)");
  return MI_OK;
}

extern "C" int mi_gated_scan_tile_rows(int dtype) { return dtype == MI_F32 ? tile_rows<float>() : tile_rows<bf16_t>(); }

template <typename T, int VEC>
static int gated_scan_launch(const void* zxg, int64_t in_stride, const float* bz, const float* bx, float* state,
                             int64_t state_stride, const int* cu, const int* slots, void* out, int64_t out_stride,
                             int num_requests, int width, int num_slots, int chunk, int chunks_per_request,
                             float* summaries, hipStream_t stream) {
  const int col_blocks = ceil_div(ceil_div(width, VEC), 64);
  if (chunk <= 0) {
    dim3 grid(col_blocks, num_requests);
    gated_scan_kernel<T, VEC><<<grid, 64, 0, stream>>>((const T*)zxg, in_stride, bz, bx, state, state_stride, cu, slots,
                                                       (T*)out, out_stride, width, num_slots);
    MI_CHECK_LAUNCH("gated_scan");
    return MI_OK;
  }
  dim3 grid(col_blocks, chunks_per_request, num_requests);
  gated_scan_summaries_kernel<T, VEC><<<grid, 64, 0, stream>>>((const T*)zxg, in_stride, bz, bx, cu, summaries, width,
                                                               chunk, chunks_per_request);
  MI_CHECK_LAUNCH("gated_scan (summaries)");
  gated_scan_carry_kernel<<<dim3(ceil_div(width, 64), num_requests), 64, 0, stream>>>(
      summaries, state, state_stride, cu, slots, width, chunk, chunks_per_request, num_slots);
  MI_CHECK_LAUNCH("gated_scan (carry)");
  gated_scan_outputs_kernel<T, VEC><<<grid, 64, 0, stream>>>((const T*)zxg, in_stride, bz, bx, cu, summaries, (T*)out,
                                                             out_stride, width, chunk, chunks_per_request);
  MI_CHECK_LAUNCH("gated_scan (outputs)");
  return MI_OK;
}

// `chunk` = 0: the sequential form.  `chunk` > 0: the chunked form; no request may bring more
// than chunk * chunks_per_request rows (the caller's bound), and `summaries` holds
// num_requests * (chunks_per_request + 1) * 2 * width floats.  `state_stride`: floats between the
// state rows of two slots.
extern "C" int mi_gated_scan(int dtype, const void* zxg, int64_t in_stride, const float* bz, const float* bx,
                             float* state, int64_t state_stride, const int* cu, const int* slots, void* out,
                             int64_t out_stride, int num_requests, int width, int num_slots, int chunk,
                             int chunks_per_request, float* summaries, hipStream_t stream) {
  MI_REQUIRE(num_requests >= 0 && width > 0 && num_slots >= 0, "gated_scan: bad sizes requests=%d width=%d slots=%d",
             num_requests, width, num_slots);
  MI_REQUIRE(in_stride >= 3 * (int64_t)width && out_stride >= width && state_stride >= width,
             "gated_scan: rows hold [z | x | g], %d each", width);
  MI_REQUIRE(chunk >= 0 && (chunk == 0 || (chunks_per_request > 0 && summaries != nullptr)),
             "gated_scan: the chunked form needs a chunk count and a summaries buffer");
  MI_REQUIRE(num_requests <= 65535 && chunks_per_request <= 65535, "gated_scan: too many requests or chunks for one launch");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "gated_scan: unknown dtype %d", dtype);
  if (num_requests == 0) return MI_OK;
  const int64_t step = dtype == MI_F32 ? 4 : 8;  // elements of a 16-byte boundary
  const bool vec = width % 4 == 0 && in_stride % step == 0 && out_stride % step == 0 && width % step == 0 &&
                   aligned16(zxg) && aligned16(out) && aligned16(summaries);
  if (vec && aligned16(bz) && aligned16(bx) && chunk > 0 && chunk == mi_gated_scan_tile_rows(dtype)) {
    if (dtype == MI_F32)
      return gated_scan_tiles_launch<float>(zxg, in_stride, bz, bx, state, state_stride, cu, slots, out, out_stride,
                                            num_requests, width, num_slots, chunks_per_request, summaries, stream);
    return gated_scan_tiles_launch<bf16_t>(zxg, in_stride, bz, bx, state, state_stride, cu, slots, out, out_stride,
                                           num_requests, width, num_slots, chunks_per_request, summaries, stream);
  }
#define MI_SCAN(T, VEC)                                                                                              \
  return gated_scan_launch<T, VEC>(zxg, in_stride, bz, bx, state, state_stride, cu, slots, out, out_stride,           \
                                   num_requests, width, num_slots, chunk, chunks_per_request, summaries, stream)
  if (dtype == MI_F32) {
    if (vec) MI_SCAN(float, 4);
    MI_SCAN(float, 1);
  }
  if (vec) MI_SCAN(bf16_t, 4);
  MI_SCAN(bf16_t, 1);
#undef MI_SCAN
}

// ---------------------------------------------------------------------------
// q and k normed over their whole projection, and the cache write.
//   row layout of qk: [q: q_width | k: kv_heads * head_dim]
//   q <- q * rsqrt(mean(q^2) + eps) * qw      (in place)
//   key page slot   <- k * rsqrt(mean(k^2) + eps) * kw
//   value page slot <- k as it came           (the values are the keys before their norm)
// Page layouts and slot numbering are those of rope_kv_write.  kv_heads = 0: q only.
// ---------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(1024) void qk_norm_kv_write_kernel(
    T* __restrict__ qk, int64_t row_stride, const float* __restrict__ qw, const float* __restrict__ kw,
    const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages, int q_width,
    int kv_heads, int head_dim, int page_size, int v_transposed, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x;
  T* row = qk + (int64_t)t * row_stride;
  const int k_width = kv_heads * head_dim;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;
  A q_squares = 0, k_squares = 0;
  for (int i = first; i < q_width; i += stride) {
    float v[VEC];
    load_cols<T, VEC>(row + i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) q_squares += (A)v[j] * (A)v[j];
  }
  for (int i = first; i < k_width; i += stride) {
    float v[VEC];
    load_cols<T, VEC>(row + q_width + i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) k_squares += (A)v[j] * (A)v[j];
  }
  const A q_inv = inv_root(block_total<A>(q_squares, scratch) / (A)q_width, (A)eps);
  const bool writes = k_width > 0 && slot_mapping != nullptr;
  const A k_inv = writes ? inv_root(block_total<A>(k_squares, scratch) / (A)k_width, (A)eps) : (A)0;
  for (int i = first; i < q_width; i += stride) {
    float v[VEC], w[VEC];
    load_cols<T, VEC>(row + i, v);
    load_cols<float, VEC>(qw + i, w);
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = (float)(((A)v[j] * q_inv) * (A)w[j]);
    store_cols<T, VEC>(row + i, v);
  }
  if (!writes) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  for (int e = first; e < k_width; e += stride) {
    const int h = e / head_dim, d = e % head_dim;  // (VEC divides head_dim: the VEC values lie in one head)
    float raw[VEC], w[VEC], normed[VEC];
    load_cols<T, VEC>(row + q_width + e, raw);
    load_cols<float, VEC>(kw + e, w);
#pragma unroll
    for (int j = 0; j < VEC; ++j) normed[j] = (float)(((A)raw[j] * k_inv) * (A)w[j]);
    const int64_t chunk = ((int64_t)page * kv_heads + h) * page_size * head_dim;
    store_cols<T, VEC>(k_pages + chunk + (int64_t)off * head_dim + d, normed);
    if (v_transposed) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v_pages[chunk + (int64_t)(d + j) * page_size + off] = from_f32<T>(raw[j]);
    } else {
      store_cols<T, VEC>(v_pages + chunk + (int64_t)off * head_dim + d, raw);
    }
  }
}

extern "C" int mi_qk_norm_kv_write(int dtype, void* qk, int64_t row_stride, const float* qw, const float* kw,
                                   const int* slot_mapping, void* k_pages, void* v_pages, int num_tokens, int q_width,
                                   int kv_heads, int head_dim, int page_size, int num_pages, int v_transposed,
                                   float eps, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && q_width > 0 && kv_heads >= 0 && head_dim > 0,
             "qk_norm_kv_write: bad sizes tokens=%d q_width=%d kv_heads=%d head_dim=%d", num_tokens, q_width, kv_heads,
             head_dim);
  MI_REQUIRE(row_stride >= (int64_t)q_width + (int64_t)kv_heads * head_dim,
             "qk_norm_kv_write: row stride %lld is shorter than q and k together", (long long)row_stride);
  MI_REQUIRE(kv_heads == 0 || slot_mapping == nullptr || (page_size > 0 && num_pages > 0 && k_pages && v_pages && kw),
             "qk_norm_kv_write: pages and the key norm's weight are needed to write keys and values");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "qk_norm_kv_write: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int64_t step = dtype == MI_F32 ? 4 : 8;
  const bool vec = q_width % step == 0 && head_dim % step == 0 && row_stride % step == 0 && aligned16(qk) && aligned16(qw) &&
                   aligned16(kw) && aligned16(k_pages) && aligned16(v_pages);
  const int threads = row_block(num_tokens, (q_width + kv_heads * head_dim) / (vec ? 4 : 1));
#define MI_QK(T, VEC)                                                                                               \
  qk_norm_kv_write_kernel<T, VEC><<<num_tokens, threads, 0, stream>>>((T*)qk, row_stride, qw, kw, slot_mapping,      \
                                                                      (T*)k_pages, (T*)v_pages, q_width, kv_heads,   \
                                                                      head_dim, page_size, v_transposed, eps)
  if (dtype == MI_F32) {
    if (vec) MI_QK(float, 4);
    else MI_QK(float, 1);
  } else {
    if (vec) MI_QK(bf16_t, 4);
    else MI_QK(bf16_t, 1);
  }
#undef MI_QK
  MI_CHECK_LAUNCH("qk_norm_kv_write");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// The same with values of their own: row layout [q: q_width | k: kv_heads * head_dim | v: kv_heads * v_dim].
//   q <- q * rsqrt(mean(q^2) + eps) * qw      (in place)
//   key page slot   <- k * rsqrt(mean(k^2) + eps) * kw
//   value page slot <- v, or (1 - mix) * v + mix * other[t] where another layer's values of the
//                      same tokens are given (`other` [tokens, kv_heads * v_dim], `mix` one float32)
// kv_heads = 0 or no slots: q only.
// ---------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(1024) void qkv_norm_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ qw, const float* __restrict__ kw,
    const T* __restrict__ other, int64_t other_stride, const float* __restrict__ mix,
    const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages, int q_width,
    int kv_heads, int head_dim, int v_dim, int page_size, int v_transposed, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x;
  T* row = qkv + (int64_t)t * row_stride;
  const int k_width = kv_heads * head_dim, v_width = kv_heads * v_dim;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;
  A q_squares = 0, k_squares = 0;
  for (int i = first; i < q_width; i += stride) {
    float v[VEC];
    load_cols<T, VEC>(row + i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) q_squares += (A)v[j] * (A)v[j];
  }
  for (int i = first; i < k_width; i += stride) {
    float v[VEC];
    load_cols<T, VEC>(row + q_width + i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) k_squares += (A)v[j] * (A)v[j];
  }
  const A q_inv = inv_root(block_total<A>(q_squares, scratch) / (A)q_width, (A)eps);
  const bool writes = k_width > 0 && slot_mapping != nullptr;
  const A k_inv = writes ? inv_root(block_total<A>(k_squares, scratch) / (A)k_width, (A)eps) : (A)0;
  for (int i = first; i < q_width; i += stride) {
    float v[VEC], w[VEC];
    load_cols<T, VEC>(row + i, v);
    load_cols<float, VEC>(qw + i, w);
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = (float)(((A)v[j] * q_inv) * (A)w[j]);
    store_cols<T, VEC>(row + i, v);
  }
  if (!writes) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  for (int e = first; e < k_width; e += stride) {
    const int h = e / head_dim, d = e % head_dim;  // (VEC divides head_dim: the VEC values lie in one head)
    float raw[VEC], w[VEC];
    load_cols<T, VEC>(row + q_width + e, raw);
    load_cols<float, VEC>(kw + e, w);
#pragma unroll
    for (int j = 0; j < VEC; ++j) raw[j] = (float)(((A)raw[j] * k_inv) * (A)w[j]);
    store_cols<T, VEC>(k_pages + (((int64_t)page * kv_heads + h) * page_size + off) * head_dim + d, raw);
  }
  const A lam = (other != nullptr) ? (A)mix[0] : (A)0;
  for (int e = first; e < v_width; e += stride) {
    const int h = e / v_dim, d = e % v_dim;  // (VEC divides v_dim)
    float val[VEC];
    load_cols<T, VEC>(row + q_width + k_width + e, val);
    if (other != nullptr) {
      float first_val[VEC];
      load_cols<T, VEC>(other + (int64_t)t * other_stride + e, first_val);
#pragma unroll
      for (int j = 0; j < VEC; ++j) val[j] = (float)(((A)1 - lam) * (A)val[j] + lam * (A)first_val[j]);
    }
    const int64_t chunk = ((int64_t)page * kv_heads + h) * page_size * v_dim;
    if (v_transposed) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v_pages[chunk + (int64_t)(d + j) * page_size + off] = from_f32<T>(val[j]);
    } else {
      store_cols<T, VEC>(v_pages + chunk + (int64_t)off * v_dim + d, val);
    }
  }
}

extern "C" int mi_qkv_norm_write(int dtype, void* qkv, int64_t row_stride, const float* qw, const float* kw,
                                 const void* other, int64_t other_stride, const float* mix, const int* slot_mapping,
                                 void* k_pages, void* v_pages, int num_tokens, int q_width, int kv_heads, int head_dim,
                                 int v_dim, int page_size, int num_pages, int v_transposed, float eps,
                                 hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && q_width > 0 && kv_heads >= 0 && head_dim > 0 && v_dim > 0,
             "qkv_norm_write: bad sizes tokens=%d q_width=%d kv_heads=%d head_dim=%d v_dim=%d", num_tokens, q_width, kv_heads,
             head_dim, v_dim);
  MI_REQUIRE(row_stride >= (int64_t)q_width + (int64_t)kv_heads * (head_dim + v_dim),
             "qkv_norm_write: row stride %lld is shorter than q, k and v together", (long long)row_stride);
  MI_REQUIRE(kv_heads == 0 || slot_mapping == nullptr || (page_size > 0 && num_pages > 0 && k_pages && v_pages && kw),
             "qkv_norm_write: pages and the key norm's weight are needed to write keys and values");
  MI_REQUIRE(other == nullptr || (mix != nullptr && other_stride >= (int64_t)kv_heads * v_dim),
             "qkv_norm_write: values to mix in come with their weight and rows at least as wide as the values");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "qkv_norm_write: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int64_t step = dtype == MI_F32 ? 4 : 8;
  const bool vec = q_width % step == 0 && head_dim % step == 0 && v_dim % step == 0 && row_stride % step == 0 &&
                   other_stride % step == 0 && aligned16(qkv) && aligned16(qw) && aligned16(kw) && aligned16(other) &&
                   aligned16(k_pages) && aligned16(v_pages);
  const int threads = row_block(num_tokens, (q_width + kv_heads * (head_dim + v_dim)) / (vec ? 4 : 1));
#define MI_QKV(T, VEC)                                                                                              \
  qkv_norm_write_kernel<T, VEC><<<num_tokens, threads, 0, stream>>>(                                                \
      (T*)qkv, row_stride, qw, kw, (const T*)other, other_stride, mix, slot_mapping, (T*)k_pages, (T*)v_pages,      \
      q_width, kv_heads, head_dim, v_dim, page_size, v_transposed, eps)
  if (dtype == MI_F32) {
    if (vec) MI_QKV(float, 4);
    else MI_QKV(float, 1);
  } else {
    if (vec) MI_QKV(bf16_t, 4);
    else MI_QKV(bf16_t, 1);
  }
#undef MI_QKV
  MI_CHECK_LAUNCH("qkv_norm_write");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// PolyNorm over a token's feed-forward values z [width]:
//   out = a * z / rms(z) + b * z^2 / rms(z^2) + c * z^3 / rms(z^3) + e,   rms(v) = sqrt(mean(v^2) + eps)
// `coef` = (a, b, c, e) float32.  One block a row.
// ---------------------------------------------------------------------------

template <typename T, int VEC>
__global__ __launch_bounds__(1024) void poly_norm_kernel(const T* __restrict__ z, int64_t in_stride,
                                                        const float* __restrict__ coef, T* __restrict__ out,
                                                        int64_t out_stride, int width, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x;
  const T* row = z + (int64_t)t * in_stride;
  A s2 = 0, s4 = 0, s6 = 0;
  for (int i = threadIdx.x * VEC; i < width; i += blockDim.x * VEC) {
    float x[VEC];
    if constexpr (VEC == 4) load4(row + i, x);
    else x[0] = to_f32(row[i]);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const A v2 = (A)x[k] * (A)x[k];
      s2 += v2;
      s4 += v2 * v2;
      s6 += v2 * v2 * v2;
    }
  }
  const A n = (A)width;
  const A i1 = inv_root(block_total<A>(s2, scratch) / n, (A)eps);
  const A i2 = inv_root(block_total<A>(s4, scratch) / n, (A)eps);
  const A i3 = inv_root(block_total<A>(s6, scratch) / n, (A)eps);
  const A a = (A)coef[0] * i1, b = (A)coef[1] * i2, c = (A)coef[2] * i3, e = (A)coef[3];
  for (int i = threadIdx.x * VEC; i < width; i += blockDim.x * VEC) {
    float x[VEC];
    if constexpr (VEC == 4) load4(row + i, x);
    else x[0] = to_f32(row[i]);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const A v = (A)x[k], v2 = v * v;
      x[k] = (float)(a * v + b * v2 + c * (v2 * v) + e);
    }
    if constexpr (VEC == 4) store4(out + (int64_t)t * out_stride + i, x);
    else out[(int64_t)t * out_stride + i] = from_f32<T>(x[0]);
  }
}

template <typename T>
static int poly_norm_launch(const void* z, int64_t in_stride, const float* coef, void* out, int64_t out_stride,
                            int num_tokens, int width, float eps, hipStream_t stream) {
  const int64_t step = sizeof(T) == 4 ? 4 : 8;
  const bool vec = width % 4 == 0 && in_stride % step == 0 && out_stride % step == 0 && aligned16(z) && aligned16(out);
  const int threads = row_block(num_tokens, vec ? width / 4 : width);
  if (vec) {
    poly_norm_kernel<T, 4><<<num_tokens, threads, 0, stream>>>((const T*)z, in_stride, coef, (T*)out, out_stride, width, eps);
  } else {
    poly_norm_kernel<T, 1><<<num_tokens, threads, 0, stream>>>((const T*)z, in_stride, coef, (T*)out, out_stride, width, eps);
  }
  MI_CHECK_LAUNCH("poly_norm");
  return MI_OK;
}

extern "C" int mi_poly_norm(int dtype, const void* z, int64_t in_stride, const float* coef, void* out,
                            int64_t out_stride, int num_tokens, int width, float eps, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && in_stride >= width && out_stride >= width,
             "poly_norm: bad sizes tokens=%d width=%d", num_tokens, width);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "poly_norm: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  if (dtype == MI_F32) return poly_norm_launch<float>(z, in_stride, coef, out, out_stride, num_tokens, width, eps, stream);
  return poly_norm_launch<bf16_t>(z, in_stride, coef, out, out_stride, num_tokens, width, eps, stream);
}

// ---------------------------------------------------------------------------
// out[t, j] = gelu_tanh(gate[t, j]) * table[ids[t], first_col + j],  j < width
//   gelu_tanh(z) = z/2 * (1 + tanh(sqrt(2/pi) * (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void gated_table_rows_kernel(
    const T* __restrict__ gate, int64_t gate_stride, const T* __restrict__ table, int64_t table_stride,
    const int* __restrict__ ids, T* __restrict__ out, int width, int first_col, int64_t total) {
  using A = typename Wide<T>::type;
  const int64_t at = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const int64_t t = at / width;
  const int j = (int)(at % width);
  const A z = (A)to_f32(gate[t * gate_stride + j]);
  const A inner = (A)0.7978845608028654 * (z + (A)0.044715 * z * z * z);
  const A act = (A)0.5 * z * ((A)1 + tanh_of(inner));
  const A e = (A)to_f32(table[(int64_t)ids[t] * table_stride + first_col + j]);
  out[at] = from_f32<T>((float)(act * e));
}

extern "C" int mi_gated_table_rows(int dtype, const void* gate, int64_t gate_stride, const void* table,
                                   int64_t table_stride, const int* ids, void* out, int num_tokens, int width,
                                   int first_col, int vocab, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && first_col >= 0 && vocab > 0 && gate_stride >= width &&
                 table_stride >= (int64_t)first_col + width,
             "gated_table_rows: bad sizes tokens=%d width=%d first_col=%d", num_tokens, width, first_col);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "gated_table_rows: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int64_t total = (int64_t)num_tokens * width;
  const unsigned blocks = (unsigned)ceil_div64(total, 256);
  if (dtype == MI_F32) {
    gated_table_rows_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate, gate_stride, (const float*)table,
                                                               table_stride, ids, (float*)out, width, first_col, total);
  } else {
    gated_table_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gate, gate_stride, (const bf16_t*)table,
                                                                table_stride, ids, (bf16_t*)out, width, first_col, total);
  }
  MI_CHECK_LAUNCH("gated_table_rows");
  return MI_OK;
}
