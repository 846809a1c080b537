// What stands between the projections of a latent attention layer and its attention.
//
// Such a layer keeps ONE small row per token for all heads: a latent c (RMS-normed) from
// which every head's keys and values are linear maps, and a rotated part r that all heads
// share.  With the key map folded into the query (q' = W_uk^T q per head) a head's score is
// q' . c + q_rot . r: attention with a single key/value head whose key row is [c | r] and
// whose value row is c itself, the value map applied to the attention's output afterwards.
//
//   latent_prepare   per token: c = x_c / sqrt(mean(x_c^2) + eps) * weight and the rotated r go
//                    into the token's slot of the key pages as one row [c | r]; each head's
//                    rotated query part goes behind that head's folded part in the query rows
//                    the attention reads ([head][rank + rot]).
//
// Rotation pairs entry 2i with 2i+1; cos and sin come as float32 tables [tokens, rot/2].
#include "common.h"

#include <math.h>

namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_col, int q_head_width, int q_rot_at, int c_col,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const float* __restrict__ norm_weight,
    const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ queries, int64_t queries_stride,
    T* __restrict__ latent_out, int heads, int rank, int rot, float eps, const T* __restrict__ down,
    int64_t down_stride) {
  __shared__ float scratch[4];
  __shared__ double scratch_wide[4];
  constexpr bool WIDE = sizeof(T) == 4;
  const int t = blockIdx.x;
  const int half = rot / 2;
  const T* row = proj + (int64_t)t * proj_stride;
  const float* c = cos_t + (int64_t)t * half;
  const float* s = sin_t + (int64_t)t * half;
  const int width = rank + rot;

  auto turn = [&](float x0, float x1, int i, float& y0, float& y1) {
    if constexpr (WIDE) {
      y0 = (float)((double)x0 * c[i] - (double)x1 * s[i]);
      y1 = (float)((double)x1 * c[i] + (double)x0 * s[i]);
    } else {
      y0 = x0 * c[i] - x1 * s[i];
      y1 = x1 * c[i] + x0 * s[i];
    }
  };

  T* q_out = queries + (int64_t)t * queries_stride;
  for (int e = threadIdx.x; queries != nullptr && e < heads * half; e += blockDim.x) {
    const int h = e / half, i = e % half;
    const T* x = row + q_col + h * q_head_width + q_rot_at;
    float y0, y1;
    turn(to_f32(x[2 * i]), to_f32(x[2 * i + 1]), i, y0, y1);
    T* dst = q_out + (int64_t)h * width + rank;
    dst[2 * i] = from_f32<T>(y0);
    dst[2 * i + 1] = from_f32<T>(y1);
  }

  const int slot = slot_mapping != nullptr ? slot_mapping[t] : -1;
  if (slot < 0 && latent_out == nullptr) return;  // (the whole block leaves together)
  // ([x_c | x_r] lie in `proj`'s rows, or in rows of their own where the queries come from a product of their own)
  const T* x = (down != nullptr ? down + (int64_t)t * down_stride : row) + c_col;
  float squares = 0.f;
  double squares_wide = 0.0;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    const float v = to_f32(x[d]);
    if constexpr (WIDE) squares_wide += (double)v * v;
    else squares += v * v;
  }
  T* dst = slot >= 0 ? k_pages + (int64_t)slot * width : nullptr;
  T* copy = latent_out ? latent_out + (int64_t)t * rank : nullptr;
  if constexpr (WIDE) {
    // (a fixed order: lanes by butterfly, waves one after another)
#pragma unroll
    for (int off = MI_WAVE / 2; off > 0; off >>= 1) squares_wide += __shfl_xor(squares_wide, off, MI_WAVE);
    if (threadIdx.x % MI_WAVE == 0) scratch_wide[threadIdx.x / MI_WAVE] = squares_wide;
    __syncthreads();
    double total = 0.0;
    for (int w = 0; w < (int)blockDim.x / MI_WAVE; ++w) total += scratch_wide[w];
    const double inv = 1.0 / sqrt(total / (double)rank + (double)eps);
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
      const float c_d = (float)((double)x[d] * inv * (double)norm_weight[d]);
      if (dst) dst[d] = c_d;
      if (copy) copy[d] = c_d;
    }
  } else {
    const float inv = rsqrtf(block_sum(squares, scratch) / (float)rank + eps);
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
      const T c_d = from_f32<T>(to_f32(x[d]) * inv * norm_weight[d]);
      if (dst) dst[d] = c_d;
      if (copy) copy[d] = c_d;
    }
  }
  for (int i = threadIdx.x; dst != nullptr && i < half; i += blockDim.x) {
    float y0, y1;
    turn(to_f32(x[rank + 2 * i]), to_f32(x[rank + 2 * i + 1]), i, y0, y1);
    dst[rank + 2 * i] = from_f32<T>(y0);
    dst[rank + 2 * i + 1] = from_f32<T>(y1);
  }
}

// Keys and values written out per head, for a prompt that is in the step from its first token:
// one row [q | k | v] per token with heads of D = dim + rot columns each,
//   q head: [query's plain part | its rotated part]      k head: [W_uk c | rotated shared part]
//   v head: [W_uv c | zeros up to D]
// which the paged attention kernels take like any other stacked projection.
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_head_width, int q_rot_at, int r_col,
    const T* __restrict__ k_up, int64_t k_up_stride, const T* __restrict__ v_up, int64_t v_up_stride,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, T* __restrict__ qkv, int64_t qkv_stride, int heads,
    int dim, int rot, int vdim, const T* __restrict__ down, int64_t down_stride) {
  const int t = blockIdx.x;
  const int half = rot / 2, D = dim + rot;
  const T* row = proj + (int64_t)t * proj_stride;
  const float* c = cos_t + (int64_t)t * half;
  const float* s = sin_t + (int64_t)t * half;
  T* out = qkv + (int64_t)t * qkv_stride;
  const T* ku = k_up + (int64_t)t * k_up_stride;
  const T* vu = v_up + (int64_t)t * v_up_stride;
  for (int e = threadIdx.x; e < heads * D; e += blockDim.x) {
    const int h = e / D, d = e % D;
    T qv, kv;
    if (d < dim) {
      qv = row[h * q_head_width + d];  // (plain parts lie in front of a query head: q_rot_at == dim)
      kv = ku[h * dim + d];
    } else {
      const int i = (d - dim) / 2, odd = (d - dim) & 1;
      const T* qx = row + h * q_head_width + q_rot_at + 2 * i;
      const T* kx = (down != nullptr ? down + (int64_t)t * down_stride : row) + r_col + 2 * i;
      const float q0 = to_f32(qx[0]), q1 = to_f32(qx[1]), k0 = to_f32(kx[0]), k1 = to_f32(kx[1]);
      qv = from_f32<T>(odd ? q1 * c[i] + q0 * s[i] : q0 * c[i] - q1 * s[i]);
      kv = from_f32<T>(odd ? k1 * c[i] + k0 * s[i] : k0 * c[i] - k1 * s[i]);
    }
    out[e] = qv;
    out[(int64_t)heads * D + e] = kv;
    out[2 * (int64_t)heads * D + e] = d < vdim ? vu[h * vdim + d] : from_f32<T>(0.f);
  }
}

}  // namespace

extern "C" int mi_latent_expand(int dtype, const void* proj, int64_t proj_stride, int q_head_width, int q_rot_at, int r_col,
                                const void* k_up, int64_t k_up_stride, const void* v_up, int64_t v_up_stride,
                                const float* cos_t, const float* sin_t, void* qkv, int64_t qkv_stride, int num_tokens,
                                int heads, int dim, int rot, int vdim, const void* down, int64_t down_stride,
                                hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && heads > 0 && dim > 0 && rot >= 0 && rot % 2 == 0 && vdim > 0 && vdim <= dim + rot,
             "latent_expand: bad sizes tokens=%d heads=%d dim=%d rot=%d vdim=%d", num_tokens, heads, dim, rot, vdim);
  MI_REQUIRE(q_rot_at == dim && q_head_width >= dim + rot, "latent_expand: a query head is [plain (dim) | to rotate (rot)]");
  MI_REQUIRE(proj_stride >= (int64_t)heads * q_head_width && (down != nullptr ? down_stride : proj_stride) >= r_col + (int64_t)rot && r_col >= 0 &&
                 k_up_stride >= (int64_t)heads * dim && v_up_stride >= (int64_t)heads * vdim &&
                 qkv_stride >= 3 * (int64_t)heads * (dim + rot),
             "latent_expand: row strides shorter than a row");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "latent_expand: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  if (dtype == MI_F32)
    latent_expand_kernel<float><<<num_tokens, 256, 0, stream>>>(
        (const float*)proj, proj_stride, q_head_width, q_rot_at, r_col, (const float*)k_up, k_up_stride, (const float*)v_up,
        v_up_stride, cos_t, sin_t, (float*)qkv, qkv_stride, heads, dim, rot, vdim, (const float*)down, down_stride);
  else
    latent_expand_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(
        (const bf16_t*)proj, proj_stride, q_head_width, q_rot_at, r_col, (const bf16_t*)k_up, k_up_stride,
        (const bf16_t*)v_up, v_up_stride, cos_t, sin_t, (bf16_t*)qkv, qkv_stride, heads, dim, rot, vdim, (const bf16_t*)down,
        down_stride);
  MI_CHECK_LAUNCH("latent_expand");
  return MI_OK;
}

// proj: rows that hold the query projection (heads of q_head_width columns from q_col on, the
// part to rotate rot columns wide from q_rot_at inside a head) and, from c_col on, [x_c (rank) |
// x_r (rot)].  k_pages: [num_pages * page_size][rank + rot] (one key head); slot_mapping may be
// null (nothing is written: a call that reads another's pages).  queries: [tokens, heads * (rank
// + rot)] (row stride) or null; only the last rot columns of every head are written here.
// latent_out: [tokens, rank] or null, a copy of the normed latents.  down (may be null): rows of their own
// that hold [x_c | x_r] from c_col on, where the queries come from a product of their own.
extern "C" int mi_latent_prepare(int dtype, const void* proj, int64_t proj_stride, int q_col, int q_head_width,
                                 int q_rot_at, int c_col, const float* cos_t, const float* sin_t,
                                 const float* norm_weight, const int* slot_mapping, void* k_pages, void* queries,
                                 int64_t queries_stride, void* latent_out, int num_tokens, int heads, int rank, int rot,
                                 float eps, const void* down, int64_t down_stride, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && heads > 0 && rank > 0 && rot >= 0 && rot % 2 == 0,
             "latent_prepare: bad sizes tokens=%d heads=%d rank=%d rot=%d", num_tokens, heads, rank, rot);
  MI_REQUIRE(q_rot_at >= 0 && q_rot_at + rot <= q_head_width, "latent_prepare: the rotated part lies outside a query head");
  MI_REQUIRE(q_col >= 0 && c_col >= 0 && proj_stride >= q_col + (int64_t)heads * q_head_width &&
                 (down != nullptr ? down_stride : proj_stride) >= c_col + (int64_t)rank + rot,
             "latent_prepare: columns outside a row of the projections");
  MI_REQUIRE(queries == nullptr || queries_stride >= (int64_t)heads * (rank + rot),
             "latent_prepare: query rows shorter than heads * (rank + rot)");
  MI_REQUIRE(slot_mapping == nullptr || k_pages != nullptr, "latent_prepare: pages are needed to write keys");
  MI_REQUIRE(eps > 0.f, "latent_prepare: eps must be positive, got %g", (double)eps);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "latent_prepare: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  if (dtype == MI_F32)
    latent_prepare_kernel<float><<<num_tokens, 256, 0, stream>>>(
        (const float*)proj, proj_stride, q_col, q_head_width, q_rot_at, c_col, cos_t, sin_t, norm_weight, slot_mapping,
        (float*)k_pages, (float*)queries, queries_stride, (float*)latent_out, heads, rank, rot, eps, (const float*)down, down_stride);
  else
    latent_prepare_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(
        (const bf16_t*)proj, proj_stride, q_col, q_head_width, q_rot_at, c_col, cos_t, sin_t, norm_weight, slot_mapping,
        (bf16_t*)k_pages, (bf16_t*)queries, queries_stride, (bf16_t*)latent_out, heads, rank, rot, eps, (const bf16_t*)down,
        down_stride);
  MI_CHECK_LAUNCH("latent_prepare");
  return MI_OK;
}
