// A recurrent mixer with a matrix state per head, written by the gated delta rule, and the short
// causal convolution in front of it.
//
//   short_conv        y[t, c] = silu(sum_j w[c, j] * x[t - (taps-1) + j, c]) over the rows of each
//                     request; rows before a portion's first come from the request's tail (its
//                     last taps-1 inputs, kept in its state slot), zeros at a sequence's start.
//   short_conv_tail   the tail after the portion (runs after short_conv: it overwrites what
//                     that one reads).
//   gated_delta       per request and head, token by token (S is dim x vdim, float32):
//                       S <- decay * S;  u = write * (v - S^T k);  S <- S + k u^T;  o = S^T q
//                     with q, k made unit vectors per head first (q also times dim^-1/2),
//                       write = logistic(b),  decay = exp(-exp(A_log) * softplus(a + dt_bias)),
//                     and the read-out o divided by its root mean square over vdim, times a weight
//                     per column and silu(g).
//
// The state of a head lies in memory transposed and padded, [vdim][dim_pad].  Column j of S is
// kept by 16 or 32 neighbouring lanes, each holding a run of its rows: a token costs a lane a few
// multiply-adds per pass and the partial sums meet through register moves between the lanes,
// with no barrier inside a tile of tokens.  Columns are independent of one another, so a head's
// work spreads over 16 or 32 times vdim threads however short the step.
// Everything that enters the recurrence is float32 (the projections and the convolution's
// outputs are read in the element type); in the 32-bit engine the scalar gates, the unit norms
// and the read-out's norm are evaluated in 64-bit and rounded once.
#include "common.h"

#include <math.h>

#define DELTA_MAX_TAPS 16
#define SHORT_CONV_WALK_ROWS 64  // steps of at most this many rows: convolution and tail in one launch

namespace {

template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, const T* __restrict__ tail,
    int64_t tail_stride, const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ token_request, T* __restrict__ y, int64_t y_stride, int channels, int taps,
    int num_slots, int row0, const float* __restrict__ bias) {
  const int t = row0 + blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int b = token_request[t];
  const int i = t - cu[b];  // the row's place in its portion
  const int slot = slots[b];
  const T* mine = tail + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * tail_stride;
  const float* wc = w + (int64_t)c * taps;
  const int back = taps - 1;
  const float start = bias ? bias[c] : 0.f;  // (a convolution with a bias per channel starts its sum there)
  if constexpr (sizeof(T) == 4) {
    double sum = (double)start;
    for (int j = 0; j < taps; ++j) {
      const int at = i - back + j;  // row of the portion, negative: of the tail
      const float v = at >= 0 ? x[(int64_t)(t - back + j) * x_stride + c] : mine[(int64_t)(back + at) * channels + c];
      sum = fma((double)wc[j], (double)v, sum);
    }
    y[(int64_t)t * y_stride + c] = (float)(sum / (1.0 + exp(-sum)));
  } else {
    float sum = start;
    for (int j = 0; j < taps; ++j) {
      const int at = i - back + j;
      const float v = at >= 0 ? to_f32(x[(int64_t)(t - back + j) * x_stride + c])
                              : to_f32(mine[(int64_t)(back + at) * channels + c]);
      sum = fmaf(wc[j], v, sum);
    }
    y[(int64_t)t * y_stride + c] = from_f32<T>(sum * mi_logistic(sum));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_tail_kernel(const T* __restrict__ x, int64_t x_stride,
                                                              T* __restrict__ tail, int64_t tail_stride,
                                                              const int* __restrict__ cu, const int* __restrict__ slots,
                                                              int channels, int taps, int num_slots) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu[b], n = cu[b + 1] - first;
  if (n <= 0) return;
  const int slot = slots[b];
  T* mine = tail + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * tail_stride;
  const int back = taps - 1;
  T old[DELTA_MAX_TAPS];
  for (int j = 0; j < back; ++j) old[j] = mine[(int64_t)j * channels + c];
  for (int j = 0; j < back; ++j) {
    const int at = n - back + j;
    mine[(int64_t)j * channels + c] = at >= 0 ? x[(int64_t)(first + at) * x_stride + c] : old[n + j];
  }
}

// Steps of few rows (decoded tokens, short portions): a thread walks the rows of one request on one
// channel with the last taps-1 inputs in registers, and leaves them as the new tail: convolution
// and tail in one launch.  The arithmetic is that of short_conv_kernel, term by term.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_walk_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, T* __restrict__ tail, int64_t tail_stride,
    const int* __restrict__ cu, const int* __restrict__ slots, T* __restrict__ y, int64_t y_stride, int channels, int taps,
    int num_slots, const float* __restrict__ bias) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu[b], last = cu[b + 1];
  if (last <= first) return;
  const float start = bias ? bias[c] : 0.f;
  const int slot = slots[b];
  T* mine = tail + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * tail_stride;
  const int back = taps - 1;
  float window[DELTA_MAX_TAPS], wc[DELTA_MAX_TAPS];  // window[j]: the input `back - j` rows ago
#pragma unroll
  for (int j = 0; j < DELTA_MAX_TAPS; ++j) {
    window[j] = j < back ? to_f32(mine[(int64_t)j * channels + c]) : 0.f;
    wc[j] = j < taps ? w[(int64_t)c * taps + j] : 0.f;
  }
  for (int t = first; t < last; ++t) {
    const float now = to_f32(x[(int64_t)t * x_stride + c]);
    if constexpr (sizeof(T) == 4) {
      double sum = (double)start;
#pragma unroll
      for (int j = 0; j < DELTA_MAX_TAPS; ++j)
        if (j < back) sum = fma((double)wc[j], (double)window[j], sum);
      sum = fma((double)w[(int64_t)c * taps + back], (double)now, sum);
      y[(int64_t)t * y_stride + c] = (float)(sum / (1.0 + exp(-sum)));
    } else {
      float sum = start;
#pragma unroll
      for (int j = 0; j < DELTA_MAX_TAPS; ++j)
        if (j < back) sum = fmaf(wc[j], window[j], sum);
      sum = fmaf(w[(int64_t)c * taps + back], now, sum);
      y[(int64_t)t * y_stride + c] = from_f32<T>(sum * mi_logistic(sum));
    }
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS - 1; ++j)
      if (j + 1 < back) window[j] = window[j + 1];
#pragma unroll
    for (int j = 0; j < DELTA_MAX_TAPS; ++j)
      if (j == back - 1) window[j] = now;
  }
#pragma unroll
  for (int j = 0; j < DELTA_MAX_TAPS; ++j)
    if (j < back) mine[(int64_t)j * channels + c] = from_f32<T>(window[j]);
}

// what a token's step needs beside q and k, made once per tile
struct TokenGates {
  float decay, write;
};

// Sum over the R neighbouring lanes that keep one column (R = 4, 8, 16 inside a row of 16
// lanes, or 32: two rows); every lane gets the total.  Lane exchanges inside a row are register moves (DPP):
// neighbours, pairs, then the mirror image inside 8 and inside 16 lanes, which after the first
// two steps holds the other half's sum.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float lanes_sum(float v) {
  v += dpp_move<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);  // quad_perm [2,3,0,1]
  if constexpr (R >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
  if constexpr (R >= 16) v += dpp_move<0x140>(v);  // row_mirror
  // (the other row of 16 inside 32 lanes: lane ^ 16, through the LDS crossbar without touching memory)
  if constexpr (R >= 32) v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
  return v;
}

// R lanes (16 or 32) keep a column of S, lane r of them its rows r * ROWS .. (r + 1) * ROWS - 1
// (rows past dim are zero and stay zero).  The columns of S do not meet in the recurrence, so a
// head's columns are shared out among blocks: 256 threads keep 256 / R columns; thread = R *
// column + r.  The state of a head lies in memory as S transposed and padded, [vdim][R * ROWS].
// The read-outs leave as float32 [tokens, heads * vdim]; their norm over a head's columns is the
// next kernel's.
//
// Tokens are taken a tile (32, or 16) at a time.  A tile's rows are asked of memory while the
// tile before it is worked on (they wait in registers); then a group of lanes per token makes q
// and k unit vectors and puts them into LDS with the tile's values and gates, all tokens at once;
// then the recurrence walks the tile with LDS reads only, each token's operands read while the
// one before it is worked on.  A step of the recurrence is 4 * ROWS multiply-adds a lane and two
// sums over R lanes by register moves.  Counters at heads of 128 x 128, 16 lanes a column: 100
// vector instructions and 6 LDS reads a token and wave, one wave a SIMD, a token every 250 issue
// turns.  32 lanes a column (half the work a wave, two waves a SIMD, twice the LDS reads a CU)
// measured no faster, 961 against 912 us for 2,048 tokens, so 16 it is.
template <typename T, int R, int ROWS>
__global__ __launch_bounds__(256) void gated_delta_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, const T* __restrict__ proj, int64_t proj_stride, int col_b,
    int col_a, const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
    int64_t state_stride, const int* __restrict__ cu, const int* __restrict__ slots, float* __restrict__ readout,
    int heads, int kv_heads, int dim, int vdim, int chunks, int num_slots) {
  constexpr bool WIDE = sizeof(T) == 4;
  constexpr int PAD = R * ROWS;    // rows of S as kept: dim rounded up
  constexpr int COLS = 256 / R;    // columns of S this block keeps
  // In LDS a lane's run of ROWS entries of q (and k) is followed by unused ones where runs of 32
  // or 64 bytes would otherwise meet 2 or 4 to a bank in a 16-byte read of all lanes (runs of 16
  // bytes lie side by side as they are).
  constexpr int RUN = ROWS == 4 ? 4 : ROWS + 4;
  constexpr int LPAD = R * RUN;
  constexpr int TILE = LPAD <= 192 ? 32 : 16;  // tokens prepared together (two tiles of LPAD floats each fit LDS)
  constexpr int GROUP = 256 / TILE;            // lanes that prepare one token
  constexpr int EACH = PAD / GROUP;            // entries of a token's q (and k) row a lane prepares
  constexpr int VALUES = (TILE * COLS + 255) / 256;  // of the tile's values a thread fetches
  static_assert(EACH % 4 == 0 && ROWS % 4 == 0, "entries are moved four at a time");
  __shared__ __align__(16) float q_tile[TILE * LPAD];
  __shared__ __align__(16) float k_tile[TILE * LPAD];
  __shared__ float v_tile[VALUES * 256];
  __shared__ TokenGates gates[TILE];

  const int h = blockIdx.x / chunks, chunk = blockIdx.x % chunks, b = blockIdx.y;
  const int first = cu[b], last = cu[b + 1];
  if (last <= first) return;
  const int slot = slots[b];
  const int tid = threadIdx.x;
  const int j = chunk * COLS + tid / R, r = tid % R;
  const bool owns = j < vdim;
  const int group = heads / kv_heads;
  const int kvh = h / group;
  float* mine = state + (int64_t)((slot < 0 || slot >= num_slots) ? num_slots : slot) * state_stride +
                ((int64_t)h * vdim + (owns ? j : 0)) * PAD + r * ROWS;
  float s[ROWS];
#pragma unroll
  for (int ii = 0; ii < ROWS; ii += 4) {
    const float4 four = owns ? *reinterpret_cast<const float4*>(mine + ii) : make_float4(0.f, 0.f, 0.f, 0.f);
    s[ii] = four.x, s[ii + 1] = four.y, s[ii + 2] = four.z, s[ii + 3] = four.w;
  }

  const int q_col = kvh * dim, k_col = kv_heads * dim + kvh * dim, v_col = 2 * kv_heads * dim + h * vdim + chunk * COLS;
  const int my_cols = min(COLS, vdim - chunk * COLS);
  const float rate = expf(a_log[h]);
  const double rate_wide = exp((double)a_log[h]);
  const float q_scale = 1.0f / sqrtf((float)dim);
  const float bias = dt_bias[h];

  // what this thread prepares of a tile: token `mine_token` (GROUP lanes a token), entries
  // sub * EACH .. of its q and k rows; and one or two of the tile's values
  const int mine_token = tid / GROUP, sub = tid % GROUP;
  float q_raw[EACH], k_raw[EACH], v_raw[VALUES], b_raw = 0.f, a_raw = 0.f;
  auto ask = [&](int t0, int nt) {
    const bool live = mine_token < nt;
    const T* row = qkv + (int64_t)(t0 + (live ? mine_token : 0)) * qkv_stride;
#pragma unroll
    for (int e = 0; e < EACH; ++e) {
      const int d = sub * EACH + e;
      q_raw[e] = (live && d < dim) ? to_f32(row[q_col + d]) : 0.f;
      k_raw[e] = (live && d < dim) ? to_f32(row[k_col + d]) : 0.f;
    }
    if (sub == 0) {
      const T* p = proj + (int64_t)(t0 + (live ? mine_token : 0)) * proj_stride;
      b_raw = to_f32(p[col_b + h]);
      a_raw = to_f32(p[col_a + h]);
    }
#pragma unroll
    for (int n = 0; n < VALUES; ++n) {
      const int e = tid + n * 256, i = e / COLS, c = e % COLS;
      v_raw[n] = (i < nt && c < my_cols) ? to_f32(qkv[(int64_t)(t0 + i) * qkv_stride + v_col + c]) : 0.f;
    }
  };
  ask(first, min(TILE, last - first));

  for (int t0 = first; t0 < last; t0 += TILE) {
    const int nt = min(TILE, last - t0);
    __syncthreads();  // the last tile's steps have read what is overwritten now
    {
      float q_inv, k_inv;
      if constexpr (WIDE) {
        double qq = 0.0, kk = 0.0;
#pragma unroll
        for (int e = 0; e < EACH; ++e) {
          qq += (double)q_raw[e] * q_raw[e];
          kk += (double)k_raw[e] * k_raw[e];
        }
#pragma unroll
        for (int off = 1; off < GROUP; off <<= 1) {
          qq += __shfl_xor(qq, off, MI_WAVE);
          kk += __shfl_xor(kk, off, MI_WAVE);
        }
        q_inv = (float)(1.0 / sqrt((qq + 1e-6) * (double)dim));
        k_inv = (float)(1.0 / sqrt(kk + 1e-6));
      } else {
        float qq = 0.f, kk = 0.f;
#pragma unroll
        for (int e = 0; e < EACH; ++e) {
          qq = fmaf(q_raw[e], q_raw[e], qq);
          kk = fmaf(k_raw[e], k_raw[e], kk);
        }
        q_inv = rsqrtf(lanes_sum<GROUP>(qq) + 1e-6f) * q_scale;
        k_inv = rsqrtf(lanes_sum<GROUP>(kk) + 1e-6f);
      }
      // (entry d of a token's row lies at d + (d / ROWS) * (RUN - ROWS): runs of ROWS, each padded to RUN)
      float* q_at = q_tile + mine_token * LPAD;
      float* k_at = k_tile + mine_token * LPAD;
#pragma unroll
      for (int e = 0; e < EACH; e += 4) {
        const int d = sub * EACH + e;
        const int at = d + (d / ROWS) * (RUN - ROWS);
        *reinterpret_cast<float4*>(q_at + at) = make_float4(q_raw[e] * q_inv, q_raw[e + 1] * q_inv, q_raw[e + 2] * q_inv, q_raw[e + 3] * q_inv);
        *reinterpret_cast<float4*>(k_at + at) = make_float4(k_raw[e] * k_inv, k_raw[e + 1] * k_inv, k_raw[e + 2] * k_inv, k_raw[e + 3] * k_inv);
      }
      if (sub == 0) {
        TokenGates gt;
        if constexpr (WIDE) {
          const double z = (double)a_raw + (double)bias;
          const double soft = z > 30.0 ? z : log1p(exp(z));
          gt.decay = (float)exp(-rate_wide * soft);
          gt.write = (float)(1.0 / (1.0 + exp(-(double)b_raw)));
        } else {
          const float z = a_raw + bias;
          const float soft = z > 20.f ? z : log1pf(expf(z));
          gt.decay = expf(-rate * soft);
          gt.write = 1.f / (1.f + expf(-b_raw));
        }
        gates[mine_token] = gt;
      }
#pragma unroll
      for (int n = 0; n < VALUES; ++n) v_tile[tid + n * 256] = v_raw[n];
    }
    __syncthreads();
    if (t0 + TILE < last) ask(t0 + TILE, min(TILE, last - t0 - TILE));  // (waits in registers through the steps below)
    // -- the recurrence over the tile's tokens: no barrier, the lanes of a column meet by register moves
    float kr[ROWS], qr[ROWS], k_next[ROWS], q_next[ROWS];
    float v = 0.f, v_after = 0.f;
    TokenGates gt = {1.f, 0.f}, gt_after = {1.f, 0.f};
    auto fetch = [&](int i, float* kd, float* qd, float& vd, TokenGates& gd) {
      const float4* kt = reinterpret_cast<const float4*>(k_tile + i * LPAD + r * RUN);
      const float4* qt = reinterpret_cast<const float4*>(q_tile + i * LPAD + r * RUN);
#pragma unroll
      for (int ii = 0; ii < ROWS; ii += 4) {
        const float4 kf = kt[ii / 4], qf = qt[ii / 4];
        kd[ii] = kf.x, kd[ii + 1] = kf.y, kd[ii + 2] = kf.z, kd[ii + 3] = kf.w;
        qd[ii] = qf.x, qd[ii + 1] = qf.y, qd[ii + 2] = qf.z, qd[ii + 3] = qf.w;
      }
      vd = v_tile[i * COLS + tid / R];
      gd = gates[i];
    };
    fetch(0, k_next, q_next, v_after, gt_after);
    for (int i = 0; i < nt; ++i) {
#pragma unroll
      for (int ii = 0; ii < ROWS; ++ii) kr[ii] = k_next[ii], qr[ii] = q_next[ii];
      v = v_after, gt = gt_after;
      if (i + 1 < nt) fetch(i + 1, k_next, q_next, v_after, gt_after);
      // (four running sums each: a chain of dependent multiply-adds would be the step's time)
      float seen4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < ROWS; ii += 4)
#pragma unroll
        for (int e = 0; e < 4; ++e) seen4[e] = fmaf(s[ii + e], kr[ii + e], seen4[e]);
      // (S^T k of the decayed state is the decay times S^T k of the old one)
      const float seen = lanes_sum<R>((seen4[0] + seen4[1]) + (seen4[2] + seen4[3])) * gt.decay;
      const float u = gt.write * (v - seen);
      float read4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < ROWS; ii += 4)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[ii + e] = fmaf(kr[ii + e], u, s[ii + e] * gt.decay);
          read4[e] = fmaf(s[ii + e], qr[ii + e], read4[e]);
        }
      const float read = lanes_sum<R>((read4[0] + read4[1]) + (read4[2] + read4[3]));
      if (owns && r == 0) readout[(int64_t)(t0 + i) * heads * vdim + (int64_t)h * vdim + j] = read;
    }
  }
  if (owns) {
#pragma unroll
    for (int ii = 0; ii < ROWS; ii += 4) *reinterpret_cast<float4*>(mine + ii) = make_float4(s[ii], s[ii + 1], s[ii + 2], s[ii + 3]);
  }
}

// The read-outs of a step, head by head: divided by their root mean square over the head's
// columns, times a weight per column, times silu of the output gate's projection.  A wave a head.
template <typename T>
__global__ __launch_bounds__(256) void delta_readout_norm_kernel(const float* __restrict__ readout, const T* __restrict__ proj,
                                                                 int64_t proj_stride, int col_g,
                                                                 const float* __restrict__ norm_weight, T* __restrict__ out,
                                                                 int64_t out_stride, int heads, int vdim, float eps) {
  constexpr bool WIDE = sizeof(T) == 4;
  const int t = blockIdx.x;
  const int lane = threadIdx.x % MI_WAVE;
  for (int h = blockIdx.y * (blockDim.x / MI_WAVE) + threadIdx.x / MI_WAVE; h < heads; h += gridDim.y * (blockDim.x / MI_WAVE)) {
    const float* o = readout + ((int64_t)t * heads + h) * vdim;
    float sq = 0.f;
    double sq_wide = 0.0;
    for (int d = lane; d < vdim; d += MI_WAVE) {
      if constexpr (WIDE) sq_wide += (double)o[d] * o[d];
      else sq += o[d] * o[d];
    }
    float inv;
    double inv_wide = 0.0;
    if constexpr (WIDE) {
#pragma unroll
      for (int off = MI_WAVE / 2; off > 0; off >>= 1) sq_wide += __shfl_xor(sq_wide, off, MI_WAVE);
      inv_wide = 1.0 / sqrt(sq_wide / (double)vdim + (double)eps);
      inv = (float)inv_wide;
    } else {
      inv = rsqrtf(wave_sum(sq) / (float)vdim + eps);
    }
    const T* p = proj + (int64_t)t * proj_stride + col_g + h * vdim;
    T* dst = out + (int64_t)t * out_stride + h * vdim;
    for (int d = lane; d < vdim; d += MI_WAVE) {
      const float g = to_f32(p[d]);
      if constexpr (WIDE) {
        const double gate = (double)g / (1.0 + exp(-(double)g));
        dst[d] = (float)((double)o[d] * inv_wide * (double)norm_weight[d] * gate);
      } else {
        dst[d] = from_f32<T>(o[d] * inv * norm_weight[d] * (g * mi_logistic(g)));
      }
    }
  }
}

// How a head's state is kept for these sizes: 16 lanes a column, 4, 8 or 16 rows a lane (the next of
// them that holds dim / 16).
static void delta_layout(int dim, int vdim, int* lanes, int* rows) {
  (void)vdim;
  *lanes = 16;
  *rows = dim <= 64 ? 4 : (dim <= 128 ? 8 : 16);
}

}  // namespace

// x: the projections [tokens, >= channels] (row stride); w float32 [channels, taps]; tail
// [slots + 1, (taps-1) * channels] in the element type (row stride); y [tokens, channels]; bias float32
// [channels] or null.
extern "C" int mi_short_conv(int dtype, const void* x, int64_t x_stride, const float* w, void* tail,
                             int64_t tail_stride, const int* cu, const int* slots, const int* token_request,
                             void* y, int64_t y_stride, int num_tokens, int num_requests, int channels, int taps,
                             int num_slots, const float* bias, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && num_requests >= 0 && channels > 0, "short_conv: bad sizes tokens=%d requests=%d channels=%d",
             num_tokens, num_requests, channels);
  MI_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "short_conv: taps=%d must be 1..%d", taps, DELTA_MAX_TAPS);
  MI_REQUIRE(x_stride >= channels && y_stride >= channels && tail_stride >= (int64_t)(taps - 1) * channels,
             "short_conv: row strides shorter than a row");
  MI_REQUIRE(num_slots >= 1, "short_conv: no state slots");
  MI_REQUIRE(num_requests <= 65535, "short_conv: too many requests");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "short_conv: unknown dtype %d", dtype);
  if (num_tokens == 0 || num_requests == 0) return MI_OK;
  const int blocks = ceil_div(channels, 256);
  if (num_tokens <= SHORT_CONV_WALK_ROWS) {
    dim3 grid(blocks, num_requests);
    if (dtype == MI_F32)
      short_conv_walk_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, w, (float*)tail, tail_stride, cu, slots,
                                                              (float*)y, y_stride, channels, taps, num_slots, bias);
    else
      short_conv_walk_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, w, (bf16_t*)tail, tail_stride, cu,
                                                               slots, (bf16_t*)y, y_stride, channels, taps, num_slots, bias);
    MI_CHECK_LAUNCH("short_conv_walk");
    return MI_OK;
  }
  for (int first = 0; first < num_tokens; first += 65535) {
    dim3 grid(blocks, min(65535, num_tokens - first));
    if (dtype == MI_F32)
      short_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, w, (const float*)tail, tail_stride, cu,
                                                         slots, token_request, (float*)y, y_stride, channels, taps,
                                                         num_slots, first, bias);
    else
      short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, w, (const bf16_t*)tail, tail_stride,
                                                          cu, slots, token_request, (bf16_t*)y, y_stride, channels, taps,
                                                          num_slots, first, bias);
  }
  MI_CHECK_LAUNCH("short_conv");
  if (taps > 1) {
    dim3 grid(blocks, num_requests);
    if (dtype == MI_F32)
      short_conv_tail_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, (float*)tail, tail_stride, cu,
                                                              slots, channels, taps, num_slots);
    else
      short_conv_tail_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, (bf16_t*)tail, tail_stride,
                                                               cu, slots, channels, taps, num_slots);
    MI_CHECK_LAUNCH("short_conv_tail");
  }
  return MI_OK;
}

// qkv: the convolved q | k | v [tokens, 2 * kv_heads * dim + heads * vdim]; proj: the row that
// holds the write gates' (col_b), the decays' (col_a, heads columns each) and the output gates'
// (col_g, heads * vdim columns) projections; state float32 [slots + 1, heads * vdim * dim_pad], dim_pad what
// mi_gated_delta_rows says for these sizes; readout: float32 scratch [tokens, heads * vdim].
extern "C" int mi_gated_delta_rows(int dim, int vdim) {
  int lanes = 0, rows = 0;
  delta_layout(dim, vdim, &lanes, &rows);
  return lanes * rows;
}

extern "C" int mi_gated_delta(int dtype, const void* qkv, int64_t qkv_stride, const void* proj, int64_t proj_stride,
                              int col_b, int col_a, int col_g, const float* a_log, const float* dt_bias,
                              const float* norm_weight, float* state, int64_t state_stride, const int* cu,
                              const int* slots, float* readout, void* out, int64_t out_stride, int num_tokens, int num_requests, int heads,
                              int kv_heads, int dim, int vdim, int dim_pad, float eps, int num_slots, hipStream_t stream) {
  MI_REQUIRE(num_requests >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
             "gated_delta: bad sizes requests=%d heads=%d kv_heads=%d", num_requests, heads, kv_heads);
  MI_REQUIRE(dim > 0 && dim <= 256, "gated_delta: dim=%d must be 1..256", dim);
  MI_REQUIRE(vdim > 0 && vdim <= 256, "gated_delta: vdim=%d must be 1..256", vdim);
  int lanes = 0, rows = 0;
  delta_layout(dim, vdim, &lanes, &rows);
  const int pad = lanes * rows;
  MI_REQUIRE(qkv_stride >= 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim && out_stride >= (int64_t)heads * vdim,
             "gated_delta: row strides shorter than a row");
  MI_REQUIRE(dim_pad == pad && state_stride >= (int64_t)heads * vdim * pad && state_stride % 4 == 0 &&
                 (uintptr_t)state % 16 == 0,
             "gated_delta: heads of %d x %d keep their state as [vdim][%d] float32 on 16-byte boundaries, the caller has [vdim][%d]",
             dim, vdim, pad, dim_pad);
  MI_REQUIRE(col_b >= 0 && col_a >= 0 && col_g >= 0 && proj_stride >= col_b + heads && proj_stride >= col_a + heads &&
                 proj_stride >= col_g + (int64_t)heads * vdim,
             "gated_delta: the gates' columns lie outside a row of the projections");
  MI_REQUIRE(eps > 0.f, "gated_delta: eps must be positive, got %g", (double)eps);
  MI_REQUIRE(num_slots >= 1 && num_requests <= 65535, "gated_delta: bad slot or request count");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "gated_delta: unknown dtype %d", dtype);
  if (num_requests == 0) return MI_OK;
  MI_REQUIRE(readout != nullptr, "gated_delta: no buffer for the read-outs");
  const int cols = 256 / lanes, chunks = ceil_div(vdim, cols);
  MI_REQUIRE((int64_t)heads * chunks <= 2147483647, "gated_delta: too many heads");
  dim3 grid(heads * chunks, num_requests);
#define MI_DELTA_LAUNCH(T, RR, ROWS)                                                                             \
  gated_delta_kernel<T, RR, ROWS><<<grid, 256, 0, stream>>>(                                                     \
      (const T*)qkv, qkv_stride, (const T*)proj, proj_stride, col_b, col_a, a_log, dt_bias, state, state_stride, \
      cu, slots, readout, heads, kv_heads, dim, vdim, chunks, num_slots)
#define MI_DELTA_LANES(T)                          \
  if (rows == 4) MI_DELTA_LAUNCH(T, 16, 4);        \
  else if (rows == 8) MI_DELTA_LAUNCH(T, 16, 8);   \
  else MI_DELTA_LAUNCH(T, 16, 16);
  if (dtype == MI_F32) { MI_DELTA_LANES(float) }
  else { MI_DELTA_LANES(bf16_t) }
#undef MI_DELTA_LANES
#undef MI_DELTA_LAUNCH
  MI_CHECK_LAUNCH("gated_delta");
  if (num_tokens > 0) {
    dim3 ngrid(num_tokens, min(ceil_div(heads, 4), 64));
    if (dtype == MI_F32)
      delta_readout_norm_kernel<float><<<ngrid, 256, 0, stream>>>(readout, (const float*)proj, proj_stride, col_g, norm_weight,
                                                                  (float*)out, out_stride, heads, vdim, eps);
    else
      delta_readout_norm_kernel<bf16_t><<<ngrid, 256, 0, stream>>>(readout, (const bf16_t*)proj, proj_stride, col_g, norm_weight,
                                                                   (bf16_t*)out, out_stride, heads, vdim, eps);
    MI_CHECK_LAUNCH("delta_readout_norm");
  }
  return MI_OK;
}
