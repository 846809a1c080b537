// Recurrent mixers whose state is a matrix per head that decays and takes one outer product a
// token:
//
//     S_t = diag(a_t) S_(t-1) + k_t v_t^T          o_t = S_t^T q_t          (S is dim x vdim, float32)
//
//   DECAY_PER_CHANNEL  a_t is a vector over the key channels, a = logistic(z + bias)^(1/tau)
//                      (gated linear attention); q comes times a constant.
//   DECAY_PER_HEAD     a_t is one number per head, a = exp(-exp(rate) * dt), dt = softplus(raw +
//                      bias); the value row enters times dt, and the read-out gets skip * value
//                      added (a state-space layer in its recurrent form: k, q are its B, C rows,
//                      shared by the heads of a group).
//
// A head's state lies in memory transposed and padded, [vdim][dim_pad].  Column j of S is kept
// by L neighbouring lanes, each holding a run of R rows in registers (dim_pad = R * L), so a
// token costs a lane R multiply-adds for the update and R for the read-out, and the partial
// read-outs of a column meet through register moves between its lanes.  Columns never meet, so
// a head's columns may be shared out among blocks.  Tokens are taken a tile at a time: all
// threads fetch the tile's rows, evaluate decays and step sizes and leave them in LDS as
// float32; the walk over the tile's tokens reads LDS only.
//
//   readout_gate_norm  what follows the read-out: an RMS norm over groups of columns times a
//                      weight, and a gate silu(g), before the norm or after it.
//
// Everything that enters the recurrence is float32 (projections and convolution outputs are read
// in the element type); in the 32-bit engine decays, step sizes, the read-out's sums and the
// norm's statistics are evaluated in 64-bit and rounded once.
#include "common.h"

#include <math.h>

#define SCAN_TILE 16  // tokens fetched at once

namespace {

enum { DECAY_PER_CHANNEL = 0, DECAY_PER_HEAD = 1 };

struct ScanArgs {
  const void *q, *k, *v, *gate;  // rows in the element type
  int64_t q_stride, k_stride, v_stride, gate_stride;
  int q_col, k_col, v_col, gate_col;  // first column of head (or group) 0 in a row
  const float* gate_bias;             // per channel [heads * dim] or per head [heads]
  const float* rate;                  // per head (DECAY_PER_HEAD)
  const float* skip;                  // per head (DECAY_PER_HEAD), may be null
  float inv_tau, q_scale;
  float* state;  // [slots + 1][heads][vdim][dim_pad]
  int64_t state_stride;
  const int *cu, *slots;
  int num_slots;
  float* out;  // float32 [tokens, heads * vdim]
  int heads, groups, dim, vdim;
};

template <typename T>
struct Wide {
  using type = float;
};
template <>
struct Wide<float> {
  using type = double;
};

// log(logistic(z)), stable on both sides
template <typename A>
__device__ __forceinline__ A log_logistic(A z) {
  if constexpr (sizeof(A) == 8) return z >= 0 ? -log1p(exp(-z)) : z - log1p(exp(z));
  else return z >= 0 ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

template <typename A>
__device__ __forceinline__ A soft_plus(A z) {
  if constexpr (sizeof(A) == 8) return fmax(z, 0.0) + log1p(exp(-fabs(z)));
  else return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
}

template <typename T, int MODE, int R, int L>
__global__ __launch_bounds__(256) void decay_scan_kernel(ScanArgs p) {
  using A = typename Wide<T>::type;
  constexpr int DP = R * L;  // padded dim
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  const int cols = blockDim.x / L;
  float* q_lds = reinterpret_cast<float*>(lds_bytes);  // [SCAN_TILE][DP]
  float* k_lds = q_lds + SCAN_TILE * DP;
  float* a_lds = k_lds + SCAN_TILE * DP;                                  // per channel: [SCAN_TILE][DP]; per head: [SCAN_TILE]
  float* v_lds = a_lds + (MODE == DECAY_PER_CHANNEL ? SCAN_TILE * DP : SCAN_TILE);  // [SCAN_TILE][cols], the value rows as read
  float* dt_lds = v_lds + SCAN_TILE * cols;                               // [SCAN_TILE]

  const int b = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * cols;
  const int grp = head / (p.heads / p.groups);
  const int part = threadIdx.x % L, c = threadIdx.x / L, col = col0 + c;
  const bool live = col < p.vdim;
  const int first = p.cu[b], last = p.cu[b + 1];
  const int slot = p.slots[b];
  float* mine = p.state + (int64_t)((slot < 0 || slot >= p.num_slots) ? p.num_slots : slot) * p.state_stride +
                ((int64_t)head * p.vdim + (live ? col : 0)) * DP + part * R;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; i += 4) {
    const float4 got = *reinterpret_cast<const float4*>(mine + i);
    S[i] = got.x, S[i + 1] = got.y, S[i + 2] = got.z, S[i + 3] = got.w;
  }
  const T* q_rows = (const T*)p.q + p.q_col + (int64_t)grp * p.dim;
  const T* k_rows = (const T*)p.k + p.k_col + (int64_t)grp * p.dim;
  const T* v_rows = (const T*)p.v + p.v_col + (int64_t)head * p.vdim + col0;
  const T* g_rows = (const T*)p.gate + p.gate_col;
  const float skip = (MODE == DECAY_PER_HEAD && p.skip) ? p.skip[head] : 0.f;

  for (int t0 = first; t0 < last; t0 += SCAN_TILE) {
    const int n = min(SCAN_TILE, last - t0);
    __syncthreads();  // the last tile has been walked
    for (int e = threadIdx.x; e < n * DP; e += blockDim.x) {
      const int tt = e / DP, d = e % DP;
      const int64_t t = t0 + tt;
      float qv = 0.f, kv = 0.f, av = 0.f;
      if (d < p.dim) {
        qv = to_f32(q_rows[t * p.q_stride + d]) * p.q_scale;
        kv = to_f32(k_rows[t * p.k_stride + d]);
        if (MODE == DECAY_PER_CHANNEL) {
          const int ch = head * p.dim + d;
          const A z = (A)to_f32(g_rows[t * p.gate_stride + ch]) + (A)p.gate_bias[ch];
          if constexpr (sizeof(A) == 8) av = (float)exp(log_logistic<A>(z) * (A)p.inv_tau);
          else av = expf(log_logistic<A>(z) * p.inv_tau);
        }
      }
      q_lds[e] = qv;
      k_lds[e] = kv;
      if (MODE == DECAY_PER_CHANNEL) a_lds[e] = av;
    }
    for (int e = threadIdx.x; e < n * cols; e += blockDim.x) {
      const int tt = e / cols, cc = e % cols;
      v_lds[e] = (col0 + cc < p.vdim) ? to_f32(v_rows[(int64_t)(t0 + tt) * p.v_stride + cc]) : 0.f;
    }
    if (MODE == DECAY_PER_HEAD && threadIdx.x < n) {
      const int64_t t = t0 + threadIdx.x;
      const A step = soft_plus<A>((A)to_f32(g_rows[t * p.gate_stride + head]) + (A)p.gate_bias[head]);
      if constexpr (sizeof(A) == 8) {
        a_lds[threadIdx.x] = (float)exp(-exp((A)p.rate[head]) * step);
      } else {
        a_lds[threadIdx.x] = expf(-expf(p.rate[head]) * step);
      }
      dt_lds[threadIdx.x] = (float)step;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float xv = v_lds[tt * cols + c];
      const float vv = MODE == DECAY_PER_HEAD ? xv * dt_lds[tt] : xv;
      const float* qr = q_lds + tt * DP + part * R;
      const float* kr = k_lds + tt * DP + part * R;
      const float* ar = a_lds + tt * DP + part * R;
      const float a_head = MODE == DECAY_PER_HEAD ? a_lds[tt] : 0.f;
      A acc = 0;
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 q4 = *reinterpret_cast<const float4*>(qr + i);
        const float4 k4 = *reinterpret_cast<const float4*>(kr + i);
        float4 a4 = make_float4(a_head, a_head, a_head, a_head);
        if (MODE == DECAY_PER_CHANNEL) a4 = *reinterpret_cast<const float4*>(ar + i);
        S[i] = fmaf(k4.x, vv, a4.x * S[i]);
        S[i + 1] = fmaf(k4.y, vv, a4.y * S[i + 1]);
        S[i + 2] = fmaf(k4.z, vv, a4.z * S[i + 2]);
        S[i + 3] = fmaf(k4.w, vv, a4.w * S[i + 3]);
        if constexpr (sizeof(A) == 8) {
          acc = fma((double)S[i], (double)q4.x, acc);
          acc = fma((double)S[i + 1], (double)q4.y, acc);
          acc = fma((double)S[i + 2], (double)q4.z, acc);
          acc = fma((double)S[i + 3], (double)q4.w, acc);
        } else {
          acc = fmaf(S[i], q4.x, acc);
          acc = fmaf(S[i + 1], q4.y, acc);
          acc = fmaf(S[i + 2], q4.z, acc);
          acc = fmaf(S[i + 3], q4.w, acc);
        }
      }
#pragma unroll
      for (int off = 1; off < L; off <<= 1) acc += __shfl_xor(acc, off, MI_WAVE);
      if (part == 0 && live) {
        if constexpr (sizeof(A) == 8) acc = fma((double)skip, (double)xv, acc);
        else acc = fmaf(skip, xv, acc);
        p.out[(int64_t)(t0 + tt) * ((int64_t)p.heads * p.vdim) + (int64_t)head * p.vdim + col] = (float)acc;
      }
    }
  }
  if (live && last > first) {
#pragma unroll
    for (int i = 0; i < R; i += 4) *reinterpret_cast<float4*>(mine + i) = make_float4(S[i], S[i + 1], S[i + 2], S[i + 3]);
  }
}

// rows per lane and lanes per column for a head whose keys are `dim` wide
inline void scan_shape(int dim, int* rows, int* lanes) {
  if (dim <= 16) *rows = 4, *lanes = 4;
  else if (dim <= 32) *rows = 8, *lanes = 4;
  else if (dim <= 64) *rows = 8, *lanes = 8;
  else if (dim <= 128) *rows = 8, *lanes = 16;
  else *rows = 16, *lanes = 16;
}

template <typename T, int MODE>
int launch_scan(const ScanArgs& p, int requests, hipStream_t stream) {
  int rows, lanes;
  scan_shape(p.dim, &rows, &lanes);
  const int dp = rows * lanes;
  // columns a block keeps: as many as fill it, fewer for narrow heads (whole waves)
  const int per_wave = MI_WAVE / lanes;
  int cols = min(256 / lanes, ceil_div(p.vdim, per_wave) * per_wave);
  // short steps of few requests: share a head's columns out among more blocks
  while (cols > per_wave && (int64_t)requests * p.heads * ceil_div(p.vdim, cols) < 512) cols = max(per_wave, cols / 2 / per_wave * per_wave);
  const int threads = cols * lanes;
  dim3 grid(requests, p.heads, ceil_div(p.vdim, cols));
  const size_t lds =
      sizeof(float) * ((size_t)SCAN_TILE * dp * (MODE == DECAY_PER_CHANNEL ? 3 : 2) + (size_t)SCAN_TILE * cols + 2 * SCAN_TILE);
#define MI_SCAN(RR, LL) decay_scan_kernel<T, MODE, RR, LL><<<grid, threads, lds, stream>>>(p)
  if (rows == 4) MI_SCAN(4, 4);
  else if (rows == 8 && lanes == 4) MI_SCAN(8, 4);
  else if (rows == 8 && lanes == 8) MI_SCAN(8, 8);
  else if (rows == 8 && lanes == 16) MI_SCAN(8, 16);
  else MI_SCAN(16, 16);
#undef MI_SCAN
  MI_CHECK_LAUNCH("decay_scan");
  return MI_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void readout_gate_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                int64_t gate_stride, const float* __restrict__ weight,
                                                                int weight_period, T* __restrict__ out, int64_t out_stride,
                                                                int width, int group_width, int gate_first, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[4];
  const int t = blockIdx.x, g = blockIdx.y;
  const float* orow = o + (int64_t)t * width + (int64_t)g * group_width;
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)g * group_width;
  T* dst = out + (int64_t)t * out_stride + (int64_t)g * group_width;
  auto gate_of = [&](int c) -> A {
    const A z = (A)to_f32(grow[c]);
    if constexpr (sizeof(A) == 8) return z / (1.0 + exp(-z));
    else return z / (1.f + expf(-z));
  };
  A ss = 0;
  for (int c = threadIdx.x; c < group_width; c += blockDim.x) {
    A y = (A)orow[c];
    if (gate_first) y = (A)(float)(y * gate_of(c));
    ss += y * y;
  }
  // (fixed order: lanes by butterfly, waves one after another)
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, MI_WAVE);
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  if (threadIdx.x % MI_WAVE == 0) scratch[threadIdx.x / MI_WAVE] = ss;
  __syncthreads();
  ss = 0;
  for (int w = 0; w < n_waves; ++w) ss += scratch[w];
  A r;
  if constexpr (sizeof(A) == 8) r = 1.0 / sqrt(ss / (double)group_width + (double)eps);
  else r = 1.0f / sqrtf(ss / (float)group_width + eps);
  for (int c = threadIdx.x; c < group_width; c += blockDim.x) {
    const A w = (A)weight[(g * group_width + c) % weight_period];
    A y = (A)orow[c];
    if (gate_first) y = (A)(float)(y * gate_of(c)) * r * w;
    else y = y * r * w * gate_of(c);
    dst[c] = from_f32<T>((float)y);
  }
}

}  // namespace

extern "C" int mi_decay_scan_dim_pad(int dim) {
  int rows, lanes;
  scan_shape(dim, &rows, &lanes);
  return rows * lanes;
}

// mode 0: decay per key channel (gate: [tokens, heads * dim] logits, gate_bias [heads * dim], inv_tau);
// mode 1: decay per head (gate: [tokens, heads] raw step sizes, gate_bias [heads], rate [heads], skip [heads] or null).
// q, k: rows holding `groups` heads of `dim` from q_col / k_col on (head h reads group h / (heads / groups));
// v: rows holding `heads` heads of `vdim` from v_col on.  state float32 [slots + 1][heads][vdim][dim_pad].
// out float32 [tokens, heads * vdim].
extern "C" int mi_decay_scan(int dtype, int mode, const void* q, int64_t q_stride, int q_col, const void* k, int64_t k_stride,
                             int k_col, const void* v, int64_t v_stride, int v_col, const void* gate, int64_t gate_stride,
                             int gate_col, const float* gate_bias, const float* rate, const float* skip, float inv_tau,
                             float q_scale, float* state, int64_t state_stride, const int* cu, const int* slots, int num_slots,
                             float* out, int num_tokens, int num_requests, int heads, int groups, int dim, int vdim,
                             hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && num_requests >= 0 && heads > 0 && groups > 0 && dim > 0 && vdim > 0,
             "decay_scan: bad sizes tokens=%d requests=%d heads=%d groups=%d dim=%d vdim=%d", num_tokens, num_requests, heads,
             groups, dim, vdim);
  MI_REQUIRE(heads % groups == 0, "decay_scan: heads=%d is not a multiple of groups=%d", heads, groups);
  MI_REQUIRE(dim <= 256, "decay_scan: dim=%d is above 256", dim);
  MI_REQUIRE(mode == 0 || mode == 1, "decay_scan: mode %d (0 per channel, 1 per head)", mode);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "decay_scan: unknown dtype %d", dtype);
  MI_REQUIRE(num_slots >= 1 && num_requests <= 65535 * 32 && heads <= 65535, "decay_scan: bad slot or grid counts");
  MI_REQUIRE(q_stride >= q_col + (int64_t)groups * dim && k_stride >= k_col + (int64_t)groups * dim &&
                 v_stride >= v_col + (int64_t)heads * vdim,
             "decay_scan: row strides shorter than the columns read");
  MI_REQUIRE(gate_stride >= gate_col + (int64_t)heads * (mode == 0 ? dim : 1), "decay_scan: the gates' rows are too short");
  MI_REQUIRE(gate_bias != nullptr && (mode == 0 || rate != nullptr), "decay_scan: missing gate constants");
  MI_REQUIRE(state_stride >= (int64_t)heads * vdim * mi_decay_scan_dim_pad(dim) && ((uintptr_t)state % 16 == 0) &&
                 state_stride % 4 == 0,
             "decay_scan: the state rows are too short or not 16-byte aligned");
  if (num_tokens == 0 || num_requests == 0) return MI_OK;
  ScanArgs p;
  p.q = q, p.k = k, p.v = v, p.gate = gate;
  p.q_stride = q_stride, p.k_stride = k_stride, p.v_stride = v_stride, p.gate_stride = gate_stride;
  p.q_col = q_col, p.k_col = k_col, p.v_col = v_col, p.gate_col = gate_col;
  p.gate_bias = gate_bias, p.rate = rate, p.skip = skip, p.inv_tau = inv_tau, p.q_scale = q_scale;
  p.state = state, p.state_stride = state_stride, p.cu = cu, p.slots = slots, p.num_slots = num_slots, p.out = out;
  p.heads = heads, p.groups = groups, p.dim = dim, p.vdim = vdim;
  if (dtype == MI_F32) return mode == 0 ? launch_scan<float, DECAY_PER_CHANNEL>(p, num_requests, stream)
                                        : launch_scan<float, DECAY_PER_HEAD>(p, num_requests, stream);
  return mode == 0 ? launch_scan<bf16_t, DECAY_PER_CHANNEL>(p, num_requests, stream)
                   : launch_scan<bf16_t, DECAY_PER_HEAD>(p, num_requests, stream);
}

// o float32 [tokens, width]; gate [tokens, >= width] in the element type (row stride, from its first column);
// weight float32 [weight_period] (column c takes weight[c % weight_period]); the norm runs over
// groups of `group_width` columns.  gate_first: out = norm(o * silu(g)) * w, else norm(o) * w * silu(g).
extern "C" int mi_readout_gate_norm(int dtype, const float* o, const void* gate, int64_t gate_stride, const float* weight,
                                    int weight_period, void* out, int64_t out_stride, int num_tokens, int width,
                                    int group_width, int gate_first, float eps, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && width > 0 && group_width > 0 && width % group_width == 0,
             "readout_gate_norm: bad sizes tokens=%d width=%d group=%d", num_tokens, width, group_width);
  MI_REQUIRE(weight_period > 0 && gate_stride >= width && out_stride >= width, "readout_gate_norm: rows or weight too short");
  MI_REQUIRE(width / group_width <= 65535, "readout_gate_norm: too many groups");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "readout_gate_norm: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  dim3 grid(num_tokens, width / group_width);
  const int threads = min(256, ceil_div(group_width, MI_WAVE) * MI_WAVE);
  if (dtype == MI_F32)
    readout_gate_norm_kernel<float><<<grid, threads, 0, stream>>>(o, (const float*)gate, gate_stride, weight, weight_period,
                                                                  (float*)out, out_stride, width, group_width, gate_first, eps);
  else
    readout_gate_norm_kernel<bf16_t><<<grid, threads, 0, stream>>>(o, (const bf16_t*)gate, gate_stride, weight, weight_period,
                                                                   (bf16_t*)out, out_stride, width, group_width, gate_first, eps);
  MI_CHECK_LAUNCH("readout_gate_norm");
  return MI_OK;
}
