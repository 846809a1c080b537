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
// a head's columns are shared out among blocks of 256 / L columns.  Tokens are taken a tile at
// a time: the next tile's rows are asked of memory while this one is walked, all threads
// evaluate decays and step sizes and leave them in LDS as float32; the walk over the tile's
// tokens reads LDS only.
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

// Sum over the L neighbouring lanes that keep one column (4, 8 or 16, inside a row of 16
// lanes); every lane gets the total.  The exchanges are register moves (DPP): neighbours,
// pairs, then the mirror image inside 8 and inside 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int L>
__device__ __forceinline__ float lanes_sum(float v) {
  v += dpp_move<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);  // quad_perm [2,3,0,1]
  if constexpr (L >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
  if constexpr (L >= 16) v += dpp_move<0x140>(v);  // row_mirror
  return v;
}
template <int L>
__device__ __forceinline__ double lanes_sum(double v) {
#pragma unroll
  for (int off = 1; off < L; off <<= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

// log(1 + e) for 0 <= e <= 1 on the hardware's logarithm (one ulp), with the series where 1 + e
// would round e away
__device__ __forceinline__ float log1p_small(float e) {
  return e < 1e-3f ? e * (1.f - e * (0.5f - e * 0.33333334f)) : 0.6931471805599453f * __builtin_amdgcn_logf(1.f + e);
}
// log(logistic(z)) = -softplus(-z), and softplus, float32 on the hardware's exponential and logarithm
__device__ __forceinline__ float soft_plus_fast(float z) {
  return fmaxf(z, 0.f) + log1p_small(__builtin_amdgcn_exp2f(-fabsf(z) * 1.4426950408889634f));
}

// 256 threads keep 256 / L columns of a head's S, L lanes a column, R rows a lane.  Tokens are
// taken SCAN_TILE at a time: a tile's rows are asked of memory while the tile before it is
// walked (they wait in registers), then all threads turn them into float32 q, k, decays and
// step sizes in LDS, and the walk reads LDS only, each token's operands one token ahead.  In LDS
// a lane's run of R entries is followed by four unused ones where runs of 32 or 64 bytes would
// otherwise meet 2 or 4 to a bank in a 16-byte read of all lanes.
template <typename T, int MODE, int R, int L>
__global__ __launch_bounds__(256) void decay_scan_kernel(ScanArgs p) {
  using A = typename Wide<T>::type;
  constexpr bool WIDE = sizeof(T) == 4;
  constexpr int DP = R * L;  // padded dim
  constexpr int RUN = R == 4 ? 4 : R + 4;
  constexpr int LP = L * RUN;  // a token's row in LDS
  constexpr int COLS = 256 / L;
  constexpr int EACH = SCAN_TILE * DP / 256;       // entries of the tile's q (k, decay) rows a thread prepares
  constexpr int VALUES = SCAN_TILE * COLS / 256;   // of the tile's values
  static_assert(EACH >= 1 && VALUES >= 1, "a tile gives every thread something to prepare");
  __shared__ __align__(16) float q_lds[SCAN_TILE * LP];
  __shared__ __align__(16) float k_lds[SCAN_TILE * LP];
  __shared__ __align__(16) float a_lds[MODE == DECAY_PER_CHANNEL ? SCAN_TILE * LP : SCAN_TILE];
  __shared__ float v_lds[SCAN_TILE * COLS];  // the value rows as read
  __shared__ float dt_lds[SCAN_TILE];

  const int b = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * COLS;
  const int tid = threadIdx.x;
  const int grp = head / (p.heads / p.groups);
  const int part = tid % L, c = tid / L, col = col0 + c;
  const bool live = col < p.vdim;
  const int first = p.cu[b], last = p.cu[b + 1];
  if (last <= first) return;
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
  float rate = 0.f, head_bias = 0.f;
  double rate_wide = 0.0;
  if constexpr (MODE == DECAY_PER_HEAD) {
    head_bias = p.gate_bias[head];
    rate = expf(p.rate[head]) * 1.4426950408889634f;  // (times log2 e: the decay is an exp2)
    rate_wide = exp((double)p.rate[head]);
  }
  float ch_bias[EACH];
  if constexpr (MODE == DECAY_PER_CHANNEL) {
#pragma unroll
    for (int i = 0; i < EACH; ++i) {
      const int d = (tid + i * 256) % DP;
      ch_bias[i] = d < p.dim ? p.gate_bias[head * p.dim + d] : 0.f;
    }
  }

  float q_raw[EACH], k_raw[EACH], g_raw[MODE == DECAY_PER_CHANNEL ? EACH : 1], v_raw[VALUES];
  auto ask = [&](int t0, int n) {
#pragma unroll
    for (int i = 0; i < EACH; ++i) {
      const int e = tid + i * 256, tt = e / DP, d = e % DP;
      const bool in = tt < n && d < p.dim;
      const int64_t t = t0 + (in ? tt : 0);
      q_raw[i] = in ? to_f32(q_rows[t * p.q_stride + d]) : 0.f;
      k_raw[i] = in ? to_f32(k_rows[t * p.k_stride + d]) : 0.f;
      if constexpr (MODE == DECAY_PER_CHANNEL) g_raw[i] = in ? to_f32(g_rows[t * p.gate_stride + head * p.dim + d]) : 0.f;
    }
    if constexpr (MODE == DECAY_PER_HEAD) g_raw[0] = tid < n ? to_f32(g_rows[(int64_t)(t0 + tid) * p.gate_stride + head]) : 0.f;
#pragma unroll
    for (int i = 0; i < VALUES; ++i) {
      const int e = tid + i * 256, tt = e / COLS, cc = e % COLS;
      v_raw[i] = (tt < n && col0 + cc < p.vdim) ? to_f32(v_rows[(int64_t)(t0 + tt) * p.v_stride + cc]) : 0.f;
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int i = 0; i < EACH; ++i) {
      const int e = tid + i * 256, tt = e / DP, d = e % DP;
      const int at = tt * LP + d + (d / R) * (RUN - R);
      q_lds[at] = q_raw[i] * p.q_scale;
      k_lds[at] = k_raw[i];
      if constexpr (MODE == DECAY_PER_CHANNEL) {
        float av = 0.f;
        if (d < p.dim) {
          if constexpr (WIDE) av = (float)exp(log_logistic<double>((double)g_raw[i] + (double)ch_bias[i]) * (double)p.inv_tau);
          else av = __builtin_amdgcn_exp2f(-soft_plus_fast(-(g_raw[i] + ch_bias[i])) * (p.inv_tau * 1.4426950408889634f));
        }
        a_lds[at] = av;
      }
    }
    if constexpr (MODE == DECAY_PER_HEAD) if (tid < SCAN_TILE) {
      if constexpr (WIDE) {
        const double step = soft_plus<double>((double)g_raw[0] + (double)head_bias);
        a_lds[tid] = (float)exp(-rate_wide * step);
        dt_lds[tid] = (float)step;
      } else {
        const float step = soft_plus_fast(g_raw[0] + head_bias);
        a_lds[tid] = __builtin_amdgcn_exp2f(-rate * step);
        dt_lds[tid] = step;
      }
    }
#pragma unroll
    for (int i = 0; i < VALUES; ++i) v_lds[tid + i * 256] = v_raw[i];
  };

  struct Operands {
    float q[R], k[R], a[R], x, dt;
  };
  auto fetch = [&](int tt, Operands& o) {
    const float4* qt = reinterpret_cast<const float4*>(q_lds + tt * LP + part * RUN);
    const float4* kt = reinterpret_cast<const float4*>(k_lds + tt * LP + part * RUN);
#pragma unroll
    for (int i = 0; i < R; i += 4) {
      const float4 q4 = qt[i / 4], k4 = kt[i / 4];
      o.q[i] = q4.x, o.q[i + 1] = q4.y, o.q[i + 2] = q4.z, o.q[i + 3] = q4.w;
      o.k[i] = k4.x, o.k[i + 1] = k4.y, o.k[i + 2] = k4.z, o.k[i + 3] = k4.w;
    }
    if constexpr (MODE == DECAY_PER_CHANNEL) {
      const float4* at = reinterpret_cast<const float4*>(a_lds + tt * LP + part * RUN);
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 a4 = at[i / 4];
        o.a[i] = a4.x, o.a[i + 1] = a4.y, o.a[i + 2] = a4.z, o.a[i + 3] = a4.w;
      }
      o.dt = 1.f;
    } else {
      o.a[0] = a_lds[tt];
      o.dt = dt_lds[tt];
    }
    o.x = v_lds[tt * COLS + c];
  };

  ask(first, min(SCAN_TILE, last - first));
  float* out_at = p.out + (int64_t)head * p.vdim + (live ? col : 0);
  const int64_t out_stride = (int64_t)p.heads * p.vdim;
  for (int t0 = first; t0 < last; t0 += SCAN_TILE) {
    const int n = min(SCAN_TILE, last - t0);
    __syncthreads();  // the last tile has been walked
    put();
    __syncthreads();
    if (t0 + SCAN_TILE < last) ask(t0 + SCAN_TILE, min(SCAN_TILE, last - t0 - SCAN_TILE));  // (waits in registers through the walk)
    auto step = [&](int tt, const Operands& o) {
      const float vv = MODE == DECAY_PER_HEAD ? o.x * o.dt : o.x;
      A acc = 0;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const float a = MODE == DECAY_PER_HEAD ? o.a[0] : o.a[i];
        S[i] = fmaf(o.k[i], vv, a * S[i]);
        if constexpr (WIDE) acc = fma((double)S[i], (double)o.q[i], acc);
        else acc = fmaf(S[i], o.q[i], acc);
      }
      acc = lanes_sum<L>(acc);
      if (part == 0 && live) {
        if constexpr (WIDE) acc = fma((double)skip, (double)o.x, acc);
        else acc = fmaf(skip, o.x, acc);
        out_at[(int64_t)(t0 + tt) * out_stride] = (float)acc;
      }
    };
    // two tokens a turn, each one's operands read from LDS while the one before it is worked on
    Operands even, odd;
    fetch(0, even);
    for (int tt = 0; tt < n; tt += 2) {
      if (tt + 1 < n) fetch(tt + 1, odd);
      step(tt, even);
      if (tt + 1 < n) {
        if (tt + 2 < n) fetch(tt + 2, even);
        step(tt + 1, odd);
      }
    }
  }
  if (live) {
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
  dim3 grid(requests, p.heads, ceil_div(p.vdim, 256 / lanes));
#define MI_SCAN(RR, LL) decay_scan_kernel<T, MODE, RR, LL><<<grid, 256, 0, stream>>>(p)
  if (rows == 4) MI_SCAN(4, 4);
  else if (rows == 8 && lanes == 4) MI_SCAN(8, 4);
  else if (rows == 8 && lanes == 8) MI_SCAN(8, 8);
  else if (rows == 8 && lanes == 16) MI_SCAN(8, 16);
  else MI_SCAN(16, 16);
#undef MI_SCAN
  MI_CHECK_LAUNCH("decay_scan");
  return MI_OK;
}

// A block takes one group of one row; V columns a thread at once, as many threads as the group
// has runs of V columns, up to 1,024.
template <typename T, int V>
__global__ __launch_bounds__(1024) void readout_gate_norm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                 int64_t gate_stride, const float* __restrict__ weight,
                                                                 int weight_period, T* __restrict__ out, int64_t out_stride,
                                                                 int width, int group_width, int gate_first, float eps) {
  using A = typename Wide<T>::type;
  __shared__ A scratch[16];
  const int t = blockIdx.x, g = blockIdx.y;
  const float* orow = o + (int64_t)t * width + (int64_t)g * group_width;
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)g * group_width;
  T* dst = out + (int64_t)t * out_stride + (int64_t)g * group_width;
  auto gate_of = [&](float raw) -> A {
    const A z = (A)raw;
    if constexpr (sizeof(A) == 8) return z / (1.0 + exp(-z));
    else return z / (1.f + expf(-z));
  };
  A ss = 0;
  for (int c = threadIdx.x * V; c < group_width; c += blockDim.x * V) {
    float y[V], z[V];
    mi_load_cols<float, V>(orow + c, y);
    if (gate_first) mi_load_cols<T, V>(grow + c, z);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      A v = (A)y[j];
      if (gate_first) v = (A)(float)(v * gate_of(z[j]));
      ss += v * v;
    }
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
  for (int c = threadIdx.x * V; c < group_width; c += blockDim.x * V) {
    float y[V], z[V], res[V];
    mi_load_cols<float, V>(orow + c, y);
    mi_load_cols<T, V>(grow + c, z);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const A w = (A)weight[(g * group_width + c + j) % weight_period];
      A v = (A)y[j];
      if (gate_first) v = (A)(float)(v * gate_of(z[j])) * r * w;
      else v = v * r * w * gate_of(z[j]);
      res[j] = (float)v;
    }
    mi_store_cols<T, V>(dst + c, res);
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
  const size_t elem = dtype == MI_F32 ? 4 : 2;
  const bool wide = group_width % 4 == 0 && gate_stride % 4 == 0 && out_stride % 4 == 0 && (uintptr_t)o % 16 == 0 &&
                    (uintptr_t)gate % (4 * elem) == 0 && (uintptr_t)out % (4 * elem) == 0;
  const int threads = min(1024, ceil_div(wide ? group_width / 4 : group_width, MI_WAVE) * MI_WAVE);
#define MI_READOUT(TT, VV)                                                                                                   \
  readout_gate_norm_kernel<TT, VV><<<grid, threads, 0, stream>>>(o, (const TT*)gate, gate_stride, weight, weight_period, (TT*)out, \
                                                                 out_stride, width, group_width, gate_first, eps)
  if (dtype == MI_F32) {
    if (wide) MI_READOUT(float, 4);
    else MI_READOUT(float, 1);
  } else {
    if (wide) MI_READOUT(bf16_t, 4);
    else MI_READOUT(bf16_t, 1);
  }
#undef MI_READOUT
  MI_CHECK_LAUNCH("readout_gate_norm");
  return MI_OK;
}
