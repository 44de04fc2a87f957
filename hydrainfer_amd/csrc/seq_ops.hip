// seq_ops.hip — the row kernels of mixers that keep per-sequence state beside the paged cache: short causal convolutions
// (the inputs of the last taps - 1 positions live in the sequence's slot), token shift with several mixes (the slot
// holds the last token's input), the clamped gated feed-forward activation, per-head decays / step sizes / write
// strengths of a recurrence, unit norms, per-head RMS norm + rotary positions + cache append, and the gate / group norm
// that finishes a mixer.  Everything that is not a matrix product's operand is float.
#include <type_traits>

#include "hx_common.h"
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

// A sigmoid for results that are rounded to bfloat16 right away: the hardware's exponential and reciprocal (about one unit
// in the last place of a float each) instead of the library's exact forms; float32 activations take the exact ones.
template <typename A>
__device__ __forceinline__ float sigmoid_of(float x) {
  if constexpr (A::kDtype == HX_F32) return 1.f / (1.f + expf(-x));
  else return __builtin_amdgcn_rcpf(1.f + __expf(-x));
}

template <typename A>
__device__ __forceinline__ float act_apply(float x, int act) {
  switch (act) {
    case HXM_ACT_SILU: return x * sigmoid_of<A>(x);
    case HXM_ACT_SIGMOID: return sigmoid_of<A>(x);
    case HXM_ACT_TANH: return tanhf(x);
    default: return x;
  }
}

__device__ __forceinline__ float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// ------------------------------------------------------------------------------------------------ causal convolution
// (y2, w2, bias2: a second convolution of the same inputs, or NULL; skip: the input itself is added to every result)
template <typename A>
__global__ __launch_bounds__(256) void causal_conv_kernel(typename A::storage* y, int64_t y_stride, const typename A::storage* u,
                                                          int64_t u_stride, const float* w, const float* bias, int act,
                                                          const float* state, int64_t slot_stride, const int32_t* slots,
                                                          const int32_t* tok_seq, const int32_t* q_cu, const int32_t* positions,
                                                          int C, int taps, typename A::storage* y2, int64_t y2_stride,
                                                          const float* w2, const float* bias2, int skip) {
  const int64_t t = blockIdx.x;
  const int seq = tok_seq[t];
  const int64_t t0 = q_cu[seq];
  const bool fresh = positions[t0] == 0;
  const float* st = state + (int64_t)slots[seq] * slot_stride;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    float acc = bias ? bias[c] : 0.f, acc2 = bias2 ? bias2[c] : 0.f, x = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int64_t src = t - (taps - 1) + j;
      x = 0.f;
      if (src >= t0) x = A::to_float(u[src * u_stride + c]);
      else if (!fresh) x = st[(int64_t)((taps - 1) - (int)(t0 - src)) * C + c];
      acc += w[(int64_t)c * taps + j] * x;
      if (y2) acc2 += w2[(int64_t)c * taps + j] * x;
    }
    const float own = skip ? x : 0.f;      // (the last tap's input is the token's own)
    y[t * y_stride + c] = A::from_float(act_apply<A>(acc, act) + own);
    if (y2) y2[t * y2_stride + c] = A::from_float(act_apply<A>(acc2, act) + own);
  }
}

// The same for up to MT taps, a thread keeping one channel's last inputs in registers over a tile of kConvTile tokens: every
// input is read once instead of once per tap.  A tile may hold the ends and starts of several sequences: the history is
// taken afresh (from the rows before, the slot, or zeros) at the tile's first token and at every portion's first token.
constexpr int kConvTile = 16;

template <typename A, int NC> struct Chan;      // NC neighbouring channels of an activation row at once
template <typename A> struct Chan<A, 1> {
  static __device__ __forceinline__ void load(const typename A::storage* p, float (&v)[1]) { v[0] = A::to_float(p[0]); }
  static __device__ __forceinline__ void store(typename A::storage* p, const float (&v)[1]) { p[0] = A::from_float(v[0]); }
};
template <> struct Chan<F32, 2> {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ void load(const float* p, float (&v)[2]) {
    const f32x2 t = *reinterpret_cast<const f32x2*>(p);
    v[0] = t[0]; v[1] = t[1];
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[2]) { *reinterpret_cast<f32x2*>(p) = f32x2{v[0], v[1]}; }
};
template <> struct Chan<BF16, 2> {
  static __device__ __forceinline__ void load(const u16* p, float (&v)[2]) {
    const uint32_t t = *reinterpret_cast<const uint32_t*>(p);
    v[0] = __builtin_bit_cast(float, t << 16); v[1] = __builtin_bit_cast(float, t & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(u16* p, const float (&v)[2]) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)BF16::from_float(v[0]) | ((uint32_t)BF16::from_float(v[1]) << 16);
  }
};

template <typename A, int MT, int NC, bool TWO>
__global__ __launch_bounds__(256) void causal_conv_tile_kernel(typename A::storage* y, int64_t y_stride, const typename A::storage* u,
                                                               int64_t u_stride, const float* w, const float* bias, int act,
                                                               const float* state, int64_t slot_stride, const int32_t* slots,
                                                               const int32_t* tok_seq, const int32_t* q_cu, const int32_t* positions,
                                                               int64_t T, int C, int taps, typename A::storage* y2, int64_t y2_stride,
                                                               const float* w2, const float* bias2, int skip) {
  const int c = NC * (blockIdx.y * 256 + threadIdx.x);
  if (c >= C) return;
  const int64_t tile0 = (int64_t)blockIdx.x * kConvTile;
  const int64_t tile1 = tile0 + kConvTile < T ? tile0 + kConvTile : T;
  const int keep = taps - 1;
  float wt[NC][MT], hist[NC][MT], b[NC];    // wt[.][j]: the weight of the input j tokens back; hist[.][j]: the input j + 1 tokens back
  float wt2[TWO ? NC : 1][TWO ? MT : 1], b2[TWO ? NC : 1];      // the second convolution's
#pragma unroll
  for (int n = 0; n < NC; ++n) {
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      wt[n][j] = j < taps ? w[(int64_t)(c + n) * taps + (taps - 1 - j)] : 0.f;
      if constexpr (TWO) wt2[n][j] = j < taps ? w2[(int64_t)(c + n) * taps + (taps - 1 - j)] : 0.f;
      hist[n][j] = 0.f;
    }
    b[n] = bias ? bias[c + n] : 0.f;
    if constexpr (TWO) b2[n] = bias2 ? bias2[c + n] : 0.f;
  }
  // the tile's sequence ids and inputs are requested at once, before anything waits for them: a portion starts where
  // the id changes, and only there (and at the tile's first token) is the history taken afresh
  int sid[kConvTile];
  float xs[kConvTile][NC];
#pragma unroll
  for (int i = 0; i < kConvTile; ++i) {
    const int64_t t = tile0 + i < tile1 ? tile0 + i : tile1 - 1;
    sid[i] = tok_seq[t];
    Chan<A, NC>::load(u + t * u_stride + c, xs[i]);
  }
#pragma unroll
  for (int i = 0; i < kConvTile; ++i) {
    const int64_t t = tile0 + i;
    if (t < tile1) {
    if (i == 0 || sid[i] != sid[i > 0 ? i - 1 : 0]) {
      const int seq = sid[i];
      const int64_t t0 = q_cu[seq];
      const bool fresh = positions[t0] == 0;
      const float* st = state + (int64_t)slots[seq] * slot_stride;
#pragma unroll
      for (int j = 0; j < MT - 1; ++j) {
        const int64_t src = t - 1 - j;
        float x[NC];
#pragma unroll
        for (int n = 0; n < NC; ++n) x[n] = 0.f;
        if (j < keep) {
          if (src >= t0) {
            Chan<A, NC>::load(u + src * u_stride + c, x);
          } else if (!fresh) {
#pragma unroll
            for (int n = 0; n < NC; ++n) x[n] = st[(int64_t)(keep - (int)(t0 - src)) * C + c + n];
          }
        }
#pragma unroll
        for (int n = 0; n < NC; ++n) hist[n][j] = x[n];
      }
    }
    float x[NC], o[NC], o2[NC];
#pragma unroll
    for (int n = 0; n < NC; ++n) x[n] = xs[i][n];
#pragma unroll
    for (int n = 0; n < NC; ++n) {
      float acc = b[n] + wt[n][0] * x[n];
#pragma unroll
      for (int j = 0; j < MT - 1; ++j) acc += wt[n][j + 1] * hist[n][j];
      const float own = skip ? x[n] : 0.f;
      o[n] = act_apply<A>(acc, act) + own;
      if constexpr (TWO) {
        float acc2 = b2[n] + wt2[n][0] * x[n];
#pragma unroll
        for (int j = 0; j < MT - 1; ++j) acc2 += wt2[n][j + 1] * hist[n][j];
        o2[n] = act_apply<A>(acc2, act) + own;
      }
#pragma unroll
      for (int j = MT - 2; j > 0; --j) hist[n][j] = hist[n][j - 1];
      hist[n][0] = x[n];
    }
    Chan<A, NC>::store(y + t * y_stride + c, o);
    if constexpr (TWO) Chan<A, NC>::store(y2 + t * y2_stride + c, o2);
    }
  }
}

// the slot afterwards: the last taps - 1 inputs of (what the slot held, then the portion); one thread a channel, ascending
template <typename A>
__global__ __launch_bounds__(256) void causal_conv_state_kernel(const typename A::storage* u, int64_t u_stride, float* state,
                                                                int64_t slot_stride, const int32_t* slots, const int32_t* q_cu,
                                                                const int32_t* positions, int C, int taps) {
  const int seq = blockIdx.x;
  const int64_t t0 = q_cu[seq], n = q_cu[seq + 1] - t0;
  if (n <= 0) return;
  const bool fresh = positions[t0] == 0;
  float* st = state + (int64_t)slots[seq] * slot_stride;
  const int keep = taps - 1;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    for (int s = 0; s < keep; ++s) {
      const int64_t at = n + s;                       // index into [the slot's keep entries | the portion's n inputs]
      float x;
      if (at >= keep) x = A::to_float(u[(t0 + at - keep) * u_stride + c]);
      else x = fresh ? 0.f : st[(int64_t)at * C + c];
      st[(int64_t)s * C + c] = x;
    }
  }
}

// ------------------------------------------------------------------------------------------------ token shift
template <typename A>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(typename A::storage* out, const typename A::storage* h, int64_t h_stride,
                                                              const float* mu, int n_mix, const float* state, int64_t slot_stride,
                                                              const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                                                              const int32_t* positions, int64_t T, int64_t W, int vec) {
  const int64_t t = blockIdx.x;
  const int seq = tok_seq[t];
  const int64_t t0 = q_cu[seq];
  const bool first = t == t0, fresh = positions[t0] == 0;
  const float* st = state + (int64_t)slots[seq] * slot_stride;
  if (vec) {
    for (int64_t c = 4 * (int64_t)threadIdx.x; c < W; c += 1024) {
      const f32x4 x = Row4<A>::load(h + t * h_stride + c);
      f32x4 prev = f32x4{0.f, 0.f, 0.f, 0.f};
      if (!first) prev = Row4<A>::load(h + (t - 1) * h_stride + c);
      else if (!fresh) prev = *reinterpret_cast<const f32x4*>(st + c);
      for (int m = 0; m < n_mix; ++m) {
        const f32x4 w = *reinterpret_cast<const f32x4*>(mu + (int64_t)m * W + c);
        f32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = x[k] + (prev[k] - x[k]) * w[k];
        Row4<A>::store(out + ((int64_t)m * T + t) * W + c, o);
      }
    }
    return;
  }
  for (int64_t c = threadIdx.x; c < W; c += 256) {
    const float x = A::to_float(h[t * h_stride + c]);
    const float prev = first ? (fresh ? 0.f : st[c]) : A::to_float(h[(t - 1) * h_stride + c]);
    const float d = prev - x;
    for (int m = 0; m < n_mix; ++m) out[((int64_t)m * T + t) * W + c] = A::from_float(x + d * mu[(int64_t)m * W + c]);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void token_shift_state_kernel(const typename A::storage* h, int64_t h_stride, float* state,
                                                                int64_t slot_stride, const int32_t* slots, const int32_t* q_cu, int64_t W) {
  const int seq = blockIdx.x;
  const int64_t t0 = q_cu[seq], t1 = q_cu[seq + 1];
  if (t1 <= t0) return;
  float* st = state + (int64_t)slots[seq] * slot_stride;
  for (int64_t c = threadIdx.x; c < W; c += 256) st[c] = A::to_float(h[(t1 - 1) * h_stride + c]);
}

// ------------------------------------------------------------------------------------------------ element-wise rows
template <typename A>
__global__ __launch_bounds__(256) void clamped_glu_kernel(typename A::storage* y, int64_t y_stride, const typename A::storage* gate,
                                                          int64_t gate_stride, const typename A::storage* up, int64_t up_stride,
                                                          float limit, float alpha, float up_shift, int64_t rows, int64_t n, int vec) {
  if (vec) {
    const int64_t n4 = n >> 2, total = rows * n4;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
      const int64_t r = e / n4, i = (e - r * n4) * 4;
      f32x4 g = Row4<A>::load(gate + r * gate_stride + i), u = Row4<A>::load(up + r * up_stride + i), o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float gg = limit > 0.f ? fminf(g[k], limit) : g[k];
        const float uu = limit > 0.f ? fminf(fmaxf(u[k], -limit), limit) : u[k];
        o[k] = gg * sigmoid_of<A>(alpha * gg) * (uu + up_shift);
      }
      Row4<A>::store(y + r * y_stride + i, o);
    }
    return;
  }
  const int64_t total = rows * n;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t r = e / n, i = e - r * n;
    const float g = A::to_float(gate[r * gate_stride + i]), u = A::to_float(up[r * up_stride + i]);
    const float gg = limit > 0.f ? fminf(g, limit) : g;
    const float uu = limit > 0.f ? fminf(fmaxf(u, -limit), limit) : u;
    y[r * y_stride + i] = A::from_float(gg * sigmoid_of<A>(alpha * gg) * (uu + up_shift));
  }
}

template <typename A>
__global__ __launch_bounds__(256) void unary_kernel(typename A::storage* out, int64_t out_stride, const typename A::storage* x,
                                                    int64_t x_stride, int act, int64_t rows, int64_t n) {
  const int64_t total = rows * n;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t r = e / n, i = e - r * n;
    out[r * out_stride + i] = A::from_float(act_apply<A>(A::to_float(x[r * x_stride + i]), act));
  }
}

template <typename A>
__global__ __launch_bounds__(256) void head_gates_kernel(float* decay, float* step, float* beta, const typename A::storage* a,
                                                         int64_t a_stride, const typename A::storage* b, int64_t b_stride,
                                                         const float* log_rate, const float* step_bias, int64_t T, int H) {
  const int64_t total = T * H;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t t = e / H;
    const int h = (int)(e - t * H);
    const float sp = softplus(A::to_float(a[t * a_stride + h]) + step_bias[h]);
    decay[e] = expf(-expf(log_rate[h]) * sp);
    if (step) step[e] = sp;
    if (beta) beta[e] = 1.f / (1.f + expf(-A::to_float(b[t * b_stride + h])));
  }
}

template <typename A>
__global__ __launch_bounds__(256) void decay_exp_kernel(float* decay, const typename A::storage* x, int64_t x_stride, const float* bias,
                                                        int64_t rows, int64_t n) {
  const int64_t total = rows * n;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t r = e / n, i = e - r * n;
    decay[e] = expf(-expf(A::to_float(x[r * x_stride + i]) + (bias ? bias[i] : 0.f)));
  }
}

// one wave per (token, head)
template <typename A>
__global__ __launch_bounds__(256) void unit_norm_kernel(float* out, const typename A::storage* x, int64_t x_stride, float eps, float scale,
                                                        int64_t T, int H, int D) {
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= T * H) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = item / H;
  const int h = (int)(item - t * H);
  const typename A::storage* xr = x + t * x_stride + (int64_t)h * D;
  float ss = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float v = A::to_float(xr[d]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss + eps);
  float* o = out + (t * H + h) * D;
  for (int d = lane; d < D; d += 64) o[d] = A::to_float(xr[d]) * inv;
}

// ------------------------------------------------------------------------------------------------ head norm + rotation + cache
// two neighbouring elements of an activation row in one store (p on a multiple of two elements)
template <typename A> struct Pair;
template <> struct Pair<F32> {
  static __device__ __forceinline__ void store(float* p, float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    *reinterpret_cast<f32x2*>(p) = f32x2{a, b};
  }
};
template <> struct Pair<BF16> {
  static __device__ __forceinline__ void store(u16* p, float a, float b) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)BF16::from_float(a) | ((uint32_t)BF16::from_float(b) << 16);
  }
};

// one workgroup per token: the token's cos and sin of every pair and all its query and key heads go once into LDS (one
// round trip to memory), then the four waves take the heads in turn (heads 0 .. q_heads - 1 are queries, the rest keys).
// LDS: [cos | sin] of the pairs, then (q_heads + kv_heads) * dim floats.
template <typename A>
__global__ __launch_bounds__(256) void head_norm_rope_cache_kernel(hxm_head_rope_args a) {
  extern __shared__ float lds[];
  typedef typename A::storage T;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int NH = a.q_heads + a.kv_heads, D = a.dim, R = a.rot_dims, half = R >> 1;
  const int64_t t = blockIdx.x;
  float* cs = lds;
  float* sn = lds + half;
  float* all = lds + 2 * half;
  const int nq = a.q_heads * D, nk = a.kv_heads * D;
  const T* qrow = (const T*)a.q + t * a.q_stride;
  const T* krow = (const T*)a.k + t * a.k_stride;
  const bool rows4 = nq % 4 == 0 && nk % 4 == 0 && R % 2 == 0 && a.q_stride % 4 == 0 && a.k_stride % 4 == 0 &&
                     (((uintptr_t)a.q | (uintptr_t)a.k) % (4 * sizeof(T))) == 0;
  if (rows4) {
    for (int e = 4 * threadIdx.x; e < nq; e += 1024) *reinterpret_cast<f32x4*>(all + e) = Row4<A>::load(qrow + e);
    for (int e = 4 * threadIdx.x; e < nk; e += 1024) *reinterpret_cast<f32x4*>(all + nq + e) = Row4<A>::load(krow + e);
  } else {
    for (int e = threadIdx.x; e < nq; e += 256) all[e] = A::to_float(qrow[e]);
    for (int e = threadIdx.x; e < nk; e += 256) all[nq + e] = A::to_float(krow[e]);
  }
  const float p = (float)a.positions[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float s_, c_;
    sincosf(p * a.inv_freq[i], &s_, &c_);
    cs[i] = c_ * a.cos_sin_scale;
    sn[i] = s_ * a.cos_sin_scale;
  }
  __syncthreads();
  const int64_t slot = a.kv_heads ? a.slot_ids[t] : 0;
  const uintptr_t pair_bytes = 2 * sizeof(T);
  if (D % 2 == 0 && R % 4 == 0 && D <= 512 && (((uintptr_t)a.q_w | (uintptr_t)a.k_w) & 7) == 0 && ((a.cache_row_stride | a.head_stride) & 1) == 0 &&
      (((uintptr_t)a.q_out | (uintptr_t)a.key_cache | (uintptr_t)a.value_cache) % pair_bytes) == 0) {
    // two neighbouring channels a lane, the same ones for every head: their cos and sin stay in registers, the sum of
    // squares is a DPP row sum and four lane reads, and a head costs three LDS accesses a lane
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 c2[4], s2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = 2 * (lane + 64 * i);
      c2[i] = f32x2{1.f, 1.f};
      s2[i] = f32x2{0.f, 0.f};
      if (d < R) {
        const int j = d < half ? d : d - half;
        c2[i] = *reinterpret_cast<const f32x2*>(cs + j);
        s2[i] = *reinterpret_cast<const f32x2*>(sn + j);
        if (d < half) s2[i] = -s2[i];                 // the first half turns against its partner, the second with it
      }
    }
    for (int h = wave; h < NH; h += 4) {
      const bool is_q = h < a.q_heads;
      const int g = is_q ? h : h - a.q_heads;
      float* nb = all + (int64_t)h * D;
      const float* w = is_q ? a.q_w : a.k_w;
      T* orow = is_q ? (T*)a.q_out + (t * a.q_heads + g) * D : (T*)a.key_cache + slot * a.cache_row_stride + (int64_t)g * a.head_stride;
      T* vrow = is_q ? nullptr : (T*)a.value_cache + slot * a.cache_row_stride + (int64_t)g * a.head_stride;
      f32x2 x[4];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 2 * (lane + 64 * i);
        x[i] = f32x2{0.f, 0.f};
        if (d < D) {
          x[i] = *reinterpret_cast<const f32x2*>(nb + d);
          if (vrow) Pair<A>::store(vrow + d, x[i][0], x[i][1]);
          ss += x[i][0] * x[i][0] + x[i][1] * x[i][1];
        }
      }
      ss = row16_sum(ss);
      const float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ss), 0)) +
                        __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ss), 16)) +
                        __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ss), 32)) +
                        __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ss), 48));
      const float inv = 1.0f / sqrtf(tot / (float)D + a.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 2 * (lane + 64 * i);
        if (d < D) {
          const f32x2 w2 = *reinterpret_cast<const f32x2*>(w + d);
          x[i][0] *= inv * w2[0];
          x[i][1] *= inv * w2[1];
          if (d < R) *reinterpret_cast<f32x2*>(nb + d) = x[i];
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 2 * (lane + 64 * i);
        if (d < D) {
          f32x2 o = x[i];
          if (d < R) {
            const f32x2 pr = *reinterpret_cast<const f32x2*>(nb + (d < half ? d + half : d - half));
            o[0] = x[i][0] * c2[i][0] + pr[0] * s2[i][0];
            o[1] = x[i][1] * c2[i][1] + pr[1] * s2[i][1];
          }
          Pair<A>::store(orow + d, o[0], o[1]);
        }
      }
    }
    return;
  }
  for (int h = wave; h < NH; h += 4) {
    const bool is_q = h < a.q_heads;
    const int g = is_q ? h : h - a.q_heads;
    float* nb = all + (int64_t)h * D;
    const float* w = is_q ? a.q_w : a.k_w;
    T* vrow = nullptr;
    T* orow;
    if (is_q) {
      orow = (T*)a.q_out + (t * a.q_heads + g) * D;
    } else {
      orow = (T*)a.key_cache + slot * a.cache_row_stride + (int64_t)g * a.head_stride;
      vrow = (T*)a.value_cache + slot * a.cache_row_stride + (int64_t)g * a.head_stride;
    }
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = nb[d];
      if (vrow) vrow[d] = A::from_float(v);          // (exactly the element that came in)
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)D + a.eps);
    for (int d = lane; d < D; d += 64) nb[d] = nb[d] * inv * w[d];      // (a lane rewrites the channels it read)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int d = lane; d < D; d += 64) {
      float o = nb[d];
      if (d < half) o = nb[d] * cs[d] - nb[d + half] * sn[d];
      else if (d < R) o = nb[d] * cs[d - half] + nb[d - half] * sn[d - half];
      orow[d] = A::from_float(o);
    }
  }
}

// ------------------------------------------------------------------------------------------------ gate / group norm
template <typename A, typename X>
__device__ __forceinline__ float gn_value(const hxm_group_norm_args& a, int64_t r, int64_t c) {
  float v = X::to_float(((const typename X::storage*)a.x)[r * a.x_stride + c]);
  if (a.skip) v += a.skip_w[c / a.skip_group] * A::to_float(((const typename A::storage*)a.skip)[r * a.skip_stride + c]);
  if (a.gate && a.gate_first) v *= act_apply<A>(A::to_float(((const typename A::storage*)a.gate)[r * a.gate_stride + c]), a.gate_act);
  return v;
}

template <typename A, typename X>
__device__ __forceinline__ f32x4 gn_value4(const hxm_group_norm_args& a, int64_t r, int64_t c) {
  f32x4 v = Row4<X>::load((const typename X::storage*)a.x + r * a.x_stride + c);
  if (a.skip) {
    const f32x4 sk = Row4<A>::load((const typename A::storage*)a.skip + r * a.skip_stride + c);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] += a.skip_w[(uint32_t)(c + k) / (uint32_t)a.skip_group] * sk[k];
  }
  if (a.gate && a.gate_first) {
    const f32x4 g = Row4<A>::load((const typename A::storage*)a.gate + r * a.gate_stride + c);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] *= act_apply<A>(g[k], a.gate_act);
  }
  return v;
}

// one wave per (row, group): the group's sum of squares, then the elements once more (vec: four elements a lane, the first
// 1024 of a group kept in registers between the two passes)
template <typename A, typename X>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(hxm_group_norm_args a, int vec) {
  typedef typename A::storage T;
  const int lane = threadIdx.x & 63;
  const int64_t gs = a.group > 0 ? a.group : (a.n < 1024 ? a.n : 1024);        // no norm: the groups only deal the work
  const int64_t n_groups = (a.n + gs - 1) / gs;
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= a.rows * n_groups) return;
  const int64_t r = item / n_groups, c0 = (item - r * n_groups) * gs;
  const int64_t c1 = c0 + gs < a.n ? c0 + gs : a.n;
  T* o = (T*)a.out + r * a.out_stride;
  if (vec) {
    f32x4 keep[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t c = c0 + 4 * (lane + 64 * i);
      if (c < c1) {
        keep[i] = gn_value4<A, X>(a, r, c);
        ss += (keep[i][0] * keep[i][0] + keep[i][1] * keep[i][1]) + (keep[i][2] * keep[i][2] + keep[i][3] * keep[i][3]);
      }
    }
    if (a.group > 0)
      for (int64_t c = c0 + 4 * (lane + 256); c < c1; c += 256) {
        const f32x4 v = gn_value4<A, X>(a, r, c);
        ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
      }
    float inv = 1.f;
    if (a.group > 0) inv = 1.0f / sqrtf(wave_sum(ss) / (float)gs + a.eps);
    auto finish = [&](f32x4 v, int64_t c) {
      f32x4 g = f32x4{1.f, 1.f, 1.f, 1.f};
      if (a.gate && !a.gate_first) g = Row4<A>::load((const T*)a.gate + r * a.gate_stride + c);
      const uint32_t cw = a.w ? (uint32_t)c % (uint32_t)a.w_len : 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float x = v[k] * inv;
        if (a.w) x *= a.w[cw + k < (uint32_t)a.w_len ? cw + k : cw + k - (uint32_t)a.w_len];
        if (a.gate && !a.gate_first) x *= act_apply<A>(g[k], a.gate_act);
        v[k] = x * a.scale;
      }
      Row4<A>::store(o + c, v);
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t c = c0 + 4 * (lane + 64 * i);
      if (c < c1) finish(keep[i], c);
    }
    for (int64_t c = c0 + 4 * (lane + 256); c < c1; c += 256) finish(gn_value4<A, X>(a, r, c), c);
    return;
  }
  float inv = 1.f;
  if (a.group > 0) {
    float ss = 0.f;
    for (int64_t c = c0 + lane; c < c1; c += 64) {
      const float v = gn_value<A, X>(a, r, c);
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)gs + a.eps);
  }
  for (int64_t c = c0 + lane; c < c1; c += 64) {
    float v = gn_value<A, X>(a, r, c) * inv;
    if (a.w) v *= a.w[c % a.w_len];
    if (a.gate && !a.gate_first) v *= act_apply<A>(A::to_float(((const T*)a.gate)[r * a.gate_stride + c]), a.gate_act);
    o[c] = A::from_float(v * a.scale);
  }
}

// Groups of at most 128 elements, four elements a lane: LPG lanes a group, 64 / LPG groups a wave; everything a group needs
// is requested before its sum is known.
template <typename A, typename X>
__global__ __launch_bounds__(256) void gated_group_norm_small_kernel(hxm_group_norm_args a, int lpg) {
  typedef typename A::storage T;
  const int lane = threadIdx.x & 63;
  const int64_t gs = a.group > 0 ? a.group : (a.n < 128 ? a.n : 128);
  const int64_t n_groups = (a.n + gs - 1) / gs;
  const int64_t item = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / lpg) + lane / lpg;
  const int64_t r = item / n_groups, c0 = (item - r * n_groups) * gs;
  const int64_t c1 = c0 + gs < a.n ? c0 + gs : a.n;
  const int64_t c = c0 + 4 * (lane % lpg);
  const bool ok = item < a.rows * n_groups && c < c1;
  f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f}, g = f32x4{1.f, 1.f, 1.f, 1.f};
  if (ok) {
    v = gn_value4<A, X>(a, r, c);
    if (a.gate && !a.gate_first) g = Row4<A>::load((const T*)a.gate + r * a.gate_stride + c);
  }
  float inv = 1.f;
  if (a.group > 0) {
    float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    for (int off = lpg >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    inv = 1.0f / sqrtf(ss / (float)gs + a.eps);
  }
  if (!ok) return;
  const uint32_t cw = a.w ? (uint32_t)c % (uint32_t)a.w_len : 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float x = v[k] * inv;
    if (a.w) x *= a.w[cw + k < (uint32_t)a.w_len ? cw + k : cw + k - (uint32_t)a.w_len];
    if (a.gate && !a.gate_first) x *= act_apply<A>(g[k], a.gate_act);
    v[k] = x * a.scale;
  }
  Row4<A>::store((T*)a.out + r * a.out_stride + c, v);
}

inline unsigned flat_blocks(int64_t total) {
  const int64_t b = (total + 255) / 256;
  return (unsigned)(b < 1 ? 1 : (b > 16384 ? 16384 : b));
}

}  // namespace

#define HXM_BY_DTYPE(dtype, CALL_F32, CALL_BF16) \
  switch (dtype) {                               \
    case HX_F32: CALL_F32; break;                \
    case HX_BF16: CALL_BF16; break;              \
    default: return HX_ERR_DTYPE;                \
  }

static int causal_conv_launch(void* y, int64_t y_stride, const void* u, int64_t u_stride, const float* w, const float* bias, int act,
                              float* state, int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                              const int32_t* positions, int64_t n_tokens, int32_t n_seq, int32_t channels, int32_t taps, int dtype,
                              void* stream, void* y2, int64_t y2_stride, const float* w2, const float* bias2, int skip) {
  if (n_tokens < 0 || n_seq < 0 || channels < 1 || taps < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0 || n_seq == 0) return HX_OK;
  if (!y || !u || !w || !state || !slots || !tok_seq || !q_cu || !positions || (y2 && !w2)) return HX_ERR_NULL;
  if (y_stride < channels || u_stride < channels || (y2 && y2_stride < channels)) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const unsigned cb = (unsigned)((channels + 255) / 256);
  const dim3 grid((unsigned)n_tokens, cb < 64 ? cb : 64), sgrid((unsigned)n_seq, cb < 64 ? cb : 64), block(256);
  const uintptr_t pair = dtype == HX_F32 ? 8 : 4;
  const bool two = channels % 2 == 0 && y_stride % 2 == 0 && u_stride % 2 == 0 && (uintptr_t)y % pair == 0 && (uintptr_t)u % pair == 0 &&
                   y2_stride % 2 == 0 && (uintptr_t)y2 % pair == 0;
  const dim3 tgrid((unsigned)((n_tokens + kConvTile - 1) / kConvTile), two ? (unsigned)((channels / 2 + 255) / 256) : cb);
  auto tile = [&](auto tag, auto mt) {
    typedef decltype(tag) A;
    constexpr int MT = decltype(mt)::value;
    typedef typename A::storage E;
#define HXM_CONV_TILE(NC_, TWO_)                                                                                                      \
  causal_conv_tile_kernel<A, MT, NC_, TWO_><<<tgrid, block, 0, s>>>((E*)y, y_stride, (const E*)u, u_stride, w, bias, act, state, slot_stride, \
                                                                    slots, tok_seq, q_cu, positions, n_tokens, channels, taps, (E*)y2,   \
                                                                    y2_stride, w2, bias2, skip)
    if (two) {
      if (y2) HXM_CONV_TILE(2, true);
      else HXM_CONV_TILE(2, false);
    } else {
      if (y2) HXM_CONV_TILE(1, true);
      else HXM_CONV_TILE(1, false);
    }
#undef HXM_CONV_TILE
  };
  typedef std::integral_constant<int, 4> Taps4;
  typedef std::integral_constant<int, 8> Taps8;
  // (a batch of few tokens — decode steps — has nothing to keep in registers from one token to the next: a thread a token and channel)
  if (taps <= 8 && n_tokens >= 8 * kConvTile) {
    if (taps <= 4) {
      HXM_BY_DTYPE(dtype, (tile(F32{}, Taps4{})), (tile(BF16{}, Taps4{})))
    } else {
      HXM_BY_DTYPE(dtype, (tile(F32{}, Taps8{})), (tile(BF16{}, Taps8{})))
    }
  } else {
    HXM_BY_DTYPE(dtype,
                 (causal_conv_kernel<F32><<<grid, block, 0, s>>>((float*)y, y_stride, (const float*)u, u_stride, w, bias, act, state, slot_stride,
                                                                 slots, tok_seq, q_cu, positions, channels, taps, (float*)y2, y2_stride, w2,
                                                                 bias2, skip)),
                 (causal_conv_kernel<BF16><<<grid, block, 0, s>>>((u16*)y, y_stride, (const u16*)u, u_stride, w, bias, act, state, slot_stride,
                                                                  slots, tok_seq, q_cu, positions, channels, taps, (u16*)y2, y2_stride, w2,
                                                                  bias2, skip)))
  }
  int rc = hxm::check_launch();
  if (rc != HX_OK || taps == 1) return rc;
  HXM_BY_DTYPE(dtype,
               (causal_conv_state_kernel<F32><<<sgrid, block, 0, s>>>((const float*)u, u_stride, state, slot_stride, slots, q_cu, positions,
                                                                      channels, taps)),
               (causal_conv_state_kernel<BF16><<<sgrid, block, 0, s>>>((const u16*)u, u_stride, state, slot_stride, slots, q_cu, positions,
                                                                       channels, taps)))
  return hxm::check_launch();
}

extern "C" int hxm_causal_conv(void* y, int64_t y_stride, const void* u, int64_t u_stride, const float* w, const float* bias, int act,
                               float* state, int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                               const int32_t* positions, int64_t n_tokens, int32_t n_seq, int32_t channels, int32_t taps, int dtype,
                               void* stream) {
  return causal_conv_launch(y, y_stride, u, u_stride, w, bias, act, state, slot_stride, slots, tok_seq, q_cu, positions, n_tokens, n_seq,
                            channels, taps, dtype, stream, nullptr, 0, nullptr, nullptr, 0);
}

extern "C" int hxm_causal_conv_pair(void* y, int64_t y_stride, void* y2, int64_t y2_stride, const void* u, int64_t u_stride,
                                    const float* w, const float* w2, const float* bias, const float* bias2, int act, int skip,
                                    float* state, int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq,
                                    const int32_t* q_cu, const int32_t* positions, int64_t n_tokens, int32_t n_seq, int32_t channels,
                                    int32_t taps, int dtype, void* stream) {
  return causal_conv_launch(y, y_stride, u, u_stride, w, bias, act, state, slot_stride, slots, tok_seq, q_cu, positions, n_tokens, n_seq,
                            channels, taps, dtype, stream, y2, y2_stride, w2, bias2, skip);
}

extern "C" int hxm_token_shift_mix(void* out, const void* h, int64_t h_stride, const float* mu, int32_t n_mix, float* state,
                                   int64_t slot_stride, const int32_t* slots, const int32_t* tok_seq, const int32_t* q_cu,
                                   const int32_t* positions, int64_t n_tokens, int32_t n_seq, int64_t width, int dtype, void* stream) {
  if (n_tokens < 0 || n_seq < 0 || width < 1 || n_mix < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0 || n_seq == 0) return HX_OK;
  if (!out || !h || !mu || !state || !slots || !tok_seq || !q_cu || !positions) return HX_ERR_NULL;
  if (h_stride < width) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), sgrid((unsigned)n_seq), block(256);
  const uintptr_t es = dtype == HX_F32 ? 4 : 2;
  const int vec = width % 4 == 0 && h_stride % 4 == 0 && slot_stride % 4 == 0 && (uintptr_t)h % (4 * es) == 0 && (uintptr_t)out % (4 * es) == 0 &&
                  (uintptr_t)mu % 16 == 0 && (uintptr_t)state % 16 == 0;
  HXM_BY_DTYPE(dtype,
               (token_shift_mix_kernel<F32><<<grid, block, 0, s>>>((float*)out, (const float*)h, h_stride, mu, n_mix, state, slot_stride, slots,
                                                                   tok_seq, q_cu, positions, n_tokens, width, vec)),
               (token_shift_mix_kernel<BF16><<<grid, block, 0, s>>>((u16*)out, (const u16*)h, h_stride, mu, n_mix, state, slot_stride, slots,
                                                                    tok_seq, q_cu, positions, n_tokens, width, vec)))
  int rc = hxm::check_launch();
  if (rc != HX_OK) return rc;
  HXM_BY_DTYPE(dtype,
               (token_shift_state_kernel<F32><<<sgrid, block, 0, s>>>((const float*)h, h_stride, state, slot_stride, slots, q_cu, width)),
               (token_shift_state_kernel<BF16><<<sgrid, block, 0, s>>>((const u16*)h, h_stride, state, slot_stride, slots, q_cu, width)))
  return hxm::check_launch();
}

extern "C" int hxm_clamped_glu(void* y, int64_t y_stride, const void* gate, int64_t gate_stride, const void* up, int64_t up_stride,
                               float limit, float alpha, float up_shift, int64_t rows, int64_t n, int dtype, void* stream) {
  if (rows < 0 || n < 1) return HX_ERR_SHAPE;
  if (rows == 0) return HX_OK;
  if (!y || !gate || !up) return HX_ERR_NULL;
  if (y_stride < n || gate_stride < n || up_stride < n) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const uintptr_t es = dtype == HX_F32 ? 4 : 2;
  const int vec = n % 4 == 0 && y_stride % 4 == 0 && gate_stride % 4 == 0 && up_stride % 4 == 0 && (uintptr_t)y % (4 * es) == 0 &&
                  (uintptr_t)gate % (4 * es) == 0 && (uintptr_t)up % (4 * es) == 0;
  const dim3 grid(flat_blocks(vec ? rows * n / 4 : rows * n)), block(256);
  HXM_BY_DTYPE(dtype,
               (clamped_glu_kernel<F32><<<grid, block, 0, s>>>((float*)y, y_stride, (const float*)gate, gate_stride, (const float*)up, up_stride,
                                                               limit, alpha, up_shift, rows, n, vec)),
               (clamped_glu_kernel<BF16><<<grid, block, 0, s>>>((u16*)y, y_stride, (const u16*)gate, gate_stride, (const u16*)up, up_stride,
                                                                limit, alpha, up_shift, rows, n, vec)))
  return hxm::check_launch();
}

extern "C" int hxm_unary(void* out, int64_t out_stride, const void* x, int64_t x_stride, int act, int64_t rows, int64_t n, int dtype,
                         void* stream) {
  if (rows < 0 || n < 1) return HX_ERR_SHAPE;
  if (rows == 0) return HX_OK;
  if (!out || !x) return HX_ERR_NULL;
  if (out_stride < n || x_stride < n) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_blocks(rows * n)), block(256);
  HXM_BY_DTYPE(dtype, (unary_kernel<F32><<<grid, block, 0, s>>>((float*)out, out_stride, (const float*)x, x_stride, act, rows, n)),
               (unary_kernel<BF16><<<grid, block, 0, s>>>((u16*)out, out_stride, (const u16*)x, x_stride, act, rows, n)))
  return hxm::check_launch();
}

extern "C" int hxm_head_gates(float* decay, float* step, float* beta, const void* a, int64_t a_stride, const void* b, int64_t b_stride,
                              const float* log_rate, const float* step_bias, int64_t n_tokens, int32_t heads, int dtype, void* stream) {
  if (n_tokens < 0 || heads < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!decay || !a || !log_rate || !step_bias || (beta && !b)) return HX_ERR_NULL;
  if (a_stride < heads || (b && b_stride < heads)) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_blocks(n_tokens * heads)), block(256);
  HXM_BY_DTYPE(dtype,
               (head_gates_kernel<F32><<<grid, block, 0, s>>>(decay, step, beta, (const float*)a, a_stride, (const float*)b, b_stride, log_rate,
                                                              step_bias, n_tokens, heads)),
               (head_gates_kernel<BF16><<<grid, block, 0, s>>>(decay, step, beta, (const u16*)a, a_stride, (const u16*)b, b_stride, log_rate,
                                                               step_bias, n_tokens, heads)))
  return hxm::check_launch();
}

extern "C" int hxm_decay_exp(float* decay, const void* x, int64_t x_stride, const float* bias, int64_t rows, int64_t n, int dtype,
                             void* stream) {
  if (rows < 0 || n < 1) return HX_ERR_SHAPE;
  if (rows == 0) return HX_OK;
  if (!decay || !x) return HX_ERR_NULL;
  if (x_stride < n) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_blocks(rows * n)), block(256);
  HXM_BY_DTYPE(dtype, (decay_exp_kernel<F32><<<grid, block, 0, s>>>(decay, (const float*)x, x_stride, bias, rows, n)),
               (decay_exp_kernel<BF16><<<grid, block, 0, s>>>(decay, (const u16*)x, x_stride, bias, rows, n)))
  return hxm::check_launch();
}

extern "C" int hxm_unit_norm(float* out, const void* x, int64_t x_stride, float eps, float scale, int64_t n_tokens, int32_t heads,
                             int32_t dim, int dtype, void* stream) {
  if (n_tokens < 0 || heads < 1 || dim < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!out || !x) return HX_ERR_NULL;
  if (x_stride < (int64_t)heads * dim) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((n_tokens * heads + 3) / 4)), block(256);
  HXM_BY_DTYPE(dtype, (unit_norm_kernel<F32><<<grid, block, 0, s>>>(out, (const float*)x, x_stride, eps, scale, n_tokens, heads, dim)),
               (unit_norm_kernel<BF16><<<grid, block, 0, s>>>(out, (const u16*)x, x_stride, eps, scale, n_tokens, heads, dim)))
  return hxm::check_launch();
}

extern "C" int hxm_head_norm_rope_cache(const hxm_head_rope_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_head_rope_args& a = *args;
  if (a.n_tokens < 0 || a.q_heads < 0 || a.kv_heads < 0 || a.q_heads + a.kv_heads < 1 || a.dim < 1 || a.rot_dims < 0 || a.rot_dims > a.dim ||
      (a.rot_dims & 1))
    return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.positions || (a.rot_dims && !a.inv_freq)) return HX_ERR_NULL;
  if (a.q_heads && (!a.q || !a.q_out || !a.q_w)) return HX_ERR_NULL;
  if (a.kv_heads && (!a.k || !a.k_w || !a.slot_ids || !a.key_cache || !a.value_cache)) return HX_ERR_NULL;
  if ((a.q_heads && a.q_stride < (int64_t)a.q_heads * a.dim) || (a.kv_heads && a.k_stride < (int64_t)a.kv_heads * a.dim)) return HX_ERR_STRIDE;
  if (a.kv_heads && (a.head_stride < a.dim || a.cache_row_stride < a.head_stride * a.kv_heads)) return HX_ERR_STRIDE;
  const size_t lds = ((size_t)(a.q_heads + a.kv_heads) * a.dim + (size_t)a.rot_dims) * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)a.n_tokens), block(256);
  HXM_BY_DTYPE(a.dtype, (head_norm_rope_cache_kernel<F32><<<grid, block, lds, s>>>(a)),
               (head_norm_rope_cache_kernel<BF16><<<grid, block, lds, s>>>(a)))
  return hxm::check_launch();
}

extern "C" int hxm_gated_group_norm(const hxm_group_norm_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_group_norm_args& a = *args;
  if (a.rows < 0 || a.n < 1 || a.n > 0x7fffffff || a.group < 0 || (a.group > 0 && a.n % a.group) || (a.w && a.w_len < 1) || (a.skip && a.skip_group < 1))
    return HX_ERR_SHAPE;
  if (a.rows == 0) return HX_OK;
  if (!a.out || !a.x || (a.skip && !a.skip_w)) return HX_ERR_NULL;
  if (a.out_stride < a.n || a.x_stride < a.n || (a.skip && a.skip_stride < a.n) || (a.gate && a.gate_stride < a.n)) return HX_ERR_STRIDE;
  if (a.x_dtype != HX_F32 && a.x_dtype != a.dtype) return HX_ERR_DTYPE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t gs = a.group > 0 ? a.group : (a.n < 1024 ? a.n : 1024);
  const int64_t items = a.rows * ((a.n + gs - 1) / gs);
  const dim3 grid((unsigned)((items + 3) / 4)), block(256);
  const uintptr_t es = a.dtype == HX_F32 ? 4 : 2, xs = a.x_dtype == HX_F32 ? 4 : 2;
  auto by4 = [](const void* p, int64_t stride, uintptr_t e) { return ((uintptr_t)p % (4 * e)) == 0 && stride % 4 == 0; };
  const int vec = gs % 4 == 0 && a.n % 4 == 0 && by4(a.x, a.x_stride, xs) && by4(a.out, a.out_stride, es) && by4(a.skip, a.skip_stride, es) &&
                  by4(a.gate, a.gate_stride, es);
  const int64_t small_gs = a.group > 0 ? a.group : (a.n < 128 ? a.n : 128);
  if (vec && small_gs <= 128) {
    int lpg = 1;
    while (4 * lpg < small_gs) lpg <<= 1;
    const int64_t small_items = a.rows * ((a.n + small_gs - 1) / small_gs);
    const int64_t waves = (small_items + 64 / lpg - 1) / (64 / lpg);
    const dim3 sgrid((unsigned)((waves + 3) / 4));
    if (a.dtype == HX_F32) gated_group_norm_small_kernel<F32, F32><<<sgrid, block, 0, s>>>(a, lpg);
    else if (a.dtype == HX_BF16 && a.x_dtype == HX_F32) gated_group_norm_small_kernel<BF16, F32><<<sgrid, block, 0, s>>>(a, lpg);
    else if (a.dtype == HX_BF16) gated_group_norm_small_kernel<BF16, BF16><<<sgrid, block, 0, s>>>(a, lpg);
    else return HX_ERR_DTYPE;
    return hxm::check_launch();
  }
  if (a.dtype == HX_F32) {
    gated_group_norm_kernel<F32, F32><<<grid, block, 0, s>>>(a, vec);
  } else if (a.dtype == HX_BF16) {
    if (a.x_dtype == HX_F32) gated_group_norm_kernel<BF16, F32><<<grid, block, 0, s>>>(a, vec);
    else gated_group_norm_kernel<BF16, BF16><<<grid, block, 0, s>>>(a, vec);
  } else {
    return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
