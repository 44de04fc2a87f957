// moe_mix.hip — mixture of experts for the mix library: a softmax router whose choice can carry a bias, the plan that puts
// the (token, choice) pairs in expert-major order, the grouped product Y = act(X W_e^T) over the rows of every expert,
// and the weighted combine with an optional gated shared expert.  Nothing returns to the host between the router and the
// combine: the products are launched for the most rows there can be and find their expert from the plan's segments.
#include <cfloat>
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

constexpr int kMaxExperts = 1024;
constexpr int kPerLane = kMaxExperts / 64;

// one wave per token, lane l owns experts l, l + 64, ... (PER of them)
template <int PER>
__global__ __launch_bounds__(256) void route_softmax_topk_kernel(const float* __restrict__ logits, int64_t stride,
                                                                 const float* __restrict__ bias, int64_t n_tokens, int E,
                                                                 int top, float scale, float* __restrict__ weights,
                                                                 int32_t* __restrict__ experts, int renorm) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= n_tokens) return;
  const float* row = logits + t * stride;
  constexpr int per = PER;
  float s[PER], c[PER];
  float mx = -FLT_MAX;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    const int e = lane + 64 * i;
    s[i] = e < E ? row[e] : -FLT_MAX;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    const int e = lane + 64 * i;
    s[i] = e < E ? expf(s[i] - mx) : 0.f;
    sum += s[i];
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    const int e = lane + 64 * i;
    s[i] *= inv;
    c[i] = e < E ? s[i] + (bias ? bias[e] : 0.f) : -FLT_MAX;
  }
  float chosen_sum = 0.f, my_w = 0.f;      // lane k keeps the k-th choice
  int my_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -FLT_MAX;
    int best_e = INT32_MAX;
    float best_s = 0.f;
  #pragma unroll
  for (int i = 0; i < per; ++i) {
      const int e = lane + 64 * i;
      if (e < E && (c[i] > best)) {      // within a lane experts go up: the first of equals is the lower one
        best = c[i];
        best_e = e;
        best_s = s[i];
      }
    }
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oe = __shfl_xor(best_e, off, 64);
      const float os = __shfl_xor(best_s, off, 64);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
        best_s = os;
      }
    }
#pragma unroll
    for (int i = 0; i < per; ++i)
      if (lane + 64 * i == best_e) c[i] = -FLT_MAX;      // taken
    chosen_sum += best_s;
    if (lane == k % 64) {      // (top <= 64 is checked by the host)
      my_w = best_s;
      my_e = best_e;
    }
  }
  if (lane < top) {
    weights[t * top + lane] = (renorm ? my_w / (chosen_sum + 1e-20f) : my_w) * scale;
    experts[t * top + lane] = my_e;
  }
}

// one workgroup of 1024 threads: histogram, exclusive scan, scatter, all through LDS counters
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ experts, int64_t n, int top, int E,
                                                        int32_t* __restrict__ seg, int32_t* __restrict__ row_of,
                                                        int32_t* __restrict__ src) {
  __shared__ int32_t count[kMaxExperts];
  __shared__ int32_t cursor[kMaxExperts];
  for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += 1024) {
    const int e = experts[i];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
      cursor[e] = run;
      seg[e] = run;
      run += count[e];
    }
    seg[E] = run;
  }
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += 1024) {
    const int e = experts[i];
    if (e >= 0 && e < E) {
      const int32_t row = atomicAdd(&cursor[e], 1);
      row_of[i] = row;
      src[row] = (int32_t)(i / top);
    } else {
      row_of[i] = -1;
    }
  }
}

// the expert and the first row of row tile `tile` (tiles of TM rows, every expert's rows starting a tile of their own);
// false: the tile lies beyond the last expert's rows
__device__ __forceinline__ bool find_tile(const int32_t* __restrict__ seg, int E, int TM, int tile, int& expert, int& row0, int& row1) {
  int passed = 0;
  for (int e = 0; e < E; ++e) {
    const int lo = seg[e], hi = seg[e + 1];
    const int nt = (hi - lo + TM - 1) / TM;
    if (tile < passed + nt) {
      expert = e;
      row0 = lo + (tile - passed) * TM;
      row1 = hi < row0 + TM ? hi : row0 + TM;
      return true;
    }
    passed += nt;
  }
  return false;
}

__device__ __forceinline__ float act_apply(float v, int act) {
  if (act == 1) {
    v = fmaxf(v, 0.f);
    return v * v;
  }
  return v;
}

// General form (any dtype, any sizes): a workgroup takes 16 rows of one expert and 64 output columns; the rows' inputs go
// through LDS in slices of 64 k; thread (r, c): row r = tid / 16 ... each thread 4 columns.
constexpr int kGM = 16, kGN = 64, kGK = 64;
template <typename A>
__global__ __launch_bounds__(256) void grouped_linear_kernel(typename A::storage* __restrict__ y, const typename A::storage* __restrict__ x,
                                                             int64_t x_stride, const int32_t* __restrict__ src,
                                                             const typename A::storage* __restrict__ w,
                                                             const int32_t* __restrict__ seg, int E, int64_t N, int64_t K, int act) {
  __shared__ float xs[kGM][kGK + 1];
  __shared__ float ws[kGN][kGK + 1];
  int e, row0, row1;
  if (!find_tile(seg, E, kGM, blockIdx.y, e, row0, row1)) return;
  const int64_t col0 = (int64_t)blockIdx.x * kGN;
  const int r = threadIdx.x >> 4, cg = threadIdx.x & 15;      // row r, columns cg, cg + 16, cg + 32, cg + 48
  const typename A::storage* we = w + (int64_t)e * N * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int64_t k0 = 0; k0 < K; k0 += kGK) {
    for (int i = threadIdx.x; i < kGM * kGK; i += 256) {
      const int rr = i / kGK, kk = i - rr * kGK;
      float v = 0.f;
      if (row0 + rr < row1 && k0 + kk < K) {
        const int64_t sr = src ? (int64_t)src[row0 + rr] : (int64_t)(row0 + rr);
        v = A::to_float(x[sr * x_stride + k0 + kk]);
      }
      xs[rr][kk] = v;
    }
    for (int i = threadIdx.x; i < kGN * kGK; i += 256) {
      const int cc = i / kGK, kk = i - cc * kGK;
      ws[cc][kk] = (col0 + cc < N && k0 + kk < K) ? A::to_float(we[(col0 + cc) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kGK; ++kk) {
      const float xv = xs[r][kk];
      acc[0] += xv * ws[cg][kk];
      acc[1] += xv * ws[cg + 16][kk];
      acc[2] += xv * ws[cg + 32][kk];
      acc[3] += xv * ws[cg + 48][kk];
    }
    __syncthreads();
  }
  if (row0 + r < row1) {
    for (int j = 0; j < 4; ++j) {
      const int64_t c = col0 + cg + 16 * j;
      if (c < N) y[(int64_t)(row0 + r) * N + c] = A::from_float(act_apply(acc[j], act));
    }
  }
}

// MFMA form (bfloat16, K a multiple of 8, rows 16-byte aligned): a workgroup of four waves takes TM rows of one expert and
// TN output columns; the rows' inputs (gathered through src) and the expert's weight rows go through LDS in slices of 64
// k — the next slice is on its way into registers while the current one is multiplied — and every wave multiplies its
// (TM / WGM) x (TN / WGN) part with 16x16x32 MFMAs: lane l holds k 8 (l / 16) .. + 7 of row (A) or column (B) l % 16, the
// accumulator's lane l column l % 16 of rows 4 (l / 16) .. + 3.  Rows of LDS are padded to 72 elements (144 bytes): the
// sixteen rows a 16-byte read touches fall into different banks.
constexpr int kKS = 64, kLDK = 72;
template <int TM, int TN, int WGM, int WGN>
__global__ __launch_bounds__(256) void grouped_linear_tiled_kernel(u16* __restrict__ y, const u16* __restrict__ x, int64_t x_stride,
                                                                   const int32_t* __restrict__ src, const u16* __restrict__ w,
                                                                   const int32_t* __restrict__ seg, int E, int64_t N, int64_t K,
                                                                   int act) {
  constexpr int FM = TM / WGM / 16, FN = TN / WGN / 16;
  constexpr int PA = TM * 8 / 256, PB = TN * 8 / 256;      // 16-byte pieces of a slice a thread moves
  __shared__ __attribute__((aligned(16))) u16 As[TM * kLDK];
  __shared__ __attribute__((aligned(16))) u16 Bs[TN * kLDK];
  int e, row0, row1;
  if (!find_tile(seg, E, TM, blockIdx.y, e, row0, row1)) return;      // (the whole workgroup: no barrier is left waiting)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm0 = (wave / WGN) * (TM / WGM), wn0 = (wave % WGN) * (TN / WGN);
  const int64_t col0 = (int64_t)blockIdx.x * TN;
  const u16* we = w + (int64_t)e * N * K;
  const u16x8 zero8 = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
  const u16* pa[PA];
  const u16* pb[PB];
  int ka[PA], kb[PB];
#pragma unroll
  for (int p = 0; p < PA; ++p) {
    const int idx = threadIdx.x + 256 * p, r = idx >> 3;
    ka[p] = (idx & 7) * 8;
    pa[p] = nullptr;
    if (row0 + r < row1) pa[p] = x + (src ? (int64_t)src[row0 + r] : (int64_t)(row0 + r)) * x_stride + ka[p];
  }
#pragma unroll
  for (int p = 0; p < PB; ++p) {
    const int idx = threadIdx.x + 256 * p, c = idx >> 3;
    kb[p] = (idx & 7) * 8;
    pb[p] = col0 + c < N ? we + (col0 + c) * K + kb[p] : nullptr;
  }
  u16x8 ra[PA], rb[PB];
  auto fetch = [&](int64_t k0) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < PA; ++p) ra[p] = (pa[p] && k0 + ka[p] < K) ? *reinterpret_cast<const u16x8*>(pa[p] + k0) : zero8;
#pragma unroll
    for (int p = 0; p < PB; ++p) rb[p] = (pb[p] && k0 + kb[p] < K) ? *reinterpret_cast<const u16x8*>(pb[p] + k0) : zero8;
  };
  f32x4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int l16 = lane & 15, kq = lane >> 4;
  fetch(0);
  for (int64_t k0 = 0; k0 < K; k0 += kKS) {
#pragma unroll
    for (int p = 0; p < PA; ++p) *reinterpret_cast<u16x8*>(As + ((threadIdx.x + 256 * p) >> 3) * kLDK + ka[p]) = ra[p];
#pragma unroll
    for (int p = 0; p < PB; ++p) *reinterpret_cast<u16x8*>(Bs + ((threadIdx.x + 256 * p) >> 3) * kLDK + kb[p]) = rb[p];
    lds_barrier();      // (LDS only: the next slice's loads stay in flight)
    if (k0 + kKS < K) fetch(k0 + kKS);
#pragma unroll
    for (int ks = 0; ks < kKS / 32; ++ks) {
      u16x8 af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = *reinterpret_cast<const u16x8*>(As + (wm0 + 16 * i + l16) * kLDK + 32 * ks + 8 * kq);
#pragma unroll
      for (int j = 0; j < FN; ++j) bf[j] = *reinterpret_cast<const u16x8*>(Bs + (wn0 + 16 * j + l16) * kLDK + 32 * ks + 8 * kq);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[i]), __builtin_bit_cast(bf16x8, bf[j]),
                                                              acc[i][j], 0, 0, 0);
    }
    lds_barrier();      // (LDS only: the next slice's loads stay in flight)
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int64_t c = col0 + wn0 + 16 * j + l16;
      if (c >= N) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rr = row0 + wm0 + 16 * i + 4 * kq + r;
        if (rr < row1) y[(int64_t)rr * N + c] = BF16::from_float(act_apply(acc[i][j][r], act));
      }
    }
}

template <typename A>
__global__ __launch_bounds__(256) void moe_combine_kernel(typename A::storage* __restrict__ out, const typename A::storage* __restrict__ y,
                                                          const int32_t* __restrict__ row_of, const float* __restrict__ weights,
                                                          const typename A::storage* __restrict__ shared,
                                                          const float* __restrict__ shared_gate, int64_t gate_stride, int top,
                                                          int64_t W, const typename A::storage* __restrict__ identity,
                                                          int64_t identity_stride) {
  const int64_t t = blockIdx.x;
  const float g = shared ? 1.0f / (1.0f + expf(-shared_gate[t * gate_stride])) : 0.f;
  // a choice without a row (an expert past those the plan was made for) is an identity expert when `identity` is given
  float idw = 0.f;
  if (identity)
    for (int k = 0; k < top; ++k)
      if (row_of[t * top + k] < 0) idw += weights[t * top + k];
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    float u = 0.f;
    for (int k = 0; k < top; ++k) {
      const int32_t r = row_of[t * top + k];
      if (r >= 0) u += weights[t * top + k] * A::to_float(y[(int64_t)r * W + i]);
    }
    if (idw != 0.f) u += idw * A::to_float(identity[t * identity_stride + i]);
    if (shared) u += g * A::to_float(shared[t * W + i]);
    out[t * W + i] = A::from_float(u);
  }
}

}  // namespace

extern "C" int hxm_route_softmax_topk(const float* logits, int64_t logit_stride, const float* choice_bias, int64_t n_tokens,
                                      int32_t n_experts, int32_t top, float scale, int32_t renorm, float* weights,
                                      int32_t* experts, void* stream) {
  if (n_tokens < 0 || n_experts < 1 || n_experts > kMaxExperts || top < 1 || top > n_experts || top > 64) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!logits || !weights || !experts) return HX_ERR_NULL;
  if (logit_stride < n_experts) return HX_ERR_STRIDE;
  const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
  hipStream_t s = (hipStream_t)stream;
#define HXM_ROUTE(PER_) route_softmax_topk_kernel<PER_><<<grid, block, 0, s>>>(logits, logit_stride, choice_bias, n_tokens, \
                                                                              n_experts, top, scale, weights, experts, renorm)
  if (n_experts <= 64) HXM_ROUTE(1);
  else if (n_experts <= 128) HXM_ROUTE(2);
  else if (n_experts <= 256) HXM_ROUTE(4);
  else HXM_ROUTE(kPerLane);
#undef HXM_ROUTE
  return hxm::check_launch();
}

extern "C" int hxm_moe_plan(const int32_t* experts, int64_t n_tokens, int32_t top, int32_t n_experts, int32_t* seg,
                            int32_t* row_of, int32_t* src, void* stream) {
  if (n_tokens < 0 || top < 1 || n_experts < 1 || n_experts > kMaxExperts || n_tokens * top > INT32_MAX) return HX_ERR_SHAPE;
  if (!experts || !seg || !row_of || !src) return HX_ERR_NULL;
  moe_plan_kernel<<<dim3(1), dim3(1024), 0, (hipStream_t)stream>>>(experts, n_tokens * top, top, n_experts, seg, row_of, src);
  return hxm::check_launch();
}

extern "C" int hxm_grouped_linear(void* y, const void* x, int64_t x_stride, const int32_t* src, const void* w,
                                  const int32_t* seg, int64_t max_rows, int32_t n_experts, int64_t n_dim, int64_t k_dim,
                                  int32_t act, int dtype, void* stream) {
  if (max_rows < 0 || n_experts < 1 || n_experts > kMaxExperts || n_dim < 1 || k_dim < 1 || act < 0 || act > 1) return HX_ERR_SHAPE;
  if (max_rows == 0) return HX_OK;
  if (!y || !x || !w || !seg) return HX_ERR_NULL;
  if (x_stride < k_dim) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HX_BF16 && k_dim % 8 == 0 && x_stride % 8 == 0 && aligned16(x) && aligned16(w)) {
    // few rows an expert (decode steps): tiles of 32 rows, the four waves side by side over 128 columns; else 128 x 128
    const bool small = max_rows <= (int64_t)32 * n_experts;
    const int tm = small ? 32 : 128;
    const int64_t tiles = (max_rows + tm - 1) / tm + n_experts;      // every expert's rows start a tile of their own
    if (tiles > 65535) return HX_ERR_SHAPE;
    const dim3 grid((unsigned)((n_dim + 127) / 128), (unsigned)tiles);
    if (small)
      grouped_linear_tiled_kernel<32, 128, 1, 4><<<grid, dim3(256), 0, s>>>((u16*)y, (const u16*)x, x_stride, src, (const u16*)w, seg,
                                                                            n_experts, n_dim, k_dim, act);
    else
      grouped_linear_tiled_kernel<128, 128, 2, 2><<<grid, dim3(256), 0, s>>>((u16*)y, (const u16*)x, x_stride, src, (const u16*)w, seg,
                                                                             n_experts, n_dim, k_dim, act);
    return hxm::check_launch();
  }
  const int64_t tiles = (max_rows + kGM - 1) / kGM + n_experts;
  if (tiles > 65535) return HX_ERR_SHAPE;
  const dim3 grid((unsigned)((n_dim + kGN - 1) / kGN), (unsigned)tiles), block(256);
  switch (dtype) {
    case HX_F32:
      grouped_linear_kernel<F32><<<grid, block, 0, s>>>((float*)y, (const float*)x, x_stride, src, (const float*)w, seg, n_experts,
                                                        n_dim, k_dim, act);
      break;
    case HX_BF16:
      grouped_linear_kernel<BF16><<<grid, block, 0, s>>>((u16*)y, (const u16*)x, x_stride, src, (const u16*)w, seg, n_experts, n_dim,
                                                         k_dim, act);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_moe_combine(void* out, const void* y, const int32_t* row_of, const float* weights, const void* shared,
                               const float* shared_gate, int64_t gate_stride, const void* identity, int64_t identity_stride,
                               int64_t n_tokens, int32_t top, int64_t width, int dtype, void* stream) {
  if (n_tokens < 0 || top < 1 || width < 1) return HX_ERR_SHAPE;
  if (identity && identity_stride < width) return HX_ERR_STRIDE;
  if (n_tokens == 0) return HX_OK;
  if (!out || !y || !row_of || !weights || (shared && !shared_gate)) return HX_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), block(256);
  switch (dtype) {
    case HX_F32:
      moe_combine_kernel<F32><<<grid, block, 0, s>>>((float*)out, (const float*)y, row_of, weights, (const float*)shared, shared_gate,
                                                     gate_stride, top, width, (const float*)identity, identity_stride);
      break;
    case HX_BF16:
      moe_combine_kernel<BF16><<<grid, block, 0, s>>>((u16*)out, (const u16*)y, row_of, weights, (const u16*)shared, shared_gate,
                                                      gate_stride, top, width, (const u16*)identity, identity_stride);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
