// state_scan.hip — the recurrence of a matrix state S [dim, vdim] per head and sequence, token by token in float:
//   HXM_SCAN_DECAY:  S <- a S + k (s v)^T;  o = S^T q                      (state-space duality: a, s one per head)
//   HXM_SCAN_BONUS:  o = (S + diag(u) k v^T)^T q;  S <- diag(a) S + k v^T   (time mixing: a one per key channel)
//   HXM_SCAN_DELTA:  S <- a S;  S <- S + k (b (v - S^T k))^T;  o = S^T q    (gated delta rule)
// a is either one number per (token, head) or one per key channel.  Several heads may share one q / k head.
//
// A wave takes 16 value channels (columns of S) of one (sequence, head); the four lanes of a quad share a column and hold a
// quarter of its key channels (rows of S) each, KR registers a lane.  The sums over key channels that a token needs — the
// read-out, and for the delta rule S^T k BEFORE the write — are KR products a lane and two DPP quad steps: nothing leaves
// the wave and no barrier stands in the serial chain.  The next token's operands are requested before the current one is
// worked on.  The state comes from the sequence's slot (zeros for a portion that starts at position 0) and goes back.
#include "hx_common.h"
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

// KR consecutive elements of a row starting at element `first` (rows past `n` read as zero); vec: 4 at a time
template <int KR>
__device__ __forceinline__ void load_part(float (&dst)[KR], const void* row, int dtype, int first, int n, bool vec) {
  if (vec && first + KR <= n) {
    if (dtype == HX_F32) {
      const f32x4* p = reinterpret_cast<const f32x4*>((const float*)row + first);
#pragma unroll
      for (int r = 0; r < KR / 4; ++r) {
        const f32x4 v = p[r];
        dst[4 * r] = v[0]; dst[4 * r + 1] = v[1]; dst[4 * r + 2] = v[2]; dst[4 * r + 3] = v[3];
      }
    } else {
      const u16x4* p = reinterpret_cast<const u16x4*>((const u16*)row + first);
#pragma unroll
      for (int r = 0; r < KR / 4; ++r) {
        const u16x4 v = p[r];
        dst[4 * r] = BF16::to_float(v[0]); dst[4 * r + 1] = BF16::to_float(v[1]);
        dst[4 * r + 2] = BF16::to_float(v[2]); dst[4 * r + 3] = BF16::to_float(v[3]);
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int e = first + r;
    dst[r] = e < n ? (dtype == HX_F32 ? ((const float*)row)[e] : BF16::to_float(((const u16*)row)[e])) : 0.f;
  }
}

__device__ __forceinline__ float load_one(const void* row, int dtype, int e) {
  return dtype == HX_F32 ? ((const float*)row)[e] : BF16::to_float(((const u16*)row)[e]);
}

__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  return v;
}

template <int KR, bool VEC>
struct Operands {
  float q[KR], k[KR];
  float a[VEC ? KR : 1];
  float v, s, b;
};

template <int KR, int MODE, bool VEC>
__device__ __forceinline__ void fetch(Operands<KR, VEC>& o, const hxm_state_scan_args& a, int64_t t, int head, int qk_head, int first,
                                      int col, bool col_ok, bool vq, bool vk, bool va) {
  const int K = a.dim;
  const int es_q = a.q_dtype == HX_F32 ? 4 : 2, es_k = a.k_dtype == HX_F32 ? 4 : 2, es_v = a.v_dtype == HX_F32 ? 4 : 2;
  load_part<KR>(o.q, (const char*)a.q + (t * a.q_stride + (int64_t)qk_head * K) * es_q, a.q_dtype, first, K, vq);
  load_part<KR>(o.k, (const char*)a.k + (t * a.k_stride + (int64_t)qk_head * K) * es_k, a.k_dtype, first, K, vk);
  o.v = col_ok ? load_one((const char*)a.v + (t * a.v_stride + (int64_t)head * a.vdim) * es_v, a.v_dtype, col) : 0.f;
  if constexpr (VEC) {
    load_part<KR>(o.a, a.decay + (t * a.heads + head) * (int64_t)K, HX_F32, first, K, va);
  } else {
    o.a[0] = a.decay[t * a.heads + head];
  }
  o.s = (MODE == HXM_SCAN_DECAY && a.vscale) ? a.vscale[t * a.heads + head] : 1.f;
  o.b = MODE == HXM_SCAN_DELTA ? a.beta[t * a.heads + head] : 1.f;
}

template <int KR, int MODE, bool VEC>
__global__ __launch_bounds__(256) void state_scan_kernel(hxm_state_scan_args a) {
  const int seq = blockIdx.x, head = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int part = lane & 3;
  const int col = ((int)blockIdx.z * (int)(blockDim.x >> 6) + wave) * 16 + (lane >> 2);
  const int K = a.dim, V = a.vdim;
  const bool col_ok = col < V;
  const int64_t t_begin = a.q_cu[seq], t_end = a.q_cu[seq + 1];
  if (t_end <= t_begin) return;
  const int first = part * KR;
  const int qk_head = head / (a.heads / a.qk_heads);
  float* slot = a.state + (int64_t)a.slots[seq] * a.slot_stride + (int64_t)head * K * V;
  const bool fresh = a.positions[t_begin] == 0;
  float S[KR];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int kk = first + r;
    S[r] = (!fresh && col_ok && kk < K) ? slot[(int64_t)kk * V + col] : 0.f;
  }
  float u[KR];
  if (MODE == HXM_SCAN_BONUS) load_part<KR>(u, a.bonus + (int64_t)head * K, HX_F32, first, K, false);
  // 4 elements at a time where every row of an operand starts on a multiple of four elements
  auto by4 = [&](const void* p, int dtype, int64_t stride) {
    const uintptr_t es = dtype == HX_F32 ? 4 : 2;
    return K % 4 == 0 && stride % 4 == 0 && ((uintptr_t)p % (4 * es)) == 0;
  };
  const bool vq = by4(a.q, a.q_dtype, a.q_stride), vk = by4(a.k, a.k_dtype, a.k_stride);
  const bool va = VEC && by4(a.decay, HX_F32, 4);
  Operands<KR, VEC> cur, nxt;
  fetch<KR, MODE, VEC>(cur, a, t_begin, head, qk_head, first, col, col_ok, vq, vk, va);
  for (int64_t t = t_begin; t < t_end; ++t) {
    if (t + 1 < t_end) fetch<KR, MODE, VEC>(nxt, a, t + 1, head, qk_head, first, col, col_ok, vq, vk, va);
    float o = 0.f;
    if (MODE == HXM_SCAN_DECAY) {
      const float vv = cur.v * cur.s;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        S[r] = cur.a[VEC ? r : 0] * S[r] + cur.k[r] * vv;
        o += S[r] * cur.q[r];
      }
      o = quad_sum(o);
    } else if (MODE == HXM_SCAN_BONUS) {
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const float kv = cur.k[r] * cur.v;
        o += (S[r] + u[r] * kv) * cur.q[r];
        S[r] = cur.a[VEC ? r : 0] * S[r] + kv;
      }
      o = quad_sum(o);
    } else {
      float sk = 0.f;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        S[r] *= cur.a[VEC ? r : 0];
        sk += S[r] * cur.k[r];
      }
      sk = quad_sum(sk);
      const float w = cur.b * (cur.v - sk);
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        S[r] += cur.k[r] * w;
        o += S[r] * cur.q[r];
      }
      o = quad_sum(o);
    }
    if (part == 0 && col_ok) a.out[t * ((int64_t)a.heads * V) + (int64_t)head * V + col] = o;
    cur = nxt;
  }
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int kk = first + r;
    if (col_ok && kk < K) slot[(int64_t)kk * V + col] = S[r];
  }
}

template <int KR, int MODE>
int launch_mode(const hxm_state_scan_args& a, dim3 grid, dim3 block, hipStream_t s) {
  if (a.decay_per_channel) state_scan_kernel<KR, MODE, true><<<grid, block, 0, s>>>(a);
  else state_scan_kernel<KR, MODE, false><<<grid, block, 0, s>>>(a);
  return hxm::check_launch();
}

template <int KR>
int launch_rows(const hxm_state_scan_args& a, dim3 grid, dim3 block, hipStream_t s) {
  switch (a.mode) {
    case HXM_SCAN_DECAY: return launch_mode<KR, HXM_SCAN_DECAY>(a, grid, block, s);
    case HXM_SCAN_BONUS: return launch_mode<KR, HXM_SCAN_BONUS>(a, grid, block, s);
    case HXM_SCAN_DELTA: return launch_mode<KR, HXM_SCAN_DELTA>(a, grid, block, s);
    default: return HX_ERR_UNSUPPORTED;
  }
}

}  // namespace

extern "C" int hxm_state_scan(const hxm_state_scan_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_state_scan_args& a = *args;
  if (a.n_tokens < 0 || a.n_seq < 0 || a.heads < 1 || a.qk_heads < 1 || a.heads % a.qk_heads || a.dim < 1 || a.dim > 256 || a.vdim < 1)
    return HX_ERR_SHAPE;
  if (a.n_tokens == 0 || a.n_seq == 0) return HX_OK;
  if (!a.out || !a.q || !a.k || !a.v || !a.decay || !a.state || !a.slots || !a.q_cu || !a.positions) return HX_ERR_NULL;
  if ((a.mode == HXM_SCAN_DELTA && !a.beta) || (a.mode == HXM_SCAN_BONUS && !a.bonus)) return HX_ERR_NULL;
  for (int d : {a.q_dtype, a.k_dtype, a.v_dtype})
    if (d != HX_F32 && d != HX_BF16) return HX_ERR_DTYPE;
  if (a.q_stride < (int64_t)a.qk_heads * a.dim || a.k_stride < (int64_t)a.qk_heads * a.dim || a.v_stride < (int64_t)a.heads * a.vdim)
    return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int col_waves = (a.vdim + 15) / 16;
  const int nw = col_waves < 4 ? col_waves : 4;
  const dim3 grid((unsigned)a.n_seq, (unsigned)a.heads, (unsigned)((col_waves + nw - 1) / nw)), block(64 * nw);
  if (a.dim <= 32) return launch_rows<8>(a, grid, block, s);
  if (a.dim <= 64) return launch_rows<16>(a, grid, block, s);
  if (a.dim <= 128) return launch_rows<32>(a, grid, block, s);
  return launch_rows<64>(a, grid, block, s);
}
