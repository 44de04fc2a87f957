// state_scan.hip — the recurrence of a matrix state S [dim, vdim] per head and sequence, token by token in float:
//   HXM_SCAN_DECAY:  S <- a S + k (s v)^T;  o = S^T q                      (state-space duality: a, s one per head)
//   HXM_SCAN_BONUS:  o = (S + diag(u) k v^T)^T q;  S <- diag(a) S + k v^T   (time mixing: a one per key channel)
//   HXM_SCAN_DELTA:  S <- a S;  S <- S + k (b (v - S^T k))^T;  o = S^T q    (gated delta rule)
// a is either one number per (token, head) or one per key channel.  Several heads may share one q / k head.
//
// A workgroup of four waves takes up to 4 * 64 / PARTS value channels (columns of S) of one (sequence, head).  The PARTS
// lanes that share a column sit next to each other and hold KR key channels (rows of S) each, so the sums over key
// channels that a token needs — the read-out, and for the delta rule S^T k BEFORE the write — are KR products a lane and
// a few DPP steps: nothing leaves the wave and no barrier stands in the serial chain.  Tokens go by in chunks of TC: the
// chunk's q, k (and per-channel decays) come once per workgroup as float into LDS, zero-padded to PARTS * KR channels, and
// are read back 16 bytes at a time; the next chunk is on its way into registers while the current one is scanned (two LDS
// images, one barrier a chunk), so the serial chain waits for no global load.  The state comes from the sequence's slot
// (zeros for a portion that starts at position 0) and goes back.
#include "hx_common.h"
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

__device__ __forceinline__ float load_one(const void* row, int dtype, int64_t e) {
  return dtype == HX_F32 ? ((const float*)row)[e] : BF16::to_float(((const u16*)row)[e]);
}

// sum over the PARTS neighbouring lanes that share a column; every one of them ends with the sum
template <int PARTS>
__device__ __forceinline__ float parts_sum(float v) {
  v += dpp_move<kDppXor1>(v);
  v += dpp_move<kDppXor2>(v);
  if (PARTS >= 8) v += dpp_move<kDppHalfMirror>(v);
  if (PARTS >= 16) v += dpp_move<kDppMirror>(v);
  return v;
}

// One operand's chunk [TC tokens][KP channels] on its way from global memory (rows of `dtype`, K valid channels) to LDS:
// thread `tid` of 256 holds NI groups of four channels.
template <int TC, int KP>
struct ChunkRegs {
  static constexpr int kGroups = TC * KP / 4;
  static constexpr int NI = (kGroups + 255) / 256;
  f32x4 r[NI];

  __device__ __forceinline__ void fetch(const void* base, int dtype, int64_t stride, int64_t first_elem, int K, int64_t t0, int n_tok,
                                        bool by4, int tid) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int g = tid + i * 256;
      const int row = g / (KP / 4), c = (g % (KP / 4)) * 4;
      f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
      if (g < kGroups && row < n_tok && c < K) {
        const int64_t e = (t0 + row) * stride + first_elem + c;
        if (by4 && c + 3 < K) {
          if (dtype == HX_F32) {
            v = *reinterpret_cast<const f32x4*>((const float*)base + e);
          } else {
            const u16x4 b = *reinterpret_cast<const u16x4*>((const u16*)base + e);
            v = f32x4{BF16::to_float(b[0]), BF16::to_float(b[1]), BF16::to_float(b[2]), BF16::to_float(b[3])};
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (c + j < K) v[j] = load_one(base, dtype, e + j);
        }
      }
      r[i] = v;
    }
  }

  __device__ __forceinline__ void store(float* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int g = tid + i * 256;
      if (g < kGroups) *reinterpret_cast<f32x4*>(lds + 4 * g) = r[i];
    }
  }
};

template <int KR, int PARTS, int TC, int MODE, bool VEC>
__global__ __launch_bounds__(256) void state_scan_kernel(hxm_state_scan_args a) {
  constexpr int KP = KR * PARTS, CPW = 64 / PARTS, COLS = 4 * CPW;
  constexpr int kImage = TC * KP * (VEC ? 3 : 2) + TC * COLS + TC * 4;       // floats of one LDS image
  __shared__ __attribute__((aligned(16))) float lds[2 * kImage];
  const int seq = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int part = lane % PARTS, colw = wave * CPW + lane / PARTS;
  const int col0 = (int)blockIdx.z * COLS, col = col0 + colw;
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
  if (MODE == HXM_SCAN_BONUS) {
#pragma unroll
    for (int r = 0; r < KR; ++r) u[r] = first + r < K ? a.bonus[(int64_t)head * K + first + r] : 0.f;
  }
  // four channels at a time where every row of an operand starts on a multiple of four elements
  auto by4 = [&](const void* p, int dtype, int64_t stride) {
    const uintptr_t es = dtype == HX_F32 ? 4 : 2;
    return K % 4 == 0 && stride % 4 == 0 && ((uintptr_t)p % (4 * es)) == 0;
  };
  const bool vq = by4(a.q, a.q_dtype, a.q_stride), vk = by4(a.k, a.k_dtype, a.k_stride), va = VEC && by4(a.decay, HX_F32, 4);
  const int64_t qk_first = (int64_t)qk_head * K;
  ChunkRegs<TC, KP> rq, rk, rd;
  float rv[(TC * COLS + 255) / 256], rs[3];
  auto fetch = [&](int64_t t0) {
    const int n_tok = (int)(t_end - t0 < TC ? t_end - t0 : TC);
    rq.fetch(a.q, a.q_dtype, a.q_stride, qk_first, K, t0, n_tok, vq, tid);
    rk.fetch(a.k, a.k_dtype, a.k_stride, qk_first, K, t0, n_tok, vk, tid);
    if (VEC) rd.fetch(a.decay, HX_F32, (int64_t)a.heads * K, (int64_t)head * K, K, t0, n_tok, va, tid);
#pragma unroll
    for (int i = 0; i < (TC * COLS + 255) / 256; ++i) {
      const int e = tid + i * 256, row = e / COLS, c = col0 + e % COLS;
      rv[i] = (e < TC * COLS && row < n_tok && c < V) ? load_one(a.v, a.v_dtype, (t0 + row) * a.v_stride + (int64_t)head * V + c) : 0.f;
    }
    if (tid < TC) {
      const bool ok = tid < n_tok;
      const int64_t th = (t0 + tid) * a.heads + head;
      rs[0] = (!VEC && ok) ? a.decay[th] : 1.f;
      rs[1] = (MODE == HXM_SCAN_DECAY && a.vscale && ok) ? a.vscale[th] : 1.f;
      rs[2] = (MODE == HXM_SCAN_DELTA && ok) ? a.beta[th] : 0.f;
    }
  };
  auto store = [&](float* img) {
    rq.store(img, tid);
    rk.store(img + TC * KP, tid);
    if (VEC) rd.store(img + 2 * TC * KP, tid);
    float* vs = img + TC * KP * (VEC ? 3 : 2);
#pragma unroll
    for (int i = 0; i < (TC * COLS + 255) / 256; ++i) {
      const int e = tid + i * 256;
      if (e < TC * COLS) vs[e] = rv[i];
    }
    if (tid < TC) {
      float* sc = vs + TC * COLS + 4 * tid;
      sc[0] = rs[0]; sc[1] = rs[1]; sc[2] = rs[2];
    }
  };
  fetch(t_begin);
  store(lds);
  __syncthreads();
  int cur = 0;
  for (int64_t t0 = t_begin; t0 < t_end; t0 += TC, cur ^= 1) {
    const bool more = t0 + TC < t_end;
    if (more) fetch(t0 + TC);
    const float* img = lds + cur * kImage;
    const float* vs = img + TC * KP * (VEC ? 3 : 2);
    const float* sc = vs + TC * COLS;
    const int n_tok = (int)(t_end - t0 < TC ? t_end - t0 : TC);
    if (col0 + wave * CPW < V) {          // (a wave whose columns all lie past vdim only helps to bring the chunks in)
      auto token = [&](int j) {
        float q[KR], k[KR], d[VEC ? KR : 1];
#pragma unroll
        for (int r = 0; r < KR / 4; ++r) {
          const f32x4 q4 = *reinterpret_cast<const f32x4*>(img + j * KP + first + 4 * r);
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(img + TC * KP + j * KP + first + 4 * r);
#pragma unroll
          for (int x = 0; x < 4; ++x) { q[4 * r + x] = q4[x]; k[4 * r + x] = k4[x]; }
          if constexpr (VEC) {
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(img + 2 * TC * KP + j * KP + first + 4 * r);
#pragma unroll
            for (int x = 0; x < 4; ++x) d[4 * r + x] = d4[x];
          }
        }
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(sc + 4 * j);
        if constexpr (!VEC) d[0] = s4[0];
        const float v = vs[j * COLS + colw];
        float o = 0.f;
        if (MODE == HXM_SCAN_DECAY) {
          const float vv = v * s4[1];
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            S[r] = d[VEC ? r : 0] * S[r] + k[r] * vv;
            o += S[r] * q[r];
          }
        } else if (MODE == HXM_SCAN_BONUS) {
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            const float kv = k[r] * v;
            o += (S[r] + u[r] * kv) * q[r];
            S[r] = d[VEC ? r : 0] * S[r] + kv;
          }
        } else {
          float sk = 0.f;
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            S[r] *= d[VEC ? r : 0];
            sk += S[r] * k[r];
          }
          sk = parts_sum<PARTS>(sk);
          const float w = s4[2] * (v - sk);
#pragma unroll
          for (int r = 0; r < KR; ++r) {
            S[r] += k[r] * w;
            o += S[r] * q[r];
          }
        }
        o = parts_sum<PARTS>(o);
        if (part == 0 && col_ok) a.out[(t0 + j) * ((int64_t)a.heads * V) + (int64_t)head * V + col] = o;
      };
      if (n_tok == TC) {                  // a whole chunk: unrolled, so that the reads of the next tokens start early
#pragma unroll 4
        for (int j = 0; j < TC; ++j) token(j);
      } else {
        for (int j = 0; j < n_tok; ++j) token(j);
      }
    }
    if (more) store(lds + (cur ^ 1) * kImage);
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int kk = first + r;
    if (col_ok && kk < K) slot[(int64_t)kk * V + col] = S[r];
  }
}

template <int KR, int PARTS, int TC, int MODE>
int launch_mode(const hxm_state_scan_args& a, hipStream_t s) {
  const int cols = 4 * (64 / PARTS);
  const dim3 grid((unsigned)a.n_seq, (unsigned)a.heads, (unsigned)((a.vdim + cols - 1) / cols)), block(256);
  if (a.decay_per_channel) state_scan_kernel<KR, PARTS, TC, MODE, true><<<grid, block, 0, s>>>(a);
  else state_scan_kernel<KR, PARTS, TC, MODE, false><<<grid, block, 0, s>>>(a);
  return hxm::check_launch();
}

template <int KR, int PARTS, int TC>
int launch_rows(const hxm_state_scan_args& a, hipStream_t s) {
  switch (a.mode) {
    case HXM_SCAN_DECAY: return launch_mode<KR, PARTS, TC, HXM_SCAN_DECAY>(a, s);
    case HXM_SCAN_BONUS: return launch_mode<KR, PARTS, TC, HXM_SCAN_BONUS>(a, s);
    case HXM_SCAN_DELTA: return launch_mode<KR, PARTS, TC, HXM_SCAN_DELTA>(a, s);
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
  // key channels a lane x lanes a column: 8 x 4, 8 x 8, 16 x 8, 16 x 16 (chunks of 16 tokens; 8 at the widest)
  if (a.dim <= 32) return launch_rows<8, 4, 16>(a, s);
  if (a.dim <= 64) return launch_rows<8, 8, 16>(a, s);
  if (a.dim <= 128) return launch_rows<16, 8, 16>(a, s);
  return launch_rows<16, 16, 8>(a, s);
}
