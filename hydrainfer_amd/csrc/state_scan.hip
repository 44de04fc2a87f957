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
// (zeros for a portion that starts at position 0) and goes back.  KR x PARTS follows the key size (8 x 4 ... 16 x 16); a
// launch of prompts with few workgroups takes more lanes a column, a batch of single tokens two columns a lane.
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
// thread `tid` of 256 holds NI groups of four channels AS THEY CAME (float bits, or four bfloat16 in two words).  Nothing is
// computed on them before store(): the scan between fetch() and store() then waits for no load.
template <int TC, int KP>
struct ChunkRegs {
  static constexpr int kGroups = TC * KP / 4;
  static constexpr int NI = (kGroups + 255) / 256;
  u32x4 r[NI];

  __device__ __forceinline__ void fetch(const void* base, int dtype, int64_t stride, int64_t first_elem, int K, int64_t t0, int n_tok,
                                        bool by4, int tid) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int g = tid + i * 256;
      const int row = g / (KP / 4), c = (g % (KP / 4)) * 4;
      u32x4 v = u32x4{0u, 0u, 0u, 0u};
      if (g < kGroups && row < n_tok && c < K) {
        const int64_t e = (t0 + row) * stride + first_elem + c;
        if (by4 && c + 3 < K) {
          if (dtype == HX_F32) {
            v = *reinterpret_cast<const u32x4*>((const float*)base + e);
          } else {
            const u32x2 b = *reinterpret_cast<const u32x2*>((const u16*)base + e);
            v[0] = b[0];
            v[1] = b[1];
          }
        } else if (dtype == HX_F32) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (c + j < K) v[j] = ((const uint32_t*)base)[e + j];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (c + j < K) v[j >> 1] |= (uint32_t)((const u16*)base)[e + j] << (16 * (j & 1));
        }
      }
      r[i] = v;
    }
  }

  __device__ __forceinline__ void store(float* lds, int dtype, int tid) const {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int g = tid + i * 256;
      if (g < kGroups) {
        u32x4 v = r[i];
        if (dtype != HX_F32) v = u32x4{v[0] << 16, v[0] & 0xffff0000u, v[1] << 16, v[1] & 0xffff0000u};
        *reinterpret_cast<u32x4*>(lds + 4 * g) = v;
      }
    }
  }
};

template <int KR, int PARTS, int TC, int CPL, int MODE, bool VEC>
__global__ __launch_bounds__(256) void state_scan_kernel(hxm_state_scan_args a) {
  constexpr int KP = KR * PARTS, CPW = 64 / PARTS, COLS = 4 * CPW * CPL;      // a lane owns CPL columns, 4 * CPW apart
  constexpr int kImage = TC * KP * (VEC ? 3 : 2) + TC * COLS + TC * 4;       // floats of one LDS image
  __shared__ __attribute__((aligned(16))) float lds[2 * kImage];
  const int seq = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int part = lane % PARTS, colw = wave * CPW + lane / PARTS;
  const int col0 = (int)blockIdx.z * COLS;
  const int K = a.dim, V = a.vdim;
  int col[CPL];
  bool col_ok[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    col[c] = col0 + c * 4 * CPW + colw;
    col_ok[c] = col[c] < V;
  }
  const int64_t t_begin = a.q_cu[seq], t_end = a.q_cu[seq + 1];
  if (t_end <= t_begin) return;
  const int first = part * KR;
  const int qk_head = head / (a.heads / a.qk_heads);
  float* slot = a.state + (int64_t)a.slots[seq] * a.slot_stride + (int64_t)head * K * V;
  const bool fresh = a.positions[t_begin] == 0;
  float S[CPL][KR];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int kk = first + r;
      S[c][r] = (!fresh && col_ok[c] && kk < K) ? slot[(int64_t)kk * V + col[c]] : 0.f;
    }
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
  constexpr int NV = (TC * COLS + 255) / 256;
  uint32_t rv[NV];                   // the chunk's values as they came (float bits or one bfloat16)
  float rs[3];
  int rs_ok = 0;
  auto fetch = [&](int64_t t0) {
    const int n_tok = (int)(t_end - t0 < TC ? t_end - t0 : TC);
    rq.fetch(a.q, a.q_dtype, a.q_stride, qk_first, K, t0, n_tok, vq, tid);
    rk.fetch(a.k, a.k_dtype, a.k_stride, qk_first, K, t0, n_tok, vk, tid);
    if (VEC) rd.fetch(a.decay, HX_F32, (int64_t)a.heads * K, (int64_t)head * K, K, t0, n_tok, va, tid);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256, row = e / COLS, c = col0 + e % COLS;
      rv[i] = 0u;
      if (e < TC * COLS && row < n_tok && c < V) {
        const int64_t at = (t0 + row) * a.v_stride + (int64_t)head * V + c;
        rv[i] = a.v_dtype == HX_F32 ? ((const uint32_t*)a.v)[at] : (uint32_t)((const u16*)a.v)[at];
      }
    }
    if (tid < TC) {
      rs_ok = tid < n_tok;
      const int64_t th = (t0 + (rs_ok ? tid : 0)) * a.heads + head;          // (a row past the portion reads the chunk's first: unused)
      rs[0] = VEC ? 1.f : a.decay[th];
      rs[1] = (MODE == HXM_SCAN_DECAY && a.vscale) ? a.vscale[th] : 1.f;
      rs[2] = MODE == HXM_SCAN_DELTA ? a.beta[th] : 0.f;
    }
  };
  auto store = [&](float* img) {
    rq.store(img, a.q_dtype, tid);
    rk.store(img + TC * KP, a.k_dtype, tid);
    if (VEC) rd.store(img + 2 * TC * KP, HX_F32, tid);
    float* vs = img + TC * KP * (VEC ? 3 : 2);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + i * 256;
      if (e < TC * COLS) vs[e] = __builtin_bit_cast(float, a.v_dtype == HX_F32 ? rv[i] : rv[i] << 16);
    }
    if (tid < TC) {
      float* sc = vs + TC * COLS + 4 * tid;
      sc[0] = rs_ok ? rs[0] : 1.f; sc[1] = rs_ok ? rs[1] : 1.f; sc[2] = rs_ok ? rs[2] : 0.f;
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
      struct Ops {
        float q[KR], k[KR], d[VEC ? KR : 1], v[CPL];
        f32x4 s4;
      };
      auto read = [&](Ops& x, int j) {
#pragma unroll
        for (int r = 0; r < KR / 4; ++r) {
          const f32x4 q4 = *reinterpret_cast<const f32x4*>(img + j * KP + first + 4 * r);
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(img + TC * KP + j * KP + first + 4 * r);
#pragma unroll
          for (int e = 0; e < 4; ++e) { x.q[4 * r + e] = q4[e]; x.k[4 * r + e] = k4[e]; }
          if constexpr (VEC) {
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(img + 2 * TC * KP + j * KP + first + 4 * r);
#pragma unroll
            for (int e = 0; e < 4; ++e) x.d[4 * r + e] = d4[e];
          }
        }
        x.s4 = *reinterpret_cast<const f32x4*>(sc + 4 * j);
        if constexpr (!VEC) x.d[0] = x.s4[0];
#pragma unroll
        for (int c = 0; c < CPL; ++c) x.v[c] = vs[j * COLS + c * 4 * CPW + colw];
      };
      auto compute = [&](const Ops& x, int j) {
        const float* q = x.q;
        const float* k = x.k;
        const float* d = x.d;
        const float* v = x.v;
        const f32x4 s4 = x.s4;
        float o[CPL];
#pragma unroll
        for (int c = 0; c < CPL; ++c) o[c] = 0.f;
        if (MODE == HXM_SCAN_DECAY) {
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            const float vv = v[c] * s4[1];
#pragma unroll
            for (int r = 0; r < KR; ++r) {
              S[c][r] = d[VEC ? r : 0] * S[c][r] + k[r] * vv;
              o[c] += S[c][r] * q[r];
            }
          }
        } else if (MODE == HXM_SCAN_BONUS) {
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
#pragma unroll
            for (int r = 0; r < KR; ++r) {
              const float kv = k[r] * v[c];
              o[c] += (S[c][r] + u[r] * kv) * q[r];
              S[c][r] = d[VEC ? r : 0] * S[c][r] + kv;
            }
          }
        } else {
          float sk[CPL];
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            sk[c] = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
              S[c][r] *= d[VEC ? r : 0];
              sk[c] += S[c][r] * k[r];
            }
          }
#pragma unroll
          for (int c = 0; c < CPL; ++c) sk[c] = parts_sum<PARTS>(sk[c]);
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            const float w = s4[2] * (v[c] - sk[c]);
#pragma unroll
            for (int r = 0; r < KR; ++r) {
              S[c][r] += k[r] * w;
              o[c] += S[c][r] * q[r];
            }
          }
        }
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          o[c] = parts_sum<PARTS>(o[c]);
          if (part == 0 && col_ok[c]) a.out[(t0 + j) * ((int64_t)a.heads * V) + (int64_t)head * V + col[c]] = o[c];
        }
      };
      if (n_tok == TC) {                  // a whole chunk: two sets of operands, one read from LDS while the other is worked on
        Ops x0, x1;
        read(x0, 0);
#pragma unroll 2
        for (int j = 0; j < TC; j += 2) {
          read(x1, j + 1);
          compute(x0, j);
          if (j + 2 < TC) read(x0, j + 2);
          compute(x1, j + 1);
        }
      } else {
        Ops x0;
        for (int j = 0; j < n_tok; ++j) {
          read(x0, j);
          compute(x0, j);
        }
      }
    }
    if (more) store(lds + (cur ^ 1) * kImage);
    __syncthreads();
  }
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int kk = first + r;
      if (col_ok[c] && kk < K) slot[(int64_t)kk * V + col[c]] = S[c][r];
    }
  }
}

template <int KR, int PARTS, int TC, int CPL, int MODE>
int launch_cols(const hxm_state_scan_args& a, hipStream_t s) {
  const int cols = 4 * (64 / PARTS) * CPL;
  const dim3 grid((unsigned)a.n_seq, (unsigned)a.heads, (unsigned)((a.vdim + cols - 1) / cols)), block(256);
  if (a.decay_per_channel) state_scan_kernel<KR, PARTS, TC, CPL, MODE, true><<<grid, block, 0, s>>>(a);
  else state_scan_kernel<KR, PARTS, TC, CPL, MODE, false><<<grid, block, 0, s>>>(a);
  return hxm::check_launch();
}

// A batch of single tokens (decode steps) is bound by the states it moves: two columns a lane, so half as many workgroups
// bring q / k / decays in.  Portions of prompts are bound by a wave's arithmetic per token: one column a lane (two measured
// 35 - 50 % slower there).
template <int KR, int PARTS, int TC, int MODE>
int launch_mode(const hxm_state_scan_args& a, hipStream_t s) {
  if (a.vdim >= 8 * (64 / PARTS) && a.n_tokens == a.n_seq) return launch_cols<KR, PARTS, TC, 2, MODE>(a, s);
  return launch_cols<KR, PARTS, TC, 1, MODE>(a, s);
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
  // key channels a lane x lanes a column: 8 x 4, 8 x 8, 16 x 8, 16 x 16 (chunks of 16 tokens; 8 at the widest).  Portions of
  // prompts in a launch that would leave compute units without a workgroup take twice the lanes a column and half the key
  // channels a lane: twice the waves, each with half the serial work per token (measured at 4 x 1024 tokens, states of
  // 128 x 128: 338 -> 290 us with 256 workgroups, 394 -> 435 us with 512; decode steps 26 -> 43 us: their state rows get
  // too short).
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 1) v = 256;
    n_cu = v;
  }
  const bool prompt = a.n_tokens > a.n_seq;
  auto few = [&](int cols) { return prompt && (int64_t)a.n_seq * a.heads * ((a.vdim + cols - 1) / cols) <= n_cu; };
  if (a.dim <= 32) return launch_rows<8, 4, 16>(a, s);
  if (a.dim <= 64) return few(32) ? launch_rows<4, 16, 16>(a, s) : launch_rows<8, 8, 16>(a, s);
  if (a.dim <= 128) return few(32) ? launch_rows<8, 16, 16>(a, s) : launch_rows<16, 8, 16>(a, s);
  return launch_rows<16, 16, 8>(a, s);
}
