// rope_ops.hip — rotary positions as one row kernel over "parts".  A part is a group of heads of a token's row (queries,
// keys, values, or a mixer's result) of which a range of channels turns by the token's position: pairs (i, i + dims / 2)
// ("halves") or (2 i, 2 i + 1) ("interleaved"), forwards or backwards, cos and sin optionally scaled; the other channels are
// copied.  A part goes to rows of an output matrix or into the paged cache (at a column offset, so that a latent and a
// rotated key part can share a cache row), and may be multiplied by a sigmoid gate per head or per element on the way.
// One launch takes up to three parts — q, k and v of an attention layer — so what a token's projection row needs before
// attention is one kernel, and what a head's result needs after it (turning rotated values back, the output gate) another.
// Angles are position * frequency in double and reduced to [-pi, pi] there; cos and sin of the remainder are float.
#include "hx_common.h"
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

constexpr int kMaxRotPairs = 512;

// two neighbouring channels of an activation row at once
template <typename A> struct Two;
template <> struct Two<F32> {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ void load(const float* p, float& a, float& b) {
    const f32x2 t = *reinterpret_cast<const f32x2*>(p);
    a = t[0]; b = t[1];
  }
  static __device__ __forceinline__ void store(float* p, float a, float b) { *reinterpret_cast<f32x2*>(p) = f32x2{a, b}; }
};
template <> struct Two<BF16> {
  static __device__ __forceinline__ void load(const u16* p, float& a, float& b) {
    const uint32_t t = *reinterpret_cast<const uint32_t*>(p);
    a = __builtin_bit_cast(float, t << 16); b = __builtin_bit_cast(float, t & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(u16* p, float a, float b) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)BF16::from_float(a) | ((uint32_t)BF16::from_float(b) << 16);
  }
};

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// `pairs`: bit q set = part q's offsets, sizes and strides are even and its pointers aligned to two elements, so a lane
// moves two neighbouring channels at a time (halves: channels c, c + 1 and their partners c + half, c + half + 1 together).
template <typename A>
__global__ __launch_bounds__(256) void rotary_parts_kernel(hxm_rotary_args a, int pairs) {
  __shared__ float cs[kMaxRotPairs], sn[kMaxRotPairs];
  typedef typename A::storage T;
  const int64_t t = blockIdx.x;
  const double p = (double)a.positions[t];
  for (int q = 0; q < a.n_parts; ++q) {
    const hxm_rotary_part& pt = a.parts[q];
    const int half = pt.inv_freq ? pt.rot_dims / 2 : 0;
    // queries and keys turn alike: the table of the part before serves when it is the same
    const bool same = q > 0 && pt.inv_freq == a.parts[q - 1].inv_freq && pt.rot_dims == a.parts[q - 1].rot_dims &&
                      pt.mag == a.parts[q - 1].mag && pt.sign == a.parts[q - 1].sign;
    if (!same) {
      __syncthreads();      // the last part's table is no longer read
      for (int i = threadIdx.x; i < half; i += 256) {
        // the angle in double, brought into [-pi, pi] there (two-term 2 pi), then the float sine and cosine of the remainder:
        // what is lost is the remainder's float rounding, whatever the position
        const double ang = p * pt.inv_freq[i];
        const double turns = rint(ang * 0.15915494309189535);
        const float r = (float)fma(-turns, 2.4492935982947064e-16, fma(-turns, 6.283185307179586, ang));
        float s_, c_;
        sincosf(r, &s_, &c_);
        cs[i] = c_ * pt.mag;
        sn[i] = s_ * pt.mag * pt.sign;
      }
      __syncthreads();
    }
    const T* src = (const T*)pt.src + t * pt.src_stride;
    T* dst;
    if (pt.to_cache) {
      const int64_t slot = a.slot_ids[t];
      if (slot < 0) continue;      // (the whole workgroup: the barriers above are still reached by all)
      dst = (T*)pt.dst + (slot / a.block_size) * pt.cache_block_stride + (slot % a.block_size) * pt.dst_stride;
    } else {
      dst = (T*)pt.dst + t * pt.dst_stride;
    }
    const T* gate = pt.gate ? (const T*)pt.gate + t * pt.gate_stride : nullptr;
    const int plain = pt.size - 2 * half;                  // channels of a head that do not turn
    const bool per_head = pt.gate_kind == HXM_GATE_PER_HEAD;
    if ((pairs >> q) & 1) {
      const bool halves = pt.layout == HXM_ROT_HALVES;
      const int turning = halves ? half / 2 : half;        // items that turn: four channels (halves) or one pair (interleaved)
      const int per_head_items = turning + plain / 2;
      const int items = pt.heads * per_head_items;
      for (int e = threadIdx.x; e < items; e += 256) {
        const int h = e / per_head_items, i = e - h * per_head_items;
        const T* s = src + (int64_t)h * pt.src_head_stride;
        T* d = dst + (int64_t)h * pt.dst_head_stride;
        const float gh = gate && per_head ? sigmoidf_(A::to_float(gate[h])) : 1.0f;
        const T* ge = gate && !per_head ? gate + (int64_t)h * pt.size : nullptr;
        if (i < turning && halves) {
          const int c0 = pt.rot_off + 2 * i, c1 = c0 + half;
          float u0, u1, v0, v1;
          Two<A>::load(s + c0, u0, u1);
          Two<A>::load(s + c1, v0, v1);
          float o0 = u0 * cs[2 * i] - v0 * sn[2 * i], o1 = u1 * cs[2 * i + 1] - v1 * sn[2 * i + 1];
          float o2 = v0 * cs[2 * i] + u0 * sn[2 * i], o3 = v1 * cs[2 * i + 1] + u1 * sn[2 * i + 1];
          if (ge) {
            float g0, g1, g2, g3;
            Two<A>::load(ge + c0, g0, g1);
            Two<A>::load(ge + c1, g2, g3);
            o0 *= sigmoidf_(g0); o1 *= sigmoidf_(g1); o2 *= sigmoidf_(g2); o3 *= sigmoidf_(g3);
          }
          Two<A>::store(d + c0, o0 * gh, o1 * gh);
          Two<A>::store(d + c1, o2 * gh, o3 * gh);
        } else if (i < turning) {
          const int c0 = pt.rot_off + 2 * i;
          float u, v;
          Two<A>::load(s + c0, u, v);
          float o0 = u * cs[i] - v * sn[i], o1 = v * cs[i] + u * sn[i];
          if (ge) {
            float g0, g1;
            Two<A>::load(ge + c0, g0, g1);
            o0 *= sigmoidf_(g0); o1 *= sigmoidf_(g1);
          }
          Two<A>::store(d + c0, o0 * gh, o1 * gh);
        } else {
          const int j = 2 * (i - turning);
          const int c = j < pt.rot_off ? j : j + 2 * half;
          float u, v;
          Two<A>::load(s + c, u, v);
          if (ge) {
            float g0, g1;
            Two<A>::load(ge + c, g0, g1);
            u *= sigmoidf_(g0); v *= sigmoidf_(g1);
          }
          Two<A>::store(d + c, u * gh, v * gh);
        }
      }
      continue;
    }
    const int per_head_items = half + plain;               // work items of a head: a pair, or a single channel
    const int items = pt.heads * per_head_items;
    for (int e = threadIdx.x; e < items; e += 256) {
      const int h = e / per_head_items, i = e - h * per_head_items;
      const T* s = src + (int64_t)h * pt.src_head_stride;
      T* d = dst + (int64_t)h * pt.dst_head_stride;
      if (i < half) {
        const int i0 = pt.rot_off + (pt.layout == HXM_ROT_HALVES ? i : 2 * i);
        const int i1 = pt.layout == HXM_ROT_HALVES ? i0 + half : i0 + 1;
        const float u = A::to_float(s[i0]), v = A::to_float(s[i1]);
        float o0 = u * cs[i] - v * sn[i], o1 = v * cs[i] + u * sn[i];
        if (gate) {
          if (per_head) {
            const float g = sigmoidf_(A::to_float(gate[h]));
            o0 *= g;
            o1 *= g;
          } else {
            o0 *= sigmoidf_(A::to_float(gate[(int64_t)h * pt.size + i0]));
            o1 *= sigmoidf_(A::to_float(gate[(int64_t)h * pt.size + i1]));
          }
        }
        d[i0] = A::from_float(o0);
        d[i1] = A::from_float(o1);
      } else {
        const int j = i - half;
        const int c = j < pt.rot_off ? j : j + 2 * half;
        if (gate) {
          const float z = A::to_float(gate[per_head ? (int64_t)h : (int64_t)h * pt.size + c]);
          d[c] = A::from_float(A::to_float(s[c]) * sigmoidf_(z));
        } else {
          d[c] = s[c];
        }
      }
    }
  }
}

// eight neighbouring channels at once: 16 bytes of bfloat16, 32 of float
template <typename A> struct Eight;
template <> struct Eight<F32> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
};
template <> struct Eight<BF16> {
  static __device__ __forceinline__ void load(const u16* p, float (&v)[8]) {
    const u16x8 a = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = BF16::to_float(a[i]);
  }
  static __device__ __forceinline__ void store(u16* p, const float (&v)[8]) {
    u16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = BF16::from_float(v[i]);
    *reinterpret_cast<u16x8*>(p) = a;
  }
};

// The same with eight neighbouring channels a lane (every part's offsets, sizes and strides multiples of eight, pointers
// aligned to eight elements) and `tpw` tokens a workgroup, 256 / tpw threads each: halves — channels c .. c + 7 and their
// partners c + half .. together; interleaved — four pairs.  A token's cos / sin table is cs[local token * half + pair].
template <typename A>
__global__ __launch_bounds__(256) void rotary_parts_wide_kernel(hxm_rotary_args a, int tpw) {
  __shared__ float cs[kMaxRotPairs], sn[kMaxRotPairs];
  typedef typename A::storage T;
  const int tpt = 256 / tpw;                                // threads of a token
  const int tl = threadIdx.x / tpt, lane = threadIdx.x - tl * tpt;
  const int64_t t0 = (int64_t)blockIdx.x * tpw, t = t0 + tl;
  const bool live = t < a.n_tokens;
  for (int q = 0; q < a.n_parts; ++q) {
    const hxm_rotary_part& pt = a.parts[q];
    const int half = pt.inv_freq ? pt.rot_dims / 2 : 0;
    const bool same = q > 0 && pt.inv_freq == a.parts[q - 1].inv_freq && pt.rot_dims == a.parts[q - 1].rot_dims &&
                      pt.mag == a.parts[q - 1].mag && pt.sign == a.parts[q - 1].sign;
    if (!same) {
      __syncthreads();
      for (int e = threadIdx.x; e < tpw * half; e += 256) {
        const int k = e / half, i = e - k * half;
        const int64_t tk = t0 + k < a.n_tokens ? t0 + k : a.n_tokens - 1;
        const double ang = (double)a.positions[tk] * pt.inv_freq[i];
        const double turns = rint(ang * 0.15915494309189535);
        const float r = (float)fma(-turns, 2.4492935982947064e-16, fma(-turns, 6.283185307179586, ang));
        float s_, c_;
        sincosf(r, &s_, &c_);
        cs[e] = c_ * pt.mag;
        sn[e] = s_ * pt.mag * pt.sign;
      }
      __syncthreads();
    }
    if (!live) continue;
    const float* ct = cs + tl * half;
    const float* st = sn + tl * half;
    const T* src = (const T*)pt.src + t * pt.src_stride;
    T* dst;
    if (pt.to_cache) {
      const int64_t slot = a.slot_ids[t];
      if (slot < 0) continue;      // (only this token's threads; the barriers above are passed by all before)
      dst = (T*)pt.dst + (slot / a.block_size) * pt.cache_block_stride + (slot % a.block_size) * pt.dst_stride;
    } else {
      dst = (T*)pt.dst + t * pt.dst_stride;
    }
    const T* gate = pt.gate ? (const T*)pt.gate + t * pt.gate_stride : nullptr;
    const bool per_head = pt.gate_kind == HXM_GATE_PER_HEAD;
    const bool halves = pt.layout == HXM_ROT_HALVES;
    const int turning = halves ? half / 8 : half / 4;       // items that turn: 8 + 8 channels (halves) or 8 channels = 4 pairs
    const int per_head_items = turning + (pt.size - 2 * half) / 8;
    const int items = pt.heads * per_head_items;
    for (int e = lane; e < items; e += tpt) {
      const int h = e / per_head_items, i = e - h * per_head_items;
      const T* s = src + (int64_t)h * pt.src_head_stride;
      T* d = dst + (int64_t)h * pt.dst_head_stride;
      const float gh = gate && per_head ? sigmoidf_(A::to_float(gate[h])) : 1.0f;
      const T* ge = gate && !per_head ? gate + (int64_t)h * pt.size : nullptr;
      float u[8], v[8], g[8];
      if (i < turning && halves) {
        const int c0 = pt.rot_off + 8 * i, c1 = c0 + half;
        Eight<A>::load(s + c0, u);
        Eight<A>::load(s + c1, v);
        float o0[8], o1[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float c_ = ct[8 * i + k], s_ = st[8 * i + k];
          o0[k] = (u[k] * c_ - v[k] * s_) * gh;
          o1[k] = (v[k] * c_ + u[k] * s_) * gh;
        }
        if (ge) {
          Eight<A>::load(ge + c0, g);
#pragma unroll
          for (int k = 0; k < 8; ++k) o0[k] *= sigmoidf_(g[k]);
          Eight<A>::load(ge + c1, g);
#pragma unroll
          for (int k = 0; k < 8; ++k) o1[k] *= sigmoidf_(g[k]);
        }
        Eight<A>::store(d + c0, o0);
        Eight<A>::store(d + c1, o1);
      } else {
        const bool turns = i < turning;
        const int j = 8 * (i - turning);
        const int c = turns ? pt.rot_off + 8 * i : (j < pt.rot_off ? j : j + 2 * half);
        Eight<A>::load(s + c, u);
        if (turns) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float c_ = ct[4 * i + k], s_ = st[4 * i + k];
            v[2 * k] = u[2 * k] * c_ - u[2 * k + 1] * s_;
            v[2 * k + 1] = u[2 * k + 1] * c_ + u[2 * k] * s_;
          }
        } else {
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] = u[k];
        }
        if (ge) {
          Eight<A>::load(ge + c, g);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] *= sigmoidf_(g[k]);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] *= gh;
        Eight<A>::store(d + c, v);
      }
    }
  }
}

}  // namespace

extern "C" int hxm_rotary_parts(const hxm_rotary_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_rotary_args& a = *args;
  if (a.n_tokens < 0 || a.n_parts < 1 || a.n_parts > HXM_ROT_MAX_PARTS) return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.positions) return HX_ERR_NULL;
  for (int q = 0; q < a.n_parts; ++q) {
    const hxm_rotary_part& p = a.parts[q];
    if (!p.src || !p.dst) return HX_ERR_NULL;
    if (p.heads < 1 || p.size < 1 || p.rot_off < 0) return HX_ERR_SHAPE;
    if (p.inv_freq && (p.rot_dims < 2 || p.rot_dims % 2 || p.rot_off + p.rot_dims > p.size || p.rot_dims / 2 > kMaxRotPairs)) return HX_ERR_SHAPE;
    if (p.layout != HXM_ROT_HALVES && p.layout != HXM_ROT_INTERLEAVED) return HX_ERR_SHAPE;
    if (p.src_head_stride < p.size || p.dst_head_stride < p.size) return HX_ERR_STRIDE;
    if (p.to_cache && (!a.slot_ids || a.block_size < 1)) return HX_ERR_NULL;
    if (p.gate && p.gate_kind != HXM_GATE_PER_HEAD && p.gate_kind != HXM_GATE_PER_ELEMENT) return HX_ERR_SHAPE;
  }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)a.n_tokens), block(256);
  int pairs = 0;
  const uintptr_t two = a.dtype == HX_F32 ? 8 : 4;
  for (int q = 0; q < a.n_parts; ++q) {
    const hxm_rotary_part& p = a.parts[q];
    const int half = p.inv_freq ? p.rot_dims / 2 : 0;
    const bool even = p.size % 2 == 0 && p.rot_off % 2 == 0 && (p.layout == HXM_ROT_INTERLEAVED || half % 2 == 0) &&
                      p.src_stride % 2 == 0 && p.src_head_stride % 2 == 0 && p.dst_stride % 2 == 0 && p.dst_head_stride % 2 == 0 &&
                      p.cache_block_stride % 2 == 0 && (uintptr_t)p.src % two == 0 && (uintptr_t)p.dst % two == 0 &&
                      (!p.gate || p.gate_kind == HXM_GATE_PER_HEAD || (p.gate_stride % 2 == 0 && (uintptr_t)p.gate % two == 0));
    if (even) pairs |= 1 << q;
  }
  // eight channels a lane where every part allows it; tokens a workgroup so that a part's items fill its threads
  bool wide = true;
  int most = 1, widest = 0;
  const uintptr_t eight = a.dtype == HX_F32 ? 16 : 16;
  for (int q = 0; q < a.n_parts; ++q) {
    const hxm_rotary_part& p = a.parts[q];
    const int half = p.inv_freq ? p.rot_dims / 2 : 0;
    wide = wide && p.size % 8 == 0 && p.rot_off % 8 == 0 && half % 8 == 0 && p.src_stride % 8 == 0 && p.src_head_stride % 8 == 0 &&
           p.dst_stride % 8 == 0 && p.dst_head_stride % 8 == 0 && p.cache_block_stride % 8 == 0 && (uintptr_t)p.src % eight == 0 &&
           (uintptr_t)p.dst % eight == 0 && (!p.gate || p.gate_kind == HXM_GATE_PER_HEAD || (p.gate_stride % 8 == 0 && (uintptr_t)p.gate % eight == 0));
    const int turning = p.layout == HXM_ROT_HALVES ? half / 8 : half / 4;
    const int items = p.heads * (turning + (p.size - 2 * half) / 8);
    most = items > most ? items : most;
    widest = half > widest ? half : widest;
  }
  if (wide) {
    int tpw = 1;
    while (tpw < 8 && most * tpw * 2 <= 256 && widest * tpw * 2 <= kMaxRotPairs) tpw *= 2;
    const dim3 wgrid((unsigned)((a.n_tokens + tpw - 1) / tpw));
    switch (a.dtype) {
      case HX_F32: rotary_parts_wide_kernel<F32><<<wgrid, block, 0, s>>>(a, tpw); break;
      case HX_BF16: rotary_parts_wide_kernel<BF16><<<wgrid, block, 0, s>>>(a, tpw); break;
      default: return HX_ERR_DTYPE;
    }
    return hxm::check_launch();
  }
  switch (a.dtype) {
    case HX_F32: rotary_parts_kernel<F32><<<grid, block, 0, s>>>(a, pairs); break;
    case HX_BF16: rotary_parts_kernel<BF16><<<grid, block, 0, s>>>(a, pairs); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
