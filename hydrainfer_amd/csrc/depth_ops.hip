// depth_ops.hip — the row kernels of depth-averaged hybrids: token + learned position embedding, the kernel that serves
// every place where a residual meets a layer norm (a sublayer's normed result enters the residual, the layer's result
// joins the stack of levels, the depth-weighted average of the levels becomes the next input, the next sublayer's input
// is normed), and the PolyNorm / squared-ReLU activations.  One 256-thread workgroup per row, the row staged in LDS,
// all arithmetic in float; only what a matrix product reads or writes has the activation dtype.
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

// sum of v over the 256 threads of the workgroup; part: 4 floats of LDS.  Ends with every thread holding the sum, and
// part free to be used again after the next barrier.
__device__ __forceinline__ float block_sum(float v, float* part) {
  v = wave_sum(v);
  __syncthreads();                       // the previous use of part is over
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  return part[0] + part[1] + part[2] + part[3];
}

// buf[0 .. W) -> (shift, 1 / spread): layer norm (mean, 1 / sqrt(var + eps)) or RMS norm (0, 1 / sqrt(mean square + eps))
__device__ __forceinline__ void row_stats(const float* buf, float* part, int64_t W, float eps, int rms, float& shift, float& inv) {
  float mean = 0.f;
  if (!rms) {
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < W; i += 256) s += buf[i];
    mean = block_sum(s, part) / (float)W;
  }
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    const float d = buf[i] - mean;
    ss += d * d;
  }
  ss = block_sum(ss, part);
  shift = mean;
  inv = 1.0f / sqrtf(ss / (float)W + eps);
}

template <typename A>
__global__ __launch_bounds__(256) void embed_positions_kernel(float* __restrict__ out, const typename A::storage* __restrict__ table,
                                                              const typename A::storage* __restrict__ pos_table,
                                                              const void* __restrict__ ids, int ids64,
                                                              const int32_t* __restrict__ positions, int64_t W, int64_t vocab,
                                                              int64_t n_pos) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids64 ? ((const int64_t*)ids)[t] : (int64_t)((const int32_t*)ids)[t];
  const int64_t p = pos_table ? (int64_t)positions[t] : -1;
  const bool ok = id >= 0 && id < vocab, pok = p >= 0 && p < n_pos;
  for (int64_t i = threadIdx.x; i < W; i += 256) {
    float v = ok ? A::to_float(table[id * W + i]) : 0.f;
    if (pok) v += A::to_float(pos_table[p * W + i]);
    out[t * W + i] = v;
  }
}

template <typename A>
__global__ __launch_bounds__(256) void depth_norm_kernel(hxm_depth_norm_args a) {
  extern __shared__ float lds[];
  float* buf = lds;                // [W]
  float* part = lds + a.width;     // [4]
  typedef typename A::storage T;
  const int64_t W = a.width, i_out = blockIdx.x;
  const int64_t r = a.rows ? (int64_t)a.rows[i_out] : i_out;
  const float* xin = a.x_in ? a.x_in + r * W : nullptr;
  if (a.y) {
    const T* y = (const T*)a.y + r * a.y_stride;
    for (int64_t i = threadIdx.x; i < W; i += 256) buf[i] = A::to_float(y[i]);
    float shift = 0.f, inv = 1.f;
    if (a.post_norm != HXM_POST_PLAIN) {
      __syncthreads();
      row_stats(buf, part, W, a.eps, a.post_norm == HXM_POST_SAME ? a.rms : a.post_norm == HXM_POST_RMS, shift, inv);
    }
    for (int64_t i = threadIdx.x; i < W; i += 256)
      buf[i] = (xin ? xin[i] : 0.f) + a.mult * ((buf[i] - shift) * inv * (a.post_w ? a.post_w[i] : 1.f));
  } else {
    for (int64_t i = threadIdx.x; i < W; i += 256) buf[i] = xin ? xin[i] : 0.f;
  }
  if (a.y2) {
    const T* y2 = (const T*)a.y2 + r * a.y2_stride;
    for (int64_t i = threadIdx.x; i < W; i += 256) buf[i] += A::to_float(y2[i]);
  }
  if (a.bias) {
    for (int64_t i = threadIdx.x; i < W; i += 256) buf[i] += a.bias[i];
  }
  // (every thread keeps to the elements i = tid + 256 k from here on: no barrier is needed until the next statistics)
  if (a.level_out) {
    float* lo = a.level_out + r * W;
    for (int64_t i = threadIdx.x; i < W; i += 256) lo[i] = buf[i];
  }
  if (a.depth_w) {
    for (int64_t i = threadIdx.x; i < W; i += 256) {
      float u = 0.f;
      for (int j = 0; j < a.n_levels; ++j) {
        const float* lv = a.levels + (int64_t)j * a.level_stride + r * W;
        // the level written above is taken from LDS: the store to it need not have landed
        const float v = (a.level_out && lv == a.level_out + r * W) ? buf[i] : lv[i];
        u += a.depth_w[j] * v;
      }
      buf[i] = u;
    }
  }
  if (a.x_out) {
    float* xo = a.x_out + i_out * W;
    for (int64_t i = threadIdx.x; i < W; i += 256) xo[i] = buf[i];
  }
  if (a.next_w) {
    __syncthreads();
    float shift, inv;
    row_stats(buf, part, W, a.eps, a.rms, shift, inv);
    T* h = (T*)a.h_out + i_out * a.h_stride;
    for (int64_t i = threadIdx.x; i < W; i += 256) h[i] = A::from_float((buf[i] - shift) * inv * a.next_w[i]);
  } else if (a.h_out) {      // no norm: the row itself in the activations' type
    T* h = (T*)a.h_out + i_out * a.h_stride;
    for (int64_t i = threadIdx.x; i < W; i += 256) h[i] = A::from_float(buf[i]);
  }
}

// The same, four elements a lane at a time: width, y's stride and every pointer are multiples of four elements.
__device__ __forceinline__ void row_stats4(const float* buf, float* part, int64_t W, float eps, int rms, float& shift, float& inv) {
  const f32x4* b4 = reinterpret_cast<const f32x4*>(buf);
  const int64_t n4 = W >> 2;
  float mean = 0.f;
  if (!rms) {
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      const f32x4 v = b4[i];
      s += (v[0] + v[1]) + (v[2] + v[3]);
    }
    mean = block_sum(s, part) / (float)W;
  }
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < n4; i += 256) {
    const f32x4 v = b4[i];
#pragma unroll
    for (int k = 0; k < 4; ++k) ss += (v[k] - mean) * (v[k] - mean);
  }
  ss = block_sum(ss, part);
  shift = mean;
  inv = 1.0f / sqrtf(ss / (float)W + eps);
}

template <typename A>
__global__ __launch_bounds__(256) void depth_norm_vec_kernel(hxm_depth_norm_args a) {
  extern __shared__ float lds[];
  f32x4* buf = reinterpret_cast<f32x4*>(lds);      // [W / 4]
  float* part = lds + a.width;                      // [4]
  typedef typename A::storage T;
  const int64_t W = a.width, n4 = W >> 2, i_out = blockIdx.x;
  const int64_t r = a.rows ? (int64_t)a.rows[i_out] : i_out;
  const f32x4* xin = a.x_in ? reinterpret_cast<const f32x4*>(a.x_in + r * W) : nullptr;
  const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f}, one4 = f32x4{1.f, 1.f, 1.f, 1.f};
  if (a.y) {
    const T* y = (const T*)a.y + r * a.y_stride;
    for (int64_t i = threadIdx.x; i < n4; i += 256) buf[i] = Row4<A>::load(y + 4 * i);
    float shift = 0.f, inv = 1.f;
    if (a.post_norm != HXM_POST_PLAIN) {
      __syncthreads();
      row_stats4(lds, part, W, a.eps, a.post_norm == HXM_POST_SAME ? a.rms : a.post_norm == HXM_POST_RMS, shift, inv);
    }
    const f32x4* pw = reinterpret_cast<const f32x4*>(a.post_w);
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      const f32x4 v = buf[i], x = xin ? xin[i] : zero4, w = pw ? pw[i] : one4;
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = x[k] + a.mult * ((v[k] - shift) * inv * w[k]);
      buf[i] = o;
    }
  } else {
    for (int64_t i = threadIdx.x; i < n4; i += 256) buf[i] = xin ? xin[i] : zero4;
  }
  if (a.y2) {
    const T* y2 = (const T*)a.y2 + r * a.y2_stride;
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      const f32x4 v = Row4<A>::load(y2 + 4 * i);
      f32x4 o = buf[i];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] += v[k];
      buf[i] = o;
    }
  }
  if (a.bias) {
    const f32x4* bw = reinterpret_cast<const f32x4*>(a.bias);
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      const f32x4 v = bw[i];
      f32x4 o = buf[i];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] += v[k];
      buf[i] = o;
    }
  }
  // (every thread keeps to the elements i = tid + 256 k from here on: no barrier is needed until the next statistics)
  if (a.level_out) {
    f32x4* lo = reinterpret_cast<f32x4*>(a.level_out + r * W);
    for (int64_t i = threadIdx.x; i < n4; i += 256) lo[i] = buf[i];
  }
  if (a.depth_w) {
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      f32x4 u = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int j = 0; j < a.n_levels; ++j) {
        const float* lv = a.levels + (int64_t)j * a.level_stride + r * W;
        // the level written above is taken from LDS: the store to it need not have landed
        const f32x4 v = (a.level_out && lv == a.level_out + r * W) ? buf[i] : reinterpret_cast<const f32x4*>(lv)[i];
        const float w = a.depth_w[j];
#pragma unroll
        for (int k = 0; k < 4; ++k) u[k] += w * v[k];
      }
      buf[i] = u;
    }
  }
  if (a.x_out) {
    f32x4* xo = reinterpret_cast<f32x4*>(a.x_out + i_out * W);
    for (int64_t i = threadIdx.x; i < n4; i += 256) xo[i] = buf[i];
  }
  if (a.next_w) {
    __syncthreads();
    float shift, inv;
    row_stats4(lds, part, W, a.eps, a.rms, shift, inv);
    T* h = (T*)a.h_out + i_out * a.h_stride;
    const f32x4* nw = reinterpret_cast<const f32x4*>(a.next_w);
    for (int64_t i = threadIdx.x; i < n4; i += 256) {
      const f32x4 v = buf[i], w = nw[i];
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = (v[k] - shift) * inv * w[k];
      Row4<A>::store(h + 4 * i, o);
    }
  } else if (a.h_out) {      // no norm: the row itself in the activations' type
    T* h = (T*)a.h_out + i_out * a.h_stride;
    for (int64_t i = threadIdx.x; i < n4; i += 256) Row4<A>::store(h + 4 * i, buf[i]);
  }
}

// vec: rows let a lane move four elements at a time (n, strides and pointers multiples of four elements)
template <typename A>
__global__ __launch_bounds__(256) void poly_norm_kernel(typename A::storage* __restrict__ out, int64_t out_stride,
                                                        const typename A::storage* __restrict__ z, int64_t z_stride,
                                                        const float* __restrict__ coef, float eps, int64_t n, int vec) {
  extern __shared__ float lds[];
  float* buf = lds;
  float* part = lds + n;       // [12]
  const int64_t row = blockIdx.x;
  float s[3] = {0.f, 0.f, 0.f};
  if (vec) {
    for (int64_t i = (int64_t)threadIdx.x * 4; i < n; i += 1024) {
      const f32x4 v = Row4<A>::load(z + row * z_stride + i);
      *reinterpret_cast<f32x4*>(buf + i) = v;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float v2 = v[k] * v[k];
        s[0] += v2;
        s[1] += v2 * v2;
        s[2] += v2 * v2 * v2;
      }
    }
  } else {
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      const float v = A::to_float(z[row * z_stride + i]);
      buf[i] = v;
      const float v2 = v * v;
      s[0] += v2;
      s[1] += v2 * v2;
      s[2] += v2 * v2 * v2;
    }
  }
  block_sums<3>(s, part);
  const float r1 = coef[0] / sqrtf(s[0] / (float)n + eps), r2 = coef[1] / sqrtf(s[1] / (float)n + eps),
              r3 = coef[2] / sqrtf(s[2] / (float)n + eps), c3 = coef[3];
  // (a thread reads back the elements of buf it wrote itself)
  if (vec) {
    for (int64_t i = (int64_t)threadIdx.x * 4; i < n; i += 1024) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(buf + i);
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = v[k] * r1 + v[k] * v[k] * r2 + v[k] * v[k] * v[k] * r3 + c3;
      Row4<A>::store(out + row * out_stride + i, o);
    }
  } else {
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      const float v = buf[i];
      out[row * out_stride + i] = A::from_float(v * r1 + v * v * r2 + v * v * v * r3 + c3);
    }
  }
}

template <typename A>
__global__ __launch_bounds__(256) void relu_squared_kernel(typename A::storage* __restrict__ out, int64_t out_stride,
                                                           const typename A::storage* __restrict__ z, int64_t z_stride,
                                                           int64_t rows, int64_t n) {
  const int64_t total = rows * n;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t r = e / n, c = e - r * n;
    const float v = fmaxf(A::to_float(z[r * z_stride + c]), 0.f);
    out[r * out_stride + c] = A::from_float(v * v);
  }
}

}  // namespace

extern "C" int hxm_embed_positions(float* out, const void* table, const void* pos_table, const void* ids, int ids_are_int64,
                                   const int32_t* positions, int64_t n_tokens, int64_t width, int64_t vocab,
                                   int64_t n_positions, int dtype, void* stream) {
  if (n_tokens < 0 || width < 1 || vocab < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!out || !table || !ids || (pos_table && !positions)) return HX_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), block(256);
  switch (dtype) {
    case HX_F32:
      embed_positions_kernel<F32><<<grid, block, 0, s>>>(out, (const float*)table, (const float*)pos_table, ids, ids_are_int64,
                                                         positions, width, vocab, n_positions);
      break;
    case HX_BF16:
      embed_positions_kernel<BF16><<<grid, block, 0, s>>>(out, (const u16*)table, (const u16*)pos_table, ids, ids_are_int64,
                                                          positions, width, vocab, n_positions);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_depth_norm(const hxm_depth_norm_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_depth_norm_args& a = *args;
  if (a.n_out < 0 || a.width < 1 || a.n_levels < 0) return HX_ERR_SHAPE;
  if (a.n_out == 0) return HX_OK;
  if (a.post_norm < HXM_POST_SAME || a.post_norm > HXM_POST_PLAIN) return HX_ERR_SHAPE;
  if ((!a.x_in && !a.y) || (a.y && !a.post_w && a.post_norm != HXM_POST_PLAIN) || (a.depth_w && !a.levels) || (a.next_w && !a.h_out))
    return HX_ERR_NULL;
  if ((a.y && a.y_stride < a.width) || (a.y2 && a.y2_stride < a.width) || (a.h_out && a.h_stride < a.width)) return HX_ERR_STRIDE;
  const size_t lds = ((size_t)a.width + 4) * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)a.n_out), block(256);
  const uintptr_t es = a.dtype == HX_F32 ? 4 : 2;
  auto by16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = a.width % 4 == 0 && by16(a.x_in) && by16(a.post_w) && by16(a.level_out) && by16(a.levels) && a.level_stride % 4 == 0 &&
                   by16(a.x_out) && by16(a.next_w) && ((uintptr_t)a.y % (4 * es)) == 0 && a.y_stride % 4 == 0 &&
                   ((uintptr_t)a.h_out % (4 * es)) == 0 && a.h_stride % 4 == 0 && ((uintptr_t)a.y2 % (4 * es)) == 0 &&
                   a.y2_stride % 4 == 0 && by16(a.bias);
  switch (a.dtype) {
    case HX_F32:
      if (vec) depth_norm_vec_kernel<F32><<<grid, block, lds, s>>>(a);
      else depth_norm_kernel<F32><<<grid, block, lds, s>>>(a);
      break;
    case HX_BF16:
      if (vec) depth_norm_vec_kernel<BF16><<<grid, block, lds, s>>>(a);
      else depth_norm_kernel<BF16><<<grid, block, lds, s>>>(a);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_poly_norm(void* out, int64_t out_stride, const void* z, int64_t z_stride, const float* coef, float eps,
                             int64_t rows, int64_t n, int dtype, void* stream) {
  if (rows < 0 || n < 1) return HX_ERR_SHAPE;
  if (rows == 0) return HX_OK;
  if (!out || !z || !coef) return HX_ERR_NULL;
  if (out_stride < n || z_stride < n) return HX_ERR_STRIDE;
  const size_t lds = ((size_t)n + 12) * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)rows), block(256);
  const int es = dtype == HX_F32 ? 4 : 2;
  const int vec = n % 4 == 0 && out_stride % 4 == 0 && z_stride % 4 == 0 && ((uintptr_t)out % (4 * es)) == 0 && ((uintptr_t)z % (4 * es)) == 0;
  switch (dtype) {
    case HX_F32: poly_norm_kernel<F32><<<grid, block, lds, s>>>((float*)out, out_stride, (const float*)z, z_stride, coef, eps, n, vec); break;
    case HX_BF16: poly_norm_kernel<BF16><<<grid, block, lds, s>>>((u16*)out, out_stride, (const u16*)z, z_stride, coef, eps, n, vec); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_relu_squared(void* out, int64_t out_stride, const void* z, int64_t z_stride, int64_t rows, int64_t n,
                                int dtype, void* stream) {
  if (rows < 0 || n < 1) return HX_ERR_SHAPE;
  if (rows == 0) return HX_OK;
  if (!out || !z) return HX_ERR_NULL;
  if (out_stride < n || z_stride < n) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t blocks = (rows * n + 255) / 256;
  const dim3 grid((unsigned)(blocks < 8192 ? blocks : 8192)), block(256);
  switch (dtype) {
    case HX_F32: relu_squared_kernel<F32><<<grid, block, 0, s>>>((float*)out, out_stride, (const float*)z, z_stride, rows, n); break;
    case HX_BF16: relu_squared_kernel<BF16><<<grid, block, 0, s>>>((u16*)out, out_stride, (const u16*)z, z_stride, rows, n); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
