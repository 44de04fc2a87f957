// biased_attn.hip — grouped-query attention over a paged key/value cache whose scores carry a linear distance bias,
// score(i, j) = q_i . k_j * scale - slope_h (i - j), under a causal, sliding-window or chunked mask (chunks counted from
// position 0 of the sequence).  Key and value rows may differ in size.  Scores, weights and sums are float.  Also the
// kernel in front of it: one RMS norm over a token's whole query projection and one over its whole key projection
// (all heads at once), keys and values straight into the cache.
#include <cfloat>
#include "attn_common.h"
#include "mix_rows.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int& last_hip_error();
int check_launch();
}  // namespace hxm

namespace {

using namespace hx;

// one workgroup per token.  vec: every offset, size, stride and pointer lets a lane move four elements at a time (and a
// head's key / value rows are multiples of four)
template <typename A>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(const typename A::storage* __restrict__ proj, int64_t proj_stride,
                                                            int64_t q_off, int64_t q_size, int64_t k_off, int64_t k_size,
                                                            int64_t v_off, int64_t v_size, const float* __restrict__ q_w,
                                                            const float* __restrict__ k_w, float eps,
                                                            typename A::storage* __restrict__ q_out,
                                                            const int32_t* __restrict__ slot_ids,
                                                            typename A::storage* __restrict__ key_cache,
                                                            typename A::storage* __restrict__ value_cache,
                                                            int64_t cache_row_stride, int64_t head_stride, int kv_heads, int vec) {
  __shared__ float part[8];
  const int64_t t = blockIdx.x;
  const typename A::storage* row = proj + t * proj_stride;
  const int step = vec ? 4 : 1;
  float ss[2] = {0.f, 0.f};      // sums of squares of the query and of the key projection, one pass
  if (q_w) {
    for (int64_t i = (int64_t)threadIdx.x * step; i < q_size; i += 256 * step) {
      if (vec) {
        const f32x4 v = Row4<A>::load(row + q_off + i);
        ss[0] += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
      } else {
        const float v = A::to_float(row[q_off + i]);
        ss[0] += v * v;
      }
    }
  }
  if (k_w) {
    for (int64_t i = (int64_t)threadIdx.x * step; i < k_size; i += 256 * step) {
      if (vec) {
        const f32x4 v = Row4<A>::load(row + k_off + i);
        ss[1] += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
      } else {
        const float v = A::to_float(row[k_off + i]);
        ss[1] += v * v;
      }
    }
  }
  if (q_w || k_w) block_sums<2>(ss, part);
  const float q_inv = 1.0f / sqrtf(ss[0] / (float)q_size + eps);
  for (int64_t i = (int64_t)threadIdx.x * step; i < q_size; i += 256 * step) {
    if (vec) {
      f32x4 v = Row4<A>::load(row + q_off + i);
      if (q_w) {
        const f32x4 w = *reinterpret_cast<const f32x4*>(q_w + i);
        v = f32x4{v[0] * q_inv * w[0], v[1] * q_inv * w[1], v[2] * q_inv * w[2], v[3] * q_inv * w[3]};
      }
      Row4<A>::store(q_out + t * q_size + i, v);
    } else {
      q_out[t * q_size + i] = q_w ? A::from_float(A::to_float(row[q_off + i]) * q_inv * q_w[i]) : row[q_off + i];
    }
  }
  if (k_size <= 0) return;
  const int64_t slot = slot_ids[t];
  if (slot < 0) return;
  const float k_inv = 1.0f / sqrtf(ss[1] / (float)k_size + eps);
  const int64_t kd = k_size / kv_heads, vd = v_size / kv_heads;
  typename A::storage* kr = key_cache + slot * cache_row_stride;
  typename A::storage* vr = value_cache + slot * cache_row_stride;
  for (int64_t i = (int64_t)threadIdx.x * step; i < k_size; i += 256 * step) {
    const int64_t at = (i / kd) * head_stride + i % kd;
    if (vec) {
      f32x4 v = Row4<A>::load(row + k_off + i);
      if (k_w) {
        const f32x4 w = *reinterpret_cast<const f32x4*>(k_w + i);
        v = f32x4{v[0] * k_inv * w[0], v[1] * k_inv * w[1], v[2] * k_inv * w[2], v[3] * k_inv * w[3]};
      }
      Row4<A>::store(kr + at, v);
    } else {
      kr[at] = k_w ? A::from_float(A::to_float(row[k_off + i]) * k_inv * k_w[i]) : row[k_off + i];
    }
  }
  for (int64_t i = (int64_t)threadIdx.x * step; i < v_size; i += 256 * step) {
    const int64_t at = (i / vd) * head_stride + i % vd;
    if (vec) Row4<A>::store(vr + at, Row4<A>::load(row + v_off + i));
    else vr[at] = row[v_off + i];
  }
}

// the wave's LDS writes so far are visible to all its lanes
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// a score under a soft cap: cap * tanh(s / cap); cap 0: the score itself
__device__ __forceinline__ float capped(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// the first key a query at position i sees
__device__ __forceinline__ int first_visible(int i, int kind, int size) {
  if (kind == HXM_MASK_WINDOW) return i - size + 1 > 0 ? i - size + 1 : 0;
  if (kind == HXM_MASK_CHUNK) return i / size * size;
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Row form: one wave per (token, head), four a workgroup, no barriers.  Keys go by in groups of 64: lane l scores key
// lo + l (its row of the cache against the query in LDS), the group's maximum and sum are wave reductions, then the lanes
// turn to the value's columns (lane l owns columns l, l + 64, ...) and add the 64 rows, each weighted by its lane's p.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxVCols = 8;      // value columns per lane: vdim <= 512
template <typename A>
__global__ __launch_bounds__(256) void biased_attn_rows_kernel(hxm_biased_attn_args a) {
  extern __shared__ float lds[];
  typedef typename A::storage T;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= (int64_t)a.n_tokens * a.n_heads) return;
  const int t = (int)(item / a.n_heads), h = (int)(item - (int64_t)t * a.n_heads);
  const int D = a.dim, V = a.vdim, BS = a.block_size;
  float* qs = lds + wave * (D + 64);       // the query, then the group's weights
  float* ps = qs + D;
  const T* q = (const T*)a.q + ((int64_t)t * a.n_heads + h) * D;
  const float qscale = a.head_scale ? a.scale * a.head_scale[h] : a.scale;
  for (int d = lane; d < D; d += 64) qs[d] = A::to_float(q[d]) * qscale;
  wave_lds_sync();
  const int seq = a.tok_seq[t], i = a.positions[t];
  const int32_t* table = a.block_table + a.cu_block_lens[seq];
  const int g = h / (a.n_heads / a.kv_heads);
  const T* kc = (const T*)a.key_cache + (int64_t)g * a.head_stride;
  const T* vc = (const T*)a.value_cache + (int64_t)g * a.head_stride;
  const float slope = a.slopes ? a.slopes[h] : 0.f;
  const int lo = first_visible(i, a.mask_kind, a.mask_size);
  float m = -FLT_MAX, l = 0.f;
  float acc[kMaxVCols];
#pragma unroll
  for (int c = 0; c < kMaxVCols; ++c) acc[c] = 0.f;
  for (int j0 = lo; j0 <= i; j0 += 64) {
    const int j = j0 + lane;
    float s = -FLT_MAX;
    if (j <= i) {
      const T* kr = kc + (int64_t)table[j / BS] * a.cache_block_stride + (int64_t)(j % BS) * a.cache_row_stride;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * A::to_float(kr[d]);
      if (a.softcap > 0.f) dot = a.softcap * tanhf(dot / a.softcap);
      s = dot - slope * (float)(i - j);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = j <= i ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    wave_lds_sync();
    ps[lane] = p;
    wave_lds_sync();
#pragma unroll
    for (int c = 0; c < kMaxVCols; ++c) acc[c] *= corr;
    const int n = i - j0 + 1 < 64 ? i - j0 + 1 : 64;
    for (int jj = 0; jj < n; ++jj) {
      const int jk = j0 + jj;
      const T* vr = vc + (int64_t)table[jk / BS] * a.cache_block_stride + (int64_t)(jk % BS) * a.cache_row_stride;
      const float pj = ps[jj];
#pragma unroll
      for (int c = 0; c < kMaxVCols; ++c) {
        const int col = lane + 64 * c;
        if (col < V) acc[c] += pj * A::to_float(vr[col]);
      }
    }
  }
  T* o = (T*)a.out + ((int64_t)t * a.n_heads + h) * V;
  if (a.sinks) l += expf(a.sinks[h] - m);      // the sink: one more term of the denominator, without a value
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < kMaxVCols; ++c) {
    const int col = lane + 64 * c;
    if (col < V) o[col] = A::from_float(acc[c] * inv);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Tile form (bfloat16): one wave per 16 rows, a row being a (token, query head) pair of ONE sequence's portion and ONE
// key/value head, the group's query heads fastest — the heads of a decoded token that share a key head, or a few tokens
// times those heads.  All rows of a tile read the same keys, which go by in chunks of 32: S = Q K^T and O += P V are
// 16x16x32 MFMAs.  Key rows come straight from the paged cache into the B operands of S (a lane's 16 bytes are 8
// consecutive columns of one key's row); value rows are written to the wave's LDS as they come (row-major image of the
// chunk) and return through the transposing LDS read as B operands of the second product; P goes through LDS from the
// accumulator layout to the A layout.  Bias and mask are applied to the float scores, row by row.  With n_splits > 1 the
// key range of a tile is dealt to several waves whose partial results a second kernel merges.  No workgroup barriers.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kPStride = 36;       // u16 per row of P in LDS: 32 slots + 4

template <int KK>                  // ceil(max(dim, vdim) / 32): 1, 2, 4, 8
__global__ __launch_bounds__(256) void biased_attn_tile_kernel(hxm_biased_attn_args a, int tiles_per_seq, int waves_per_block) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave >= waves_per_block) return;
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1;
  const int G = a.kv_heads, R = a.n_heads / a.kv_heads, D = a.dim, V = a.vdim;
  const int64_t witem = (int64_t)blockIdx.x * waves_per_block + wave;      // (sequence, kv head, row tile, key split), splits fastest
  if (witem >= (int64_t)a.n_seq * G * tiles_per_seq * n_splits) return;
  const int64_t item = witem / n_splits;
  const int split = (int)(witem % n_splits);
  const int tile = (int)(item % tiles_per_seq);
  const int kvh = (int)((item / tiles_per_seq) % G);
  const int b = (int)(item / ((int64_t)tiles_per_seq * G));
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * R;
  if (tile * 16 >= n_rows) return;
  const int g = lane >> 4, c = lane & 15;
  const int RS = 2 * (KK * 32) + 32;      // bytes per row of the value image (a key's columns, padded)
  char* img = reinterpret_cast<char*>(lds) + (size_t)wave * (32 * RS + 16 * kPStride * 2);
  u16* pl = reinterpret_cast<u16*>(img + 32 * RS);
  const u16* kc = (const u16*)a.key_cache + (int64_t)kvh * a.head_stride;
  const u16* vc = (const u16*)a.value_cache + (int64_t)kvh * a.head_stride;
  const int32_t* table = a.block_table + a.cu_block_lens[b];
  const u16x8 zero8 = u16x8{0, 0, 0, 0, 0, 0, 0, 0};

  // the queries: lane (g, c) holds row c, columns 32 kk + 8 g .. + 7
  const int last_row = min(tile * 16 + 15, n_rows - 1);
  u16x8 qf[KK];
  {
    const int r = min(tile * 16 + c, n_rows - 1);
    const u16* qg = (const u16*)a.q + ((int64_t)(q0 + r / R) * a.n_heads + kvh * R + r % R) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      qf[kk] = col < D ? *reinterpret_cast<const u16x8*>(qg + col) : zero8;
    }
  }
  // the rows this lane holds of S and O: 4 g + i
  int pos[4], lo[4];
  float slope[4], hsc[4], snk[4];      // per row: distance slope, score scale (scale * head_scale), sink term's logit
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    hsc[i] = a.scale;
    snk[i] = -INFINITY;
    if (r < n_rows) {
      const int h = kvh * R + r % R;
      pos[i] = a.positions[q0 + r / R];
      lo[i] = first_visible(pos[i], a.mask_kind, a.mask_size);
      slope[i] = a.slopes ? a.slopes[h] : 0.f;
      if (a.head_scale) hsc[i] = a.scale * a.head_scale[h];
      if (a.sinks) snk[i] = a.sinks[h];
    } else {
      pos[i] = -1;      // sees nothing
      lo[i] = 0;
      slope[i] = 0.f;
    }
  }
  // the keys any row of the tile sees
  int k_min, k_max;
  {
    const int r = min(tile * 16 + c, last_row);
    const int pr = a.positions[q0 + r / R];
    k_max = pr;
    k_min = first_visible(pr, a.mask_kind, a.mask_size);
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      k_max = max(k_max, __shfl_xor(k_max, off, 64));
      k_min = min(k_min, __shfl_xor(k_min, off, 64));
    }
  }
  float m[4], l[4];
  f32x4 acc[KK * 2];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m[i] = -1.0e30f; l[i] = 0.f; }
#pragma unroll
  for (int n = 0; n < KK * 2; ++n) acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  int k_begin = k_min, k_end = k_max;
  if (n_splits > 1) {
    const int chunks = (k_max - k_min + 32) / 32;
    const int per = (chunks + n_splits - 1) / n_splits;
    k_begin = k_min + split * per * 32;
    k_end = min(k_max, k_begin + per * 32 - 1);
  }
  const int bs = a.block_size;
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  // a chunk's key or value rows, this lane's part: key 16 s + c, columns 32 kk + 8 g .. + 7
  auto fetch = [&](int key0, const u16* base, int width, u16x8 (&f)[2][KK]) __attribute__((always_inline)) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int key = min(key0 + 16 * s + c, k_max);        // (a key past the last one repeats it; masked below)
      const int page = bshift >= 0 ? key >> bshift : key / bs;
      const int64_t off = (int64_t)table[page] * a.cache_block_stride + (int64_t)(key - page * bs) * a.cache_row_stride;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const int col = 32 * kk + 8 * g;
        f[s][kk] = col < width ? *reinterpret_cast<const u16x8*>(base + off + col) : zero8;
      }
    }
  };
  // One register set each for keys and values: a chunk's values are asked for before its scores are multiplied, and the
  // next chunk's keys as soon as the scores are done — both loads are in flight behind the softmax and the products.
  u16x8 kf[2][KK], vf[2][KK];
  if (k_begin <= k_end) fetch(k_begin, kc, D, kf);
  for (int key0 = k_begin; key0 <= k_end; key0 += 32) {
    fetch(key0, vc, V, vf);
    f32x4 sc[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      sc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) sc[s] = Mfma<BF16>::mma(qf[kk], kf[s][kk], sc[s]);
    }
    if (key0 + 32 <= k_end) fetch(key0 + 32, kc, D, kf);
    // softmax of the rows 4 g + i over this chunk (sc[s][i] is key key0 + 16 s + c)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float p[2];
      float mx = -INFINITY;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int key = key0 + 16 * s + c;
        const bool seen = key >= lo[i] && key <= pos[i];
        p[s] = seen ? capped(sc[s][i] * hsc[i], a.softcap) - slope[i] * (float)(pos[i] - key) : -INFINITY;
        mx = fmaxf(mx, p[s]);
      }
      mx = row16_max(mx);      // (the sixteen lanes that hold the row's scores: one DPP row)
      const float m_new = fmaxf(m[i], mx);
      const float corr = __expf(m[i] - m_new);
      p[0] = __expf(p[0] - m_new);       // exp(-inf) = 0 for a key the row does not see
      p[1] = __expf(p[1] - m_new);
      float ps = p[0] + p[1];
      ps = row16_sum(ps);
      l[i] = l[i] * corr + ps;
      m[i] = m_new;
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) acc[n][i] *= corr;
      // key 16 s + c sits in slot 8 (c / 4) + c % 4 + 4 s of its row: the order the transposing read delivers the keys in
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3)] = BF16::from_float(p[0]);
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3) + 4] = BF16::from_float(p[1]);
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) *reinterpret_cast<u16x8*>(img + (16 * s + c) * RS + (32 * kk + 8 * g) * 2) = vf[s][kk];
    wave_lds_sync();
    // O += P V: A = P[row c][slots 8 g ..], B = the image's column 16 n + c at the keys of those slots
    u16x8 pf;
    {
      const u16x4 x0 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g);
      const u16x4 x1 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g + 4);
      pf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
    const char* vrd = img + (4 * g + (c >> 2)) * RS + (c & 3) * 8;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const u16x4 x0 = lds_tr_read(vrd + n * 32);
      const u16x4 x1 = lds_tr_read(vrd + 16 * RS + n * 32);
      const u16x8 vv = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
      acc[n] = Mfma<BF16>::mma(pf, vv, acc[n]);
    }
    wave_lds_sync();      // the reads are done before the next chunk is written
  }
  const int V16 = (V + 15) / 16 * 16;
  if (n_splits > 1) {
    // unnormalised partial result of this split: ws_o [item][split][16 rows][V16], ws_ml [item][split][16 rows][m, l]
    float* wo = a.ws_o + ((size_t)witem * 16) * V16;
    float* wml = a.ws_ml + (size_t)witem * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * g + i;
      if (c == 0) {
        wml[2 * row] = m[i];
        wml[2 * row + 1] = l[i];
      }
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) {
        const int col = 16 * n + c;
        if (col < V16) wo[(size_t)row * V16 + col] = acc[n][i];
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r >= n_rows) continue;
    const float inv = 1.0f / (l[i] + expf(snk[i] - m[i]));      // (no sink: exp(-inf) = 0)
    u16* og = (u16*)a.out + ((int64_t)(q0 + r / R) * a.n_heads + kvh * R + r % R) * V;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const int col = 16 * n + c;
      if (col < V) og[col] = BF16::from_float(acc[n][i] * inv);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Group form (bfloat16, portions of prompts, head sizes up to 128): a workgroup of four waves takes four consecutive row
// tiles (64 rows) of ONE (sequence, key head) and ONE image of every 32-key chunk.  The tile form is bound by its loads —
// sixteen 16-byte load instructions per chunk and wave, each touching sixteen half cache lines; here the workgroup brings
// a chunk's key and value rows once, in whole rows (two to four loads a thread), into one of two LDS images, and all four
// waves read the B operands of both products from there (16-byte reads for S, transposing reads for O).  The next chunk
// is on its way into registers while this one is multiplied and goes to the other image afterwards: one workgroup barrier
// a chunk, one that orders LDS only.  A wave skips the chunks none of its rows sees.
// ---------------------------------------------------------------------------------------------------------------
template <int KK>                  // ceil(max(dim, vdim) / 32): 1, 2, 4
__global__ __launch_bounds__(256) void biased_attn_group_kernel(hxm_biased_attn_args a, int groups_per_seq) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int G = a.kv_heads, R = a.n_heads / a.kv_heads, D = a.dim, V = a.vdim;
  const int64_t item = blockIdx.x;                                   // (sequence, kv head, group of four row tiles)
  const int group = (int)(item % groups_per_seq);
  const int kvh = (int)((item / groups_per_seq) % G);
  const int b = (int)(item / ((int64_t)groups_per_seq * G));
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * R;
  if (group * 64 >= n_rows) return;                                  // (the whole workgroup: no barrier is left waiting)
  const int tile = group * 4 + wave;
  const bool live = tile * 16 < n_rows;                              // a wave past the portion's rows only helps to load
  const int g = lane >> 4, c = lane & 15;
  constexpr int RS = 2 * (KK * 32) + 32;                             // bytes per row of an image (a key's columns, padded)
  constexpr int PR = KK * 4;                                         // 16-byte pieces per row
  constexpr int NP = (32 * PR + 255) / 256;                          // pieces of a chunk's keys (or values) a thread brings
  char* base = reinterpret_cast<char*>(lds);
  char* img_k[2] = {base, base + 32 * RS};
  char* img_v[2] = {base + 64 * RS, base + 96 * RS};
  u16* pl = reinterpret_cast<u16*>(base + 128 * RS) + wave * (16 * kPStride);
  const u16* kc = (const u16*)a.key_cache + (int64_t)kvh * a.head_stride;
  const u16* vc = (const u16*)a.value_cache + (int64_t)kvh * a.head_stride;
  const int32_t* table = a.block_table + a.cu_block_lens[b];
  const u16x8 zero8 = u16x8{0, 0, 0, 0, 0, 0, 0, 0};

  u16x8 qf[KK];
  {
    const int r = min(tile * 16 + c, n_rows - 1);
    const u16* qg = (const u16*)a.q + ((int64_t)(q0 + r / R) * a.n_heads + kvh * R + r % R) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      qf[kk] = col < D ? *reinterpret_cast<const u16x8*>(qg + col) : zero8;
    }
  }
  int pos[4], lo[4];
  float slope[4], hsc[4], snk[4];      // per row: distance slope, score scale (scale * head_scale), sink term's logit
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    hsc[i] = a.scale;
    snk[i] = -INFINITY;
    if (r < n_rows) {
      const int h = kvh * R + r % R;
      pos[i] = a.positions[q0 + r / R];
      lo[i] = first_visible(pos[i], a.mask_kind, a.mask_size);
      slope[i] = a.slopes ? a.slopes[h] : 0.f;
      if (a.head_scale) hsc[i] = a.scale * a.head_scale[h];
      if (a.sinks) snk[i] = a.sinks[h];
    } else {
      pos[i] = -1;      // sees nothing
      lo[i] = 0;
      slope[i] = 0.f;
    }
  }
  // rows of a portion are in the order of their positions: the group's first row sees the earliest key, its last the latest
  const int k_begin = first_visible(a.positions[q0 + (group * 64) / R], a.mask_kind, a.mask_size);
  const int k_end = a.positions[q0 + min(group * 64 + 63, n_rows - 1) / R];
  int w_min = 0x7fffffff, w_max = -1;      // the keys this wave's rows see
  if (live) {
    w_min = first_visible(a.positions[q0 + (tile * 16) / R], a.mask_kind, a.mask_size);
    w_max = a.positions[q0 + min(tile * 16 + 15, n_rows - 1) / R];
  }
  float m[4], l[4];
  f32x4 acc[KK * 2];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m[i] = -1.0e30f; l[i] = 0.f; }
#pragma unroll
  for (int n = 0; n < KK * 2; ++n) acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int bs = a.block_size;
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  // piece p of a chunk: row p / PR (a key), columns 8 (p % PR) .. + 7
  u16x8 kr[NP], vr[NP];
  auto fetch = [&](int key0) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      const int p = threadIdx.x + 256 * n;
      kr[n] = zero8;
      vr[n] = zero8;
      if (p < 32 * PR) {
        const int key = min(key0 + p / PR, k_end), col = (p % PR) * 8;      // (a key past the last one repeats it; masked below)
        const int page = bshift >= 0 ? key >> bshift : key / bs;
        const int64_t off = (int64_t)table[page] * a.cache_block_stride + (int64_t)(key - page * bs) * a.cache_row_stride + col;
        if (col < D) kr[n] = *reinterpret_cast<const u16x8*>(kc + off);
        if (col < V) vr[n] = *reinterpret_cast<const u16x8*>(vc + off);
      }
    }
  };
  auto store = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      const int p = threadIdx.x + 256 * n;
      if (p < 32 * PR) {
        const int at = (p / PR) * RS + (p % PR) * 16;
        *reinterpret_cast<u16x8*>(img_k[buf] + at) = kr[n];
        *reinterpret_cast<u16x8*>(img_v[buf] + at) = vr[n];
      }
    }
  };
  fetch(k_begin);
  store(0);
  lds_barrier();
  int buf = 0;
  for (int key0 = k_begin; key0 <= k_end; key0 += 32, buf ^= 1) {
    const bool more = key0 + 32 <= k_end;
    if (more) fetch(key0 + 32);
    if (key0 <= w_max && key0 + 31 >= w_min) {
      f32x4 sc[2];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        sc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const u16x8 kf = *reinterpret_cast<const u16x8*>(img_k[buf] + (16 * s + c) * RS + (32 * kk + 8 * g) * 2);
          sc[s] = Mfma<BF16>::mma(qf[kk], kf, sc[s]);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float p[2];
        float mx = -INFINITY;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int key = key0 + 16 * s + c;
          const bool seen = key >= lo[i] && key <= pos[i];
          p[s] = seen ? capped(sc[s][i] * hsc[i], a.softcap) - slope[i] * (float)(pos[i] - key) : -INFINITY;
          mx = fmaxf(mx, p[s]);
        }
        mx = row16_max(mx);
        const float m_new = fmaxf(m[i], mx);
        const float corr = __expf(m[i] - m_new);
        p[0] = __expf(p[0] - m_new);
        p[1] = __expf(p[1] - m_new);
        float ps = p[0] + p[1];
        ps = row16_sum(ps);
        l[i] = l[i] * corr + ps;
        m[i] = m_new;
#pragma unroll
        for (int n = 0; n < KK * 2; ++n) acc[n][i] *= corr;
        pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3)] = BF16::from_float(p[0]);
        pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3) + 4] = BF16::from_float(p[1]);
      }
      wave_lds_sync();
      u16x8 pf;
      {
        const u16x4 x0 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g);
        const u16x4 x1 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g + 4);
        pf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
      }
      const char* vrd = img_v[buf] + (4 * g + (c >> 2)) * RS + (c & 3) * 8;
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) {
        const u16x4 x0 = lds_tr_read(vrd + n * 32);
        const u16x4 x1 = lds_tr_read(vrd + 16 * RS + n * 32);
        const u16x8 vv = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        acc[n] = Mfma<BF16>::mma(pf, vv, acc[n]);
      }
      wave_lds_sync();      // this wave's reads of P are done before it writes the next chunk's
    }
    if (more) store(buf ^ 1);      // (the other image: every wave finished with it before the last barrier)
    lds_barrier();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r >= n_rows) continue;
    const float inv = 1.0f / (l[i] + expf(snk[i] - m[i]));      // (no sink: exp(-inf) = 0)
    u16* og = (u16*)a.out + ((int64_t)(q0 + r / R) * a.n_heads + kvh * R + r % R) * V;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const int col = 16 * n + c;
      if (col < V) og[col] = BF16::from_float(acc[n][i] * inv);
    }
  }
}

// the splits of a (sequence, kv head, row tile) merged: out = sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M)
__global__ __launch_bounds__(256) void biased_attn_combine_kernel(hxm_biased_attn_args a, int tiles_per_seq) {
  const int64_t item = blockIdx.x;
  const int G = a.kv_heads, R = a.n_heads / a.kv_heads, V = a.vdim, V16 = (V + 15) / 16 * 16, NS = a.n_splits;
  const int tile = (int)(item % tiles_per_seq);
  const int kvh = (int)((item / tiles_per_seq) % G);
  const int b = (int)(item / ((int64_t)tiles_per_seq * G));
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * R;
  if (tile * 16 >= n_rows) return;
  __shared__ float wgt[16][65];      // [row][split] weight e^(m_s - M) / L (NS <= 64)
  if (threadIdx.x < 16) {
    const int row = threadIdx.x;
    const float* wml = a.ws_ml + (size_t)item * NS * 32;
    float M = -1.0e30f;
    for (int s = 0; s < NS; ++s) M = fmaxf(M, wml[s * 32 + 2 * row]);
    float L = 0.f;
    for (int s = 0; s < NS; ++s) L += wml[s * 32 + 2 * row + 1] * __expf(wml[s * 32 + 2 * row] - M);
    if (a.sinks) L += expf(a.sinks[kvh * R + (tile * 16 + row) % R] - M);      // the sink counts once, here
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    for (int s = 0; s < NS; ++s) wgt[row][s] = __expf(wml[s * 32 + 2 * row] - M) * inv;
  }
  __syncthreads();
  const float* wo = a.ws_o + (size_t)item * NS * 16 * V16;
  for (int e = threadIdx.x; e < 16 * V; e += 256) {
    const int row = e / V, col = e % V;
    const int r = tile * 16 + row;
    if (r >= n_rows) continue;
    float v = 0.f;
    for (int s = 0; s < NS; ++s) v += wo[((size_t)s * 16 + row) * V16 + col] * wgt[row][s];
    ((u16*)a.out)[((int64_t)(q0 + r / R) * a.n_heads + kvh * R + r % R) * V + col] = BF16::from_float(v);
  }
}

template <int KK>
int launch_tile(const hxm_biased_attn_args& a, hipStream_t s) {
  const size_t per_wave = (size_t)32 * (2 * (KK * 32) + 32) + 16 * kPStride * 2;
  int waves = 4;
  while (waves > 1 && per_wave * waves > 64 * 1024) waves >>= 1;
  const int R = a.n_heads / a.kv_heads;
  const int tiles_per_seq = (int)(((int64_t)a.max_q_len * R + 15) / 16);
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1;
  if constexpr (KK <= 4) {
    if (n_splits == 1 && tiles_per_seq >= 4 && a.form != 2) {      // portions of prompts: four row tiles share every chunk
      const int groups_per_seq = (tiles_per_seq + 3) / 4;
      const size_t lds_g = (size_t)128 * (2 * (KK * 32) + 32) + 4 * 16 * kPStride * 2;
      biased_attn_group_kernel<KK><<<dim3((unsigned)((int64_t)a.n_seq * a.kv_heads * groups_per_seq)), dim3(256), lds_g, s>>>(a, groups_per_seq);
      return hxm::check_launch();
    }
  }
  const int64_t items = (int64_t)a.n_seq * a.kv_heads * tiles_per_seq;
  const dim3 grid((unsigned)((items * n_splits + waves - 1) / waves));
  biased_attn_tile_kernel<KK><<<grid, dim3(64 * waves), per_wave * waves, s>>>(a, tiles_per_seq, waves);
  if (n_splits > 1) biased_attn_combine_kernel<<<dim3((unsigned)items), dim3(256), 0, s>>>(a, tiles_per_seq);
  return hxm::check_launch();
}

bool tile_form_serves(const hxm_biased_attn_args& a) {
  const bool aligned = a.dim % 8 == 0 && a.vdim % 8 == 0 && a.head_stride % 8 == 0 && a.cache_row_stride % 8 == 0 &&
                       a.cache_block_stride % 8 == 0 && aligned16(a.key_cache) && aligned16(a.value_cache) && aligned16(a.q);
  return a.dtype == HX_BF16 && aligned && a.dim <= 256 && a.vdim <= 256 && a.q_cu && a.n_seq > 0 && a.max_q_len > 0 && a.form != 1;
}

}  // namespace

extern "C" int hxm_qk_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_size, int64_t k_off,
                                 int64_t k_size, int64_t v_off, int64_t v_size, const float* q_w, const float* k_w, float eps,
                                 void* q_out, const int32_t* slot_ids, void* key_cache, void* value_cache,
                                 int64_t cache_row_stride, int64_t head_stride, int32_t kv_heads, int64_t n_tokens, int dtype,
                                 void* stream) {
  if (n_tokens < 0 || q_size < 1 || k_size < 0 || v_size < 0 || kv_heads < 1) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!proj || !q_out) return HX_ERR_NULL;
  if (k_size > 0) {
    if (!slot_ids || !key_cache || !value_cache) return HX_ERR_NULL;
    if (k_size % kv_heads || v_size % kv_heads || v_size < 1) return HX_ERR_SHAPE;
    if (k_size / kv_heads > head_stride || v_size / kv_heads > head_stride || cache_row_stride < head_stride * kv_heads) return HX_ERR_STRIDE;
  }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_tokens), block(256);
  const uintptr_t es = dtype == HX_F32 ? 4 : 2;
  auto by4 = [&](const void* p) { return ((uintptr_t)p % (4 * es)) == 0; };
  int vec = q_off % 4 == 0 && q_size % 4 == 0 && proj_stride % 4 == 0 && by4(proj) && by4(q_out) &&
            (!q_w || (uintptr_t)q_w % 16 == 0);
  if (k_size > 0)
    vec = vec && k_off % 4 == 0 && v_off % 4 == 0 && (k_size / kv_heads) % 4 == 0 && (v_size / kv_heads) % 4 == 0 &&
          cache_row_stride % 4 == 0 && head_stride % 4 == 0 && by4(key_cache) && by4(value_cache) && (!k_w || (uintptr_t)k_w % 16 == 0);
  switch (dtype) {
    case HX_F32:
      qk_norm_cache_kernel<F32><<<grid, block, 0, s>>>((const float*)proj, proj_stride, q_off, q_size, k_off, k_size, v_off, v_size,
                                                       q_w, k_w, eps, (float*)q_out, slot_ids, (float*)key_cache, (float*)value_cache,
                                                       cache_row_stride, head_stride, kv_heads, vec);
      break;
    case HX_BF16:
      qk_norm_cache_kernel<BF16><<<grid, block, 0, s>>>((const u16*)proj, proj_stride, q_off, q_size, k_off, k_size, v_off, v_size,
                                                        q_w, k_w, eps, (u16*)q_out, slot_ids, (u16*)key_cache, (u16*)value_cache,
                                                        cache_row_stride, head_stride, kv_heads, vec);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

extern "C" int hxm_biased_attention(const hxm_biased_attn_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_biased_attn_args& a = *args;
  if (a.n_tokens < 0 || a.n_heads < 1 || a.kv_heads < 1 || a.n_heads % a.kv_heads || a.dim < 1 || a.vdim < 1 ||
      a.vdim > 64 * kMaxVCols || a.block_size < 1)
    return HX_ERR_SHAPE;
  if (a.mask_kind < HXM_MASK_CAUSAL || a.mask_kind > HXM_MASK_CHUNK || (a.mask_kind != HXM_MASK_CAUSAL && a.mask_size < 1)) return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.out || !a.q || !a.key_cache || !a.value_cache || !a.tok_seq || !a.positions || !a.block_table || !a.cu_block_lens) return HX_ERR_NULL;
  if (a.dim > a.head_stride || a.vdim > a.head_stride) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  if (a.n_splits > 1 && (a.n_splits > 64 || !a.ws_o || !a.ws_ml || !tile_form_serves(a))) return HX_ERR_WORKSPACE;
  if (tile_form_serves(a)) {
    const int kk = ((a.dim > a.vdim ? a.dim : a.vdim) + 31) / 32;
    if (kk <= 1) return launch_tile<1>(a, s);
    if (kk <= 2) return launch_tile<2>(a, s);
    if (kk <= 4) return launch_tile<4>(a, s);
    return launch_tile<8>(a, s);
  }
  const int64_t items = (int64_t)a.n_tokens * a.n_heads;
  const size_t lds = 4 * ((size_t)a.dim + 64) * sizeof(float);
  if (lds > 64 * 1024) return HX_ERR_SHAPE;
  const dim3 grid((unsigned)((items + 3) / 4)), block(256);
  switch (a.dtype) {
    case HX_F32: biased_attn_rows_kernel<F32><<<grid, block, lds, s>>>(a); break;
    case HX_BF16: biased_attn_rows_kernel<BF16><<<grid, block, lds, s>>>(a); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
