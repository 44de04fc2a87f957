// latent_attn.hip — attention over a paged cache of low-rank latents.  A token leaves ONE row c (kv_rank numbers) in the
// cache; every head's key and value are linear maps of it, so with the key map folded into the query (q~ = W_uk^T q) and
// the value map applied afterwards (o = W_uv sum_j p_j c_j) the kernel is multi-query attention whose keys and values
// are the same rows: score = q~ . c_j * scale, out = sum_j softmax(score)_j c_j.  Scores, weights and sums are float.
// Sliding window: a query at position i sees keys j with 0 <= i - j < window.
#include "attn_common.h"
#include "../../include/hydra_mix.h"

namespace hxm {
int check_launch();
int& tile_form();      // 0: row form only (A/B measurements), 1: tile form where it applies
}

namespace {

using namespace hx;

// one WAVE per token (four tokens a workgroup, no barriers): both latents of the token from its projection row.  vec:
// every pointer, offset and stride lets a lane move four elements at a time.
template <typename A>
__global__ __launch_bounds__(256) void latent_norm_cache_kernel(const typename A::storage* __restrict__ proj, int64_t proj_stride,
                                                                int64_t q_off, int64_t q_rank, int64_t kv_off, int64_t kv_rank,
                                                                const float* __restrict__ q_w, const float* __restrict__ kv_w, float eps,
                                                                typename A::storage* __restrict__ cq_out,
                                                                const int32_t* __restrict__ slot_ids,
                                                                typename A::storage* __restrict__ cache, int64_t cache_block_stride,
                                                                int64_t cache_row_stride, int32_t block_size, int64_t n_tokens, int vec) {
  typedef typename A::storage ST;
  typedef ST ST4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= n_tokens) return;
  const ST* p = proj + t * proj_stride;
  const int32_t slot = slot_ids[t];
  ST* dst = slot >= 0 ? cache + (int64_t)(slot / block_size) * cache_block_stride + (int64_t)(slot % block_size) * cache_row_stride : nullptr;
  // the two latents in turn: (source offset, length, weight, destination)
  for (int which = 0; which < 2; ++which) {
    const int64_t off = which ? kv_off : q_off, n = which ? kv_rank : q_rank;
    const float* w = which ? kv_w : q_w;
    ST* out = which ? dst : cq_out + t * q_rank;
    if (!out) break;
    float ss = 0.f;
    if (vec) {
      for (int64_t i = 4 * lane; i < n; i += 256) {
        const ST4 v = *reinterpret_cast<const ST4*>(p + off + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += A::to_float(v[e]) * A::to_float(v[e]);
      }
    } else {
      for (int64_t i = lane; i < n; i += 64) ss += A::to_float(p[off + i]) * A::to_float(p[off + i]);
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)n + eps);
    if (vec) {
      for (int64_t i = 4 * lane; i < n; i += 256) {
        const ST4 v = *reinterpret_cast<const ST4*>(p + off + i);
        const f32x4 wv = *reinterpret_cast<const f32x4*>(w + i);
        ST4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = A::from_float(A::to_float(v[e]) * inv * wv[e]);
        *reinterpret_cast<ST4*>(out + i) = o;
      }
    } else {
      for (int64_t i = lane; i < n; i += 64) out[i] = A::from_float(A::to_float(p[off + i]) * inv * w[i]);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Row form: one wave per (token, head).  Keys go by in groups of 64: lane l scores key lo + l (its own row of the
// cache against the query in LDS), the group's maximum and sum are wave reductions, then the lanes turn to the latent's
// columns (lane l owns columns l, l + 64, ...) and add the 64 rows, each weighted by its lane's p.  Serves float32 runs
// and layouts that are not 16-byte aligned; bfloat16 runs take the MFMA forms below.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxCols = HXM_MAX_LATENT / 64;

template <typename A>
__global__ __launch_bounds__(256) void latent_attn_rows_kernel(hxm_latent_attn_args a) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t total = (int64_t)a.n_tokens * a.n_heads;
  const bool live = (int64_t)blockIdx.x * 4 + wave < total;
  const int64_t item = live ? (int64_t)blockIdx.x * 4 + wave : total - 1;      // (a spare wave repeats the last row and stores nothing)
  const int32_t t = (int32_t)(item / a.n_heads), h = (int32_t)(item % a.n_heads);
  const int32_t R = a.kv_rank;
  float* q = lds + wave * R;
  const typename A::storage* qg = (const typename A::storage*)a.q + (int64_t)t * a.q_token_stride + (int64_t)h * a.q_head_stride;
  for (int i = lane; i < R; i += 64) q[i] = A::to_float(qg[i]) * a.scale;
  __syncthreads();
  const int32_t b = a.tok_seq[t];
  const int32_t pos = a.positions[t];
  const int32_t lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int32_t* table = a.block_table + a.cu_block_lens[b];
  const typename A::storage* cache = (const typename A::storage*)a.cache;
  constexpr int kVec = 16 / sizeof(typename A::storage);
  const bool vec = R % kVec == 0 && a.cache_row_stride % kVec == 0 && a.cache_block_stride % kVec == 0 &&
                   (reinterpret_cast<uintptr_t>(a.cache) & 15u) == 0;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxCols];
#pragma unroll
  for (int k = 0; k < kMaxCols; ++k) acc[k] = 0.f;
  for (int32_t j0 = lo; j0 <= pos; j0 += 64) {
    const int32_t j = j0 + lane;
    const bool valid = j <= pos;
    int64_t off = 0;
    float s = -INFINITY;
    if (valid) {
      off = (int64_t)table[j / a.block_size] * a.cache_block_stride + (int64_t)(j % a.block_size) * a.cache_row_stride;
      const typename A::storage* c = cache + off;
      float d = 0.f;
      if (vec) {      // 16-byte loads of the row
        constexpr int N = 16 / sizeof(typename A::storage);
        typedef typename A::storage VecT __attribute__((ext_vector_type(N)));
        for (int i = 0; i < R; i += N) {
          const VecT v = *reinterpret_cast<const VecT*>(c + i);
#pragma unroll
          for (int e = 0; e < N; ++e) d += q[i + e] * A::to_float(v[e]);
        }
      } else {
        for (int i = 0; i < R; ++i) d += q[i] * A::to_float(c[i]);
      }
      s = d;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);      // (m = -inf on the first group: 0)
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int k = 0; k < kMaxCols; ++k) acc[k] *= corr;
    const int n = min(64, pos - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int64_t oj = __shfl(off, jj, 64);
      const typename A::storage* c = cache + oj;
#pragma unroll
      for (int k = 0; k < kMaxCols; ++k) {
        const int i = lane + 64 * k;
        if (i < R) acc[k] += pj * A::to_float(c[i]);
      }
    }
  }
  if (a.sinks) l += expf(a.sinks[h] - m);      // the sink: one more term of the denominator, without a value
  float g = 1.0f / l;
  if (a.gate_pre) {
    const float z = A::to_float(((const typename A::storage*)a.gate_pre)[(int64_t)t * a.gate_stride + h]);
    g = g / (1.0f + expf(-z));
  }
  typename A::storage* og = (typename A::storage*)a.out + (int64_t)t * a.out_token_stride + (int64_t)h * a.out_head_stride;
#pragma unroll
  for (int k = 0; k < kMaxCols; ++k) {
    const int i = lane + 64 * k;
    if (i < R && live) og[i] = A::from_float(acc[k] * g);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Tile form (bfloat16): one wave per 16 rows, a row being a (token, head) pair of ONE sequence's portion, heads fastest —
// sixteen heads of a decoded token, or a few tokens times a few heads.  All rows of a tile read the same keys, which go
// by in chunks of 32: S = Q C^T and O += P C are 16x16x32 MFMAs.  The chunk's rows come straight from the paged cache
// into the B operands of S (a lane's 16 bytes are 8 consecutive columns of one key's row); for O the same registers are
// written to the wave's LDS as they are (row-major image of the chunk, 16 bytes a write) and come back through the
// transposing LDS read (ds_read_b64_tr_b16: a lane gets one column of four rows) as B operands; P goes through LDS from
// the accumulator layout to the A layout.  Inside a chunk the 32 keys are summed in the order the transposing read
// delivers them — lane group g: keys 4g .. 4g+3, then 16+4g .. 16+4g+3 — in both operands.  No workgroup barriers: a wave
// shares nothing with its neighbours.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kPStride = 36;       // u16 per row of P in LDS: 32 slots + 4

template <int KK>                  // ceil(kv_rank / 32), 1 .. 16
__global__ __launch_bounds__(256) void latent_attn_tile_kernel(hxm_latent_attn_args a, int tiles_per_seq, int waves_per_block) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave >= waves_per_block) return;
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1;
  const int64_t witem = (int64_t)blockIdx.x * waves_per_block + wave;      // (sequence, row tile, key split), splits fastest
  if (witem >= (int64_t)a.n_seq * tiles_per_seq * n_splits) return;
  const int64_t item = witem / n_splits;
  const int split = (int)(witem % n_splits);
  const int b = (int)(item / tiles_per_seq), tile = (int)(item % tiles_per_seq);
  const int H = a.n_heads, R = a.kv_rank;
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * H;
  if (tile * 16 >= n_rows) return;
  const int g = lane >> 4, c = lane & 15;
  const int R16 = (R + 15) / 16 * 16;
  const int RS = 2 * (KK * 32) + 32;      // bytes per row of the chunk's image (a key's columns, padded)
  char* img = reinterpret_cast<char*>(lds) + (size_t)wave * (32 * RS + 16 * kPStride * 2);
  u16* pl = reinterpret_cast<u16*>(img + 32 * RS);
  const u16* cache = (const u16*)a.cache;
  const int32_t* table = a.block_table + a.cu_block_lens[b];

  // the queries: lane (g, c) holds row c, columns 32 kk + 8 g .. + 7
  const int last_row = min(tile * 16 + 15, n_rows - 1);
  u16x8 qf[KK];
  {
    const int r = min(tile * 16 + c, n_rows - 1);
    const u16* qg = (const u16*)a.q + (int64_t)(q0 + r / H) * a.q_token_stride + (int64_t)(r % H) * a.q_head_stride;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      if (col < R) qf[kk] = *reinterpret_cast<const u16x8*>(qg + col);
      else qf[kk] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  // the rows this lane holds of S and O: 4 g + i
  int pos[4], lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r < n_rows) {
      pos[i] = a.positions[q0 + r / H];
      lo[i] = a.window > 0 ? max(0, pos[i] - a.window + 1) : 0;
    } else {
      pos[i] = -1;      // sees nothing
      lo[i] = 0;
    }
  }
  // the keys any row of the tile sees: lane (., c) looks at row c, the sixteen are reduced by shuffles
  int k_min, k_max;
  {
    const int r = min(tile * 16 + c, last_row);
    const int pr = a.positions[q0 + r / H];
    k_max = pr;
    k_min = a.window > 0 ? max(0, pr - a.window + 1) : 0;
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

  // a key split takes a run of whole 32-key chunks of the tile's range (the last splits may get none)
  int k_begin = k_min, k_end = k_max;
  if (n_splits > 1) {
    const int chunks = (k_max - k_min + 32) / 32;
    const int per = (chunks + n_splits - 1) / n_splits;
    k_begin = k_min + split * per * 32;
    k_end = min(k_max, k_begin + per * 32 - 1);
  }
  const int bs = a.block_size;
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  // half a chunk's rows, this lane's part: key 16 s + c, columns 32 kk + 8 g .. + 7
  auto fetch = [&](int key0, int s, u16x8 (&cf)[KK]) __attribute__((always_inline)) {
    const int key = min(key0 + 16 * s + c, k_max);        // (a key past the last one repeats it; masked below)
    const int page = bshift >= 0 ? key >> bshift : key / bs;
    const u16* row = cache + (int64_t)table[page] * a.cache_block_stride + (int64_t)(key - page * bs) * a.cache_row_stride;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      if (col < R) cf[kk] = *reinterpret_cast<const u16x8*>(row + col);
      else cf[kk] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  };
  // scores of half a chunk, and its rows into the image for the second product (row = key 16 s + c, the lane's eight
  // columns as they came)
  auto score = [&](int s, const u16x8 (&cf)[KK]) __attribute__((always_inline)) -> f32x4 {
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      v = Mfma<BF16>::mma(qf[kk], cf[kk], v);
      *reinterpret_cast<u16x8*>(img + (16 * s + c) * RS + (32 * kk + 8 * g) * 2) = cf[kk];
    }
    return v;
  };
  auto finish = [&](int key0, const f32x4 (&sc)[2]) __attribute__((always_inline)) {
    // softmax of the rows 4 g + i over this chunk (sc[s][i] is key key0 + 16 s + c)
    float p[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = -INFINITY;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int key = key0 + 16 * s + c;
        const bool seen = key >= lo[i] && key <= pos[i];
        const float v = seen ? sc[s][i] * a.scale : -INFINITY;
        p[s][i] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
      const float m_new = fmaxf(m[i], mx);
      const float corr = __expf(m[i] - m_new);
      float ps = 0.f;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        p[s][i] = __expf(p[s][i] - m_new);       // exp(-inf) = 0 for a key the row does not see
        ps += p[s][i];
      }
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      ps += __shfl_xor(ps, 4, 64);
      ps += __shfl_xor(ps, 8, 64);
      l[i] = l[i] * corr + ps;
      m[i] = m_new;
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) acc[n][i] *= corr;
      // key 16 s + c sits in slot 8 (c / 4) + c % 4 + 4 s of its row
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3)] = BF16::from_float(p[0][i]);
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3) + 4] = BF16::from_float(p[1][i]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // O += P C: A = P[row c][slots 8 g ..], B = the image's column 16 n + c at the keys of those slots
    u16x8 pf;
    {
      const u16x4 x0 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g);
      const u16x4 x1 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g + 4);
      pf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
    const char* vrd = img + (4 * g + (c >> 2)) * RS + (c & 3) * 8;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      {      // (column tiles past the latent's width read zeros of the image: no branch around an MFMA)
        const u16x4 x0 = lds_tr_read(vrd + n * 32);
        const u16x4 x1 = lds_tr_read(vrd + 16 * RS + n * 32);
        const u16x8 vf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        acc[n] = Mfma<BF16>::mma(pf, vf, acc[n]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();      // the reads are done before the next chunk is written
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  {
    // two register sets: the next chunk's rows are on their way while this one is worked on
    u16x8 ca[2][KK], cb[2][KK];
    f32x4 sc[2];
    if (k_begin <= k_end) {
      fetch(k_begin, 0, ca[0]);
      fetch(k_begin, 1, ca[1]);
    }
    for (int key0 = k_begin; key0 <= k_end; key0 += 64) {
      const bool more = key0 + 32 <= k_end;
      if (more) {
        fetch(key0 + 32, 0, cb[0]);
        fetch(key0 + 32, 1, cb[1]);
      }
      sc[0] = score(0, ca[0]);
      sc[1] = score(1, ca[1]);
      finish(key0, sc);
      if (more) {
        if (key0 + 64 <= k_end) {
          fetch(key0 + 64, 0, ca[0]);
          fetch(key0 + 64, 1, ca[1]);
        }
        sc[0] = score(0, cb[0]);
        sc[1] = score(1, cb[1]);
        finish(key0 + 32, sc);
      }
    }
  }
  if (n_splits > 1) {
    // unnormalised partial result of this split: ws_o [item][split][16 rows][R16], ws_ml [item][split][16 rows][m, l]
    float* wo = a.ws_o + ((size_t)witem * 16) * R16;
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
        if (col < R16) wo[(size_t)row * R16 + col] = acc[n][i];
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r >= n_rows) continue;
    const int t = q0 + r / H, h = r % H;
    float gsc = 1.0f / (a.sinks ? l[i] + expf(a.sinks[h] - m[i]) : l[i]);
    if (a.gate_pre) {
      const float z = BF16::to_float(((const u16*)a.gate_pre)[(int64_t)t * a.gate_stride + h]);
      gsc = gsc / (1.0f + __expf(-z));
    }
    u16* og = (u16*)a.out + (int64_t)t * a.out_token_stride + (int64_t)h * a.out_head_stride;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const int col = 16 * n + c;
      if (col < R) og[col] = BF16::from_float(acc[n][i] * gsc);
    }
  }
}

// The same for latents of more than 256 columns: no second register set for the rows on their way (the accumulators
// and the queries leave no room), a whole chunk in registers between its two products.
template <int KK>                  // ceil(kv_rank / 32), 9 .. 16
__global__ __launch_bounds__(256) void latent_attn_tile_wide_kernel(hxm_latent_attn_args a, int tiles_per_seq, int waves_per_block) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave >= waves_per_block) return;
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1;
  const int64_t witem = (int64_t)blockIdx.x * waves_per_block + wave;      // (sequence, row tile, key split), splits fastest
  if (witem >= (int64_t)a.n_seq * tiles_per_seq * n_splits) return;
  const int64_t item = witem / n_splits;
  const int split = (int)(witem % n_splits);
  const int b = (int)(item / tiles_per_seq), tile = (int)(item % tiles_per_seq);
  const int H = a.n_heads, R = a.kv_rank;
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * H;
  if (tile * 16 >= n_rows) return;
  const int g = lane >> 4, c = lane & 15;
  const int R16 = (R + 15) / 16 * 16;
  const int RS = 2 * (KK * 32) + 32;      // bytes per row of the chunk's image (a key's columns, padded)
  char* img = reinterpret_cast<char*>(lds) + (size_t)wave * (32 * RS + 16 * kPStride * 2);
  u16* pl = reinterpret_cast<u16*>(img + 32 * RS);
  const u16* cache = (const u16*)a.cache;
  const int32_t* table = a.block_table + a.cu_block_lens[b];

  // the queries: lane (g, c) holds row c, columns 32 kk + 8 g .. + 7
  const int last_row = min(tile * 16 + 15, n_rows - 1);
  u16x8 qf[KK];
  {
    const int r = min(tile * 16 + c, n_rows - 1);
    const u16* qg = (const u16*)a.q + (int64_t)(q0 + r / H) * a.q_token_stride + (int64_t)(r % H) * a.q_head_stride;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      if (col < R) qf[kk] = *reinterpret_cast<const u16x8*>(qg + col);
      else qf[kk] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  // the rows this lane holds of S and O: 4 g + i
  int pos[4], lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r < n_rows) {
      pos[i] = a.positions[q0 + r / H];
      lo[i] = a.window > 0 ? max(0, pos[i] - a.window + 1) : 0;
    } else {
      pos[i] = -1;      // sees nothing
      lo[i] = 0;
    }
  }
  // the keys any row of the tile sees: lane (., c) looks at row c, the sixteen are reduced by shuffles
  int k_min, k_max;
  {
    const int r = min(tile * 16 + c, last_row);
    const int pr = a.positions[q0 + r / H];
    k_max = pr;
    k_min = a.window > 0 ? max(0, pr - a.window + 1) : 0;
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

  // a key split takes a run of whole 32-key chunks of the tile's range (the last splits may get none)
  int k_begin = k_min, k_end = k_max;
  if (n_splits > 1) {
    const int chunks = (k_max - k_min + 32) / 32;
    const int per = (chunks + n_splits - 1) / n_splits;
    k_begin = k_min + split * per * 32;
    k_end = min(k_max, k_begin + per * 32 - 1);
  }
  for (int key0 = k_begin; key0 <= k_end; key0 += 32) {
    f32x4 sc[2];
    u16x8 cf[2][KK];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int key = min(key0 + 16 * s + c, k_max);        // (a key past the last one repeats it; masked below)
      const u16* row = cache + (int64_t)table[key / a.block_size] * a.cache_block_stride +
                       (int64_t)(key % a.block_size) * a.cache_row_stride;
      sc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const int col = 32 * kk + 8 * g;
        if (col < R) cf[s][kk] = *reinterpret_cast<const u16x8*>(row + col);
        else cf[s][kk] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
        sc[s] = Mfma<BF16>::mma(qf[kk], cf[s][kk], sc[s]);
      }
    }
    // the chunk's image for the second product: row = key 16 s + c, the lane's eight columns as they came
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        *reinterpret_cast<u16x8*>(img + (16 * s + c) * RS + (32 * kk + 8 * g) * 2) = cf[s][kk];
    // softmax of the rows 4 g + i over this chunk (sc[s][i] is key key0 + 16 s + c)
    float p[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = -INFINITY;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int key = key0 + 16 * s + c;
        const bool seen = key >= lo[i] && key <= pos[i];
        const float v = seen ? sc[s][i] * a.scale : -INFINITY;
        p[s][i] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
      const float m_new = fmaxf(m[i], mx);
      const float corr = __expf(m[i] - m_new);
      float ps = 0.f;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        p[s][i] = __expf(p[s][i] - m_new);       // exp(-inf) = 0 for a key the row does not see
        ps += p[s][i];
      }
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      ps += __shfl_xor(ps, 4, 64);
      ps += __shfl_xor(ps, 8, 64);
      l[i] = l[i] * corr + ps;
      m[i] = m_new;
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) acc[n][i] *= corr;
      // key 16 s + c sits in slot 8 (c / 4) + c % 4 + 4 s of its row
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3)] = BF16::from_float(p[0][i]);
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3) + 4] = BF16::from_float(p[1][i]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // O += P C: A = P[row c][slots 8 g ..], B = the image's column 16 n + c at the keys of those slots
    u16x8 pf;
    {
      const u16x4 x0 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g);
      const u16x4 x1 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g + 4);
      pf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
    const char* vrd = img + (4 * g + (c >> 2)) * RS + (c & 3) * 8;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      {      // (column tiles past the latent's width read zeros of the image: no branch around an MFMA)
        const u16x4 x0 = lds_tr_read(vrd + n * 32);
        const u16x4 x1 = lds_tr_read(vrd + 16 * RS + n * 32);
        const u16x8 vf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        acc[n] = Mfma<BF16>::mma(pf, vf, acc[n]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();      // the reads are done before the next chunk is written
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }

  if (n_splits > 1) {
    // unnormalised partial result of this split: ws_o [item][split][16 rows][R16], ws_ml [item][split][16 rows][m, l]
    float* wo = a.ws_o + ((size_t)witem * 16) * R16;
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
        if (col < R16) wo[(size_t)row * R16 + col] = acc[n][i];
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r >= n_rows) continue;
    const int t = q0 + r / H, h = r % H;
    float gsc = 1.0f / (a.sinks ? l[i] + expf(a.sinks[h] - m[i]) : l[i]);
    if (a.gate_pre) {
      const float z = BF16::to_float(((const u16*)a.gate_pre)[(int64_t)t * a.gate_stride + h]);
      gsc = gsc / (1.0f + __expf(-z));
    }
    u16* og = (u16*)a.out + (int64_t)t * a.out_token_stride + (int64_t)h * a.out_head_stride;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const int col = 16 * n + c;
      if (col < R) og[col] = BF16::from_float(acc[n][i] * gsc);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Group form (bfloat16, portions of prompts): a workgroup of four waves takes four consecutive row tiles (64 rows) of a
// sequence and ONE image of every 32-key chunk: each wave brings eight of the chunk's rows from the paged cache into
// LDS, then all four read their B operands of both products from there (16-byte reads for S, transposing reads for O).
// Against the tile form: a quarter of the global reads and LDS writes per wave, and no registers spent on the chunk.
// Two workgroup barriers a chunk (image complete / image free).  Used for latents of more than 256 columns.
// ---------------------------------------------------------------------------------------------------------------
template <int KK>
__global__ __launch_bounds__(256) void latent_attn_group_kernel(hxm_latent_attn_args a, int groups_per_seq) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = blockIdx.x;      // (sequence, group of four row tiles)
  const int b = (int)(item / groups_per_seq), grp = (int)(item % groups_per_seq);
  const int H = a.n_heads, R = a.kv_rank;
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * H;
  if (grp * 64 >= n_rows) return;       // (the whole workgroup)
  const int tile = grp * 4 + wave;
  const bool live = tile * 16 < n_rows; // a wave without rows still brings its share of every chunk
  const int g = lane >> 4, c = lane & 15;
  const int RS = 2 * (KK * 32) + 32;    // bytes per row of the chunk's image (a key's columns, padded)
  char* img = reinterpret_cast<char*>(lds);
  u16* pl = reinterpret_cast<u16*>(img + 32 * RS) + wave * 16 * kPStride;
  const u16* cache = (const u16*)a.cache;
  const int32_t* table = a.block_table + a.cu_block_lens[b];
  // the image's columns past the latent's width stay zero (the loads below never touch them)
  for (int i = threadIdx.x; i < 2 * RS; i += 256) reinterpret_cast<u16x8*>(img)[i] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};

  u16x8 qf[KK];
  {
    const int r = min(tile * 16 + c, n_rows - 1);
    const u16* qg = (const u16*)a.q + (int64_t)(q0 + r / H) * a.q_token_stride + (int64_t)(r % H) * a.q_head_stride;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int col = 32 * kk + 8 * g;
      if (col < R) qf[kk] = *reinterpret_cast<const u16x8*>(qg + col);
      else qf[kk] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  int pos[4], lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r < n_rows) {
      pos[i] = a.positions[q0 + r / H];
      lo[i] = a.window > 0 ? max(0, pos[i] - a.window + 1) : 0;
    } else {
      pos[i] = -1;      // sees nothing
      lo[i] = 0;
    }
  }
  // the keys any row of the GROUP sees (the same in every wave): lane l looks at row 64 grp + l
  int k_min, k_max;
  {
    const int r = min(grp * 64 + lane, n_rows - 1);
    const int pr = a.positions[q0 + r / H];
    k_max = pr;
    k_min = a.window > 0 ? max(0, pr - a.window + 1) : 0;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
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
  const int bs = a.block_size;
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  auto finish = [&](int key0, const f32x4 (&sc)[2]) __attribute__((always_inline)) {
    // softmax of the rows 4 g + i over this chunk (sc[s][i] is key key0 + 16 s + c)
    float p[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = -INFINITY;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int key = key0 + 16 * s + c;
        const bool seen = key >= lo[i] && key <= pos[i];
        const float v = seen ? sc[s][i] * a.scale : -INFINITY;
        p[s][i] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
      const float m_new = fmaxf(m[i], mx);
      const float corr = __expf(m[i] - m_new);
      float ps = 0.f;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        p[s][i] = __expf(p[s][i] - m_new);       // exp(-inf) = 0 for a key the row does not see
        ps += p[s][i];
      }
      ps += __shfl_xor(ps, 1, 64);
      ps += __shfl_xor(ps, 2, 64);
      ps += __shfl_xor(ps, 4, 64);
      ps += __shfl_xor(ps, 8, 64);
      l[i] = l[i] * corr + ps;
      m[i] = m_new;
#pragma unroll
      for (int n = 0; n < KK * 2; ++n) acc[n][i] *= corr;
      // key 16 s + c sits in slot 8 (c / 4) + c % 4 + 4 s of its row
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3)] = BF16::from_float(p[0][i]);
      pl[(4 * g + i) * kPStride + 8 * (c >> 2) + (c & 3) + 4] = BF16::from_float(p[1][i]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // O += P C: A = P[row c][slots 8 g ..], B = the image's column 16 n + c at the keys of those slots
    u16x8 pf;
    {
      const u16x4 x0 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g);
      const u16x4 x1 = *reinterpret_cast<const u16x4*>(pl + c * kPStride + 8 * g + 4);
      pf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
    const char* vrd = img + (4 * g + (c >> 2)) * RS + (c & 3) * 8;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      {      // (column tiles past the latent's width read zeros of the image: no branch around an MFMA)
        const u16x4 x0 = lds_tr_read(vrd + n * 32);
        const u16x4 x1 = lds_tr_read(vrd + 16 * RS + n * 32);
        const u16x8 vf = u16x8{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        acc[n] = Mfma<BF16>::mma(pf, vf, acc[n]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();      // the reads are done before the next chunk is written
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  __syncthreads();      // the zeroed image
  for (int key0 = k_min; key0 <= k_max; key0 += 32) {
    // this wave's eight rows of the chunk: key0 + 8 wave + kq, a lane brings eight columns
#pragma unroll
    for (int kq = 0; kq < 8; ++kq) {
      const int key = min(key0 + 8 * wave + kq, k_max);      // (a key past the last one repeats it; masked in the softmax)
      const int page = bshift >= 0 ? key >> bshift : key / bs;
      const u16* row = cache + (int64_t)table[page] * a.cache_block_stride + (int64_t)(key - page * bs) * a.cache_row_stride;
      for (int col = lane * 8; col < R; col += 512)
        *reinterpret_cast<u16x8*>(img + (8 * wave + kq) * RS + col * 2) = *reinterpret_cast<const u16x8*>(row + col);
    }
    __syncthreads();      // the image is complete
    if (live) {
      f32x4 sc[2];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        sc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
          sc[s] = Mfma<BF16>::mma(qf[kk], *reinterpret_cast<const u16x8*>(img + (16 * s + c) * RS + (32 * kk + 8 * g) * 2), sc[s]);
      }
      finish(key0, sc);
    }
    __syncthreads();      // every wave is done with the image
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 16 + 4 * g + i;
    if (r >= n_rows) continue;
    const int t = q0 + r / H, h = r % H;
    float gsc = 1.0f / (a.sinks ? l[i] + expf(a.sinks[h] - m[i]) : l[i]);
    if (a.gate_pre) {
      const float z = BF16::to_float(((const u16*)a.gate_pre)[(int64_t)t * a.gate_stride + h]);
      gsc = gsc / (1.0f + __expf(-z));
    }
    u16* og = (u16*)a.out + (int64_t)t * a.out_token_stride + (int64_t)h * a.out_head_stride;
#pragma unroll
    for (int n = 0; n < KK * 2; ++n) {
      const int col = 16 * n + c;
      if (col < R) og[col] = BF16::from_float(acc[n][i] * gsc);
    }
  }
}

// the splits of a (sequence, row tile) merged: out = sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M), times the head gate
__global__ __launch_bounds__(256) void latent_attn_combine_kernel(hxm_latent_attn_args a, int tiles_per_seq) {
  const int64_t item = blockIdx.x;
  const int b = (int)(item / tiles_per_seq), tile = (int)(item % tiles_per_seq);
  const int H = a.n_heads, R = a.kv_rank, R16 = (R + 15) / 16 * 16, NS = a.n_splits;
  const int q0 = a.q_cu[b];
  const int n_rows = (a.q_cu[b + 1] - q0) * H;
  if (tile * 16 >= n_rows) return;
  __shared__ float wgt[16][65];      // [row][split] weight e^(m_s - M) / L (NS <= 64)
  if (threadIdx.x < 16) {
    const int row = threadIdx.x;
    const float* wml = a.ws_ml + (size_t)item * NS * 32;
    float M = -1.0e30f;
    for (int s = 0; s < NS; ++s) M = fmaxf(M, wml[s * 32 + 2 * row]);
    float L = 0.f;
    for (int s = 0; s < NS; ++s) L += wml[s * 32 + 2 * row + 1] * __expf(wml[s * 32 + 2 * row] - M);
    const int r = tile * 16 + row;
    if (a.sinks && r < n_rows) L += expf(a.sinks[r % H] - M);      // the sink counts once, here
    float gsc = L > 0.f ? 1.0f / L : 0.f;
    if (a.gate_pre && r < n_rows) {
      const float z = BF16::to_float(((const u16*)a.gate_pre)[(int64_t)(q0 + r / H) * a.gate_stride + r % H]);
      gsc = gsc / (1.0f + __expf(-z));
    }
    for (int s = 0; s < NS; ++s) wgt[row][s] = __expf(wml[s * 32 + 2 * row] - M) * gsc;
  }
  __syncthreads();
  const float* wo = a.ws_o + (size_t)item * NS * 16 * R16;
  for (int e = threadIdx.x; e < 16 * R; e += 256) {
    const int row = e / R, col = e % R;
    const int r = tile * 16 + row;
    if (r >= n_rows) continue;
    float v = 0.f;
    for (int s = 0; s < NS; ++s) v += wo[((size_t)s * 16 + row) * R16 + col] * wgt[row][s];
    ((u16*)a.out)[(int64_t)(q0 + r / H) * a.out_token_stride + (int64_t)(r % H) * a.out_head_stride + col] = BF16::from_float(v);
  }
}

// key splits for a launch: enough waves to fill the chip when there are few (sequence, row tile) items — decode steps
static int tile_splits(const hxm_latent_attn_args& a) {
  const int tiles_per_seq = (int)(((int64_t)a.max_q_len * a.n_heads + 15) / 16);
  const int64_t items = (int64_t)a.n_seq * tiles_per_seq;
  int reach = a.max_kv_len > 0 ? a.max_kv_len : 1;
  if (a.window > 0 && a.window + a.max_q_len < reach) reach = a.window + a.max_q_len;
  const int chunks = (reach + 31) / 32;
  int64_t want = (2048 + items - 1) / items;      // ~8 waves per CU
  if (want > chunks / 2) want = chunks / 2;          // at least two chunks a split
  if (want > 64) want = 64;
  return want < 2 ? 1 : (int)want;
}

template <int KK>
int launch_tile(const hxm_latent_attn_args& a, hipStream_t s) {
  const size_t per_wave = (size_t)32 * (2 * (KK * 32) + 32) + 16 * kPStride * 2;
  int waves = 4;
  while (waves > 1 && per_wave * waves > 64 * 1024) waves >>= 1;
  const int tiles_per_seq = (int)(((int64_t)a.max_q_len * a.n_heads + 15) / 16);
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1;
  if (n_splits > 1 && (n_splits > 64 || !a.ws_o || !a.ws_ml)) return HX_ERR_WORKSPACE;
  // (measured: the group form wins where the tile form has no room for its second register set — latents of more than 256
  //  columns: 1136 -> 891 us at 512 columns — and loses below: 89 -> 140 us at 64 columns)
  if (KK > 8 && n_splits == 1 && tiles_per_seq >= 4 && hxm::tile_form() == 1) {
    const int groups_per_seq = (tiles_per_seq + 3) / 4;
    const size_t lds_g = (size_t)32 * (2 * (KK * 32) + 32) + 4 * 16 * kPStride * 2;
    latent_attn_group_kernel<KK><<<dim3((unsigned)((int64_t)a.n_seq * groups_per_seq)), dim3(256), lds_g, s>>>(a, groups_per_seq);
    return hxm::check_launch();
  }
  const int64_t items = (int64_t)a.n_seq * tiles_per_seq;
  const dim3 grid((unsigned)((items * n_splits + waves - 1) / waves));
  if constexpr (KK <= 8) latent_attn_tile_kernel<KK><<<grid, dim3(64 * waves), per_wave * waves, s>>>(a, tiles_per_seq, waves);
  else latent_attn_tile_wide_kernel<KK><<<grid, dim3(64 * waves), per_wave * waves, s>>>(a, tiles_per_seq, waves);
  if (n_splits > 1) latent_attn_combine_kernel<<<dim3((unsigned)items), dim3(256), 0, s>>>(a, tiles_per_seq);
  return hxm::check_launch();
}

}  // namespace

extern "C" int hxm_latent_norm_cache(const void* proj, int64_t proj_stride, int64_t q_off, int64_t q_rank, int64_t kv_off,
                                     int64_t kv_rank, const float* q_w, const float* kv_w, float eps, void* cq_out,
                                     const int32_t* slot_ids, void* cache, int64_t cache_block_stride,
                                     int64_t cache_row_stride, int32_t block_size, int64_t n_tokens, int dtype, void* stream) {
  if (n_tokens < 0 || q_rank < 1 || kv_rank < 1 || block_size < 1 || q_off < 0 || kv_off < 0) return HX_ERR_SHAPE;
  if (n_tokens == 0) return HX_OK;
  if (!proj || !q_w || !kv_w || !cq_out || !slot_ids || !cache) return HX_ERR_NULL;
  if (proj_stride < q_off + q_rank || proj_stride < kv_off + kv_rank || cache_row_stride < kv_rank) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t esz = dtype == HX_F32 ? 4 : 2;
  auto al = [&](const void* q, int64_t bytes) { return (reinterpret_cast<uintptr_t>(q) % bytes) == 0; };
  const int vec = (q_rank % 4 == 0 && kv_rank % 4 == 0 && q_off % 4 == 0 && kv_off % 4 == 0 && proj_stride % 4 == 0 &&
                   cache_row_stride % 4 == 0 && cache_block_stride % 4 == 0 && al(proj, 4 * esz) && al(cq_out, 4 * esz) &&
                   al(cache, 4 * esz) && al(q_w, 16) && al(kv_w, 16)) ? 1 : 0;
  switch (dtype) {
    case HX_F32:
      latent_norm_cache_kernel<F32><<<dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, s>>>(
          (const float*)proj, proj_stride, q_off, q_rank, kv_off, kv_rank, q_w, kv_w, eps, (float*)cq_out, slot_ids,
          (float*)cache, cache_block_stride, cache_row_stride, block_size, n_tokens, vec);
      break;
    case HX_BF16:
      latent_norm_cache_kernel<BF16><<<dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, s>>>(
          (const u16*)proj, proj_stride, q_off, q_rank, kv_off, kv_rank, q_w, kv_w, eps, (u16*)cq_out, slot_ids,
          (u16*)cache, cache_block_stride, cache_row_stride, block_size, n_tokens, vec);
      break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}

static bool tile_form_serves(const hxm_latent_attn_args& a) {
  const bool aligned = a.kv_rank % 8 == 0 && a.cache_row_stride % 8 == 0 && a.cache_block_stride % 8 == 0 &&
                       a.q_token_stride % 8 == 0 && a.q_head_stride % 8 == 0 && aligned16(a.cache) && aligned16(a.q);
  return a.dtype == HX_BF16 && aligned && a.kv_rank <= 512 && hxm::tile_form();
}

extern "C" int hxm_latent_attention_plan(const hxm_latent_attn_args* args, int32_t* n_splits, int64_t* ws_floats) {
  if (!args || !n_splits || !ws_floats) return HX_ERR_NULL;
  *n_splits = 1;
  *ws_floats = 0;
  if (args->n_tokens <= 0 || args->max_q_len < 1 || args->n_seq < 1 || !tile_form_serves(*args)) return HX_OK;
  const int ns = tile_splits(*args);
  if (ns > 1) {
    const int64_t tiles_per_seq = ((int64_t)args->max_q_len * args->n_heads + 15) / 16;
    const int64_t R16 = (args->kv_rank + 15) / 16 * 16;
    *n_splits = ns;
    *ws_floats = (int64_t)args->n_seq * tiles_per_seq * ns * 16 * (R16 + 2);
  }
  return HX_OK;
}

extern "C" int hxm_latent_attention(const hxm_latent_attn_args* args, void* stream) {
  if (!args) return HX_ERR_NULL;
  const hxm_latent_attn_args& a = *args;
  if (a.n_tokens < 0 || a.n_seq < 1 || a.n_heads < 1 || a.kv_rank < 1 || a.kv_rank > HXM_MAX_LATENT || a.block_size < 1)
    return HX_ERR_SHAPE;
  if (a.n_tokens == 0) return HX_OK;
  if (!a.out || !a.q || !a.cache || !a.tok_seq || !a.positions || !a.q_cu || !a.block_table || !a.cu_block_lens) return HX_ERR_NULL;
  if (a.cache_row_stride < a.kv_rank) return HX_ERR_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  if (a.max_q_len < 1) return HX_ERR_SHAPE;
  if (tile_form_serves(a)) {
    switch ((a.kv_rank + 31) / 32) {
      case 1: return launch_tile<1>(a, s);
      case 2: return launch_tile<2>(a, s);
      case 3: return launch_tile<3>(a, s);
      case 4: return launch_tile<4>(a, s);
      case 5: case 6: return launch_tile<6>(a, s);
      case 7: case 8: return launch_tile<8>(a, s);
      case 9: case 10: return launch_tile<10>(a, s);
      case 11: case 12: return launch_tile<12>(a, s);
      default: return launch_tile<16>(a, s);
    }
  }
  const int64_t items = (int64_t)a.n_tokens * a.n_heads;
  const dim3 grid((unsigned)((items + 3) / 4));
  const size_t lds = (size_t)4 * a.kv_rank * sizeof(float);
  switch (a.dtype) {
    case HX_F32: latent_attn_rows_kernel<F32><<<grid, dim3(256), lds, s>>>(a); break;
    case HX_BF16: latent_attn_rows_kernel<BF16><<<grid, dim3(256), lds, s>>>(a); break;
    default: return HX_ERR_DTYPE;
  }
  return hxm::check_launch();
}
