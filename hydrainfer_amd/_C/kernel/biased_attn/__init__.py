"""Grouped-query attention over a paged key/value cache with a per-head linear distance bias and a causal, windowed or
chunked mask (csrc/biased_attn.hip, libhydra_mix.so):
    score(i, j) = cap(q_i . k_j * scale) - slopes[h] * (i - j),   softmax over the keys j that position i sees,
with cap(s) = softcap * tanh(s / softcap) when a soft cap is given and s otherwise.
Key rows (dim) and value rows (vdim) may differ in size; a cache row holds kv_heads heads of `head_size` elements and the
keys / values fill the first dim / vdim of each.  The caches are the pool planes [n_blocks, block_size, kv_heads, head_size]
of the block manager; a layer with fewer heads than the pool's rows hold uses the first of each row."""
import ctypes
from typing import Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib

MASK_KINDS = {"causal": 0, "window": 1, "chunk": 2}


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"biased attention: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


def _cache_layout(cache: Tensor, kv_heads: int):
    if cache.dim() != 4 or cache.shape[2] < kv_heads or cache.stride(3) != 1:
        raise _lib.HydraHipError("cache planes must be [n_blocks, block_size, >= kv_heads, head_size] with contiguous rows")
    if cache.stride(0) % cache.stride(1) or cache.stride(0) // cache.stride(1) != cache.shape[1]:
        raise _lib.HydraHipError("cache planes: a block's rows must follow each other (slot = block * block_size + row)")
    return cache.stride(0), cache.stride(1), cache.stride(2), cache.shape[1]


def qk_norm_cache(proj: Tensor, q_size: int, k_size: int, v_size: int, q_w: Optional[Tensor], k_w: Optional[Tensor],
                  eps: float, kv_heads: int, slot_ids: Optional[Tensor] = None, key_cache: Optional[Tensor] = None,
                  value_cache: Optional[Tensor] = None) -> Tensor:
    """proj: [n_tokens, q_size + k_size + v_size] (q | k | v).  Returns q = rms_norm(q part) * q_w (ONE norm over the whole
    projection, all heads at once; q_w None: unchanged); with k_size > 0 the keys — normed the same way with k_w — and the
    values go to the cache rows slot_ids (int32, slot = block * block_size + row)."""
    _lib.require_gpu(proj, q_w, k_w, slot_ids, key_cache, value_cache)
    if proj.dim() != 2 or proj.stride(1) != 1 or proj.shape[1] < q_size + k_size + v_size:
        raise _lib.HydraHipError("qk_norm_cache: proj must be 2-D with contiguous rows of q | k | v")
    for w, n in ((q_w, q_size), (k_w, k_size)):
        if w is not None and (w.dtype != torch.float32 or not w.is_contiguous() or w.numel() != n):
            raise _lib.HydraHipError("qk_norm_cache: norm weights must be contiguous float32 of the projection's length")
    T = proj.shape[0]
    bstride = rstride = hstride = 0
    if k_size > 0:
        if key_cache is None or value_cache is None or slot_ids is None or key_cache.dtype != proj.dtype or \
                value_cache.dtype != proj.dtype or value_cache.stride() != key_cache.stride():
            raise _lib.HydraHipError("qk_norm_cache: key and value caches of proj's dtype and one layout, with slot_ids")
        if slot_ids.dtype != torch.int32 or not slot_ids.is_contiguous() or slot_ids.numel() != T:
            raise _lib.HydraHipError("qk_norm_cache: slot_ids must be contiguous int32 [n_tokens]")
        bstride, rstride, hstride, _ = _cache_layout(key_cache, kv_heads)
    q = torch.empty((T, q_size), dtype=proj.dtype, device=proj.device)
    _lib.mix_check(_lib.mix_lib().hxm_qk_norm_cache(
        proj.data_ptr(), proj.stride(0), 0, q_size, q_size, k_size, q_size + k_size, v_size,
        None if q_w is None else q_w.data_ptr(), None if k_w is None else k_w.data_ptr(), float(eps), q.data_ptr(),
        None if slot_ids is None else slot_ids.data_ptr(), None if key_cache is None else key_cache.data_ptr(),
        None if value_cache is None else value_cache.data_ptr(), rstride, hstride, int(kv_heads), T, _code(proj.dtype),
        _lib.current_stream()), "qk_norm_cache")
    return q


def biased_attention(q: Tensor, key_cache: Tensor, value_cache: Tensor, vdim: int, tok_seq: Tensor, positions: Tensor,
                     q_cu: Tensor, block_table: Tensor, cu_block_lens: Tensor, scale: float,
                     slopes: Optional[Tensor] = None, mask: str = "causal", mask_size: int = 0, max_q_len: int = 0,
                     kv_heads: Optional[int] = None, max_kv_len: int = 0, form: str = "auto", softcap: float = 0.0,
                     head_scale: Optional[Tensor] = None, sinks: Optional[Tensor] = None) -> Tensor:
    """q: [n_tokens, n_heads, dim] contiguous.  kv_heads: the key / value heads in use (the first of every cache row;
    default: all the plane has).  max_q_len: the longest portion of the batch; max_kv_len: the most keys a sequence holds —
    with few rows in the launch (decode steps) the keys of every tile are dealt to several waves.  form: "auto" (bfloat16
    with sizes that are multiples of 8: the MFMA forms — portions of prompts share every chunk of keys between four row
    tiles, decode steps split the keys), "tile" (the MFMA tile form throughout) or "rows" (one wave per token and head, any
    dtype and size).  head_scale [n_heads]: head h's scores are multiplied by head_scale[h] as well (a temperature per head);
    sinks [n_heads]: the softmax's denominator of head h holds one more term exp(sinks[h]) without a key or a value.
    Returns [n_tokens, n_heads, vdim]."""
    _lib.require_gpu(q, key_cache, value_cache, tok_seq, positions, q_cu, block_table, cu_block_lens, slopes, head_scale, sinks)
    if q.dim() != 3 or not q.is_contiguous() or key_cache.dtype != q.dtype or value_cache.dtype != q.dtype:
        raise _lib.HydraHipError("biased_attention: q contiguous [n_tokens, n_heads, dim], caches of the same dtype")
    T, H, D = q.shape
    G = int(kv_heads) if kv_heads else key_cache.shape[2]
    if value_cache.stride() != key_cache.stride() or H % G:
        raise _lib.HydraHipError("biased_attention: key and value caches of one layout; heads a multiple of kv heads")
    bstride, rstride, hstride, bs = _cache_layout(key_cache, G)
    if D > key_cache.shape[3] or vdim > key_cache.shape[3]:
        raise _lib.HydraHipError("biased_attention: dim / vdim exceed the cache's head size")
    n_seq = q_cu.numel() - 1
    for t, name, n in ((tok_seq, "tok_seq", T), (positions, "positions", T), (q_cu, "q_cu", n_seq + 1),
                       (cu_block_lens, "cu_block_lens", n_seq + 1), (block_table, "block_table", block_table.numel())):
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
            raise _lib.HydraHipError(f"biased_attention: {name} must be contiguous int32 [{n}]")
    if slopes is not None and (slopes.dtype != torch.float32 or not slopes.is_contiguous() or slopes.numel() != H):
        raise _lib.HydraHipError("biased_attention: slopes must be contiguous float32 [n_heads]")
    for w, name in ((head_scale, "head_scale"), (sinks, "sinks")):
        if w is not None and (w.dtype != torch.float32 or not w.is_contiguous() or w.numel() != H):
            raise _lib.HydraHipError(f"biased_attention: {name} must be contiguous float32 [n_heads]")
    if mask not in MASK_KINDS or (mask != "causal" and mask_size < 1):
        raise _lib.HydraHipError(f"biased_attention: mask {mask!r} of size {mask_size}")
    out = torch.empty((T, H, vdim), dtype=q.dtype, device=q.device)
    a = _lib.hxm_biased_attn_args()
    a.head_scale = None if head_scale is None else head_scale.data_ptr()
    a.sinks = None if sinks is None else sinks.data_ptr()
    a.out, a.q, a.key_cache, a.value_cache = out.data_ptr(), q.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr()
    a.slopes = None if slopes is None else slopes.data_ptr()
    a.tok_seq, a.positions, a.q_cu = tok_seq.data_ptr(), positions.data_ptr(), q_cu.data_ptr()
    a.block_table, a.cu_block_lens = block_table.data_ptr(), cu_block_lens.data_ptr()
    a.cache_block_stride, a.cache_row_stride, a.head_stride, a.block_size = bstride, rstride, hstride, bs
    a.n_tokens, a.n_heads, a.kv_heads, a.dim, a.vdim = T, H, G, D, int(vdim)
    a.mask_kind, a.mask_size, a.scale, a.dtype = MASK_KINDS[mask], int(mask_size), float(scale), _code(q.dtype)
    a.n_seq, a.max_q_len, a.softcap = n_seq, int(max_q_len), float(softcap or 0.0)
    a.form, a.n_splits, a.ws_o, a.ws_ml = {"auto": 0, "rows": 1, "tile": 2}[form], 1, None, None
    if form in ("auto", "tile") and q.dtype == torch.bfloat16 and max_q_len > 0 and max_kv_len > 0 and D % 8 == 0 and vdim % 8 == 0 \
            and D <= 256 and vdim <= 256:
        # key splits: enough waves to fill the chip when the launch has few row tiles, at least two 32-key chunks a split
        tiles = n_seq * G * ((max_q_len * (H // G) + 15) // 16)
        reach = max_kv_len
        if mask != "causal":
            reach = min(reach, mask_size + (max_q_len if mask == "window" else 0))
        ns = min((2048 + tiles - 1) // tiles, ((reach + 31) // 32) // 2, 64)
        if ns > 1:
            v16 = (vdim + 15) // 16 * 16
            ws = torch.empty(tiles * ns * 16 * (v16 + 2), dtype=torch.float32, device=q.device)
            a.n_splits, a.ws_o, a.ws_ml = ns, ws.data_ptr(), ws.data_ptr() + 4 * tiles * ns * 16 * v16
    _lib.mix_check(_lib.mix_lib().hxm_biased_attention(ctypes.byref(a), _lib.current_stream()), "biased_attention")
    return out
