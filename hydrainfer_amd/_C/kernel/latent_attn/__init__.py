"""Attention over a paged cache of low-rank latents (csrc/latent_attn.hip, libhydra_mix.so).

A token leaves one row c of kv_rank numbers in the cache; a head's key and value are linear maps of c.  With the key map
folded into the query and the value map applied to the result, every head attends over the same rows:
    out[t, h] = sum_j softmax_j(q[t, h] . c_j * scale) c_j      over the keys j that position i = positions[t] sees
(0 <= i - j < window, or every j <= i without a window).  The cache is a pool plane [n_blocks, block_size, 1, row_width]
of the block manager (row_width >= kv_rank), addressed through the batch's block tables."""
import ctypes
from typing import Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"latent attention: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


def _cache_strides(cache: Tensor, kv_rank: int):
    if cache.dim() != 4 or cache.shape[2] != 1 or cache.shape[3] < kv_rank or cache.stride(3) != 1:
        raise _lib.HydraHipError("latent cache must be [n_blocks, block_size, 1, >= kv_rank] with contiguous rows")
    return cache.stride(0), cache.stride(1), cache.shape[1]


def latent_norm_cache(proj: Tensor, q_off: int, q_rank: int, kv_off: int, kv_rank: int, q_w: Tensor, kv_w: Tensor,
                      eps: float, slot_ids: Tensor, cache: Tensor) -> Tensor:
    """cq = rms_norm(proj[:, q_off : q_off + q_rank]) * q_w is returned; c = rms_norm(proj[:, kv_off : kv_off + kv_rank])
    * kv_w goes to the cache rows slot_ids (int32, slot = block * block_size + row)."""
    _lib.require_gpu(proj, q_w, kv_w, slot_ids, cache)
    if proj.dim() != 2 or proj.stride(1) != 1 or cache.dtype != proj.dtype:
        raise _lib.HydraHipError("latent_norm_cache: proj 2-D with contiguous rows, cache of the same dtype")
    for w, n in ((q_w, q_rank), (kv_w, kv_rank)):
        if w.dtype != torch.float32 or not w.is_contiguous() or w.numel() != n:
            raise _lib.HydraHipError("latent_norm_cache: norm weights must be contiguous float32 of the latent's length")
    if slot_ids.dtype != torch.int32 or not slot_ids.is_contiguous() or slot_ids.numel() != proj.shape[0]:
        raise _lib.HydraHipError("latent_norm_cache: slot_ids must be contiguous int32 [n_tokens]")
    bstride, rstride, bs = _cache_strides(cache, kv_rank)
    cq = torch.empty((proj.shape[0], q_rank), dtype=proj.dtype, device=proj.device)
    _lib.mix_check(_lib.mix_lib().hxm_latent_norm_cache(
        proj.data_ptr(), proj.stride(0), q_off, q_rank, kv_off, kv_rank, q_w.data_ptr(), kv_w.data_ptr(), float(eps),
        cq.data_ptr(), slot_ids.data_ptr(), cache.data_ptr(), bstride, rstride, bs, proj.shape[0], _code(proj.dtype),
        _lib.current_stream()), "latent_norm_cache")
    return cq


def latent_attention(q: Tensor, cache: Tensor, tok_seq: Tensor, positions: Tensor, q_cu: Tensor, block_table: Tensor,
                     cu_block_lens: Tensor, scale: float, window: Optional[int], max_q_len: int,
                     gate_pre: Optional[Tensor] = None, out: Optional[Tensor] = None, max_kv_len: int = 0,
                     sinks: Optional[Tensor] = None) -> Tensor:
    """q: [n_tokens, n_heads, kv_rank] (any token / head strides, contiguous rows).  max_kv_len: the most keys a sequence
    of the batch holds — lets a launch with few rows (decode steps) deal every row tile's keys to several waves.  gate_pre [n_tokens, >= n_heads]:
    the result of head h is multiplied by sigmoid(gate_pre[t, h]).  sinks [n_heads] float32: the softmax's denominator of
    head h holds one more term exp(sinks[h]) without a key or a value.  Returns [n_tokens, n_heads, kv_rank]."""
    _lib.require_gpu(q, cache, tok_seq, positions, q_cu, block_table, cu_block_lens, gate_pre, out, sinks)
    if q.dim() != 3 or q.stride(2) != 1 or cache.dtype != q.dtype:
        raise _lib.HydraHipError("latent_attention: q [n_tokens, n_heads, kv_rank] with contiguous rows, cache of the same dtype")
    T, H, R = q.shape
    if R > _lib.HXM_MAX_LATENT:
        raise _lib.HydraHipError(f"latent_attention: kv_rank {R} > {_lib.HXM_MAX_LATENT}")
    n_seq = q_cu.numel() - 1
    for t, name, n in ((tok_seq, "tok_seq", T), (positions, "positions", T), (q_cu, "q_cu", n_seq + 1),
                       (cu_block_lens, "cu_block_lens", n_seq + 1), (block_table, "block_table", block_table.numel())):
        if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
            raise _lib.HydraHipError(f"latent_attention: {name} must be contiguous int32 [{n}]")
    if out is None:
        out = torch.empty((T, H, R), dtype=q.dtype, device=q.device)
    elif out.shape != q.shape or out.dtype != q.dtype or out.stride(2) != 1:
        raise _lib.HydraHipError("latent_attention: out must look like q")
    if sinks is not None and (sinks.dtype != torch.float32 or not sinks.is_contiguous() or sinks.numel() != H):
        raise _lib.HydraHipError("latent_attention: sinks must be contiguous float32 [n_heads]")
    a = _lib.hxm_latent_attn_args()
    a.sinks = None if sinks is None else sinks.data_ptr()
    a.out, a.q, a.cache = out.data_ptr(), q.data_ptr(), cache.data_ptr()
    a.gate_pre = None
    a.gate_stride = 0
    if gate_pre is not None:
        if gate_pre.dtype != q.dtype or gate_pre.dim() != 2 or gate_pre.shape[0] != T or gate_pre.shape[1] < H or gate_pre.stride(1) != 1:
            raise _lib.HydraHipError("latent_attention: gate_pre must be [n_tokens, >= n_heads] of q's dtype")
        a.gate_pre, a.gate_stride = gate_pre.data_ptr(), gate_pre.stride(0)
    a.tok_seq, a.positions, a.q_cu = tok_seq.data_ptr(), positions.data_ptr(), q_cu.data_ptr()
    a.block_table, a.cu_block_lens = block_table.data_ptr(), cu_block_lens.data_ptr()
    a.q_token_stride, a.q_head_stride = q.stride(0), q.stride(1)
    a.out_token_stride, a.out_head_stride = out.stride(0), out.stride(1)
    a.cache_block_stride, a.cache_row_stride, a.block_size = _cache_strides(cache, R)
    a.n_tokens, a.n_seq, a.n_heads, a.kv_rank = T, n_seq, H, R
    a.window = int(window) if window else 0
    a.max_q_len = int(max_q_len)
    a.scale = float(scale)
    a.dtype = _code(q.dtype)
    a.max_kv_len = int(max_kv_len)      # (0: unknown — no key splits)
    a.n_splits, a.ws_o, a.ws_ml = 1, None, None
    if max_kv_len > 0:
        ns, need = ctypes.c_int32(1), ctypes.c_int64(0)
        _lib.mix_check(_lib.mix_lib().hxm_latent_attention_plan(ctypes.byref(a), ctypes.byref(ns), ctypes.byref(need)), "latent_attention_plan")
        if ns.value > 1:
            ws = torch.empty(need.value, dtype=torch.float32, device=q.device)
            n_o = need.value // ((R + 15) // 16 * 16 + 2) * ((R + 15) // 16 * 16)
            a.n_splits, a.ws_o, a.ws_ml = ns.value, ws.data_ptr(), ws.data_ptr() + 4 * n_o
    _lib.mix_check(_lib.mix_lib().hxm_latent_attention(ctypes.byref(a), _lib.current_stream()), "latent_attention")
    return out
