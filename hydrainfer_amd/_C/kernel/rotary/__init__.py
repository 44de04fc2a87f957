"""Rotary positions over parts of a token's row (csrc/rope_ops.hip, libhydra_mix.so).

A part is a group of heads (queries, keys, values, or a mixer's result) of which a range of channels turns by the
token's position — pairs (i, i + dims / 2) ("halves") or (2 i, 2 i + 1) ("interleaved"), forwards or back — while the
other channels are copied.  A part lands in an output matrix or in the paged cache (at a column offset of the cache row,
so a latent and a rotated key part can share a row) and may be multiplied by a sigmoid gate per head or per element.
One launch takes up to three parts: what a token's q | k | v projection needs before attention is one kernel."""
import ctypes
from dataclasses import dataclass
from typing import List, Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib

LAYOUTS = {"halves": 0, "interleaved": 1}
GATES = {"head": 1, "element": 2}
MAX_PARTS = 3


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"rotary: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


@dataclass
class RotaryPart:
    src: Tensor                          # [n_tokens, >= heads * size] rows (a view of a projection's columns will do)
    heads: int
    size: int                            # elements of a head
    inv_freq: Optional[Tensor] = None    # float64 [rot_dims / 2] on the device; None: nothing turns
    rot_off: int = 0                     # first turning channel of every head
    layout: str = "halves"
    mag: float = 1.0                     # factor on cos and sin
    back: bool = False                   # turn by - position
    dst: Optional[Tensor] = None         # [n_tokens, heads * size] rows; None with no cache: a new tensor
    cache: Optional[Tensor] = None       # a pool plane [n_blocks, block_size, rows..., head_size]: the part goes to the token's row
    cache_col: int = 0                   # first column of the cache row the part's first head takes
    cache_head_stride: Optional[int] = None   # columns from one head to the next in the cache row (default: size)
    gate: Optional[Tensor] = None        # [n_tokens, heads] ("head") or [n_tokens, heads * size] ("element") rows of pre-sigmoid gates
    gate_kind: str = "head"
    src_head_stride: Optional[int] = None


def rotary_parts(parts: List[RotaryPart], positions: Tensor, slot_ids: Optional[Tensor] = None) -> List[Optional[Tensor]]:
    """Runs the parts in one launch; returns, per part, the output matrix [n_tokens, heads * size] (None for a cache part)."""
    if not 1 <= len(parts) <= MAX_PARTS:
        raise _lib.HydraHipError(f"rotary_parts: 1 .. {MAX_PARTS} parts a launch")
    T = positions.numel()
    if positions.dtype != torch.int32 or not positions.is_contiguous():
        raise _lib.HydraHipError("rotary_parts: positions must be contiguous int32 [n_tokens]")
    _lib.require_gpu(positions, slot_ids)
    a = _lib.hxm_rotary_args()
    outs: List[Optional[Tensor]] = []
    dtype = parts[0].src.dtype
    block_size = 1
    for i, p in enumerate(parts):
        _lib.require_gpu(p.src, p.inv_freq, p.dst, p.cache, p.gate)
        s = p.src
        shs = p.size if p.src_head_stride is None else int(p.src_head_stride)
        if s.dim() != 2 or s.shape[0] != T or s.stride(1) != 1 or s.dtype != dtype or s.shape[1] < (p.heads - 1) * shs + p.size:
            raise _lib.HydraHipError(f"rotary_parts: part {i}: src must be [n_tokens, >= heads * size] rows of one dtype")
        q = a.parts[i]
        q.src, q.src_stride, q.src_head_stride = s.data_ptr(), s.stride(0), shs
        q.heads, q.size, q.rot_off, q.rot_dims = int(p.heads), int(p.size), int(p.rot_off), 0
        q.inv_freq = None
        if p.inv_freq is not None:
            if p.inv_freq.dtype != torch.float64 or not p.inv_freq.is_contiguous() or p.inv_freq.numel() < 1:
                raise _lib.HydraHipError(f"rotary_parts: part {i}: inv_freq must be contiguous float64 [rot_dims / 2]")
            q.inv_freq, q.rot_dims = p.inv_freq.data_ptr(), 2 * p.inv_freq.numel()
        q.layout, q.mag, q.sign = LAYOUTS[p.layout], float(p.mag), -1.0 if p.back else 1.0
        q.gate, q.gate_stride, q.gate_kind = None, 0, 0
        if p.gate is not None:
            need = p.heads if p.gate_kind == "head" else p.heads * p.size
            if p.gate.dtype != dtype or p.gate.dim() != 2 or p.gate.shape[0] != T or p.gate.shape[1] < need or p.gate.stride(1) != 1:
                raise _lib.HydraHipError(f"rotary_parts: part {i}: gate must be [n_tokens, >= {need}] rows of the activations' dtype")
            q.gate, q.gate_stride, q.gate_kind = p.gate.data_ptr(), p.gate.stride(0), GATES[p.gate_kind]
        if p.cache is not None:
            c = p.cache
            chs = p.size if p.cache_head_stride is None else int(p.cache_head_stride)
            row = c.stride(1)
            if c.dtype != dtype or c.dim() != 4 or c.stride(3) != 1 or slot_ids is None or \
                    p.cache_col + (p.heads - 1) * chs + p.size > c.shape[2] * c.stride(2):
                raise _lib.HydraHipError(f"rotary_parts: part {i}: the cache plane must hold the part's columns in a row, with slot_ids")
            q.dst = c.data_ptr() + c.element_size() * int(p.cache_col)
            q.dst_stride, q.dst_head_stride, q.cache_block_stride, q.to_cache = row, chs, c.stride(0), 1
            block_size = c.shape[1]
            outs.append(None)
        else:
            d = p.dst if p.dst is not None else torch.empty((T, p.heads * p.size), dtype=dtype, device=s.device)
            if d.dtype != dtype or d.dim() != 2 or d.shape[0] != T or d.shape[1] < p.heads * p.size or d.stride(1) != 1:
                raise _lib.HydraHipError(f"rotary_parts: part {i}: dst must be [n_tokens, >= heads * size] rows")
            q.dst, q.dst_stride, q.dst_head_stride, q.cache_block_stride, q.to_cache = d.data_ptr(), d.stride(0), p.size, 0, 0
            outs.append(d)
    if slot_ids is not None and (slot_ids.dtype != torch.int32 or not slot_ids.is_contiguous() or slot_ids.numel() != T):
        raise _lib.HydraHipError("rotary_parts: slot_ids must be contiguous int32 [n_tokens]")
    a.positions, a.slot_ids = positions.data_ptr(), None if slot_ids is None else slot_ids.data_ptr()
    a.n_tokens, a.n_parts, a.block_size, a.dtype = T, len(parts), int(block_size), _code(dtype)
    _lib.mix_check(_lib.mix_lib().hxm_rotary_parts(ctypes.byref(a), _lib.current_stream()), "rotary_parts")
    return outs
