"""Mixture of experts on the mix library (csrc/moe_mix.hip): softmax router with a choice bias, expert-major plan, grouped
products over the rows of every expert, weighted combine with an optional gated shared expert.  No step returns to the
host: buffers are sized for n_tokens * top rows and the kernels find the experts' segments on the device."""
from typing import Optional, Tuple

import torch
from torch import Tensor

from hydrainfer_amd import _lib


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"moe: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


def route_softmax_topk(logits: Tensor, n_experts: int, top: int, scale: float,
                       choice_bias: Optional[Tensor] = None, renorm: bool = True) -> Tuple[Tensor, Tensor]:
    """logits: float32 [n_tokens, >= n_experts] (contiguous rows).  s = softmax(logits[:, :n_experts]); the `top` largest of
    s + choice_bias are chosen (ties: the lower expert); weights = chosen s / (their sum + 1e-20) * scale, or with
    renorm=False the chosen scores themselves, s * scale.
    Returns (weights float32 [n_tokens, top], experts int32 [n_tokens, top])."""
    _lib.require_gpu(logits, choice_bias)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or logits.shape[1] < n_experts:
        raise _lib.HydraHipError("route_softmax_topk: logits must be float32 [n_tokens, >= n_experts] with contiguous rows")
    if choice_bias is not None and (choice_bias.dtype != torch.float32 or not choice_bias.is_contiguous()
                                    or choice_bias.numel() != n_experts):
        raise _lib.HydraHipError("route_softmax_topk: choice_bias must be contiguous float32 [n_experts]")
    T = logits.shape[0]
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    experts = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    _lib.mix_check(_lib.mix_lib().hxm_route_softmax_topk(
        logits.data_ptr(), logits.stride(0), None if choice_bias is None else choice_bias.data_ptr(), T, int(n_experts),
        int(top), float(scale), 1 if renorm else 0, weights.data_ptr(), experts.data_ptr(), _lib.current_stream()),
        "route_softmax_topk")
    return weights, experts


def moe_plan(experts: Tensor, n_experts: int) -> Tuple[Tensor, Tensor, Tensor]:
    """experts: int32 [n_tokens, top].  Returns (seg int32 [n_experts + 1], row_of int32 [n_tokens, top], src int32
    [n_tokens * top]): rows seg[e] .. seg[e + 1] of the expert-major order belong to expert e, pair (t, k) is row
    row_of[t, k], and row r comes from token src[r]."""
    _lib.require_gpu(experts)
    if experts.dtype != torch.int32 or experts.dim() != 2 or not experts.is_contiguous():
        raise _lib.HydraHipError("moe_plan: experts must be contiguous int32 [n_tokens, top]")
    T, top = experts.shape
    seg = torch.empty(n_experts + 1, dtype=torch.int32, device=experts.device)
    row_of = torch.empty((T, top), dtype=torch.int32, device=experts.device)
    src = torch.empty(T * top, dtype=torch.int32, device=experts.device)
    _lib.mix_check(_lib.mix_lib().hxm_moe_plan(experts.data_ptr(), T, top, int(n_experts), seg.data_ptr(), row_of.data_ptr(),
                                               src.data_ptr(), _lib.current_stream()), "moe_plan")
    return seg, row_of, src


def grouped_linear(x: Tensor, w: Tensor, seg: Tensor, max_rows: int, src: Optional[Tensor] = None, act: str = "none") -> Tensor:
    """y[r] = act(x[src[r] (or r)] @ w[e].T) for the rows r of every expert e.  x: [n, k] (contiguous rows); w: [n_experts,
    n_out, k] contiguous; returns [max_rows, n_out] (rows beyond seg[-1] are not written).  act: "none" | "relu2"."""
    _lib.require_gpu(x, w, seg, src)
    if x.dim() != 2 or x.stride(1) != 1 or w.dim() != 3 or not w.is_contiguous() or w.dtype != x.dtype or w.shape[2] != x.shape[1]:
        raise _lib.HydraHipError("grouped_linear: x [n, k] with contiguous rows, w [n_experts, n_out, k] contiguous, one dtype")
    E, N, K = w.shape
    if seg.dtype != torch.int32 or not seg.is_contiguous() or seg.numel() != E + 1:
        raise _lib.HydraHipError("grouped_linear: seg must be contiguous int32 [n_experts + 1]")
    if src is not None and (src.dtype != torch.int32 or not src.is_contiguous() or src.numel() < max_rows):
        raise _lib.HydraHipError("grouped_linear: src must be contiguous int32 [>= max_rows]")
    if src is None and x.shape[0] < max_rows:
        raise _lib.HydraHipError("grouped_linear: x has fewer rows than max_rows")
    y = torch.empty((max_rows, N), dtype=x.dtype, device=x.device)
    _lib.mix_check(_lib.mix_lib().hxm_grouped_linear(
        y.data_ptr(), x.data_ptr(), x.stride(0), None if src is None else src.data_ptr(), w.data_ptr(), seg.data_ptr(),
        int(max_rows), E, N, K, {"none": 0, "relu2": 1}[act], _code(x.dtype), _lib.current_stream()), "grouped_linear")
    return y


def moe_combine(y: Tensor, row_of: Tensor, weights: Tensor, shared: Optional[Tensor] = None,
                shared_gate: Optional[Tensor] = None, identity: Optional[Tensor] = None) -> Tensor:
    """out[t] = sum_k weights[t, k] * y[row_of[t, k]] + sigmoid(shared_gate[t]) * shared[t].  shared_gate: float32, one
    number per token (any row stride: a column of a wider matrix will do).  identity [n_tokens, width] (the experts' input):
    a choice without a row (row_of < 0: an expert beyond those moe_plan was called with) is an identity expert and adds
    weights[t, k] * identity[t]; without it such a choice adds nothing."""
    _lib.require_gpu(y, row_of, weights, shared, shared_gate, identity)
    T, top = row_of.shape
    W = y.shape[1]
    if y.dim() != 2 or not y.is_contiguous() or weights.dtype != torch.float32 or not weights.is_contiguous() or \
            weights.shape != row_of.shape or row_of.dtype != torch.int32 or not row_of.is_contiguous():
        raise _lib.HydraHipError("moe_combine: y contiguous [rows, width], row_of int32 / weights float32 [n_tokens, top]")
    gate_stride = 0
    if shared is not None:
        if shared.shape != (T, W) or shared.dtype != y.dtype or not shared.is_contiguous() or shared_gate is None or \
                shared_gate.dtype != torch.float32 or shared_gate.shape[0] != T:
            raise _lib.HydraHipError("moe_combine: shared [n_tokens, width] of y's dtype with a float32 gate per token")
        gate_stride = shared_gate.stride(0)
    if identity is not None and (identity.dtype != y.dtype or identity.dim() != 2 or identity.shape[0] != T or
                                 identity.shape[1] < W or identity.stride(1) != 1):
        raise _lib.HydraHipError("moe_combine: identity must be [n_tokens, >= width] of y's dtype with contiguous rows")
    out = torch.empty((T, W), dtype=y.dtype, device=y.device)
    _lib.mix_check(_lib.mix_lib().hxm_moe_combine(
        out.data_ptr(), y.data_ptr(), row_of.data_ptr(), weights.data_ptr(), None if shared is None else shared.data_ptr(),
        None if shared is None else shared_gate.data_ptr(), gate_stride, None if identity is None else identity.data_ptr(),
        0 if identity is None else identity.stride(0), T, top, W, _code(y.dtype), _lib.current_stream()), "moe_combine")
    return out
