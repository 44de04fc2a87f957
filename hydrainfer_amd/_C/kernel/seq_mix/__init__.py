"""Mixers that keep per-sequence state beside the paged cache (csrc/seq_ops.hip, csrc/state_scan.hip, libhydra_mix.so):
short causal convolutions, token shift with several mixes, per-head RMS norm + rotary positions + cache append, the
decays / step sizes / write strengths of a recurrence, the scan over a matrix state per head (decayed sum, read before
write with a bonus, delta rule), the gate / group norm that finishes a mixer, and the clamped gated feed-forward
activation.

A sequence's state is a flat run of floats in its slot of memory.state_slots.StateSlotManager (`seq.state`
[n_slots, rows, width], contiguous); every mixer owns a piece of it, named here by `offset` (floats from the slot's
start).  A portion that starts at position 0 starts from zeros without reading its slot."""
import ctypes
from typing import Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib
from hydrainfer_amd._C.kernel.stream_ops import SequenceState

ACT = {None: 0, "none": 0, "silu": 1, "sigmoid": 2, "tanh": 3}
SCAN_MODES = {"decay": 0, "bonus": 1, "delta": 2}


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"sequence mixers: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


def _ptr(t: Optional[Tensor]):
    return None if t is None else t.data_ptr()


def _rows(t: Tensor, n: int, name: str, rows: Optional[int] = None, dtype: Optional[torch.dtype] = None) -> None:
    if t.dim() != 2 or t.shape[1] != n or t.stride(1) != 1 or (rows is not None and t.shape[0] != rows) or \
            (dtype is not None and t.dtype != dtype):
        raise _lib.HydraHipError(f"{name} must be [{'n' if rows is None else rows}, {n}] with contiguous rows"
                                 + (f" of {dtype}" if dtype is not None else ""))


def _f32(t: Optional[Tensor], n: int, name: str) -> None:
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n):
        raise _lib.HydraHipError(f"{name} must be contiguous float32 [{n}]")


def _i32(t: Tensor, n: int, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() != n:
        raise _lib.HydraHipError(f"{name} must be contiguous int32 [{n}]")


def _piece(seq: SequenceState, offset: int, size: int, what: str):
    """(pointer to the piece in slot 0, floats from one slot to the next)."""
    st = seq.state
    if st.dtype != torch.float32 or st.dim() != 3 or not st.is_contiguous():
        raise _lib.HydraHipError(f"{what}: state must be contiguous float32 [n_slots, rows, width]")
    if offset < 0 or offset + size > st.shape[1] * st.shape[2]:
        raise _lib.HydraHipError(f"{what}: the piece [{offset}, {offset + size}) lies outside a slot of {st.shape[1] * st.shape[2]} floats")
    return st.data_ptr() + 4 * offset, st.stride(0)


def _batch(seq: SequenceState, q_cu: Tensor, positions: Tensor, T: int, what: str) -> int:
    n_seq = q_cu.numel() - 1
    _i32(q_cu, n_seq + 1, f"{what}: q_cu"); _i32(positions, T, f"{what}: positions"); _i32(seq.slots, n_seq, f"{what}: slots")
    _i32(seq.tok_seq, T, f"{what}: tok_seq")
    _lib.require_gpu(seq.state, seq.slots, seq.tok_seq, q_cu, positions)
    return n_seq


def causal_conv(u: Tensor, w: Tensor, bias: Optional[Tensor], act: Optional[str], seq: SequenceState, offset: int,
                q_cu: Tensor, positions: Tensor) -> Tensor:
    """y[t, c] = act(sum_j w[c, j] u[t - taps + 1 + j, c] + bias[c]) within each sequence.  u: [n_tokens, channels] (a view
    of a projection's columns will do); w: float32 [channels, taps]; the slot's piece: (taps - 1) * channels floats."""
    _lib.require_gpu(u, w, bias)
    if u.dim() != 2 or u.stride(1) != 1:
        raise _lib.HydraHipError("causal_conv: u must be 2-D with contiguous rows")
    T, C = u.shape
    if w.dim() != 2 or w.shape[0] != C:
        raise _lib.HydraHipError("causal_conv: w must be [channels, taps]")
    taps = w.shape[1]
    _f32(w, C * taps, "causal_conv: w"); _f32(bias, C, "causal_conv: bias")
    n_seq = _batch(seq, q_cu, positions, T, "causal_conv")
    base, stride = _piece(seq, offset, max(taps - 1, 1) * C, "causal_conv")
    y = torch.empty((T, C), dtype=u.dtype, device=u.device)
    _lib.mix_check(_lib.mix_lib().hxm_causal_conv(
        y.data_ptr(), y.stride(0), u.data_ptr(), u.stride(0), w.data_ptr(), _ptr(bias), ACT[act], base, stride,
        seq.slots.data_ptr(), seq.tok_seq.data_ptr(), q_cu.data_ptr(), positions.data_ptr(), T, n_seq, C, taps, _code(u.dtype),
        _lib.current_stream()), "causal_conv")
    return y


def causal_conv_pair(u: Tensor, w: Tensor, w2: Optional[Tensor], seq: SequenceState, offset: int, q_cu: Tensor, positions: Tensor,
                     bias: Optional[Tensor] = None, bias2: Optional[Tensor] = None, act: Optional[str] = None,
                     skip: bool = True):
    """Two short causal convolutions of the same input in one pass: y = act(conv_w(u) + bias) + u, y2 = act(conv_w2(u) +
    bias2) + u (skip=False: without the + u).  The inputs are read once and the slot's piece ((taps - 1) * channels floats,
    the inputs of the last positions) is brought up to date once.  w2 None: only y.  Returns (y, y2 or None)."""
    _lib.require_gpu(u, w, w2, bias, bias2)
    if u.dim() != 2 or u.stride(1) != 1:
        raise _lib.HydraHipError("causal_conv_pair: u must be 2-D with contiguous rows")
    T, C = u.shape
    if w.dim() != 2 or w.shape[0] != C or (w2 is not None and w2.shape != w.shape):
        raise _lib.HydraHipError("causal_conv_pair: w and w2 must be [channels, taps]")
    taps = w.shape[1]
    _f32(w, C * taps, "causal_conv_pair: w"); _f32(w2, C * taps, "causal_conv_pair: w2")
    _f32(bias, C, "causal_conv_pair: bias"); _f32(bias2, C, "causal_conv_pair: bias2")
    n_seq = _batch(seq, q_cu, positions, T, "causal_conv_pair")
    base, stride = _piece(seq, offset, max(taps - 1, 1) * C, "causal_conv_pair")
    y = torch.empty((T, C), dtype=u.dtype, device=u.device)
    y2 = torch.empty((T, C), dtype=u.dtype, device=u.device) if w2 is not None else None
    _lib.mix_check(_lib.mix_lib().hxm_causal_conv_pair(
        y.data_ptr(), y.stride(0), _ptr(y2), C if y2 is not None else 0, u.data_ptr(), u.stride(0), w.data_ptr(), _ptr(w2),
        _ptr(bias), _ptr(bias2), ACT[act], 1 if skip else 0, base, stride, seq.slots.data_ptr(), seq.tok_seq.data_ptr(),
        q_cu.data_ptr(), positions.data_ptr(), T, n_seq, C, taps, _code(u.dtype), _lib.current_stream()), "causal_conv_pair")
    return y, y2


def token_shift_mix(h: Tensor, mu: Tensor, seq: SequenceState, offset: int, q_cu: Tensor, positions: Tensor) -> Tensor:
    """out[m] = h + (h_prev - h) * mu[m], h_prev the row of the token before in the same sequence (zeros before position 0).
    h: [n_tokens, width]; mu: float32 [n_mix, width]; the slot's piece: width floats.  Returns [n_mix, n_tokens, width]."""
    _lib.require_gpu(h, mu)
    if h.dim() != 2 or h.stride(1) != 1:
        raise _lib.HydraHipError("token_shift_mix: h must be 2-D with contiguous rows")
    T, W = h.shape
    if mu.dim() != 2 or mu.shape[1] != W:
        raise _lib.HydraHipError("token_shift_mix: mu must be [n_mix, width]")
    _f32(mu, mu.numel(), "token_shift_mix: mu")
    n_seq = _batch(seq, q_cu, positions, T, "token_shift_mix")
    base, stride = _piece(seq, offset, W, "token_shift_mix")
    out = torch.empty((mu.shape[0], T, W), dtype=h.dtype, device=h.device)
    _lib.mix_check(_lib.mix_lib().hxm_token_shift_mix(
        out.data_ptr(), h.data_ptr(), h.stride(0), mu.data_ptr(), mu.shape[0], base, stride, seq.slots.data_ptr(),
        seq.tok_seq.data_ptr(), q_cu.data_ptr(), positions.data_ptr(), T, n_seq, W, _code(h.dtype), _lib.current_stream()),
        "token_shift_mix")
    return out


def clamped_glu(gate: Tensor, up: Tensor, limit: float, alpha: float = 1.702, up_shift: float = 1.0) -> Tensor:
    """g sigmoid(alpha g) (u + up_shift) with g = min(gate, limit), u = clamp(up, -limit, limit); limit <= 0: no clamp."""
    _lib.require_gpu(gate, up)
    if gate.dim() != 2 or gate.shape != up.shape or gate.stride(1) != 1 or up.stride(1) != 1 or gate.dtype != up.dtype:
        raise _lib.HydraHipError("clamped_glu: gate / up must be 2-D, one shape and dtype, contiguous rows")
    y = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    _lib.mix_check(_lib.mix_lib().hxm_clamped_glu(
        y.data_ptr(), y.stride(0), gate.data_ptr(), gate.stride(0), up.data_ptr(), up.stride(0), float(limit), float(alpha),
        float(up_shift), gate.shape[0], gate.shape[1], _code(gate.dtype), _lib.current_stream()), "clamped_glu")
    return y


def unary(x: Tensor, act: str) -> Tensor:
    _lib.require_gpu(x)
    if x.dim() != 2 or x.stride(1) != 1:
        raise _lib.HydraHipError("unary: x must be 2-D with contiguous rows")
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _lib.mix_check(_lib.mix_lib().hxm_unary(out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), ACT[act], x.shape[0],
                                            x.shape[1], _code(x.dtype), _lib.current_stream()), "unary")
    return out


def head_gates(a: Tensor, log_rate: Tensor, step_bias: Tensor, b: Optional[Tensor] = None, want_step: bool = False):
    """Per token and head, float32: step = softplus(a + step_bias), decay = exp(-exp(log_rate) * step), beta = sigmoid(b).
    a, b: [n_tokens, heads] (views will do).  Returns (decay, step or None, beta or None)."""
    _lib.require_gpu(a, b, log_rate, step_bias)
    if a.dim() != 2 or a.stride(1) != 1 or (b is not None and (b.shape != a.shape or b.stride(1) != 1 or b.dtype != a.dtype)):
        raise _lib.HydraHipError("head_gates: a (and b) must be [n_tokens, heads] with contiguous rows, one dtype")
    T, H = a.shape
    _f32(log_rate, H, "head_gates: log_rate"); _f32(step_bias, H, "head_gates: step_bias")
    f = dict(dtype=torch.float32, device=a.device)
    decay = torch.empty((T, H), **f)
    step = torch.empty((T, H), **f) if want_step else None
    beta = torch.empty((T, H), **f) if b is not None else None
    _lib.mix_check(_lib.mix_lib().hxm_head_gates(
        decay.data_ptr(), _ptr(step), _ptr(beta), a.data_ptr(), a.stride(0), _ptr(b), b.stride(0) if b is not None else 0,
        log_rate.data_ptr(), step_bias.data_ptr(), T, H, _code(a.dtype), _lib.current_stream()), "head_gates")
    return decay, step, beta


def decay_exp(x: Tensor, bias: Optional[Tensor]) -> Tensor:
    """exp(-exp(x + bias)) in float32."""
    _lib.require_gpu(x, bias)
    if x.dim() != 2 or x.stride(1) != 1:
        raise _lib.HydraHipError("decay_exp: x must be 2-D with contiguous rows")
    _f32(bias, x.shape[1], "decay_exp: bias")
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _lib.mix_check(_lib.mix_lib().hxm_decay_exp(out.data_ptr(), x.data_ptr(), x.stride(0), _ptr(bias), x.shape[0], x.shape[1],
                                                _code(x.dtype), _lib.current_stream()), "decay_exp")
    return out


def unit_norm(x: Tensor, heads: int, dim: int, eps: float, scale: float = 1.0) -> Tensor:
    """Every head's vector divided by sqrt(sum of squares + eps), times scale; float32 [n_tokens, heads * dim]."""
    _lib.require_gpu(x)
    _rows(x, heads * dim, "unit_norm: x")
    out = torch.empty((x.shape[0], heads * dim), dtype=torch.float32, device=x.device)
    _lib.mix_check(_lib.mix_lib().hxm_unit_norm(out.data_ptr(), x.data_ptr(), x.stride(0), float(eps), float(scale), x.shape[0],
                                                int(heads), int(dim), _code(x.dtype), _lib.current_stream()), "unit_norm")
    return out


def head_norm_rope_cache(q: Tensor, k: Tensor, q_w: Tensor, k_w: Tensor, eps: float, q_heads: int, kv_heads: int, dim: int,
                         inv_freq: Optional[Tensor], cos_sin_scale: float, positions: Tensor, slot_ids: Tensor,
                         key_cache: Tensor, value_cache: Tensor) -> Tensor:
    """Per-head RMS norm of q and k (weights [dim], shared by the heads), rotation of the first 2 * len(inv_freq) channels
    of every head (channel i with channel i + len(inv_freq); angle = position * inv_freq[i], cos and sin times
    cos_sin_scale), the turned keys to key_cache and the keys as they came to value_cache (rows slot_ids).
    Returns q [n_tokens, q_heads * dim]."""
    _lib.require_gpu(q, k, q_w, k_w, inv_freq, positions, slot_ids, key_cache, value_cache)
    _rows(q, q_heads * dim, "head_norm_rope_cache: q")
    T = q.shape[0]
    _rows(k, kv_heads * dim, "head_norm_rope_cache: k", T, q.dtype)
    _f32(q_w, dim, "head_norm_rope_cache: q_w"); _f32(k_w, dim, "head_norm_rope_cache: k_w")
    _i32(positions, T, "head_norm_rope_cache: positions"); _i32(slot_ids, T, "head_norm_rope_cache: slot_ids")
    rot = 0 if inv_freq is None else 2 * inv_freq.numel()
    _f32(inv_freq, rot // 2, "head_norm_rope_cache: inv_freq")
    if rot > dim:
        raise _lib.HydraHipError("head_norm_rope_cache: more rotary channels than a head has")
    for c in (key_cache, value_cache):
        if c.dim() != 4 or c.dtype != q.dtype or c.shape[2] < kv_heads or c.shape[3] < dim or c.stride(3) != 1 or \
                c.stride(0) != c.stride(1) * c.shape[1] or c.stride() != key_cache.stride():
            raise _lib.HydraHipError("head_norm_rope_cache: cache planes [n_blocks, block_size, >= kv_heads, >= dim] of q's dtype, "
                                     "one layout, a block's rows following each other")
    out = torch.empty((T, q_heads * dim), dtype=q.dtype, device=q.device)
    a = _lib.hxm_head_rope_args()
    a.q_out, a.q, a.k, a.q_stride, a.k_stride = out.data_ptr(), q.data_ptr(), k.data_ptr(), q.stride(0), k.stride(0)
    a.q_w, a.k_w, a.inv_freq = q_w.data_ptr(), k_w.data_ptr(), _ptr(inv_freq)
    a.positions, a.slot_ids = positions.data_ptr(), slot_ids.data_ptr()
    a.key_cache, a.value_cache = key_cache.data_ptr(), value_cache.data_ptr()
    a.cache_row_stride, a.head_stride = key_cache.stride(1), key_cache.stride(2)
    a.n_tokens, a.q_heads, a.kv_heads, a.dim, a.rot_dims = T, int(q_heads), int(kv_heads), int(dim), rot
    a.eps, a.cos_sin_scale, a.dtype = float(eps), float(cos_sin_scale), _code(q.dtype)
    _lib.mix_check(_lib.mix_lib().hxm_head_norm_rope_cache(ctypes.byref(a), _lib.current_stream()), "head_norm_rope_cache")
    return out


def state_scan(mode: str, q: Tensor, k: Tensor, v: Tensor, decay: Tensor, seq: SequenceState, offset: int, q_cu: Tensor,
               positions: Tensor, heads: int, qk_heads: int, dim: int, vdim: int, vscale: Optional[Tensor] = None,
               beta: Optional[Tensor] = None, bonus: Optional[Tensor] = None) -> Tensor:
    """The recurrence of a matrix state S [dim, vdim] per head, token by token in float32, continued from and left in the
    slot's piece of heads * dim * vdim floats:
        "decay": S <- a S + k (s v)^T, o = S^T q;   "bonus": o = (S + diag(u) k v^T)^T q, then S <- a S + k v^T;
        "delta": S <- a S, S <- S + k (b (v - S^T k))^T, o = S^T q.
    q, k: [n_tokens, qk_heads * dim], v: [n_tokens, heads * vdim] (float32 or bfloat16, each its own; views will do);
    decay a: float32 [n_tokens, heads] or [n_tokens, heads * dim] (one per key channel); vscale s, beta b: float32
    [n_tokens, heads]; bonus u: float32 [heads * dim].  Returns o: float32 [n_tokens, heads * vdim]."""
    _lib.require_gpu(q, k, v, decay, vscale, beta, bonus)
    _rows(q, qk_heads * dim, "state_scan: q")
    T = q.shape[0]
    _rows(k, qk_heads * dim, "state_scan: k", T); _rows(v, heads * vdim, "state_scan: v", T)
    per_channel = decay.dim() == 2 and decay.shape[1] == heads * dim and dim > 1
    _f32(decay, T * heads * (dim if per_channel else 1), "state_scan: decay")
    _f32(vscale, T * heads, "state_scan: vscale"); _f32(beta, T * heads, "state_scan: beta"); _f32(bonus, heads * dim, "state_scan: bonus")
    if mode not in SCAN_MODES or (mode == "delta" and beta is None) or (mode == "bonus" and bonus is None):
        raise _lib.HydraHipError(f"state_scan: mode {mode!r} (delta needs beta, bonus needs bonus)")
    n_seq = _batch(seq, q_cu, positions, T, "state_scan")
    base, stride = _piece(seq, offset, heads * dim * vdim, "state_scan")
    out = torch.empty((T, heads * vdim), dtype=torch.float32, device=q.device)
    a = _lib.hxm_state_scan_args()
    a.out, a.q, a.k, a.v = out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr()
    a.q_stride, a.k_stride, a.v_stride = q.stride(0), k.stride(0), v.stride(0)
    a.q_dtype, a.k_dtype, a.v_dtype = _code(q.dtype), _code(k.dtype), _code(v.dtype)
    a.decay_per_channel, a.decay, a.vscale, a.beta, a.bonus = int(per_channel), decay.data_ptr(), _ptr(vscale), _ptr(beta), _ptr(bonus)
    a.state, a.slot_stride, a.slots, a.q_cu, a.positions = base, stride, seq.slots.data_ptr(), q_cu.data_ptr(), positions.data_ptr()
    a.n_tokens, a.n_seq, a.heads, a.qk_heads, a.dim, a.vdim, a.mode = T, n_seq, int(heads), int(qk_heads), int(dim), int(vdim), SCAN_MODES[mode]
    _lib.mix_check(_lib.mix_lib().hxm_state_scan(ctypes.byref(a), _lib.current_stream()), "state_scan")
    return out


def gated_group_norm(x: Tensor, dtype: torch.dtype, group: int = 0, eps: float = 0.0, w: Optional[Tensor] = None,
                     gate: Optional[Tensor] = None, gate_act: str = "silu", gate_first: bool = False,
                     skip: Optional[Tensor] = None, skip_w: Optional[Tensor] = None, skip_group: int = 1, scale: float = 1.0,
                     out: Optional[Tensor] = None) -> Tensor:
    """out = scale * [act(gate)] * w[c % len(w)] * N(x + skip_w[c // skip_group] * skip [* act(gate) if gate_first]) per row,
    N dividing every `group` consecutive elements by their root mean square (eps inside the root; group 0: no norm).
    x: float32 or `dtype` [rows, n]; gate, skip: `dtype` rows; out: `dtype` [rows, n] (a view of a wider buffer will do)."""
    _lib.require_gpu(x, w, gate, skip, skip_w, out)
    if x.dim() != 2 or x.stride(1) != 1 or x.dtype not in (torch.float32, dtype):
        raise _lib.HydraHipError("gated_group_norm: x must be 2-D float32 or of the activation dtype, contiguous rows")
    R, n = x.shape
    for t, name in ((gate, "gate"), (skip, "skip")):
        if t is not None:
            _rows(t, n, f"gated_group_norm: {name}", R, dtype)
    if w is not None:
        _f32(w, w.numel(), "gated_group_norm: w")
    if skip is not None:
        _f32(skip_w, (n + skip_group - 1) // skip_group, "gated_group_norm: skip_w")
    if out is None:
        out = torch.empty((R, n), dtype=dtype, device=x.device)
    _rows(out, n, "gated_group_norm: out", R, dtype)
    a = _lib.hxm_group_norm_args()
    a.out, a.out_stride, a.x, a.x_stride, a.x_dtype = out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), _code(x.dtype)
    a.skip, a.skip_stride, a.skip_w, a.skip_group = _ptr(skip), skip.stride(0) if skip is not None else 0, _ptr(skip_w), int(skip_group)
    a.gate, a.gate_stride, a.gate_act, a.gate_first = _ptr(gate), gate.stride(0) if gate is not None else 0, ACT[gate_act], int(gate_first)
    a.group, a.eps, a.w, a.w_len, a.scale = int(group), float(eps), _ptr(w), w.numel() if w is not None else 0, float(scale)
    a.rows, a.n, a.dtype = R, n, _code(dtype)
    _lib.mix_check(_lib.mix_lib().hxm_gated_group_norm(ctypes.byref(a), _lib.current_stream()), "gated_group_norm")
    return out
