"""Row kernels of depth-averaged hybrids (csrc/depth_ops.hip, libhydra_mix.so): token + learned position embedding, the
one kernel for every place where a residual meets a norm (`depth_norm`), PolyNorm and squared ReLU.  The residual and the
stack of levels are float32; activations (what the matrix products read and write) are float32 or bfloat16."""
import ctypes
from typing import Optional

import torch
from torch import Tensor

from hydrainfer_amd import _lib


def _code(dtype: torch.dtype) -> int:
    if dtype not in (torch.float32, torch.bfloat16):
        raise _lib.HydraHipError(f"depth ops: activations are float32 or bfloat16, not {dtype}")
    return _lib._DTYPE[dtype]


def _f32(t: Optional[Tensor], name: str, n: Optional[int] = None) -> None:
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or (n is not None and t.numel() < n)):
        raise _lib.HydraHipError(f"{name} must be a contiguous float32 tensor" + (f" of at least {n} elements" if n else ""))


def _ptr(t: Optional[Tensor]):
    return None if t is None else t.data_ptr()


def embed_positions(ids: Tensor, positions: Optional[Tensor], table: Tensor, pos_table: Optional[Tensor],
                    out: Optional[Tensor] = None) -> Tensor:
    """out[t] = table[ids[t]] + pos_table[positions[t]] as float32 [n_tokens, width] (no position table: the first term)."""
    _lib.require_gpu(ids, positions, table, pos_table, out)
    if ids.dim() != 1 or ids.dtype not in (torch.int32, torch.int64) or not ids.is_contiguous():
        raise _lib.HydraHipError("embed_positions: ids must be a contiguous 1-D int32 / int64 tensor")
    if table.dim() != 2 or not table.is_contiguous():
        raise _lib.HydraHipError("embed_positions: table must be contiguous [vocab, width]")
    T, W = ids.shape[0], table.shape[1]
    if pos_table is not None:
        if pos_table.dtype != table.dtype or pos_table.dim() != 2 or pos_table.shape[1] != W or not pos_table.is_contiguous():
            raise _lib.HydraHipError("embed_positions: pos_table must be contiguous [n_positions, width] of the table's dtype")
        if positions is None or positions.dtype != torch.int32 or not positions.is_contiguous() or positions.numel() != T:
            raise _lib.HydraHipError("embed_positions: positions must be contiguous int32 [n_tokens]")
    if out is None:
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
    _f32(out, "out", T * W)
    _lib.mix_check(_lib.mix_lib().hxm_embed_positions(
        out.data_ptr(), table.data_ptr(), _ptr(pos_table), ids.data_ptr(), 1 if ids.dtype == torch.int64 else 0,
        _ptr(positions) if pos_table is not None else None, T, W, table.shape[0],
        pos_table.shape[0] if pos_table is not None else 0, _code(table.dtype), _lib.current_stream()), "embed_positions")
    return out


POST_NORMS = {None: 0, "same": 0, "layer": 1, "rms": 2, "plain": 3}


def depth_norm(x_in: Optional[Tensor], dtype: torch.dtype, eps: float, y: Optional[Tensor] = None, post_w: Optional[Tensor] = None,
               mult: float = 1.0, level_out: Optional[Tensor] = None, levels: Optional[Tensor] = None,
               depth_w: Optional[Tensor] = None, x_out: Optional[Tensor] = None, next_w: Optional[Tensor] = None,
               rows: Optional[Tensor] = None, rms: bool = False, post_norm: Optional[str] = None, y2: Optional[Tensor] = None,
               bias: Optional[Tensor] = None, cast_out: Optional[Tensor] = None) -> Optional[Tensor]:
    """For every output row i (input row r = rows[i], or i):
        x = x_in[r] (None: zeros);  with y: x += mult * N(y[r]) * post_w;  with y2: x += y2[r];  with bias: x += bias;
        with level_out: level_out[r] = x;  with depth_w [n]: x = sum_j depth_w[j] * levels[j, r];  with x_out: x_out[i] = x;
        with next_w: returns h[i] = norm(x) * next_w in `dtype`;  with cast_out (and no next_w): cast_out[i] = x in `dtype`.
    norm = layer norm without bias (rms=True: RMS norm), eps inside the root.  N = the same norm, or by post_norm "layer",
    "rms" or "plain" (y as it is; post_w may then be None).  x_in, level_out, x_out: float32 [n, width]; levels: float32
    [>= n_levels, n, width]; y, y2: `dtype` [n, >= width] with contiguous rows; cast_out: `dtype` [n, >= width] rows (a
    column range of a wider matrix will do)."""
    _lib.require_gpu(x_in, y, post_w, level_out, levels, depth_w, x_out, next_w, rows, y2, bias, cast_out)
    ref = x_in if x_in is not None else y
    if ref is None or ref.dim() != 2:
        raise _lib.HydraHipError("depth_norm: x_in (or y, when there is no x_in) must be [n_tokens, width]")
    T = ref.shape[0]
    W = x_in.shape[1] if x_in is not None else (post_w.numel() if post_w is not None else (bias.numel() if bias is not None else y.shape[1]))
    if post_norm not in POST_NORMS:
        raise _lib.HydraHipError(f"depth_norm: post_norm {post_norm!r}")
    _f32(x_in, "x_in"); _f32(post_w, "post_w", W); _f32(level_out, "level_out", T * W); _f32(levels, "levels")
    _f32(depth_w, "depth_w"); _f32(x_out, "x_out"); _f32(next_w, "next_w", W); _f32(bias, "bias", W)
    a = _lib.hxm_depth_norm_args()
    a.x_in = _ptr(x_in)
    a.y, a.y_stride, a.y2, a.y2_stride = None, 0, None, 0
    if y is not None:
        if y.dtype != dtype or y.dim() != 2 or y.shape[0] != T or y.shape[1] < W or y.stride(1) != 1 or \
                (post_w is None and POST_NORMS[post_norm] != 3):
            raise _lib.HydraHipError("depth_norm: y must be [n_tokens, >= width] of the activation dtype, with post_w")
        a.y, a.y_stride = y.data_ptr(), y.stride(0)
    if y2 is not None:
        if y2.dtype != dtype or y2.dim() != 2 or y2.shape[0] != T or y2.shape[1] < W or y2.stride(1) != 1:
            raise _lib.HydraHipError("depth_norm: y2 must be [n_tokens, >= width] of the activation dtype")
        a.y2, a.y2_stride = y2.data_ptr(), y2.stride(0)
    a.post_w, a.level_out, a.bias, a.post_norm = _ptr(post_w), _ptr(level_out), _ptr(bias), POST_NORMS[post_norm]
    a.levels, a.depth_w, a.n_levels, a.level_stride = None, None, 0, 0
    if depth_w is not None:
        n = depth_w.numel()
        if levels is None or levels.dim() != 3 or levels.shape[0] < n or levels.shape[1] != T or levels.shape[2] != W:
            raise _lib.HydraHipError("depth_norm: levels must be float32 [>= len(depth_w), n_tokens, width]")
        a.levels, a.depth_w, a.n_levels, a.level_stride = levels.data_ptr(), depth_w.data_ptr(), n, levels.stride(0)
    n_out = T
    a.rows = None
    if rows is not None:
        if rows.dtype != torch.int32 or not rows.is_contiguous():
            raise _lib.HydraHipError("depth_norm: rows must be contiguous int32")
        n_out, a.rows = rows.numel(), rows.data_ptr()
    if x_out is not None and x_out.numel() < n_out * W:
        raise _lib.HydraHipError("depth_norm: x_out too small")
    h = None
    if next_w is not None:
        h = torch.empty((n_out, W), dtype=dtype, device=ref.device)
    elif cast_out is not None:
        if cast_out.dtype != dtype or cast_out.dim() != 2 or cast_out.shape[0] < n_out or cast_out.shape[1] < W or cast_out.stride(1) != 1:
            raise _lib.HydraHipError("depth_norm: cast_out must be [>= n_out, >= width] of the activation dtype with contiguous rows")
        h = cast_out
    a.x_out, a.next_w, a.h_out, a.h_stride = _ptr(x_out), _ptr(next_w), _ptr(h), (h.stride(0) if h is not None else W)
    a.n_out, a.width, a.rms, a.dtype, a.mult, a.eps = n_out, W, 1 if rms else 0, _code(dtype), float(mult), float(eps)
    _lib.mix_check(_lib.mix_lib().hxm_depth_norm(ctypes.byref(a), _lib.current_stream()), "depth_norm")
    return h


def _rows2d(t: Tensor, name: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise _lib.HydraHipError(f"{name} must be 2-D with contiguous rows")


def poly_norm(z: Tensor, coef: Tensor, eps: float) -> Tensor:
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] per row, N(u) = u / sqrt(mean(u^2) + eps); coef: float32 [4]
    on the device."""
    _lib.require_gpu(z, coef)
    _rows2d(z, "poly_norm: z"); _f32(coef, "coef", 4)
    out = torch.empty((z.shape[0], z.shape[1]), dtype=z.dtype, device=z.device)
    _lib.mix_check(_lib.mix_lib().hxm_poly_norm(out.data_ptr(), out.stride(0), z.data_ptr(), z.stride(0), coef.data_ptr(),
                                                float(eps), z.shape[0], z.shape[1], _code(z.dtype), _lib.current_stream()),
                   "poly_norm")
    return out


def relu_squared(z: Tensor) -> Tensor:
    _lib.require_gpu(z)
    _rows2d(z, "relu_squared: z")
    out = torch.empty((z.shape[0], z.shape[1]), dtype=z.dtype, device=z.device)
    _lib.mix_check(_lib.mix_lib().hxm_relu_squared(out.data_ptr(), out.stride(0), z.data_ptr(), z.stride(0), z.shape[0],
                                                   z.shape[1], _code(z.dtype), _lib.current_stream()), "relu_squared")
    return out
