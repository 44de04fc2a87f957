"""A plain, slow restatement of the Fasanex design in float64 on the CPU, one function per mechanism, written from the
design's equations (it shares no code with hydrainfer_amd).  Weights are a dict under the checkpoint's tensor names; the
configuration is the dict config.json holds.  Whole sequences only: no cache, no state slots, no batching — what the
engine must reproduce however it cuts and batches the work."""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms_div(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x ** 2).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layer norms and the final norm: weights are stored as their distance from one."""
    return rms_div(x, eps) * (1.0 + w)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def short_conv(u: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [n, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j) (+ b), with zeros before the first token."""
    n, taps = u.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + n] * w[:, j]
    return y if b is None else y + b


# ---------------------------------------------------------------------------------------------- state-space mixer
def mamba2(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, P, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(n, H, P)
    B = xbc[:, inner:inner + G * N].reshape(n, G, N)
    C = xbc[:, inner + G * N:].reshape(n, G, N)
    dt = softplus(dt + W[p + "dt_bias"])                       # [n, H]
    a = torch.exp(-torch.exp(W[p + "A_log"]) * dt)             # [n, H]
    S = torch.zeros(H, N, P, dtype=F)
    y = torch.zeros(n, H, P, dtype=F)
    for t in range(n):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = a[t, hd] * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_div(y.reshape(n, parts, inner // parts), eps).reshape(n, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- attention side
def yarn_frequencies(rot: dict):
    """-> (frequency of every pair [dims / 2], the factor on cos and sin)."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    turn = lambda t: dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(turn(sc["fast"])), 0)
    hi = min(math.ceil(turn(sc["slow"])), dims - 1)
    ramp = torch.clamp((torch.arange(dims // 2, dtype=F) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [n, heads, dim]; the first rot.dims channels of every head turn, channel i with channel i + dims / 2."""
    dims = rot["dims"]
    f, m = yarn_frequencies(rot)
    ang = positions.to(F)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * m)[:, None, :], (torch.sin(ang) * m)[:, None, :]
    a, b = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def window_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, G, D = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = short_conv(h @ W[p + "q"].T, W[p + "q.conv"]).reshape(n, H, D)
    k = short_conv(h @ W[p + "k"].T, W[p + "k.conv"]).reshape(n, G, D)
    v = k                                                     # values: the keys before norm and rotation
    pos = torch.arange(n)
    q, k = rms_div(q, eps) * W[p + "q.norm"], rms_div(k, eps) * W[p + "k.norm"]
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    i, j = pos[:, None], pos[None, :]
    see = j <= i
    if m.get("mask"):
        see = see & (i - j < m["mask"]["size"])
    out = torch.zeros(n, H, v.shape[-1], dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if m.get("softcap"):
            s = m["softcap"] * torch.tanh(s / m["softcap"])
        s = s.masked_fill(~see, float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    out = out.reshape(n, -1) * torch.sigmoid(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- time mixing
def time_mix(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, D = h.shape[0], m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, h.shape[1], dtype=F), h[:-1]], dim=0)
    mix = lambda s: h + (prev - h) * W[p + "mu." + s]
    r = (mix("r") @ W[p + "r"].T).reshape(n, H, D)
    k = (mix("k") @ W[p + "k"].T).reshape(n, H, D)
    v = (mix("v") @ W[p + "v"].T).reshape(n, H, D)
    gate = silu(mix("g") @ W[p + "g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mix("w") @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).reshape(n, H, D)
    u = W[p + "u"]                                            # [H, D]
    S = torch.zeros(H, D, D, dtype=F)
    o = torch.zeros(n, H, D, dtype=F)
    for t in range(n):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[t])
        S = w[t][:, :, None] * S + kv
    o = rms_div(o, eps).reshape(n, H * D) * W[p + "norm"] * gate
    return o @ W[p + "o"].T


def parallel(h, W, p, m, eps):
    return m["left_scale"] * window_attention(h, W, p + "left.", m["left"], eps) + \
        m["right_scale"] * time_mix(h, W, p + "right.", m["right"], eps)


# ---------------------------------------------------------------------------------------------- delta rule
def delta(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, G, D, V = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(n, G, D)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(n, G, D)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(n, H, V)
    unit = lambda x: x / torch.sqrt((x ** 2).sum(dim=-1, keepdim=True) + 1e-6)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = torch.sigmoid(h @ W[p + "b"].T)                     # [n, H]
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    S = torch.zeros(H, D, V, dtype=F)
    o = torch.zeros(n, H, V, dtype=F)
    for t in range(n):
        for hd in range(H):
            kh, qh = k[t, hd // (H // G)], q[t, hd // (H // G)]
            S[hd] = g[t, hd] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ kh)
            S[hd] = S[hd] + torch.outer(kh, u)
            o[t, hd] = S[hd].T @ qh
    o = rms_div(o, eps) * W[p + "norm"]
    o = o.reshape(n, H * V) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forward, model
def dense_ff(h, W, p, mlp):
    lim = mlp.get("limit")
    g, u = h @ W[p + "gate"].T, h @ W[p + "up"].T
    if lim is not None:
        g, u = torch.clamp(g, max=lim), torch.clamp(u, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


MIXERS = {"mamba2": mamba2, "parallel": parallel, "delta": delta}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence; layers_out (a list) receives the residual after every layer."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[l["type"]](norm_one_plus(x, W[p + "norm1"], eps), W, p + "mix.", l["mixer"], eps)
        x = x + norm_one_plus(y, W[p + "norm1b"], eps)
        if l.get("mlp") is not None:
            y = dense_ff(norm_one_plus(x, W[p + "norm2"], eps), W, p + "mlp.", l["mlp"])
            x = x + norm_one_plus(y, W[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_one_plus(x, W["final.norm"], eps) @ W["head"].T


def greedy(cfg, weights, prompt: List[int], n_new: int):
    """(tokens generated greedily, top-1 margin of every step)."""
    toks, out, margins = list(prompt), [], []
    for _ in range(n_new):
        last = forward(cfg, weights, toks)[-1]
        top = torch.topk(last, 2).values
        out.append(int(torch.argmax(last)))
        margins.append(float(top[0] - top[1]))
        toks.append(out[-1])
    return out, margins
