"""A plain, slow restatement of the Pemalorn design in float64 on the CPU, one function per mechanism, written from the
design's equations (it shares no code with hydrainfer_amd).  Weights are a dict under the checkpoint's tensor names; the
configuration is the dict config.json holds.  Whole sequences only: no cache, no state slots, no batching, keys and values
of the latent attention materialised per head — what the engine must reproduce however it cuts and batches the work."""
import math
from typing import Dict, List, Optional, Tuple

import torch

F = torch.float64


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    d = x - x.mean(dim=-1, keepdim=True)
    return d / torch.sqrt((d ** 2).mean(dim=-1, keepdim=True) + eps) * w


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x ** 2).mean(dim=-1, keepdim=True) + eps) * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def input_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """h [n, C], w [C, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the first token."""
    n, taps = h.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, h.shape[1], dtype=h.dtype), h], dim=0)
    y = h.clone()
    for j in range(taps):
        y = y + pad[j:j + n] * w[:, j]
    return y


# ---------------------------------------------------------------------------------------------- rotations
def pair_frequencies(dims: int, base: float, scaling: Optional[dict] = None) -> Tuple[torch.Tensor, float]:
    """(angle per position of pair i < dims / 2, factor on cos and sin).  With a scaling block the slowly turning pairs are
    slowed down by `factor`, the fast ones kept, a linear ramp between; cos and sin grow by 0.1 ln(factor) + 1."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    where = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((torch.arange(dims // 2, dtype=F) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, layout: str, mag: float = 1.0) -> torch.Tensor:
    """x [n, ..., d] with d = 2 len(freq): every pair of channels turns by pos * freq[pair].  layout "halves": channel i
    with i + d / 2; "interleaved": 2 i with 2 i + 1.  pos [n] may be negative (turning back)."""
    d = 2 * freq.numel()
    assert x.shape[-1] == d
    ang = pos.to(F).reshape(-1, *([1] * (x.dim() - 1))) * freq
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    if layout == "halves":
        u, v = x[..., :d // 2], x[..., d // 2:]
        return torch.cat([u * c - v * s, v * c + u * s], dim=-1)
    assert layout == "interleaved"
    u, v = x[..., 0::2], x[..., 1::2]
    return torch.stack([u * c - v * s, v * c + u * s], dim=-1).reshape(x.shape)


# ---------------------------------------------------------------------------------------------- attention
def sink_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, head_scale: torch.Tensor, sink: torch.Tensor,
                           window: Optional[int]) -> torch.Tensor:
    """q [n, H, d], k [n, H, d], v [n, H, dv]; score_ij = q_i . k_j * head_scale[h] for the j that i sees (j <= i, and
    i - j < window when there is one); the softmax's denominator holds one more term exp(sink[h]) that carries no value."""
    n, H, _ = q.shape
    out = torch.zeros(n, H, v.shape[-1], dtype=F)
    for h in range(H):
        for i in range(n):
            lo = 0 if window is None else max(0, i - window + 1)
            s = (k[lo:i + 1, h] @ q[i, h]) * head_scale[h]
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, h]).sum(dim=0) / (e.sum() + torch.exp(sink[h] - m))
    return out


def attention_mixer(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    """Grouped-query attention: partial rotation (halves) of q and k, values turned by their own position over all their
    channels and the heads' sums turned back by the query's, a temperature and a sink per head, a sigmoid gate per head."""
    n, H, G, D, V = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    q = (h @ W[p + "q"].T).reshape(n, H, D)
    k = (h @ W[p + "k"].T).reshape(n, G, D)
    v = (h @ W[p + "v"].T).reshape(n, G, V)
    rot = m.get("rot")
    base = float(rot["base"]) if rot else 10000.0
    if rot and int(rot["dims"]) >= 2:
        r = int(rot["dims"])
        f, mag = pair_frequencies(r, base, rot.get("scaling"))
        q = torch.cat([rotate(q[..., :r], pos, f, "halves", mag), q[..., r:]], dim=-1)
        k = torch.cat([rotate(k[..., :r], pos, f, "halves", mag), k[..., r:]], dim=-1)
    fv, _ = pair_frequencies(V, base)
    v = rotate(v, pos, fv, "halves")
    rep = H // G
    k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    mask = m.get("mask") or {}
    o = sink_softmax_attention(q, k, v, float(m["scale"]) * W[p + "temp"], W[p + "sink"], mask.get("size"))
    o = rotate(o, -pos, fv, "halves")
    o = o * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(n, H * V) @ W[p + "o"].T


def latent_attention_mixer(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Attention through low-rank latents: queries from a normed latent; keys = [W_uk c | one rotated part shared by all
    heads], values = W_uv c, c the normed key/value latent; interleaved rotation with scaled frequencies; sliding window;
    a sink per head; an element-wise sigmoid gate."""
    n, H, D, R, V, C = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(n, H, D + R)
    dkv = h @ W[p + "dkv"].T
    c = rms_norm(dkv[:, :C], W[p + "dkv.norm"], eps)
    k_rot = dkv[:, C:C + R]
    rot = m.get("rot") or {}
    if R >= 2:
        f, mag = pair_frequencies(R, float(rot["base"]), rot.get("scaling"))
        q = torch.cat([q[..., :D], rotate(q[..., D:], pos, f, "interleaved", mag)], dim=-1)
        k_rot = rotate(k_rot, pos, f, "interleaved", mag)
    k = torch.cat([(c @ W[p + "uk"].T).reshape(n, H, D), k_rot[:, None, :].expand(n, H, R)], dim=-1)
    v = (c @ W[p + "uv"].T).reshape(n, H, V)
    mask = m.get("mask") or {}
    o = sink_softmax_attention(q, k, v, torch.full((H,), float(m["scale"]), dtype=F), W[p + "sink"], mask.get("size"))
    o = o.reshape(n, H * V) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forward
def route(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, r: dict) -> Tuple[torch.Tensor, torch.Tensor]:
    """(weights [n, top], experts [n, top]): softmax over every router output (identity experts included); the choice adds
    a correction to the scores, the weights are the chosen scores themselves."""
    s = torch.softmax(h @ W[p + "router"].T, dim=-1)
    choice = s + W[p + "correction"] if p + "correction" in W else s
    idx = torch.topk(choice, int(r["top"]), dim=-1).indices
    return torch.gather(s, 1, idx), idx


def expert_mixture(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    E = int(r["experts"])
    weights, idx = route(h, W, p, r)
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0] if E else h.shape[1], dtype=F)
    for t in range(h.shape[0]):
        for wk, e in zip(weights[t], idx[t].tolist()):
            if e >= E:                                    # an identity expert hands its input on
                out[t] += wk * h[t]
            else:
                x = p + f"e{e}."
                out[t] += wk * ((silu(h[t] @ W[x + "gate"].T) * (h[t] @ W[x + "up"].T)) @ W[x + "down"].T)
    return out


def token_side_input(x: torch.Tensor, tokens: torch.Tensor, W: Dict[str, torch.Tensor], p: str, layer: int, dim: int,
                     eps: float) -> torch.Tensor:
    """x + rms_norm(W_proj (gelu_tanh(W_gate x) * e)) with e the layer's part of the token's side embedding."""
    e = W["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ W[p + "side.gate"].T) * e) @ W[p + "side.proj"].T
    return x + rms_norm(y, W[p + "side.norm"], eps)


# ---------------------------------------------------------------------------------------------- the model
def run_order(cfg: dict) -> List[Tuple[int, int, bool]]:
    """(layer, pass number, first layer of a pass?) of every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    out = [(i, 0, False) for i in range(a)]
    for t in range(times):
        out += [(i, t, i == a) for i in range(a, b)]
    return out + [(i, 0, False) for i in range(b, n)]


def layer(x: torch.Tensor, tokens: torch.Tensor, W: Dict[str, torch.Tensor], cfg: dict, i: int) -> torch.Tensor:
    l, p, eps = cfg["layers"][i], f"l{i}.", float(cfg["norm"]["eps"])
    h = layer_norm(x, W[p + "norm1"], eps)
    hm = input_conv(h, W[p + "canon1"]) if p + "canon1" in W else h
    if l["type"] == "attention":
        y = attention_mixer(hm, W, p + "mix.", l["mixer"])
    elif l["type"] == "latent_attention":
        y = latent_attention_mixer(hm, W, p + "mix.", l["mixer"], eps)
    else:
        raise ValueError(l["type"])
    if l.get("mlp") is not None:
        hf = input_conv(h, W[p + "canon2"]) if p + "canon2" in W else h
        y = y + expert_mixture(hf, W, p + "mlp.", l["mlp"])
    x = x + y
    if cfg.get("token_side") and p + "side.gate" in W:
        x = token_side_input(x, tokens, W, p, i, int(cfg["token_side"]["dim"]), eps)
    return x


def forward(tokens: List[int], W: Dict[str, torch.Tensor], cfg: dict, trace: Optional[list] = None) -> torch.Tensor:
    """float64 logits [n, vocab] of a whole sequence; `trace` (a list) receives the residual after every layer run."""
    W = {k: (v.to(F) if v.is_floating_point() else v) for k, v in W.items()}
    tok = torch.tensor(tokens, dtype=torch.long)
    x0 = W["embed"][tok]
    x = x0
    for i, t, first in run_order(cfg):
        if first:
            x = torch.cat([x, x0], dim=-1) @ W["loop.in"].T + W["loop.step"][t]
        x = layer(x, tok, W, cfg, i)
        if trace is not None:
            trace.append(x.clone())
    return layer_norm(x, W["final.norm"], float(cfg["norm"]["eps"])) @ W["head"].T


def greedy(tokens: List[int], W: Dict[str, torch.Tensor], cfg: dict, n_new: int) -> Tuple[List[int], List[float]]:
    """n_new greedy tokens after the prompt, and the margin of each over the runner-up (a small one: a near-tie)."""
    toks, out, margins = list(tokens), [], []
    for _ in range(n_new):
        top = torch.topk(forward(toks, W, cfg)[-1], 2)
        out.append(int(top.indices[0]))
        margins.append(float(top.values[0] - top.values[1]))
        toks.append(out[-1])
    return out, margins
