"""Fasanex — a decoder-only hybrid whose layers pick one of three sequence mixers, every sublayer between two RMS norms:

  * x = embed[token] * embedding scale; a layer is x <- x + norm_1b(mixer(norm_1(x))), then (if it has a feed-forward)
    x <- x + norm_2b(ff(norm_2(x))); every such norm is x / rms(x) * (1 + w), the weight stored as its distance from one;
  * mixer `mamba2`: one projection -> [z | x | B | C | dt]; a short causal convolution with bias and silu over x, B, C;
    dt = softplus(dt + bias); per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x (heads share B / C in groups);
    y * silu(z), RMS norm in equal parts, times a weight, then the output projection;
  * mixer `parallel`: two mixers read the same input and their results are added with a weight each.  Left: grouped-query
    attention whose values ARE the keys (as they leave the convolution): a short causal convolution on q and k, per-head
    RMS norm with a weight, rotary positions with YaRN-scaled frequencies on the first channels of every head, score
    = cap * tanh(q . k * scale / cap) under a sliding window, softmax, a sigmoid output gate.  Right: time mixing — r, k,
    v, g, w each read their own blend of the token's input and the previous token's; decay w = exp(-exp(low-rank(w mix)
    + w0)) per key channel; o = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T; per-head RMS, a weight, silu gate;
  * mixer `delta`: the gated delta rule — short causal convolution + silu on q, k, v; q, k unit vectors per head (q also
    times dim^-1/2); beta = sigmoid(.), g = exp(-exp(A_log) softplus(. + bias)) per head; S <- g S, S <- S + k (beta (v -
    S^T k))^T, o = S^T q; per-head RMS norm, a weight, silu gate;
  * feed-forward: g = min(W_gate h, limit), u = clamp(W_up h, +-limit), W_down (g sigmoid(1.702 g) (u + 1));
  * logits = head . norm(x).

Every size and constant comes from config.json (`FasanexShape.from_config`), every tensor from model.safetensors under the
names of `tensor_shapes`.  The residual, norms, angles, scores and softmax weights, decays, step sizes, write strengths,
unit norms and the recurrent states are float32; the matrix products run in the model's dtype (bfloat16 with float
accumulation, or float32).

The compute path: library GEMMs (torch.matmul / bmm) for the projections and the kernels of libhydra_mix.so
(_C.kernel.seq_mix, .biased_attn, .depth_ops, .stream_ops).  The model plugs into the engine through the interface
LlamaForCausalLM has; `cache_spec` asks the block manager for a key and a value plane per attention mixer, `state_spec`
asks the state-slot manager for one flat row per sequence in which every mixer owns a piece (convolution tails, the last
token's input, matrix states)."""
import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor

from hydrainfer_amd._C.kernel.biased_attn import biased_attention
from hydrainfer_amd._C.kernel.depth_ops import depth_norm
from hydrainfer_amd._C.kernel.seq_mix import (causal_conv, clamped_glu, decay_exp, gated_group_norm, head_gates,
                                              head_norm_rope_cache, state_scan, token_shift_mix, unary, unit_norm)
from hydrainfer_amd._C.kernel.stream_ops import SequenceState, stream_embed
from hydrainfer_amd.layer.rotary_spec import RotarySpec

ARCHITECTURE = "Fasanex"
GLU_ALPHA = 1.702             # the feed-forward's gate: g sigmoid(GLU_ALPHA g)
UNIT_NORM_EPS = 1e-6          # delta rule: q, k / sqrt(sum of squares + UNIT_NORM_EPS)
SHIFT_MIXES = ("r", "k", "v", "g", "w")


@dataclass
class AttentionSpec:                  # the left side of a `parallel` mixer
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float
    softcap: float = 0.0
    window: Optional[int] = None
    rot: Optional[RotarySpec] = None


@dataclass
class TimeMixSpec:                    # the right side of a `parallel` mixer
    heads: int
    dim: int
    decay_rank: int = 16              # inner size of the decay's low-rank map: a checkpoint's tensors say


@dataclass
class MixerSpec:
    type: str                         # "mamba2" | "parallel" | "delta"
    heads: int = 0
    vdim: int = 0
    conv: int = 1
    state: int = 0                    # mamba2: rows of a head's state
    groups: int = 1                   # mamba2: groups of heads sharing B and C
    norm_groups: int = 1              # mamba2: parts of the output norm
    dim: int = 0                      # delta: q / k size per head
    kv_heads: int = 0                 # delta: q / k heads
    left: Optional[AttentionSpec] = None
    right: Optional[TimeMixSpec] = None
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass
class FeedForwardSpec:
    ff: int
    limit: Optional[float] = None     # None: gate and up are not clamped


@dataclass
class FasanexLayer:
    mixer: MixerSpec
    mlp: Optional[FeedForwardSpec]


def _round4(n: int) -> int:
    return (n + 3) // 4 * 4


@dataclass
class FasanexShape:
    vocab_size: int
    hidden_size: int
    layers: List[FasanexLayer]
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    cache_plane: Dict[int, int] = field(default_factory=dict)          # layer with attention -> its cache plane
    state_piece: Dict[Tuple[int, str], int] = field(default_factory=dict)   # (layer, piece) -> first float in a slot
    state_floats: int = 0
    max_position_embeddings: int = 1 << 24      # positions are computed, not looked up: no table bounds them

    def __post_init__(self):
        self.cache_plane, self.state_piece, at = {}, {}, 0
        W = self.hidden_size

        def piece(i: int, name: str, size: int):
            nonlocal at
            self.state_piece[(i, name)] = at
            at += _round4(max(size, 1))

        for i, l in enumerate(self.layers):
            m = l.mixer
            if m.type == "mamba2":
                if m.heads % m.groups or (m.heads * m.vdim) % m.norm_groups:
                    raise ValueError(f"layer {i}: heads must be a multiple of groups and the inner size of norm_groups")
                piece(i, "conv", (m.conv - 1) * (m.heads * m.vdim + 2 * m.groups * m.state))
                piece(i, "S", m.heads * m.state * m.vdim)
            elif m.type == "parallel":
                a, r = m.left, m.right
                if a.heads % a.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if a.vdim != a.dim:
                    raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
                if a.rot and (a.rot.dims % 2 or a.rot.dims > a.dim):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
                self.cache_plane[i] = len(self.cache_plane)
                piece(i, "conv", (a.conv - 1) * (a.heads + a.kv_heads) * a.dim)
                piece(i, "shift", W)
                piece(i, "S", r.heads * r.dim * r.dim)
            elif m.type == "delta":
                if m.heads % m.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                piece(i, "conv", (m.conv - 1) * (2 * m.kv_heads * m.dim + m.heads * m.vdim))
                piece(i, "S", m.heads * m.dim * m.vdim)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {m.type!r}")
        self.state_floats = at

    # what the engine's cache pool and parameter builders ask of a model's shape
    def _attn(self):
        return [l.mixer.left for l in self.layers if l.mixer.type == "parallel"]

    @property
    def num_hidden_layers(self) -> int:          # cache planes: one per attention mixer
        return max(1, len(self.cache_plane))

    @property
    def num_attention_heads(self) -> int:
        return max([a.heads for a in self._attn()] or [1])

    @property
    def num_key_value_heads(self) -> int:
        return max([a.kv_heads for a in self._attn()] or [1])

    @property
    def head_dim(self) -> int:
        return max([a.dim for a in self._attn()] or [1])

    @classmethod
    def from_config(cls, cfg: dict) -> "FasanexShape":
        if cfg.get("architecture") != ARCHITECTURE:
            raise ValueError(f"not a {ARCHITECTURE} configuration: {cfg.get('architecture')!r}")
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, kind = l["mixer"], l["type"]
            if kind == "mamba2":
                mixer = MixerSpec(kind, heads=int(m["heads"]), vdim=int(m["vdim"]), conv=int(m["conv"]), state=int(m["state"]),
                                  groups=int(m.get("groups", 1)), norm_groups=int(m.get("norm_groups", 1)))
            elif kind == "parallel":
                a, r = m["left"], m["right"]
                rot = None
                if a.get("rot"):
                    sc = a["rot"].get("scaling") or {}
                    rot = RotarySpec(int(a["rot"]["dims"]), float(a["rot"]["base"]),
                                     float(sc["factor"]) if sc.get("factor") else None, float(sc.get("original", 0.0)),
                                     float(sc.get("fast", 32.0)), float(sc.get("slow", 1.0)))
                mask = a.get("mask") or {}
                left = AttentionSpec(int(a["heads"]), int(a.get("kv_heads") or a["heads"]), int(a["dim"]), int(a.get("vdim", a["dim"])),
                                     int(a.get("conv", 1)), float(a["scale"]), float(a.get("softcap") or 0.0),
                                     int(mask["size"]) if mask.get("size") else None, rot)
                right = TimeMixSpec(int(r["heads"]), int(r["dim"]), int(r.get("decay_rank", 16)))
                mixer = MixerSpec(kind, left=left, right=right, left_scale=float(m.get("left_scale", 1.0)),
                                  right_scale=float(m.get("right_scale", 1.0)))
            elif kind == "delta":
                mixer = MixerSpec(kind, heads=int(m["heads"]), vdim=int(m["vdim"]), conv=int(m["conv"]), dim=int(m["dim"]),
                                  kv_heads=int(m.get("kv_heads") or m["heads"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp, spec = l.get("mlp"), None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
                spec = FeedForwardSpec(int(mlp["ff"]), float(mlp["limit"]) if mlp.get("limit") is not None else None)
            layers.append(FasanexLayer(mixer, spec))
        return cls(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                   norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-5)),
                   embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)))

    def to_config(self) -> dict:
        out = []
        for l in self.layers:
            m = l.mixer
            if m.type == "mamba2":
                mixer = {"conv": m.conv, "groups": m.groups, "heads": m.heads, "norm_groups": m.norm_groups, "state": m.state,
                         "vdim": m.vdim}
            elif m.type == "parallel":
                a, r = m.left, m.right
                left = {"conv": a.conv, "dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads, "scale": a.scale, "vdim": a.vdim}
                if a.softcap:
                    left["softcap"] = a.softcap
                if a.window:
                    left["mask"] = {"size": a.window}
                if a.rot:
                    left["rot"] = {"base": a.rot.base, "dims": a.rot.dims}
                    if a.rot.factor:
                        left["rot"]["scaling"] = {"factor": a.rot.factor, "original": a.rot.original, "fast": a.rot.fast,
                                                  "slow": a.rot.slow}
                mixer = {"left": left, "left_scale": m.left_scale, "right_scale": m.right_scale,
                         "right": {"dim": r.dim, "heads": r.heads, "decay_rank": r.decay_rank}}
            else:
                mixer = {"conv": m.conv, "dim": m.dim, "heads": m.heads, "kv_heads": m.kv_heads, "vdim": m.vdim}
            mlp = None if l.mlp is None else {"kind": "dense", "ff": l.mlp.ff}
            if mlp is not None and l.mlp.limit is not None:
                mlp["limit"] = l.mlp.limit
            out.append({"type": m.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": ARCHITECTURE, "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "layers": out}


def tensor_shapes(shape: FasanexShape) -> Dict[str, tuple]:
    """Name -> shape of every tensor of a checkpoint of this shape (linear weights are [out, in])."""
    W = shape.hidden_size
    out = {"embed": (shape.vocab_size, W), "final.norm": (W,), "head": (shape.vocab_size, W)}
    for i, l in enumerate(shape.layers):
        m, p = l.mixer, f"l{i}."
        out.update({p + "norm1": (W,), p + "norm1b": (W,)})
        x = p + "mix."
        if m.type == "mamba2":
            inner, gn = m.heads * m.vdim, m.groups * m.state
            out.update({x + "in": (2 * inner + 2 * gn + m.heads, W), x + "conv": (inner + 2 * gn, m.conv),
                        x + "conv.b": (inner + 2 * gn,), x + "dt_bias": (m.heads,), x + "A_log": (m.heads,), x + "D": (m.heads,),
                        x + "norm": (inner,), x + "o": (W, inner)})
        elif m.type == "parallel":
            a, r = m.left, m.right
            hd = r.heads * r.dim
            out.update({x + "left.q": (a.heads * a.dim, W), x + "left.k": (a.kv_heads * a.dim, W), x + "left.q.norm": (a.dim,),
                        x + "left.k.norm": (a.dim,), x + "left.q.conv": (a.heads * a.dim, a.conv),
                        x + "left.k.conv": (a.kv_heads * a.dim, a.conv), x + "left.g": (a.heads * a.vdim, W),
                        x + "left.o": (W, a.heads * a.vdim)})
            out.update({x + f"right.mu.{s}": (W,) for s in SHIFT_MIXES})
            out.update({x + f"right.{s}": (hd, W) for s in ("r", "k", "v", "g")})
            out.update({x + "right.w1": (r.decay_rank, W), x + "right.w2": (hd, r.decay_rank), x + "right.w0": (hd,),
                        x + "right.u": (r.heads, r.dim), x + "right.norm": (hd,), x + "right.o": (W, hd)})
        else:
            qk, hv = m.kv_heads * m.dim, m.heads * m.vdim
            out.update({x + "q": (qk, W), x + "q.conv": (qk, m.conv), x + "k": (qk, W), x + "k.conv": (qk, m.conv),
                        x + "v": (hv, W), x + "v.conv": (hv, m.conv), x + "b": (m.heads, W), x + "a": (m.heads, W),
                        x + "A_log": (m.heads,), x + "dt_bias": (m.heads,), x + "norm": (m.vdim,), x + "g": (hv, W),
                        x + "o": (W, hv)})
        if l.mlp is not None:
            out.update({p + "norm2": (W,), p + "norm2b": (W,), p + "mlp.gate": (l.mlp.ff, W), p + "mlp.up": (l.mlp.ff, W),
                        p + "mlp.down": (W, l.mlp.ff)})
    return out


class _LayerWeights:
    pass


class FasanexForCausalLM:
    supports_graph_decode = False      # the engine's captured decode step is built around the Llama launch sequence

    def __init__(self, shape: FasanexShape, dtype: torch.dtype, device, state: Dict[str, Tensor]):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("Fasanex runs in bfloat16 or float32")
        self.shape, self.dtype, self.device = shape, dtype, torch.device(device)
        self.layer_trace: Optional[List[Tensor]] = None    # tests: when a list, the residual after every layer
        dev = self.device
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        one_plus = lambda t: (1.0 + t.to(device=dev, dtype=torch.float32)).contiguous()
        act = lambda t: t.to(device=dev, dtype=dtype).contiguous()
        self.embed_table, self.head = act(state["embed"]), act(state["head"])
        self.final_norm = one_plus(state["final.norm"])
        self.lw: List[_LayerWeights] = []
        for i, l in enumerate(shape.layers):
            m, p = l.mixer, f"l{i}."
            x = p + "mix."
            w = _LayerWeights()
            w.norm1, w.norm1b = one_plus(state[p + "norm1"]), one_plus(state[p + "norm1b"])
            if m.type == "mamba2":
                w.w_in, w.o = act(state[x + "in"]), act(state[x + "o"])
                w.conv_w, w.conv_b = f32(state[x + "conv"]), f32(state[x + "conv.b"])
                w.step_bias, w.log_rate, w.skip = f32(state[x + "dt_bias"]), f32(state[x + "A_log"]), f32(state[x + "D"])
                w.o_norm = f32(state[x + "norm"])
            elif m.type == "parallel":
                a, r = m.left, m.right
                w.w_in = act(torch.cat([state[x + "left.q"], state[x + "left.k"], state[x + "left.g"]], dim=0))
                w.conv_w = f32(torch.cat([state[x + "left.q.conv"], state[x + "left.k.conv"]], dim=0))
                w.q_norm, w.k_norm = f32(state[x + "left.q.norm"]), f32(state[x + "left.k.norm"])
                w.inv_freq, w.cos_sin_scale = None, 1.0
                if a.rot and a.rot.dims >= 2:
                    freq, w.cos_sin_scale = a.rot.frequencies()
                    w.inv_freq = torch.tensor(freq, dtype=torch.float64).to(device=dev, dtype=torch.float32)
                w.mu = f32(torch.stack([state[x + f"right.mu.{s}"] for s in SHIFT_MIXES]))
                w.w_rkvg = act(torch.stack([state[x + f"right.{s}"].t() for s in ("r", "k", "v", "g")]))     # [4, W, heads * dim]
                w.w1, w.w2, w.w0 = act(state[x + "right.w1"]), act(state[x + "right.w2"]), f32(state[x + "right.w0"])
                w.bonus, w.o_norm = f32(state[x + "right.u"]).reshape(-1), f32(state[x + "right.norm"])
                w.o = act(torch.cat([state[x + "left.o"], state[x + "right.o"]], dim=1))      # both sides through one product
            else:
                w.w_in = act(torch.cat([state[x + s] for s in ("q", "k", "v", "b", "a", "g")], dim=0))
                w.conv_w = f32(torch.cat([state[x + "q.conv"], state[x + "k.conv"], state[x + "v.conv"]], dim=0))
                w.log_rate, w.step_bias, w.o_norm = f32(state[x + "A_log"]), f32(state[x + "dt_bias"]), f32(state[x + "norm"])
                w.o = act(state[x + "o"])
            if l.mlp is not None:
                w.norm2, w.norm2b = one_plus(state[p + "norm2"]), one_plus(state[p + "norm2b"])
                w.gate_up = act(torch.cat([state[p + "mlp.gate"], state[p + "mlp.up"]], dim=0))
                w.down = act(state[p + "mlp.down"])
            self.lw.append(w)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_state_dict(cls, shape: FasanexShape, sd: Dict[str, Tensor], dtype, device) -> "FasanexForCausalLM":
        for i, l in enumerate(shape.layers):          # sizes that only a tensor's shape gives
            key = f"l{i}.mix.right.w1"
            if l.mixer.type == "parallel" and key in sd:
                l.mixer.right.decay_rank = int(sd[key].shape[0])
        want = tensor_shapes(shape)
        missing = [k for k in want if k not in sd]
        if missing:
            raise RuntimeError(f"{len(missing)} tensors missing from the checkpoint, e.g. {missing[:3]}")
        for k, shp in want.items():
            if tuple(sd[k].shape) != shp:
                raise RuntimeError(f"tensor {k}: shape {tuple(sd[k].shape)} in the checkpoint, {shp} by config.json")
        return cls(shape, dtype, device, {k: sd[k] for k in want})

    @staticmethod
    def random_state_dict(shape: FasanexShape, seed: int = 0) -> Dict[str, Tensor]:
        """Random bfloat16 weights of a size that keeps activations O(1): linears N(0, 1/fan_in), stored norm offsets and
        biases small, decays spread between fast and slow."""
        g = torch.Generator().manual_seed(seed)
        sd = {}
        for k, shp in tensor_shapes(shape).items():
            leaf = k.split(".", 1)[-1] if k[0] == "l" and k[1].isdigit() else k
            tail = leaf.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm1b", "norm2", "norm2b", "final.norm"):
                t = 0.1 * torch.randn(shp, generator=g)
            elif tail == "norm":
                t = 1.0 + 0.1 * torch.randn(shp, generator=g)
            elif tail == "conv":
                t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
            elif tail in ("b",) and leaf.endswith("conv.b"):
                t = 0.1 * torch.randn(shp, generator=g)
            elif tail in ("dt_bias", "w0"):
                t = torch.randn(shp, generator=g) - 1.0
            elif tail == "A_log":
                t = torch.rand(shp, generator=g) * 1.5 - 1.0
            elif tail in ("D", "u"):
                t = 0.5 + 0.3 * torch.randn(shp, generator=g)
            elif ".mu." in leaf:
                t = torch.rand(shp, generator=g)
            elif k == "embed":
                t = torch.randn(shp, generator=g) * 0.7
            else:
                t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
            sd[k] = t.to(torch.bfloat16)      # checkpoints hold bfloat16
        return sd

    @classmethod
    def random_init(cls, shape: FasanexShape, dtype, device, seed: int = 0) -> "FasanexForCausalLM":
        return cls(shape, dtype, device, cls.random_state_dict(shape, seed))

    # ------------------------------------------------------------------ what the engine asks
    def cache_spec(self) -> dict:
        """Planes and row size of the paged cache: a key and a value plane per attention mixer."""
        sh = self.shape
        return {"n_layers": sh.num_hidden_layers, "n_tokens": 2, "n_heads": sh.num_key_value_heads, "head_size": sh.head_dim}

    def state_spec(self) -> Optional[dict]:
        """What a sequence carries from step to step beside the cache: one flat row, a piece of it for every mixer's
        convolution tail, last input and matrix state."""
        return {"rows": 1, "width": self.shape.state_floats} if self.shape.state_floats else None

    def prepare_decode(self, max_rows: int = 64, keep_row_major: bool = True) -> None:
        """Nothing to prepare: decode steps run on the same weights as portions of prompts."""

    def weight_bytes(self, tokens: int = 1) -> int:
        e = torch.empty((), dtype=self.dtype).element_size()
        n = self.head.numel()
        for l, w in zip(self.shape.layers, self.lw):
            n += w.w_in.numel() + w.o.numel()
            if l.mixer.type == "parallel":
                n += w.w_rkvg.numel() + w.w1.numel() + w.w2.numel()
            if l.mlp is not None:
                n += w.gate_up.numel() + w.down.numel()
        return n * e

    def embed(self, input_ids: Tensor) -> Tensor:
        return input_ids

    # ------------------------------------------------------------------ mixers
    def _mamba2(self, i: int, h: Tensor, pos: Tensor, q_cu: Tensor, params, seq: SequenceState) -> Tensor:
        m, w, sh = self.shape.layers[i].mixer, self.lw[i], self.shape
        inner, gn = m.heads * m.vdim, m.groups * m.state
        proj = torch.matmul(h, w.w_in.t())                                   # [T, z | x | B | C | dt]
        xbc = causal_conv(proj[:, inner:2 * inner + 2 * gn], w.conv_w, w.conv_b, "silu", seq, sh.state_piece[(i, "conv")], q_cu, pos)
        decay, step, _ = head_gates(proj[:, 2 * inner + 2 * gn:], w.log_rate, w.step_bias, want_step=True)
        x = xbc[:, :inner]
        o = state_scan("decay", xbc[:, inner + gn:], xbc[:, inner:inner + gn], x, decay, seq, sh.state_piece[(i, "S")], q_cu, pos,
                       m.heads, m.groups, m.state, m.vdim, vscale=step)
        y = gated_group_norm(o, self.dtype, group=inner // m.norm_groups, eps=sh.norm_eps, w=w.o_norm, gate=proj[:, :inner],
                             gate_act="silu", gate_first=True, skip=x, skip_w=w.skip, skip_group=m.vdim)
        return torch.matmul(y, w.o.t())

    def _parallel(self, i: int, h: Tensor, pos: Tensor, q_cu: Tensor, params, seq: SequenceState) -> Tensor:
        m, w, sh = self.shape.layers[i].mixer, self.lw[i], self.shape
        a, r = m.left, m.right
        T, H, G, D = h.shape[0], a.heads, a.kv_heads, a.dim
        hd = r.heads * r.dim
        both = torch.empty((T, H * a.vdim + hd), dtype=self.dtype, device=self.device)
        # left: attention over the paged cache
        ap = params.attention_params[sh.cache_plane[i]]
        kc, vc = ap.kv_cache.get_kv_cache()
        proj = torch.matmul(h, w.w_in.t())                                   # [T, q | k | gate]
        qk = causal_conv(proj[:, :(H + G) * D], w.conv_w, None, None, seq, sh.state_piece[(i, "conv")], q_cu, pos)
        q = head_norm_rope_cache(qk[:, :H * D], qk[:, H * D:], w.q_norm, w.k_norm, sh.norm_eps, H, G, D, w.inv_freq,
                                 w.cos_sin_scale, pos, ap.new_cache_slots, kc, vc)
        o = biased_attention(q.view(T, H, D), kc, vc, a.vdim, seq.tok_seq, pos, ap.q_cu_seq_lens, ap.block_tables, ap.cu_blocks_lens,
                             a.scale, None, "window" if a.window else "causal", a.window or 0, max_q_len=ap.q_max_seq_len,
                             kv_heads=G, max_kv_len=ap.kv_max_seq_len, softcap=a.softcap)
        gated_group_norm(o.view(T, H * a.vdim), self.dtype, gate=proj[:, (H + G) * D:], gate_act="sigmoid", scale=m.left_scale,
                         out=both[:, :H * a.vdim])
        # right: time mixing
        mixes = token_shift_mix(h, w.mu, seq, sh.state_piece[(i, "shift")], q_cu, pos)             # [5, T, W]
        rkvg = torch.bmm(mixes[:4], w.w_rkvg)                                                      # [4, T, heads * dim]
        low = torch.matmul(unary(torch.matmul(mixes[4], w.w1.t()), "tanh"), w.w2.t())
        o = state_scan("bonus", rkvg[0], rkvg[1], rkvg[2], decay_exp(low, w.w0), seq, sh.state_piece[(i, "S")], q_cu, pos,
                       r.heads, r.heads, r.dim, r.dim, bonus=w.bonus)
        gated_group_norm(o, self.dtype, group=r.dim, eps=sh.norm_eps, w=w.o_norm, gate=rkvg[3], gate_act="silu", scale=m.right_scale,
                         out=both[:, H * a.vdim:])
        return torch.matmul(both, w.o.t())

    def _delta(self, i: int, h: Tensor, pos: Tensor, q_cu: Tensor, params, seq: SequenceState) -> Tensor:
        m, w, sh = self.shape.layers[i].mixer, self.lw[i], self.shape
        qk, hv, H = m.kv_heads * m.dim, m.heads * m.vdim, m.heads
        proj = torch.matmul(h, w.w_in.t())                                   # [T, q | k | v | b | a | gate]
        c = causal_conv(proj[:, :2 * qk + hv], w.conv_w, None, "silu", seq, sh.state_piece[(i, "conv")], q_cu, pos)
        q = unit_norm(c[:, :qk], m.kv_heads, m.dim, UNIT_NORM_EPS, m.dim ** -0.5)
        k = unit_norm(c[:, qk:2 * qk], m.kv_heads, m.dim, UNIT_NORM_EPS)
        at = 2 * qk + hv
        decay, _, beta = head_gates(proj[:, at + H:at + 2 * H], w.log_rate, w.step_bias, b=proj[:, at:at + H])
        o = state_scan("delta", q, k, c[:, 2 * qk:], decay, seq, sh.state_piece[(i, "S")], q_cu, pos, H, m.kv_heads, m.dim, m.vdim,
                       beta=beta)
        y = gated_group_norm(o, self.dtype, group=m.vdim, eps=sh.norm_eps, w=w.o_norm, gate=proj[:, at + 2 * H:], gate_act="silu")
        return torch.matmul(y, w.o.t())

    def _feed_forward(self, i: int, h: Tensor) -> Tensor:
        f, w = self.shape.layers[i].mlp, self.lw[i]
        gu = torch.matmul(h, w.gate_up.t())
        return torch.matmul(clamped_glu(gu[:, :f.ff], gu[:, f.ff:], f.limit if f.limit is not None else 0.0, GLU_ALPHA, 1.0), w.down.t())

    # ------------------------------------------------------------------ forward
    def forward_hidden(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """The normed output [n_selected, width] of model_params.selected_token_ids (all rows if None).  Every token's keys
        and values go to the cache and every sequence's state slot is brought up to date."""
        sh, dt = self.shape, self.dtype
        if input_ids.dtype not in (torch.int32, torch.int64):
            raise ValueError("Fasanex takes token ids (its embedding is scaled in float)")
        if position_ids.dtype != torch.int32:
            position_ids = position_ids.to(torch.int32)
        input_ids, position_ids = input_ids.contiguous(), position_ids.contiguous()
        seq = model_params.sequence_state
        if seq is None:
            raise ValueError("Fasanex needs LanguageModelParameters.sequence_state (the batch's sequences and their state slots)")
        q_cu = model_params.attention_params[0].q_cu_seq_lens
        L, eps = len(sh.layers), sh.norm_eps
        x = stream_embed(input_ids, self.embed_table, sh.embedding_scale, 1).view(input_ids.shape[0], sh.hidden_size)
        sel = model_params.selected_token_ids
        rows = sel.to(torch.int32).contiguous() if sel is not None and self.layer_trace is None else None
        if L == 0:
            return depth_norm(x, dt, eps, next_w=self.final_norm, rows=rows, rms=True)
        h = depth_norm(x, dt, eps, next_w=self.lw[0].norm1, rms=True)
        mixers = {"mamba2": self._mamba2, "parallel": self._parallel, "delta": self._delta}
        for i, (l, w) in enumerate(zip(sh.layers, self.lw)):
            y = mixers[l.mixer.type](i, h, position_ids, q_cu, model_params, seq)
            post = w.norm1b
            if l.mlp is not None:
                h = depth_norm(x, dt, eps, y=y, post_w=post, x_out=x, next_w=w.norm2, rms=True)
                y, post = self._feed_forward(i, h), w.norm2b
            last = i == L - 1
            # the sublayer's normed result joins the residual, which is normed for what comes next (the final norm on the
            # selected rows only)
            h = depth_norm(x, dt, eps, y=y, post_w=post, x_out=None if (last and rows is not None) else x,
                           next_w=self.final_norm if last else self.lw[i + 1].norm1, rows=rows if last else None, rms=True)
            if self.layer_trace is not None:
                self.layer_trace.append(x.clone())
        if rows is None and sel is not None:
            h = h.index_select(0, sel.to(torch.int64))
        return h

    def forward_logits(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """float32 logits [n_selected, vocab]."""
        x = self.forward_hidden(input_ids, position_ids, model_params)
        return torch.matmul(x, self.head.t()).float()

    def forward(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """Greedy token ids of the selected rows, like the framework's other models."""
        return torch.argmax(self.forward_logits(input_ids, position_ids, model_params), dim=-1)

    __call__ = forward


def read_shape(model_path: str) -> FasanexShape:
    with open(os.path.join(model_path, "config.json")) as f:
        return FasanexShape.from_config(json.load(f))
