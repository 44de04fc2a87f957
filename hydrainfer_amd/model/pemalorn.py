"""Pemalorn — a decoder-only model whose layers run a mixer and a feed-forward side by side on one normed input:

  * x = embed[token]; a layer is h = layer_norm(x) * w (no bias), x <- x + mixer(h + conv_1(h)) + ff(h + conv_2(h)), the
    convolutions short, causal and per channel (their last inputs travel with the sequence), then a per-layer token input
    x <- x + rms_norm(W_proj (gelu_tanh(W_gate x) * e)) * w with e the layer's slice of a second embedding of the token;
  * mixer `attention`: grouped-query attention, rotary positions on the first channels of every head (pairs i, i + dims / 2),
    values that turn by their own position over all their channels and whose weighted sum is turned back by the query's,
    scores q . k * scale * temperature_h, a sink per head in the softmax's denominator, a sigmoid gate per head;
  * mixer `latent_attention`: queries through a normed latent, keys and values through ONE normed latent c per token plus
    one rotated key part shared by the heads (pairs 2 i, 2 i + 1; YaRN-scaled frequencies); sliding window; a sink per
    head; a sigmoid gate per element.  Only [c | rotated part] is cached: W_uk is folded into the query and W_uv applied
    after the weighted sum, so every head attends over the same cached rows;
  * feed-forward: a mixture of silu-gated experts — softmax router over all outputs, the choice carries a correction, the
    weights are the chosen scores themselves, and the last outputs of the router are identity experts (input * weight);
  * a span of layers may run several times with the same weights; each pass starts from W_in [x; x0] + step[pass], x0 the
    embedding, and has caches and convolution state of its own;
  * logits = head . layer_norm(x).

Every size and constant comes from config.json (`PemalornShape.from_config`), every tensor from model.safetensors under the
names of `tensor_shapes`.  The residual, norms, angles, scores and softmax weights and the router are float32; the matrix
products run in the model's dtype (bfloat16 with float accumulation, or float32).

The compute path: library GEMMs (torch.matmul / bmm) and the kernels of libhydra_mix.so (_C.kernel.depth_ops, .seq_mix,
.rotary, .biased_attn, .latent_attn, .moe_mix, .stream_ops).  The model plugs into the engine through the interface
LlamaForCausalLM has; `cache_spec` asks the block manager for one plane per cached row kind and layer run (keys and values
of an attention mixer are two planes, a latent mixer's row one), `state_spec` asks the state-slot manager for one flat row
per sequence in which every layer run owns the tail of its convolutions' input."""
import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor

from hydrainfer_amd._C.kernel.biased_attn import biased_attention
from hydrainfer_amd._C.kernel.depth_ops import depth_norm
from hydrainfer_amd._C.kernel.latent_attn import latent_attention, latent_norm_cache
from hydrainfer_amd._C.kernel.moe_mix import grouped_linear, moe_combine, moe_plan, route_softmax_topk
from hydrainfer_amd._C.kernel.rotary import RotaryPart, rotary_parts
from hydrainfer_amd._C.kernel.seq_mix import causal_conv_pair, clamped_glu, gated_group_norm
from hydrainfer_amd._C.kernel.stream_ops import SequenceState, gelu_tanh_and_mul, stream_embed
from hydrainfer_amd.layer.rotary_spec import RotarySpec

ARCHITECTURE = "Pemalorn"


def _round8(n: int) -> int:
    return (n + 7) // 8 * 8


@dataclass
class MixerSpec:
    type: str                         # "attention" | "latent_attention"
    heads: int
    dim: int                          # attention: q / k size per head; latent: the unrotated part of it
    vdim: int
    scale: float
    kv_heads: int = 0                 # attention
    kv_rank: int = 0                  # latent: the cached latent
    q_rank: int = 0                   # latent: the query's latent
    rot_dim: int = 0                  # latent: the rotated part of q / k
    window: Optional[int] = None      # position i sees j with 0 <= i - j < window; None: every j <= i
    rot: Optional[RotarySpec] = None

    @property
    def row(self) -> int:
        """Elements a token leaves in ONE cache plane of this mixer."""
        if self.type == "attention":
            return self.kv_heads * self.head_stride
        return self.kv_rank + self.rot_dim

    @property
    def head_stride(self) -> int:     # attention: from one key / value head to the next within a cache row
        return _round8(max(self.dim, self.vdim))

    @property
    def planes(self) -> int:
        return 2 if self.type == "attention" else 1


@dataclass
class ExpertsSpec:
    experts: int                      # experts with tensors
    identity: int                     # router outputs beyond them: experts that hand their input on
    top: int
    ff: int


@dataclass
class PemalornLayer:
    mixer: MixerSpec
    mlp: Optional[ExpertsSpec]


@dataclass
class PemalornShape:
    vocab_size: int
    hidden_size: int
    layers: List[PemalornLayer]
    norm_eps: float = 1e-5
    taps: int = 0                     # taps of the input convolutions (one tap: h (1 + w)); 0: the design's layers have none
    side_dim: int = 0                 # per-layer slice of the token's second embedding; 0: no per-layer token input
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    has_loop: bool = False
    runs: List[Tuple[int, int, bool]] = field(default_factory=list)   # (layer, pass, first of its pass) of every layer run
    run_plane: List[int] = field(default_factory=list)                # first cache plane of every layer run
    n_planes: int = 0
    state_floats: int = 0
    max_position_embeddings: int = 1 << 24      # positions are computed, not looked up: no table bounds them

    def __post_init__(self):
        n = len(self.layers)
        if self.has_loop:
            if not (0 <= self.loop_start < self.loop_stop <= n) or self.loop_times < 1:
                raise ValueError(f"loop {self.loop_start}..{self.loop_stop} x {self.loop_times} does not fit {n} layers")
            a, b = self.loop_start, self.loop_stop
            self.runs = [(i, 0, False) for i in range(a)]
            for t in range(self.loop_times):
                self.runs += [(i, t, i == a) for i in range(a, b)]
            self.runs += [(i, 0, False) for i in range(b, n)]
        else:
            self.runs = [(i, 0, False) for i in range(n)]
        self.run_plane, at = [], 0
        for i, _, _ in self.runs:
            self.run_plane.append(at)
            at += self.layers[i].mixer.planes
        self.n_planes = at
        for i, l in enumerate(self.layers):
            m = l.mixer
            if m.type == "attention":
                if m.heads % m.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if m.vdim % 2:
                    raise ValueError(f"layer {i}: values turn in pairs, so vdim must be even")
                if m.rot and (m.rot.dims % 2 or m.rot.dims > m.dim):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
            elif m.type == "latent_attention":
                if m.rot_dim % 2:
                    raise ValueError(f"layer {i}: rot_dim must be even")
            else:
                raise ValueError(f"layer {i}: unknown mixer type {m.type!r}")
            if self.taps < 0:
                raise ValueError("canon.taps must not be negative")
            if l.mlp is not None and (l.mlp.experts < 1 or not 1 <= l.mlp.top <= l.mlp.experts + l.mlp.identity):
                raise ValueError(f"layer {i}: at least one expert with tensors, and top within the router's outputs")
        # a layer run's piece of a sequence's state: the last taps - 1 inputs of its convolutions
        self.state_floats = len(self.runs) * self.state_piece_floats

    @property
    def state_piece_floats(self) -> int:
        # (one tap keeps nothing, but its kernel is handed a piece like the others: a row of `width` nobody reads)
        return max(self.taps - 1, 1) * self.hidden_size if self.taps >= 1 else 0

    def state_piece(self, run: int) -> int:
        return run * self.state_piece_floats

    # what the engine's cache pool and parameter builders ask of a model's shape
    @property
    def num_hidden_layers(self) -> int:          # cache planes
        return max(1, self.n_planes)

    @property
    def num_attention_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    @property
    def num_key_value_heads(self) -> int:        # a plane's row is one run of elements; a mixer lays its heads out in it
        return 1

    @property
    def head_dim(self) -> int:                   # width of a cache row: the widest any mixer needs
        return _round8(max(l.mixer.row for l in self.layers))

    @classmethod
    def from_config(cls, cfg: dict) -> "PemalornShape":
        if cfg.get("architecture") != ARCHITECTURE:
            raise ValueError(f"not a {ARCHITECTURE} configuration: {cfg.get('architecture')!r}")
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, kind = l["mixer"], l["type"]
            mask = m.get("mask") or {}
            window = int(mask["size"]) if mask.get("size") else None
            rot = RotarySpec.from_config(m.get("rot"))
            if kind == "attention":
                mixer = MixerSpec(kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                  scale=float(m["scale"]), kv_heads=int(m.get("kv_heads") or m["heads"]), window=window, rot=rot)
            elif kind == "latent_attention":
                mixer = MixerSpec(kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                                  kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), rot_dim=int(m.get("rot_dim", 0)),
                                  window=window, rot=rot)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp, spec = l.get("mlp"), None
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
                r = mlp["router"]
                spec = ExpertsSpec(int(r["experts"]), int(r.get("identity", 0)), int(r["top"]), int(mlp["expert"]["ff"]))
            layers.append(PemalornLayer(mixer, spec))
        loop = cfg.get("loop") or None
        if loop and int(loop["stop"]) <= int(loop["start"]):
            loop = None               # a span without layers: nothing runs twice, and no pass is ever entered
        return cls(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                   norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-5)), taps=int((cfg.get("canon") or {}).get("taps", 0)),
                   side_dim=int((cfg.get("token_side") or {}).get("dim", 0)),
                   loop_start=int(loop["start"]) if loop else 0, loop_stop=int(loop["stop"]) if loop else 0,
                   loop_times=int(loop.get("times", 1)) if loop else 1, has_loop=bool(loop))

    def to_config(self) -> dict:
        out = []
        for l in self.layers:
            m = l.mixer
            if m.type == "attention":
                mixer = {"dim": m.dim, "heads": m.heads, "kv_heads": m.kv_heads, "scale": m.scale, "vdim": m.vdim}
            else:
                mixer = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank, "q_rank": m.q_rank, "rot_dim": m.rot_dim,
                         "scale": m.scale, "vdim": m.vdim}
            if m.rot:
                mixer["rot"] = m.rot.to_config()
            if m.window:
                mixer["mask"] = {"size": m.window}
            mlp = None
            if l.mlp is not None:
                mlp = {"kind": "moe", "expert": {"ff": l.mlp.ff},
                       "router": {"experts": l.mlp.experts, "identity": l.mlp.identity, "top": l.mlp.top}}
            out.append({"type": m.type, "mixer": mixer, "mlp": mlp})
        cfg = {"architecture": ARCHITECTURE, "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "layers": out}
        if self.taps >= 1:
            cfg["canon"] = {"taps": self.taps}
        if self.side_dim:
            cfg["token_side"] = {"dim": self.side_dim}
        if self.has_loop:
            cfg["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return cfg


def tensor_shapes(shape: PemalornShape) -> Dict[str, tuple]:
    """Name -> shape of every tensor of a checkpoint of this shape (linear weights are [out, in])."""
    W, L = shape.hidden_size, len(shape.layers)
    out = {"embed": (shape.vocab_size, W), "final.norm": (W,), "head": (shape.vocab_size, W)}
    if shape.has_loop:
        out.update({"loop.in": (W, 2 * W), "loop.step": (shape.loop_times, W)})
    if shape.side_dim:
        out["side.embed"] = (shape.vocab_size, L * shape.side_dim)
    for i, l in enumerate(shape.layers):
        m, p = l.mixer, f"l{i}."
        x = p + "mix."
        out[p + "norm1"] = (W,)
        if m.type == "attention":
            out.update({x + "q": (m.heads * m.dim, W), x + "k": (m.kv_heads * m.dim, W), x + "v": (m.kv_heads * m.vdim, W),
                        x + "temp": (m.heads,), x + "sink": (m.heads,), x + "g": (m.heads, W), x + "o": (W, m.heads * m.vdim)})
        else:
            out.update({x + "dq": (m.q_rank, W), x + "dq.norm": (m.q_rank,), x + "uq": (m.heads * (m.dim + m.rot_dim), m.q_rank),
                        x + "dkv": (m.kv_rank + m.rot_dim, W), x + "dkv.norm": (m.kv_rank,), x + "uk": (m.heads * m.dim, m.kv_rank),
                        x + "uv": (m.heads * m.vdim, m.kv_rank), x + "sink": (m.heads,), x + "g": (m.heads * m.vdim, W),
                        x + "o": (W, m.heads * m.vdim)})
        if l.mlp is not None:
            f = l.mlp
            for e in range(f.experts):
                out.update({p + f"mlp.e{e}.gate": (f.ff, W), p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
            out.update({p + "mlp.router": (f.experts + f.identity, W), p + "mlp.correction": (f.experts + f.identity,)})
        if shape.taps >= 1:
            out[p + "canon1"] = (W, shape.taps)
            if l.mlp is not None:
                out[p + "canon2"] = (W, shape.taps)
        if shape.side_dim:
            out.update({p + "side.gate": (shape.side_dim, W), p + "side.proj": (W, shape.side_dim), p + "side.norm": (W,)})
    return out


class _LayerWeights:
    pass


class PemalornForCausalLM:
    supports_graph_decode = False      # the engine's captured decode step is built around the Llama launch sequence

    def __init__(self, shape: PemalornShape, dtype: torch.dtype, device, state: Dict[str, Tensor]):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("Pemalorn runs in bfloat16 or float32")
        self.shape, self.dtype, self.device = shape, dtype, torch.device(device)
        self.layer_trace: Optional[List[Tensor]] = None    # tests: when a list, the residual after every layer run
        dev = self.device
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        act = lambda t: t.to(device=dev, dtype=dtype).contiguous()
        f64 = lambda v: torch.tensor(v, dtype=torch.float64, device=dev)
        self.embed_table, self.head, self.final_norm = act(state["embed"]), act(state["head"]), f32(state["final.norm"])
        self.loop_in = act(state["loop.in"]) if shape.has_loop else None
        self.loop_step = f32(state["loop.step"]) if shape.has_loop else None
        self.side_table = act(state["side.embed"]) if shape.side_dim else None
        self.lw: List[_LayerWeights] = []
        for i, l in enumerate(shape.layers):
            m, p = l.mixer, f"l{i}."
            x = p + "mix."
            w = _LayerWeights()
            w.norm1 = f32(state[p + "norm1"])
            w.canon1 = f32(state[p + "canon1"]) if p + "canon1" in state else None
            w.canon2 = f32(state[p + "canon2"]) if p + "canon2" in state else None
            w.sink = f32(state[x + "sink"]) if x + "sink" in state else None
            w.o = act(state[x + "o"])
            w.freq, w.mag = None, 1.0
            rot_dims = (m.rot.dims if m.type == "attention" else m.rot_dim) if m.rot else 0
            if m.rot and rot_dims >= 2:
                freq, w.mag = RotarySpec(rot_dims, m.rot.base, m.rot.factor, m.rot.original, m.rot.fast, m.rot.slow).frequencies()
                w.freq = f64(freq)
            if m.type == "attention":
                w.w_in = act(torch.cat([state[x + "q"], state[x + "k"], state[x + "v"], state[x + "g"]], dim=0))
                w.temp = f32(state[x + "temp"]) if x + "temp" in state else None
                # the values turn over all their channels, by plain frequencies of the keys' base
                base = m.rot.base if m.rot else 10000.0
                w.vfreq = f64([base ** (-2.0 * j / m.vdim) for j in range(m.vdim // 2)])
            else:
                H, D, R, C, V = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
                w.w_in = act(torch.cat([state[x + "dq"], state[x + "dkv"], state[x + "g"]], dim=0))
                w.dq_norm, w.dkv_norm = f32(state[x + "dq.norm"]), f32(state[x + "dkv.norm"])
                w.uq = act(state[x + "uq"])
                # a head's query in the space of the cached row [c | rotated part]: q~ = [W_uk,h^T q_plain | q_rotated]
                uk = torch.zeros(H, D + R, C + R, dtype=torch.float32)
                uk[:, :D, :C] = state[x + "uk"].float().reshape(H, D, C)
                uk[:, D:, C:] = torch.eye(R)
                w.uk = act(uk)
                # and its result back from it: o_h = W_uv,h (sum_j p_j c_j); the rotated columns of the sum carry nothing
                uv = torch.zeros(H, C + R, V, dtype=torch.float32)
                uv[:, :C, :] = state[x + "uv"].float().reshape(H, V, C).transpose(1, 2)
                w.uv_t = act(uv)
            if l.mlp is not None:
                f = l.mlp
                w.router = f32(state[p + "mlp.router"]).t().contiguous()          # [W, experts + identity]
                w.correction = f32(state[p + "mlp.correction"]) if p + "mlp.correction" in state else None
                w.gate_up = act(torch.stack([torch.cat([state[p + f"mlp.e{e}.gate"], state[p + f"mlp.e{e}.up"]], dim=0)
                                             for e in range(f.experts)]))         # [E, 2 ff, W]
                w.down = act(torch.stack([state[p + f"mlp.e{e}.down"] for e in range(f.experts)]))      # [E, W, ff]
            w.has_side = bool(shape.side_dim) and p + "side.gate" in state
            if w.has_side:
                w.side_gate, w.side_proj, w.side_norm = act(state[p + "side.gate"]), act(state[p + "side.proj"]), f32(state[p + "side.norm"])
            self.lw.append(w)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_state_dict(cls, shape: PemalornShape, sd: Dict[str, Tensor], dtype, device) -> "PemalornForCausalLM":
        want = tensor_shapes(shape)
        # a checkpoint without these tensors has no such mechanism (no temperature, no sink, no correction of the choice)
        optional = lambda k: k.rsplit(".", 1)[-1] in ("temp", "sink", "correction")
        missing = [k for k in want if k not in sd and not optional(k)]
        if missing:
            raise RuntimeError(f"{len(missing)} tensors missing from the checkpoint, e.g. {missing[:3]}")
        for k, shp in want.items():
            if k in sd and tuple(sd[k].shape) != shp:
                raise RuntimeError(f"tensor {k}: shape {tuple(sd[k].shape)} in the checkpoint, {shp} by config.json")
        return cls(shape, dtype, device, {k: sd[k] for k in want if k in sd})

    @staticmethod
    def random_state_dict(shape: PemalornShape, seed: int = 0) -> Dict[str, Tensor]:
        """Random bfloat16 weights of a size that keeps activations O(1): linears N(0, 1/fan_in), norm weights near one,
        temperatures near one, sinks and corrections small."""
        g = torch.Generator().manual_seed(seed)
        sd = {}
        for k, shp in tensor_shapes(shape).items():
            tail = k.rsplit(".", 1)[-1]
            if tail in ("norm1", "norm") or k == "final.norm":
                t = 1.0 + 0.1 * torch.randn(shp, generator=g)
            elif tail == "temp":
                t = 1.0 + 0.2 * torch.randn(shp, generator=g)
            elif tail == "sink":
                t = 0.5 * torch.randn(shp, generator=g)
            elif tail == "correction":
                t = 0.05 * torch.randn(shp, generator=g)
            elif tail in ("canon1", "canon2"):
                t = 0.3 * torch.randn(shp, generator=g)
            elif k == "loop.step":
                t = 0.1 * torch.randn(shp, generator=g)
            elif k in ("embed", "side.embed"):
                t = torch.randn(shp, generator=g)
            else:
                t = torch.randn(shp, generator=g) / math.sqrt(shp[-1])
            sd[k] = t.to(torch.bfloat16)      # checkpoints hold bfloat16
        return sd

    @classmethod
    def random_init(cls, shape: PemalornShape, dtype, device, seed: int = 0) -> "PemalornForCausalLM":
        return cls(shape, dtype, device, cls.random_state_dict(shape, seed))

    # ------------------------------------------------------------------ what the engine asks
    def cache_spec(self) -> dict:
        """Planes and row size of the paged cache: per layer run a key and a value plane (attention) or one plane of
        [latent | rotated key part] rows (latent attention); a row is as wide as the widest of them."""
        sh = self.shape
        return {"n_layers": sh.num_hidden_layers, "n_tokens": 1, "n_heads": 1, "head_size": sh.head_dim}

    def state_spec(self) -> Optional[dict]:
        """What a sequence carries from step to step beside the cache: one flat row, a piece of it for every layer run's
        last convolution inputs."""
        return {"rows": 1, "width": self.shape.state_floats} if self.shape.state_floats else None

    def prepare_decode(self, max_rows: int = 64, keep_row_major: bool = True) -> None:
        """Nothing to prepare: decode steps run on the same weights as portions of prompts."""

    def weight_bytes(self, tokens: int = 1) -> int:
        """Bytes of matrix weights a step of `tokens` tokens streams at most (looped layers every time they run; of the
        experts those that the tokens can choose)."""
        e = torch.empty((), dtype=self.dtype).element_size()
        n = self.head.numel() + (self.loop_in.numel() * self.shape.loop_times if self.loop_in is not None else 0)
        for li, _, _ in self.shape.runs:
            l, w = self.shape.layers[li], self.lw[li]
            n += w.w_in.numel() + w.o.numel()
            if l.mixer.type == "latent_attention":
                n += w.uq.numel() + w.uk.numel() + w.uv_t.numel()
            if l.mlp is not None:
                used = min(l.mlp.experts, tokens * l.mlp.top)
                n += (w.gate_up.numel() + w.down.numel()) // l.mlp.experts * used
            if w.has_side:
                n += w.side_gate.numel() + w.side_proj.numel()
        return n * e

    def embed(self, input_ids: Tensor) -> Tensor:
        return input_ids

    # ------------------------------------------------------------------ mixers
    def _attention(self, run: int, li: int, h: Tensor, pos: Tensor, params, seq: SequenceState) -> Tensor:
        m, w = self.shape.layers[li].mixer, self.lw[li]
        T, H, G, D, V, hs = h.shape[0], m.heads, m.kv_heads, m.dim, m.vdim, m.head_stride
        plane = self.shape.run_plane[run]
        ap = params.attention_params[plane]
        kp, vp = ap.kv_cache.key_cache, params.attention_params[plane + 1].kv_cache.key_cache
        proj = torch.matmul(h, w.w_in.t())                                    # [T, q | k | v | gate]
        at_k, at_v, at_g = H * D, (H + G) * D, (H + G) * D + G * V
        q = rotary_parts([
            RotaryPart(proj[:, :at_k], H, D, w.freq, layout="halves", mag=w.mag),
            RotaryPart(proj[:, at_k:at_v], G, D, w.freq, layout="halves", mag=w.mag, cache=kp, cache_head_stride=hs),
            RotaryPart(proj[:, at_v:at_g], G, V, w.vfreq, layout="halves", cache=vp, cache_head_stride=hs),
        ], pos, ap.new_cache_slots)[0]
        # the planes' rows as this layer's heads
        heads = lambda c: c.as_strided((c.shape[0], c.shape[1], G, hs), (c.stride(0), c.stride(1), hs, 1))
        o = biased_attention(q.view(T, H, D), heads(kp), heads(vp), V, seq.tok_seq, pos, ap.q_cu_seq_lens, ap.block_tables,
                             ap.cu_blocks_lens, m.scale, None, "window" if m.window else "causal", m.window or 0,
                             max_q_len=ap.q_max_seq_len, kv_heads=G, max_kv_len=ap.kv_max_seq_len, head_scale=w.temp, sinks=w.sink)
        # every head's sum of turned values is turned back by the query's position, then gated
        og = rotary_parts([RotaryPart(o.view(T, H * V), H, V, w.vfreq, layout="halves", back=True, gate=proj[:, at_g:],
                                      gate_kind="head")], pos)[0]
        return torch.matmul(og, w.o.t())

    def _latent_attention(self, run: int, li: int, h: Tensor, pos: Tensor, params, seq: SequenceState) -> Tensor:
        sh, m, w = self.shape, self.shape.layers[li].mixer, self.lw[li]
        T, H, D, R, C, V, Q = h.shape[0], m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim, m.q_rank
        ap = params.attention_params[sh.run_plane[run]]
        cache = ap.kv_cache.key_cache                                         # [n_blocks, block_size, 1, row]
        proj = torch.matmul(h, w.w_in.t())                                    # [T, q latent | kv latent | rotated key part | gate]
        cq = latent_norm_cache(proj, 0, Q, Q, C, w.dq_norm, w.dkv_norm, sh.norm_eps, ap.new_cache_slots, cache)
        q = torch.matmul(cq, w.uq.t())                                        # [T, H * (plain | rotated)]
        if R:
            rotary_parts([
                RotaryPart(q, H, D + R, w.freq, rot_off=D, layout="interleaved", mag=w.mag, dst=q),
                RotaryPart(proj[:, Q + C:Q + C + R], 1, R, w.freq, layout="interleaved", mag=w.mag, cache=cache, cache_col=C),
            ], pos, ap.new_cache_slots)
        q_lat = torch.bmm(q.view(T, H, D + R).transpose(0, 1), w.uk)          # [H, T, C + R]: the queries in the cached rows' space
        o_lat = torch.empty_like(q_lat)
        latent_attention(q_lat.transpose(0, 1), cache, seq.tok_seq, pos, ap.q_cu_seq_lens, ap.block_tables, ap.cu_blocks_lens,
                         m.scale, m.window, ap.q_max_seq_len, out=o_lat.transpose(0, 1), max_kv_len=ap.kv_max_seq_len, sinks=w.sink)
        o = torch.bmm(o_lat, w.uv_t)                                          # [H, T, V]
        og = gated_group_norm(o.transpose(0, 1).reshape(T, H * V), self.dtype, gate=proj[:, Q + C + R:], gate_act="sigmoid")
        return torch.matmul(og, w.o.t())

    def _experts(self, li: int, h: Tensor) -> Tensor:
        f, w = self.shape.layers[li].mlp, self.lw[li]
        T = h.shape[0]
        logits = torch.matmul(h.float(), w.router)                            # the router in float
        weights, experts = route_softmax_topk(logits, f.experts + f.identity, f.top, 1.0, w.correction, renorm=False)
        seg, row_of, src = moe_plan(experts, f.experts)                       # (a choice of an identity expert gets no row)
        gu = grouped_linear(h, w.gate_up, seg, T * f.top, src=src)            # [rows, gate | up]
        y = grouped_linear(clamped_glu(gu[:, :f.ff], gu[:, f.ff:], 0.0, 1.0, 0.0), w.down, seg, T * f.top)
        return moe_combine(y, row_of, weights, identity=h)

    # ------------------------------------------------------------------ forward
    def forward_hidden(self, input_ids: Tensor, position_ids: Tensor, model_params) -> Tensor:
        """The normed output [n_selected, width] of model_params.selected_token_ids (all rows if None).  Every token's keys,
        values and latents go to the cache and every sequence's state slot is brought up to date."""
        sh, dt = self.shape, self.dtype
        if input_ids.dtype not in (torch.int32, torch.int64):
            raise ValueError("Pemalorn takes token ids")
        if position_ids.dtype != torch.int32:
            position_ids = position_ids.to(torch.int32)
        input_ids, pos = input_ids.contiguous(), position_ids.contiguous()
        q_cu = model_params.attention_params[0].q_cu_seq_lens
        seq = model_params.sequence_state
        if seq is None:
            if self.state_spec() is not None:
                raise ValueError("Pemalorn with input convolutions needs LanguageModelParameters.sequence_state (the batch's "
                                 "sequences and their state slots)")
            tok_seq = torch.repeat_interleave(torch.arange(q_cu.numel() - 1, device=q_cu.device), q_cu.diff().long(),
                                              output_size=input_ids.shape[0]).to(torch.int32)
            seq = SequenceState(None, None, tok_seq)
        T, W, eps = input_ids.shape[0], sh.hidden_size, sh.norm_eps
        x = stream_embed(input_ids, self.embed_table, 1.0, 1).view(T, W)      # the residual, float
        side = torch.nn.functional.embedding(input_ids, self.side_table) if self.side_table is not None else None
        xcat = None
        if sh.has_loop:
            # [x | x0] as the operand of every pass's input product; the embedding's half is written once
            xcat = torch.empty((T, 2 * W), dtype=dt, device=self.device)
            depth_norm(x, dt, eps, cast_out=xcat[:, W:])
        sel = model_params.selected_token_ids
        rows = sel.to(torch.int32).contiguous() if sel is not None and self.layer_trace is None else None
        n_runs = len(sh.runs)

        def enter(run: int, y=None, post_w=None, post=None, y2=None):
            """What stands between layer runs: results y (normed as `post` says, weighted) and y2 join the residual, then the
            next run's first norm — behind a pass's input product when the run starts one — or, after the last run, the
            final norm of the selected rows."""
            if run == n_runs:
                return depth_norm(x, dt, eps, y=y, post_w=post_w, post_norm=post, y2=y2, x_out=None if rows is not None else x,
                                  next_w=self.final_norm, rows=rows)
            li, t, first = sh.runs[run]
            if not first:
                return depth_norm(x, dt, eps, y=y, post_w=post_w, post_norm=post, y2=y2, x_out=x if y is not None else None,
                                  next_w=self.lw[li].norm1)
            depth_norm(x, dt, eps, y=y, post_w=post_w, post_norm=post, y2=y2, cast_out=xcat[:, :W])
            z = torch.matmul(xcat, self.loop_in.t())
            return depth_norm(None, dt, eps, y=z, post_norm="plain", bias=self.loop_step[t], x_out=x, next_w=self.lw[li].norm1)

        h = enter(0)
        for run, (li, _, _) in enumerate(sh.runs):
            l, w = sh.layers[li], self.lw[li]
            h1, h2 = h, h
            if w.canon1 is not None:
                h1, h2 = causal_conv_pair(h, w.canon1, w.canon2 if l.mlp is not None else None, seq, sh.state_piece(run), q_cu, pos)
                if h2 is None:
                    h2 = h
            mixer = self._attention if l.mixer.type == "attention" else self._latent_attention
            y = mixer(run, li, h1, pos, model_params, seq)
            y2 = self._experts(li, h2) if l.mlp is not None else None
            if w.has_side:
                # both sublayers join the residual, which the token input's gate reads as a matrix operand
                xb = torch.empty((T, W), dtype=dt, device=self.device)
                depth_norm(x, dt, eps, y=y, post_norm="plain", y2=y2, x_out=x, cast_out=xb)
                e = side[:, li * sh.side_dim:(li + 1) * sh.side_dim]
                y = torch.matmul(gelu_tanh_and_mul(torch.matmul(xb, w.side_gate.t()), e), w.side_proj.t())
                post_w, post, y2 = w.side_norm, "rms", None
            else:
                post_w, post = None, "plain"
            if self.layer_trace is None:
                h = enter(run + 1, y, post_w, post, y2)
            else:
                depth_norm(x, dt, eps, y=y, post_w=post_w, post_norm=post, y2=y2, x_out=x)
                self.layer_trace.append(x.clone())
                h = enter(run + 1)
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


def read_shape(model_path: str) -> PemalornShape:
    with open(os.path.join(model_path, "config.json")) as f:
        return PemalornShape.from_config(json.load(f))
