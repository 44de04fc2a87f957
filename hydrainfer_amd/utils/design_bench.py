"""`bench.py --design tetepel|kezolix|fasanex|pemalorn`: prefill and decode throughput of a model design at sizes that resemble a real
model's layers (random weights, a few layers), beside the Llama decoder at equal width / feed-forward / heads (Fasanex:
also beside Kezolix, the closest design), and a table of the design's own kernels against the like kernels of the models
beside it, each as a fraction of its roofline (HBM bytes or MFMA flops, algorithmic counts).  All models run their eager
step (no captured graph / launch plan) on hand-built batches."""
import math
import time
from typing import Callable, Dict, List

import torch

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0

SIZES = {
    # width, ff, heads, head dim, latent (kv_rank), query latent, window, streams, norm groups, layers
    "w2048": dict(width=2048, ff=5632, heads=16, dim=128, kv_rank=256, q_rank=768, window=2048, streams=4, groups=8, layers=4),
    "w4096": dict(width=4096, ff=11008, heads=32, dim=128, kv_rank=512, q_rank=1536, window=4096, streams=4, groups=8, layers=4),
}
VOCAB = 32064


def _tetepel(size: dict, dtype, dev):
    from hydrainfer_amd.model.tetepel import LatentAttentionSpec, TetepelForCausalLM, TetepelLayer, TetepelShape
    m = LatentAttentionSpec(size["heads"], size["dim"], size["dim"], size["kv_rank"], size["q_rank"],
                            1.0 / math.sqrt(size["dim"]), size["window"])
    shape = TetepelShape(VOCAB, size["width"], [TetepelLayer("latent_attention", m, size["ff"]) for _ in range(size["layers"])],
                         norm_groups=size["groups"], streams=size["streams"], embedding_scale=1.0)
    return TetepelForCausalLM.random_init(shape, dtype, dev, seed=0)


def _kezolix(size: dict, dtype, dev):
    """Four layers: recurrent + dense, attention + experts, recurrent + experts, attention on the second layer's keys +
    experts.  Attention as wide as the Llama decoder's (a quarter of the heads carry keys), chunks of 512; the recurrent
    layers keep a 128 x 128 state per head; 16 experts of a quarter of the dense inner size, four a token, and a shared one."""
    from hydrainfer_amd.model.kezolix import FeedForwardSpec, KezolixForCausalLM, KezolixLayer, KezolixShape, MixerSpec
    H, D, ff = size["heads"], size["dim"], size["ff"]
    att = lambda kv_from: MixerSpec("attention", H, D, D, H // 4, 1.0 / math.sqrt(D), 512, kv_from)
    rec = MixerSpec("hgrn2", H, D, D)
    moe = FeedForwardSpec("moe", ff // 4 // 32 * 32, 16, 4, 1.0, ff // 4 // 32 * 32)
    layers = [KezolixLayer(rec, FeedForwardSpec("dense", ff)), KezolixLayer(att(None), moe), KezolixLayer(rec, moe),
              KezolixLayer(att(1), moe)][:size["layers"]]
    shape = KezolixShape(VOCAB, size["width"], layers, max_position_embeddings=8192, norm_eps=1e-5, residual_mult=0.5)
    return KezolixForCausalLM.random_init(shape, dtype, dev, seed=0)


def _fasanex(size: dict, dtype, dev):
    """Four layers, a dense feed-forward each: state-space (heads of 64 channels over the model's width, a 128 x 64 state
    each, 8 groups, 4 taps), attention beside time mixing (attention as wide as the Llama decoder's with a quarter of the
    heads carrying keys, a window of 512, half of every head turning; time mixing heads of 64), the delta rule (128 x 128
    states, half of the heads carrying queries and keys), and the parallel mixer once more."""
    from hydrainfer_amd.model.fasanex import (AttentionSpec, FasanexForCausalLM, FasanexLayer, FasanexShape, FeedForwardSpec, MixerSpec,
                                              RotarySpec, TimeMixSpec)
    H, D, ff, W = size["heads"], size["dim"], size["ff"], size["width"]
    ssm = MixerSpec("mamba2", heads=W // 64, vdim=64, conv=4, state=128, groups=8, norm_groups=1)
    par = MixerSpec("parallel", left=AttentionSpec(H, H // 4, D, D, 3, 1.0 / math.sqrt(D), 30.0, 512, RotarySpec(D // 2, 10000.0, 8.0, 4096.0, 32.0, 1.0)),
                    right=TimeMixSpec(H, 64, 64), left_scale=1.0, right_scale=1.0)
    dl = MixerSpec("delta", heads=H, vdim=D, conv=4, dim=D, kv_heads=H // 2)
    layers = [FasanexLayer(m, FeedForwardSpec(ff, 7.0)) for m in (ssm, par, dl, par)][:size["layers"]]
    shape = FasanexShape(VOCAB, W, layers, norm_eps=1e-5, embedding_scale=1.0)
    return FasanexForCausalLM.random_init(shape, dtype, dev, seed=0)


def _pemalorn_sizes(size: dict) -> dict:
    """Attention as wide as the Llama decoder's, a quarter of the heads carrying keys, half of every head turning; latent
    attention with the size's latents, 64 rotated channels beside them (a cached row of at most 512 columns keeps the
    matrix-core form) and a window of 512; 16 experts of a quarter of the dense inner size, four a token, two identity
    experts; four taps; 64 channels of per-layer token input."""
    H, D = size["heads"], size["dim"]
    return dict(H=H, G=H // 4, D=D, V=D, rot=D // 2, R=64, C=min(size["kv_rank"], 512 - 64), Q=size["q_rank"], window=512,
                E=16, I=2, top=4, eff=size["ff"] // 4 // 32 * 32, taps=4, side=64)


def _pemalorn(size: dict, dtype, dev):
    """Four layers — attention, latent attention, attention, latent attention, a mixture of experts beside each — the two
    in the middle entered through the loop's input product (one pass)."""
    from hydrainfer_amd.layer.rotary_spec import RotarySpec
    from hydrainfer_amd.model.pemalorn import ExpertsSpec, MixerSpec, PemalornForCausalLM, PemalornLayer, PemalornShape
    z = _pemalorn_sizes(size)
    att = MixerSpec("attention", heads=z["H"], dim=z["D"], vdim=z["V"], scale=1.0 / math.sqrt(z["D"]), kv_heads=z["G"],
                    rot=RotarySpec(z["rot"], 10000.0))
    lat = MixerSpec("latent_attention", heads=z["H"], dim=z["D"], vdim=z["V"], scale=1.0 / math.sqrt(z["D"] + z["R"]), kv_rank=z["C"],
                    q_rank=z["Q"], rot_dim=z["R"], window=z["window"], rot=RotarySpec(z["R"], 10000.0, 4.0, 4096.0, 32.0, 1.0))
    moe = ExpertsSpec(z["E"], z["I"], z["top"], z["eff"])
    layers = [PemalornLayer(m, moe) for m in (att, lat, att, lat)][:size["layers"]]
    shape = PemalornShape(VOCAB, size["width"], layers, norm_eps=1e-5, taps=z["taps"], side_dim=z["side"], loop_start=1,
                          loop_stop=min(3, len(layers)), loop_times=1, has_loop=len(layers) > 1)
    return PemalornForCausalLM.random_init(shape, dtype, dev, seed=0)


def _llama(size: dict, dtype, dev):
    from hydrainfer_amd.model.llama import LlamaForCausalLM, LlamaShape
    shape = LlamaShape(size["width"], size["ff"], size["layers"], size["heads"], size["heads"], size["dim"], VOCAB)
    return LlamaForCausalLM.random_init(shape, dtype, dev, seed=0)


def _batch(model, n_seqs: int, q_len: int, kv_len: int, dtype, dev):
    """(ids, positions, LanguageModelParameters) of n_seqs sequences that feed their last q_len of kv_len tokens."""
    from hydrainfer_amd.layer.causal_attention import AttentionParametersBuilder
    from hydrainfer_amd.memory.kv_cache import KVCache
    from hydrainfer_amd.model.llama import LanguageModelParameters
    sh = model.shape
    bs, nb = 16, (kv_len + 15) // 16
    b = AttentionParametersBuilder(sh.num_attention_heads, sh.num_key_value_heads, sh.head_dim, bs, dev)
    for s in range(n_seqs):
        table = list(range(s * nb, (s + 1) * nb))
        b.add_request(q_len, kv_len, [table[p // bs] * bs + p % bs for p in range(kv_len - q_len, kv_len)], table)
    spec = model.cache_spec() if hasattr(model, "cache_spec") else {
        "n_layers": sh.num_hidden_layers, "n_tokens": 2, "n_heads": sh.num_key_value_heads, "head_size": sh.head_dim}
    for _ in range(spec["n_layers"]):
        k = torch.randn((n_seqs * nb, bs, spec["n_heads"], spec["head_size"]), device=dev).to(dtype)
        b.add_kv_cache(KVCache(k, k if spec["n_tokens"] == 1 else torch.randn_like(k)))
    ap = b.build_attention_parameters()
    pos = torch.arange(kv_len - q_len, kv_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    sel = torch.arange(q_len - 1, n_seqs * q_len, q_len, device=dev)
    params = LanguageModelParameters(ap, q_len == 1, sel)
    sspec = model.state_spec() if hasattr(model, "state_spec") else None
    if sspec is not None:
        from hydrainfer_amd._C.kernel.stream_ops import SequenceState
        state = torch.zeros((n_seqs, sspec["rows"], sspec["width"]), dtype=torch.float32, device=dev)
        params.sequence_state = SequenceState(state, torch.arange(n_seqs, dtype=torch.int32, device=dev),
                                              torch.arange(n_seqs, dtype=torch.int32, device=dev).repeat_interleave(q_len))
    ids = torch.randint(0, VOCAB, (n_seqs * q_len,), device=dev, dtype=torch.int32)
    return ids, pos, params


# the models a design's throughput is set beside: the closest existing one first
BESIDE = {"fasanex": ("kezolix", "llama"), "pemalorn": ("kezolix", "tetepel", "llama")}


def _time_eager(fn: Callable, dev, reps: int = 5, warm: int = 2) -> float:
    for _ in range(warm):
        fn()
    torch.cuda.synchronize(dev)
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize(dev)
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def _time_graph(fn: Callable, dev, launches: int = 10, reps: int = 3) -> float:
    """Microseconds per launch: a hipGraph of `launches` launches, mean of `reps` replays, HIP events."""
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(launches):
            fn()
    graph.replay()
    torch.cuda.synchronize(dev)
    ts = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); graph.replay(); e1.record()
        torch.cuda.synchronize(dev)
        ts.append(e0.elapsed_time(e1) / launches * 1e3)
    return sum(ts) / len(ts)


def _row(name, us, nbytes=None, flops=None):
    r = {"kernel": name, "us": round(us, 2)}
    if nbytes is not None:
        r.update(bound="hbm", achieved_GBps=round(nbytes / us / 1e3, 1), frac=round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4))
    else:
        r.update(bound="mfma", achieved_TFLOPs=round(flops / us / 1e6, 1), frac=round(flops / us / 1e6 / MFMA_PEAK_TFLOPS, 4))
    return r


def throughput(size_name: str, dtype, dev, prefill=(4, 1024), decode=(32, 1024), design: str = "tetepel") -> dict:
    size = SIZES[size_name]
    out = {}
    makers = {"tetepel": _tetepel, "kezolix": _kezolix, "fasanex": _fasanex, "pemalorn": _pemalorn, "llama": _llama}
    beside = BESIDE.get(design, ("llama",))
    for name, make in [(n, makers[n]) for n in (design,) + beside]:
        model = make(size, dtype, dev)
        if name == "llama":
            model.prepare_decode(max_rows=decode[0])
        with torch.inference_mode():
            ids, pos, params = _batch(model, prefill[0], prefill[1], prefill[1], dtype, dev)
            tp = _time_eager(lambda: model(ids, pos, params), dev)
            ids, pos, params = _batch(model, decode[0], 1, decode[1], dtype, dev)
            td = _time_eager(lambda: model(ids, pos, params), dev, reps=9, warm=3)
        out[name] = {"prefill_tok_s": round(prefill[0] * prefill[1] / tp, 1), "prefill_ms": round(tp * 1e3, 3),
                     "decode_tok_s": round(decode[0] / td, 1), "decode_step_ms": round(td * 1e3, 3),
                     "weight_GB": round(model.weight_bytes() / 1e9, 3)}
        del model, params
        torch.cuda.empty_cache()
    out["workload"] = {"prefill": f"{prefill[0]} x {prefill[1]} tokens", "decode": f"{decode[0]} sequences at {decode[1]} keys",
                       "layers": size["layers"], "size": size}
    return out


def kernel_table(size_name: str, dtype, dev, T: int = 4096, n_seqs: int = 4, B: int = 32, ctx: int = 2048) -> dict:
    """Every kernel of the design at a prefill batch of T tokens (n_seqs portions) — the attention also at a decode batch
    of B sequences with ctx keys — and the Llama path's like kernels at the same sizes."""
    from hydrainfer_amd._C.kernel import stream_ops as so
    from hydrainfer_amd._C.kernel.activation import silu_and_mul
    from hydrainfer_amd._C.kernel.flash_attn import mha_varlen_fwd
    from hydrainfer_amd._C.kernel.latent_attn import latent_attention, latent_norm_cache
    from hydrainfer_amd._C.kernel.norm import add_rms_norm
    from hydrainfer_amd._C.kernel.position_embedding import rope_set_kv_cache
    sz = SIZES[size_name]
    W, S, ff, H, D, R, QR, win = sz["width"], sz["streams"], sz["ff"], sz["heads"], sz["dim"], sz["kv_rank"], sz["q_rank"], sz["window"]
    e = 2
    rnd = lambda *s: torch.randn(s, device=dev).to(dtype)
    f32 = lambda *s: torch.randn(s, device=dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev) if not torch.is_tensor(v) else v.to(torch.int32).to(dev)
    rows: Dict[str, List[dict]] = {"tetepel": [], "llama": []}
    q_len = T // n_seqs
    q_cu = i32(list(range(0, T + 1, q_len)))
    pos = torch.arange(q_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    tok_seq = torch.arange(n_seqs, dtype=torch.int32, device=dev).repeat_interleave(q_len)
    x, y, gp = f32(T, S, W), rnd(T, W), rnd(T, W)
    seq = so.SequenceState(torch.zeros((n_seqs, 1, W), device=dev), i32(list(range(n_seqs))), tok_seq)
    in_w, nw, shw, gb, mix, ow = f32(S), f32(W), f32(W), f32(W), f32(S, S), f32(S)
    us = _time_graph(lambda: so.stream_norm(x, in_w, nw, sz["groups"], 1e-6, dtype, shift_w=shw, seq=seq, q_cu=q_cu, positions=pos), dev)
    rows["tetepel"].append(_row("stream_norm + token shift (reads S streams, writes h and hs)", us, T * W * (4 * S + 2 * e)))
    us = _time_graph(lambda: so.stream_norm(x, in_w, nw, sz["groups"], 1e-6, dtype), dev)
    rows["tetepel"].append(_row("stream_norm (feed-forward side)", us, T * W * (4 * S + e)))
    us = _time_graph(lambda: so.stream_update(x, y, mix, ow, gp, gb), dev)
    rows["tetepel"].append(_row("stream_update (gated result into S streams)", us, T * W * (8 * S + 2 * e)))
    gu = rnd(T, 2 * ff)
    us = _time_graph(lambda: so.gelu_tanh_and_mul(gu[:, :ff], gu[:, ff:]), dev)
    rows["tetepel"].append(_row("gelu_tanh_and_mul", us, 3 * T * ff * e))
    nb = (q_len + 15) // 16
    cache = rnd(n_seqs * nb, 16, 1, R)
    table, cu_b = i32(torch.randperm(n_seqs * nb)), i32(list(range(0, n_seqs * nb + 1, nb)))
    slots = i32([int(table[s * nb + p // 16]) * 16 + p % 16 for s in range(n_seqs) for p in range(q_len)])
    proj = rnd(T, QR + R + H)
    qw, kw = f32(QR), f32(R)
    us = _time_graph(lambda: latent_norm_cache(proj, 0, QR, QR, R, qw, kw, 1e-6, slots, cache), dev)
    rows["tetepel"].append(_row("latent_norm_cache (two norms + cache append)", us, 2 * T * (QR + R) * e))
    ql = rnd(T, H, R)
    seen = n_seqs * sum(min(i + 1, win) for i in range(q_len))
    us = _time_graph(lambda: latent_attention(ql, cache, tok_seq, pos, q_cu, table, cu_b, 1 / math.sqrt(D), win, q_len, gate_pre=proj[:, QR + R:], max_kv_len=q_len), dev, launches=4)
    rows["tetepel"].append(_row(f"latent_attention, prefill {n_seqs} x {q_len} (MFMA tile form, latent {R})", us, flops=4 * H * R * seen))
    # decode: B sequences, one token each, ctx keys
    nbd = (ctx + 15) // 16
    cache_d = rnd(B * nbd, 16, 1, R)
    table_d, cu_bd = i32(torch.randperm(B * nbd)), i32(list(range(0, B * nbd + 1, nbd)))
    qd, posd, seqd, qcud = rnd(B, H, R), i32([ctx - 1] * B), i32(list(range(B))), i32(list(range(B + 1)))
    us = _time_graph(lambda: latent_attention(qd, cache_d, seqd, posd, qcud, table_d, cu_bd, 1 / math.sqrt(D), win, 1, max_kv_len=ctx), dev)
    rows["tetepel"].append(_row(f"latent_attention, decode {B} x {min(ctx, win)} keys", us, B * min(ctx, win) * R * e + 2 * B * H * R * e))

    # ---- the Llama path's like kernels
    res, xx, out, w16 = rnd(T, W), rnd(T, W), rnd(T, W), rnd(W)
    us = _time_graph(lambda: add_rms_norm(out, res, xx, w16, 1e-6), dev)
    rows["llama"].append(_row("add_rms_norm (residual add + norm)", us, 4 * T * W * e))
    us = _time_graph(lambda: silu_and_mul(gu[:, :ff], gu[:, ff:]), dev)
    rows["llama"].append(_row("silu_and_mul", us, 3 * T * ff * e))
    q, k, v = rnd(T, H, D), rnd(T, H, D), rnd(T, H, D)
    kc, vc = rnd(n_seqs * nb, 16, H, D), rnd(n_seqs * nb, 16, H, D)
    cos_sin = rnd(max(q_len, ctx), 2, D // 2)
    us = _time_graph(lambda: rope_set_kv_cache(q, k, v, pos, cos_sin, D, slots, kc, vc), dev)
    rows["llama"].append(_row("rope_set_kv_cache (rotary + cache append)", us, (2 * 2 * T * H * D + 2 * T * H * D) * e))
    o = torch.empty_like(q)
    cu_k = q_cu
    us = _time_graph(lambda: mha_varlen_fwd(o, q, kc, vc, q_cu, cu_k, table, cu_b, None, q_len, q_len, 1 / math.sqrt(D), 0, -1, 0, 0), dev, launches=4)
    rows["llama"].append(_row(f"mha_varlen_fwd, prefill {n_seqs} x {q_len} (causal, head_dim {D})", us,
                              flops=4 * H * D * n_seqs * sum(i + 1 for i in range(q_len))))
    kcd, vcd = rnd(B * nbd, 16, H, D), rnd(B * nbd, 16, H, D)
    qd2, od2 = rnd(B, H, D), rnd(B, H, D)
    cu_kd = i32(list(range(0, B * ctx + 1, ctx)))
    us = _time_graph(lambda: mha_varlen_fwd(od2, qd2, kcd, vcd, qcud, cu_kd, table_d, cu_bd, None, 1, ctx, 1 / math.sqrt(D), 0, -1, 0, 0), dev)
    rows["llama"].append(_row(f"mha_varlen_fwd, decode {B} x {ctx} keys", us, 2 * B * ctx * H * D * e + 2 * B * H * D * e))
    rows["workload"] = {"prefill_tokens": T, "portions": n_seqs, "decode_batch": B, "decode_keys": ctx, "size": sz,
                        "timing": "hipGraph of 10 (attention prefill: 4) launches, mean of 3 replays, HIP events",
                        "roofline": f"HBM {HBM_PEAK_GBS} GB/s, MFMA {MFMA_PEAK_TFLOPS} TFLOP/s dense bf16; algorithmic bytes / flops"}
    return rows


def _llama_rows(size_name: str, dtype, dev, T: int, n_seqs: int, B: int, ctx: int) -> List[dict]:
    """The Llama path's kernels that the designs' kernels are set beside, at the same sizes."""
    from hydrainfer_amd._C.kernel.activation import silu_and_mul
    from hydrainfer_amd._C.kernel.flash_attn import mha_varlen_fwd
    from hydrainfer_amd._C.kernel.norm import add_rms_norm
    from hydrainfer_amd._C.kernel.position_embedding import rope_set_kv_cache
    sz = SIZES[size_name]
    W, ff, H, D = sz["width"], sz["ff"], sz["heads"], sz["dim"]
    e = 2
    rnd = lambda *s: torch.randn(s, device=dev).to(dtype)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev) if not torch.is_tensor(v) else v.to(torch.int32).to(dev)
    rows = []
    q_len = T // n_seqs
    nb, nbd = (q_len + 15) // 16, (ctx + 15) // 16
    q_cu = i32(list(range(0, T + 1, q_len)))
    pos = torch.arange(q_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    table, cu_b = i32(torch.randperm(n_seqs * nb)), i32(list(range(0, n_seqs * nb + 1, nb)))
    slots = i32([int(table[s * nb + p // 16]) * 16 + p % 16 for s in range(n_seqs) for p in range(q_len)])
    res, xx, out, w16, gu = rnd(T, W), rnd(T, W), rnd(T, W), rnd(W), rnd(T, 2 * ff)
    us = _time_graph(lambda: add_rms_norm(out, res, xx, w16, 1e-6), dev)
    rows.append(_row("add_rms_norm (residual add + norm)", us, 4 * T * W * e))
    us = _time_graph(lambda: silu_and_mul(gu[:, :ff], gu[:, ff:]), dev)
    rows.append(_row("silu_and_mul", us, 3 * T * ff * e))
    q, k, v = rnd(T, H, D), rnd(T, H, D), rnd(T, H, D)
    kc, vc = rnd(n_seqs * nb, 16, H, D), rnd(n_seqs * nb, 16, H, D)
    cos_sin = rnd(max(q_len, ctx), 2, D // 2)
    us = _time_graph(lambda: rope_set_kv_cache(q, k, v, pos, cos_sin, D, slots, kc, vc), dev)
    rows.append(_row("rope_set_kv_cache (rotary + cache append)", us, (2 * 2 * T * H * D + 2 * T * H * D) * e))
    o = torch.empty_like(q)
    us = _time_graph(lambda: mha_varlen_fwd(o, q, kc, vc, q_cu, q_cu, table, cu_b, None, q_len, q_len, 1 / math.sqrt(D), 0, -1, 0, 0), dev, launches=4)
    rows.append(_row(f"mha_varlen_fwd, prefill {n_seqs} x {q_len} (causal, head_dim {D})", us,
                     flops=4 * H * D * n_seqs * sum(i + 1 for i in range(q_len))))
    table_d, cu_bd = i32(torch.randperm(B * nbd)), i32(list(range(0, B * nbd + 1, nbd)))
    kcd, vcd = rnd(B * nbd, 16, H, D), rnd(B * nbd, 16, H, D)
    qd2, od2 = rnd(B, H, D), rnd(B, H, D)
    qcud, cu_kd = i32(list(range(B + 1))), i32(list(range(0, B * ctx + 1, ctx)))
    us = _time_graph(lambda: mha_varlen_fwd(od2, qd2, kcd, vcd, qcud, cu_kd, table_d, cu_bd, None, 1, ctx, 1 / math.sqrt(D), 0, -1, 0, 0), dev)
    rows.append(_row(f"mha_varlen_fwd, decode {B} x {ctx} keys", us, 2 * B * ctx * H * D * e + 2 * B * H * D * e))
    return rows


def kezolix_kernel_table(size_name: str, dtype, dev, T: int = 4096, n_seqs: int = 4, B: int = 32, ctx: int = 2048) -> dict:
    """Every kernel of the Kezolix design at a prefill batch of T tokens (n_seqs portions) — attention and recurrence also
    at a decode batch of B sequences — and the Llama path's like kernels at the same sizes."""
    from hydrainfer_amd._C.kernel import biased_attn as ba, depth_ops as do, moe_mix as mm
    from hydrainfer_amd._C.kernel.recurrence import gated_recurrence
    from hydrainfer_amd._C.kernel.stream_ops import SequenceState
    sz = SIZES[size_name]
    W, ff, H, D = sz["width"], sz["ff"], sz["heads"], sz["dim"]
    G, V, chunk, E, top, n_lv = H // 4, D, 512, 16, 4, 5
    eff = ff // 4 // 32 * 32
    e = 2
    rnd = lambda *s: torch.randn(s, device=dev).to(dtype)
    f32 = lambda *s: torch.randn(s, device=dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev) if not torch.is_tensor(v) else v.to(torch.int32).to(dev)
    rows: Dict[str, List[dict]] = {"kezolix": [], "llama": []}
    add = lambda *a, **k: rows["kezolix"].append(_row(*a, **k))
    q_len = T // n_seqs
    q_cu = i32(list(range(0, T + 1, q_len)))
    pos = torch.arange(q_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    tok_seq = torch.arange(n_seqs, dtype=torch.int32, device=dev).repeat_interleave(q_len)
    x, y, w1, w2 = f32(T, W), rnd(T, W), f32(W), f32(W)
    xo, levels, dw = torch.empty_like(x), f32(n_lv, T, W), f32(n_lv)
    us = _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_w=w1, mult=0.5, x_out=xo, next_w=w2), dev)
    add("depth_norm, mid-layer (norm of y into the residual + next norm)", us, T * W * (8 + 2 * e))
    us = _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_w=w1, mult=0.5, level_out=levels[n_lv - 1], levels=levels,
                                           depth_w=dw, x_out=xo, next_w=w2), dev)
    add(f"depth_norm, layer end (+ level written, average of {n_lv} levels)", us, T * W * (4 * (n_lv + 2) + 2 * e))
    z, coef = rnd(T, ff), f32(4)
    us = _time_graph(lambda: do.poly_norm(z, coef, 1e-5), dev)
    add("poly_norm", us, 2 * T * ff * e)
    # recurrence: prefill portions from position 0, then one token for B sequences
    proj = rnd(T, 3 * H * D)
    fb, low, nw = f32(H * D), torch.rand(H * D, device=dev), f32(V)
    state = torch.zeros((max(n_seqs, B), 1, H * D * V), device=dev)
    seq = SequenceState(state, i32(list(range(n_seqs))), tok_seq)
    us = _time_graph(lambda: gated_recurrence(proj[:, :H * D], proj[:, H * D:2 * H * D], proj[:, 2 * H * D:], fb, low, nw, 1e-5, seq, 0,
                                              q_cu, pos, H, D, V), dev, launches=2)
    add(f"gated_recurrence, prefill {n_seqs} x {q_len} ({H} heads, state {D} x {V})", us, flops=6 * T * H * D * V)
    posd, qcud = i32([ctx - 1] * B), i32(list(range(B + 1)))
    seqd = SequenceState(state, i32(list(range(B))), i32(list(range(B))))
    us = _time_graph(lambda: gated_recurrence(proj[:B, :H * D], proj[:B, H * D:2 * H * D], proj[:B, 2 * H * D:], fb, low, nw, 1e-5, seqd,
                                              0, qcud, posd, H, D, V, max_q_len=1), dev)
    add(f"gated_recurrence, decode {B} sequences (state read and written)", us, 2 * B * H * D * V * 4)
    # attention
    nb, nbd = (q_len + 15) // 16, (ctx + 15) // 16
    kc, vc = rnd(n_seqs * nb, 16, G, D), rnd(n_seqs * nb, 16, G, D)
    table, cu_b = i32(torch.randperm(n_seqs * nb)), i32(list(range(0, n_seqs * nb + 1, nb)))
    slots = i32([int(table[s * nb + p // 16]) * 16 + p % 16 for s in range(n_seqs) for p in range(q_len)])
    qkv, qw, kw = rnd(T, (H + 2 * G) * D), f32(H * D), f32(G * D)
    us = _time_graph(lambda: ba.qk_norm_cache(qkv, H * D, G * D, G * V, qw, kw, 1e-5, G, slots, kc, vc), dev)
    add("qk_norm_cache (two norms + cache append)", us, T * (2 * H * D + 2 * G * D + 2 * G * V) * e)
    q = rnd(T, H, D)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], device=dev)
    seen = n_seqs * sum(i % chunk + 1 for i in range(q_len))
    us = _time_graph(lambda: ba.biased_attention(q, kc, vc, V, tok_seq, pos, q_cu, table, cu_b, 1 / math.sqrt(D), slopes, "chunk", chunk,
                                                 max_q_len=q_len, max_kv_len=q_len), dev, launches=2)
    add(f"biased_attention, prefill {n_seqs} x {q_len} (chunks of {chunk}, head_dim {D})", us, flops=2 * H * (D + V) * seen)
    kcd, vcd = rnd(B * nbd, 16, G, D), rnd(B * nbd, 16, G, D)
    table_d, cu_bd = i32(torch.randperm(B * nbd)), i32(list(range(0, B * nbd + 1, nbd)))
    qd, seq_ids = rnd(B, H, D), i32(list(range(B)))
    keys = (ctx - 1) % chunk + 1
    us = _time_graph(lambda: ba.biased_attention(qd, kcd, vcd, V, seq_ids, posd, qcud, table_d, cu_bd, 1 / math.sqrt(D), slopes, "chunk",
                                                 chunk, max_q_len=1, max_kv_len=ctx), dev)
    add(f"biased_attention, decode {B} x {keys} keys of its chunk", us, 2 * B * keys * G * D * e + 2 * B * H * D * e)
    posd2 = i32([ctx - 1] * B)
    us = _time_graph(lambda: ba.biased_attention(qd, kcd, vcd, V, seq_ids, posd2, qcud, table_d, cu_bd, 1 / math.sqrt(D), slopes, "causal",
                                                 0, max_q_len=1, max_kv_len=ctx), dev)
    add(f"biased_attention, decode {B} x {ctx} keys (causal mask)", us, 2 * B * ctx * G * D * e + 2 * B * H * D * e)
    # experts
    logits, corr = f32(T, E + 1), f32(E) * 0.01
    us = _time_graph(lambda: mm.route_softmax_topk(logits, E, top, 1.0, corr), dev)
    add(f"route_softmax_topk ({E} experts, top {top})", us, T * (E + 1 + 2 * top) * 4)
    wts, idx = mm.route_softmax_topk(logits, E, top, 1.0, corr)
    us = _time_graph(lambda: mm.moe_plan(idx, E), dev)
    add("moe_plan (one workgroup)", us, 3 * T * top * 4)
    seg, row_of, src = mm.moe_plan(idx, E)
    h, up, down = rnd(T, W), rnd(E, eff, W) / math.sqrt(W), rnd(E, W, eff) / math.sqrt(eff)
    us = _time_graph(lambda: mm.grouped_linear(h, up, seg, T * top, src=src, act="relu2"), dev, launches=2)
    add(f"grouped_linear up + squared ReLU ({T * top} rows, {W} -> {eff})", us, flops=2 * T * top * W * eff)
    y1 = mm.grouped_linear(h, up, seg, T * top, src=src, act="relu2")
    us = _time_graph(lambda: mm.grouped_linear(y1, down, seg, T * top), dev, launches=2)
    add(f"grouped_linear down ({T * top} rows, {eff} -> {W})", us, flops=2 * T * top * W * eff)
    y2, shared = mm.grouped_linear(y1, down, seg, T * top), rnd(T, W)
    us = _time_graph(lambda: mm.moe_combine(y2, row_of, wts, shared, logits[:, E:]), dev)
    add("moe_combine (+ gated shared expert)", us, T * W * (top + 2) * e)
    # decode-sized expert products: B tokens, weights of the chosen experts stream once
    hd = rnd(B, W)
    wd, idd = mm.route_softmax_topk(logits[:B].contiguous(), E, top, 1.0, corr)
    segd, rowd, srcd = mm.moe_plan(idd, E)
    us = _time_graph(lambda: mm.grouped_linear(hd, up, segd, B * top, src=srcd, act="relu2"), dev)
    used = int(torch.unique(idd).numel())
    add(f"grouped_linear up, decode ({B} tokens, {used} experts' weights)", us, used * eff * W * e)
    rows["llama"] = _llama_rows(size_name, dtype, dev, T, n_seqs, B, ctx)
    a = rnd(T * top, W)
    bw = rnd(eff, W)
    us = _time_graph(lambda: torch.matmul(a, bw.t()), dev, launches=2)
    rows["llama"].append(_row(f"library GEMM of the expert products' size ({T * top} x {W} -> {eff})", us, flops=2 * T * top * W * eff))
    rows["workload"] = {"prefill_tokens": T, "portions": n_seqs, "decode_batch": B, "decode_keys": ctx, "size": sz,
                        "timing": "hipGraph of 10 (long kernels: 2) launches, mean of 3 replays, HIP events",
                        "roofline": f"HBM {HBM_PEAK_GBS} GB/s, MFMA {MFMA_PEAK_TFLOPS} TFLOP/s dense bf16; algorithmic bytes / flops"}
    return rows


def fasanex_kernel_table(size_name: str, dtype, dev, T: int = 4096, n_seqs: int = 4, B: int = 32, ctx: int = 2048) -> dict:
    """Every kernel of the Fasanex design at a prefill batch of T tokens (n_seqs portions) — attention and the scans also at
    a decode batch of B sequences — beside the like kernels of the closest design (Kezolix: recurrent / attention hybrid)
    and of the Llama path at the same sizes."""
    from hydrainfer_amd._C.kernel import biased_attn as ba, depth_ops as do, seq_mix as sm
    from hydrainfer_amd._C.kernel.recurrence import gated_recurrence
    from hydrainfer_amd._C.kernel.stream_ops import SequenceState
    from hydrainfer_amd.model.fasanex import RotarySpec
    sz = SIZES[size_name]
    W, ff, H, D = sz["width"], sz["ff"], sz["heads"], sz["dim"]
    G, window = H // 4, 512
    e = 2
    rnd = lambda *s: torch.randn(s, device=dev).to(dtype)
    f32 = lambda *s: torch.randn(s, device=dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev) if not torch.is_tensor(v) else v.to(torch.int32).to(dev)
    rows: Dict[str, List[dict]] = {"fasanex": [], "kezolix": [], "llama": []}
    add = lambda *a, **k: rows["fasanex"].append(_row(*a, **k))
    kez = lambda *a, **k: rows["kezolix"].append(_row(*a, **k))
    q_len = T // n_seqs
    q_cu = i32(list(range(0, T + 1, q_len)))
    pos = torch.arange(q_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    tok_seq = torch.arange(n_seqs, dtype=torch.int32, device=dev).repeat_interleave(q_len)
    posd, qcud, seq_ids = i32([ctx - 1] * B), i32(list(range(B + 1))), i32(list(range(B)))
    # residual + norms: the kernel both designs share
    x, y, w1, w2 = f32(T, W), rnd(T, W), f32(W), f32(W)
    us = _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_w=w1, x_out=x, next_w=w2, rms=True), dev)
    add("depth_norm (RMS norm of y into the residual + next norm)", us, T * W * (8 + 2 * e))
    kez("depth_norm, mid-layer (the same kernel, layer norms)", _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_w=w1, mult=0.5, x_out=x, next_w=w2), dev),
        T * W * (8 + 2 * e))
    gu, coef = rnd(T, 2 * ff), f32(4)
    us = _time_graph(lambda: sm.clamped_glu(gu[:, :ff], gu[:, ff:], 7.0), dev)
    add("clamped_glu", us, 3 * T * ff * e)
    kez("poly_norm", _time_graph(lambda: do.poly_norm(gu[:, :ff], coef, 1e-5), dev), 2 * T * ff * e)
    # state pieces of one slot: [conv tail | shift | S]
    n_slots = max(n_seqs, B)
    inner, gn, N, P = W, 8 * 128, 128, 64
    C = inner + 2 * gn
    state = torch.zeros((n_slots, 1, 3 * C + W + H * D * D), device=dev)
    seq = SequenceState(state, i32(list(range(n_seqs))), tok_seq)
    seqd = SequenceState(state, seq_ids, seq_ids)
    off_S = 3 * C + W
    proj = rnd(T, 2 * inner + 2 * gn + inner // P)
    cw, cb = f32(C, 4), f32(C)
    us = _time_graph(lambda: sm.causal_conv(proj[:, inner:inner + C], cw, cb, "silu", seq, 0, q_cu, pos), dev)
    add(f"causal_conv + bias + silu ({C} channels, 4 taps)", us, 2 * T * C * e)
    hh, mu = rnd(T, W), torch.rand(5, W, device=dev)
    us = _time_graph(lambda: sm.token_shift_mix(hh, mu, seq, 3 * C, q_cu, pos), dev)
    add("token_shift_mix (five mixes)", us, 6 * T * W * e)
    # attention side
    nb, nbd = (q_len + 15) // 16, (ctx + 15) // 16
    kc, vc = rnd(n_seqs * nb, 16, G, D), rnd(n_seqs * nb, 16, G, D)
    table, cu_b = i32(torch.randperm(n_seqs * nb)), i32(list(range(0, n_seqs * nb + 1, nb)))
    slots = i32([int(table[s * nb + p // 16]) * 16 + p % 16 for s in range(n_seqs) for p in range(q_len)])
    qk, qw, kw = rnd(T, (H + G) * D), f32(D), f32(D)
    freq, cs = RotarySpec(D // 2, 10000.0, 8.0, 4096.0, 32.0, 1.0).frequencies()
    inv = torch.tensor(freq, device=dev, dtype=torch.float32)
    us = _time_graph(lambda: sm.head_norm_rope_cache(qk[:, :H * D], qk[:, H * D:], qw, kw, 1e-5, H, G, D, inv, cs, pos, slots, kc, vc), dev)
    add("head_norm_rope_cache (head norms + rotation + cache append)", us, T * (2 * H * D + 3 * G * D) * e)
    qkv, qw2, kw2 = rnd(T, (H + 2 * G) * D), f32(H * D), f32(G * D)
    kez("qk_norm_cache (two norms + cache append)", _time_graph(lambda: ba.qk_norm_cache(qkv, H * D, G * D, G * D, qw2, kw2, 1e-5, G, slots, kc, vc), dev),
        T * (2 * H * D + 2 * G * D + 2 * G * D) * e)
    q = rnd(T, H, D)
    seen = n_seqs * sum(min(i + 1, window) for i in range(q_len))
    us = _time_graph(lambda: ba.biased_attention(q, kc, vc, D, tok_seq, pos, q_cu, table, cu_b, 1 / math.sqrt(D), None, "window", window,
                                                 max_q_len=q_len, max_kv_len=q_len, softcap=30.0), dev, launches=2)
    add(f"biased_attention, prefill {n_seqs} x {q_len} (window {window}, soft cap, head_dim {D})", us, flops=4 * H * D * seen)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], device=dev)
    seen_c = n_seqs * sum(i % window + 1 for i in range(q_len))
    kez(f"biased_attention, prefill {n_seqs} x {q_len} (chunks of {window}, distance bias)",
        _time_graph(lambda: ba.biased_attention(q, kc, vc, D, tok_seq, pos, q_cu, table, cu_b, 1 / math.sqrt(D), slopes, "chunk", window,
                                                max_q_len=q_len, max_kv_len=q_len), dev, launches=2), flops=4 * H * D * seen_c)
    kcd, vcd = rnd(B * nbd, 16, G, D), rnd(B * nbd, 16, G, D)
    table_d, cu_bd = i32(torch.randperm(B * nbd)), i32(list(range(0, B * nbd + 1, nbd)))
    qd = rnd(B, H, D)
    us = _time_graph(lambda: ba.biased_attention(qd, kcd, vcd, D, seq_ids, posd, qcud, table_d, cu_bd, 1 / math.sqrt(D), None, "window", window,
                                                 max_q_len=1, max_kv_len=ctx, softcap=30.0), dev)
    add(f"biased_attention, decode {B} x {window} keys of the window (soft cap)", us, 2 * B * window * G * D * e + 2 * B * H * D * e)
    pos_chunk_end = i32([window * (ctx // window) - 1] * B)
    kez(f"biased_attention, decode {B} x {window} keys of its chunk",
        _time_graph(lambda: ba.biased_attention(qd, kcd, vcd, D, seq_ids, pos_chunk_end, qcud, table_d, cu_bd,
                                                1 / math.sqrt(D), slopes, "chunk", window, max_q_len=1, max_kv_len=ctx), dev),
        2 * B * window * G * D * e + 2 * B * H * D * e)
    og, gate = rnd(T, H * D), rnd(T, H * D)
    both = rnd(T, H * D + 64)
    us = _time_graph(lambda: sm.gated_group_norm(og, dtype, gate=gate, gate_act="sigmoid", scale=0.8, out=both[:, :H * D]), dev)
    add("gated_group_norm: sigmoid gate on the attention's result", us, 3 * T * H * D * e)
    # the scans, each at a state of H x 128 x 128 floats a sequence (the state-space form: W / 64 heads of 128 x 64)
    Hs = inner // P
    xbc, dtr = rnd(T, C), rnd(T, Hs)
    rate, bias = f32(Hs) * 0.3, f32(Hs)
    us = _time_graph(lambda: sm.head_gates(dtr, rate, bias, want_step=True), dev)
    add("head_gates (decay and step size of every head)", us, T * Hs * (e + 8))
    decay, step, _ = sm.head_gates(dtr, rate, bias, want_step=True)
    flops_state = lambda n_tok, heads, k, v, per: per * n_tok * heads * k * v
    us = _time_graph(lambda: sm.state_scan("decay", xbc[:, inner + gn:], xbc[:, inner:inner + gn], xbc[:, :inner], decay, seq, off_S, q_cu, pos,
                                           Hs, 8, N, P, vscale=step), dev, launches=2)
    add(f"state_scan decay form, prefill {n_seqs} x {q_len} ({Hs} heads, state {N} x {P})", us, flops=flops_state(T, Hs, N, P, 5))
    us = _time_graph(lambda: sm.state_scan("decay", xbc[:B, inner + gn:], xbc[:B, inner:inner + gn], xbc[:B, :inner], decay[:B].contiguous(), seqd,
                                           off_S, qcud, posd, Hs, 8, N, P, vscale=step[:B].contiguous()), dev)
    add(f"state_scan decay form, decode {B} sequences (state read and written)", us, 2 * B * Hs * N * P * 4)
    Hr, Dr = H, 64
    rkv, dch, bonus = rnd(3, T, Hr * Dr), torch.rand(T, Hr * Dr, device=dev) * 0.5 + 0.5, f32(Hr * Dr)
    us = _time_graph(lambda: sm.decay_exp(rkv[0], bonus), dev)
    add("decay_exp (a decay per key channel)", us, T * Hr * Dr * (e + 4))
    us = _time_graph(lambda: sm.state_scan("bonus", rkv[0], rkv[1], rkv[2], dch, seq, off_S, q_cu, pos, Hr, Hr, Dr, Dr, bonus=bonus), dev, launches=2)
    add(f"state_scan bonus form, prefill {n_seqs} x {q_len} ({Hr} heads, state {Dr} x {Dr})", us, flops=flops_state(T, Hr, Dr, Dr, 7))
    us = _time_graph(lambda: sm.state_scan("bonus", rkv[0, :B], rkv[1, :B], rkv[2, :B], dch[:B].contiguous(), seqd, off_S, qcud, posd, Hr, Hr, Dr, Dr,
                                           bonus=bonus), dev)
    add(f"state_scan bonus form, decode {B} sequences", us, 2 * B * Hr * Dr * Dr * 4)
    Gd = H // 2
    cqkv = rnd(T, 2 * Gd * D + H * D)
    us = _time_graph(lambda: sm.unit_norm(cqkv[:, :Gd * D], Gd, D, 1e-6, D ** -0.5), dev)
    add("unit_norm (queries or keys of the delta rule)", us, T * Gd * D * (e + 4))
    qn, kn = sm.unit_norm(cqkv[:, :Gd * D], Gd, D, 1e-6, D ** -0.5), sm.unit_norm(cqkv[:, Gd * D:2 * Gd * D], Gd, D, 1e-6)
    ab = rnd(T, 2 * H)
    dec_d, _, beta = sm.head_gates(ab[:, H:], f32(H) * 0.3, f32(H), b=ab[:, :H])
    us = _time_graph(lambda: sm.state_scan("delta", qn, kn, cqkv[:, 2 * Gd * D:], dec_d, seq, off_S, q_cu, pos, H, Gd, D, D, beta=beta), dev, launches=2)
    add(f"state_scan delta form, prefill {n_seqs} x {q_len} ({H} heads, state {D} x {D})", us, flops=flops_state(T, H, D, D, 8))
    us = _time_graph(lambda: sm.state_scan("delta", qn[:B], kn[:B], cqkv[:B, 2 * Gd * D:], dec_d[:B].contiguous(), seqd, off_S, qcud, posd, H, Gd, D, D,
                                           beta=beta[:B].contiguous()), dev)
    add(f"state_scan delta form, decode {B} sequences (state read and written)", us, 2 * B * H * D * D * 4)
    o32, nw = f32(T, H * D), f32(D)
    us = _time_graph(lambda: sm.gated_group_norm(o32, dtype, group=D, eps=1e-5, w=nw, gate=gate, gate_act="silu"), dev)
    add("gated_group_norm: head norm + weight + silu gate after a scan", us, T * H * D * (4 + 2 * e))
    # the closest design's recurrence at the same state size
    pr = rnd(T, 3 * H * D)
    fb, low, nw2 = f32(H * D), torch.rand(H * D, device=dev), f32(D)
    st2 = torch.zeros((n_slots, 1, H * D * D), device=dev)
    sq2, sq2d = SequenceState(st2, i32(list(range(n_seqs))), tok_seq), SequenceState(st2, seq_ids, seq_ids)
    kez(f"gated_recurrence (scan + head norm), prefill {n_seqs} x {q_len} ({H} heads, state {D} x {D})",
        _time_graph(lambda: gated_recurrence(pr[:, :H * D], pr[:, H * D:2 * H * D], pr[:, 2 * H * D:], fb, low, nw2, 1e-5, sq2, 0, q_cu, pos, H, D, D), dev,
                    launches=2), flops=flops_state(T, H, D, D, 6))
    kez(f"gated_recurrence, decode {B} sequences (state read and written)",
        _time_graph(lambda: gated_recurrence(pr[:B, :H * D], pr[:B, H * D:2 * H * D], pr[:B, 2 * H * D:], fb, low, nw2, 1e-5, sq2d, 0, qcud, posd, H, D, D,
                                             max_q_len=1), dev), 2 * B * H * D * D * 4)
    rows["llama"] = _llama_rows(size_name, dtype, dev, T, n_seqs, B, ctx)
    rows["workload"] = {"prefill_tokens": T, "portions": n_seqs, "decode_batch": B, "decode_keys": ctx, "size": sz,
                        "timing": "hipGraph of 10 (long kernels: 2) launches, mean of 3 replays, HIP events",
                        "roofline": f"HBM {HBM_PEAK_GBS} GB/s, MFMA {MFMA_PEAK_TFLOPS} TFLOP/s dense bf16; algorithmic bytes / flops "
                                    "(the scans are float vector work: their flops are counted, not priced against the MFMA peak)"}
    return rows


def pemalorn_kernel_table(size_name: str, dtype, dev, T: int = 4096, n_seqs: int = 4, B: int = 32, ctx: int = 2048) -> dict:
    """Every kernel of the Pemalorn design at a prefill batch of T tokens (n_seqs portions) — the attentions also at a decode
    batch of B sequences — and beside them the tables of the two closest designs at the same sizes: Kezolix (grouped-query
    attention of the same kernel family, experts, the same residual kernel) and Tetepel (latent attention)."""
    from hydrainfer_amd._C.kernel import biased_attn as ba, depth_ops as do, moe_mix as mm
    from hydrainfer_amd._C.kernel.latent_attn import latent_attention, latent_norm_cache
    from hydrainfer_amd._C.kernel.rotary import RotaryPart, rotary_parts
    from hydrainfer_amd._C.kernel.seq_mix import causal_conv_pair, clamped_glu, gated_group_norm
    from hydrainfer_amd._C.kernel.stream_ops import SequenceState, gelu_tanh_and_mul
    from hydrainfer_amd.layer.rotary_spec import RotarySpec
    sz = SIZES[size_name]
    z = _pemalorn_sizes(sz)
    W, H, G, D, V, C, R, Q = sz["width"], z["H"], z["G"], z["D"], z["V"], z["C"], z["R"], z["Q"]
    E, I, top, eff, taps, side, win = z["E"], z["I"], z["top"], z["eff"], z["taps"], z["side"], z["window"]
    e = 2
    rnd = lambda *s: torch.randn(s, device=dev).to(dtype)
    f32 = lambda *s: torch.randn(s, device=dev)
    f64 = lambda v: torch.tensor(v, dtype=torch.float64, device=dev)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev) if not torch.is_tensor(v) else v.to(torch.int32).to(dev)
    rows: Dict[str, List[dict]] = {"pemalorn": []}
    add = lambda *a, **k: rows["pemalorn"].append(_row(*a, **k))
    q_len = T // n_seqs
    q_cu = i32(list(range(0, T + 1, q_len)))
    pos = torch.arange(q_len, dtype=torch.int32, device=dev).repeat(n_seqs)
    tok_seq = torch.arange(n_seqs, dtype=torch.int32, device=dev).repeat_interleave(q_len)
    posd, qcud, seq_ids = i32([ctx - 1] * B), i32(list(range(B + 1))), i32(list(range(B)))
    # residual
    x, y, y2, w1, w2 = f32(T, W), rnd(T, W), rnd(T, W), f32(W), f32(W)
    xo, xb = torch.empty_like(x), torch.empty((T, W), dtype=dtype, device=dev)
    us = _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_norm="plain", y2=y2, x_out=xo, cast_out=xb), dev)
    add("depth_norm: mixer and experts into the residual + operand copy", us, T * W * (8 + 3 * e))
    us = _time_graph(lambda: do.depth_norm(x, dtype, 1e-5, y=y, post_w=w1, post_norm="rms", x_out=xo, next_w=w2), dev)
    add("depth_norm: RMS norm of the token input into the residual + next layer norm", us, T * W * (8 + 2 * e))
    # input convolutions
    h, cw1, cw2 = rnd(T, W), f32(W, taps), f32(W, taps)
    state = torch.zeros((max(n_seqs, B), 1, (taps - 1) * W), device=dev)
    seq = SequenceState(state, i32(list(range(n_seqs))), tok_seq)
    us = _time_graph(lambda: causal_conv_pair(h, cw1, cw2, seq, 0, q_cu, pos), dev)
    add(f"causal_conv_pair: two convolutions of {taps} taps added to their input", us, 3 * T * W * e)
    # attention mixer
    hs = max(D, V)
    nb, nbd = (q_len + 15) // 16, (ctx + 15) // 16
    table, cu_b = i32(torch.randperm(n_seqs * nb)), i32(list(range(0, n_seqs * nb + 1, nb)))
    slots = i32([int(table[s * nb + p // 16]) * 16 + p % 16 for s in range(n_seqs) for p in range(q_len)])
    kp, vp = rnd(n_seqs * nb, 16, 1, G * hs), rnd(n_seqs * nb, 16, 1, G * hs)
    proj = rnd(T, (H + G) * D + G * V + H)
    fq = f64(RotarySpec(z["rot"], 10000.0).frequencies()[0])
    fv = f64([10000.0 ** (-2.0 * j / V) for j in range(V // 2)])
    at_k, at_v, at_g = H * D, (H + G) * D, (H + G) * D + G * V
    pre = lambda: rotary_parts([RotaryPart(proj[:, :at_k], H, D, fq), RotaryPart(proj[:, at_k:at_v], G, D, fq, cache=kp, cache_head_stride=hs),
                                RotaryPart(proj[:, at_v:at_g], G, V, fv, cache=vp, cache_head_stride=hs)], pos, slots)
    us = _time_graph(pre, dev)
    add("rotary_parts: q, k and turning values of a token, k and v to the cache", us, 2 * T * ((H + G) * D + G * V) * e)
    heads = lambda c: c.as_strided((c.shape[0], c.shape[1], G, hs), (c.stride(0), c.stride(1), hs, 1))
    q, temp, sink = rnd(T, H, D), 1 + 0.1 * f32(H), f32(H)
    seen = n_seqs * sum(i + 1 for i in range(q_len))
    us = _time_graph(lambda: ba.biased_attention(q, heads(kp), heads(vp), V, tok_seq, pos, q_cu, table, cu_b, 1 / math.sqrt(D), None, "causal",
                                                 0, max_q_len=q_len, kv_heads=G, max_kv_len=q_len, head_scale=temp, sinks=sink), dev, launches=2)
    add(f"biased_attention, prefill {n_seqs} x {q_len} (causal, sinks, temperatures, head_dim {D})", us, flops=2 * H * (D + V) * seen)
    kpd, vpd = rnd(B * nbd, 16, 1, G * hs), rnd(B * nbd, 16, 1, G * hs)
    table_d, cu_bd = i32(torch.randperm(B * nbd)), i32(list(range(0, B * nbd + 1, nbd)))
    qd = rnd(B, H, D)
    us = _time_graph(lambda: ba.biased_attention(qd, heads(kpd), heads(vpd), V, seq_ids, posd, qcud, table_d, cu_bd, 1 / math.sqrt(D), None,
                                                 "causal", 0, max_q_len=1, kv_heads=G, max_kv_len=ctx, head_scale=temp, sinks=sink), dev)
    add(f"biased_attention, decode {B} x {ctx} keys (sinks, temperatures)", us, B * ctx * G * (D + V) * e + 2 * B * H * D * e)
    o = rnd(T, H * V)
    us = _time_graph(lambda: rotary_parts([RotaryPart(o, H, V, fv, back=True, gate=proj[:, at_g:], gate_kind="head")], pos), dev)
    add("rotary_parts: heads' results turned back + gate per head", us, 2 * T * H * V * e)
    # latent attention mixer
    row = C + R
    cache = rnd(n_seqs * nb, 16, 1, row)
    lproj = rnd(T, Q + C + R + H * V)
    qw, kw = f32(Q), f32(C)
    us = _time_graph(lambda: latent_norm_cache(lproj, 0, Q, Q, C, qw, kw, 1e-5, slots, cache), dev)
    add("latent_norm_cache (two norms + cache append)", us, 2 * T * (Q + C) * e)
    ql = rnd(T, H * (D + R))
    fl, mag = RotarySpec(R, 10000.0, 4.0, 4096.0, 32.0, 1.0).frequencies()
    fl = f64(fl)
    us = _time_graph(lambda: rotary_parts([RotaryPart(ql, H, D + R, fl, rot_off=D, layout="interleaved", mag=mag, dst=ql),
                                           RotaryPart(lproj[:, Q + C:Q + C + R], 1, R, fl, layout="interleaved", mag=mag, cache=cache,
                                                      cache_col=C)], pos, slots), dev)
    add("rotary_parts: rotated part of the latent queries in place + shared key part to the cache", us, 2 * T * (H * (D + R) + R) * e)
    qlat = rnd(T, H, row)
    seen_w = n_seqs * sum(min(i + 1, win) for i in range(q_len))
    us = _time_graph(lambda: latent_attention(qlat, cache, tok_seq, pos, q_cu, table, cu_b, 0.1, win, q_len, max_kv_len=q_len, sinks=sink), dev,
                     launches=2)
    add(f"latent_attention, prefill {n_seqs} x {q_len} (window {win}, sinks, cached row {row})", us, flops=4 * H * row * seen_w)
    cache_d, qld = rnd(B * nbd, 16, 1, row), rnd(B, H, row)
    us = _time_graph(lambda: latent_attention(qld, cache_d, seq_ids, posd, qcud, table_d, cu_bd, 0.1, win, 1, max_kv_len=ctx, sinks=sink), dev)
    add(f"latent_attention, decode {B} x {min(ctx, win)} keys of the window", us, B * min(ctx, win) * row * e + 2 * B * H * row * e)
    og = rnd(T, H * V)
    us = _time_graph(lambda: gated_group_norm(og, dtype, gate=lproj[:, Q + C + R:], gate_act="sigmoid"), dev)
    add("gated_group_norm: sigmoid gate per element on the latent attention's result", us, 3 * T * H * V * e)
    # experts
    logits, corr = f32(T, E + I), f32(E + I) * 0.01
    us = _time_graph(lambda: mm.route_softmax_topk(logits, E + I, top, 1.0, corr, renorm=False), dev)
    add(f"route_softmax_topk ({E} + {I} identity experts, top {top}, plain weights)", us, T * (E + I + 2 * top) * 4)
    wts, idx = mm.route_softmax_topk(logits, E + I, top, 1.0, corr, renorm=False)
    us = _time_graph(lambda: mm.moe_plan(idx, E), dev)
    add("moe_plan (one workgroup)", us, 3 * T * top * 4)
    seg, row_of, src = mm.moe_plan(idx, E)
    n_rows = int(seg[-1])
    gate_up, down = rnd(E, 2 * eff, W) / math.sqrt(W), rnd(E, W, eff) / math.sqrt(eff)
    us = _time_graph(lambda: mm.grouped_linear(h, gate_up, seg, T * top, src=src), dev, launches=2)
    add(f"grouped_linear gate | up ({n_rows} rows, {W} -> 2 x {eff})", us, flops=2 * n_rows * W * 2 * eff)
    gu = mm.grouped_linear(h, gate_up, seg, T * top, src=src)
    us = _time_graph(lambda: clamped_glu(gu[:, :eff], gu[:, eff:], 0.0, 1.0, 0.0), dev)
    add("clamped_glu as silu(gate) * up over the experts' rows", us, 3 * T * top * eff * e)
    act = clamped_glu(gu[:, :eff], gu[:, eff:], 0.0, 1.0, 0.0)
    us = _time_graph(lambda: mm.grouped_linear(act, down, seg, T * top), dev, launches=2)
    add(f"grouped_linear down ({n_rows} rows, {eff} -> {W})", us, flops=2 * n_rows * W * eff)
    yd = mm.grouped_linear(act, down, seg, T * top)
    us = _time_graph(lambda: mm.moe_combine(yd, row_of, wts, identity=h), dev)
    add("moe_combine (+ identity experts)", us, T * W * (top + 2) * e)
    # per-layer token input
    gp, emb = rnd(T, side), rnd(T, 4 * side)
    us = _time_graph(lambda: gelu_tanh_and_mul(gp, emb[:, side:2 * side]), dev)
    add(f"gelu_tanh_and_mul (token input, {side} channels)", us, 3 * T * side * e)
    del kp, vp, kpd, vpd, cache, cache_d, gate_up, down, gu, act, yd
    torch.cuda.empty_cache()
    kz = kezolix_kernel_table(size_name, dtype, dev, T, n_seqs, B, ctx)
    rows["kezolix"], rows["llama"] = kz["kezolix"], kz["llama"]
    rows["tetepel"] = kernel_table(size_name, dtype, dev, T, n_seqs, B, ctx)["tetepel"]
    rows["workload"] = {"prefill_tokens": T, "portions": n_seqs, "decode_batch": B, "decode_keys": ctx, "size": sz, "pemalorn": z,
                        "timing": "hipGraph of 10 (long kernels: 2) launches, mean of 3 replays, HIP events",
                        "roofline": f"HBM {HBM_PEAK_GBS} GB/s, MFMA {MFMA_PEAK_TFLOPS} TFLOP/s dense bf16; algorithmic bytes / flops"}
    return rows


def run(dtype, dev, sizes=("w2048", "w4096"), design: str = "tetepel") -> dict:
    from hydrainfer_amd import _lib
    _lib.lib(); _lib.mix_lib()
    res = {"throughput": {}, "kernels": {}}
    table = {"tetepel": kernel_table, "kezolix": kezolix_kernel_table, "fasanex": fasanex_kernel_table,
             "pemalorn": pemalorn_kernel_table}[design]
    for s in sizes:
        res["throughput"][s] = throughput(s, dtype, dev, design=design)
        res["kernels"][s] = table(s, dtype, dev)
    return res
