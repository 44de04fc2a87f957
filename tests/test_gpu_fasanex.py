"""GPU: the Fasanex path (kernels of libhydra_mix.so, the model, the engine's scheduler / cache / state-slot managers)
against the float64 restatement in tests/fasanex_oracle.py.  Small made-up configurations and random weights; float32
runs are held to a tight tolerance (a window that is one token off, a lost state or a stale page moves the logits by
percents), bfloat16 runs to a loose one."""
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fasanex_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL32, TOL16 = 2e-4, 6e-2
F = torch.float64


@pytest.fixture(autouse=True)
def _leave_the_device_rng_alone():
    state = torch.cuda.get_rng_state(DEV) if torch.cuda.is_available() else None
    yield
    if state is not None:
        torch.cuda.set_rng_state(state, DEV)


def _shape(kind: str):
    from hydrainfer_amd.model.fasanex import (AttentionSpec as A, FasanexLayer as L, FasanexShape, FeedForwardSpec as FF, MixerSpec as M,
                                              RotarySpec as R, TimeMixSpec as TM)
    par = lambda left, right, ls=1.0, rs=1.0: M("parallel", left=left, right=right, left_scale=ls, right_scale=rs)
    if kind == "hybrid":      # attention first; partial rotation with and without scaled frequencies; a layer without feed-forward
        return FasanexShape(101, 96, [
            L(par(A(4, 2, 16, 16, 2, 0.3, 5.0, 24, R(8, 1000.0, 4.0, 32.0, 4.0, 1.0)), TM(3, 16, 8), 0.7, 1.3), FF(72, 1.5)),
            L(M("mamba2", heads=4, vdim=8, conv=3, state=16, groups=2, norm_groups=1), None),
            L(M("delta", heads=4, vdim=24, conv=2, dim=16, kv_heads=2), FF(40, 0.8)),
            L(par(A(2, 2, 32, 32, 4, 0.2, 0.0, None, R(32, 50.0)), TM(1, 24, 5), 1.0, 0.5), FF(48, None)),
            L(M("mamba2", heads=2, vdim=16, conv=4, state=8, groups=1, norm_groups=4), FF(64, 3.0))],
            norm_eps=1e-5, embedding_scale=2.0)
    if kind == "odd":         # nothing a multiple of four: every kernel's element-by-element path; taps 1 and 5
        return FasanexShape(45, 38, [
            L(M("mamba2", heads=3, vdim=5, conv=5, state=7, groups=3, norm_groups=3), FF(26, 1.0)),
            L(M("delta", heads=3, vdim=10, conv=3, dim=6, kv_heads=3), None),
            L(par(A(3, 1, 6, 6, 4, 0.45, 3.0, 5, R(6, 77.0, 2.0, 16.0, 3.0, 0.5)), TM(1, 9, 3), 0.9, 1.1), FF(11, 2.5)),
            L(par(A(3, 3, 10, 10, 1, 0.4, 8.0, 11, None), TM(2, 7, 2), 1.2, 0.6), None),
            L(M("delta", heads=2, vdim=7, conv=1, dim=9, kv_heads=1), FF(30, 1.2))],
            norm_eps=1e-4, embedding_scale=0.5)
    if kind == "wide":        # states wider than a quad's registers at the smaller sizes; one mixer each, no attention first
        return FasanexShape(61, 64, [
            L(M("delta", heads=2, vdim=32, conv=4, dim=130, kv_heads=1), FF(48, 2.0)),
            L(M("mamba2", heads=2, vdim=64, conv=2, state=128, groups=1, norm_groups=2), None),
            L(par(A(8, 2, 32, 32, 3, 0.18, 30.0, 40, R(16, 10000.0, 16.0, 64.0, 32.0, 1.0)), TM(2, 64, 12), 0.5, 1.0), FF(96, 7.0))],
            norm_eps=1e-6, embedding_scale=1.0)
    if kind == "recurrent":   # no attention mixer: the cache pool has a plane nobody uses
        return FasanexShape(33, 48, [
            L(M("delta", heads=6, vdim=8, conv=3, dim=16, kv_heads=3), None),
            L(M("mamba2", heads=6, vdim=8, conv=3, state=24, groups=3, norm_groups=2), FF(32, 1.0))],
            norm_eps=1e-5, embedding_scale=1.5)
    raise KeyError(kind)


def _weights(shape, seed=0):
    from hydrainfer_amd.model.fasanex import tensor_shapes
    g = torch.Generator().manual_seed(seed)
    W = {}
    for k, s in tensor_shapes(shape).items():
        leaf = k.split(".", 1)[-1] if k[0] == "l" and k[1].isdigit() else k
        tail = leaf.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm1b", "norm2", "norm2b", "final.norm"):
            t = 0.3 * torch.randn(s, generator=g)               # stored as the distance from one
        elif tail == "norm":
            t = 1.0 + 0.2 * torch.randn(s, generator=g)
        elif tail == "conv":
            t = torch.randn(s, generator=g)
        elif leaf.endswith("conv.b") or tail in ("dt_bias", "w0"):
            t = torch.randn(s, generator=g) - 0.5
        elif tail == "A_log":
            t = torch.rand(s, generator=g) * 2.0 - 1.5
        elif tail in ("D", "u"):
            t = torch.randn(s, generator=g)
        elif ".mu." in leaf:
            t = torch.rand(s, generator=g)
        elif k == "embed":
            t = torch.randn(s, generator=g)
        else:
            t = 1.5 * torch.randn(s, generator=g) / math.sqrt(s[-1])
        W[k] = t.to(torch.bfloat16).float()       # representable in a bfloat16 checkpoint: both dtypes see the same weights
    return W


def _model(shape, W, dtype):
    from hydrainfer_amd.model.fasanex import FasanexForCausalLM
    from hydrainfer_amd.model.llava import TextLanguageModel
    return TextLanguageModel(FasanexForCausalLM.from_state_dict(shape, W, dtype, DEV))


def _replayer(lm, dtype, max_tokens, max_live=4):
    from hydrainfer_amd.engine.trace import TraceReplayer
    return TraceReplayer(lm, dtype, DEV, max_tokens, max_live_requests=max_live)


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _run(rp, requests, schedule):
    """schedule: steps of [(request, n_tokens)]; every position's logits are wanted.  Returns {request: [n, vocab]}."""
    at = {r: 0 for r in requests}
    got = {r: [] for r in requests}
    with torch.inference_mode():
        for step in schedule:
            entries, end = [], []
            for r, n in step:
                toks = requests[r][at[r]:at[r] + n]
                entries.append({"id": r, "tokens": toks, "want": list(range(len(toks)))})
                at[r] += n
                if at[r] == len(requests[r]):
                    end.append(r)
            lg = rp.step(entries, end).float().cpu()
            o = 0
            for e in entries:
                got[e["id"]].append(lg[o:o + len(e["tokens"])])
                o += len(e["tokens"])
    return {r: torch.cat(v) for r, v in got.items()}


def _close(got, ref, tol, what=""):
    d = got.double().cpu() - ref
    if tol < 1e-2:
        err = d.abs().max().item() / max(1.0, ref.abs().max().item())
    else:
        err = d.pow(2).mean().sqrt().item() / max(1e-6, ref.pow(2).mean().sqrt().item())
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol}"


def _dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


class _Portions:
    """Sequences cut into portions that travel through state slots: per step, for each sequence that takes part, its next
    tokens; the batch's q_cu / positions / tok_seq and the SequenceState over `state`."""

    def __init__(self, n_slots, floats, poison=7.0):
        self.state = torch.full((n_slots, 1, floats), poison, dtype=torch.float32, device=DEV)     # stale: never read at position 0

    def batch(self, parts):
        """parts: [(slot, first position, n tokens)] -> (SequenceState, q_cu, positions)."""
        from hydrainfer_amd._C.kernel.stream_ops import SequenceState
        q_cu, pos, tok_seq = [0], [], []
        for s, (slot, p0, n) in enumerate(parts):
            q_cu.append(q_cu[-1] + n)
            pos += list(range(p0, p0 + n))
            tok_seq += [s] * n
        return SequenceState(self.state, _i32([p[0] for p in parts]), _i32(tok_seq)), _i32(q_cu), _i32(pos)


# the cuts every stateful kernel is run through: two sequences of lengths (n_a, n_b); b joins late, sits a step out, both
# are cut down to one and two tokens; a third sequence then takes a's slot
def _cuts(n_a, n_b):
    steps, a, b = [], 0, 0
    plan = [(5, 0), (1, 2), (2, 0), (0, 1), (1, 1), (n_a - 9, 3), (0, n_b - 7)]
    for da, db in plan:
        parts = []
        if da:
            parts.append(("a", 0, a, da)); a += da
        if db:
            parts.append(("b", 1, b, db)); b += db
        steps.append(parts)
    assert a == n_a and b == n_b
    return steps


def _through_portions(fn, inputs, n_a, n_b, floats):
    """fn(rows of the batch [dict name -> tensor], seq, q_cu, positions) -> [n, ...]; inputs: {"a": dict, "b": dict} of
    per-token tensors.  Returns the outputs of a and b put together again, and of c — b's inputs through a's slot."""
    P = _Portions(3, floats)
    out = {"a": [], "b": [], "c": []}
    for parts in _cuts(n_a, n_b):
        seq, q_cu, pos = P.batch([(slot, p0, n) for _, slot, p0, n in parts])
        rows = {k: torch.cat([inputs[r][k][p0:p0 + n] for r, _, p0, n in parts]) for k in inputs["a"]}
        y = fn(rows, seq, q_cu, pos)
        o = 0
        for r, _, _, n in parts:
            out[r].append(y[o:o + n]); o += n
    seq, q_cu, pos = P.batch([(0, 0, n_b)])            # a slot that held another sequence, from position 0
    out["c"].append(fn(inputs["b"], seq, q_cu, pos))
    return {r: torch.cat(v).cpu() for r, v in out.items()}


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("C,taps,bias,act", [(38, 4, True, "silu"), (64, 3, False, None), (7, 1, False, "silu"), (130, 5, True, None),
                                             (16, 2, False, "silu"), (20, 9, True, "silu"), (600, 8, False, None)])
def test_short_convolution_through_portions_and_slots(C, taps, bias, act):
    from hydrainfer_amd._C.kernel.seq_mix import causal_conv
    g = torch.Generator().manual_seed(C + taps)
    n_a, n_b = 23, 12
    w, b = torch.randn(C, taps, generator=g), (torch.randn(C, generator=g) if bias else None)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        u = {r: torch.randn(n, C + 3, generator=g).to(dtype) for r, n in (("a", n_a), ("b", n_b))}
        ref = {}
        for r in u:
            y = oracle.short_conv(u[r][:, 1:C + 1].to(F), w.to(F), None if b is None else b.to(F))
            ref[r] = oracle.silu(y) if act else y
        fn = lambda rows, seq, q_cu, pos: causal_conv(_dev(rows["u"], dtype)[:, 1:C + 1], _dev(w), None if b is None else _dev(b), act,
                                                      seq, 8, q_cu, pos)             # a view into wider rows, a piece that starts at 8
        got = _through_portions(fn, {r: {"u": u[r]} for r in u}, n_a, n_b, 8 + max(taps - 1, 1) * C)
        _close(got["a"], ref["a"], tol, "a"); _close(got["b"], ref["b"], tol, "b"); _close(got["c"], ref["b"], tol, "a used slot")


@pytest.mark.parametrize("W_,n_mix", [(38, 5), (64, 1), (130, 3)])
def test_token_shift_mixes_through_portions_and_slots(W_, n_mix):
    from hydrainfer_amd._C.kernel.seq_mix import token_shift_mix
    g = torch.Generator().manual_seed(W_)
    n_a, n_b = 21, 13
    mu = torch.rand(n_mix, W_, generator=g)
    h = {r: torch.randn(n, W_, generator=g) for r, n in (("a", n_a), ("b", n_b))}
    ref = {}
    for r in h:
        prev = torch.cat([torch.zeros(1, W_), h[r][:-1]]).to(F)
        ref[r] = torch.stack([h[r].to(F) + (prev - h[r].to(F)) * mu[m].to(F) for m in range(n_mix)], dim=1)      # [n, n_mix, W]
    fn = lambda rows, seq, q_cu, pos: token_shift_mix(_dev(rows["h"]), _dev(mu), seq, 4, q_cu, pos).transpose(0, 1)
    got = _through_portions(fn, {r: {"h": h[r]} for r in h}, n_a, n_b, 4 + W_)
    _close(got["a"], ref["a"], 1e-6, "a"); _close(got["b"], ref["b"], 1e-6, "b"); _close(got["c"], ref["b"], 1e-6, "a used slot")


def _scan_reference(mode, q, k, v, decay, vscale, beta, bonus, H, G, K, V):
    """Token by token in float64.  q, k: [n, G * K]; v: [n, H * V]; decay: [n, H] or [n, H * K]."""
    n = q.shape[0]
    q, k, v = q.to(F).reshape(n, G, K), k.to(F).reshape(n, G, K), v.to(F).reshape(n, H, V)
    a = decay.to(F).reshape(n, H, -1)
    S, out = torch.zeros(H, K, V, dtype=F), torch.zeros(n, H, V, dtype=F)
    for t in range(n):
        for h in range(H):
            kh, qh, at = k[t, h // (H // G)], q[t, h // (H // G)], a[t, h][:, None]
            if mode == "decay":
                S[h] = at * S[h] + torch.outer(kh, v[t, h] * (vscale[t, h].to(F) if vscale is not None else 1.0))
                out[t, h] = S[h].T @ qh
            elif mode == "bonus":
                kv = torch.outer(kh, v[t, h])
                out[t, h] = (S[h] + bonus.to(F).reshape(H, K)[h][:, None] * kv).T @ qh
                S[h] = at * S[h] + kv
            else:
                S[h] = at * S[h]
                S[h] = S[h] + torch.outer(kh, beta[t, h].to(F) * (v[t, h] - S[h].T @ kh))
                out[t, h] = S[h].T @ qh
    return out.reshape(n, H * V)


@pytest.mark.parametrize("mode,H,G,K,V,per_channel", [("decay", 4, 2, 16, 8, False), ("decay", 3, 3, 7, 5, False), ("decay", 2, 1, 128, 64, False),
                                                      ("bonus", 3, 3, 16, 16, True), ("bonus", 1, 1, 9, 9, True), ("bonus", 2, 2, 64, 64, True),
                                                      ("delta", 4, 2, 16, 24, False), ("delta", 3, 3, 6, 10, False), ("delta", 2, 1, 130, 32, False),
                                                      ("delta", 1, 1, 40, 200, False), ("decay", 2, 2, 24, 40, True),
                                                      # enough heads that a launch of prompts fills the chip: the layouts of large launches
                                                      ("decay", 130, 65, 128, 32, False), ("bonus", 132, 132, 64, 32, True),
                                                      ("delta", 134, 67, 72, 32, False)])
def test_state_scan_forms_sizes_portions_and_slots(mode, H, G, K, V, per_channel):
    from hydrainfer_amd._C.kernel.seq_mix import state_scan
    g = torch.Generator().manual_seed(H * K + V)
    n_a, n_b = 22, 14
    bonus = torch.randn(H * K, generator=g) if mode == "bonus" else None
    for kdtype in (torch.float32, torch.bfloat16):      # the operands' dtype; the state and the sums are float either way
        x = {}
        for r, n in (("a", n_a), ("b", n_b)):
            k = torch.randn(n, G * K, generator=g)
            if mode == "delta":
                k = k.reshape(n, G, K)
                k = (k / k.norm(dim=-1, keepdim=True)).reshape(n, G * K)          # a delta rule is stable for unit keys
            x[r] = {"q": torch.randn(n, G * K, generator=g).to(kdtype), "k": k.to(kdtype), "v": torch.randn(n, H * V, generator=g).to(kdtype),
                    "decay": torch.rand(n, H * (K if per_channel else 1), generator=g) * 0.6 + 0.4,
                    "vscale": torch.rand(n, H, generator=g) + 0.5, "beta": torch.rand(n, H, generator=g)}
        ref = {r: _scan_reference(mode, x[r]["q"], x[r]["k"], x[r]["v"], x[r]["decay"], x[r]["vscale"] if mode == "decay" else None,
                                  x[r]["beta"], bonus, H, G, K, V) for r in x}

        def fn(rows, seq, q_cu, pos):
            return state_scan(mode, _dev(rows["q"], kdtype), _dev(rows["k"], kdtype), _dev(rows["v"], kdtype), _dev(rows["decay"]), seq, 12,
                              q_cu, pos, H, G, K, V, vscale=_dev(rows["vscale"]) if mode == "decay" else None,
                              beta=_dev(rows["beta"]) if mode == "delta" else None, bonus=None if bonus is None else _dev(bonus))
        got = _through_portions(fn, x, n_a, n_b, 12 + H * K * V)
        for r, want in (("a", "a"), ("b", "b"), ("c", "b")):
            _close(got[r], ref[want], 2e-5, f"{mode} {kdtype} {r}")


def test_head_gates_decays_unit_norms_and_activations():
    from hydrainfer_amd._C.kernel.seq_mix import clamped_glu, decay_exp, head_gates, unary, unit_norm
    g = torch.Generator().manual_seed(3)
    T, H = 37, 5
    a, b = torch.randn(T, H + 2, generator=g) * 4, torch.randn(T, H, generator=g) * 3
    a[0, 1], a[1, 1] = 60.0, -60.0                       # softplus far out on both sides
    rate, bias = torch.randn(H, generator=g), torch.randn(H, generator=g)
    decay, step, beta = head_gates(_dev(a)[:, 1:H + 1], _dev(rate), _dev(bias), b=_dev(b), want_step=True)
    sp = oracle.softplus(a[:, 1:H + 1].to(F) + bias.to(F))
    _close(step, sp, 1e-6, "step"); _close(decay, torch.exp(-torch.exp(rate.to(F)) * sp), 1e-6, "decay")
    _close(beta, torch.sigmoid(b.to(F)), 1e-6, "beta")
    x, w0 = torch.randn(T, 23, generator=g), torch.randn(23, generator=g)
    _close(decay_exp(_dev(x), _dev(w0)), torch.exp(-torch.exp(x.to(F) + w0.to(F))), 1e-6, "decay_exp")
    _close(unary(_dev(x), "tanh"), torch.tanh(x.to(F)), 1e-6, "tanh")
    u = torch.randn(T, 3 * 11, generator=g)
    ref = u.to(F).reshape(T, 3, 11)
    ref = ref / torch.sqrt((ref ** 2).sum(-1, keepdim=True) + 1e-6) * 0.3
    _close(unit_norm(_dev(u), 3, 11, 1e-6, 0.3), ref.reshape(T, 33), 1e-6, "unit norm")
    for n in (26, 64):                                   # element by element, and four at a time
        gate, up = torch.randn(T, n, generator=g) * 3, torch.randn(T, n, generator=g) * 3
        for limit in (1.5, 0.0):
            gg = torch.clamp(gate.to(F), max=limit) if limit else gate.to(F)
            uu = torch.clamp(up.to(F), -limit, limit) if limit else up.to(F)
            ref = gg * torch.sigmoid(1.3 * gg) * (uu + 0.5)
            _close(clamped_glu(_dev(gate), _dev(up), limit, 1.3, 0.5), ref, 1e-6, f"clamped glu {n} {limit}")
            both = _dev(torch.cat([gate, up], dim=1), torch.bfloat16)
            ref16 = both.float().cpu().to(F)
            gg = torch.clamp(ref16[:, :n], max=limit) if limit else ref16[:, :n]
            uu = torch.clamp(ref16[:, n:], -limit, limit) if limit else ref16[:, n:]
            _close(clamped_glu(both[:, :n], both[:, n:], limit, 1.3, 0.5), gg * torch.sigmoid(1.3 * gg) * (uu + 0.5), 2e-2, "bf16 halves")


@pytest.mark.parametrize("n,group,w_len,gate,first,skip", [(48, 8, 8, "silu", False, False), (48, 24, 48, "silu", True, True),
                                                          (35, 7, 35, "silu", False, False), (30, 0, 0, "sigmoid", False, False),
                                                          (2048, 2048, 2048, "silu", True, True), (64, 0, 0, "sigmoid", False, False),
                                                          (1280, 0, 0, "silu", False, True), (512, 256, 256, "silu", False, False),
                                                          (384, 128, 128, "silu", False, True)])
def test_gate_and_group_norm(n, group, w_len, gate, first, skip):
    from hydrainfer_amd._C.kernel.seq_mix import gated_group_norm
    g = torch.Generator().manual_seed(n + group)
    T, sg = 9, max(1, n // 6)
    x, gt, sk = torch.randn(T, n, generator=g), torch.randn(T, n, generator=g), torch.randn(T, n, generator=g)
    w = torch.randn(w_len, generator=g) if w_len else None
    sw = torch.randn((n + sg - 1) // sg, generator=g)
    act = oracle.silu if gate == "silu" else torch.sigmoid
    v = x.to(F) + (sw.to(F).repeat_interleave(sg)[:n] * sk.to(F) if skip else 0.0)
    if first:
        v = v * act(gt.to(F))
    if group:
        v = oracle.rms_div(v.reshape(T, n // group, group), 1e-5).reshape(T, n)
    if w is not None:
        v = v * w.to(F).repeat(n // w_len)
    if not first:
        v = v * act(gt.to(F))
    out = torch.zeros(T, n + 5, device=DEV)
    gated_group_norm(_dev(x), torch.float32, group=group, eps=1e-5, w=None if w is None else _dev(w), gate=_dev(gt), gate_act=gate,
                     gate_first=first, skip=_dev(sk) if skip else None, skip_w=_dev(sw) if skip else None, skip_group=sg, scale=0.7,
                     out=out[:, 2:n + 2])
    _close(out[:, 2:n + 2], 0.7 * v, 1e-5, "gate / group norm")
    assert torch.all(out[:, :2] == 0) and torch.all(out[:, n + 2:] == 0)


def _paged_planes(n_blocks, bs, G, head, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    pool = torch.randn(2, n_blocks, bs, G, head, generator=g).to(device=DEV, dtype=dtype)      # stale rows: finite garbage
    return pool[0], pool[1]


@pytest.mark.parametrize("H,G,D,rot", [(4, 2, 16, (8, 1000.0, 4.0, 32.0, 4.0, 1.0)), (3, 1, 6, (6, 77.0, None, 0, 0, 0)), (2, 2, 70, (64, 1e4, 16.0, 64.0, 32.0, 1.0)),
                                       (3, 3, 10, None)])
def test_head_norm_rotation_and_cache_rows(H, G, D, rot):
    from hydrainfer_amd._C.kernel.seq_mix import head_norm_rope_cache
    from hydrainfer_amd.model.fasanex import RotarySpec
    g = torch.Generator().manual_seed(D)
    T, bs = 29, 16
    q, k = torch.randn(T, H * D, generator=g), torch.randn(T, G * D, generator=g)
    qw, kw = torch.randn(D, generator=g), torch.randn(D, generator=g)
    pos = torch.randint(0, 3000, (T,), generator=g)
    pos[0], pos[1] = 0, 2999
    slots = torch.randperm(4 * bs, generator=g)[:T]
    cfg = None if rot is None else {"dims": rot[0], "base": rot[1], "scaling": None if rot[2] is None else
                                    {"factor": rot[2], "original": rot[3], "fast": rot[4], "slow": rot[5]}}
    turn = (lambda x: oracle.rotate(x, pos, cfg)) if cfg else (lambda x: x)
    qref = turn(oracle.rms_div(q.to(F).reshape(T, H, D), 1e-5) * qw.to(F)).reshape(T, H * D)
    kref = turn(oracle.rms_div(k.to(F).reshape(T, G, D), 1e-5) * kw.to(F))
    inv_freq, cs = None, 1.0
    if rot is not None:
        freq, cs = RotarySpec(*rot).frequencies()
        inv_freq = torch.tensor(freq, dtype=torch.float64).to(device=DEV, dtype=torch.float32)
    kc, vc = _paged_planes(4, bs, G + 1, D + 2, torch.float32, 5)
    before = kc.clone()
    qo = head_norm_rope_cache(_dev(q), _dev(k), _dev(qw), _dev(kw), 1e-5, H, G, D, inv_freq, cs, _i32(pos.tolist()), _i32(slots.tolist()), kc, vc)
    _close(qo, qref, 2e-4, "queries")          # (angles of thousands of radians in float32)
    kf, vf = kc.view(4 * bs, G + 1, D + 2), vc.view(4 * bs, G + 1, D + 2)
    _close(kf[slots.to(DEV), :G, :D], kref, 2e-4, "cached keys")
    _close(vf[slots.to(DEV), :G, :D], k.to(F).reshape(T, G, D), 1e-7, "cached values: the keys as they came")
    untouched = torch.ones(4 * bs, dtype=torch.bool); untouched[slots] = False
    assert torch.equal(kc.view(4 * bs, G + 1, D + 2)[untouched.to(DEV)], before.view(4 * bs, G + 1, D + 2)[untouched.to(DEV)])
    assert torch.equal(kf[:, G], before.view(4 * bs, G + 1, D + 2)[:, G])


@pytest.mark.parametrize("H,G,D,window,cap,dtype", [(4, 2, 16, 24, 5.0, torch.bfloat16), (4, 2, 16, 24, 5.0, torch.float32), (3, 1, 6, 5, 3.0, torch.float32),
                                                    (8, 2, 32, 40, 30.0, torch.bfloat16), (2, 2, 64, 300, 0.0, torch.bfloat16),
                                                    (2, 1, 128, 33, 12.0, torch.bfloat16)])
def test_capped_window_attention_one_key_standing_out(H, G, D, window, cap, dtype):
    """Values are the keys' plane twin.  One key far back is made to stand out (its query asks for exactly it): a query whose
    window still holds it must return its value, the next query must not see it — in rows of a prompt's portion and in
    rows decoded alone, at page borders, with the keys of other sequences in the pool."""
    from hydrainfer_amd._C.kernel.biased_attn import biased_attention
    g = torch.Generator().manual_seed(D + window)
    bs, scale = 16, 0.4
    n = window + 70
    mark = 37                                      # the key that stands out; seen by queries mark .. mark + window - 1
    k = torch.randn(n, G, D, generator=g) * 0.3
    v = torch.randn(n, G, D, generator=g)
    q = torch.randn(n, H, D, generator=g) * 0.3
    spike = torch.randn(D, generator=g)
    spike = spike / spike.norm() * 6.0
    k[mark] = spike
    for i in (mark, mark + 1, mark + window - 1, mark + window, n - 1):
        q[i] = spike * 3.0                         # asks for the marked key: far back, just inside, just outside
    k, v, q = (t.to(dtype).to(F) for t in (k, v, q))
    i_, j_ = torch.arange(n)[:, None], torch.arange(n)[None, :]
    see = (j_ <= i_) & (i_ - j_ < window)
    ref = torch.zeros(n, H, D, dtype=F)
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        ref[:, h] = torch.softmax(s.masked_fill(~see, float("-inf")), dim=-1) @ v[:, h // (H // G)]
    n_blocks = (n + bs - 1) // bs
    kc, vc = _paged_planes(2 * n_blocks + 3, bs, G, D, dtype, 9)
    table = torch.randperm(2 * n_blocks + 3, generator=g)[:n_blocks]
    rows = (table[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)[:n].to(DEV)
    kc.view(-1, G, D)[rows] = k.to(device=DEV, dtype=dtype)
    vc.view(-1, G, D)[rows] = v.to(device=DEV, dtype=dtype)
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-5
    forms = ("auto", "tile", "rows") if dtype == torch.bfloat16 and D % 8 == 0 else ("rows",)
    for form in forms:
        # the whole prompt; then portions [0, 50), [50, n - 20) and 20 rows decoded alone, each seeing the cache so far
        for lo, hi in ((0, n), (0, 50), (50, n - 20)) + tuple((t, t + 1) for t in range(n - 20, n)):
            T = hi - lo
            out = biased_attention(_dev(q[lo:hi], dtype), kc, vc, D, _i32([0] * T), _i32(list(range(lo, hi))), _i32([0, T]),
                                   _i32(table.tolist()), _i32([0, n_blocks]), scale, None, "window", window, max_q_len=T, kv_heads=G,
                                   max_kv_len=hi, form=form, softcap=cap)
            _close(out, ref[lo:hi], tol, f"{form} rows {lo}..{hi}")
    # the marked key decides those rows: inside the window the result is mostly its value (as far as the cap lets one score
    # stand out), one row later it is not
    inside, outside = ref[mark + window - 1, 0], ref[mark + window, 0]
    assert (inside - v[mark, 0]).abs().mean() < 0.35 * (outside - v[mark, 0]).abs().mean()


# ------------------------------------------------------------------------------------------------ the model in the engine
@pytest.mark.parametrize("kind", ["hybrid", "odd", "wide", "recurrent"])
def test_whole_prompts_match_the_oracle_layer_by_layer(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=11)
    toks = _tokens(70, shape.vocab_size, 4)
    passed = []
    ref = oracle.forward(shape.to_config(), W, toks, passed)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, 0.1 if kind == "odd" else TOL16)):
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 128)
        lm.language_model.layer_trace = []
        got = _run(rp, {"a": toks}, [[("a", 70)]])["a"]
        trace, lm.language_model.layer_trace = lm.language_model.layer_trace, None
        assert len(trace) == len(passed) == len(shape.layers)
        for r, (a, b) in enumerate(zip(trace, passed)):
            _close(a.cpu(), b, tol, f"{kind} {dtype}: the residual after layer {r}")
        _close(got, ref, tol, f"{kind} {dtype}: logits")


def test_specs_the_engine_reads():
    h, r = (_model(_shape(k), _weights(_shape(k)), torch.float32).language_model for k in ("hybrid", "recurrent"))
    assert h.cache_spec() == {"n_layers": 2, "n_tokens": 2, "n_heads": 2, "head_size": 32} and h.shape.cache_plane == {0: 0, 3: 1}
    assert r.cache_spec()["n_layers"] == 1 and r.shape.cache_plane == {}
    pieces = sorted(h.shape.state_piece.items(), key=lambda kv: kv[1])
    assert [k for k, _ in pieces][:5] == [(0, "conv"), (0, "shift"), (0, "S"), (1, "conv"), (1, "S")]
    assert h.shape.state_piece[(0, "shift")] == (2 - 1) * (4 + 2) * 16 and h.shape.state_piece[(0, "S")] == 96 + 96
    assert h.state_spec() == {"rows": 1, "width": h.shape.state_floats} and h.shape.state_floats % 4 == 0
    assert r.state_spec()["width"] == 2 * (2 * 3 * 16 + 6 * 8) + 6 * 16 * 8 + 2 * (6 * 8 + 2 * 3 * 24) + 6 * 24 * 8


@pytest.mark.parametrize("kind", ["hybrid", "odd", "wide"])
def test_decoding_token_by_token_and_portions_of_every_size_equal_the_whole_prompt(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=13)
    n = 90
    toks = _tokens(n, shape.vocab_size, 6)
    ref = oracle.forward(shape.to_config(), W, toks)
    lm = _model(shape, W, torch.float32)
    rp = _replayer(lm, torch.float32, 96)
    # from the very first token on, one token a step: the first tokens of a sequence, every window and page edge
    got = _run(rp, {"a": toks}, [[("a", 1)] for _ in range(n)])["a"]
    _close(got, ref, TOL32, "decoded from the first token")
    # portions down to two tokens, cut inside pages and windows and shorter than the convolutions; then single tokens
    cuts = [2, 3, 2, 9, 16, 1, 15, 2, 7]
    cuts += [1] * (n - sum(cuts))
    got = _run(rp, {"b": toks}, [[("b", c)] for c in cuts])["b"]
    _close(got, ref, TOL32, "portions")
    got = _run(rp, {"c": toks}, [[("c", 33)], [("c", 31)], [("c", 26)]])["c"]
    _close(got, ref, TOL32, "three portions")


def test_mixed_batches_reused_pages_and_slots():
    """Five unequal requests through a pool for two and a half of them and three state slots: portions beside single
    tokens in one batch, requests that sit steps out, pages and slots handed on to later requests."""
    shape = _shape("hybrid")
    W = _weights(shape, seed=14)
    lens = {"a": 70, "b": 23, "c": 41, "d": 1, "e": 64}
    reqs = {r: _tokens(n, shape.vocab_size, 20 + i) for i, (r, n) in enumerate(lens.items())}
    ref = {r: oracle.forward(shape.to_config(), W, t) for r, t in reqs.items()}
    schedule = [[("a", 30), ("b", 2)], [("b", 1), ("a", 1)], [("a", 17), ("b", 20), ("c", 3)], [("c", 1)],
                [("a", 22), ("c", 30)],                                  # a ends: its pages and slot go back
                [("d", 1), ("c", 2)],                                    # d takes a's slot, ends at once
                [("e", 2), ("c", 1)], [("e", 31), ("c", 1)], [("c", 1), ("e", 1)], [("e", 30), ("c", 2)]]
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 80 + 32 + 48, max_live=3)
        kv, sm = rp.node.kv_cache_block_manager, rp.node.batch_scheduler.context.state_manager
        free0 = len(kv.shared_cache.to_be_evicted)       # blocks no request holds
        assert free0 == kv.n_blocks
        got = _run(rp, reqs, schedule)
        for r in reqs:
            _close(got[r], ref[r], tol, f"request {r} in mixed batches ({dtype})")
        assert len(kv.shared_cache.to_be_evicted) == free0 and sm.get_num_available_slots() == 3
        assert sm.n_allocated_total == 5
        # and again on the used pool: every page and slot now has had an owner before
        got = _run(rp, {"a": reqs["a"], "e": reqs["e"]}, [[("a", 35), ("e", 64)], [("a", 35)]])
        _close(got["a"], ref["a"], tol, "second use of the pool")
        _close(got["e"], ref["e"], tol, "second use of the pool")


def test_long_decoding_past_several_windows():
    shape = _shape("hybrid")
    W = _weights(shape, seed=15)
    toks = _tokens(10 + 150, shape.vocab_size, 8)
    ref = oracle.forward(shape.to_config(), W, toks)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        lm = _model(shape, W, dtype)
        got = _run(_replayer(lm, dtype, 160), {"a": toks}, [[("a", 10)]] + [[("a", 1)] for _ in range(150)])["a"]
        _close(got, ref, tol, f"150 decoded tokens ({dtype})")


def test_greedy_generation_through_the_offline_engine():
    """The framework's own entry point: requests in, the scheduler batches prompts (chunked under a small token budget)
    and decode steps, greedy tokens out.  Compared with the oracle wherever its top-1 margin is not a near-tie."""
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    shape = _shape("hybrid")
    W = _weights(shape, seed=16)
    lm = _model(shape, W, torch.float32)
    eng = OfflineInferenceEngine(lm, None, torch.float32, device=DEV, max_running_requests=3, token_budgets=24,
                                 max_context=96, warm_up=False)
    prompts = [_tokens(n, shape.vocab_size, 30 + i) for i, n in enumerate((37, 5, 18, 50, 1))]
    n_new = 12
    outs = eng.generate([OfflineRequest(token_ids=p, max_tokens=n_new) for p in prompts])
    for p, o in zip(prompts, outs):
        want, margins = oracle.greedy(shape.to_config(), W, p, n_new)
        assert len(o.output_token_ids) == n_new
        for i, (a, b, m) in enumerate(zip(o.output_token_ids, want, margins)):
            if m < 1e-3:
                break            # a near-tie: either token is right, what follows depends on it
            assert a == b, f"prompt of {len(p)}: token {i} is {a}, the oracle says {b} (margin {m:.3g})"
    kv, sm = eng.node.kv_cache_block_manager, eng.node.batch_scheduler.context.state_manager
    assert sm.get_num_available_slots() == 3 and sm.n_allocated_total == 5
    assert len(kv.shared_cache.to_be_evicted) == kv.n_blocks


def test_registry_and_trace_run_command_line(tmp_path):
    """A checkpoint directory through the registry (the decay's inner size comes from its tensors), and bin/trace_run as a
    user starts it: steps on standard input, `done <step>` lines and .f32 files out."""
    import subprocess
    import numpy as np
    import safetensors.torch
    from hydrainfer_amd.model.registry import architecture_of, load_model
    shape = _shape("odd")
    W = _weights(shape, seed=18)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    cfg = shape.to_config()
    for l in cfg["layers"]:
        if l["type"] == "parallel":
            del l["mixer"]["right"]["decay_rank"]            # a configuration that leaves it to the tensors
    (model_dir / "config.json").write_text(json.dumps(cfg))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(model_dir / "model.safetensors"))
    assert architecture_of(str(model_dir)) == "Fasanex"
    lm, vision = load_model(str(model_dir), torch.float32, DEV)
    assert vision is None and lm.language_model.shape.to_config() == shape.to_config()
    a, b = _tokens(21, shape.vocab_size, 40), _tokens(9, shape.vocab_size, 41)
    ra, rb = oracle.forward(shape.to_config(), W, a), oracle.forward(shape.to_config(), W, b)
    _close(_run(_replayer(lm, torch.float32, 32), {"a": a}, [[("a", 21)]])["a"], ra, TOL32, "loaded checkpoint")
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                        "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    read = lambda n: torch.from_numpy(np.fromfile(str(out_dir / f"{n}.f32"), dtype="<f4")).view(-1, shape.vocab_size)
    _close(read(0), ra[[0, 16]], TOL32, "step 0")
    _close(read(1), ra[[17]], TOL32, "step 1")
    _close(read(2), torch.cat([ra[[20]], rb[[8]]]), TOL32, "step 2")


def test_chat_endpoint_serves_a_checkpoint_directory(tmp_path):
    """`python -m hydrainfer_amd.entrypoint --checkpoint DIR` in parts: registry -> node -> front end -> HTTP endpoint.  The
    streams carry the tokens the offline engine generates for the same token ids."""
    import asyncio
    from types import SimpleNamespace
    import safetensors.torch
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    from hydrainfer_amd.entrypoint.__main__ import build_checkpoint_server
    from hydrainfer_amd.entrypoint.api_protocol import parse_chat_completion_request as parse
    from tests.test_api_server import _client_stream, _payload
    shape = _shape("hybrid")
    W = _weights(shape, seed=19)
    (tmp_path / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    args = SimpleNamespace(checkpoint=str(tmp_path), max_running=4, max_tokens=128, tokenizer=None, host="127.0.0.1", port=0, dtype="fp32")
    server, front = build_checkpoint_server(args, torch.float32, torch.device(DEV))
    jobs = [("what a fine day it is today", 6), ("one two three four five six seven eight nine ten eleven twelve", 9), ("hello", 4)]

    async def go():
        await server.start()
        front.start()
        try:
            return await asyncio.gather(*[_client_stream(f"http://127.0.0.1:{server.port}/v1", _payload(t, None, n)) for t, n in jobs])
        finally:
            front.stop()
            await server.close()
    got = asyncio.run(go())
    assert front.error is None and front.n_admitted == len(jobs)
    eng = OfflineInferenceEngine.from_checkpoint(str(tmp_path), torch.float32, DEV, max_running_requests=4, max_context=128, warm_up=False)
    for (text, n_events, done), (prompt, n) in zip(got, jobs):
        assert done and n_events == n + 1 and len(text.split()) == n
        ids = server._token_request(parse(_payload(prompt, None, n))).token_ids
        want = eng.generate([OfflineRequest(token_ids=ids, max_tokens=n)])[0].output_token_ids
        assert text == "".join(server.tokenizer.decode(t) for t in want)
