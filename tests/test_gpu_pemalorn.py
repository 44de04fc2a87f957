"""GPU: the Pemalorn path (kernels of libhydra_mix.so, the model, the engine's scheduler / cache / state-slot managers)
against the float64 restatement in tests/pemalorn_oracle.py.  Small made-up configurations and random weights; float32
runs are held to a tight tolerance (a window that is one token off, a sink left out, a lost convolution input or a stale
page moves the logits by percents), bfloat16 runs to a loose one."""
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import pemalorn_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL32, TOL16 = 2e-4, 0.1      # (bfloat16: up to eight layer runs of weights with a gain above one)
F = torch.float64


@pytest.fixture(autouse=True)
def _leave_the_device_rng_alone():
    state = torch.cuda.get_rng_state(DEV) if torch.cuda.is_available() else None
    yield
    if state is not None:
        torch.cuda.set_rng_state(state, DEV)


def _shape(kind: str):
    from hydrainfer_amd.layer.rotary_spec import RotarySpec as R
    from hydrainfer_amd.model.pemalorn import ExpertsSpec as E, MixerSpec as M, PemalornLayer as L, PemalornShape
    att = lambda H, G, D, V, scale, window=None, rot=None: M("attention", heads=H, dim=D, vdim=V, scale=scale, kv_heads=G, window=window, rot=rot)
    lat = lambda H, D, RD, V, C, Q, scale, window=None, rot=None: M("latent_attention", heads=H, dim=D, vdim=V, scale=scale, kv_rank=C,
                                                                   q_rank=Q, rot_dim=RD, window=window, rot=rot)
    if kind == "mix":         # attention first, a loop over the middle, identity experts, both rotations, a layer without feed-forward
        return PemalornShape(101, 64, [
            L(att(4, 2, 16, 24, 0.3, None, R(8, 1000.0)), E(5, 2, 3, 24)),
            L(lat(3, 8, 16, 12, 24, 20, 0.25, 21, R(16, 1000.0, 4.0, 32.0, 4.0, 1.0)), E(4, 1, 2, 16)),
            L(att(2, 1, 32, 16, 0.2, 30, R(32, 50.0, 2.0, 16.0, 3.0, 0.5)), None),
            L(lat(2, 16, 8, 24, 40, 16, 0.2, None, R(8, 300.0)), E(6, 0, 1, 40))],
            norm_eps=1e-5, taps=3, side_dim=6, loop_start=1, loop_stop=3, loop_times=3, has_loop=True)
    if kind == "odd":         # nothing a multiple of four: every kernel's element-by-element path; a loop from the first layer
        return PemalornShape(45, 38, [
            L(lat(3, 5, 6, 7, 10, 7, 0.4, 5, R(6, 77.0, 2.0, 16.0, 3.0, 0.5)), E(3, 1, 1, 11)),
            L(att(3, 1, 6, 10, 0.45, 7, R(4, 77.0)), E(2, 3, 4, 9)),
            L(att(3, 3, 10, 6, 0.4, None, R(10, 20.0)), None)],
            norm_eps=1e-4, taps=2, side_dim=3, loop_start=0, loop_stop=2, loop_times=2, has_loop=True)
    if kind == "wide":        # sizes that take the matrix-core forms in bfloat16; no loop, no token input, five taps
        return PemalornShape(61, 128, [
            L(lat(4, 32, 32, 40, 64, 48, 0.12, 40, R(32, 10000.0, 16.0, 64.0, 32.0, 1.0)), E(4, 0, 2, 64)),
            L(att(8, 2, 64, 32, 0.12, 48, R(16, 10000.0)), E(8, 2, 3, 32)),
            L(lat(2, 64, 16, 64, 112, 32, 0.1, None, R(16, 500.0)), None),
            L(att(4, 4, 32, 64, 0.15, None, R(32, 10000.0, 8.0, 32.0, 8.0, 2.0)), E(3, 1, 2, 48))],
            norm_eps=1e-6, taps=5)
    if kind == "plain":       # convolutions of ONE tap (nothing to carry), no token input, one pass through a whole-model loop
        return PemalornShape(33, 48, [
            L(att(6, 3, 8, 8, 0.35, 9, R(8, 100.0)), E(2, 0, 2, 20)),
            L(lat(2, 12, 4, 20, 24, 12, 0.3, None, R(4, 100.0)), E(1, 1, 1, 32))],
            norm_eps=1e-5, taps=1, loop_start=0, loop_stop=2, loop_times=1, has_loop=True)
    if kind == "bare":        # no convolutions at all (no state slots), no token input, no loop
        return PemalornShape(33, 48, [
            L(lat(2, 12, 4, 20, 24, 12, 0.3, 13, R(4, 100.0)), E(3, 1, 2, 32)),
            L(att(6, 2, 8, 12, 0.35, None, R(4, 100.0)), None)],
            norm_eps=1e-5)
    raise KeyError(kind)


def _all_chosen(shape):
    """The same shape with every expert chosen by every token (top = all the router's outputs): no choice is left that a
    bfloat16 rounding could turn round, so bfloat16 runs differ from the restatement by rounding alone.  The choice itself is
    checked in float32, and in bfloat16 on the feed-forward alone."""
    import copy
    sh = copy.deepcopy(shape)
    for l in sh.layers:
        if l.mlp is not None:
            l.mlp.top = l.mlp.experts + l.mlp.identity
    return type(sh).from_config(sh.to_config())


def _weights(shape, seed=0, drop=()):
    from hydrainfer_amd.model.pemalorn import tensor_shapes
    g = torch.Generator().manual_seed(seed)
    W = {}
    for k, s in tensor_shapes(shape).items():
        tail = k.rsplit(".", 1)[-1]
        if tail in drop:
            continue
        if tail in ("norm1", "norm") or k == "final.norm":
            t = 1.0 + 0.3 * torch.randn(s, generator=g)
        elif tail == "temp":
            t = 1.0 + 0.4 * torch.randn(s, generator=g)
        elif tail == "sink":
            t = 1.0 + torch.randn(s, generator=g)            # large enough to take a visible share of every softmax
        elif tail == "correction":
            t = 0.2 * torch.randn(s, generator=g)            # large enough to change choices
        elif tail in ("canon1", "canon2"):
            t = 0.7 * torch.randn(s, generator=g)
        elif k == "loop.step":
            t = 0.5 * torch.randn(s, generator=g)
        elif k in ("embed", "side.embed"):
            t = torch.randn(s, generator=g)
        else:
            t = 1.5 * torch.randn(s, generator=g) / math.sqrt(s[-1])
        W[k] = t.to(torch.bfloat16).float()       # representable in a bfloat16 checkpoint: both dtypes see the same weights
    return W


def _model(shape, W, dtype):
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.pemalorn import PemalornForCausalLM
    return TextLanguageModel(PemalornForCausalLM.from_state_dict(shape, W, dtype, DEV))


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


def _batch(state, parts):
    """parts: [(slot, first position, n tokens)] -> (SequenceState over `state`, q_cu, positions)."""
    from hydrainfer_amd._C.kernel.stream_ops import SequenceState
    q_cu, pos, tok_seq = [0], [], []
    for s, (slot, p0, n) in enumerate(parts):
        q_cu.append(q_cu[-1] + n)
        pos += list(range(p0, p0 + n))
        tok_seq += [s] * n
    return SequenceState(state, _i32([p[0] for p in parts]), _i32(tok_seq)), _i32(q_cu), _i32(pos)


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("C,taps,two,n_a,n_b", [(38, 3, True, 23, 12), (64, 2, True, 23, 12), (7, 4, False, 23, 12), (130, 5, True, 23, 12),
                                                 (600, 9, True, 23, 12), (16, 1, True, 23, 12),
                                                 # launches of hundreds of tokens: a thread keeps a channel's inputs over a tile of tokens
                                                 (38, 3, True, 300, 180), (64, 4, False, 300, 180), (130, 8, True, 300, 180), (33, 5, False, 300, 180)])
def test_paired_input_convolutions_through_portions_and_slots(C, taps, two, n_a, n_b):
    """Two sequences cut into portions of one, two and more tokens (shorter than the convolution), one joining late and
    sitting a step out, a third on a used slot; stale slots hold poison that position 0 must not read."""
    from hydrainfer_amd._C.kernel.seq_mix import causal_conv_pair
    g = torch.Generator().manual_seed(C + taps)
    w1, w2 = torch.randn(C, taps, generator=g), torch.randn(C, taps, generator=g)
    plan = [[("a", 0, 0, 5)], [("a", 0, 5, 1), ("b", 1, 0, 2)], [("a", 0, 6, 2)], [("b", 1, 2, 1)], [("a", 0, 8, 1), ("b", 1, 3, 1)],
            [("a", 0, 9, n_a - 9), ("b", 1, 4, 3)], [("b", 1, 7, n_b - 7)], [("c", 0, 0, n_b)]]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        u = {r: torch.randn(n, C + 3, generator=g).to(dtype) for r, n in (("a", n_a), ("b", n_b))}
        u["c"] = u["b"]
        ref = {r: (oracle.input_conv(u[r][:, 1:C + 1].to(F), w1.to(F)), oracle.input_conv(u[r][:, 1:C + 1].to(F), w2.to(F))) for r in u}
        state = torch.full((3, 1, 8 + max(taps - 1, 1) * C), 7.0, dtype=torch.float32, device=DEV)
        got = {r: ([], []) for r in u}
        for parts in plan:
            seq, q_cu, pos = _batch(state, [(slot, p0, n) for _, slot, p0, n in parts])
            rows = _dev(torch.cat([u[r][p0:p0 + n] for r, _, p0, n in parts]), dtype)[:, 1:C + 1]      # a view into wider rows
            y1, y2 = causal_conv_pair(rows, _dev(w1), _dev(w2) if two else None, seq, 8, q_cu, pos)     # a piece that starts at 8
            assert (y2 is not None) == two
            o = 0
            for r, _, _, n in parts:
                got[r][0].append(y1[o:o + n]); got[r][1].append((y2 if two else y1)[o:o + n]); o += n
        for r in u:
            _close(torch.cat(got[r][0]), ref[r][0], tol, f"{r}: first convolution")
            if two:
                _close(torch.cat(got[r][1]), ref[r][1], tol, f"{r}: second convolution")


@pytest.mark.parametrize("H,D,off,rd,layout,mag,pad", [(4, 16, 0, 8, "halves", 1.0, 2), (3, 10, 4, 6, "interleaved", 1.2, 2), (2, 64, 0, 64, "halves", 1.0, 2),
                                                       (5, 7, 1, 6, "interleaved", 0.9, 2), (1, 32, 16, 16, "interleaved", 1.3, 2),
                                                       # everything a multiple of eight: eight channels a lane, several tokens a workgroup
                                                       (2, 64, 0, 64, "halves", 1.0, 8), (8, 128, 0, 64, "halves", 1.1, 8), (1, 32, 16, 16, "interleaved", 1.3, 8),
                                                       (4, 192, 128, 64, "interleaved", 1.2, 8), (16, 32, 8, 16, "halves", 1.0, 8)])
def test_rotary_parts_layouts_offsets_gates_and_cache_columns(H, D, off, rd, layout, mag, pad):
    from hydrainfer_amd._C.kernel.rotary import RotaryPart, rotary_parts
    g = torch.Generator().manual_seed(H * D + rd)
    T, bs, n_blocks = 37, 16, 6
    pos = torch.randint(0, 3000, (T,), generator=g)
    freq, _ = oracle.pair_frequencies(rd, 500.0)
    x = torch.randn(T, H, D, generator=g)
    gate_h, gate_e = torch.randn(T, H, generator=g), torch.randn(T, H, D, generator=g)
    slots = torch.randperm(n_blocks * bs, generator=g)[:T]
    slots[5] = -1                                          # a token without a cache row
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        xs = x.to(dtype).to(F)
        turned = lambda sign: torch.cat([xs[..., :off], oracle.rotate(xs[..., off:off + rd], sign * pos, freq, layout, mag), xs[..., off + rd:]], dim=-1)
        fwd, back = turned(1), turned(-1)
        xd = _dev(torch.cat([x, torch.zeros(T, H, pad)], dim=-1).reshape(T, H * (D + pad)), dtype)    # heads D + pad apart in the source
        cache = torch.full((n_blocks, bs, 1, H * D + 24), 3.0, dtype=dtype, device=DEV)
        fd = _dev(freq, torch.float64)
        gh, ge = _dev(gate_h, dtype), _dev(gate_e.reshape(T, H * D), dtype)
        outs = rotary_parts([
            RotaryPart(xd, H, D, fd, rot_off=off, layout=layout, mag=mag, src_head_stride=D + pad),
            RotaryPart(xd, H, D, fd, rot_off=off, layout=layout, mag=mag, src_head_stride=D + pad, cache=cache, cache_col=16),
            RotaryPart(xd, H, D, fd, rot_off=off, layout=layout, mag=mag, src_head_stride=D + pad, back=True, gate=gh, gate_kind="head"),
        ], _i32(pos.tolist()), _i32(slots.tolist()))
        _close(outs[0].view(T, H, D), fwd, tol, "turned forwards")
        assert outs[1] is None
        _close(outs[2].view(T, H, D), back * torch.sigmoid(gh.to(F).cpu())[:, :, None], tol, "turned back, gate per head")
        rows = cache.view(n_blocks * bs, -1).cpu()
        live = slots >= 0
        _close(rows[slots[live], 16:16 + H * D].reshape(-1, H, D), fwd[live], tol, "cache rows")
        untouched = torch.ones(n_blocks * bs, dtype=torch.bool)
        untouched[slots[live]] = False
        assert (rows[untouched] == 3.0).all() and (rows[:, :16] == 3.0).all() and (rows[:, 16 + H * D:] == 3.0).all()
        out = rotary_parts([RotaryPart(xd, H, D, None, src_head_stride=D + pad, gate=ge, gate_kind="element")], _i32(pos.tolist()))[0]
        _close(out.view(T, H, D), xs * torch.sigmoid(ge.to(F).cpu()).view(T, H, D), tol, "a gate per element, nothing turns")
        # in place
        y = xd.view(T, H, D + pad)[:, :, :D].reshape(T, H * D).contiguous()
        rotary_parts([RotaryPart(y, H, D, fd, rot_off=off, layout=layout, mag=mag, dst=y)], _i32(pos.tolist()))
        _close(y.view(T, H, D), fwd, tol, "in place")


def _paged(n_blocks, bs, width, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n_blocks, bs, 1, width, generator=g).to(device=DEV, dtype=dtype)      # stale rows: finite garbage


def _spans(n):
    # the whole prompt; portions [0, 50), [50, n - 20); then 20 rows decoded alone, each seeing the cache so far
    return ((0, n), (0, 50), (50, n - 20)) + tuple((t, t + 1) for t in range(n - 20, n))


@pytest.mark.parametrize("H,G,D,V,window,dtype", [(4, 2, 16, 24, 24, torch.bfloat16), (4, 2, 16, 24, None, torch.float32), (3, 1, 6, 10, 5, torch.float32),
                                                  (8, 2, 64, 32, 40, torch.bfloat16), (2, 2, 32, 64, None, torch.bfloat16),
                                                  (6, 3, 128, 128, 33, torch.bfloat16)])
def test_attention_with_sinks_and_temperatures_one_key_standing_out(H, G, D, V, window, dtype):
    """One key far back is made to stand out (its query asks for exactly it): a query whose window still holds it returns its
    value, the next one does not see it.  Sinks large enough to take a tenth to a half of every softmax, a temperature per
    head between a half and two; rows of a prompt's portion and rows decoded alone, at page borders, keys and values of
    different sizes in rows of a wider cache plane."""
    from hydrainfer_amd._C.kernel.biased_attn import biased_attention
    g = torch.Generator().manual_seed(D + V)
    bs, scale = 16, 0.4
    n = (window or 60) + 70
    mark = 37
    k = torch.randn(n, G, D, generator=g) * 0.3
    v = torch.randn(n, G, V, generator=g)
    q = torch.randn(n, H, D, generator=g) * 0.3
    spike = torch.randn(D, generator=g)
    spike = spike / spike.norm() * 6.0
    k[mark] = spike
    asked = (mark, mark + 1, n - 1) + ((mark + window - 1, mark + window) if window else ())
    for i in asked:
        q[i] = spike * 3.0
    temp = 0.5 + 1.5 * torch.rand(H, generator=g)
    sink = 1.0 + 2.0 * torch.rand(H, generator=g)
    k, v, q = (t.to(dtype).to(F) for t in (k, v, q))
    rep = H // G
    ref = oracle.sink_softmax_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), scale * temp.to(F), sink.to(F), window)
    without = oracle.sink_softmax_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), scale * temp.to(F),
                                            torch.full((H,), -1e9, dtype=F), window)
    assert (ref - without).abs().max() > 0.05              # the sink shows
    hs = (max(D, V) + 7) // 8 * 8
    n_blocks = (n + bs - 1) // bs
    kp, vp = _paged(2 * n_blocks + 3, bs, G * hs + 8, dtype, 9), _paged(2 * n_blocks + 3, bs, G * hs + 8, dtype, 10)
    heads = lambda c: c.as_strided((c.shape[0], c.shape[1], G, hs), (c.stride(0), c.stride(1), hs, 1))
    table = torch.randperm(2 * n_blocks + 3, generator=g)[:n_blocks]
    rows = (table[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)[:n].to(DEV)
    kv_k, kv_v = heads(kp), heads(vp)
    for r_, row in enumerate(rows.tolist()):
        kv_k[row // bs, row % bs, :, :D] = k[r_].to(device=DEV, dtype=dtype)
        kv_v[row // bs, row % bs, :, :V] = v[r_].to(device=DEV, dtype=dtype)
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-5
    forms = ("auto", "tile", "rows") if dtype == torch.bfloat16 and D % 8 == 0 and V % 8 == 0 else ("rows",)
    for form in forms:
        for lo, hi in _spans(n):
            T = hi - lo
            out = biased_attention(_dev(q[lo:hi], dtype), kv_k, kv_v, V, _i32([0] * T), _i32(list(range(lo, hi))), _i32([0, T]),
                                   _i32(table.tolist()), _i32([0, n_blocks]), scale, None, "window" if window else "causal", window or 0,
                                   max_q_len=T, kv_heads=G, max_kv_len=hi, form=form, head_scale=_dev(temp), sinks=_dev(sink))
            _close(out, ref[lo:hi], tol, f"{form} rows {lo}..{hi}")
    if window:
        inside, outside = ref[mark + window - 1, 0], ref[mark + window, 0]
        assert (inside - v[mark, 0]).abs().mean() < 0.35 * (outside - v[mark, 0]).abs().mean()
    else:
        assert (ref[n - 1, 0] - v[mark, 0]).abs().mean() < 0.2 * v[mark, 0].abs().mean() + 0.05      # far back, still found


@pytest.mark.parametrize("H,R,window,dtype", [(4, 40, 24, torch.bfloat16), (3, 10, 5, torch.float32), (2, 96, None, torch.bfloat16),
                                              (5, 72, 33, torch.float32), (16, 128, 40, torch.bfloat16), (2, 320, 50, torch.bfloat16)])
def test_latent_attention_with_sinks_one_key_standing_out(H, R, window, dtype):
    from hydrainfer_amd._C.kernel.latent_attn import latent_attention
    g = torch.Generator().manual_seed(H + R)
    bs, scale = 16, 0.3
    n = (window or 60) + 70
    mark = 37
    c = torch.randn(n, R, generator=g) * 0.3
    q = torch.randn(n, H, R, generator=g) * 0.3
    spike = torch.randn(R, generator=g)
    spike = spike / spike.norm() * 6.0
    c[mark] = spike
    for i in (mark, mark + 1, n - 1) + ((mark + window - 1, mark + window) if window else ()):
        q[i] = spike * 3.0
    sink = 1.0 + 2.0 * torch.rand(H, generator=g)
    c, q = c.to(dtype).to(F), q.to(dtype).to(F)
    kv = c[:, None, :].expand(n, H, R)
    ref = oracle.sink_softmax_attention(q, kv, kv, torch.full((H,), scale, dtype=F), sink.to(F), window)
    without = oracle.sink_softmax_attention(q, kv, kv, torch.full((H,), scale, dtype=F), torch.full((H,), -1e9, dtype=F), window)
    assert (ref - without).abs().max() > 0.05
    n_blocks = (n + bs - 1) // bs
    cache = _paged(2 * n_blocks + 3, bs, R + 8, dtype, 11)
    table = torch.randperm(2 * n_blocks + 3, generator=g)[:n_blocks]
    rows = (table[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)[:n].to(DEV)
    cache.view(-1, R + 8)[rows, :R] = c.to(device=DEV, dtype=dtype)
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-5
    for lo, hi in _spans(n):
        T = hi - lo
        out = latent_attention(_dev(q[lo:hi], dtype), cache, _i32([0] * T), _i32(list(range(lo, hi))), _i32([0, T]), _i32(table.tolist()),
                               _i32([0, n_blocks]), scale, window, T, max_kv_len=hi, sinks=_dev(sink))
        _close(out, ref[lo:hi], tol, f"rows {lo}..{hi}")
    if window:
        inside, outside = ref[mark + window - 1, 0], ref[mark + window, 0]
        assert (inside - c[mark]).abs().mean() < 0.35 * (outside - c[mark]).abs().mean()


@pytest.mark.parametrize("W_", [38, 64, 129])
def test_residual_kernel_two_results_bias_norm_kinds_and_operand_copy(W_):
    from hydrainfer_amd._C.kernel.depth_ops import depth_norm
    g = torch.Generator().manual_seed(W_)
    T, eps = 19, 1e-4
    x, b = torch.randn(T, W_, generator=g), torch.randn(W_, generator=g)
    pw, nw = 1 + 0.3 * torch.randn(W_, generator=g), 1 + 0.3 * torch.randn(W_, generator=g)
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        y, y2 = (torch.randn(T, W_ + 4, generator=g).to(dtype) for _ in range(2))
        yf, y2f = y[:, :W_].to(F), y2[:, 2:W_ + 2].to(F)
        # two results join as they are; the row leaves as an operand into a column range of a wider matrix, and as the next norm
        want = x.to(F) + yf + y2f
        wide = torch.zeros(T, 2 * W_ + 8, dtype=dtype, device=DEV)
        x_out = torch.empty(T, W_, device=DEV)
        depth_norm(_dev(x), dtype, eps, y=_dev(y, dtype)[:, :W_], post_norm="plain", y2=_dev(y2, dtype)[:, 2:W_ + 2], x_out=x_out,
                   cast_out=wide[:, 8:8 + W_] if W_ % 2 == 0 else wide[:, 7:7 + W_])
        _close(x_out, want, 2e-6, "x + y + y2")
        at = 8 if W_ % 2 == 0 else 7
        _close(wide[:, at:at + W_], want, tol, "the operand copy")
        assert (wide[:, :at] == 0).all() and (wide[:, at + W_:] == 0).all()
        h = depth_norm(_dev(x), dtype, eps, y=_dev(y, dtype)[:, :W_], post_w=_dev(pw), post_norm="rms", x_out=x_out, next_w=_dev(nw))
        want = x.to(F) + oracle.rms_norm(yf, pw.to(F), eps)
        _close(x_out, want, 2e-6, "x + rms_norm(y) w")
        _close(h, oracle.layer_norm(want, nw.to(F), eps), tol, "layer norm of it")
        # no residual to start from: a product's result plus a vector becomes the residual
        h = depth_norm(None, dtype, eps, y=_dev(y, dtype)[:, :W_], post_norm="plain", bias=_dev(b), x_out=x_out, next_w=_dev(nw))
        _close(x_out, yf + b.to(F), 2e-6, "y + bias")
        _close(h, oracle.layer_norm(yf + b.to(F), nw.to(F), eps), tol, "its layer norm")
        h = depth_norm(_dev(x), dtype, eps, y=_dev(y, dtype)[:, :W_], post_w=_dev(pw), post_norm="layer", next_w=_dev(nw), rms=True,
                       rows=_i32([3, 0, 18]))
        want = (x.to(F) + oracle.layer_norm(yf, pw.to(F), eps))[[3, 0, 18]]
        _close(h, oracle.rms_norm(want, nw.to(F), eps), tol, "layer norm in, RMS norm out, chosen rows")


@pytest.mark.parametrize("E,I,top,W_,ff", [(5, 2, 3, 64, 24), (3, 1, 1, 38, 11), (2, 3, 4, 40, 9), (70, 5, 6, 32, 16), (1, 1, 2, 16, 8)])
def test_router_with_correction_plain_weights_and_identity_experts(E, I, top, W_, ff):
    """The model's feed-forward (router in float, plan, grouped products, silu gate, combine) against the restatement: a
    correction large enough to change the choice, weights that are the scores themselves, experts that hand their input on."""
    from hydrainfer_amd._C.kernel.moe_mix import route_softmax_topk
    from hydrainfer_amd.layer.rotary_spec import RotarySpec as R
    from hydrainfer_amd.model.pemalorn import ExpertsSpec, MixerSpec, PemalornLayer, PemalornShape
    shape = PemalornShape(17, W_, [PemalornLayer(MixerSpec("attention", heads=1, dim=8, vdim=8, scale=0.3, kv_heads=1, rot=R(8, 100.0)),
                                                 ExpertsSpec(E, I, top, ff))])
    W = _weights(shape, seed=E + top)
    g = torch.Generator().manual_seed(3)
    T = 50
    h = torch.randn(T, W_, generator=g)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        hd = h.to(dtype)
        Wd = {k: v.to(dtype).to(F) for k, v in W.items()}
        mlp = shape.to_config()["layers"][0]["mlp"]
        weights, idx = oracle.route(hd.to(F), Wd, "l0.mlp.", mlp["router"])
        plain, _ = oracle.route(hd.to(F), {k: v for k, v in Wd.items() if not k.endswith("correction")}, "l0.mlp.", mlp["router"])
        lm = _model(shape, W, dtype).language_model
        logits = torch.matmul(_dev(hd, dtype).float(), lm.lw[0].router)
        gw, ge = route_softmax_topk(logits, E + I, top, 1.0, lm.lw[0].correction, renorm=False)
        # (where two choice scores all but tie the two may order them differently: compare as sets, through the output)
        same = (ge.cpu().long().sort(dim=1).values == idx.sort(dim=1).values).all(dim=1)
        assert same.float().mean() > 0.9
        assert top == E + I or (weights.sum(dim=1) < 0.999).any()          # not renormalised
        if top < E + I and E + I > 2:
            assert (weights.sort(dim=1).values - plain.sort(dim=1).values).abs().max() > 1e-3      # the correction changes choices
        with torch.inference_mode():
            out = lm._experts(0, _dev(hd, dtype))
        ref = oracle.expert_mixture(hd.to(F), Wd, "l0.mlp.", mlp)
        _close(out[same.to(DEV)], ref[same], tol, "the mixture's output")
        assert I == 0 or (idx >= E).any()                                   # identity experts were chosen


# ------------------------------------------------------------------------------------------------ the model in the engine
@pytest.mark.parametrize("kind", ["mix", "odd", "wide", "plain", "bare"])
def test_whole_prompts_match_the_oracle_layer_by_layer(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=11)
    toks = _tokens(70, shape.vocab_size, 4)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        if dtype == torch.bfloat16:
            shape = _all_chosen(shape)
        passed = []
        ref = oracle.forward(toks, W, shape.to_config(), passed)
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 128)
        lm.language_model.layer_trace = []
        got = _run(rp, {"a": toks}, [[("a", 70)]])["a"]
        trace, lm.language_model.layer_trace = lm.language_model.layer_trace, None
        assert len(trace) == len(passed) == len(shape.runs)
        for r, (a, b) in enumerate(zip(trace, passed)):
            _close(a.cpu(), b, tol, f"{kind} {dtype}: the residual after layer run {r}")
        _close(got, ref, tol, f"{kind} {dtype}: logits")
        got = _run(rp, {"b": toks}, [[("b", 70)]])["b"]          # and on the product path proper (fused layer ends)
        _close(got, ref, tol, f"{kind} {dtype}: logits, fused layer ends")


def test_specs_the_engine_reads():
    m, p = (_model(_shape(k), _weights(_shape(k)), torch.float32).language_model for k in ("mix", "plain"))
    # runs: layer 0, three passes over layers 1 and 2, layer 3; an attention run takes two planes, a latent run one
    assert [r[0] for r in m.shape.runs] == [0, 1, 2, 1, 2, 1, 2, 3] and [r[2] for r in m.shape.runs] == [False, True, False, True, False, True, False, False]
    assert m.shape.run_plane == [0, 2, 3, 5, 6, 8, 9, 11] and m.cache_spec() == {"n_layers": 12, "n_tokens": 1, "n_heads": 1, "head_size": 48}
    assert m.state_spec() == {"rows": 1, "width": 8 * 2 * 64} and m.shape.state_piece(3) == 3 * 128
    assert p.state_spec() == {"rows": 1, "width": 2 * 48} and p.cache_spec()["n_layers"] == 3
    b = _model(_shape("bare"), _weights(_shape("bare")), torch.float32).language_model
    assert b.state_spec() is None and "l0.canon1" not in b.shape.to_config() and b.shape.to_config().get("canon") is None
    assert m.shape.to_config() == type(m.shape).from_config(m.shape.to_config()).to_config()


@pytest.mark.parametrize("kind", ["mix", "odd", "wide", "plain", "bare"])
def test_decoding_token_by_token_and_portions_of_every_size_equal_the_whole_prompt(kind):
    shape = _shape(kind)
    W = _weights(shape, seed=13)
    n = 90
    toks = _tokens(n, shape.vocab_size, 6)
    ref = oracle.forward(toks, W, shape.to_config())
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
    if kind == "wide":                                           # the matrix-core forms through the same cuts
        shape = _all_chosen(shape)
        ref = oracle.forward(toks, W, shape.to_config())
        lm = _model(shape, W, torch.bfloat16)
        got = _run(_replayer(lm, torch.bfloat16, 96), {"b": toks}, [[("b", c)] for c in cuts])["b"]
        _close(got, ref, TOL16, "portions, bfloat16")


def test_mixed_batches_reused_pages_and_slots():
    """Five unequal requests through a pool for two and a half of them and three state slots: portions beside single
    tokens in one batch, requests that sit steps out, pages and slots handed on to later requests."""
    shape = _shape("mix")
    W = _weights(shape, seed=14)
    lens = {"a": 70, "b": 23, "c": 41, "d": 1, "e": 64}
    reqs = {r: _tokens(n, shape.vocab_size, 20 + i) for i, (r, n) in enumerate(lens.items())}
    schedule = [[("a", 30), ("b", 2)], [("b", 1), ("a", 1)], [("a", 17), ("b", 20), ("c", 3)], [("c", 1)],
                [("a", 22), ("c", 30)],                                  # a ends: its pages and slot go back
                [("d", 1), ("c", 2)],                                    # d takes a's slot, ends at once
                [("e", 2), ("c", 1)], [("e", 31), ("c", 1)], [("c", 1), ("e", 1)], [("e", 30), ("c", 2)]]
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        if dtype == torch.bfloat16:
            shape = _all_chosen(shape)
        ref = {r: oracle.forward(t, W, shape.to_config()) for r, t in reqs.items()}
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
    shape = _shape("mix")
    W = _weights(shape, seed=15)
    toks = _tokens(10 + 150, shape.vocab_size, 8)
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        if dtype == torch.bfloat16:
            shape = _all_chosen(shape)
        ref = oracle.forward(toks, W, shape.to_config())
        lm = _model(shape, W, dtype)
        got = _run(_replayer(lm, dtype, 160), {"a": toks}, [[("a", 10)]] + [[("a", 1)] for _ in range(150)])["a"]
        _close(got, ref, tol, f"150 decoded tokens ({dtype})")


def test_long_prompts_far_keys_in_portions_and_decoded():
    """Several hundred positions: angles far out, keys far back (two layers see every earlier token), many pages, the key
    splits of decode steps over long ranges — whole, in portions that end inside pages and windows, and decoded."""
    shape = _shape("wide")
    W = _weights(shape, seed=21)
    n = 600
    toks = _tokens(n, shape.vocab_size, 12)
    cuts = [37] * 15 + [5]
    cuts += [1] * (n - sum(cuts))
    for dtype, tol in ((torch.float32, TOL32), (torch.bfloat16, TOL16)):
        if dtype == torch.bfloat16:
            shape = _all_chosen(shape)
        ref = oracle.forward(toks, W, shape.to_config())
        lm = _model(shape, W, dtype)
        rp = _replayer(lm, dtype, 640 + 608)
        got = _run(rp, {"a": toks, "b": toks}, [[("a", n)]] + [[("b", c)] for c in cuts])
        _close(got["a"], ref, tol, f"whole ({dtype})")
        _close(got["b"], ref, tol, f"portions and decoded ({dtype})")
        _close(got["b"][-40:], ref[-40:], tol, f"the decoded rows ({dtype})")


def test_checkpoints_without_temperatures_sinks_and_corrections():
    shape = _shape("odd")
    W = _weights(shape, seed=17, drop=("temp", "sink", "correction"))
    toks = _tokens(40, shape.vocab_size, 9)
    full = {k: v for k, v in W.items()}
    for i, l in enumerate(shape.layers):                  # what the restatement takes instead: ones, no sink, no correction
        if l.mixer.type == "attention":
            full[f"l{i}.mix.temp"] = torch.ones(l.mixer.heads)
        full[f"l{i}.mix.sink"] = torch.full((l.mixer.heads,), -1e9)
    ref = oracle.forward(toks, full, shape.to_config())
    lm = _model(shape, W, torch.float32)
    got = _run(_replayer(lm, torch.float32, 48), {"a": toks}, [[("a", 25)], [("a", 15)]])["a"]
    _close(got, ref, TOL32, "no temperatures, sinks or corrections")


def test_greedy_generation_through_the_offline_engine():
    """The framework's own entry point: requests in, the scheduler batches prompts (chunked under a small token budget)
    and decode steps, greedy tokens out.  Compared with the oracle wherever its top-1 margin is not a near-tie."""
    from hydrainfer_amd.engine.offline import OfflineInferenceEngine, OfflineRequest
    shape = _shape("mix")
    W = _weights(shape, seed=16)
    lm = _model(shape, W, torch.float32)
    eng = OfflineInferenceEngine(lm, None, torch.float32, device=DEV, max_running_requests=3, token_budgets=24,
                                 max_context=96, warm_up=False)
    prompts = [_tokens(n, shape.vocab_size, 30 + i) for i, n in enumerate((37, 5, 18, 50, 1))]
    n_new = 12
    outs = eng.generate([OfflineRequest(token_ids=p, max_tokens=n_new) for p in prompts])
    for p, o in zip(prompts, outs):
        want, margins = oracle.greedy(p, W, shape.to_config(), n_new)
        assert len(o.output_token_ids) == n_new
        for i, (a, b, m) in enumerate(zip(o.output_token_ids, want, margins)):
            if m < 1e-3:
                break            # a near-tie: either token is right, what follows depends on it
            assert a == b, f"prompt of {len(p)}: token {i} is {a}, the oracle says {b} (margin {m:.3g})"
    kv, sm = eng.node.kv_cache_block_manager, eng.node.batch_scheduler.context.state_manager
    assert sm.get_num_available_slots() == 3 and sm.n_allocated_total == 5
    assert len(kv.shared_cache.to_be_evicted) == kv.n_blocks


def test_registry_and_trace_run_command_line(tmp_path):
    """A checkpoint directory through the registry, and bin/trace_run as a user starts it: steps on standard input,
    `done <step>` lines and .f32 files out."""
    import subprocess
    import numpy as np
    import safetensors.torch
    from hydrainfer_amd.model.registry import architecture_of, load_model
    shape = _shape("odd")
    W = _weights(shape, seed=18)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(shape.to_config()))
    safetensors.torch.save_file({k: v.to(torch.bfloat16) for k, v in W.items()}, str(model_dir / "model.safetensors"))
    assert architecture_of(str(model_dir)) == "Pemalorn"
    lm, vision = load_model(str(model_dir), torch.float32, DEV)
    assert vision is None and lm.language_model.shape.to_config() == shape.to_config()
    a, b = _tokens(21, shape.vocab_size, 40), _tokens(9, shape.vocab_size, 41)
    ra, rb = oracle.forward(a, W, shape.to_config()), oracle.forward(b, W, shape.to_config())
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
    shape = _shape("mix")
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
