"""CPU: the host side of the Pemalorn integration — configuration reading, layer runs, cache planes and state pieces, tensor
names, the model registry — and the float64 restatement's own mechanisms on cases worked out by hand."""
import json
import math

import pytest
import torch

import tests.pemalorn_oracle as oracle
from hydrainfer_amd.model.pemalorn import PemalornForCausalLM, PemalornShape, tensor_shapes

F = torch.float64


def _config(**over):
    att = {"dim": 8, "heads": 6, "kv_heads": 3, "vdim": 12, "scale": 0.25, "rot": {"base": 500.0, "dims": 4}}
    lat = {"dim": 6, "heads": 5, "kv_rank": 20, "q_rank": 14, "rot_dim": 4, "vdim": 10, "scale": 0.3, "mask": {"size": 11},
           "rot": {"base": 500.0, "dims": 4, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}}}
    moe = lambda e, i, t, ff: {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": e, "identity": i, "top": t}}
    cfg = {"architecture": "Pemalorn", "vocab": 33, "width": 24, "norm": {"eps": 1e-4}, "canon": {"taps": 4}, "token_side": {"dim": 5},
           "loop": {"start": 1, "stop": 3, "times": 2},
           "layers": [{"type": "latent_attention", "mixer": json.loads(json.dumps(lat)), "mlp": moe(3, 2, 2, 16)},
                      {"type": "attention", "mixer": json.loads(json.dumps(att)), "mlp": None},
                      {"type": "latent_attention", "mixer": json.loads(json.dumps(lat)), "mlp": moe(4, 0, 1, 8)},
                      {"type": "attention", "mixer": json.loads(json.dumps(att)), "mlp": moe(2, 1, 3, 12)}]}
    cfg.update(over)
    return cfg


def test_shape_from_config_runs_planes_pieces_and_names():
    sh = PemalornShape.from_config(_config())
    assert [(r[0], r[1], r[2]) for r in sh.runs] == [(0, 0, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (3, 0, False)]
    assert sh.run_plane == [0, 1, 3, 4, 6, 7] and sh.n_planes == sh.num_hidden_layers == 9
    # an attention row: three heads, sixteen (twelve rounded up to eight) apart; a latent row: latent + rotated part
    assert sh.layers[1].mixer.head_stride == 16 and sh.layers[1].mixer.row == 48 and sh.layers[0].mixer.row == 24 and sh.head_dim == 48
    assert sh.num_key_value_heads == 1 and sh.num_attention_heads == 6
    assert sh.state_floats == 6 * 3 * 24 and sh.state_piece(4) == 4 * 72
    m = sh.layers[0].mixer
    assert (m.window, m.rot.factor, m.rot.original, m.rot_dim, m.kv_rank, m.q_rank) == (11, 4.0, 64.0, 4, 20, 14)
    assert sh.layers[1].mixer.window is None and sh.layers[1].mlp is None and sh.layers[3].mlp.identity == 1
    assert PemalornShape.from_config(sh.to_config()).to_config() == sh.to_config() == _config()
    names = tensor_shapes(sh)
    assert names["l0.mix.dkv"] == (24, 24) and names["l0.mix.uq"] == (50, 14) and names["l0.mix.uk"] == (30, 20) and names["l0.mix.g"] == (50, 24)
    assert names["l1.mix.k"] == (24, 24) and names["l1.mix.v"] == (36, 24) and names["l1.mix.g"] == (6, 24) and names["l1.mix.temp"] == (6,)
    assert names["l0.mlp.router"] == (5, 24) and names["l0.mlp.correction"] == (5,) and "l0.mlp.e3.up" not in names and names["l0.mlp.e2.down"] == (24, 16)
    assert "l1.mlp.router" not in names and "l1.canon2" not in names and names["l1.canon1"] == (24, 4) and names["l2.canon2"] == (24, 4)
    assert names["side.embed"] == (33, 20) and names["l3.side.proj"] == (24, 5) and names["loop.in"] == (24, 48) and names["loop.step"] == (2, 24)
    sd = PemalornForCausalLM.random_state_dict(sh, seed=1)
    assert set(sd) == set(names) and all(tuple(sd[k].shape) == v for k, v in names.items())


def test_configurations_without_loop_convolutions_or_token_input():
    cfg = _config()
    for k in ("loop", "canon", "token_side"):
        del cfg[k]
    sh = PemalornShape.from_config(cfg)
    assert [r[0] for r in sh.runs] == [0, 1, 2, 3] and not any(r[2] for r in sh.runs) and sh.state_floats == 0
    names = tensor_shapes(sh)
    assert not any(k.startswith(("loop.", "side.")) or "canon" in k or ".side." in k for k in names)
    assert sh.to_config() == cfg
    one = PemalornShape.from_config(_config(canon={"taps": 1}))          # one tap is still a convolution: h (1 + w)
    assert tensor_shapes(one)["l0.canon1"] == (24, 1) and one.state_floats == 6 * 24 and one.to_config()["canon"] == {"taps": 1}
    whole = PemalornShape.from_config(_config(loop={"start": 0, "stop": 4, "times": 1}))      # one pass still enters through the loop's input
    assert [r[2] for r in whole.runs] == [True, False, False, False]
    empty = PemalornShape.from_config(_config(loop={"start": 3, "stop": 3, "times": 4}))      # a span without layers is no loop
    assert [r[0] for r in empty.runs] == [0, 1, 2, 3] and not empty.has_loop and "loop.in" not in tensor_shapes(empty)


def test_configurations_that_cannot_be():
    with pytest.raises(ValueError):
        PemalornShape.from_config(_config(architecture="Other"))
    for change in (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), lambda c: c["layers"][1]["mixer"].update(vdim=7),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), lambda c: c["layers"][0]["mixer"].update(rot_dim=3),
                   lambda c: c["layers"][0].update(type="other"), lambda c: c["layers"][0]["mlp"]["router"].update(top=6),
                   lambda c: c["layers"][0]["mlp"].update(kind="dense"), lambda c: c["loop"].update(stop=5)):
        cfg = _config()
        change(cfg)
        with pytest.raises(ValueError):
            PemalornShape.from_config(cfg)


def test_registry_knows_the_design(tmp_path):
    from hydrainfer_amd.model.registry import architecture_of, registered
    (tmp_path / "config.json").write_text(json.dumps(_config()))
    assert architecture_of(str(tmp_path)) == "Pemalorn" and "Pemalorn" in registered()


def test_restatement_rotations_by_hand():
    f, mag = oracle.pair_frequencies(4, 100.0)
    assert torch.allclose(f, torch.tensor([1.0, 0.1], dtype=F)) and mag == 1.0
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=F)
    quarter = torch.tensor([math.pi / 2], dtype=F)
    one = torch.tensor([1.0, 1.0], dtype=F)          # both pairs a quarter turn at this position
    assert torch.allclose(oracle.rotate(x, quarter, one, "halves"), torch.tensor([[-3.0, -4.0, 1.0, 2.0]], dtype=F))
    assert torch.allclose(oracle.rotate(x, quarter, one, "interleaved"), torch.tensor([[-2.0, 1.0, -4.0, 3.0]], dtype=F))
    pos = torch.tensor([7.0, 123.0], dtype=F)
    y = torch.randn(2, 3, 4, generator=torch.Generator().manual_seed(0)).to(F)
    for layout in ("halves", "interleaved"):
        assert torch.allclose(oracle.rotate(oracle.rotate(y, pos, f, layout), -pos, f, layout), y)
    # scaled frequencies: the fast pairs keep theirs, the slow ones are divided by the factor, cos and sin grow
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 0.5}
    fs, mag = oracle.pair_frequencies(16, 500.0, sc)
    f0, _ = oracle.pair_frequencies(16, 500.0)
    assert fs[0] == f0[0] and abs(fs[-1] - f0[-1] / 4.0) < 1e-15 and abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert ((fs <= f0 + 1e-18) & (fs >= f0 / 4.0 - 1e-18)).all()


def test_restatement_sink_window_and_identity_experts_by_hand():
    # two equal keys and a sink of the same score: each key gets a third, the sink's third carries no value
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]], dtype=F)
    k = torch.tensor([[[2.0, 5.0]], [[2.0, -1.0]]], dtype=F)
    v = torch.tensor([[[3.0]], [[9.0]]], dtype=F)
    out = oracle.sink_softmax_attention(q, k, v, torch.tensor([0.5], dtype=F), torch.tensor([1.0], dtype=F), None)
    assert torch.allclose(out[:, 0, 0], torch.tensor([1.5, 4.0], dtype=F))
    out = oracle.sink_softmax_attention(q, k, v, torch.tensor([0.5], dtype=F), torch.tensor([1.0], dtype=F), 1)      # a window of one: itself
    assert torch.allclose(out[:, 0, 0], torch.tensor([1.5, 4.5], dtype=F))
    # the convolution adds to its input; before the first token there are zeros
    h = torch.tensor([[1.0], [10.0], [100.0]], dtype=F)
    assert torch.allclose(oracle.input_conv(h, torch.tensor([[0.5, 0.25, 2.0]], dtype=F)), torch.tensor([[3.0], [30.25], [303.0]], dtype=F))
    # a router that prefers its identity output: the token comes back, times its (unnormalised) score
    W = {"m.router": torch.tensor([[0.0, 0.0], [4.0, 0.0]], dtype=F), "m.correction": torch.zeros(2, dtype=F),
         "m.e0.gate": torch.ones(3, 2, dtype=F), "m.e0.up": torch.ones(3, 2, dtype=F), "m.e0.down": torch.ones(2, 3, dtype=F)}
    x = torch.tensor([[1.0, -2.0]], dtype=F)
    out = oracle.expert_mixture(x, W, "m.", {"router": {"experts": 1, "identity": 1, "top": 1}})
    assert torch.allclose(out, x * torch.sigmoid(torch.tensor(4.0, dtype=F)))
    # a correction turns the choice round, the weight stays the score
    W["m.correction"] = torch.tensor([5.0, 0.0], dtype=F)
    out = oracle.expert_mixture(x, W, "m.", {"router": {"experts": 1, "identity": 1, "top": 1}})
    inner = oracle.silu(torch.tensor(-1.0, dtype=F)) * -1.0
    assert torch.allclose(out, (1 - torch.sigmoid(torch.tensor(4.0, dtype=F))) * 3.0 * inner * torch.ones(1, 2, dtype=F))


def test_restatement_loop_runs_and_layer_count():
    cfg = _config()
    assert [(i, t, f) for i, t, f in oracle.run_order(cfg)] == [(0, 0, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (3, 0, False)]
    sh = PemalornShape.from_config(cfg)
    W = {k: v.float() for k, v in PemalornForCausalLM.random_state_dict(sh, seed=2).items()}
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7]
    trace = []
    logits = oracle.forward(toks, W, cfg, trace)
    assert logits.shape == (len(toks), 33) and len(trace) == 6 and torch.isfinite(logits).all()
    # causal: a longer sequence's first positions are the shorter one's
    assert torch.allclose(oracle.forward(toks[:9], W, cfg), logits[:9], atol=1e-12)
