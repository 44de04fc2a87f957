"""CPU: the host side of the Fasanex integration — configuration reading, cache planes and state pieces, tensor names,
rotary frequencies, the model registry — and the float64 restatement's own mechanisms on cases worked out by hand."""
import json
import math

import pytest
import torch

import tests.fasanex_oracle as oracle
from hydrainfer_amd.model.fasanex import FasanexForCausalLM, FasanexShape, RotarySpec, tensor_shapes


def _config(**over):
    left = {"conv": 2, "dim": 8, "heads": 6, "kv_heads": 3, "vdim": 8, "scale": 0.25, "softcap": 9.0, "mask": {"size": 11},
            "rot": {"base": 500.0, "dims": 4, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}}}
    par = {"left": left, "left_scale": 0.6, "right": {"dim": 4, "heads": 5}, "right_scale": 1.4}
    ssm = {"conv": 3, "groups": 2, "heads": 4, "norm_groups": 4, "state": 6, "vdim": 10}
    dl = {"conv": 5, "dim": 4, "heads": 6, "kv_heads": 2, "vdim": 3}
    cfg = {"architecture": "Fasanex", "vocab": 33, "width": 24, "norm": {"eps": 1e-4}, "embedding": {"scale": 2.5},
           "layers": [{"type": "delta", "mixer": dict(dl), "mlp": {"kind": "dense", "ff": 40, "limit": 3.0}},
                      {"type": "parallel", "mixer": json.loads(json.dumps(par)), "mlp": None},
                      {"type": "mamba2", "mixer": dict(ssm), "mlp": {"kind": "dense", "ff": 8, "limit": 0.5}},
                      {"type": "parallel", "mixer": json.loads(json.dumps(par)), "mlp": {"kind": "dense", "ff": 16}}]}
    cfg.update(over)
    return cfg


def test_shape_from_config_planes_pieces_and_names():
    sh = FasanexShape.from_config(_config())
    assert sh.cache_plane == {1: 0, 3: 1} and sh.num_hidden_layers == 2
    assert (sh.num_attention_heads, sh.num_key_value_heads, sh.head_dim) == (6, 3, 8)
    assert sh.norm_eps == 1e-4 and sh.embedding_scale == 2.5 and sh.layers[1].mlp is None
    assert sh.layers[0].mlp.limit == 3.0 and sh.layers[3].mlp.limit is None
    a = sh.layers[1].mixer.left
    assert (a.window, a.softcap, a.conv, a.rot.dims, a.rot.factor, a.rot.original) == (11, 9.0, 2, 4, 4.0, 64.0)
    assert (sh.layers[1].mixer.left_scale, sh.layers[1].mixer.right_scale) == (0.6, 1.4)
    # a slot's pieces follow each other in layer order, each starting on a multiple of four floats
    want, at = {}, 0
    for key, size in (((0, "conv"), 4 * (2 * 2 * 4 + 6 * 3)), ((0, "S"), 6 * 4 * 3), ((1, "conv"), 1 * 9 * 8), ((1, "shift"), 24),
                      ((1, "S"), 5 * 4 * 4), ((2, "conv"), 2 * (40 + 24)), ((2, "S"), 4 * 6 * 10), ((3, "conv"), 72), ((3, "shift"), 24),
                      ((3, "S"), 80)):
        want[key] = at
        at += (size + 3) // 4 * 4
    assert sh.state_piece == want and sh.state_floats == at
    assert FasanexShape.from_config(sh.to_config()).to_config() == sh.to_config()
    names = tensor_shapes(sh)
    assert names["l0.mix.q"] == (8, 24) and names["l0.mix.v.conv"] == (18, 5) and names["l0.mix.b"] == (6, 24) and names["l0.mix.norm"] == (3,)
    assert names["l1.mix.left.k"] == (24, 24) and names["l1.mix.left.q.conv"] == (48, 2) and names["l1.mix.left.k.norm"] == (8,)
    assert names["l1.mix.right.w2"] == (20, 16) and names["l1.mix.right.u"] == (5, 4) and names["l1.mix.right.mu.w"] == (24,)
    assert "l1.mix.left.v" not in names and "l1.norm2" not in names and "l1.mlp.up" not in names
    assert names["l2.mix.in"] == (2 * 40 + 2 * 12 + 4, 24) and names["l2.mix.conv"] == (64, 3) and names["l2.mix.D"] == (4,)
    assert names["l3.mlp.down"] == (24, 16) and names["head"] == (33, 24)
    sd = FasanexForCausalLM.random_state_dict(sh, seed=1)
    assert set(sd) == set(names) and all(tuple(sd[k].shape) == v for k, v in names.items())


def test_configurations_that_cannot_be():
    with pytest.raises(ValueError):
        FasanexShape.from_config(_config(architecture="Other"))
    for layer, key, value in ((1, ("left", "kv_heads"), 4), (1, ("left", "vdim"), 6), (2, ("groups",), 3), (2, ("norm_groups",), 7),
                              (0, ("kv_heads",), 4)):
        bad = _config()
        m = bad["layers"][layer]["mixer"]
        for k in key[:-1]:
            m = m[k]
        m[key[-1]] = value
        with pytest.raises(ValueError):
            FasanexShape.from_config(bad)
    bad = _config()
    bad["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        FasanexShape.from_config(bad)
    bad = _config()
    bad["layers"][1]["mixer"]["left"]["rot"]["dims"] = 10          # more turning channels than a head has
    with pytest.raises(ValueError):
        FasanexShape.from_config(bad)


def test_rotary_frequencies_plain_and_scaled():
    f, m = RotarySpec(8, 100.0).frequencies()
    assert m == 1.0 and f == pytest.approx([1.0, 100.0 ** -0.25, 0.1, 100.0 ** -0.75])
    # scaled: the pair index at which a full turn takes `original / t` positions; fast pairs keep their frequency, slow ones are
    # divided by the factor
    spec = RotarySpec(16, 10000.0, 8.0, 256.0, 16.0, 1.0)
    f, m = spec.frequencies()
    plain = [10000.0 ** (-2.0 * i / 16) for i in range(8)]
    turn = lambda t: 16 * math.log(256.0 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(turn(16.0)), 0), min(math.ceil(turn(1.0)), 15)
    assert (lo, hi) == (0, 4) and m == pytest.approx(0.1 * math.log(8.0) + 1.0)
    for i in range(8):
        r = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        assert f[i] == pytest.approx(plain[i] / 8.0 * r + plain[i] * (1.0 - r))
    assert f[0] == plain[0] and f[7] == pytest.approx(plain[7] / 8.0)
    of, om = oracle.yarn_frequencies({"dims": 16, "base": 10000.0, "scaling": {"factor": 8.0, "original": 256.0, "fast": 16.0, "slow": 1.0}})
    assert om == pytest.approx(m) and of.tolist() == pytest.approx(f)


def test_registry_knows_the_design(tmp_path):
    from hydrainfer_amd.model.registry import architecture_of, registered
    (tmp_path / "config.json").write_text(json.dumps(_config()))
    assert "Fasanex" in registered() and architecture_of(str(tmp_path)) == "Fasanex"


def test_oracle_mechanisms_by_hand():
    F = oracle.F
    # a convolution of three taps: y_t = w0 u_(t-2) + w1 u_(t-1) + w2 u_t
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=F)
    assert oracle.short_conv(u, torch.tensor([[100.0, 10.0, 1.0]], dtype=F)).flatten().tolist() == [1.0, 12.0, 124.0]
    # the rotation turns channel i with channel i + dims / 2 and leaves the rest
    x = torch.tensor([[[1.0, 0.0, 5.0]]], dtype=F)
    out = oracle.rotate(x, torch.tensor([1]), {"dims": 2, "base": 10.0})
    assert out.flatten().tolist() == pytest.approx([math.cos(1.0), math.sin(1.0), 5.0])
    # the feed-forward's clamp: the gate from above only, the other side from both
    W = {"gate": torch.tensor([[10.0], [-10.0]], dtype=F), "up": torch.tensor([[10.0], [-10.0]], dtype=F), "down": torch.eye(2, dtype=F)}
    y = oracle.dense_ff(torch.ones(1, 1, dtype=F), W, "", {"limit": 2.0})
    assert y.flatten().tolist() == pytest.approx([2.0 / (1 + math.exp(-3.404)) * 3.0, -10.0 / (1 + math.exp(17.02)) * -1.0])
    # the delta rule with unit decay, full write strength: the state answers a written key with its value, and a second write
    # to the same key replaces it
    cfg = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "conv": 1}
    big = 30.0
    Wd = {"q": torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=F), "k": torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=F), "v": torch.tensor([[0.0, 0.0]], dtype=F),
          "q.conv": torch.ones(2, 1, dtype=F), "k.conv": torch.ones(2, 1, dtype=F), "v.conv": torch.ones(1, 1, dtype=F),
          "b": torch.tensor([[big, big]], dtype=F), "a": torch.tensor([[-big, -big]], dtype=F), "A_log": torch.zeros(1, dtype=F),
          "dt_bias": torch.zeros(1, dtype=F), "norm": torch.ones(1, dtype=F), "g": torch.tensor([[big, big]], dtype=F), "o": torch.ones(1, 1, dtype=F)}
    h = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 0.0]], dtype=F)
    Wd["v"] = torch.tensor([[3.0, -2.0]], dtype=F)
    out = oracle.delta(h, Wd, "", cfg, 0.0)
    assert torch.sign(out.flatten()).tolist() == [1.0, -1.0, 1.0]          # after its norm only the sign of each read-out is left
