"""The Ronavik design on the CPU: its configuration, the tensors its parts declare, and the plain
implementation's own properties (what the GPU tests compare the engine with)."""
import copy
import math

import pytest
import torch

import plain_ronavik as pr
import ronavik_util as ru


def test_configuration_round_trip_and_errors():
    from hfee_amd.config import ConfigError, config_from_dict
    for cj in list(ru.CONFIGS.values()) + list(ru.SINGLE.values()):
        cfg = config_from_dict(cj)
        again = cfg.to_dict()
        assert config_from_dict(again) == cfg
        assert len(cfg.layers) == len(cj["layers"])
    # what the file leaves out has its default: no temperature, scales of one, as many key heads as heads
    cfg = config_from_dict(ru.R_B)
    left = cfg.layers[1].mixer.left
    assert left.q_temp is None and left.kv_heads == left.heads and cfg.layers[1].mixer.left_scale == 1.0
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.top == 4
    bad = copy.deepcopy(ru.R_A)
    bad["layers"][0]["mixer"]["left"]["kv_heads"] = 3
    bad["layers"][1]["mixer"]["norm_groups"] = 5
    del bad["max_positions"]
    with pytest.raises(ConfigError) as e:
        config_from_dict(bad)
    assert "max_positions" in str(e.value)
    bad = copy.deepcopy(ru.R_A)
    bad["layers"][0]["mixer"]["left"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="kv_heads"):
        config_from_dict(bad)
    bad = copy.deepcopy(ru.R_A)
    bad["layers"][1]["type"] = "mamba3"
    with pytest.raises(ConfigError, match="unknown mixer type"):
        config_from_dict(bad)
    bad = copy.deepcopy(ru.R_A)
    bad["layers"][0]["mixer"]["right"]["blocks"] = 5
    with pytest.raises(ConfigError, match="equal blocks"):
        config_from_dict(bad)


def test_declared_tensors():
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    specs = {s.name: tuple(s.shape) for s in declared_tensors(config_from_dict(ru.R_A))}
    assert specs["embed"] == (131, 64) and specs["pos"] == (512, 64) and "head" not in specs
    assert specs["l0.mix.left.q"] == (64, 64) and specs["l0.mix.left.k"] == (32, 64) and specs["l0.mix.left.v"] == (64, 64)
    assert specs["l0.mix.left.o"] == (64, 128) and specs["l0.mix.left.q.norm"] == (16,) and specs["l0.mix.left.pb"] == (4,)
    assert specs["l0.mix.right.ra"] == (3, 16, 16) and specs["l0.mix.right.ri.b"] == (3, 16) and specs["l0.mix.right.conv"] == (48, 4)
    assert specs["l1.mix.in"] == (2 * 32 + 2 * 32 + 4, 64) and specs["l1.mix.conv"] == (32 + 64, 4) and specs["l1.mix.D"] == (4,)
    assert specs["l1.mix.norm"] == (32,) and specs["l0.rg1"] == (64, 64) and specs["l0.rg2.b"] == (64,)
    assert specs["l0.mlp.router"] == (5, 64) and specs["l0.mlp.e4.up"] == (24, 64) and specs["l0.mlp.e4.down"] == (64, 24)
    assert "l2.mlp.router" not in specs and "l2.rg2" not in specs and "l2.norm2" not in specs and "l2.rg1" in specs


def _w(cj, seed=3):
    return ru.make_tensors(cj, seed)


def test_a_prefix_does_not_change_with_what_follows():
    w = _w(ru.R_A)
    toks = torch.randint(0, 131, (40,), generator=torch.Generator().manual_seed(0)).tolist()
    full = pr.forward(ru.R_A, w, toks)
    part = pr.forward(ru.R_A, w, toks[:23])
    assert torch.allclose(full[:23], part, atol=1e-10)


def test_a_first_token_shows_far_behind_it_through_every_mixer():
    for name in ("sigmoid attention", "recurrent unit", "state space"):
        cj = ru.SINGLE[name]
        w = _w(cj)
        g = torch.Generator().manual_seed(1)
        toks = torch.randint(0, 50, (60,), generator=g).tolist()
        other = [(toks[0] + 1) % 50] + toks[1:]
        a, b = pr.forward(cj, w, toks), pr.forward(cj, w, other)
        assert (a[-1] - b[-1]).abs().max() > 1e-9 * a[-1].abs().max(), name


def test_sigmoid_weights_by_hand():
    """One head, one key: the output is sigmoid(q.k * scale + b) * v; a second key adds its own share and takes
    nothing from the first (no normalization)."""
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "q_temp": {"coef": 2.0, "every": 2}}
    g = torch.Generator().manual_seed(2)
    w = {"a.q": torch.randn(4, 6, generator=g), "a.k": torch.randn(4, 6, generator=g), "a.v": torch.randn(3, 6, generator=g),
         "a.q.norm": torch.rand(4, generator=g) + 0.5, "a.k.norm": torch.rand(4, generator=g) + 0.5,
         "a.pb": torch.tensor([-0.3]), "a.o": torch.eye(3)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(2, 6, generator=g).double()
    out = pr.sigmoid_attention(h, w, "a.", m, 1e-6)

    def normed(x, weight):
        return x / torch.sqrt((x * x).mean() + 1e-6) * weight
    q = [normed(w["a.q"] @ h[i], w["a.q.norm"]) for i in range(2)]
    k = [normed(w["a.k"] @ h[i], w["a.k.norm"]) for i in range(2)]
    v = [w["a.v"] @ h[i] for i in range(2)]
    q[1] = q[1] * (1 + 2.0 * math.log(2 // 2 + 1))           # position 1: floor((1 + 1) / 2) = 1
    first = torch.sigmoid(q[0] @ k[0] * 0.5 - 0.3) * v[0]
    second = torch.sigmoid(q[1] @ k[0] * 0.5 - 0.3) * v[0] + torch.sigmoid(q[1] @ k[1] * 0.5 - 0.3) * v[1]
    assert torch.allclose(out[0], first, atol=1e-12) and torch.allclose(out[1], second, atol=1e-12)


def test_an_expert_weight_multiplies_the_input():
    """With the square of relu, a weight w on the input is w^2 on the output; on the output it would be w."""
    g = torch.Generator().manual_seed(4)
    mlp = {"kind": "moe", "expert": {"ff": 5}, "router": {"experts": 3, "top": 2}}
    w = {"m.router": torch.randn(3, 6, generator=g).double()}
    for e in range(3):
        w[f"m.e{e}.up"] = torch.randn(5, 6, generator=g).double()
        w[f"m.e{e}.down"] = torch.randn(6, 5, generator=g).double()
    h = torch.randn(1, 6, generator=g).double()
    out = pr.routed_experts(h, w, "m.", mlp)[0]
    s = torch.sigmoid(w["m.router"] @ h[0])
    best = torch.argsort(s, descending=True)[:2]
    want = sum(s[e] ** 2 * (w[f"m.e{int(e)}.down"] @ torch.relu(w[f"m.e{int(e)}.up"] @ h[0]) ** 2) for e in best)
    assert torch.allclose(out, want, atol=1e-12)


def test_the_recurrent_unit_keeps_what_a_closed_gate_lets_through():
    """A decay gate far below zero leaves a = 1 - tiny: the state keeps its first input for hundreds of tokens;
    far above zero the state forgets within a few."""
    W = 4
    base = {"r.y": torch.zeros(W, 3), "r.y.b": torch.full((W,), 3.0), "r.x": torch.zeros(W, 3), "r.x.b": torch.zeros(W),
            "r.conv": torch.ones(W, 1), "r.conv.b": torch.zeros(W), "r.ra": torch.zeros(1, W, W), "r.ri": torch.zeros(1, W, W),
            "r.ri.b": torch.full((1, W), 30.0), "r.lam": torch.zeros(W), "r.o": torch.eye(W)}
    base["r.x"][:, 0] = 1.0
    h = torch.zeros(200, 3)
    h[0, 0] = 1.0
    for gate, kept in ((-30.0, True), (30.0, False)):
        w = {k: v.double() for k, v in dict(base, **{"r.ra.b": torch.full((1, W), gate)}).items()}
        out = pr.gated_linear_recurrent_unit(h.double(), w, "r.", {"width": W, "blocks": 1, "conv": 1})
        assert (out[199].abs().max() > 0.5 * out[0].abs().max()) == kept
