"""The Saposun design without a GPU: the configuration's round trip and its errors, the declared tensors, and the
plain implementation pinned by hand-worked cases: what a query sees around the window's edge and around a pooled
block's completion, the pooled softmax by hand, the retention against its closed form, the router's correction,
and the two rotations' pairings."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_saposun as ps
import saposun_util as su


def test_configuration_round_trip_and_what_it_leaves_out():
    from hfee_amd.config import ConfigError, config_from_dict
    for cj in list(su.CONFIGS.values()) + list(su.SINGLE.values()):
        cfg = config_from_dict(cj)
        assert cfg.to_dict() == cj
        assert config_from_dict(cfg.to_dict()) == cfg
    cfg = config_from_dict(su.P_A)
    assert cfg.residual_mult == 0.5 and cfg.layers[3].mixer.kv_from == 0 and cfg.layers[3].mlp is None
    assert cfg.layers[2].mixer.pool == 5 and cfg.layers[2].mixer.conv == 3 and cfg.layers[5].mixer.softcap == 0.0
    bare = config_from_dict(su.SINGLE["attention without anything"]).layers[0].mixer
    assert (bare.window, bare.pool, bare.conv, bare.softcap, bare.rot) == (0, 0, 0, 0.0, None)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_rank=16), "must equal"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5, 1.5]), "between 0 and 1"),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(pool=4), "pooled"),
    (lambda c: c["layers"][2].update(type="other"), "unknown mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense", ff=8), "moe"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "cannot use"),
    (lambda c: c.pop("width"), "width"),
])
def test_configuration_errors(change, message):
    from hfee_amd.config import ConfigError, config_from_dict
    cj = copy.deepcopy(su.P_A)
    change(cj)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(cj)


def test_declared_tensors():
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    shapes = {s.name: tuple(s.shape) for s in declared_tensors(config_from_dict(su.P_A))}
    assert shapes["l0.mix.dkv"] == (32 + 16, 64) and shapes["l0.mix.uq"] == (4 * 32, 24) and shapes["l0.mix.dq.norm"] == (24,)
    assert "l3.mix.dkv" not in shapes and "l3.mix.dkv.norm" not in shapes and shapes["l3.mix.uk"] == (4 * 16, 32)
    assert shapes["l1.mix.g"] == (64, 64) and shapes["l1.mix.o"] == (64, 64)
    assert shapes["l2.mix.q.conv"] == (128, 3) and shapes["l2.mix.k.conv"] == (64, 3) and shapes["l2.mix.v.conv"] == (32, 3)
    assert shapes["l2.mix.g"] == (4, 64) and shapes["l2.mlp.correction"] == (6,) and shapes["l2.mlp.e5.down"] == (64, 32)
    assert not any(n.startswith("l3.mlp") for n in shapes) and shapes["final.norm"] == (64,) and shapes["head"] == (131, 64)
    bare = {s.name for s in declared_tensors(config_from_dict(su.SINGLE["attention without anything"]))}
    assert "l0.mix.q.conv" not in bare and "l0.mix.g" in bare


def _one_layer(layer, width=24, vocab=40, seed=0):
    cj = su.config(vocab, width, 1e-6, 1.0, [su.bare(layer)])
    return cj, {n: t.double() for n, t in su.make_tensors(cj, seed, std=0.3).items()}


def _moved_by(cj, w, tokens, at, change):
    """Whether the logits at `at` move when the token at `change` is another one."""
    other = list(tokens)
    other[change] = (other[change] + 1) % cj["vocab"]
    a, b = ps.forward(tokens, w, cj)[at], ps.forward(other, w, cj)[at]
    return bool((a - b).abs().max() > 1e-9)


def test_what_a_query_sees_around_a_window_and_a_block():
    """One layer, so a position's input is its own token: the logits at i move with token j exactly if i sees j."""
    tokens = list(np.random.default_rng(0).integers(0, 40, size=40))
    cj, w = _one_layer(su.latent(2, 4, 4, 4, 6, 8, 0.5, window=6))
    assert _moved_by(cj, w, tokens, 30, 25) and not _moved_by(cj, w, tokens, 30, 24) and _moved_by(cj, w, tokens, 30, 30)
    assert not _moved_by(cj, w, tokens, 30, 31) and _moved_by(cj, w, tokens, 3, 0)
    # window 10 and blocks of 3: position 30 sees 21..30 and the blocks that end at or before 20: 0..6 (18..20)
    cj, w = _one_layer(su.attention(2, 1, 4, 4, 0.5, window=10, pool=3))
    assert _moved_by(cj, w, tokens, 30, 21) and _moved_by(cj, w, tokens, 30, 20) and _moved_by(cj, w, tokens, 30, 0)
    # position 31 sees 22..31 and blocks up to the one that ends at 20: token 21 has left the window and its block
    # (21..23) is not seen before position 33
    assert not _moved_by(cj, w, tokens, 31, 21) and not _moved_by(cj, w, tokens, 32, 21) and _moved_by(cj, w, tokens, 33, 21)
    assert not _moved_by(cj, w, tokens, 32, 22) and _moved_by(cj, w, tokens, 33, 23) and _moved_by(cj, w, tokens, 33, 24)
    # the convolution reaches taps - 1 tokens further back
    cj, w = _one_layer(su.attention(2, 1, 4, 4, 0.5, window=4, conv=3))
    assert _moved_by(cj, w, tokens, 30, 25) and not _moved_by(cj, w, tokens, 30, 24)


def test_the_pooled_softmax_by_hand():
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "mask": {"size": 2, "pool": 2}, "softcap": 1.5}
    k = torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.0], [0.0, 2.0], [1.0, 1.0]], dtype=torch.float64)
    h = k.clone()
    eye = torch.eye(2, dtype=torch.float64)
    w = {"q": eye, "k": eye, "v": eye, "g": torch.zeros(1, 2, dtype=torch.float64), "o": eye}
    out = ps.pooled_window_attention(h, w, "", m, 0.0)
    # position 4 sees tokens 3, 4 and block 0 (tokens 0, 1; block 1 ends at 3 > 4 - 2)
    q = k[4]
    v = k / torch.sqrt((k * k).mean(-1, keepdim=True))
    keys = torch.stack([k[3], k[4], (k[0] + k[1]) / 2])
    values = torch.stack([v[3], v[4], (v[0] + v[1]) / 2])
    s = 1.5 * torch.tanh(keys @ q / 1.5)
    want = 0.5 * (torch.softmax(s, 0) @ values)           # (the gate's logits are zero: sigmoid 1/2)
    assert torch.allclose(out[4], want, atol=1e-12)


def test_retention_against_its_closed_form():
    cj, w = _one_layer(su.retention(2, 4, 6, (0.9, 1.0), rot_dims=4), seed=3)
    m, T = cj["layers"][0]["mixer"], 12
    h = torch.randn(T, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    pre = "l0.mix."
    pos = torch.arange(T)
    q = ps.rotate_half((h @ w[pre + "q"].T).view(T, 2, 4), pos, 4, 10000.0)
    k = ps.rotate_half((h @ w[pre + "k"].T).view(T, 2, 4), pos, 4, 10000.0) / 2.0
    v = (h @ w[pre + "v"].T).view(T, 2, 6)
    o = torch.zeros(T, 2, 6, dtype=torch.float64)
    for t in range(T):
        for j in range(t + 1):
            for hd, d in enumerate((0.9, 1.0)):
                o[t, hd] += d ** (t - j) * (q[t, hd] @ k[j, hd]) * v[j, hd]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6)
    want = (o.reshape(T, 12) * torch.nn.functional.silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T
    assert torch.allclose(ps.retention(h, w, pre, m, 1e-6), want, atol=1e-10)


def test_the_correction_chooses_and_does_not_weigh():
    g = torch.Generator().manual_seed(0)
    h = torch.randn(5, 8, dtype=torch.float64, generator=g)
    w = {"router": torch.randn(4, 8, dtype=torch.float64, generator=g), "correction": torch.zeros(4, dtype=torch.float64)}
    chosen, weights, _ = ps.router(h, w, "", {"top": 2})
    scores = torch.softmax(h @ w["router"].T, -1)
    assert torch.equal(chosen, scores.argsort(-1, descending=True)[:, :2]) and torch.allclose(weights, torch.gather(scores, 1, chosen))
    w["correction"][3] = 5.0
    chosen, weights, _ = ps.router(h, w, "", {"top": 2})
    assert (chosen[:, 0] == 3).all() and torch.allclose(weights[:, 0], scores[:, 3])
    assert float(weights.sum(-1).max()) < 1.0            # (not renormalized)


def test_pairs_side_by_side_are_pairs_half_apart_in_another_order():
    """What the product does for the latent layers: with the rotated dims of q and k in the order evens, odds,
    turning pairs (i, i + half) gives the same scores as turning pairs (2i, 2i + 1) in the file's order."""
    g = torch.Generator().manual_seed(4)
    q, k = torch.randn(7, 2, 8, dtype=torch.float64, generator=g), torch.randn(7, 1, 8, dtype=torch.float64, generator=g)
    pos = torch.arange(7) + 11
    a = torch.einsum("ihd,jd->hij", ps.rotate_interleaved(q, pos, 8, 100.0), ps.rotate_interleaved(k, pos, 8, 100.0)[:, 0])
    order = torch.cat([torch.arange(0, 8, 2), torch.arange(1, 8, 2)])
    b = torch.einsum("ihd,jd->hij", ps.rotate_half(q[..., order], pos, 8, 100.0), ps.rotate_half(k[..., order], pos, 8, 100.0)[:, 0])
    assert torch.allclose(a, b, atol=1e-12)
    first = ps.rotate_interleaved(q, pos, 8, 100.0)
    ang = 11 * 100.0 ** (-2.0 / 8)
    assert math.isclose(float(first[0, 0, 2]), float(q[0, 0, 2] * math.cos(ang) - q[0, 0, 3] * math.sin(ang)), abs_tol=1e-12)


def test_a_prefix_does_not_depend_on_what_follows():
    cj = su.P_A
    w = su.make_tensors(cj, 5)
    tokens = list(np.random.default_rng(2).integers(0, cj["vocab"], size=50))
    full = ps.forward(tokens, w, cj)
    assert torch.allclose(ps.forward(tokens[:31], w, cj), full[:31], atol=1e-9)
