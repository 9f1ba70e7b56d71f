"""The Ronavik decoder as a list of parts.

The lookup adds a learned vector a position.  Every layer is a "sandwich" block whose sub-layers' results
pass a gate before their norm: with h = norm_a(x), x += norm_b(mixer(h) * sigmoid(W_g h + b_g)), then the
same around the feed-forward; all norms are RMS norms with plain weights.  The mixer of a layer is two
mixers side by side ("side_by_side": attention without a softmax, "sigmoid_attention", beside a real-gated
linear recurrent unit, "rglru", their results weighted by two numbers of the file) or a state-space mixer
("state_space"); the feed-forward is experts that a router chooses ("routed_moe"), or none.  The head
shares the lookup's table.  Which layer has which, and every size and constant, is config.json's.

What is fixed here is what the design fixes: no rotation, the norms of q and k with a weight shared by
the heads, the 8 in the recurrent unit's decay, sigmoid scores that are not renormalized and multiply an
expert's input, the square of relu, a gate on every sub-layer.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.ronavik import RonavikConfig, SideBySideConfig, StateSpaceConfig
from ..config.specs import EmbeddingSpec, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, ScheduleEntry, params


def _mixer(cfg: RonavikConfig, m) -> MixerSpec:
    if isinstance(m, SideBySideConfig):
        a, u = m.left, m.right
        left = MixerSpec("sigmoid_attention", params(
            hidden=cfg.width, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim, scale=a.scale,
            norm_eps=cfg.norm_eps, temperature=None if a.q_temp is None else (a.q_temp.coef, a.q_temp.every),
            names=(("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"),
                   ("head_bias", "pb"))))
        right = MixerSpec("rglru", params(
            hidden=cfg.width, width=u.width, blocks=u.blocks, conv=u.conv, decay_scale=8.0,
            names=(("y", "y"), ("y_bias", "y.b"), ("x", "x"), ("x_bias", "x.b"), ("conv", "conv"), ("conv_bias", "conv.b"),
                   ("decay_gate", "ra"), ("decay_gate_bias", "ra.b"), ("input_gate", "ri"), ("input_gate_bias", "ri.b"),
                   ("lam", "lam"), ("o", "o"))))
        return MixerSpec("side_by_side", params(hidden=cfg.width, left=left, right=right, left_scale=m.left_scale,
                                                right_scale=m.right_scale, names=(("left", "left."), ("right", "right."))))
    if isinstance(m, StateSpaceConfig):
        return MixerSpec("state_space", params(
            hidden=cfg.width, num_heads=m.heads, vdim=m.vdim, state=m.state, groups=m.groups, conv=m.conv,
            norm_groups=m.norm_groups, norm_eps=cfg.norm_eps,
            names=(("in", "in"), ("conv", "conv"), ("conv_bias", "conv.b"), ("dt_bias", "dt_bias"), ("a_log", "A_log"),
                   ("skip", "D"), ("norm", "norm"), ("o", "o"))))
    raise ValueError(f"no part for a mixer of type {m.type!r}")


def _feed_forward(cfg: RonavikConfig, mlp):
    if mlp is None:
        return None
    return FeedForwardSpec("routed_moe", params(
        hidden=cfg.width, intermediate=mlp.ff, experts=mlp.experts, top=mlp.top, activation="relu2", score="sigmoid",
        weight_on="input", renormalize=False,
        names=(("expert", "e{}."), ("up", "up"), ("down", "down"), ("router", "router"))))


def ronavik_model_spec(cfg: RonavikConfig) -> ModelSpec:
    norm = NormSpec("rmsnorm", cfg.width, cfg.norm_eps)
    layers = tuple(
        LayerSpec(arrangement="sandwich", hidden=cfg.width, mixer=_mixer(cfg, layer.mixer),
                  feed_forward=_feed_forward(cfg, layer.mlp), mixer_norm=norm, feed_forward_norm=norm, prefix=f"l{i}.",
                  names=(("mixer", "mix."), ("feed_forward", "mlp."), ("mixer_norm", "norm1"), ("mixer_post_norm", "norm1b"),
                         ("feed_forward_norm", "norm2"), ("feed_forward_post_norm", "norm2b"), ("mixer_gate", "rg1"),
                         ("mixer_gate_bias", "rg1.b"), ("feed_forward_gate", "rg2"), ("feed_forward_gate_bias", "rg2.b")),
                  params=params(residual_gate=True))
        for i, layer in enumerate(cfg.layers))
    schedule = tuple(ScheduleEntry(layer=i, cache=i) for i in range(len(layers)))
    return ModelSpec(
        architecture=cfg.architecture, hidden=cfg.width, vocab=cfg.vocab, layers=layers, schedule=schedule,
        final_norm=norm, embedding_name="embed", final_norm_name="final.norm", head_name=None,
        max_positions=cfg.max_positions, eos_token_ids=tuple(cfg.eos_token_ids), bos_token_id=cfg.bos_token_id,
        embedding=EmbeddingSpec("lookup", params(position_table="pos", positions=cfg.max_positions)))


register_architecture("Ronavik", RonavikConfig, ronavik_model_spec)
