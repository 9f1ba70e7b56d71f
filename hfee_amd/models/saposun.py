"""The Saposun decoder as a list of parts.

Every layer is a "parallel" block: one RMS norm whose output both the mixer and the feed-forward read,
x += m * (mixer(h) + feed_forward(h)) with one number m for the whole model.  The mixer of a layer is latent
attention over a sliding window, possibly reading the keys that an earlier latent layer keeps
("latent_attention"); retention, linear attention with a fixed decay a head ("retention"); or grouped
attention behind short convolutions, with normed values, capped scores, a sliding window with pooled blocks
before it and a gate a head ("window_attention").  The feed-forward is gated experts that a router chooses
by the softmax of its logits plus a learned correction ("routed_moe"), or none.  Which layer has which, and
every size and constant, is config.json's.

What is fixed here is what the design fixes: rotation pairs (2i, 2i + 1) in the latent layers and
(i, i + dims/2) in the others, the latents' norms with plain weights and the layer's eps, the weightless norms
of the values and of the retention's heads, the gate a head, scores that are not renormalized and multiply an
expert's output.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.saposun import PooledAttentionConfig, RetentionConfig, SaposunConfig, WindowLatentConfig
from ..config.specs import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec, ScheduleEntry, params


def _rope(head_dim: int, rot, pairing: str):
    if rot is None:
        return None
    return PositionSpec("rope", params(head_dim=head_dim, rotary_dim=rot.dims, theta=rot.base, scaling=None, pairing=pairing))


def _kept_positions(cfg: SaposunConfig, i: int) -> int:
    """How many positions the cache layer that latent layer i reads must keep: the widest window of the layers
    that read it (0: one of them sees every earlier position, so every token is kept)."""
    source = cfg.layers[i].mixer.kv_from if cfg.layers[i].mixer.kv_from is not None else i
    windows = [l.mixer.window for k, l in enumerate(cfg.layers)
               if isinstance(l.mixer, WindowLatentConfig) and (k == source or l.mixer.kv_from == source)]
    return 0 if not all(windows) else max(windows)


def _mixer(cfg: SaposunConfig, m, i: int = 0) -> MixerSpec:
    if isinstance(m, WindowLatentConfig):
        return MixerSpec("latent_attention", params(
            hidden=cfg.width, num_heads=m.heads, plain_dim=m.dim, rotated_dim=m.rot_dim, value_dim=m.vdim,
            q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, norm_eps=cfg.norm_eps, window=m.window,
            own_keys=m.kv_from is None, cache_window=_kept_positions(cfg, i),
            names=(("q_down", "dq"), ("q_norm", "dq.norm"), ("q_up", "uq"), ("kv_down", "dkv"),
                   ("kv_norm", "dkv.norm"), ("k_up", "uk"), ("v_up", "uv"), ("o", "o"))),
            position=_rope(m.rot_dim, m.rot, "interleaved"))
    if isinstance(m, RetentionConfig):
        return MixerSpec("retention", params(
            hidden=cfg.width, num_heads=m.heads, dim=m.dim, vdim=m.vdim, decay=m.decay, norm_eps=cfg.norm_eps,
            names=(("q", "q"), ("k", "k"), ("v", "v"), ("g", "g"), ("o", "o"))),
            position=_rope(m.dim, m.rot, "half"))
    if isinstance(m, PooledAttentionConfig):
        return MixerSpec("window_attention", params(
            hidden=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim, scale=m.scale,
            softcap=m.softcap, conv=m.conv, window=m.window, pool=m.pool, value_norm_eps=cfg.norm_eps, head_gate=True,
            names=(("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_conv", "q.conv"), ("k_conv", "k.conv"),
                   ("v_conv", "v.conv"), ("head_gate", "g"))),
            position=_rope(m.dim, m.rot, "half"))
    raise ValueError(f"no part for a mixer of type {m.type!r}")


def _feed_forward(cfg: SaposunConfig, mlp):
    if mlp is None:
        return None
    return FeedForwardSpec("routed_moe", params(
        hidden=cfg.width, intermediate=mlp.ff, experts=mlp.experts, top=mlp.top, activation="silu", score="softmax",
        weight_on="output", renormalize=False, correction=True,
        names=(("expert", "e{}."), ("gate", "gate"), ("up", "up"), ("down", "down"), ("router", "router"),
               ("correction", "correction"))))


def saposun_model_spec(cfg: SaposunConfig) -> ModelSpec:
    norm = NormSpec("rmsnorm", cfg.width, cfg.norm_eps)
    layers = tuple(
        LayerSpec(arrangement="parallel", hidden=cfg.width, mixer=_mixer(cfg, layer.mixer, i),
                  feed_forward=_feed_forward(cfg, layer.mlp), mixer_norm=norm, feed_forward_norm=norm, prefix=f"l{i}.",
                  names=(("mixer", "mix."), ("feed_forward", "mlp."), ("mixer_norm", "norm1")),
                  params=params(residual_scale=cfg.residual_mult))
        for i, layer in enumerate(cfg.layers))
    # a layer that reads another's keys runs on that layer's cache layer and writes nothing
    schedule = []
    for i, layer in enumerate(cfg.layers):
        source = getattr(layer.mixer, "kv_from", None)
        schedule.append(ScheduleEntry(layer=i, cache=i) if source is None else ScheduleEntry(layer=i, cache=source, writes_cache=False))
    return ModelSpec(
        architecture=cfg.architecture, hidden=cfg.width, vocab=cfg.vocab, layers=layers, schedule=tuple(schedule),
        final_norm=norm, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_ids=tuple(cfg.eos_token_ids), bos_token_id=cfg.bos_token_id)


register_architecture("Saposun", SaposunConfig, saposun_model_spec)
