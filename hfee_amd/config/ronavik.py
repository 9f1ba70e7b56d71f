"""RonavikConfig: the Ronavik decoder's configuration, read from config.json.

The file lists the layers one by one: each entry names its mixer (`type`: "parallel", two mixers side by
side, or "mamba2") with that mixer's sizes and constants (`mixer`), and its feed-forward (`mlp`:
{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}, or null for a layer without one).  Beside
the list it gives the vocabulary, the width, the norms' eps and the number of positions that have a
learned vector.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .base import ConfigError, KeyReader
from .sabezen import MoeConfig, _positive, _read_mlp


@dataclass(frozen=True)
class QueryTemperature:
    coef: float
    every: int

    def to_dict(self) -> dict:
        return {"coef": self.coef, "every": self.every}


@dataclass(frozen=True)
class SigmoidAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp: Optional[QueryTemperature]

    @staticmethod
    def read(data: dict, where: str) -> "SigmoidAttentionConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        kv_heads, vdim = r.int("kv_heads", heads), r.int("vdim", dim)
        scale = r.float("scale")
        temp = r.object("q_temp", None)
        r.require(not heads or not kv_heads or (heads > 0 and kv_heads > 0 and heads % kv_heads == 0),
                  f"{heads} heads are not a multiple of {kv_heads} kv_heads")
        _positive(r, dim=dim, vdim=vdim)
        r.finish()
        q_temp = None
        if temp is not None:
            rt = KeyReader(temp, where + ".q_temp")
            coef, every = rt.float("coef"), rt.int("every")
            _positive(rt, every=every)
            rt.finish()
            q_temp = QueryTemperature(coef, every)
        return SigmoidAttentionConfig(heads, kv_heads, dim, vdim, scale, q_temp)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.q_temp is not None:
            out["q_temp"] = self.q_temp.to_dict()
        return out


@dataclass(frozen=True)
class RecurrentUnitConfig:
    width: int
    blocks: int
    conv: int

    @staticmethod
    def read(data: dict, where: str) -> "RecurrentUnitConfig":
        r = KeyReader(data, where)
        width, blocks, conv = r.int("width"), r.int("blocks", 1), r.int("conv")
        _positive(r, width=width, blocks=blocks, conv=conv)
        r.require(not width or not blocks or blocks < 1 or width % blocks == 0, f"{width} channels are not {blocks} equal blocks")
        r.finish()
        return RecurrentUnitConfig(width, blocks, conv)

    def to_dict(self) -> dict:
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


@dataclass(frozen=True)
class SideBySideConfig:
    left: SigmoidAttentionConfig
    right: RecurrentUnitConfig
    left_scale: float
    right_scale: float
    type: str = "parallel"

    @staticmethod
    def read(data: dict, where: str) -> "SideBySideConfig":
        r = KeyReader(data, where)
        left, right = r.object("left"), r.object("right")
        ls, rs = r.float("left_scale", 1.0), r.float("right_scale", 1.0)
        r.finish()
        return SideBySideConfig(SigmoidAttentionConfig.read(left, where + ".left"),
                                RecurrentUnitConfig.read(right, where + ".right"), ls, rs)

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int
    type: str = "mamba2"

    @staticmethod
    def read(data: dict, where: str) -> "StateSpaceConfig":
        r = KeyReader(data, where)
        heads, vdim, state = r.int("heads"), r.int("vdim"), r.int("state")
        groups, conv, norm_groups = r.int("groups", 1), r.int("conv"), r.int("norm_groups", 1)
        _positive(r, heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups)
        r.require(not heads or not groups or groups < 1 or heads % groups == 0, f"{heads} heads are not a multiple of {groups} groups")
        r.require(not heads or not vdim or not norm_groups or norm_groups < 1 or (heads * vdim) % norm_groups == 0,
                  f"the heads' values are not {norm_groups} equal parts")
        r.finish()
        return StateSpaceConfig(heads, vdim, state, groups, conv, norm_groups)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


MIXERS = {"parallel": SideBySideConfig, "mamba2": StateSpaceConfig}


@dataclass(frozen=True)
class LayerConfig:
    mixer: object                   # one of MIXERS' classes
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class RonavikConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    layers: tuple                   # of LayerConfig
    max_positions: int
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None

    @staticmethod
    def from_dict(data: dict, where: str = "config.json") -> "RonavikConfig":
        r = KeyReader(data, where)
        arch = r.str("architecture", "Ronavik")
        vocab, width = r.int("vocab"), r.int("width")
        norm = r.object("norm")
        layers = data.get("layers")
        r.require(isinstance(layers, list) and len(layers) > 0, "key 'layers' must be a non-empty list")
        max_positions = r.int("max_positions")          # (the rows of the learned position vectors)
        _positive(r, vocab=vocab, width=width, max_positions=max_positions)
        eos = r.int_or_list("eos_token_id", None)
        bos = r.int("bos_token_id", None)
        r.finish()
        rn = KeyReader(norm, where + ".norm")
        eps = rn.float("eps")
        rn.require(eps is None or eps >= 0, "eps must not be negative")
        rn.finish()
        out = []
        for i, layer in enumerate(layers):
            at = f"{where}.layers[{i}]"
            rl = KeyReader(layer, at)
            kind = rl.str("type")
            mixer = rl.object("mixer")
            mlp = rl.object("mlp", None)
            rl.require(kind is None or kind in MIXERS, f"unknown mixer type {kind!r} (known: {', '.join(sorted(MIXERS))})")
            rl.finish()
            m = MIXERS[kind].read(mixer, at + ".mixer")
            f = None
            if mlp is not None:
                f = _read_mlp(mlp, at + ".mlp")
                if not isinstance(f, MoeConfig):
                    raise ConfigError(f"{at}.mlp: this design's feed-forward is of kind 'moe'")
            out.append(LayerConfig(m, f))
        return RonavikConfig(arch, vocab, width, eps, tuple(out), max_positions, tuple(eos), bos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions,
               "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                          for l in self.layers]}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out
