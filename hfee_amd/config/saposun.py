"""SaposunConfig: the Saposun decoder's configuration, read from config.json.

The file lists the layers one by one: each entry names its mixer (`type`: "latent_attention",
"retention" or "attention") with that mixer's sizes and constants (`mixer`), and its feed-forward
(`mlp`: {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}, or null for a layer without
one).  Beside the list it gives the vocabulary, the width, the norms' eps and the number that every
layer's result is multiplied by before it joins the stream (`residual_mult`).  What an entry does not
name does not exist: a mixer without `rot` is not rotated, one without `mask` sees every earlier
position, a mask without `pool` has no pooled blocks, an attention without `conv` or `softcap` has
neither.  A latent-attention layer with `kv_from` reads the keys that the layer of that number keeps.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .base import ConfigError, KeyReader
from .sabezen import MoeConfig, _read_mlp
from .vofezen import RotaryConfig


def _positive(r: KeyReader, **values):
    for name, v in values.items():
        r.require(v is None or v > 0, f"{name} must be positive")


def _rotation(rot, where: str, most: int, dims_default=None) -> Optional[RotaryConfig]:
    if rot is None:
        return None
    rc = RotaryConfig.read(rot, where + ".rot", dims_default=dims_default)
    if rc.scaling is not None:
        raise ConfigError(f"{where}.rot: this design's rotation is not stretched")
    if rc.dims > most:
        raise ConfigError(f"{where}: {rc.dims} rotated dims do not fit {most}")
    return rc


def _mask(mask, where: str):
    """(window, pool): 0 where the entry names none."""
    if mask is None:
        return 0, 0
    rm = KeyReader(mask, where + ".mask")
    size, pool = rm.int("size"), rm.int("pool", 0)
    _positive(rm, size=size)
    rm.require(pool is None or pool >= 0, "pool must not be negative")
    rm.finish()
    return size, pool


def _mask_dict(window: int, pool: int = 0):
    out = {"size": window}
    if pool:
        out["pool"] = pool
    return out


@dataclass(frozen=True)
class WindowLatentConfig:
    heads: int
    dim: int                        # unrotated query/key dims a head
    rot_dim: int                    # rotated dims a head (the key's are shared by all heads)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int                     # 0: every earlier position
    rot: Optional[RotaryConfig]
    kv_from: Optional[int]          # the layer whose latent and rotated key part this one reads
    type: str = "latent_attention"

    @staticmethod
    def read(data: dict, where: str) -> "WindowLatentConfig":
        r = KeyReader(data, where)
        heads, dim, rot_dim = r.int("heads"), r.int("dim"), r.int("rot_dim")
        vdim, q_rank, kv_rank = r.int("vdim", dim), r.int("q_rank"), r.int("kv_rank")
        scale = r.float("scale")
        rot, mask = r.object("rot", None), r.object("mask", None)
        kv_from = r.int("kv_from", None)
        _positive(r, heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank)
        r.require(kv_from is None or kv_from >= 0, "kv_from names a layer")
        r.finish()
        window, pool = _mask(mask, where)
        if pool:
            raise ConfigError(f"{where}.mask: a latent-attention layer has no pooled blocks")
        rc = _rotation(rot, where, rot_dim, dims_default=rot_dim)
        if rc is not None and rc.dims != rot_dim:
            raise ConfigError(f"{where}: the rotation covers {rc.dims} dims, the rotated part has {rot_dim}")
        return WindowLatentConfig(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window, rc, kv_from)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
               "kv_rank": self.kv_rank, "scale": self.scale}
        if self.window:
            out["mask"] = _mask_dict(self.window)
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple                    # one number a head
    rot: Optional[RotaryConfig]
    type: str = "retention"

    @staticmethod
    def read(data: dict, where: str) -> "RetentionConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        vdim = r.int("vdim", dim)
        rot = r.object("rot", None)
        decay = data.get("decay")
        _positive(r, heads=heads, dim=dim, vdim=vdim)
        numbers = isinstance(decay, list) and all(isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay)
        r.require(numbers, "key 'decay' must be a list of numbers, one a head")
        r.require(not numbers or heads is None or len(decay) == heads, f"'decay' must hold one number for each of the {heads} heads")
        r.require(not numbers or all(0.0 <= float(d) <= 1.0 for d in decay), "a decay lies between 0 and 1")
        r.finish()
        return RetentionConfig(heads, dim, vdim, tuple(float(d) for d in decay), _rotation(rot, where, dim))

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class PooledAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float                  # 0: none
    conv: int                       # taps of the short convolution on q, k and v; 0: none
    window: int                     # 0: every earlier position
    pool: int                       # tokens a pooled block; 0: none
    rot: Optional[RotaryConfig]
    type: str = "attention"

    @staticmethod
    def read(data: dict, where: str) -> "PooledAttentionConfig":
        r = KeyReader(data, where)
        heads, dim = r.int("heads"), r.int("dim")
        kv_heads, vdim = r.int("kv_heads", heads), r.int("vdim", dim)
        scale, softcap, conv = r.float("scale"), r.float("softcap", 0.0), r.int("conv", 0)
        rot, mask = r.object("rot", None), r.object("mask", None)
        r.require(not heads or not kv_heads or (heads > 0 and kv_heads > 0 and heads % kv_heads == 0),
                  f"{heads} heads are not a multiple of {kv_heads} kv_heads")
        _positive(r, dim=dim, vdim=vdim)
        r.require(softcap is None or softcap >= 0, "softcap must not be negative")
        r.require(conv is None or conv >= 0, "conv must not be negative")
        r.finish()
        window, pool = _mask(mask, where)
        return PooledAttentionConfig(heads, kv_heads, dim, vdim, scale, softcap, conv, window, pool,
                                     _rotation(rot, where, dim))

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.conv:
            out["conv"] = self.conv
        if self.window:
            out["mask"] = _mask_dict(self.window, self.pool)
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


MIXERS = {"latent_attention": WindowLatentConfig, "retention": RetentionConfig, "attention": PooledAttentionConfig}


@dataclass(frozen=True)
class LayerConfig:
    mixer: object                   # one of MIXERS' classes
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class SaposunConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: tuple                   # of LayerConfig
    max_positions: int
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None

    # the design names no longest context; the engine's tables are made for what a caller asks for, up to this
    DEFAULT_MAX_POSITIONS = 1 << 20

    @staticmethod
    def from_dict(data: dict, where: str = "config.json") -> "SaposunConfig":
        r = KeyReader(data, where)
        arch = r.str("architecture", "Saposun")
        vocab, width = r.int("vocab"), r.int("width")
        norm = r.object("norm")
        mult = r.float("residual_mult", 1.0)
        layers = data.get("layers")
        r.require(isinstance(layers, list) and len(layers) > 0, "key 'layers' must be a non-empty list")
        _positive(r, vocab=vocab, width=width)
        max_positions = r.int("max_positions", SaposunConfig.DEFAULT_MAX_POSITIONS)
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
            feed_forward = None
            if mlp is not None:
                feed_forward = _read_mlp(mlp, at + ".mlp")
                if not isinstance(feed_forward, MoeConfig):
                    raise ConfigError(f"{at}.mlp: this design's feed-forward is of kind 'moe'")
            out.append(LayerConfig(m, feed_forward))
        for i, layer in enumerate(out):
            j = getattr(layer.mixer, "kv_from", None)
            if j is None:
                continue
            at = f"{where}.layers[{i}].mixer"
            if not 0 <= j < i or not isinstance(out[j].mixer, WindowLatentConfig) or out[j].mixer.kv_from is not None:
                raise ConfigError(f"{at}: kv_from {j} must name an earlier latent-attention layer with keys of its own")
            a, b = layer.mixer, out[j].mixer
            if (a.kv_rank, a.rot_dim, a.rot) != (b.kv_rank, b.rot_dim, b.rot):
                raise ConfigError(f"{at}: the latent, the rotated part and the rotation must equal those of layer {j}")
        return SaposunConfig(arch, vocab, width, eps, mult, tuple(out), max_positions, tuple(eos), bos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
               "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                          for l in self.layers]}
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out
