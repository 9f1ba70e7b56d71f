"""Two mixers side by side.

"side_by_side": both read the same input; the result is left_scale * left + right_scale * right.  Each of
the two is a mixer of the registry with its own spec and its own tensors (under the prefixes `left` and
`right` of the pair's names); one of them may keep a growing cache (the pair's cache layer is that
mixer's; at most one of the two may ask for one) and either may keep per-request state.  Both write
float32 rows; a block that norms a sub-layer's result takes the second rows and the two scales into that
launch (`forward_into` returns them), any other block gets the weighted sum added to the stream.
"""
from __future__ import annotations

import torch

from ..config.specs import MixerSpec
from ..kernels import ops
from .base import Mixer, lookup, register_mixer


@register_mixer("side_by_side")
class SideBySide(Mixer):
    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        given = dict(spec.get("names") or ())
        left, right = spec.get("left"), spec.get("right")
        if not isinstance(left, MixerSpec) or not isinstance(right, MixerSpec):
            raise ValueError("side_by_side takes the specs of its two mixers as `left` and `right`")
        self.left = lookup("mixer", left.kind)(left, prefix + given.get("left", "left."), dtype)
        self.right = lookup("mixer", right.kind)(right, prefix + given.get("right", "right."), dtype)
        self.scales = (float(spec.get("left_scale", 1.0)), float(spec.get("right_scale", 1.0)))
        for m in (self.left, self.right):
            if not hasattr(m, "forward_into"):
                raise ValueError(f"a mixer of a pair writes rows (forward_into); {type(m).__name__} does not")
        if self.left.cache_spec() is not None and self.right.cache_spec() is not None:
            raise ValueError("at most one mixer of a pair keeps a growing cache")
        self.cached = self.right if self.right.cache_spec() is not None else self.left
        self.second_half_rows = 0

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    def parts(self):
        return [*self.left.parts(), *self.right.parts()]

    def tensor_specs(self):
        return self.left.tensor_specs() + self.right.tensor_specs()

    def bind(self, tensors):
        self.left.bind(tensors)
        self.right.bind(tensors)

    def cache_spec(self):
        return self.cached.cache_spec()

    def key_layout(self):
        return getattr(self.cached, "key_layout", lambda: None)()

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        """out = the left mixer's rows; returns the right mixer's rows and the two scales."""
        self.left.forward_into(ctx, out, h, cache_layer, writes_cache)
        y2 = ctx.rows("side_by_side.second", self.hidden, torch.float32)
        self.right.forward_into(ctx, y2, h, cache_layer, writes_cache)
        return dict(y2=y2, scales=self.scales)

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        y = ctx.rows("mixer.rows_out", self.hidden, torch.float32)
        second = self.forward_into(ctx, y, h, cache_layer, writes_cache)
        ops.scaled_add(x, y, self.scales[0], second["y2"], self.scales[1])
