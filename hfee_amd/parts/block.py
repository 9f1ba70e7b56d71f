"""How a layer's parts are arranged around the residual stream.

"prenorm" is the reference's block (/root/reference/internal/llm/forward.go:79-115):
x += mixer(norm(x)); x += feed_forward(norm(x)).

"sandwich" norms a sub-layer's output as well before it adds it:
x += norm_b(mixer(norm_a(x))); x += norm_d(feed_forward(norm_c(x))), with four norms of their own
weights, and a layer may have no feed-forward.  The sub-layers write float32 rows
(`forward_into`); one launch norms them, adds them to the stream and makes the norm of the new
stream for whatever follows (`ops.norm_add`), across layers too.  With the parameter `residual_gate`
every sub-layer's result passes a gate before its norm: y * sigmoid(W_g h + b_g), h the sub-layer's own
input, W_g [width, width] and b_g a sub-layer; the gate's product runs beside the sub-layer, its sigmoid,
the multiplication, the norm and the addition are one launch (`ops.gated_norm_add`), which also takes a
second result with the two scales of a mixer that is two mixers side by side (what its `forward_into`
returns).

"parallel" has one norm whose output both sub-layers read: with h = norm(x),
x += mixer(h) + feed_forward(h).  Both add their last product straight into the float32 stream, the
mixer first; a layer may have no feed-forward.  With the parameter `residual_scale` = m the layer adds
m * (mixer(h) + feed_forward(h)): the sub-layers then add into float32 rows of their own, which join the
stream in one launch that also makes the next layer's norm (or the head's) where that is an RMS norm.
"""
from __future__ import annotations

import torch

from ..config.specs import LayerSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import LazyNorm, Part, lookup, register_block
from .kv_attention import product, tiles_of


@register_block("prenorm")
class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, dtype: torch.dtype):
        self.spec, self.dtype = spec, dtype
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(
            spec.mixer_norm, spec.name_of("mixer_norm", "mixer_norm.") + "weight")
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, spec.name_of("mixer", "mixer."), dtype)
        self.feed_forward_norm = lookup("norm", spec.feed_forward_norm.kind)(
            spec.feed_forward_norm, spec.name_of("feed_forward_norm", "feed_forward_norm.") + "weight")
        self.feed_forward = lookup("feed_forward", spec.feed_forward.kind)(
            spec.feed_forward, spec.name_of("feed_forward", "feed_forward."), dtype)
        self.hidden = spec.hidden

    def parts(self):
        # (each with the parts it is made of itself: a mixer lists a step behind its projections)
        return [q for p in self._own() for q in p.parts()]

    def _own(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    # the layer of the paged cache that a run of this block is given belongs to its mixer
    def cache_spec(self):
        return self.mixer.cache_spec()

    def key_layout(self):
        return getattr(self.mixer, "key_layout", lambda: None)()

    def tensor_specs(self):
        return [s for p in self._own() for s in p.tensor_specs()]

    def bind(self, tensors):
        for p in self._own():
            p.bind(tensors)

    # forward takes the normed input that the block before may have begun, and that of
    # the block after, which this block's last part may begin (the engine makes both with
    # `begin` for blocks that say so)
    chains_norms = True

    def begin(self, ctx, x):
        """The block's normed input, not yet computed."""
        return LazyNorm(ctx, self.mixer_norm, x, self.mixer.second_half_rows)

    def forward(self, ctx, x, entry, h_in=None, h_next=None):
        h = h_in if h_in is not None else self.begin(ctx, x)
        h2 = LazyNorm(ctx, self.feed_forward_norm, x, self.feed_forward.second_half_rows)
        self._run(self.mixer, ctx, x, h, h2, entry.cache, entry.writes_cache)
        self._run(self.feed_forward, ctx, x, h2, h_next)

    @staticmethod
    def _run(part, ctx, x, h, then, *args):
        h = h if part.takes_lazy_norm else h.tensor()
        if then is not None and part.emits_norm:
            part.forward_add(ctx, x, h, *args, then=then)
        else:
            part.forward_add(ctx, x, h, *args)


@register_block("sandwich")
class SandwichBlock(Part):
    """Tensor names by role: mixer_norm, mixer_post_norm, feed_forward_norm, feed_forward_post_norm
    (the whole name behind the layer's prefix), mixer and feed_forward (prefixes); with `residual_gate`
    also mixer_gate, mixer_gate_bias, feed_forward_gate, feed_forward_gate_bias."""

    def __init__(self, spec: LayerSpec, dtype: torch.dtype):
        self.spec, self.dtype, self.hidden = spec, dtype, spec.hidden
        self.gated = bool(spec.get("residual_gate", False))
        self.gates = {}                  # role -> (weight, tiles, float32 bias), once bound

        def norm(norm_spec, role):
            return lookup("norm", norm_spec.kind)(norm_spec, spec.name_of(role, role + ".weight"))
        self.mixer_norm = norm(spec.mixer_norm, "mixer_norm")
        self.mixer_post_norm = norm(spec.mixer_norm, "mixer_post_norm")
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, spec.name_of("mixer", "mixer."), dtype)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_post_norm = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = norm(spec.feed_forward_norm, "feed_forward_norm")
            self.feed_forward_post_norm = norm(spec.feed_forward_norm, "feed_forward_post_norm")
            self.feed_forward = lookup("feed_forward", spec.feed_forward.kind)(
                spec.feed_forward, spec.name_of("feed_forward", "feed_forward."), dtype)
        for n in (self.mixer_post_norm, self.feed_forward_post_norm):
            if n is not None and getattr(n, "fused_form", None) is None:
                raise ValueError("a sandwich block norms its sub-layers' outputs with y / sqrt(mean(y^2) + eps) * w")

    def _own(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post_norm, self.feed_forward_norm, self.feed_forward,
                            self.feed_forward_post_norm) if p is not None]

    def parts(self):
        return [q for p in self._own() for q in p.parts()]

    def cache_spec(self):
        return self.mixer.cache_spec()

    def key_layout(self):
        return getattr(self.mixer, "key_layout", lambda: None)()

    def _gate_roles(self):
        if not self.gated:
            return []
        return ["mixer"] + (["feed_forward"] if self.feed_forward is not None else [])

    def tensor_specs(self):
        specs = [s for p in self._own() for s in p.tensor_specs()]
        for role in self._gate_roles():
            specs += [TensorSpec(self.spec.name_of(role + "_gate", role + "_gate.weight"), (self.hidden, self.hidden)),
                      TensorSpec(self.spec.name_of(role + "_gate_bias", role + "_gate.bias"), (self.hidden,), role="vector")]
        return specs

    def bind(self, tensors):
        for p in self._own():
            p.bind(tensors)
        for role in self._gate_roles():
            w = tensors.pop(self.spec.name_of(role + "_gate", role + "_gate.weight")).contiguous()
            b = tensors.pop(self.spec.name_of(role + "_gate_bias", role + "_gate.bias")).to(torch.float32).contiguous()
            self.gates[role] = (w, tiles_of(self.dtype, w)[0], b)

    chains_norms = True

    def begin(self, ctx, x):
        return LazyNorm(ctx, self.mixer_norm, x)

    def _gate_of(self, ctx, role, h):
        """The gate's logits of a sub-layer (engine dtype, before bias and sigmoid), and its bias."""
        if role not in self.gates:
            return None, None
        w, tiles, bias = self.gates[role]
        logits = ctx.rows("block.gate", self.hidden)
        product(ctx, logits, h.tensor(), w, tiles)
        return logits, bias

    @staticmethod
    def _rows_of(part, ctx, h, width, *args):
        """The sub-layer's output as float32 rows (not yet added anywhere), and what `forward_into`
        returned: None, or dict(y2, scales) of a part whose result is scales[0] * rows + scales[1] * y2."""
        y = ctx.rows("block.sublayer_rows", width, torch.float32)
        second = None
        if hasattr(part, "forward_into"):
            second = part.forward_into(ctx, y, h if part.takes_lazy_norm else h.tensor(), *args)
        else:           # a part that only knows how to add: into rows of zeros
            y.zero_()
            part.forward_add(ctx, y, h if part.takes_lazy_norm else h.tensor(), *args)
        return y, second

    @staticmethod
    def _add_normed(ctx, x, y, post_norm, bias, following, second=None, gate=None, gate_bias=None):
        """x += post_norm(y + bias), and the norm that follows in the same launch where it is of the
        same form and nobody has made it yet.  second / gate: see `ops.gated_norm_add`."""
        if second is not None or gate is not None:
            if bias is not None:
                raise ValueError("a gated sub-layer has no bias behind its last product")
            weight, eps = post_norm.fused_form_f32()
            more = dict(y2=second["y2"], scales=second["scales"]) if second is not None else {}
            nxt = following.fusable() if following is not None else None
            if nxt is not None and following._tensor is None and following.pending is None:
                out = ctx.rows("block.normed", x.shape[1])
                w2, eps2 = following.norm.fused_form_f32()
                ops.gated_norm_add(x, y, weight, eps, gate=gate, gate_bias=gate_bias, next_out=out, next_weight=w2,
                                   next_eps=eps2, **more)
                following._tensor = out
            else:
                ops.gated_norm_add(x, y, weight, eps, gate=gate, gate_bias=gate_bias, **more)
            return
        weight, eps = post_norm.fused_form()
        nxt = following.fusable() if following is not None else None
        if nxt is not None and following._tensor is None and following.pending is None and nxt[0].dtype == weight.dtype:
            out = ctx.rows("block.normed", x.shape[1])
            ops.norm_add(x, y, weight, eps, bias=bias, next_out=out, next_weight=nxt[0], next_eps=nxt[1])
            following._tensor = out
        else:
            ops.norm_add(x, y, weight, eps, bias=bias)

    def forward(self, ctx, x, entry, h_in=None, h_next=None):
        h = h_in if h_in is not None else self.begin(ctx, x)
        gate, gate_bias = self._gate_of(ctx, "mixer", h)
        y, second = self._rows_of(self.mixer, ctx, h, self.hidden, entry.cache, entry.writes_cache)
        if self.feed_forward is None:
            self._add_normed(ctx, x, y, self.mixer_post_norm, getattr(self.mixer, "output_bias", None), h_next, second, gate, gate_bias)
            return
        h2 = LazyNorm(ctx, self.feed_forward_norm, x)
        self._add_normed(ctx, x, y, self.mixer_post_norm, getattr(self.mixer, "output_bias", None), h2, second, gate, gate_bias)
        gate, gate_bias = self._gate_of(ctx, "feed_forward", h2)
        y, second = self._rows_of(self.feed_forward, ctx, h2, self.hidden)
        self._add_normed(ctx, x, y, self.feed_forward_post_norm, getattr(self.feed_forward, "output_bias", None), h_next,
                         second, gate, gate_bias)


@register_block("parallel")
class ParallelBlock(Part):
    """Tensor names by role: mixer_norm (the whole name behind the layer's prefix), mixer and
    feed_forward (prefixes)."""

    def __init__(self, spec: LayerSpec, dtype: torch.dtype):
        self.spec, self.dtype, self.hidden = spec, dtype, spec.hidden
        self.residual_scale = float(spec.get("residual_scale", 1.0))
        self.norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, spec.name_of("mixer_norm", "norm.weight"))
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, spec.name_of("mixer", "mixer."), dtype)
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward = lookup("feed_forward", spec.feed_forward.kind)(
                spec.feed_forward, spec.name_of("feed_forward", "feed_forward."), dtype)

    def _own(self):
        return [p for p in (self.norm, self.mixer, self.feed_forward) if p is not None]

    def parts(self):
        return [q for p in self._own() for q in p.parts()]

    def cache_spec(self):
        return self.mixer.cache_spec()

    def key_layout(self):
        return getattr(self.mixer, "key_layout", lambda: None)()

    def tensor_specs(self):
        return [s for p in self._own() for s in p.tensor_specs()]

    def bind(self, tensors):
        for p in self._own():
            p.bind(tensors)

    chains_norms = True

    def begin(self, ctx, x):
        return LazyNorm(ctx, self.norm, x)

    def forward(self, ctx, x, entry, h_in=None, h_next=None):
        h = (h_in if h_in is not None else self.begin(ctx, x)).tensor()
        into = x
        if self.residual_scale != 1.0:
            into = ctx.rows("block.sublayer_rows", self.hidden, torch.float32)
        if into is not x and hasattr(self.mixer, "forward_into"):       # (the mixer's last product fills the rows)
            self.mixer.forward_into(ctx, into, h, entry.cache, entry.writes_cache)
        else:
            if into is not x:
                into.zero_()
            self.mixer.forward_add(ctx, into, h, entry.cache, entry.writes_cache)
        if self.feed_forward is not None:
            self.feed_forward.forward_add(ctx, into, h)
        if into is not x:
            form = h_next.norm.fused_form_f32() if h_next is not None and hasattr(h_next.norm, "fused_form_f32") else None
            if form is not None and h_next._tensor is None and h_next.pending is None:
                out = ctx.rows("block.normed", self.hidden)
                ops.scaled_add_norm(x, into, self.residual_scale, out, form[0], form[1])
                h_next._tensor = out
            else:
                ops.scaled_add(x, into, self.residual_scale)
