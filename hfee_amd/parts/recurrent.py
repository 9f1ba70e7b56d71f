"""Mixers that keep a state of fixed size for every request instead of a growing cache.

"gated_delta", "gla" and "state_space" hold, for each head, S [dim, vdim] in float32 in the request's
state slot (zero when the request is admitted), walk a step's tokens of a request in order from it, and
leave the new state there; a decay acts on the rows of S, one number a key channel (a head in
"state_space").  "rglru" holds one number a channel.  What enters a recurrence besides the projections
and short convolutions themselves is made in float32: decays, step sizes, writing strengths, gates, unit norms.

"gated_delta": q, k (`num_qk_heads` heads of `dim`; head h reads q/k head h // (heads / qk heads)) and v
(`num_heads` heads of `vdim`) each pass a short causal convolution per channel (`conv` taps, no bias,
zeros before the sequence's start; the last conv - 1 inputs are state too) and a SiLU; q and k
become unit vectors per head, x / sqrt(sum(x^2) + unit_eps), q also times dim^(-1/2);
b = sigmoid(W_b h) a head; a = exp(-exp(A_h) softplus(W_a2 W_a1 h + dt_bias)) a head and key channel.
Per token S <- diag(a) S; u = b (v - S^T k); S <- S + k u^T; o = S^T q.  Each head's o is divided by
its root mean square (eps `norm_eps`), times a weight shared by the heads, times
sigmoid(W_g2 W_g1 h); then the output product.

"gla": q = W_q h dim^(-1/2), k, v; a = sigmoid(W_a2 W_a1 h + bias)^(1/tau);
S <- diag(a) S + k v^T; o = S^T q; each head's o normed as above with a weight shared by the heads,
the heads side by side times silu(W_g h); then the output product.

"retention": linear attention with a fixed decay a head and neither softmax nor denominator.  q, k
(`num_heads` heads of `dim`) and v (heads of `vdim`) are plain products; q and k are rotated by the token's
position (the position part's pairs (i, i + half)), k is then multiplied by dim^(-1/2);
S <- decay_h S + k v^T, o = S^T q, with one decay a head from the spec; each head's o is divided by its root
mean square (eps `norm_eps`, no weight), the heads side by side times silu(W_g h); then the output product.

"state_space" (state-space duality): one product gives [z | x | B | C | dt] (z, x: `num_heads` heads of
`vdim`; B, C: `groups` groups of `state`; dt a head).  x, B and C together pass a short causal convolution
per channel with a bias and a SiLU.  dt = softplus(dt + dt_bias); per head (head h reads group
h // (heads / groups)), with a = exp(-exp(A_h) dt): S <- a S + dt B x^T (S [state, vdim]),
y = S^T C + D_h x.  The heads side by side are multiplied by silu(z) and then divided by their root mean
square in `norm_groups` equal parts (eps `norm_eps`), times a weight an element; then the output product.

"rglru" (a real-gated linear recurrent unit between two branches of `width` channels): y =
gelu_tanh(W_y h + b_y); u = conv(W_x h + b_x), a short causal convolution per channel with a bias and no
activation.  u is cut into `blocks` equal parts; in part b, r = sigmoid(R_b u_b + c_b) and
i = sigmoid(I_b u_b + d_b) with square matrices R_b, I_b, in float32.  With a = exp(-decay_scale * r *
softplus(lam)), lam a number a channel: S <- a S + sqrt(1 - a^2) * i * u; the output product reads S * y.
"""
from __future__ import annotations

import torch

import torch.nn.functional as F

from ..config.specs import MixerSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import LazyNorm, Mixer, lookup, register_mixer
from .kv_attention import product, tiles_of


class _StateMixer(Mixer):
    graph_safe = True

    def _names(self, spec, defaults):
        given = dict(spec.get("names") or ())
        return {role: self.prefix + given.get(role, default) for role, default in defaults.items()}

    def cache_spec(self):
        return None

    def _segments(self, ctx):
        return ctx.segment_rows, ctx.segment_lengths, ctx.segment_slots


@register_mixer("gated_delta")
class GatedDelta(_StateMixer):
    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.heads = spec.get("num_heads")
        self.qk_heads = spec.get("num_qk_heads", self.heads)
        self.dim, self.vdim = spec.get("dim"), spec.get("vdim")
        self.taps = spec.get("conv")
        self.decay_rank, self.gate_rank = spec.get("decay_rank"), spec.get("gate_rank")
        self.unit_eps = float(spec.get("unit_eps", 1e-6))
        self.norm_eps = float(spec.get("norm_eps", 1e-6))
        if self.heads % self.qk_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.qk_heads} query/key heads")
        if self.taps < 1:
            raise ValueError("the short convolution has at least one tap")
        self.names = self._names(spec, dict(
            q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", q_conv="q_conv.weight", k_conv="k_conv.weight",
            v_conv="v_conv.weight", b="b_proj.weight", a_log="A_log", norm="norm.weight", a_down="a_down.weight",
            a_up="a_up.weight", dt_bias="dt_bias", g_down="g_down.weight", g_up="g_up.weight", o="o_proj.weight"))
        self.qk_width, self.v_width = self.qk_heads * self.dim, self.heads * self.vdim
        self.channels = 2 * self.qk_width + self.v_width

    def tensor_specs(self):
        n, H, D = self.names, self.heads, self.dim
        specs = [TensorSpec(n["q"], (self.qk_width, self.hidden)), TensorSpec(n["q_conv"], (self.qk_width, self.taps), role="vector"),
                 TensorSpec(n["k"], (self.qk_width, self.hidden)), TensorSpec(n["k_conv"], (self.qk_width, self.taps), role="vector"),
                 TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["v_conv"], (self.v_width, self.taps), role="vector"),
                 TensorSpec(n["b"], (H, self.hidden)), TensorSpec(n["a_log"], (H,), role="vector"),
                 TensorSpec(n["norm"], (self.vdim,), role="vector", init=("one_plus_normal",)),
                 TensorSpec(n["a_down"], (self.decay_rank, self.hidden)), TensorSpec(n["a_up"], (H * D, self.decay_rank)),
                 TensorSpec(n["dt_bias"], (H * D,), role="vector"),
                 TensorSpec(n["g_down"], (self.gate_rank, self.hidden)), TensorSpec(n["g_up"], (self.v_width, self.gate_rank)),
                 TensorSpec(n["o"], (self.hidden, self.v_width))]
        return specs

    def bind(self, tensors):
        n = self.names
        f32 = lambda name: tensors.pop(name).to(torch.float32).contiguous()      # noqa: E731
        # one product for everything that reads the layer's input: [q | k | v | a_down | g_down | b]
        self.w_in = torch.cat([tensors.pop(n[r]) for r in ("q", "k", "v", "a_down", "g_down", "b")], dim=0).contiguous()
        self.at_a = self.channels
        self.at_g = self.at_a + self.decay_rank
        self.at_b = self.at_g + self.gate_rank
        self.conv_taps = torch.cat([f32(n["q_conv"]), f32(n["k_conv"]), f32(n["v_conv"])], dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm_weight = f32(n["a_log"]), f32(n["dt_bias"]), f32(n["norm"])
        self.w_a_up, self.w_g_up = tensors.pop(n["a_up"]).contiguous(), tensors.pop(n["g_up"]).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.w_in_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_in, self.w_o)
        self.w_a_up_tiles, self.w_g_up_tiles = tiles_of(self.dtype, self.w_a_up, self.w_g_up)

    def state_specs(self):
        return [(self.prefix + "state", (self.heads, *ops.scan_state_shape(self.dim, self.vdim)), torch.float32),
                (self.prefix + "conv_state", (self.taps - 1, self.channels), self.dtype)]

    def prepare(self, info):
        self.state = info.storage.states[self.prefix + "state"]
        self.conv_state = info.storage.states[self.prefix + "conv_state"]

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, D, V = self.heads, self.qk_heads, self.dim, self.vdim
        rows, lengths, slots = self._segments(ctx)
        total = self.w_in.shape[0]       # (rows of a multiple of 8 elements, so that blocks of columns stay aligned)
        proj = ctx.rows("gated_delta.in", (total + 7) // 8 * 8)[:, :total]
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        raw = proj[:, :self.channels]
        y = ctx.rows("gated_delta.conv", self.channels, torch.float32)
        ops.short_conv_silu(y, raw, self.conv_state, self.conv_taps, ctx.token_segment, rows, slots)
        ops.short_conv_keep(self.conv_state, raw, rows, lengths, slots)
        q, k, v = y[:, :self.qk_width], y[:, self.qk_width:2 * self.qk_width], y[:, 2 * self.qk_width:]
        ops.unit_heads(q, G, D, self.unit_eps, D ** -0.5)
        ops.unit_heads(k, G, D, self.unit_eps, 1.0)
        step = ctx.rows("gated_delta.step", H * D)
        product(ctx, step, proj[:, self.at_a:self.at_g], self.w_a_up, self.w_a_up_tiles)
        decay = ctx.rows("gated_delta.decay", H * D, torch.float32)
        ops.scan_gate(decay, step, "step_decay", bias=self.dt_bias, per_head=self.a_log, head_width=D)
        beta = ctx.rows("gated_delta.beta", H, torch.float32)
        ops.scan_gate(beta, proj[:, self.at_b:self.at_b + H], "sigmoid")
        o = ctx.rows("gated_delta.read", self.v_width, torch.float32)
        ops.linear_scan(o, self.state, q, k, v, decay, beta, rows, lengths, slots, H, G, D, V, "delta")
        gate = ctx.rows("gated_delta.gate", self.v_width)
        product(ctx, gate, proj[:, self.at_g:self.at_b], self.w_g_up, self.w_g_up_tiles)
        gated = ctx.rows("gated_delta.out", self.v_width)
        ops.head_norm_gate(gated, o, gate, self.norm_weight, H, V, self.norm_eps, "sigmoid")
        product(ctx, x, gated, self.w_o, self.w_o_tiles, add=True)


@register_mixer("gla")
class GatedLinearAttention(_StateMixer):
    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.heads = spec.get("num_heads")
        self.dim, self.vdim = spec.get("dim"), spec.get("vdim")
        self.tau = float(spec.get("tau"))
        self.decay_rank = spec.get("decay_rank")
        self.norm_eps = float(spec.get("norm_eps", 1e-6))
        if self.tau <= 0:
            raise ValueError("tau must be positive")
        self.names = self._names(spec, dict(
            q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", g="g_proj.weight", o="o_proj.weight",
            norm="norm.weight", a_down="a_down.weight", a_up="a_up.weight", a_bias="a_up.bias"))
        self.qk_width, self.v_width = self.heads * self.dim, self.heads * self.vdim

    def tensor_specs(self):
        n = self.names
        return [TensorSpec(n["q"], (self.qk_width, self.hidden)), TensorSpec(n["k"], (self.qk_width, self.hidden)),
                TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["g"], (self.v_width, self.hidden)),
                TensorSpec(n["o"], (self.hidden, self.v_width)),
                TensorSpec(n["norm"], (self.vdim,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["a_down"], (self.decay_rank, self.hidden)), TensorSpec(n["a_up"], (self.qk_width, self.decay_rank)),
                TensorSpec(n["a_bias"], (self.qk_width,), role="vector")]

    def bind(self, tensors):
        n = self.names
        # one product for everything that reads the layer's input: [q | k | v | g | a_down]
        self.w_in = torch.cat([tensors.pop(n[r]) for r in ("q", "k", "v", "g", "a_down")], dim=0).contiguous()
        self.at_g = 2 * self.qk_width + self.v_width
        self.at_a = self.at_g + self.v_width
        self.w_a_up = tensors.pop(n["a_up"]).contiguous()
        self.a_bias = tensors.pop(n["a_bias"]).to(torch.float32).contiguous()
        self.norm_weight = tensors.pop(n["norm"]).to(torch.float32).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.w_in_tiles, self.w_o_tiles, self.w_a_up_tiles = tiles_of(self.dtype, self.w_in, self.w_o, self.w_a_up)

    def state_specs(self):
        return [(self.prefix + "state", (self.heads, *ops.scan_state_shape(self.dim, self.vdim)), torch.float32)]

    def prepare(self, info):
        self.state = info.storage.states[self.prefix + "state"]

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, D, V = self.heads, self.dim, self.vdim
        rows, lengths, slots = self._segments(ctx)
        total = self.w_in.shape[0]
        proj = ctx.rows("gla.in", (total + 7) // 8 * 8)[:, :total]
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        qkv = ctx.rows("gla.qkv", self.at_g, torch.float32)
        ops.scan_gate(qkv, proj[:, :self.at_g], "cast", number=D ** -0.5, first_columns=self.qk_width)
        q, k, v = qkv[:, :self.qk_width], qkv[:, self.qk_width:2 * self.qk_width], qkv[:, 2 * self.qk_width:]
        z = ctx.rows("gla.z", self.qk_width)
        product(ctx, z, proj[:, self.at_a:], self.w_a_up, self.w_a_up_tiles)
        decay = ctx.rows("gla.decay", self.qk_width, torch.float32)
        ops.scan_gate(decay, z, "root_sigmoid", bias=self.a_bias, number=self.tau)
        o = ctx.rows("gla.read", self.v_width, torch.float32)
        ops.linear_scan(o, self.state, q, k, v, decay, None, rows, lengths, slots, H, H, D, V, "decay_add")
        gated = ctx.rows("gla.out", self.v_width)
        ops.head_norm_gate(gated, o, proj[:, self.at_g:self.at_a], self.norm_weight, H, V, self.norm_eps, "silu")
        product(ctx, x, gated, self.w_o, self.w_o_tiles, add=True)


@register_mixer("retention")
class Retention(_StateMixer):
    """Tensor names by role: q, k, v, g, o (matrices)."""

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.heads = spec.get("num_heads")
        self.dim, self.vdim = spec.get("dim"), spec.get("vdim")
        self.decay = tuple(float(d) for d in spec.get("decay"))
        self.norm_eps = float(spec.get("norm_eps", 1e-6))
        if len(self.decay) != self.heads:
            raise ValueError(f"{len(self.decay)} decays for {self.heads} heads")
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        if self.position is not None and self.position.pairing != 0:
            raise ValueError("retention rotates pairs (i, i + half)")
        self.names = self._names(spec, dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", g="g_proj.weight",
                                            o="o_proj.weight"))
        self.qk_width, self.v_width = self.heads * self.dim, self.heads * self.vdim

    def tensor_specs(self):
        n = self.names
        return [TensorSpec(n["q"], (self.qk_width, self.hidden)), TensorSpec(n["k"], (self.qk_width, self.hidden)),
                TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["g"], (self.v_width, self.hidden)),
                TensorSpec(n["o"], (self.hidden, self.v_width))]

    def bind(self, tensors):
        n = self.names
        # one product for everything that reads the layer's input: [q | k | v | g]
        self.w_in = torch.cat([tensors.pop(n[r]) for r in ("q", "k", "v", "g")], dim=0).contiguous()
        self.at_v = 2 * self.qk_width
        self.at_g = self.at_v + self.v_width
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.decays = torch.tensor(self.decay, dtype=torch.float32, device=self.w_o.device)
        self.norm_weight = torch.ones(self.vdim, dtype=torch.float32, device=self.w_o.device)
        self.w_in_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_in, self.w_o)

    def state_specs(self):
        return [(self.prefix + "state", (self.heads, *ops.scan_state_shape(self.dim, self.vdim)), torch.float32)]

    def prepare(self, info):
        self.state = info.storage.states[self.prefix + "state"]
        if self.position is not None:
            self.position.prepare(info.num_positions, info.device)

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        self._run(ctx, x, h, add=True)

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        self._run(ctx, out, h, add=False)

    def _run(self, ctx, x, h, add: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, D, V = self.heads, self.dim, self.vdim
        rows, lengths, slots = self._segments(ctx)
        total = self.w_in.shape[0]
        proj = ctx.rows("retention.in", (total + 7) // 8 * 8)[:, :total]
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        qkv = ctx.rows("retention.qkv", self.at_g, torch.float32)
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        # q and k as 2 H heads of one row: rotated, the keys' heads then times dim^(-1/2)
        ops.rotate_rows(qkv[:, :self.at_v], proj[:, :self.at_v], ctx.positions, cos, sin, 2 * H, D, ctx.max_position,
                        scaled_from=H, factor=D ** -0.5)
        ops.scan_gate(qkv[:, self.at_v:], proj[:, self.at_v:self.at_g], "cast")
        q, k, v = qkv[:, :self.qk_width], qkv[:, self.qk_width:self.at_v], qkv[:, self.at_v:]
        o = ctx.rows("retention.read", self.v_width, torch.float32)
        ops.linear_scan(o, self.state, q, k, v, self.decays, None, rows, lengths, slots, H, H, D, V, "decay_add",
                        decay_per_head=True)
        gated = ctx.rows("retention.out", self.v_width)
        ops.head_norm_gate(gated, o, proj[:, self.at_g:], self.norm_weight, H, V, self.norm_eps, "silu")
        product(ctx, x, gated, self.w_o, self.w_o_tiles, add=add)


@register_mixer("state_space")
class StateSpace(_StateMixer):
    """Tensor names by role: in ([z | x | B | C | dt] rows), conv ([channels, taps]), conv_bias, dt_bias,
    a_log, skip ([heads]), norm ([inner]), o."""

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.heads, self.vdim = spec.get("num_heads"), spec.get("vdim")
        self.state_size, self.groups = spec.get("state"), spec.get("groups", 1)
        self.taps = spec.get("conv")
        self.norm_groups = spec.get("norm_groups", 1)
        self.norm_eps = float(spec.get("norm_eps", 1e-6))
        self.inner = self.heads * self.vdim
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} values are not {self.norm_groups} equal parts")
        if self.taps < 1:
            raise ValueError("the short convolution has at least one tap")
        self.names = self._names(spec, dict(
            **{"in": "in_proj.weight"}, conv="conv.weight", conv_bias="conv.bias", dt_bias="dt_bias", a_log="A_log",
            skip="D", norm="norm.weight", o="out_proj.weight"))
        self.bc_width = self.groups * self.state_size
        self.channels = self.inner + 2 * self.bc_width
        self.in_width = 2 * self.inner + 2 * self.bc_width + self.heads

    def tensor_specs(self):
        n = self.names
        return [TensorSpec(n["in"], (self.in_width, self.hidden)),
                TensorSpec(n["conv"], (self.channels, self.taps), role="vector"),
                TensorSpec(n["conv_bias"], (self.channels,), role="vector"),
                TensorSpec(n["dt_bias"], (self.heads,), role="vector"), TensorSpec(n["a_log"], (self.heads,), role="vector"),
                TensorSpec(n["skip"], (self.heads,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["norm"], (self.inner,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["o"], (self.hidden, self.inner))]

    def bind(self, tensors):
        n = self.names
        f32 = lambda name: tensors.pop(name).to(torch.float32).contiguous()      # noqa: E731
        self.w_in, self.w_o = tensors.pop(n["in"]).contiguous(), tensors.pop(n["o"]).contiguous()
        self.conv_taps, self.conv_bias = f32(n["conv"]), f32(n["conv_bias"])
        self.dt_bias, self.a_log, self.skip, self.norm_weight = f32(n["dt_bias"]), f32(n["a_log"]), f32(n["skip"]), f32(n["norm"])
        self.w_in_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_in, self.w_o)

    def state_specs(self):
        return [(self.prefix + "state", (self.heads, *ops.scan_state_shape(self.state_size, self.vdim)), torch.float32),
                (self.prefix + "conv_state", (self.taps - 1, self.channels), self.dtype)]

    def prepare(self, info):
        self.state = info.storage.states[self.prefix + "state"]
        self.conv_state = info.storage.states[self.prefix + "conv_state"]

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, N, V, inner = self.heads, self.groups, self.state_size, self.vdim, self.inner
        rows, lengths, slots = self._segments(ctx)
        proj = ctx.rows("state_space.in", (self.in_width + 7) // 8 * 8)[:, :self.in_width]
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        z, raw, dt_raw = proj[:, :inner], proj[:, inner:inner + self.channels], proj[:, inner + self.channels:]
        conv = ctx.rows("state_space.conv", self.channels, torch.float32)
        ops.short_conv_silu(conv, raw, self.conv_state, self.conv_taps, ctx.token_segment, rows, slots, out_bias=self.conv_bias)
        ops.short_conv_keep(self.conv_state, raw, rows, lengths, slots)
        xs, B, C = conv[:, :inner], conv[:, inner:inner + self.bc_width], conv[:, inner + self.bc_width:]
        steps = ctx.rows("state_space.steps", 2 * H, torch.float32)
        dt, decay = steps[:, :H], steps[:, H:]
        ops.scan_gate(dt, dt_raw, "softplus", bias=self.dt_bias)
        ops.scan_gate(decay, dt_raw, "step_decay", bias=self.dt_bias, per_head=self.a_log, head_width=1)
        o = ctx.rows("state_space.read", inner, torch.float32)
        ops.linear_scan(o, self.state, C, B, xs, decay, dt, rows, lengths, slots, H, G, N, V, "scaled_add", decay_per_head=True)
        gated = ctx.rows("state_space.out", inner)
        ops.gate_group_norm(gated, o, xs, self.skip, z, self.norm_weight, H, self.norm_groups, self.norm_eps)
        product(ctx, out, gated, self.w_o, self.w_o_tiles)

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        y = ctx.rows("mixer.rows_out", self.hidden, torch.float32)
        self.forward_into(ctx, y, h, cache_layer, writes_cache)
        ops.residual_add(x, y)


@register_mixer("rglru")
class RealGatedRecurrentUnit(_StateMixer):
    """Tensor names by role: y, y_bias, x, x_bias (the two branches), conv ([width, taps]), conv_bias,
    decay_gate and input_gate ([blocks, block, block], [out, in]) with decay_gate_bias and input_gate_bias
    ([blocks, block]), lam ([width]), o."""

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.width, self.blocks = spec.get("width"), spec.get("blocks", 1)
        self.taps = spec.get("conv")
        self.decay_scale = float(spec.get("decay_scale", 8.0))
        if self.width % self.blocks:
            raise ValueError(f"{self.width} channels are not {self.blocks} equal blocks")
        if self.taps < 1:
            raise ValueError("the short convolution has at least one tap")
        self.block = self.width // self.blocks
        self.names = self._names(spec, dict(
            y="y_proj.weight", y_bias="y_proj.bias", x="x_proj.weight", x_bias="x_proj.bias", conv="conv.weight",
            conv_bias="conv.bias", decay_gate="a_gate.weight", decay_gate_bias="a_gate.bias", input_gate="i_gate.weight",
            input_gate_bias="i_gate.bias", lam="lambda", o="out_proj.weight"))

    def tensor_specs(self):
        n, W, nb, bs = self.names, self.width, self.blocks, self.block
        return [TensorSpec(n["y"], (W, self.hidden)), TensorSpec(n["y_bias"], (W,), role="vector"),
                TensorSpec(n["x"], (W, self.hidden)), TensorSpec(n["x_bias"], (W,), role="vector"),
                TensorSpec(n["conv"], (W, self.taps), role="vector"), TensorSpec(n["conv_bias"], (W,), role="vector"),
                TensorSpec(n["decay_gate"], (nb, bs, bs), role="vector"), TensorSpec(n["decay_gate_bias"], (nb, bs), role="vector"),
                TensorSpec(n["input_gate"], (nb, bs, bs), role="vector"), TensorSpec(n["input_gate_bias"], (nb, bs), role="vector"),
                TensorSpec(n["lam"], (W,), role="vector"), TensorSpec(n["o"], (self.hidden, W))]

    def bind(self, tensors):
        n = self.names
        f32 = lambda name: tensors.pop(name).to(torch.float32).contiguous()      # noqa: E731
        # one product for both branches: [y | x]
        self.w_in = torch.cat([tensors.pop(n["y"]), tensors.pop(n["x"])], dim=0).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.y_bias, self.x_bias = f32(n["y_bias"]), f32(n["x_bias"])
        self.conv_taps, self.conv_bias = f32(n["conv"]), f32(n["conv_bias"])
        # both gates of a block as one float32 product, [block][in][decay gate's outputs | input gate's outputs]
        gates = torch.cat([f32(n["decay_gate"]), f32(n["input_gate"])], dim=1)          # [blocks, 2 block (out), block (in)]
        self.w_gates = gates.transpose(1, 2).contiguous()
        self.gate_bias = torch.cat([f32(n["decay_gate_bias"]), f32(n["input_gate_bias"])], dim=1).contiguous().view(-1)
        self.rate = (-self.decay_scale * F.softplus(f32(n["lam"]))).contiguous()       # the decay's logarithm a unit of its gate
        self.w_in_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_in, self.w_o)

    def state_specs(self):
        return [(self.prefix + "state", (self.width,), torch.float32),
                (self.prefix + "conv_state", (self.taps - 1, self.width), self.dtype)]

    def prepare(self, info):
        self.state = info.storage.states[self.prefix + "state"]
        self.conv_state = info.storage.states[self.prefix + "conv_state"]

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        W = self.width
        rows, lengths, slots = self._segments(ctx)
        proj = ctx.rows("rglru.in", 2 * W)
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        y, raw = proj[:, :W], proj[:, W:]
        u = ctx.rows("rglru.conv", W, torch.float32)
        ops.short_conv_silu(u, raw, self.conv_state, self.conv_taps, ctx.token_segment, rows, slots, in_bias=self.x_bias,
                            out_bias=self.conv_bias, activation="none")
        ops.short_conv_keep(self.conv_state, raw, rows, lengths, slots, in_bias=self.x_bias)
        gates = ctx.rows("rglru.gates", 2 * W, torch.float32)
        ops.head_linear(gates, u, self.w_gates, self.blocks, self.block, 2 * self.block)
        read = ctx.rows("rglru.read", W)
        longest = max(s.length for s in ctx.segments)
        words = ops.rglru_scan_scratch(longest, len(ctx.segments), W)
        scratch = ctx.workspace.flat("rglru.chunks", words, torch.float32) if words else None
        ops.rglru_scan(read, self.state, gates, self.gate_bias, u, self.rate, y, self.y_bias, rows, lengths, slots, self.block,
                       longest=longest, scratch=scratch)
        product(ctx, out, read, self.w_o, self.w_o_tiles)

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        y = ctx.rows("mixer.rows_out", self.hidden, torch.float32)
        self.forward_into(ctx, y, h, cache_layer, writes_cache)
        ops.residual_add(x, y)
