"""Four mixers over one family of attention kernels, whose keys and values have sizes of their own.

"kv_attention": grouped attention.  H query heads over G key/value heads (query head h reads
key/value head h // (H/G)), key size Dk, value size Dv; q and k are rotated in the first
`rotary_dim` dims of each head (the position part's tables carry the amplitude of a stretched
rotation); score = q.k * scale over the keys up to the token's own position; the softmax may have a
sink, one learned number a head that joins the denominator only (`sink`); the values may be blended
with those that the first blending layer of the model computed for the same token (`value_blend`:
"source" keeps its values of the step for the layers behind it, "mix" writes
(1 - t) v + t v_source with its own learned t, and the blended values are what the cache holds).

"latent_attention": queries and keys/values through low-rank latents.  c_q = norm(W_dq h),
q = W_uq c_q, laid out head by head as [plain dims | rotated dims]; W_dkv h gives the latent c
(normed) and one rotated key part that all heads share; per head k = [W_uk c | rotated part],
v = W_uv c.  Only c and the rotated part are cached, and the attention runs in the absorbed form:
since q_plain . (W_uk,h c) = (W_uk,h^T q_plain) . c, the query of head h becomes
[W_uk,h^T q_plain | q_rotated] against the one cached row [c | rotated part] (one key/value head of
size rank + rotated dims), the weighted sum is taken over the latents themselves (value size =
rank), and W_uv,h is applied to the result.  Prompt portions and single tokens then run the same
kernels, and a token's logits do not depend on how its prompt was cut.

With `window` a query sees the last `window` positions only, itself included; with `cache_window` (at least
the window of every layer that reads the cache layer) the layer's pages form a "window" group of the cache
manager, which takes back the pages that every such window has passed.  With `own_keys` False the
layer has no W_dkv: it reads the latent and the rotated key part that another layer of the same latent
size, rotated part and rotation keeps (the schedule names that layer's cache), with its own W_uk and W_uv.
The rotation's pairs may be (i, i + half) or (2i, 2i + 1): the score is a sum over the rotated dims, so for
the second kind the rows of W_uq's and W_dkv's rotated parts are put in the order evens, odds when they are
bound, and the kernels turn pairs (i, i + half) of that order.

"window_attention": grouped attention over a sliding window with pooled blocks.  q, k and v may pass a
short causal convolution a channel (`conv` taps, no bias, no activation; the last taps - 1 projections of a
request are state); q and k are rotated; with `value_norm_eps` a head's value is divided by its root mean
square and cached so; score = q.k * scale, with `softcap` c then c * tanh(score / c); a query sees the last
`window` positions and, with `pool` = P, one key and one value for every block of P positions that lies
wholly before the window (the means of the block's cached keys and values, made when the block's last token
is written, in a second cache layer that grows by one entry every P tokens, under the block's number); tokens
and blocks share one softmax; with `head_gate` a head's result is multiplied by sigmoid(W_g h)_h.

"sigmoid_attention": grouped attention without a softmax and without a rotation.  q and k are divided
by their root mean square over each head (eps `norm_eps`) and multiplied by a weight of the head's size
that all heads share, one for q and one for k; with `temperature` = (coef, every) the query at position p
is also multiplied by 1 + coef * ln(floor((p + 1) / every) + 1); score = q.k * scale; a key up to the
token's own position weighs sigmoid(score + b_h), b_h a learned number a head, and the weights are not
normalized over the keys: every key adds on its own, however far back it lies.

All write float32 rows for a block that norms a sub-layer's output before it adds it to the
residual stream (`forward_into`); `forward_add` is there for the other blocks.

In bfloat16 with sizes that are multiples of 16 the matrix-core kernels run (rows of a prompt
portion in tiles of 16, single tokens with the heads of a key/value head as the tile's rows and
the keys split over waves); any other size, and float32, goes through the plain kernel.
"""
from __future__ import annotations

import numpy as np
import torch

from ..config.specs import CacheNeed, MixerSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import LazyNorm, Mixer, lookup, register_mixer

_ROWS = 16             # rows of a matrix-core tile: the heads of a key/value head that one wave takes for a single token
_KEY_TILE = 32         # keys of a step of the matrix-core kernels
_WAVES_WANTED = 2048   # single tokens split their keys until about this many waves run
_MOST_SPLITS = 64
_LAYOUT = "keys by slot, then values by dimension"


def plan_items(plan, rows: int) -> None:
    """The step's work for the matrix-core kernels, once a step whichever layers ask: portions in
    tiles of `rows` rows (the most that the kernels of a layer's sizes take), single tokens one by
    one (first row, rows, first position, block-table row)."""
    if f"attention_kv.portions.{rows}" not in plan.arrays:
        portions = [(seg.row0 + off, min(rows, seg.length - off), seg.start + off, s)
                    for s, seg in enumerate(plan.segments) if seg.length > 1 for off in range(0, seg.length, rows)]
        plan.add(f"attention_kv.portions.{rows}", np.asarray(portions, dtype=np.int32).reshape(-1, 4))
    if "attention_kv.singles" not in plan.arrays:
        singles = [(seg.row0, 1, seg.start, s) for s, seg in enumerate(plan.segments) if seg.length == 1]
        plan.add("attention_kv.singles", np.asarray(singles, dtype=np.int32).reshape(-1, 4))
        plan.host["attention_kv.single_max_position"] = max([p for _, _, p, _ in singles], default=0)


def attend(ctx, out, q, cache, tables, num_heads, kv_heads, dk, dv, scale, sinks, matrix: bool, weights: str = "softmax",
           sight=None, gate=None) -> None:
    """weights "sigmoid": no softmax, `sinks` holds the number a head that joins every score.  sight: None, or
    dict(window, pool, softcap, pooled, pool_tables) of a mixer whose queries do not see every earlier key as it is."""
    sight = sight or {}
    if not matrix:
        ops.attention_kv_plain(out, q, cache, ctx.positions, ctx.token_segment, tables, num_heads, kv_heads, dk, dv,
                               ctx.page_size, scale, sinks, weights=weights, gate=gate, **sight)
        return
    portions = ctx.extra[f"attention_kv.portions.{ops.attention_kv_rows(dk, dv, num_heads // kv_heads, weights)}"]
    singles = ctx.extra["attention_kv.singles"]
    if portions.shape[0]:
        ops.attention_kv_bf16(out, q, cache, portions, 0, tables, num_heads, kv_heads, dk, dv, ctx.page_size, scale, sinks,
                              weights=weights, gate=gate, **sight)
    count = singles.shape[0]
    if count:
        # under a captured graph the split count is fixed for the whole width of the block table
        span = ctx.host.get("graph.max_context", ctx.host["attention_kv.single_max_position"] + 1)
        tiles = -(-span // _KEY_TILE)
        if sight.get("window"):        # the window's tiles, and those of the pooled blocks before it
            pooled = span // sight["pool"] if sight.get("pool") else 0
            tiles = min(tiles, -(-sight["window"] // _KEY_TILE) + 1 + -(-pooled // _KEY_TILE))
        units = kv_heads * -(-(num_heads // kv_heads) // _ROWS)
        # (a split walks four tiles at least of keys and values of 256 dims together, and fewer of larger ones)
        splits = max(1, min(tiles // max(1, 1024 // (dk + dv)), _WAVES_WANTED // (count * units), _MOST_SPLITS))
        partial = None
        if splits > 1:
            partial = ctx.workspace.flat("attention_kv.partial", ops.attention_kv_partial_words(count, num_heads, dv, splits),
                                         torch.float32)
        ops.attention_kv_bf16(out, q, cache, singles, 1, tables, num_heads, kv_heads, dk, dv, ctx.page_size, scale, sinks,
                              partial=partial, splits=splits, weights=weights, gate=gate, **sight)


def tiles_of(dtype, *weights):
    """The weights' second copies in tiles, which the products of up to 64 rows stream (None where
    the engine is not bfloat16, a width is no multiple of 8, or the memory has no room)."""
    if dtype != torch.bfloat16 or any(w.shape[0] % 8 or w.shape[1] % 8 for w in weights):
        return (None,) * len(weights)
    return ops.tile_weights_if_room(*weights) or (None,) * len(weights)


def product(ctx, out, x, weight, tiles=None, add: bool = False) -> None:
    """out = x @ weight.T: up to 64 rows stream the weight's tiles, more go through the tiled kernels.
    add: out (float32, the residual stream) += the product."""
    n = x.shape[0]
    # (the kernels that stream tiles load 16 bytes a lane: a block of columns of a wider buffer must start and
    # repeat at such a place)
    if tiles is not None and n <= ops.SKINNY_MAX_ROWS and x.data_ptr() % 16 == 0 and (n == 1 or x.stride(0) % 8 == 0):
        ops.linear_fused(out, x, tiles, "add" if add else "f32" if out.dtype == torch.float32 else "bf16",
                         **ctx.workspace.product_scratch(n, tiles))
    else:
        ops.linear(out, x, weight, accumulate=add, **ctx.workspace.split_scratch(n, weight))


class _KvMixer(Mixer):
    graph_safe = True
    weights = "softmax"       # how a key's weight comes from its score (`ops.KEY_WEIGHTS`)

    def _names(self, spec, defaults):
        given = dict(spec.get("names") or ())
        return {role: self.prefix + given.get(role, default) for role, default in defaults.items()}

    def _matrix(self, dk, dv, q_width, out_width) -> bool:
        return (self.dtype == torch.bfloat16 and ops.attention_kv_sizes_fit(dk, dv) and q_width % 8 == 0
                and out_width % 4 == 0)

    def prepare(self, info):
        if self.position is not None:
            self.position.prepare(info.num_positions, info.device)

    def plan(self, plan):
        if self.matrix:
            plan_items(plan, ops.attention_kv_rows(*self.kernel_sizes, self.weights))

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        y = ctx.rows("mixer.rows_out", self.hidden, torch.float32)
        self.forward_into(ctx, y, h, cache_layer, writes_cache)
        ops.residual_add(x, y)

    def _tables(self, ctx, cache_layer):
        return ctx.block_tables[ctx.storage.group_of(cache_layer)]


@register_mixer("kv_attention")
class KvAttention(_KvMixer):
    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.kv_heads = spec.get("num_kv_heads", self.num_heads)
        self.dk = spec.get("key_dim")
        self.dv = spec.get("value_dim", self.dk)
        self.scale = float(spec.get("scale", self.dk ** -0.5))
        self.has_sink = bool(spec.get("sink", False))
        self.blend = spec.get("value_blend")              # None | "source" | "mix"
        if self.blend not in (None, "source", "mix"):
            raise ValueError(f"value_blend is None, 'source' or 'mix', not {self.blend!r}")
        if self.num_heads % self.kv_heads:
            raise ValueError(f"{self.num_heads} heads are not a multiple of {self.kv_heads} kv heads")
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        if self.position is not None and self.position.pairing != 0:
            raise ValueError("kv_attention rotates pairs (i, i + half)")
        self.names = self._names(spec, dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", o="o_proj.weight",
                                            sink="sinks", value_blend="value_blend"))
        self.q_width, self.k_width, self.v_width = self.num_heads * self.dk, self.kv_heads * self.dk, self.kv_heads * self.dv
        self.out_width = self.num_heads * self.dv
        self.kernel_sizes = (self.dk, self.dv, self.num_heads // self.kv_heads)
        self.matrix = self._matrix(self.dk, self.dv, self.q_width + self.k_width + self.v_width, self.out_width)

    def tensor_specs(self):
        n = self.names
        specs = [TensorSpec(n["q"], (self.q_width, self.hidden)), TensorSpec(n["k"], (self.k_width, self.hidden)),
                 TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["o"], (self.hidden, self.out_width))]
        if self.has_sink:
            specs.append(TensorSpec(n["sink"], (self.num_heads,), role="vector"))
        # (a layer that blends nothing may still carry the number in its checkpoint)
        specs.append(TensorSpec(n["value_blend"], (), role="vector", optional=self.blend != "mix"))
        return specs

    def bind(self, tensors):
        n = self.names
        self.w_qkv = torch.cat([tensors.pop(n["q"]), tensors.pop(n["k"]), tensors.pop(n["v"])], dim=0).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.sinks = tensors.pop(n["sink"]).to(torch.float32).contiguous() if self.has_sink else None
        t = tensors.pop(n["value_blend"], None)
        self.blend_weight = t.reshape(1).to(self.dtype).contiguous() if (t is not None and self.blend == "mix") else None
        self.w_qkv_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_qkv, self.w_o)

    def cache_spec(self):
        return CacheNeed("full", (self.kv_heads, self.dk + self.dv), 0, layout=_LAYOUT)

    def key_layout(self):
        pos = self.position
        return (self.kv_heads, self.dk, self.dv, None if pos is None else pos.signature())

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        n = ctx.n
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, dk, dv = self.num_heads, self.kv_heads, self.dk, self.dv
        cache = ctx.storage.layer(cache_layer, (G, ctx.page_size * (dk + dv)))
        tables = self._tables(ctx, cache_layer)
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        qkv = ctx.rows("kv_attention.qkv", self.q_width + self.k_width + self.v_width)
        q = qkv[:, :self.q_width]
        if writes_cache:
            product(ctx, qkv, hn, self.w_qkv, self.w_qkv_tiles)
            k = qkv[:, self.q_width:self.q_width + self.k_width]
            v = qkv[:, self.q_width + self.k_width:]
        else:       # this run of the layer reads keys and values that another run wrote
            ops.linear(q, hn, self.w_qkv[:self.q_width])
            k = v = None
        first = None
        if self.blend is not None and writes_cache:       # the source's values of this step's tokens
            first = ctx.workspace.rows("kv_attention.blend_source", n, self.v_width, self.dtype)
        ops.kv_write(q, k, v, ctx.positions, ctx.token_segment, tables, cos, sin, cache, H, G, dk, dk, dv, ctx.page_size,
                     ctx.max_position, v_first=first, v_first_mode={None: 0, "source": 1, "mix": 2}[self.blend],
                     v_mix=self.blend_weight)
        att = ctx.rows("kv_attention.out", self.out_width)
        attend(ctx, att, q, cache, tables, H, G, dk, dv, self.scale, self.sinks, self.matrix)
        product(ctx, out, att, self.w_o, self.w_o_tiles)


@register_mixer("sigmoid_attention")
class SigmoidAttention(_KvMixer):
    """Tensor names by role: q, k, v, o (matrices), q_norm, k_norm ([key_dim]), head_bias ([heads])."""
    weights = "sigmoid"

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.kv_heads = spec.get("num_kv_heads", self.num_heads)
        self.dk = spec.get("key_dim")
        self.dv = spec.get("value_dim", self.dk)
        self.scale = float(spec.get("scale", self.dk ** -0.5))
        self.norm_eps = float(spec.get("norm_eps", 1e-6))
        self.temperature = spec.get("temperature")          # None | (coef, every)
        if self.num_heads % self.kv_heads:
            raise ValueError(f"{self.num_heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.temperature is not None and int(self.temperature[1]) < 1:
            raise ValueError("the query temperature grows in steps of at least one position")
        self.position = None
        self.names = self._names(spec, dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", o="o_proj.weight",
                                            q_norm="q_norm.weight", k_norm="k_norm.weight", head_bias="head_bias"))
        self.q_width, self.k_width, self.v_width = self.num_heads * self.dk, self.kv_heads * self.dk, self.kv_heads * self.dv
        self.out_width = self.num_heads * self.dv
        self.kernel_sizes = (self.dk, self.dv, self.num_heads // self.kv_heads)
        self.matrix = self._matrix(self.dk, self.dv, self.q_width + self.k_width + self.v_width, self.out_width)

    def tensor_specs(self):
        n = self.names
        return [TensorSpec(n["q"], (self.q_width, self.hidden)), TensorSpec(n["k"], (self.k_width, self.hidden)),
                TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["o"], (self.hidden, self.out_width)),
                TensorSpec(n["q_norm"], (self.dk,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["k_norm"], (self.dk,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["head_bias"], (self.num_heads,), role="vector")]

    def bind(self, tensors):
        n = self.names
        self.w_qkv = torch.cat([tensors.pop(n["q"]), tensors.pop(n["k"]), tensors.pop(n["v"])], dim=0).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.q_norm = tensors.pop(n["q_norm"]).to(torch.float32).contiguous()
        self.k_norm = tensors.pop(n["k_norm"]).to(torch.float32).contiguous()
        self.head_bias = tensors.pop(n["head_bias"]).to(torch.float32).contiguous()
        self.w_qkv_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_qkv, self.w_o)

    def cache_spec(self):
        return CacheNeed("full", (self.kv_heads, self.dk + self.dv), 0, layout=_LAYOUT)

    def key_layout(self):
        return (self.kv_heads, self.dk, self.dv, "normed", self.norm_eps)

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, dk, dv = self.num_heads, self.kv_heads, self.dk, self.dv
        cache = ctx.storage.layer(cache_layer, (G, ctx.page_size * (dk + dv)))
        tables = self._tables(ctx, cache_layer)
        qkv = ctx.rows("kv_attention.qkv", self.q_width + self.k_width + self.v_width)
        q = qkv[:, :self.q_width]
        k = v = None
        if writes_cache:
            product(ctx, qkv, hn, self.w_qkv, self.w_qkv_tiles)
            k = qkv[:, self.q_width:self.q_width + self.k_width]
            v = qkv[:, self.q_width + self.k_width:]
        else:       # this run of the layer reads keys and values that another run wrote
            ops.linear(q, hn, self.w_qkv[:self.q_width])
        ops.qk_norm_write(q, k, v, ctx.positions, ctx.token_segment, tables, cache, self.q_norm, self.k_norm, self.norm_eps,
                          H, G, dk, dv, ctx.page_size, temperature=self.temperature)
        att = ctx.rows("kv_attention.out", self.out_width)
        attend(ctx, att, q, cache, tables, H, G, dk, dv, self.scale, self.head_bias, self.matrix, weights="sigmoid")
        product(ctx, out, att, self.w_o, self.w_o_tiles)


@register_mixer("latent_attention")
class LatentAttention(_KvMixer):
    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.plain = spec.get("plain_dim")
        self.rotated = spec.get("rotated_dim")
        self.dv = spec.get("value_dim", self.plain)
        self.q_rank, self.kv_rank = spec.get("q_rank"), spec.get("kv_rank")
        self.scale = float(spec.get("scale", (self.plain + self.rotated) ** -0.5))
        self.eps = float(spec.get("norm_eps", 1e-6))
        self.window = int(spec.get("window", 0))
        self.cache_window = int(spec.get("cache_window", 0) or 0)
        if self.cache_window and not 0 < self.window <= self.cache_window:
            raise ValueError(f"a cache that keeps {self.cache_window} positions cannot serve a window of {self.window or 'all'}")
        self.own_keys = bool(spec.get("own_keys", True))
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        if self.position is not None and self.position.rotary_dim != self.rotated:
            raise ValueError("latent_attention rotates the whole rotated part")
        self.pairing = self.position.pairing if self.position is not None else 0
        self.names = self._names(spec, dict(q_down="q_a_proj.weight", q_norm="q_a_norm.weight", q_up="q_b_proj.weight",
                                            kv_down="kv_a_proj.weight", kv_norm="kv_a_norm.weight", k_up="k_b_proj.weight",
                                            v_up="v_b_proj.weight", o="o_proj.weight"))
        # the absorbed form: one key/value head, keys [latent | rotated part], values the latent
        self.dk_abs, self.dv_abs = self.kv_rank + self.rotated, self.kv_rank
        self.kernel_sizes = (self.dk_abs, self.dv_abs, self.num_heads)
        self.down_width = self.q_rank + (self.kv_rank + self.rotated if self.own_keys else 0)
        self.matrix = (self._matrix(self.dk_abs, self.dv_abs, self.num_heads * self.dk_abs, self.num_heads * self.dv_abs)
                       and self.down_width % 8 == 0 and self.q_rank % 8 == 0)
        self.sight = dict(window=self.window) if self.window else None

    def tensor_specs(self):
        n, H = self.names, self.num_heads
        own = [TensorSpec(n["kv_down"], (self.kv_rank + self.rotated, self.hidden)),
               TensorSpec(n["kv_norm"], (self.kv_rank,), role="vector", init=("one_plus_normal",))] if self.own_keys else []
        return [TensorSpec(n["q_down"], (self.q_rank, self.hidden)),
                TensorSpec(n["q_norm"], (self.q_rank,), role="vector", init=("one_plus_normal",)),
                TensorSpec(n["q_up"], (H * (self.plain + self.rotated), self.q_rank)), *own,
                TensorSpec(n["k_up"], (H * self.plain, self.kv_rank)),
                TensorSpec(n["v_up"], (H * self.dv, self.kv_rank)),
                TensorSpec(n["o"], (self.hidden, H * self.dv))]

    def bind(self, tensors):
        n, H = self.names, self.num_heads
        # pairs (2i, 2i + 1): the rotated rows in the order evens, odds, whose pairs are (i, i + half)
        turn = torch.arange(self.rotated)
        if self.pairing == 1:
            turn = torch.cat([turn[0::2], turn[1::2]])
        w_down = [tensors.pop(n["q_down"])]
        self.kv_norm = None
        if self.own_keys:
            kv_down = tensors.pop(n["kv_down"])
            w_down += [kv_down[:self.kv_rank], kv_down[self.kv_rank:][turn.to(kv_down.device)]]
            self.kv_norm = tensors.pop(n["kv_norm"]).to(torch.float32).contiguous()
        self.w_down = torch.cat(w_down, dim=0).contiguous()
        self.q_norm = tensors.pop(n["q_norm"]).to(torch.float32).contiguous()
        q_up = tensors.pop(n["q_up"])
        per_head = torch.cat([torch.arange(self.plain), self.plain + turn]).to(q_up.device)
        self.w_q_up = q_up.view(H, self.plain + self.rotated, self.q_rank)[:, per_head].reshape(q_up.shape).contiguous()
        # per head, as [inputs][outputs]: W_uk,h^T maps the plain query dims onto the latent, W_uv,h the
        # weighted latent onto the head's values
        self.w_k_absorb = tensors.pop(n["k_up"]).view(H, self.plain, self.kv_rank).contiguous()
        self.w_v_expand = tensors.pop(n["v_up"]).view(H, self.dv, self.kv_rank).transpose(1, 2).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.w_down_tiles, self.w_q_up_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_down, self.w_q_up, self.w_o)

    def cache_spec(self):
        if self.cache_window:
            return CacheNeed("window", (1, self.dk_abs + self.dv_abs), self.cache_window, layout=_LAYOUT)
        return CacheNeed("full", (1, self.dk_abs + self.dv_abs), 0, layout=_LAYOUT)

    def key_layout(self):
        pos = self.position
        return (1, self.dk_abs, self.dv_abs, None if pos is None else (pos.signature(), self.pairing))

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        n, H = ctx.n, self.num_heads
        if writes_cache and not self.own_keys:
            raise ValueError("a latent-attention layer without keys of its own reads another layer's cache")
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        R, Dr, Dn = self.kv_rank, self.rotated, self.plain
        dk, dv = self.dk_abs, self.dv_abs
        cache = ctx.storage.layer(cache_layer, (1, ctx.page_size * (dk + dv)))
        tables = self._tables(ctx, cache_layer)
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        down = ctx.rows("latent.down", self.down_width)
        if writes_cache or not self.own_keys:
            product(ctx, down, hn, self.w_down, self.w_down_tiles)
        else:
            ops.linear(down[:, :self.q_rank], hn, self.w_down[:self.q_rank])
        cq = ctx.rows("latent.q_latent", self.q_rank)
        ops.rmsnorm_cols(cq, down[:, :self.q_rank], self.q_norm, self.eps)
        q = ctx.rows("latent.q", H * (Dn + Dr))
        product(ctx, q, cq, self.w_q_up, self.w_q_up_tiles)
        qa = ctx.rows("latent.q_absorbed", H * dk)
        ops.head_linear(qa, q, self.w_k_absorb, H, Dn, R, tail=Dr)
        k = v = None
        if writes_cache:
            c = down[:, self.q_rank:self.q_rank + R]
            ops.rmsnorm_cols(c, c, self.kv_norm, self.eps)
            k, v = down[:, self.q_rank:], c
        ops.kv_write(qa, k, v, ctx.positions, ctx.token_segment, tables, cos, sin, cache, H, 1, dk, dk, dv, ctx.page_size,
                     ctx.max_position, q_rot_offset=R, k_rot_offset=R)
        att = ctx.rows("latent.mixed", H * dv)
        attend(ctx, att, qa, cache, tables, H, 1, dk, dv, self.scale, None, self.matrix, sight=self.sight)
        heads_out = ctx.rows("latent.values", H * self.dv)
        ops.head_linear(heads_out, att, self.w_v_expand, H, R, self.dv)
        product(ctx, out, heads_out, self.w_o, self.w_o_tiles)


@register_mixer("window_attention")
class WindowAttention(_KvMixer):
    """Tensor names by role: q, k, v, o (matrices), q_conv, k_conv, v_conv ([channels, taps]), head_gate
    ([heads, hidden])."""

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.kv_heads = spec.get("num_kv_heads", self.num_heads)
        self.dk = spec.get("key_dim")
        self.dv = spec.get("value_dim", self.dk)
        self.scale = float(spec.get("scale", self.dk ** -0.5))
        self.softcap = float(spec.get("softcap", 0.0) or 0.0)
        self.taps = int(spec.get("conv", 0) or 0)
        self.window, self.pool = int(spec.get("window", 0) or 0), int(spec.get("pool", 0) or 0)
        self.value_norm_eps = spec.get("value_norm_eps")          # None: the values as they are
        self.has_gate = bool(spec.get("head_gate", False))
        if self.num_heads % self.kv_heads:
            raise ValueError(f"{self.num_heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.window < 0 or self.pool < 0 or self.softcap < 0 or self.taps < 0:
            raise ValueError("window, pool, softcap and conv are not negative")
        if not self.window:
            self.pool = 0                  # (without a window nothing ever lies before it)
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        if self.position is not None and self.position.pairing != 0:
            raise ValueError("window_attention rotates pairs (i, i + half)")
        self.names = self._names(spec, dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", o="o_proj.weight",
                                            q_conv="q_conv.weight", k_conv="k_conv.weight", v_conv="v_conv.weight",
                                            head_gate="gate_proj.weight"))
        self.q_width, self.k_width, self.v_width = self.num_heads * self.dk, self.kv_heads * self.dk, self.kv_heads * self.dv
        self.out_width = self.num_heads * self.dv
        self.channels = self.q_width + self.k_width + self.v_width
        self.kernel_sizes = (self.dk, self.dv, self.num_heads // self.kv_heads)
        self.matrix = self._matrix(self.dk, self.dv, self.q_width, self.out_width)

    def tensor_specs(self):
        n = self.names
        specs = [TensorSpec(n["q"], (self.q_width, self.hidden)), TensorSpec(n["k"], (self.k_width, self.hidden)),
                 TensorSpec(n["v"], (self.v_width, self.hidden)), TensorSpec(n["o"], (self.hidden, self.out_width))]
        if self.taps:
            specs += [TensorSpec(n["q_conv"], (self.q_width, self.taps), role="vector"),
                      TensorSpec(n["k_conv"], (self.k_width, self.taps), role="vector"),
                      TensorSpec(n["v_conv"], (self.v_width, self.taps), role="vector")]
        if self.has_gate:
            specs.append(TensorSpec(n["head_gate"], (self.num_heads, self.hidden)))
        return specs

    def bind(self, tensors):
        n = self.names
        # one product for everything that reads the layer's input: [q | k | v | a gate a head]
        rows = [tensors.pop(n["q"]), tensors.pop(n["k"]), tensors.pop(n["v"])]
        if self.has_gate:
            rows.append(tensors.pop(n["head_gate"]))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.conv_taps = None
        if self.taps:
            self.conv_taps = torch.cat([tensors.pop(n[r]).to(torch.float32) for r in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.w_in_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_in, self.w_o)

    def cache_spec(self):
        # a token is read by the queries of the next `window` positions and, once more, when its block is pooled
        keep = max(self.window, self.pool)
        tokens = CacheNeed("window" if self.window else "full", (self.kv_heads, self.dk + self.dv), keep if self.window else 0,
                           layout=_LAYOUT)
        if not self.pool:
            return tokens
        # the pooled blocks: a second cache layer, one entry of the tokens' shape every `pool` tokens
        return (tokens, CacheNeed("full", (self.kv_heads, self.dk + self.dv), 0, layout=_LAYOUT, every=self.pool))

    def key_layout(self):
        pos = self.position
        return (self.kv_heads, self.dk, self.dv, self.pool, self.taps, self.value_norm_eps,
                None if pos is None else pos.signature())

    def state_specs(self):
        return [(self.prefix + "conv_state", (self.taps - 1, self.channels), self.dtype)] if self.taps else []

    def prepare(self, info):
        super().prepare(info)
        self.conv_state = info.storage.states[self.prefix + "conv_state"] if self.taps else None

    def forward_into(self, ctx, out, h, cache_layer: int, writes_cache: bool):
        if not writes_cache:
            raise ValueError("window_attention keeps its own keys: a request's convolution state belongs to one run of the layer")
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, dk, dv = self.num_heads, self.kv_heads, self.dk, self.dv
        cache = ctx.storage.layer(cache_layer, (G, ctx.page_size * (dk + dv)))
        tables = self._tables(ctx, cache_layer)
        sight = dict(window=self.window, pool=self.pool, softcap=self.softcap)
        if self.pool:
            sight.update(pooled=ctx.storage.layer((cache_layer, 1), (G, ctx.page_size * (dk + dv))),
                         pool_tables=self._tables(ctx, (cache_layer, 1)))
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        total = self.w_in.shape[0]       # (rows of a multiple of 8 elements, so that blocks of columns stay aligned)
        proj = ctx.rows("window_attention.in", (total + 7) // 8 * 8)[:, :total]
        product(ctx, proj, hn, self.w_in, self.w_in_tiles)
        raw = proj[:, :self.channels]
        qkv = ctx.rows("window_attention.qkv", self.channels, torch.float32)
        if self.taps:
            ops.short_conv_silu(qkv, raw, self.conv_state, self.conv_taps, ctx.token_segment, ctx.segment_rows,
                                ctx.segment_slots, activation="none")
            ops.short_conv_keep(self.conv_state, raw, ctx.segment_rows, ctx.segment_lengths, ctx.segment_slots)
        else:
            ops.scan_gate(qkv, raw, "cast")
        q = ctx.rows("window_attention.q", self.q_width)
        ops.rotate_norm_write(q, qkv[:, :self.q_width], qkv[:, self.q_width:self.q_width + self.k_width],
                              qkv[:, self.q_width + self.k_width:], ctx.positions, ctx.token_segment, tables, cos, sin, cache,
                              H, G, dk, dv, ctx.page_size, ctx.max_position, value_eps=self.value_norm_eps)
        if self.pool:
            ops.kv_pool_write(cache, sight["pooled"], self.pool, ctx.positions, ctx.token_segment, tables, sight["pool_tables"],
                              G, dk, dv, ctx.page_size)
        gate = proj[:, self.channels:self.channels + H] if self.has_gate else None
        att = ctx.rows("kv_attention.out", self.out_width)
        attend(ctx, att, q, cache, tables, H, G, dk, dv, self.scale, None, self.matrix, sight=sight, gate=gate)
        product(ctx, out, att, self.w_o, self.w_o_tiles)
