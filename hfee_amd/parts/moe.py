"""Feed-forwards of many small experts, of which every token uses `top`.

"table_moe": no router.  A table [vocabulary, top] of integers gives every token id its experts (the
entries of a row differ); each counts 1 / top.  Expert: down(act(gate(h)) * up(h)), act the SiLU, no
biases; the output is the weighted sum of the chosen experts' outputs, added to the residual stream in
float32.  The experts' matrices are stacked [experts, rows, columns] when they are bound; the lookup
runs on the device from the step's token ids, so a step may be replayed from a recorded graph.  A step
with more (token, expert) pairs than experts groups the pairs by expert on the device and multiplies them
in tiles on the matrix cores (bfloat16, sizes that are multiples of 32); a step of few tokens, and
float32, reads each token's experts row by row.

"routed_moe": a router chooses.  z = W_router h in float32; scores s = sigmoid(z); the `top` experts with
the largest scores are a token's, and their weights are those scores as they are (not renormalized).
Expert: down(relu(up(w h))^2), no gate and no biases: the weight w multiplies the expert's input (it joins
the up product's float32 sum, which is the same product).  The output is the sum of the chosen experts'
outputs.  It writes float32 rows (`forward_into`) for a block that norms them, or adds them to the stream.
Steps of many tokens go through the same grouped kernels as above, few tokens and float32 row by row.
Its parameters make other routed experts of it: `score` "softmax" takes the softmax of z over all experts as
the scores; `correction` adds a learned number an expert to the scores where the experts are chosen, and only
there; `activation` "silu" gives the experts a gate, down(silu(gate(h)) * up(h)); `weight_on` "output"
multiplies an expert's output by its weight instead of its input.
"""
from __future__ import annotations

import torch

from ..config.specs import FeedForwardSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, LazyNorm, register_feed_forward


@register_feed_forward("table_moe")
class TableMoE(FeedForward):
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.experts, self.top = spec.get("experts"), spec.get("top")
        self.vocab = spec.get("vocab")
        if spec.get("activation", "silu") != "silu":
            raise ValueError("the experts' activation is the SiLU")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"a token uses 1 to {self.experts} experts, not {self.top}")
        given = dict(spec.get("names") or ())
        self.expert_names = given.get("expert", "experts.{}.")           # a format for the expert's number
        self.roles = {r: given.get(r, d) for r, d in dict(gate="gate_proj.weight", up="up_proj.weight",
                                                         down="down_proj.weight", table="table").items()}

    def _name(self, e: int, role: str) -> str:
        return self.prefix + self.expert_names.format(e) + self.roles[role]

    def tensor_specs(self):
        specs = []
        for e in range(self.experts):
            specs += [TensorSpec(self._name(e, "gate"), (self.intermediate, self.hidden)),
                      TensorSpec(self._name(e, "up"), (self.intermediate, self.hidden)),
                      TensorSpec(self._name(e, "down"), (self.hidden, self.intermediate))]
        specs.append(TensorSpec(self.prefix + self.roles["table"], (self.vocab, self.top), role="table",
                                init=("distinct_in_row", self.experts)))
        return specs

    def bind(self, tensors):
        E = range(self.experts)
        self.w_gate = torch.stack([tensors.pop(self._name(e, "gate")) for e in E]).contiguous()
        self.w_up = torch.stack([tensors.pop(self._name(e, "up")) for e in E]).contiguous()
        self.w_down = torch.stack([tensors.pop(self._name(e, "down")) for e in E]).contiguous()
        self.table = tensors.pop(self.prefix + self.roles["table"]).contiguous()
        lo, hi = int(self.table.min()), int(self.table.max())
        if lo < 0 or hi >= self.experts:
            raise ValueError(f"{self.prefix + self.roles['table']} names experts {lo}..{hi}, the layer has {self.experts}")

    def forward_add(self, ctx, x, h):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        n, top = ctx.n, self.top
        # more pairs than experts: grouped by expert, an expert's matrices are read once for all its tokens
        if n * top > self.experts and ops.moe_grouped_fits(self.dtype, self.hidden, self.intermediate) \
                and hn.data_ptr() % 16 == 0 and hn.stride(0) % 8 == 0:
            ws = ctx.workspace
            order = ws.flat("table_moe.order", ws.capacity * top, torch.int32)
            tiles = ws.flat("table_moe.tiles", 3 * ops.moe_group_tiles(ws.capacity, top, self.experts) + 1, torch.int32)
            act = ctx.rows("table_moe.act", top * self.intermediate)
            y = ctx.rows("table_moe.rows", top * self.hidden, torch.float32) if top > 1 else None
            ops.moe_grouped(x, hn, self.w_gate, self.w_up, self.w_down, top, order, tiles, act, y, weight=1.0 / top,
                            table=self.table, token_ids=ctx.token_ids)
            return
        act = ctx.rows("table_moe.act", self.top * self.intermediate).view(ctx.n * self.top, self.intermediate)
        ops.moe_up(act, hn, self.w_gate, self.w_up, self.top, table=self.table, token_ids=ctx.token_ids)
        ops.moe_down(x, act, self.w_down, self.top, weight=1.0 / self.top, table=self.table, token_ids=ctx.token_ids)


@register_feed_forward("routed_moe")
class RoutedMoE(FeedForward):
    """Tensor names by role: router ([experts, hidden]), correction ([experts]); expert (a format for the expert's
    number), gate, up, down."""
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.experts, self.top = spec.get("experts"), spec.get("top")
        self.activation, self.score = spec.get("activation", "relu2"), spec.get("score", "sigmoid")
        self.weight_on = spec.get("weight_on", "input")
        self.has_correction = bool(spec.get("correction", False))
        if self.activation not in ("relu2", "silu") or self.score not in ops.ROUTER_SCORES:
            raise ValueError("the routed experts' activation is 'relu2' (no gate) or 'silu' (gated), their scores "
                             f"one of {sorted(ops.ROUTER_SCORES)}")
        self.gated = self.activation == "silu"
        if self.weight_on != ("output" if self.gated else "input") or spec.get("renormalize", False):
            raise ValueError("the weights multiply the inputs of experts without a gate and the outputs of gated ones, "
                             "and are not renormalized")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"a token uses 1 to {self.experts} experts, not {self.top}")
        given = dict(spec.get("names") or ())
        self.expert_names = given.get("expert", "experts.{}.")
        self.roles = {r: given.get(r, d) for r, d in dict(gate="gate_proj.weight", up="up_proj.weight", down="down_proj.weight",
                                                         router="router.weight", correction="router.correction").items()}
        self.output_bias = None
        self.correction = None

    def _name(self, e: int, role: str) -> str:
        return self.prefix + self.expert_names.format(e) + self.roles[role]

    def tensor_specs(self):
        specs = []
        for e in range(self.experts):
            if self.gated:
                specs.append(TensorSpec(self._name(e, "gate"), (self.intermediate, self.hidden)))
            specs += [TensorSpec(self._name(e, "up"), (self.intermediate, self.hidden)),
                      TensorSpec(self._name(e, "down"), (self.hidden, self.intermediate))]
        specs.append(TensorSpec(self.prefix + self.roles["router"], (self.experts, self.hidden)))
        if self.has_correction:
            specs.append(TensorSpec(self.prefix + self.roles["correction"], (self.experts,), role="vector"))
        return specs

    def bind(self, tensors):
        E = range(self.experts)
        self.w_gate = torch.stack([tensors.pop(self._name(e, "gate")) for e in E]).contiguous() if self.gated else None
        self.w_up = torch.stack([tensors.pop(self._name(e, "up")) for e in E]).contiguous()
        self.w_down = torch.stack([tensors.pop(self._name(e, "down")) for e in E]).contiguous()
        self.w_router = tensors.pop(self.prefix + self.roles["router"]).contiguous()
        if self.has_correction:
            self.correction = tensors.pop(self.prefix + self.roles["correction"]).to(torch.float32).contiguous()

    def _choose(self, ctx, hn):
        n, top = ctx.n, self.top
        logits = ctx.rows("routed_moe.logits", self.experts, torch.float32)
        ops.linear(logits, hn, self.w_router)
        ws = ctx.workspace
        chosen = ws.flat("routed_moe.chosen", ws.capacity * top, torch.int32)[:n * top].view(n, top)
        weights = ws.flat("routed_moe.weights", ws.capacity * top, torch.float32)[:n * top].view(n, top)
        ops.router_topk(chosen, weights, logits, top, score=self.score, correction=self.correction)
        return chosen, weights

    def _run(self, ctx, out, h, add: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        n, top = ctx.n, self.top
        chosen, weights = self._choose(ctx, hn)
        # (gated experts: the weight meets the output; experts without a gate: the input)
        on_input = None if self.gated else weights
        on_output = weights if self.gated else None
        if n * top > self.experts and ops.moe_grouped_fits(self.dtype, self.hidden, self.intermediate) \
                and hn.data_ptr() % 16 == 0 and hn.stride(0) % 8 == 0:
            ws = ctx.workspace
            order = ws.flat("table_moe.order", ws.capacity * top, torch.int32)
            tiles = ws.flat("table_moe.tiles", 3 * ops.moe_group_tiles(ws.capacity, top, self.experts) + 1, torch.int32)
            act = ctx.rows("table_moe.act", top * self.intermediate)
            y = ctx.rows("table_moe.rows", top * self.hidden, torch.float32) if top > 1 else None
            if not add:
                out.zero_()
            ops.moe_grouped(out, hn, self.w_gate, self.w_up, self.w_down, top, order, tiles, act, y, weight=1.0, chosen=chosen,
                            in_weights=on_input, pair_weights=on_output)
            return
        act = ctx.rows("table_moe.act", top * self.intermediate).view(n * top, self.intermediate)
        ops.moe_up(act, hn, self.w_gate, self.w_up, top, chosen=chosen, in_weights=on_input)
        ops.moe_down(out, act, self.w_down, top, weight=1.0, pair_weights=on_output, chosen=chosen, accumulate=add)

    def forward_into(self, ctx, out, h):
        self._run(ctx, out, h, add=False)

    def forward_add(self, ctx, x, h):
        self._run(ctx, x, h, add=True)
