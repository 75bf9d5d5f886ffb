"""A mixture of small gated feed-forward experts whose choice is a table over token ids.

Every token id has ``top`` experts of ``experts`` (a row of the integer table [vocab, top], its
entries distinct); the token's output is the mean of theirs (each weighs 1 / top).  No router is
computed: the experts of a token follow from the token alone, so the routing of a step is known
from its token ids (on the device: a step may take its tokens from what the step before sampled).
An optional shared expert of its own width runs for every token and is added.

An expert is a gated feed-forward without biases whose activation is a parameter
(``ops.gated_kind``); the design that brought it uses ("clamped_swish", limit, slope).

What ``forward`` returns is an ``ExpertRows``: the shared expert's output (possibly still the
unreduced slices of its down projection) beside the experts' uncombined rows; the norm that takes
the branch into the residual adds them while it reads them.

params: prefix, hidden_size, vocab_size, experts, top, intermediate_size, activation, shared
(None or {"intermediate_size", "activation"}), names (optional: "table", "expert" with {e} for
the expert's number, "shared", "gate", "up", "down").
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..weights.loader import TensorSpec
from .base import ExpertRows, FeedForward, Runtime, register_feed_forward


@register_feed_forward("table_moe")
class TableMoE(FeedForward):
    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.vocab = int(params["vocab_size"])
        self.experts = int(params["experts"])
        self.top = int(params["top"])
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"{self.prefix}: top={self.top} of {self.experts} experts")
        rt.ops.gated_kind(self.activation)  # raises for one the kernels do not know
        self.shared = params.get("shared")
        names = {"table": "table", "expert": "e{e}", "shared": "shared", "gate": "gate", "up": "up", "down": "down"}
        names.update(params.get("names", {}))
        self.names = names
        self.table = self.w_gate_up = self.w_down = None
        self.shared_gate_up = self.shared_down = None
        self.shared_group = 0

    def _name(self, owner: str, which: str) -> str:
        return f"{self.prefix}.{owner}.{self.names[which]}"

    def _expert(self, e: int) -> str:
        return self.names["expert"].format(e=e)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {f"{self.prefix}.{self.names['table']}": TensorSpec((self.vocab, self.top), "int", ("distinct", self.experts))}
        for e in range(self.experts):
            specs[self._name(self._expert(e), "gate")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(self._expert(e), "up")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(self._expert(e), "down")] = TensorSpec((self.hidden, self.inter))
        if self.shared:
            ff = int(self.shared["intermediate_size"])
            specs[self._name(self.names["shared"], "gate")] = TensorSpec((ff, self.hidden))
            specs[self._name(self.names["shared"], "up")] = TensorSpec((ff, self.hidden))
            specs[self._name(self.names["shared"], "down")] = TensorSpec((self.hidden, ff))
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        table = tensors[f"{self.prefix}.{self.names['table']}"]
        if int(table.min()) < 0 or int(table.max()) >= self.experts:
            raise ValueError(f"{self.prefix}: the table names experts outside 0..{self.experts - 1}")
        self.table = table.to(torch.int32).contiguous()
        # all experts in two tensors: [experts, 2, ff, hidden] (gate rows, then up rows) and [experts, hidden, ff]
        self.w_gate_up = torch.stack([
            torch.stack([tensors[self._name(self._expert(e), "gate")], tensors[self._name(self._expert(e), "up")]])
            for e in range(self.experts)
        ]).contiguous()
        self.w_down = torch.stack([tensors[self._name(self._expert(e), "down")] for e in range(self.experts)]).contiguous()
        if self.shared:
            s = self.names["shared"]
            self.shared_gate_up, self.shared_group = self.rt.ops.pack_gate_up(tensors[self._name(s, "gate")], tensors[self._name(s, "up")])
            self.shared_down = tensors[self._name(s, "down")]

    def products(self):
        if not self.shared:
            return ()
        ff = int(self.shared["intermediate_size"])
        return ((2 * ff, self.hidden), (self.hidden, ff))

    def forward(self, h: torch.Tensor, ctx):
        ops = self.rt.ops
        rows = ops.moe_experts(h, ctx.arrays["token_ids"], self.table, self.w_gate_up, self.w_down, self.activation)
        dense = None
        if self.shared:
            a = ops.gate_up_act(h, self.shared_gate_up, self.shared_group, self.shared["activation"], self.rt.act_dtype)
            dense = ops.linear(a, self.shared_down, self.rt.act_dtype, partial_ok=True)
        return ExpertRows(dense, rows, self.top, 1.0 / self.top)


@register_feed_forward("routed_moe")
class RoutedMoE(FeedForward):
    """A mixture whose experts a learned router chooses: logits z = W_router h in float32, scores s = sigmoid(z), the
    ``top`` experts with the largest scores; a chosen expert reads the token's input multiplied by its score (the
    score weighs what goes in, not what comes out; scores are not renormalised) and the outputs are summed.  An
    optional shared expert of the same form and a width of its own runs for every token and is added.  Experts
    are gated feed-forwards without biases, down(act(gate x) * (up x)).

    The router's product is a library product with float32 output; one kernel chooses and writes every token's row
    once per chosen expert, scaled (``ops.moe_router_topk``); the experts' two products are the grouped ones of
    ``ops.moe_experts`` with the router's choice as their table; one kernel sums a token's rows and the shared
    expert's output (``ops.moe_combine``).

    Other forms of the same mixture: ``router_bias`` (a tensor name below the prefix, [experts], added to the
    float32 logits before the choice), ``scores`` "softmax_of_chosen" (the chosen experts' weights are the softmax
    over their own logits alone; the default "sigmoid" is as above), ``weighs`` "output" (an expert reads the
    token's input as it is and its output is multiplied by the weight; the default "input" is as above),
    ``gated`` False (an expert is down(act(up x)) with ``activation`` one of the kernel library's plain ones,
    "relu2" the square of relu; no gate tensor).  With weights on the outputs ``forward`` returns the experts'
    uncombined rows beside their weights (``ExpertRows``) for whoever sums the branch into the stream.

    params: prefix, hidden_size, experts, top, intermediate_size, activation ("silu"), shared (None or
    {"intermediate_size", "activation"}), router_bias (None), scores ("sigmoid"), weighs ("input"), gated (True),
    names (optional: "router", "expert" with {e} for the expert's number, "shared", "gate", "up", "down")."""

    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.experts = int(params["experts"])
        self.top = int(params["top"])
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"{self.prefix}: top={self.top} of {self.experts} experts")
        self.gated = bool(params.get("gated", True))
        if self.gated:
            rt.ops.gated_kind(self.activation)
        else:
            rt.ops.plain_kind(self.activation)  # raises for one the kernels do not know
        self.router_bias_name = params.get("router_bias")
        self.router_bias = None
        self.scores = params.get("scores", "sigmoid")
        self.weighs = params.get("weighs", "input")
        if (self.scores, self.weighs) not in (("sigmoid", "input"), ("softmax_of_chosen", "output")):
            raise ValueError(f"{self.prefix}: scores={self.scores!r} with weighs={self.weighs!r} is not offered "
                             "(sigmoid scores weigh the inputs, a softmax over the chosen weighs the outputs)")
        self.shared = params.get("shared")
        names = {"router": "router", "expert": "e{e}", "shared": "shared", "gate": "gate", "up": "up", "down": "down"}
        names.update(params.get("names", {}))
        self.names = names
        self.router_rows = self.experts + (-self.experts % 16)
        self.w_router = self.w_gate_up = self.w_down = None
        self.shared_gate_up = self.shared_down = None
        self.shared_group = 0

    def _name(self, owner: str, which: str) -> str:
        return f"{self.prefix}.{owner}.{self.names[which]}"

    def _expert(self, e: int) -> str:
        return self.names["expert"].format(e=e)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        # (random routers are made wide enough that tokens differ in what they choose)
        specs = {f"{self.prefix}.{self.names['router']}": TensorSpec((self.experts, self.hidden), "float", ("normal", 0.5))}
        if self.router_bias_name:
            specs[f"{self.prefix}.{self.router_bias_name}"] = TensorSpec((self.experts,), "float", ("normal", 0.5))
        for e in range(self.experts):
            if self.gated:
                specs[self._name(self._expert(e), "gate")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(self._expert(e), "up")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(self._expert(e), "down")] = TensorSpec((self.hidden, self.inter))
        if self.shared:
            ff = int(self.shared["intermediate_size"])
            specs[self._name(self.names["shared"], "gate")] = TensorSpec((ff, self.hidden))
            specs[self._name(self.names["shared"], "up")] = TensorSpec((ff, self.hidden))
            specs[self._name(self.names["shared"], "down")] = TensorSpec((self.hidden, ff))
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        router = tensors[f"{self.prefix}.{self.names['router']}"]
        pad = self.router_rows - self.experts
        if pad:
            router = torch.cat([router, torch.zeros((pad, self.hidden), dtype=router.dtype, device=router.device)], dim=0)
        self.w_router = router.contiguous()
        if self.router_bias_name:
            self.router_bias = tensors[f"{self.prefix}.{self.router_bias_name}"].to(torch.float32).contiguous()
        # [experts, 2, ff, hidden] (gate rows, then up rows), or [experts, 1, ff, hidden] without gates
        self.w_gate_up = torch.stack([
            torch.stack(([tensors[self._name(self._expert(e), "gate")]] if self.gated else []) + [tensors[self._name(self._expert(e), "up")]])
            for e in range(self.experts)
        ]).contiguous()
        self.w_down = torch.stack([tensors[self._name(self._expert(e), "down")] for e in range(self.experts)]).contiguous()
        if self.shared:
            s = self.names["shared"]
            self.shared_gate_up, self.shared_group = self.rt.ops.pack_gate_up(tensors[self._name(s, "gate")], tensors[self._name(s, "up")])
            self.shared_down = tensors[self._name(s, "down")]

    def products(self):
        out = [(self.router_rows, self.hidden)]
        if self.shared:
            ff = int(self.shared["intermediate_size"])
            out += [(2 * ff, self.hidden), (self.hidden, ff)]
        return tuple(out)

    def forward(self, h: torch.Tensor, ctx):
        ops = self.rt.ops
        logits = ops.linear(h, self.w_router, torch.float32)
        if self.weighs == "output":
            choice, weights = ops.moe_router_topk(logits, None, self.top, experts=self.experts, bias=self.router_bias, scores=self.scores)
            rows = ops.moe_experts(h, None, choice, self.w_gate_up, self.w_down, self.activation, input_per_token=True)
            dense = None
            if self.shared:
                a = ops.gate_up_act(h, self.shared_gate_up, self.shared_group, self.shared.get("activation", "silu"), self.rt.act_dtype)
                dense = ops.linear(a, self.shared_down, self.rt.act_dtype, partial_ok=True)
            return ExpertRows(dense, rows, self.top, 1.0, row_weights=weights)
        choice, scaled = ops.moe_router_topk(logits, h, self.top, experts=self.experts, bias=self.router_bias)
        rows = ops.moe_experts(scaled, None, choice, self.w_gate_up, self.w_down, self.activation)
        dense = None
        if self.shared:
            a = ops.gate_up_act(h, self.shared_gate_up, self.shared_group, self.shared.get("activation", "silu"), self.rt.act_dtype)
            dense = ops.linear(a, self.shared_down, self.rt.act_dtype, partial_ok=True)
        return ops.moe_combine(dense, rows, self.top, 1.0)
