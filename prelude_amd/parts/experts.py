"""Feed-forwards of many small experts, of which every token uses a few: chosen from a table by token id
(``table_experts``) or by a router's scores (``routed_experts``, at the end of this file).

An expert is down(act(up(x))) without biases, act the square of relu.  Which experts a token uses is read from
a table by its token id (``table_experts``: a row of ``top`` distinct experts per id, each weighted 1 / top;
there is no router).  An optional shared expert of the same form runs for every token and is added.

The step's (token, choice) entries are put in the order of their experts on the device, the two products run
over tiles of that order, and a token's outputs are added in the order of its choices: no sum depends on what
else the step holds, nothing is decided on the host, and a captured step replays.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, TABLE, VECTOR, FeedForward, PartError, TensorReq, register_part


@register_part("ffn", "table_experts")
class TableExperts(FeedForward):
    NEEDS_STEP = True            # the experts are chosen by the step's token ids
    LAUNCHES = 9
    GRAPH_SAFE_PORTIONS = True   # every grid follows the step's shape; the choices are read on the device

    def __init__(self, hidden_size: int, vocab_size: int, num_experts: int, top: int, expert_size: int,
                 shared_size: int = 0):
        if not 1 <= int(top) <= int(num_experts):
            raise PartError(f"table_experts: {top} of {num_experts} experts a token")
        self.hidden_size, self.vocab_size = int(hidden_size), int(vocab_size)
        self.num_experts, self.top, self.expert_size = int(num_experts), int(top), int(expert_size)
        self.shared_size = int(shared_size or 0)
        self.table = self.up_t = self.down_t = self.shared_up = self.shared_down = None

    def tensors(self):
        h, f = self.hidden_size, self.expert_size
        t = {"table": TensorReq((self.vocab_size, self.top), TABLE, high=self.num_experts)}
        for e in range(self.num_experts):
            t[f"e{e}.up"] = TensorReq((f, h), MATRIX)
            t[f"e{e}.down"] = TensorReq((h, f), MATRIX)
        if self.shared_size:
            t["shared.up"] = TensorReq((self.shared_size, h), MATRIX)
            t["shared.down"] = TensorReq((h, self.shared_size), MATRIX)
        return t

    def load(self, tensors, dtype, device):
        n = self.num_experts
        self.table = tensors["table"]
        # one tensor [expert, out, in] per product
        self.up_t = K.GroupedWeight(torch.stack([tensors[f"e{e}.up"] for e in range(n)]))
        self.down_t = K.GroupedWeight(torch.stack([tensors[f"e{e}.down"] for e in range(n)]))
        if self.shared_size:
            self.shared_up = K.prepare_weight(tensors["shared.up"])
            self.shared_down = K.prepare_weight(tensors["shared.down"])

    def forward(self, x, step=None):
        if step is None:
            raise PartError("table_experts: the step's token ids are needed to choose the experts")
        choice = K.moe_choices_by_table(step.token_ids, self.table, self.num_experts)
        eo = K.moe_order(choice, self.num_experts, self.top)
        mid = K.moe_linear(x, self.up_t, eo, from_tokens=True, relu_squared_epilogue=True)
        y = K.moe_linear(mid, self.down_t, eo, from_tokens=False, out_dtype=torch.float32)
        base: Optional[torch.Tensor] = None
        if self.shared_size:
            base = K.as_tensor(K.linear(K.relu_squared(K.linear(x, self.shared_up)), self.shared_down))
        return K.moe_combine(y, eo, 1.0 / self.top, base, x.dtype)


@register_part("ffn", "routed_experts")
class RoutedExperts(FeedForward):
    """Experts chosen by a router.  Scores s = softmax(W_router x) over all experts, in 32-bit; a token's ``top``
    experts are those with the largest s + correction (a stored vector that bears on the choice alone); their
    weights are their s over the chosen ones' sum (+ 1e-20), times ``route_scale``.  An expert is a gated pair with
    both halves clamped, down(g * sigmoid(alpha g) * (u + 1)) with g = min(gate(x), limit) and u = clamp(up(x),
    -limit, limit), without biases.  An optional shared expert of the same form (its own size and limit) runs for
    every token and is added times sigmoid(w_sg . x), one number a token.

    The router and the shared expert's gate are one product ([experts + 1, hidden]) whose 32-bit sums one kernel turns
    into choices, weights and gates; from there on the path is that of ``table_experts``: entries in the order of
    their experts, two grouped products, the outputs added per token in the order of its choices.  Nothing is decided
    on the host."""
    LAUNCHES = 11
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, num_experts: int, top: int, expert_size: int, limit: float = 0.0, route_scale: float = 1.0,
                 alpha: float = 1.702, correction: bool = True, shared_size: int = 0, shared_limit: float = 0.0,
                 activation: str = "clamped", router_bias: bool = False, route: str = "scores"):
        """``activation``: ``"clamped"`` (the gated pair above) or ``"silu"`` (the plain gated pair silu(gate) * up, no
        clamps), for the experts and the shared expert alike.  ``router_bias``: a stored vector ``router.b`` is added to
        the router's logits.  ``route``: ``"scores"`` (above) or ``"chosen_logits"``: the ``top`` experts with the
        largest logits, weighted by the softmax over those logits alone (no correction)."""
        if not 1 <= int(top) <= int(num_experts):
            raise PartError(f"routed_experts: {top} of {num_experts} experts a token")
        if activation not in ("clamped", "silu"):
            raise PartError(f"routed_experts: activation {activation!r} is not one of 'clamped', 'silu'")
        if route not in ("scores", "chosen_logits"):
            raise PartError(f"routed_experts: route {route!r} is not one of 'scores', 'chosen_logits'")
        if route == "chosen_logits":
            correction = False
        if activation == "clamped" and (not limit > 0 or (shared_size and not shared_limit > 0)):
            raise PartError(f"routed_experts: the clamps {limit} and {shared_limit} must be positive")
        self.activation, self.has_router_bias, self.route = activation, bool(router_bias), route
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.expert_size, self.limit, self.alpha = int(expert_size), float(limit), float(alpha)
        self.route_scale, self.has_correction = float(route_scale), bool(correction)
        self.shared_size, self.shared_limit = int(shared_size or 0), float(shared_limit or 0.0)
        self.router = self.correction = self.router_bias = self.gate_up_t = self.down_t = None
        self.shared_gate_up = self.shared_down = None

    def tensors(self):
        h, f, n = self.hidden_size, self.expert_size, self.num_experts
        t = {"router": TensorReq((n, h), MATRIX)}
        if self.has_router_bias:
            t["router.b"] = TensorReq((n,), VECTOR)
        if self.has_correction:
            t["correction"] = TensorReq((n,), VECTOR)
        for e in range(n):
            t[f"e{e}.gate"] = TensorReq((f, h), MATRIX)
            t[f"e{e}.up"] = TensorReq((f, h), MATRIX)
            t[f"e{e}.down"] = TensorReq((h, f), MATRIX)
        if self.shared_size:
            s = self.shared_size
            t.update({"shared.gate": TensorReq((s, h), MATRIX), "shared.up": TensorReq((s, h), MATRIX),
                      "shared.down": TensorReq((h, s), MATRIX), "shared.sg": TensorReq((1, h), MATRIX)})
        return t

    @staticmethod
    def _pairs(gate, up):
        """Rows alternating gate_j, up_j: one product yields each pair side by side."""
        return torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()

    def load(self, tensors, dtype, device):
        n = self.num_experts
        rows = [tensors["router"]] + ([tensors["shared.sg"]] if self.shared_size else [])
        self.router = torch.cat(rows, dim=0).contiguous()
        self.correction = tensors["correction"] if self.has_correction else None
        self.router_bias = tensors["router.b"] if self.has_router_bias else None
        self.gate_up_t = K.GroupedWeight(torch.stack([self._pairs(tensors[f"e{e}.gate"], tensors[f"e{e}.up"]) for e in range(n)]))
        self.down_t = K.GroupedWeight(torch.stack([tensors[f"e{e}.down"] for e in range(n)]))
        if self.shared_size:
            self.shared_gate_up = K.prepare_weight(self._pairs(tensors["shared.gate"], tensors["shared.up"]))
            self.shared_down = K.prepare_weight(tensors["shared.down"])

    def forward(self, x, step=None):
        return self._run(x, None, None)

    def forward_into_stream(self, x, stream, other=None, step=None):
        """The kernel that adds up a token's experts adds the sum, unrounded, and ``other`` into the stream itself."""
        self._run(x, stream, None if other is None else K.as_tensor(other))

    def _run(self, x, stream, other):
        n = self.num_experts
        # the router's sums and scores are 32-bit (the operands are of the engine's type): a product of few columns
        logits = K.linear_narrow_f32(x, self.router)
        choice, weights, gate = K.moe_route(logits, n, self.top, self.route_scale, self.correction,
                                            gate_col=n if self.shared_size else -1, bias=self.router_bias,
                                            by_logit=self.route == "chosen_logits")
        eo = K.moe_order(choice, n, self.top)
        silu = self.activation == "silu"
        if silu:
            mid = K.moe_linear(x, self.gate_up_t, eo, from_tokens=True, silu_gate_epilogue=True)
        else:
            mid = K.moe_linear(x, self.gate_up_t, eo, from_tokens=True, clamped_gate_epilogue=(self.limit, self.alpha))
        y = K.moe_linear(mid, self.down_t, eo, from_tokens=False, out_dtype=torch.float32)
        base: Optional[torch.Tensor] = None
        if self.shared_size:
            mid_s = K.linear_gated(x, self.shared_gate_up, "silu") if silu else \
                K.linear_clamped_gate(x, self.shared_gate_up, self.shared_limit, self.alpha)
            base = K.as_tensor(K.linear(mid_s, self.shared_down))
        return K.moe_combine(y, eo, 1.0, base, x.dtype, weights=weights, base_scale=gate, into=stream, other=other)
