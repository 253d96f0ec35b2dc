"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases.

crates/prelude-core/src/models/qwen3.rs:383-448; silu(x) = x / (1 + e^-x) in
32-bit (crates/prelude-cuda/src/kernels/kernels_src/elementwise/silu_mul.cu:26-33).
Gate and up are one matrix [2I, H] here with rows alternating gate_j, up_j:
one product yields each (gate_j, up_j) pair side by side, so the activation
is the epilogue of that product for few rows and a pairwise kernel otherwise.
The reference's Qwen3 is wired to SiLU whatever ``hidden_act`` says
(qwen3.rs:429-447); the activation is a parameter here (SiLU, or GELU in its
tanh form: crates/prelude-core/src/models/commons/activation.rs:3-25), one
epilogue code in the same kernels.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import MATRIX, VECTOR, FeedForward, PartError, TensorReq, register_part


@register_part("ffn", "gated_mlp")
class GatedMLP(FeedForward):
    LAUNCHES = 3   # gate and up in one product, activation * up, down
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in K.GATE_ACTIVATIONS:
            raise PartError(f"gated_mlp: activation {activation!r} is not one of {sorted(K.GATE_ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.gate_up = None
        self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": TensorReq((i, h), MATRIX), "up_proj.weight": TensorReq((i, h), MATRIX),
                "down_proj.weight": TensorReq((h, i), MATRIX)}

    def load(self, tensors, dtype, device):
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.gate_up = K.prepare_weight(
            torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous())
        self.down = K.prepare_weight(tensors["down_proj.weight"])

    def forward(self, x):
        return K.linear(K.linear_gated(x, self.gate_up, self.activation), self.down, slices_ok=True)

    def forward_after_norm(self, x, residual, norm):
        # a few rows behind an RMS norm: the add and the norm ride in the gated product's staging of X
        rms = norm.as_rms() if residual is not None else None
        if rms is None or not K.gated_after_norm_supported(x, residual, self.gate_up, self.activation):
            return super().forward_after_norm(x, residual, norm)
        residual, h = K.linear_gated_after_norm(x, residual, rms[0], rms[1], self.gate_up, self.activation)
        return residual, K.linear(h, self.down, slices_ok=True)


@register_part("ffn", "clamped_gated_mlp")
class ClampedGatedMLP(FeedForward):
    """down(y) with g = min(gate(x), limit), u = clamp(up(x), -limit, limit), y = g * sigmoid(alpha * g) * (u + 1);
    ``limit`` and ``alpha`` are the model's constants.  Gate and up are one matrix with alternating rows, as in
    ``gated_mlp``; the activation is computed in 32-bit from the product's pairs."""
    LAUNCHES = 3
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702):
        if not limit > 0:
            raise PartError(f"clamped_gated_mlp: a limit of {limit} is not positive")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.limit, self.alpha = float(limit), float(alpha)
        self.gate_up = None
        self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"gate": TensorReq((i, h), MATRIX), "up": TensorReq((i, h), MATRIX), "down": TensorReq((h, i), MATRIX)}

    def load(self, tensors, dtype, device):
        self.gate_up = K.prepare_weight(torch.stack([tensors["gate"], tensors["up"]], dim=1)
                                        .reshape(2 * self.intermediate_size, self.hidden_size).contiguous())
        self.down = K.prepare_weight(tensors["down"])

    def forward(self, x):
        return K.linear(K.linear_clamped_gate(x, self.gate_up, self.limit, self.alpha), self.down, slices_ok=True)


@register_part("ffn", "squared_relu_mlp")
class SquaredReluMLP(FeedForward):
    """down(relu(up(x))^2): two products and the square of relu between them, no gate and no biases."""
    LAUNCHES = 3
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.up = self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"up": TensorReq((i, h), MATRIX), "down": TensorReq((h, i), MATRIX)}

    def load(self, tensors, dtype, device):
        self.up, self.down = K.prepare_weight(tensors["up"]), K.prepare_weight(tensors["down"])

    def forward(self, x):
        return K.linear(K.relu_squared(K.linear(x, self.up)), self.down, slices_ok=True)


@register_part("ffn", "poly_norm_mlp")
class PolyNormMLP(FeedForward):
    """down(act(up(x))) with biases on both products and act(z) = a N(z) + b N(z^2) + c N(z^3) + e: powers element by
    element, N(u) = u over sqrt(mean(u^2) + eps) across the inner size, (a, b, c, e) four learned numbers.  The first
    product's bias is added where the activation reads z."""
    LAUNCHES = 3
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, intermediate_size: int, eps: float):
        self.hidden_size, self.intermediate_size, self.eps = int(hidden_size), int(intermediate_size), float(eps)
        self.up = self.down = self.up_bias = self.down_bias = self.coeff = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"up": TensorReq((i, h), MATRIX), "up.b": TensorReq((i,), VECTOR), "down": TensorReq((h, i), MATRIX),
                "down.b": TensorReq((h,), VECTOR), "act": TensorReq((4,), VECTOR)}

    def load(self, tensors, dtype, device):
        self.up, self.down = K.prepare_weight(tensors["up"]), K.prepare_weight(tensors["down"])
        self.up_bias, self.down_bias, self.coeff = tensors["up.b"], tensors["down.b"], tensors["act"]

    def forward(self, x):
        z = K.linear(x, self.up)
        return K.linear(K.poly_norm(z, self.coeff, self.eps, bias=self.up_bias), self.down, self.down_bias)
