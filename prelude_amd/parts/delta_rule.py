"""The gated delta rule: a recurrent mixer whose memory is a matrix of fixed size per head, corrected token by token.

With h the mixer's input, per token: q = W_q h and k = W_k h (``num_kv_heads`` heads of ``head_dim``), v = W_v h
(``num_heads`` heads of ``value_dim``; head i uses q/k head floor(i / (heads / kv_heads))).  Each of q, k, v passes a short
causal convolution per channel (``conv`` taps, the last one the token's own, zeros before a request's start) and SiLU;
q and k then become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also times head_dim^(-1/2).
beta = sigmoid(W_b h), one per head.  A decay per head and key channel,
g = exp(-exp(A_log_head) softplus(W_a2 (W_a1 h) + dt_bias)).  Per head, in this order:

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

Each head's o over its own sqrt(mean^2 + eps), times a weight shared by the heads, times sigmoid(W_g2 (W_g1 h)); then
the output projection.  S (32-bit, zero at a request's start) and the convolution's last ``conv`` - 1 inputs live in a
state slot of the request.  Everything from the convolution to the norm is computed in 32-bit.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, VECTOR, Mixer, PartError, StateSpec, TensorReq, register_part


@register_part("mixer", "gated_delta_rule")
class GatedDeltaRule(Mixer):
    LAUNCHES = 8   # three projections, convolution and state, recurrence, norm and gate, output projection
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; rows and state slots are read on the device

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, conv: int,
                 norm_eps: float, rank: Optional[int] = None):
        for name, v in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads),
                        ("head_dim", head_dim), ("value_dim", value_dim), ("conv", conv)):
            if int(v) <= 0:
                raise PartError(f"gated_delta_rule: {name} {v} must be positive")
        if num_heads % num_kv_heads:
            raise PartError(f"gated_delta_rule: {num_heads} heads are not a multiple of {num_kv_heads} query/key heads")
        if head_dim > 256 or conv > 9:
            raise PartError(f"gated_delta_rule: a key width of {head_dim} (at most 256) or {conv} taps (at most 9)")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.conv, self.norm_eps = int(head_dim), int(value_dim), int(conv), float(norm_eps)
        # inner size of the two-step projections of the decay and the gate; None: whatever the tensors have
        self.rank = int(rank) if rank else None
        self.w_in = self.w_low = self.w_up = self.w_o = None
        self.conv_weight = self.a_log = self.dt_bias = self.out_norm = None

    @property
    def channels(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.value_dim

    @property
    def mixed_size(self) -> int:
        return self.num_heads * self.value_dim

    def cache_spec(self):
        return StateSpec((("conv", (self.channels, self.conv - 1), torch.float32),
                          ("s", (self.num_heads, self.head_dim, self.value_dim), torch.float32)))

    def tensors(self):
        h, qk, vv, hd = self.hidden_size, self.num_kv_heads * self.head_dim, self.mixed_size, self.num_heads * self.head_dim
        r = self.rank if self.rank else -1
        return {"q": TensorReq((qk, h), MATRIX), "k": TensorReq((qk, h), MATRIX), "v": TensorReq((vv, h), MATRIX),
                "q.conv": TensorReq((qk, self.conv), VECTOR), "k.conv": TensorReq((qk, self.conv), VECTOR),
                "v.conv": TensorReq((vv, self.conv), VECTOR), "b": TensorReq((self.num_heads, h), MATRIX),
                "A_log": TensorReq((self.num_heads,), VECTOR), "dt_bias": TensorReq((hd,), VECTOR),
                "a1": TensorReq((r, h), MATRIX), "a2": TensorReq((hd, r), MATRIX), "g1": TensorReq((r, h), MATRIX),
                "g2": TensorReq((vv, r), MATRIX), "norm": TensorReq((self.value_dim,), NORM), "o": TensorReq((h, vv), MATRIX)}

    def input_rows(self, tensors) -> torch.Tensor:
        """The rows of the product of its input this mixer wants, [q | k | v | b]; keeps its other tensors."""
        r = tensors["a1"].shape[0]
        if tensors["g1"].shape[0] != r or tensors["a2"].shape[1] != r or tensors["g2"].shape[1] != r:
            raise PartError("gated_delta_rule: the two-step projections of the decay and the gate disagree about their inner size")
        dev, dt = tensors["a1"].device, tensors["a1"].dtype
        self.conv_weight = torch.cat([tensors["q.conv"], tensors["k.conv"], tensors["v.conv"]], dim=0).contiguous()
        self.a_log, self.dt_bias, self.out_norm = tensors["A_log"], tensors["dt_bias"], tensors["norm"]
        # the first steps of the decay's and the gate's projections as one product, the second steps as one product with a
        # weight of two blocks (a2 reads the first r columns, g2 the last r; the zeros add nothing)
        self.w_low = K.prepare_weight(torch.cat([tensors["a1"], tensors["g1"]], dim=0).contiguous())
        hd, vv = self.num_heads * self.head_dim, self.mixed_size
        up = torch.zeros((hd + vv, 2 * r), dtype=dt, device=dev)
        up[:hd, :r] = tensors["a2"]
        up[hd:, r:] = tensors["g2"]
        self.w_up = K.prepare_weight(up)
        return torch.cat([tensors[n] for n in ("q", "k", "v", "b")], dim=0)

    def load(self, tensors, dtype, device):
        self.w_in = K.prepare_weight(self.input_rows(tensors).contiguous())
        self.w_o = K.prepare_weight(tensors["o"])

    def mix(self, x, p, off, step, cache, write_cache, out=None, out_scale=1.0):
        """From the mixer's input ``x`` and the product ``p`` of it (this mixer's columns start at ``off``) to the normed,
        gated heads side by side [T, heads * value_dim], times ``out_scale``, into ``out`` when given."""
        if not write_cache:
            raise PartError("gated_delta_rule: a run cannot read another run's state; every run keeps its own")
        nh, kvh, d, e = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        ag = K.linear(K.linear(x, self.w_low), self.w_up)          # [T, heads * d | heads * e]: decay input, gate input
        xs, decay, beta = K.delta_prepare(p, off, off + self.channels, self.conv_weight, cache.tensors["conv"], ag, 0,
                                          self.a_log, self.dt_bias, step, nh, kvh, d, e)
        o = K.gated_delta(xs, decay, beta, cache.tensors["s"], step, nh, kvh, d, e)
        return K.head_norm_gate(o, ag[:, nh * d:], self.out_norm, self.norm_eps, "sigmoid", out, out_scale)

    def forward(self, x, step, cache, write_cache=True):
        p = K.linear(x, self.w_in)
        return K.linear(self.mix(x, p, 0, step, cache, write_cache), self.w_o, slices_ok=True)
