"""Linear attention with a decaying state ("lightning attention"): a mixer whose memory is of fixed size.

Per head, with q, k [dim] and v [vdim] passed through an activation (SiLU):

    S_t = a_h S_(t-1) + k_t v_t^T          S [dim, vdim], from zero at a request's start
    o_t = S_t^T q_t

and no other scale.  The heads' outputs side by side are brought to unit RMS together, scaled by a weight,
multiplied by sigmoid(W_g h) and projected.  S is 32-bit and lives in a state slot of the request
(``StateSpec``), carried from step to step; the decays a_h are the model's constants.  Queries, keys, values and
the gate come from one merged product.

Variants, each a parameter: the first ``rotary_dim`` dimensions of every query and key head turned by position (in
halves, dimension i with i + rotary_dim / 2; the frequencies come from a position encoding that offers ``inv_freq``)
and the keys then multiplied by ``key_scale``, both in 32-bit on the way into the recurrence; every head brought to
unit RMS by itself (``head_norm``), with or without a weight (``norm_weight``); the gate through SiLU in place of the
sigmoid (``gate_activation``).
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, Mixer, PartError, StateSpec, TensorReq, register_part


@register_part("mixer", "lightning_attention")
class LightningAttention(Mixer):
    LAUNCHES = 4   # merged projection, the recurrence, norm and gate, output projection (one more with rotation)
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; rows and state slots are read on the device

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay: Sequence[float],
                 norm_eps: float, activation: str = "silu", position: Optional[str] = None, rotary_dim: int = 0,
                 key_scale: float = 1.0, head_norm: bool = False, norm_weight: bool = True, gate_activation: str = "sigmoid"):
        for name, v in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim), ("value_dim", value_dim)):
            if int(v) <= 0:
                raise PartError(f"lightning_attention: {name} {v} must be positive")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.decay = tuple(float(a) for a in decay)
        if len(self.decay) != self.num_heads or not all(0.0 <= a <= 1.0 for a in self.decay):
            raise PartError(f"lightning_attention: {len(self.decay)} decays {self.decay} for {self.num_heads} heads; each "
                            f"must lie in [0, 1]")
        if self.head_dim > 256:
            raise PartError(f"lightning_attention: a key width of {self.head_dim} is more than the 256 the kernels take")
        if activation not in K.LIGHTNING_ACTIVATIONS:
            raise PartError(f"lightning_attention: activation {activation!r} is not known")
        self.norm_eps, self.activation = float(norm_eps), activation
        self.position, self.rotary_dim, self.key_scale = position, int(rotary_dim) if position else 0, float(key_scale)
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise PartError(f"lightning_attention: {rotary_dim} turned dimensions must be even and at most the key width {head_dim}")
        self.head_norm, self.norm_weight = bool(head_norm), bool(norm_weight)
        if gate_activation not in K.HEAD_GATES:
            raise PartError(f"lightning_attention: gate activation {gate_activation!r} is not one of {sorted(K.HEAD_GATES)}")
        if not self.head_norm and (not self.norm_weight or gate_activation != "sigmoid"):
            raise PartError("lightning_attention: the norm over all heads together has a weight and a sigmoid gate")
        self.gate_activation = gate_activation
        self.rope = None
        self.w_in = self.w_o = self.out_norm = self.decays = None

    def cache_spec(self):
        return StateSpec((("s", (self.num_heads, self.head_dim, self.value_dim), torch.float32),))

    def bind(self, shared):
        if self.position is not None:
            self.rope = shared.get(self.position)
            if self.rope is None or not hasattr(self.rope, "inv_freq") or getattr(self.rope, "rotary_dim", None) != self.rotary_dim:
                raise PartError(f"lightning_attention: the model has no position encoding {self.position!r} that offers "
                                f"frequencies for {self.rotary_dim} turned dimensions")

    def tensors(self):
        h, qk, vv = self.hidden_size, self.num_heads * self.head_dim, self.num_heads * self.value_dim
        t = {"q": TensorReq((qk, h), MATRIX), "k": TensorReq((qk, h), MATRIX), "v": TensorReq((vv, h), MATRIX),
             "g": TensorReq((vv, h), MATRIX), "o": TensorReq((h, vv), MATRIX)}
        if self.norm_weight:
            t["norm"] = TensorReq((self.value_dim if self.head_norm else vv,), NORM)
        return t

    def load(self, tensors, dtype, device):
        # one product for queries, keys, values and the gate: rows [q | k | v | g]
        self.w_in = K.prepare_weight(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = K.prepare_weight(tensors["o"])
        self.out_norm = tensors.get("norm")
        self.decays = torch.tensor(self.decay, dtype=torch.float32, device=device)

    def forward(self, x, step, cache, write_cache=True):
        if not write_cache:
            raise PartError("lightning_attention: a run cannot read another run's state; every run keeps its own")
        nh, d, vd = self.num_heads, self.head_dim, self.value_dim
        qk, vv = nh * d, nh * vd
        p = K.linear(x, self.w_in)
        if self.rope is not None or self.key_scale != 1.0:
            # rotation and the keys' scale in 32-bit, between the product and the recurrence
            r = K.rotate_halves_f32(p, 0, qk, 2 * qk, self.rope.inv_freq if self.rope is not None else None, step.positions,
                                    nh, d, vd, self.rotary_dim, self.key_scale)
            o = K.lightning_attention(r, 0, qk, 2 * qk, self.decays, cache.tensors["s"], step, nh, d, vd, self.activation,
                                      chunk=K.LIGHTNING_CHUNK if p.dtype == torch.bfloat16 else 0)
        else:
            o = K.lightning_attention(p, 0, qk, 2 * qk, self.decays, cache.tensors["s"], step, nh, d, vd, self.activation)
        if self.head_norm:
            y = K.head_norm_gate(o, p[:, 2 * qk + vv:], self.out_norm, self.norm_eps, self.gate_activation)
        else:
            y = K.gated_rmsnorm(o.view(-1, vv), p[:, 2 * qk + vv:], self.out_norm, self.norm_eps)
        return K.linear(y, self.w_o, slices_ok=True)
