"""Attention through a latent, with a learned sink in the softmax.

Queries come through a latent of their own: c_q = RMSNorm(W_dq h) * g_q, q = W_uq c_q, laid out head by head
as [dim unrotated | rot rotated].  One down projection gives rank + rot numbers a token: the first rank,
RMS-normed, are the latent c, the rest one rotated key part shared by all heads.  Head h's unrotated key is
W_uk[h] c and its value W_uv[h] c, so only c and the rotated part are cached (``LatentCacheSpec``), and both maps
move to the query side:

    score_h(i, j) = ((W_uk[h]^T q_h^unrot(i)) . c(j)  +  q_h^rot(i) . k^rot(j)) * scale
    out_h(i)      = W_uv[h] * sum_j p_h(i, j) c(j),     p = softmax over {scores, sink_h}

A head's sink is a learned scalar s_h: its softmax divides by sum_j exp(score_j) + exp(s_h).  Nothing is attended
to through it (it adds to the denominator only), and the score scale does not apply to it.  Rotation pairs dimension 2i with 2i + 1 over the first ``rotary_dim`` rotated dimensions.  Scores,
softmax, norms and angles are 32-bit whatever the engine's type.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, VECTOR, LatentCacheSpec, Mixer, PartError, TensorReq, register_part


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    LAUNCHES = 8   # down projections, prep, query up, absorb, rotation, attention, value up, output
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 q_rank: int, norm_eps: float, scale: Optional[float] = None, position: Optional[str] = None,
                 rotary_dim: Optional[int] = None, sink: bool = False, window: int = 0, output_gate: bool = False):
        for name, v in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim),
                        ("value_dim", value_dim), ("kv_rank", kv_rank), ("q_rank", q_rank)):
            if int(v) <= 0:
                raise PartError(f"latent_attention: {name} {v} must be positive")
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.rot_dim, self.value_dim, self.kv_rank, self.q_rank = int(rot_dim), int(value_dim), int(kv_rank), int(q_rank)
        self.norm_eps, self.window, self.sink = float(norm_eps), int(window or 0), bool(sink)
        # the heads' outputs side by side times sigmoid(W_g x), element by element (tensor ``g`` [heads * value_dim,
        # hidden]); the gate reads the mixer's input, as the projections do
        self.output_gate = bool(output_gate)
        self.position = position
        self.rotary_dim = (self.rot_dim if rotary_dim is None else int(rotary_dim)) if position else 0
        if self.rot_dim < 0 or self.rotary_dim > self.rot_dim or self.rotary_dim % 2:
            raise PartError(f"latent_attention: {self.rotary_dim} rotated dimensions of a part of {self.rot_dim}")
        if self.kv_rank + self.rot_dim > K.LATENT_MAX_WIDTH:
            raise PartError(f"latent_attention: a cached vector of {self.kv_rank} + {self.rot_dim} is more than the "
                            f"{K.LATENT_MAX_WIDTH} the kernels take")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim + self.rot_dim)
        self.rope = None
        self.w_down = self.w_uq = self.w_o = self.uk_t = self.uv_t = None
        self.q_norm = self.c_norm = self.sinks = None

    def cache_spec(self):
        return LatentCacheSpec(self.kv_rank, self.rot_dim, self.window)

    def bind(self, shared):
        if self.position is not None:
            if self.position not in shared:
                raise PartError(f"latent_attention: the model has no position encoding named {self.position!r}")
            self.rope = shared[self.position]
            if getattr(self.rope, "rotary_dim", None) != self.rotary_dim or not hasattr(self.rope, "inv_freq"):
                raise PartError(f"latent_attention: position encoding {self.position!r} must give the frequencies of "
                                f"{self.rotary_dim} rotated dimensions")

    def tensors(self):
        h, nh, d, r, v = self.hidden_size, self.num_heads, self.head_dim, self.rot_dim, self.value_dim
        t = {"dq": TensorReq((self.q_rank, h), MATRIX), "dq.norm": TensorReq((self.q_rank,), NORM),
             "uq": TensorReq((nh * (d + r), self.q_rank), MATRIX),
             "dkv": TensorReq((self.kv_rank + r, h), MATRIX), "dkv.norm": TensorReq((self.kv_rank,), NORM),
             "uk": TensorReq((nh * d, self.kv_rank), MATRIX), "uv": TensorReq((nh * v, self.kv_rank), MATRIX),
             "o": TensorReq((h, nh * v), MATRIX)}
        if self.sink:
            t["sink"] = TensorReq((nh,), VECTOR)
        if self.output_gate:
            t["g"] = TensorReq((nh * v, h), MATRIX)
        return t

    def load(self, tensors, dtype, device):
        nh, d, v, rank = self.num_heads, self.head_dim, self.value_dim, self.kv_rank
        # one product for both down projections: [q_rank | kv_rank | rot] rows
        down = [tensors["dq"], tensors["dkv"]] + ([tensors["g"]] if self.output_gate else [])   # the gate's rows ride along
        self.w_down = K.prepare_weight(torch.cat(down, dim=0).contiguous())
        self.w_uq = K.prepare_weight(tensors["uq"])
        self.w_o = K.prepare_weight(tensors["o"])
        # the per-head maps as [head, out, in]: W_uk[h] is [d, rank] as stored and is applied transposed (out rank,
        # in d); W_uv[h] is [v, rank] and is applied as it is
        self.uk_t = K.GroupedWeight(tensors["uk"].reshape(nh, d, rank).transpose(1, 2))
        self.uv_t = K.GroupedWeight(tensors["uv"].reshape(nh, v, rank))
        self.q_norm, self.c_norm = tensors["dq.norm"], tensors["dkv.norm"]
        self.sinks = tensors["sink"] if self.sink else None

    def forward(self, x, step, cache, write_cache=True):
        nh, d, r, v, rank = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank
        g = step.kv[cache.group]
        freq = self.rope.inv_freq if self.rope is not None else None
        down = K.linear(x, self.w_down)
        gate = None
        if self.output_gate:
            gate = down[:, self.q_rank + rank + r:]
            down = down[:, : self.q_rank + rank + r]
        cq = K.latent_prep(down, self.q_norm, self.c_norm, freq, step.positions, g.slots if write_cache else None,
                           cache.latent if write_cache else None, self.q_rank, rank, r, self.rotary_dim, self.norm_eps,
                           cache_t=cache.latent_t if write_cache else None)
        q = K.linear(cq, self.w_uq).view(-1, nh, d + r)
        ql = torch.empty((q.shape[0], nh, rank + r), dtype=q.dtype, device=q.device)
        K.head_linear(q, self.uk_t, ql)                                             # the key map, on the query side
        if r:
            K.rotate_pairs(q, ql, freq, step.positions, d, rank, r, self.rotary_dim)
        ol = K.latent_attention(ql, cache.latent, self.sinks, g, step, rank, self.window, self.scale, cache_t=cache.latent_t)
        o = torch.empty((q.shape[0], nh, v), dtype=q.dtype, device=q.device)
        K.head_linear(ol, self.uv_t, o)                                            # the value map, after the sum
        o = o.view(-1, nh * v)
        if gate is not None:
            o = K.sigmoid_gate(o, gate)
        return K.linear(o, self.w_o, slices_ok=True)
