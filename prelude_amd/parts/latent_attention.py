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
import types
from typing import Optional

import numpy as np
import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, VECTOR, LatentCacheSpec, Mixer, PartError, TensorReq, register_part


def window_plan(step, window: int, page: int, device) -> types.SimpleNamespace:
    """For a step run directly (its host lists are its own): the cached positions every sequence of the step can see,
    from the first place of the page that holds its window's oldest key to its last token, as index arrays on the device
    -- ``seq`` / ``pos`` [N] (which cached vector), ``slots`` [N] (where its expansion goes in temporary pages that
    follow each other) -- and ``table`` [sequences, stride]: logical page -> temporary page for the pages that hold
    them (0 elsewhere: nothing visible lies there).  Built once a step and window, sent in one copy."""
    plans = step.__dict__.setdefault("_window_plans", {})
    key = (int(window), int(page))
    if key in plans:
        return plans[key]
    stride = int(step.kv[0].block_table.shape[1]) if step.kv else 1
    seqs, poss, slots = [], [], []
    table = np.zeros((step.num_seqs, stride), dtype=np.int32)
    at = 0   # temporary pages handed out so far
    for s, (start, n) in enumerate(zip(step.starts, step.q_lens)):
        end = start + n
        lo = max(0, start - (window - 1)) if window > 0 else 0
        first = lo // page
        last = (end - 1) // page
        table[s, first: last + 1] = np.arange(at, at + last + 1 - first, dtype=np.int32)
        p = np.arange(first * page, end, dtype=np.int32)
        seqs.append(np.full(p.shape, s, dtype=np.int32))
        poss.append(p)
        slots.append((at - first) * page + p)
        at += last + 1 - first
    total = sum(len(p) for p in poss)
    host = np.concatenate(seqs + poss + slots + [table.reshape(-1)]).astype(np.int32)
    dev = torch.from_numpy(host).to(device)
    plan = types.SimpleNamespace(seq=dev[:total], pos=dev[total: 2 * total], slots=dev[2 * total: 3 * total],
                                 table=dev[3 * total:].view(step.num_seqs, stride), pages=at, rows=total)
    plans[key] = plan
    return plan


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    LAUNCHES = 8   # down projections, prep, query up, absorb, rotation, attention, value up, output
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone (the expanded form below runs in direct steps only)
    # A step that brings this many tokens or more (and is run directly, in bfloat16, by a mixer without a rotated part
    # whose head sizes the matrix-core attention takes) attends in the expanded form: the keys and values of every
    # head are made from the latents its sequences can see, by one product, into temporary pages, and the queries
    # attend to them as they stand.  The form above moves both maps to the query side and pays rank + rot
    # multiplications a (query, key, head) where this one pays head_dim and value_dim; what it costs instead is the
    # product over the window's latents, which a short portion does not win back (measured at a latent of 512, heads of
    # 128 and a window of 1,024: level at some 350 tokens).
    EXPAND_FROM_TOKENS = 384

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
        self.w_down = self.w_uq = self.w_o = self.uk_t = self.uv_t = self.w_ukv = None
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
        if self.rot_dim == 0 and not self.sink and dtype == torch.bfloat16:
            # for the expanded form: every head's keys, then every head's values, from a latent by one product
            self.w_ukv = K.prepare_weight(torch.cat([tensors["uk"], tensors["uv"]], dim=0).contiguous())

    def _expands(self, x, step, cache, write_cache) -> bool:
        if not (self.w_ukv is not None and write_cache and x.dtype == torch.bfloat16 and getattr(step, "graph", None) is None
                and step.n_prefill > 0 and step.num_tokens >= self.EXPAND_FROM_TOKENS and len(step.starts) == step.num_seqs
                and K.attention_masked_mfma_supported(self.head_dim, self.value_dim, cache.latent.shape[1])):
            return False
        # not where the latents to expand outnumber the step's tokens several times (many single tokens, each with a
        # window behind it, beside a short portion)
        page = cache.latent.shape[1]
        rows = sum(min(s + n, n + (self.window or s + n) + page) for s, n in zip(step.starts, step.q_lens))
        return rows <= 4 * step.num_tokens

    def _expanded(self, q, step, cache, g):
        """The heads' outputs side by side [T, heads * value_dim] from keys and values made of the visible latents."""
        nh, d, v, rank = self.num_heads, self.head_dim, self.value_dim, self.kv_rank
        page = cache.latent.shape[1]
        plan = window_plan(step, self.window, page, q.device)
        kv = K.linear(K.latent_gather(cache.latent, g.block_table, plan.seq, plan.pos, rank), self.w_ukv)
        # zeroed: the places of a sequence's last page behind its last token are multiplied by weights of zero
        k_tmp = torch.zeros((plan.pages, nh, page, d), dtype=q.dtype, device=q.device)
        v_tmp = torch.zeros((plan.pages, nh, v, page), dtype=q.dtype, device=q.device)
        K.qkv_rope_prepare(kv, 0, 0, nh * d, None, plan.pos, plan.slots, k_tmp, v_tmp, 0, nh, nh, d, v, 0, False)
        return K.attention_masked(q.contiguous(), k_tmp, v_tmp, types.SimpleNamespace(block_table=plan.table), step, self.window, 0,
                                  self.scale)

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
        if self._expands(x, step, cache, write_cache):
            o = self._expanded(q, step, cache, g)
            if gate is not None:
                o = K.sigmoid_gate(o, gate)
            return K.linear(o, self.w_o, slices_ok=True)
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
