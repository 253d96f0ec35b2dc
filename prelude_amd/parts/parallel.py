"""Mixers side by side: several mixers read the same input, and the layer's mixer output is the sum of theirs, each
times a constant.

A member is any mixer that offers ``input_rows(tensors)`` (the rows of the product of its input it wants),
``mix(x, p, off, step, cache, write_cache, out, out_scale)`` (from that product to what its output projection reads,
written into a slice of a shared row) and ``mixed_size``, and names its output projection ``o``.  The members' input
rows are one product, and their output projections one product over the members' outputs side by side (each already
times its constant, in 32-bit before it is rounded): sum_i c_i W_i y_i = [W_1 | W_2 | ..] [c_1 y_1 | c_2 y_2 | ..].
What the members keep between steps stays their own: the layer has one cache per member that keeps something.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Sequence

import torch

from ..ops import kernels as K
from .base import Mixer, PartError, build_part, register_part


@register_part("mixer", "parallel_mixers")
class ParallelMixers(Mixer):
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, members: Sequence[Mapping[str, Any]]):
        """``members``: per member ``{"kind": ..., "params": {...}, "scale": c}``; a member's tensors are named
        ``"<index>.<its local name>"``."""
        if not members:
            raise PartError("parallel_mixers: no members")
        self.hidden_size = int(hidden_size)
        self.members, self.scales = [], []
        for m in members:
            part = build_part("mixer", m["kind"], m["params"])
            for need in ("input_rows", "mix", "mixed_size"):
                if not hasattr(part, need):
                    raise PartError(f"parallel_mixers: a {m['kind']} offers no `{need}` and cannot stand beside others")
            self.members.append(part)
            self.scales.append(float(m.get("scale", 1.0)))
        self.GRAPH_SAFE = all(p.GRAPH_SAFE for p in self.members)
        self.GRAPH_SAFE_PORTIONS = all(p.GRAPH_SAFE_PORTIONS for p in self.members)
        self.LAUNCHES = sum(p.LAUNCHES for p in self.members) - 2 * (len(self.members) - 1)
        self.ATOMIC_PREFILL = any(p.ATOMIC_PREFILL for p in self.members)
        self.w_in = self.w_o = None
        self.in_offsets, self.out_offsets = [], []

    def bind(self, shared):
        for p in self.members:
            p.bind(shared)

    def cache_spec(self):
        return tuple(cs for cs in (p.cache_spec() for p in self.members) if cs is not None)

    def tensors(self):
        return {f"{i}.{name}": req for i, p in enumerate(self.members) for name, req in p.tensors().items()}

    def load(self, tensors, dtype, device):
        rows, cols = [], []
        self.in_offsets, self.out_offsets = [], []
        n_in = n_out = 0
        for i, p in enumerate(self.members):
            own = {name[len(f"{i}."):]: t for name, t in tensors.items() if name.startswith(f"{i}.")}
            r = p.input_rows(own)
            rows.append(r)
            cols.append(own["o"])
            self.in_offsets.append(n_in)
            self.out_offsets.append(n_out)
            n_in += r.shape[0]
            n_out += p.mixed_size
        self.w_in = K.prepare_weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = K.prepare_weight(torch.cat(cols, dim=1).contiguous())
        self.total_out = n_out

    def forward(self, x, step, cache, write_cache=True):
        p = K.linear(x, self.w_in)
        mixed = torch.empty((x.shape[0], self.total_out), dtype=x.dtype, device=x.device)
        caches = iter(cache if isinstance(cache, tuple) else (cache,))
        for part, scale, off, ooff in zip(self.members, self.scales, self.in_offsets, self.out_offsets):
            c = next(caches) if part.cache_spec() is not None else None
            out = mixed[:, ooff: ooff + part.mixed_size]
            part.mix(x, p, off, step, c, write_cache, out, scale)
        return K.linear(mixed, self.w_o, slices_ok=True)
