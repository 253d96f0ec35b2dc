"""A short causal convolution over time in front of any mixer.

What the mixer reads, h, becomes h + conv(h) with conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j) on every channel by
itself (``w`` [channels, taps], no bias; zeros before the sequence's start).  The last taps - 1 inputs are part of a
request's state: a slot of its own beside whatever the mixer behind it keeps, so the layer has the mixer's cache and
this one.  The sum is taken in 32-bit and rounded once.
"""
from __future__ import annotations

from typing import Any, Mapping

import torch

from ..ops import kernels as K
from .base import VECTOR, Mixer, PartError, StateSpec, TensorReq, build_part, register_part


@register_part("mixer", "conv_input")
class ConvInputMixer(Mixer):
    def __init__(self, hidden_size: int, taps: int, inner: Mapping[str, Any]):
        """``inner``: ``{"kind": ..., "params": {...}}``, the mixer that reads the convolved input; its tensors are named
        ``"inner.<its local name>"``, the convolution's ``"conv"``."""
        if not 1 <= int(taps) <= 17:
            raise PartError(f"conv_input: {taps} taps are outside 1..17")
        self.hidden_size, self.taps = int(hidden_size), int(taps)
        self.inner = build_part("mixer", inner["kind"], inner["params"])
        self.GRAPH_SAFE = self.inner.GRAPH_SAFE
        self.GRAPH_SAFE_PORTIONS = self.inner.GRAPH_SAFE_PORTIONS
        self.LAUNCHES = self.inner.LAUNCHES + (2 if self.taps > 1 else 1)
        self.ATOMIC_PREFILL = self.inner.ATOMIC_PREFILL
        self.weight = None

    def bind(self, shared):
        self.inner.bind(shared)

    def _own_spec(self):
        return StateSpec((("inputs", (self.taps - 1, self.hidden_size), torch.float32),)) if self.taps > 1 else None

    def cache_spec(self):
        inner = self.inner.cache_spec()
        inner = tuple(inner) if isinstance(inner, (tuple, list)) else (() if inner is None else (inner,))
        own = self._own_spec()
        return (() if own is None else (own,)) + inner

    def tensors(self):
        t = {"conv": TensorReq((self.hidden_size, self.taps), VECTOR)}
        t.update({f"inner.{name}": req for name, req in self.inner.tensors().items()})
        return t

    def load(self, tensors, dtype, device):
        self.weight = tensors["conv"].t().contiguous()   # [taps, channels]: a tap's weights side by side
        self.inner.load({name[len("inner."):]: t for name, t in tensors.items() if name.startswith("inner.")}, dtype, device)

    def forward(self, x, step, cache, write_cache=True):
        caches = list(cache) if isinstance(cache, tuple) else [cache]
        state = caches.pop(0).tensors["inputs"] if self.taps > 1 else None
        x = K.time_conv_add(x, self.weight, state, step)
        inner_spec = self.inner.cache_spec()
        if isinstance(inner_spec, (tuple, list)):
            inner_cache = tuple(caches)
        else:
            inner_cache = caches[0] if caches else None
        return self.inner.forward(x, step, inner_cache, write_cache)
