"""Arrangements of parts into one layer.

``prenorm``: norm -> mixer -> (+residual) norm -> feed-forward, with the
residual carried beside the hidden state and each add deferred into the next
norm (crates/prelude-core/src/models/qwen3.rs:486-502,
crates/prelude-core/src/models/commons/linear.rs:471-488).

``branch_norm``: the norm sits on each branch's output, x <- x + norm(mixer(x)) and x <- x + norm(ffn(x)); the
branches read the stream itself.  The stream is 32-bit; beside it travels its copy in the engine's type, which is
what the branches multiply with.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import Block, PartError, register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    SLOTS = {"input_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm", "ffn": "ffn"}

    def __init__(self, input_norm, mixer, post_mixer_norm, ffn):
        self.input_norm, self.mixer, self.post_mixer_norm, self.ffn = input_norm, mixer, post_mixer_norm, ffn

    def forward(self, hidden, residual, step, cache, write_cache=True):
        # a mixer's or feed-forward's last product may come as partial sums of slices (``K.SliceSums``): a norm
        # that can adds them as it loads them, any other gets the finished tensor
        if not self.input_norm.TAKES_SLICE_SUMS:
            hidden = K.as_tensor(hidden)
        residual, h = self.input_norm.forward_residual(hidden, residual)
        h = self.mixer.forward(h, step, cache, write_cache)
        if getattr(self.ffn, "NEEDS_STEP", False):
            residual, h = self.ffn.forward_after_norm(h, residual, self.post_mixer_norm, step=step)
        else:
            residual, h = self.ffn.forward_after_norm(h, residual, self.post_mixer_norm)
        return h, residual


@register_part("block", "prenorm_mixer_only")
class PreNormMixerBlock(Block):
    """A layer without a feed-forward: norm -> mixer, the add deferred into the next norm as in ``prenorm``."""
    GRAPH_SAFE_PORTIONS = True

    SLOTS = {"input_norm": "norm", "mixer": "mixer"}

    def __init__(self, input_norm, mixer):
        self.input_norm, self.mixer = input_norm, mixer

    def forward(self, hidden, residual, step, cache, write_cache=True):
        if not self.input_norm.TAKES_SLICE_SUMS:
            hidden = K.as_tensor(hidden)
        residual, h = self.input_norm.forward_residual(hidden, residual)
        return self.mixer.forward(h, step, cache, write_cache), residual


@register_part("block", "branch_norm")
class BranchNormBlock(Block):
    """x <- x + mixer_norm(mixer(x)); x <- x + ffn_norm(ffn(x)).  Both branches read x itself, the norms sit on their
    outputs, and the sums are taken and kept in 32-bit.  ``hidden`` carried between such blocks is x in the engine's
    type (the residual itself in a 32-bit engine), written by the kernel that norms and adds."""
    GRAPH_SAFE_PORTIONS = True
    HANDS_ON_STREAM = True

    SLOTS = {"mixer": "mixer", "mixer_norm": "norm", "ffn": "ffn", "ffn_norm": "norm"}

    def __init__(self, mixer, mixer_norm, ffn, ffn_norm):
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = mixer, mixer_norm, ffn, ffn_norm

    @staticmethod
    def _enter(hidden, residual):
        if residual is None:   # the first block: the stream starts as a 32-bit copy of the embedding
            hidden = K.as_tensor(hidden)
            residual = hidden if hidden.dtype == torch.float32 else K.to_f32(hidden)
        return hidden, residual

    @staticmethod
    def _add(norm, y, hidden, residual):
        if not norm.TAKES_SLICE_SUMS:
            y = K.as_tensor(y)
        copy = norm.forward_branch(y, residual, hidden.dtype)
        return residual if copy is None else copy

    def forward(self, hidden, residual, step, cache, write_cache=True):
        hidden, residual = self._enter(hidden, residual)
        hidden = self._add(self.mixer_norm, self.mixer.forward(hidden, step, cache, write_cache), hidden, residual)
        y = self.ffn.forward(hidden, step=step) if getattr(self.ffn, "NEEDS_STEP", False) else self.ffn.forward(hidden)
        return self._add(self.ffn_norm, y, hidden, residual), residual


@register_part("block", "branch_norm_mixer_only")
class BranchNormMixerBlock(Block):
    """A ``branch_norm`` layer without a feed-forward: x <- x + mixer_norm(mixer(x))."""
    GRAPH_SAFE_PORTIONS = True
    HANDS_ON_STREAM = True

    SLOTS = {"mixer": "mixer", "mixer_norm": "norm"}

    def __init__(self, mixer, mixer_norm):
        self.mixer, self.mixer_norm = mixer, mixer_norm

    def forward(self, hidden, residual, step, cache, write_cache=True):
        hidden, residual = BranchNormBlock._enter(hidden, residual)
        y = self.mixer.forward(hidden, step, cache, write_cache)
        return BranchNormBlock._add(self.mixer_norm, y, hidden, residual), residual


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """A norm in front of and behind every branch: x <- x + post_mixer_norm(mixer(pre_mixer_norm(x))), then
    x <- x + post_ffn_norm(ffn(pre_ffn_norm(x))).  The stream x is 32-bit and is all that travels between such blocks
    (``hidden`` is handed on as None); the add behind the mixer and the norm in front of the feed-forward are one
    launch where the norms can."""
    GRAPH_SAFE_PORTIONS = True
    HANDS_ON_STREAM = True

    SLOTS = {"pre_mixer_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm", "pre_ffn_norm": "norm", "ffn": "ffn",
             "post_ffn_norm": "norm"}

    def __init__(self, pre_mixer_norm, mixer, post_mixer_norm, pre_ffn_norm, ffn, post_ffn_norm):
        self.pre_mixer_norm, self.mixer, self.post_mixer_norm = pre_mixer_norm, mixer, post_mixer_norm
        self.pre_ffn_norm, self.ffn, self.post_ffn_norm = pre_ffn_norm, ffn, post_ffn_norm

    @staticmethod
    def _enter(hidden, residual, step):
        """(the stream, the engine's element type: ``step.compute_dtype``).  The first block turns the embedding into
        the stream."""
        if residual is None:
            hidden = K.as_tensor(hidden)
            return (hidden if hidden.dtype == torch.float32 else K.to_f32(hidden)), hidden.dtype
        if residual.dtype != torch.float32:
            raise PartError("sandwich_norm: the stream between such blocks is 32-bit")
        if hidden is None and step.compute_dtype is None:
            raise PartError("sandwich_norm: the step does not say the engine's element type")
        return residual, (hidden.dtype if hidden is not None else step.compute_dtype)

    def forward(self, hidden, residual, step, cache, write_cache=True):
        residual, dtype = self._enter(hidden, residual, step)
        h = self.pre_mixer_norm.forward_stream(residual, dtype)
        y = self.mixer.forward(h, step, cache, write_cache)
        h = self.post_mixer_norm.forward_branch_then(y, residual, self.pre_ffn_norm, dtype)
        y = self.ffn.forward(h, step=step) if getattr(self.ffn, "NEEDS_STEP", False) else self.ffn.forward(h)
        self.post_ffn_norm.forward_branch_then(y, residual, None, dtype)
        return None, residual


@register_part("block", "sandwich_norm_mixer_only")
class SandwichNormMixerBlock(Block):
    """A ``sandwich_norm`` layer without a feed-forward: x <- x + post_mixer_norm(mixer(pre_mixer_norm(x)))."""
    GRAPH_SAFE_PORTIONS = True
    HANDS_ON_STREAM = True

    SLOTS = {"pre_mixer_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm"}

    def __init__(self, pre_mixer_norm, mixer, post_mixer_norm):
        self.pre_mixer_norm, self.mixer, self.post_mixer_norm = pre_mixer_norm, mixer, post_mixer_norm

    def forward(self, hidden, residual, step, cache, write_cache=True):
        residual, dtype = SandwichNormBlock._enter(hidden, residual, step)
        h = self.pre_mixer_norm.forward_stream(residual, dtype)
        y = self.mixer.forward(h, step, cache, write_cache)
        self.post_mixer_norm.forward_branch_then(y, residual, None, dtype)
        return None, residual


@register_part("block", "parallel_branches")
class ParallelBranchesBlock(Block):
    """One norm, both branches on its output: h = norm(x), x <- x + (mixer(h) + ffn(h)).  The stream x is 32-bit and is
    all that travels between such blocks (``hidden`` is handed on as None); the branches' outputs are added to each
    other and then to the stream in 32-bit, in one launch."""
    GRAPH_SAFE_PORTIONS = True
    HANDS_ON_STREAM = True

    SLOTS = {"norm": "norm", "mixer": "mixer", "ffn": "ffn"}

    def __init__(self, norm, mixer, ffn=None):
        self.norm, self.mixer, self.ffn = norm, mixer, ffn

    @staticmethod
    def _enter(hidden, residual, step):
        """(the stream, the engine's element type).  The first block turns the embedding into the stream (an embedding
        that comes in 32-bit already is the stream)."""
        if step.compute_dtype is None:
            raise PartError("parallel_branches: the step does not say the engine's element type")
        if residual is None:
            hidden = K.as_tensor(hidden)
            return (hidden if hidden.dtype == torch.float32 else K.to_f32(hidden)), step.compute_dtype
        if residual.dtype != torch.float32 or hidden is not None:
            raise PartError("parallel_branches: only a 32-bit stream travels between such blocks")
        return residual, step.compute_dtype

    def forward(self, hidden, residual, step, cache, write_cache=True):
        residual, dtype = self._enter(hidden, residual, step)
        h = self.norm.forward_stream(residual, dtype)
        a = K.as_tensor(self.mixer.forward(h, step, cache, write_cache))
        if self.ffn is None:
            K.stream_add_branches_(residual, a)
        else:   # the feed-forward's last kernel takes the mixer's output along into the stream where it can
            self.ffn.forward_into_stream(h, residual, a, step=step)
        return None, residual


@register_part("block", "parallel_branches_mixer_only")
class ParallelBranchesMixerBlock(ParallelBranchesBlock):
    """A ``parallel_branches`` layer without a feed-forward: x <- x + mixer(norm(x))."""
    SLOTS = {"norm": "norm", "mixer": "mixer"}

    def __init__(self, norm, mixer):
        super().__init__(norm, mixer, None)
