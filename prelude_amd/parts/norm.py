"""RMSNorm, alone, fused with the residual add in front of it, or on a branch's output with the add behind it.

y = x * rsqrt(mean(x^2) + eps) * w in 32-bit
(crates/prelude-core/src/models/commons/linear.rs:435-501); with a residual:
sum in 32-bit, the residual keeps the rounded sum, the norm is taken of the
unrounded one (crates/prelude-cuda/src/kernels/kernels_src/normalization/rmsnorm.cu:258-274).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import NORM, VECTOR, Norm, PartError, TensorReq, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    TAKES_SLICE_SUMS = True

    def __init__(self, size: int, eps: float, weight_offset: float = 0.0, residual_float32: bool = False):
        """``weight_offset``: the stored weight lies around zero and the gain is ``offset + weight`` (added once,
        in 32-bit, when the weight is loaded).  ``residual_float32``: the residual stream this norm adds to is
        kept in 32-bit whatever the engine's element type; the normed output is of the engine's type."""
        self.size = int(size)
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.residual_float32 = bool(residual_float32)
        self.weight: Optional[torch.Tensor] = None

    def tensors(self):
        # a weight stored around zero is drawn around zero in the random-weights mode too
        return {"weight": TensorReq((self.size,), VECTOR if self.weight_offset else NORM)}

    def load(self, tensors, dtype, device):
        w = tensors["weight"]
        self.weight = (w + self.weight_offset).contiguous() if self.weight_offset else w

    def as_rms(self):
        return self.weight, self.eps

    def forward(self, x):
        return K.rmsnorm(x, self.weight, self.eps)

    def forward_residual(self, x, residual):
        """First use in a model: residual None -> (x, norm(x)).  Afterwards the
        residual is updated in place with residual + x."""
        if residual is None:
            x = K.as_tensor(x)
            if self.residual_float32:
                # the stream starts as a 32-bit copy of x (x itself when the engine's type is 32-bit already)
                return K.to_f32(x), K.rmsnorm(x, self.weight, self.eps)
            return x, K.rmsnorm(x, self.weight, self.eps)
        if self.residual_float32:
            if residual.dtype != torch.float32:
                raise PartError("rms_norm: a norm with a 32-bit residual was handed one of another type")
            return residual, K.rmsnorm_wide(x, self.weight, self.eps, residual=residual)
        out = K.rmsnorm(x, self.weight, self.eps, residual=residual)
        return residual, out

    def forward_rows(self, x, residual, rows, out_dtype=None):
        if x is None:
            # nothing waits to be added to the stream: the norm of its wanted rows alone
            if residual is None or residual.dtype != torch.float32:
                raise PartError("rms_norm: the norm of the stream's rows alone needs a 32-bit stream")
            return K.rmsnorm_wide(None, self.weight, self.eps, residual=residual, rows=rows, out_dtype=out_dtype)
        if self.residual_float32 and residual is not None:
            return K.rmsnorm_wide(x, self.weight, self.eps, residual=residual, rows=rows)
        return K.rmsnorm(x, self.weight, self.eps, residual=residual, rows=rows)

    def forward_branch(self, y, residual, copy_dtype=None):
        """residual += norm(y), in 32-bit and in place: for a layer whose norm sits on the branch's output.  Returns
        the new residual rounded to ``copy_dtype`` (None when that is 32-bit: the residual itself serves)."""
        if residual.dtype != torch.float32:
            raise PartError("rms_norm: a branch is normed and added to a 32-bit stream only")
        return K.rmsnorm_branch(y, self.weight, self.eps, residual, copy_dtype)


@register_part("norm", "group_rms_norm")
class GroupRMSNorm(Norm):
    """RMS norm in groups around a 32-bit stream: the row is split into ``groups`` equal consecutive parts, each is
    divided by its own sqrt(mean(part^2) + eps), and the whole is multiplied by the weight.  One group is the plain
    RMS norm.  It norms the stream for a branch (``forward_stream``), norms a branch's output and adds it to the
    stream (``forward_branch``), or both in one launch (``forward_branch_then``: the add, then the next branch's
    input through another norm of this kind)."""
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, size: int, eps: float, groups: int = 1, scalar_weight: bool = False):
        """``scalar_weight``: the stored weight is a single number for all coordinates (a tensor without axes)."""
        self.size, self.eps, self.groups = int(size), float(eps), int(groups)
        if self.groups < 1 or self.size % self.groups:
            raise PartError(f"group_rms_norm: {groups} groups do not divide a row of {size}")
        self.scalar_weight = bool(scalar_weight)
        self.weight: Optional[torch.Tensor] = None

    def tensors(self):
        return {"weight": TensorReq(() if self.scalar_weight else (self.size,), NORM)}

    def load(self, tensors, dtype, device):
        w = tensors["weight"]
        # one number: spread over the row once, so that the kernels read a weight per coordinate as for any other norm
        self.weight = w.reshape(1).expand(self.size).contiguous() if self.scalar_weight else w

    def as_rms(self):
        return (self.weight, self.eps) if self.groups == 1 else None

    @staticmethod
    def _stream(residual):
        if residual is None or residual.dtype != torch.float32:
            raise PartError("group_rms_norm: works around a 32-bit stream")
        return residual

    def forward_stream(self, residual, out_dtype):
        return K.group_norm_step(self._stream(residual), self.groups, self.eps, w_out=self.weight, out_dtype=out_dtype)

    def forward_rows(self, x, residual, rows, out_dtype=None):
        if x is not None:
            raise PartError("group_rms_norm: nothing waits to be added to the stream when its rows are normed")
        return K.group_norm_step(self._stream(residual), self.groups, self.eps, w_out=self.weight,
                                 out_dtype=out_dtype or torch.float32, rows=rows)

    def forward_branch(self, y, residual, copy_dtype=None):
        if copy_dtype not in (None, torch.float32):
            raise PartError("group_rms_norm: the stream has no rounded copy; ask `forward_branch_then` for the next branch's input")
        K.group_norm_step(self._stream(residual), self.groups, self.eps, y=K.as_tensor(y), w_add=self.weight)
        return None

    def forward_branch_then(self, y, residual, then, out_dtype):
        if isinstance(then, GroupRMSNorm) and then.groups == self.groups and then.eps == self.eps:
            return K.group_norm_step(self._stream(residual), self.groups, self.eps, y=K.as_tensor(y), w_add=self.weight,
                                     w_out=then.weight, out_dtype=out_dtype)
        return super().forward_branch_then(y, residual, then, out_dtype)
