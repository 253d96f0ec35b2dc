"""Grouped-query attention over a paged cache, with optional per-head QK norm,
rotary encoding, biases and a window; optionally with the keys as projected for values and a sink in the softmax.

One merged projection [(nh + 2 nkv) hd, H] (crates/prelude-core/src/models/qwen3.rs:89-106,
crates/prelude-core/src/models/commons/attn_utils.rs:91-133; unlike the
reference's merged path, biases are kept), per-head RMSNorm of q and k with a
weight shared by all heads and RoPE straight after it
(qwen3.rs:59-62, :175-186), K and V written to the cache, causal softmax
attention with scale 1/sqrt(head_dim) (qwen3.rs:126, :191-206), output
projection (qwen3.rs:226-228).
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, VECTOR, KVCacheSpec, Mixer, PartError, TensorReq, register_part


@register_part("mixer", "gqa_attention")
class GQAAttention(Mixer):
    LAUNCHES = 4   # merged projection, norm + rotation + cache write, attention, output projection
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, norm_eps: float = 1e-6,
                 qk_norm: bool = True, bias: bool = False, window: int = 0, position: Optional[str] = None,
                 rotary_dim: Optional[int] = None, scale: Optional[float] = None, score_cap: float = 0.0,
                 values_from_keys: bool = False, sink: Optional[str] = None, head_scale: bool = False):
        if num_heads % num_kv_heads:
            raise PartError(f"gqa_attention: {num_heads} heads are not a multiple of {num_kv_heads} KV heads")
        # what the kernels take: the matrix-core attention has head sizes of its own (others go to the generic
        # kernel), the generic kernel and the norm + rotation kernel any size up to 256
        if not 1 <= head_dim <= 256:
            raise PartError(f"gqa_attention: head_dim {head_dim} is outside 1..256")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.norm_eps, self.qk_norm, self.bias, self.window = float(norm_eps), bool(qk_norm), bool(bias), int(window or 0)
        self.position = position
        self.rotary_dim = (head_dim if rotary_dim is None else int(rotary_dim)) if position else 0
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        # > 0: scaled scores are bent to cap * tanh(score / cap) before the softmax (the reference's Qwen3 has none,
        # qwen3.rs:204; a parameter for mixers of other models)
        self.score_cap = float(score_cap or 0.0)
        if self.score_cap < 0:
            raise PartError(f"gqa_attention: a score cap of {score_cap} is negative")
        # the values are the keys as projected (before norm and rotation): there is no value projection, and the
        # merged product has nh + nkv heads
        self.values_from_keys = bool(values_from_keys)
        # one more term of the softmax's denominator that brings no value: "zero" exp(0) = 1 for every head,
        # "learned" exp(s_h) with a tensor ``sinks`` [heads] (in the units of the scaled scores); None: none
        if sink not in (None, "zero", "learned"):
            raise PartError(f"gqa_attention: sink {sink!r} is not one of None, 'zero', 'learned'")
        self.sink = sink
        # a learned number per query head that its scores are multiplied by (a temperature), tensor ``head_scales``
        # [heads]: the rotated queries take it in 32-bit before they are rounded
        self.head_scale = bool(head_scale)
        if self.values_from_keys and self.bias:
            raise PartError("gqa_attention: values that are the keys come without biases")
        self.rope = None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.q_norm = self.k_norm = self.sinks = self.head_scales = None

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def bind(self, shared):
        if self.position is not None:
            if self.position not in shared:
                raise PartError(f"gqa_attention: the model has no position encoding named {self.position!r}")
            self.rope = shared[self.position]
            if (self.values_from_keys or self.head_scale) and not hasattr(self.rope, "inv_freq"):
                raise PartError("gqa_attention: values that are the keys, and a scale per head, take their rotation from "
                                "frequencies (a position encoding that offers `inv_freq`), not from tables")
            if getattr(self.rope, "rotary_dim", None) != self.rotary_dim:
                raise PartError(f"gqa_attention: position encoding {self.position!r} has width "
                                f"{getattr(self.rope, 'rotary_dim', None)}, the mixer rotates {self.rotary_dim}")

    def tensors(self):
        h, nh, nkv, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        t = {"q_proj.weight": TensorReq((nh * hd, h), MATRIX), "k_proj.weight": TensorReq((nkv * hd, h), MATRIX),
             "v_proj.weight": TensorReq((nkv * hd, h), MATRIX), "o_proj.weight": TensorReq((h, nh * hd), MATRIX)}
        if self.values_from_keys:
            del t["v_proj.weight"]
        if self.sink == "learned":
            t["sinks"] = TensorReq((nh,), VECTOR)
        if self.head_scale:
            t["head_scales"] = TensorReq((nh,), NORM)
        if self.bias:
            t.update({"q_proj.bias": TensorReq((nh * hd,), VECTOR), "k_proj.bias": TensorReq((nkv * hd,), VECTOR),
                      "v_proj.bias": TensorReq((nkv * hd,), VECTOR), "o_proj.bias": TensorReq((h,), VECTOR)})
        if self.qk_norm:
            t.update({"q_norm.weight": TensorReq((hd,), NORM), "k_norm.weight": TensorReq((hd,), NORM)})
        return t

    def load(self, tensors, dtype, device):
        merged = [tensors["q_proj.weight"], tensors["k_proj.weight"]]
        if not self.values_from_keys:
            merged.append(tensors["v_proj.weight"])
        self.w_qkv = K.prepare_weight(torch.cat(merged, dim=0).contiguous())
        if self.sink == "learned":
            self.sinks = tensors["sinks"]
        elif self.sink == "zero":
            self.sinks = torch.zeros(self.num_heads, dtype=torch.float32, device=device)
        self.w_o = K.prepare_weight(tensors["o_proj.weight"])
        if self.head_scale:
            self.head_scales = tensors["head_scales"]
        if self.bias:
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]]).contiguous()
            self.b_o = tensors["o_proj.bias"]
        if self.qk_norm:
            self.q_norm, self.k_norm = tensors["q_norm.weight"], tensors["k_norm.weight"]

    FUSED_DECODE_MAX_SEQS = 256   # measured: +3 % tokens a second at batch 1, +1 to 2 % at 8, 16, 32 and 64

    def _fused_decode(self, x, step, cache) -> bool:
        """Few sequences, each feeding one token: a kernel less per layer counts for more than the norm and the
        rotation that every workgroup of the attention kernel then does for itself."""
        return (x.dtype == torch.bfloat16 and self.rope is not None and step.decode_seqs is not None
                and getattr(self.rope, "cos", None) is not None and not self.values_from_keys and self.sinks is None
                and self.head_scales is None
                and step.n_prefill == 0 and step.n_decode == step.num_seqs <= self.FUSED_DECODE_MAX_SEQS
                and K.attention_decode_fused_supported(self.num_heads, self.num_kv_heads, self.head_dim,
                                                       self.rotary_dim, cache.k.shape[2]))

    def forward(self, x, step, cache, write_cache=True):
        nh, nkv, hd = self.num_heads, self.num_kv_heads, self.head_dim
        g = step.kv[cache.group]
        # tables by position, or the frequencies alone (the kernel then takes angle, cosine and sine itself)
        cos = getattr(self.rope, "cos", None) if self.rope is not None else None
        sin = getattr(self.rope, "sin", None) if self.rope is not None else None
        freq = getattr(self.rope, "inv_freq", None) if self.rope is not None and cos is None else None
        how = dict(inv_freq=freq, values_from_keys=self.values_from_keys) if (freq is not None or self.values_from_keys) else {}
        if self.head_scales is not None:
            how["q_scale"] = self.head_scales
        if write_cache and self._fused_decode(x, step, cache):
            # a step of single tokens: the norm, the rotation and the cache write happen inside the attention kernel
            qkv = K.linear(x, self.w_qkv, self.b_qkv)
            o = K.attention_decode_fused(qkv, self.q_norm, self.k_norm, cos, sin, g.slots, self.norm_eps,
                                         cache.k, cache.v, g.block_table, step.decode_seqs, step.cu_q, step.context_lens,
                                         nh, step.max_decode_context, self.window, self.scale, every_seq=True,
                                         softcap=self.score_cap)
            return K.linear(o.view(o.shape[0], nh * hd), self.w_o, self.b_o, slices_ok=True)
        if write_cache:
            qkv = K.linear(x, self.w_qkv, self.b_qkv)
            q = K.qknorm_rope_kv(qkv, self.q_norm, self.k_norm, cos, sin, step.positions, g.slots, cache.k, cache.v,
                                 nh, nkv, hd, self.rotary_dim, self.norm_eps, **how)
        else:  # reads keys and values another layer wrote: only the queries are projected
            bq = self.b_qkv[: nh * hd] if self.b_qkv is not None else None
            qx = K.linear(x, self.w_qkv.first_rows(nh * hd), bq)
            only_q = {"inv_freq": freq} if freq is not None else {}
            if self.head_scales is not None:
                only_q["q_scale"] = self.head_scales
            q = K.qknorm_rope_kv(qx, self.q_norm, None, cos, sin, step.positions, None, None, None, nh, 0, hd,
                                 self.rotary_dim, self.norm_eps, **only_q)
        o = K.attention(q, cache.k, cache.v, g, step, self.window, self.scale, self.score_cap, sink=self.sinks)
        return K.linear(o.view(o.shape[0], nh * hd), self.w_o, self.b_o, slices_ok=True)


@dataclasses.dataclass(frozen=True)
class KeptFirstKVCacheSpec(KVCacheSpec):
    """Keys and values in pages under a window that keeps the first tokens: pages that hold one of the first
    ``keep_first`` positions are never given back while the request lives."""
    keep_first: int = 0


@register_part("mixer", "windowed_attention")
class WindowedAttention(Mixer):
    """Grouped-query attention without rotation whose mask is a window that keeps the first tokens: the query at i
    sees the key at j <= i when i - j < ``window`` (0: no window) or j < ``keep_first``.  Values have a width of their
    own.  Optional, each a parameter: queries and keys brought to unit RMS over the whole projection (all heads at once)
    times a weight of that size (``qk_norm="whole"``); scores bent to cap * tanh(score / cap) (``score_cap``); a bias by
    distance, slope_h (i - j) taken off the score with slope_h = 2^(-``slope_exponent`` (h + 1) / heads)
    (``slope_exponent`` > 0); a learned sink per head in the softmax's denominator (``sink="learned"``); a gate per
    head, the head's output times sigmoid(W_g x)_h (``head_gate``).

    ``cache_window`` / ``cache_keep_first``: the mask the cache is kept for, where it is wider than this layer's own
    because other layers read the same keys (``window`` 0 = everything)."""
    LAUNCHES = 4   # merged projection, norm + cache write, attention, output projection
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 window: int = 0, keep_first: int = 0, qk_norm: Optional[str] = None, norm_eps: float = 1e-6,
                 score_cap: float = 0.0, slope_exponent: float = 0.0, sink: Optional[str] = None, head_gate: bool = False,
                 own_keys: bool = True, cache_window: Optional[int] = None, cache_keep_first: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise PartError(f"windowed_attention: {num_heads} heads are not a multiple of {num_kv_heads} KV heads")
        if not (1 <= head_dim <= 256 and 1 <= value_dim <= 256):
            raise PartError(f"windowed_attention: key width {head_dim} or value width {value_dim} is outside 1..256")
        if qk_norm not in (None, "whole"):
            raise PartError(f"windowed_attention: qk_norm {qk_norm!r} is not one of None, 'whole'")
        if sink not in (None, "learned"):
            raise PartError(f"windowed_attention: sink {sink!r} is not one of None, 'learned'")
        if window < 0 or keep_first < 0 or score_cap < 0 or slope_exponent < 0:
            raise PartError("windowed_attention: window, kept first tokens, score cap and slope exponent must not be negative")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.scale = int(head_dim), int(value_dim), float(scale)
        self.window, self.keep_first = int(window), int(keep_first) if window else 0
        self.qk_norm, self.norm_eps, self.score_cap = qk_norm, float(norm_eps), float(score_cap)
        self.slope_exponent, self.sink, self.head_gate = float(slope_exponent), sink, bool(head_gate)
        # False: this layer has no key and value projections and reads the keys and values another layer cached
        self.own_keys = bool(own_keys)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.cache_keep_first = self.keep_first if cache_keep_first is None else int(cache_keep_first)
        if self.cache_window and (not self.window or self.cache_window < self.window or
                                  self.cache_keep_first < self.keep_first):
            raise PartError("windowed_attention: the cache's mask must hold everything this layer's mask sees")
        self.w_in = self.w_o = self.q_norm = self.k_norm = self.sinks = self.slopes = None

    # ---- sizes of its columns in the projection of its input ----
    @property
    def nq(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def nk(self) -> int:
        return self.num_kv_heads * self.head_dim if self.own_keys else 0

    @property
    def nv(self) -> int:
        return self.num_kv_heads * self.value_dim if self.own_keys else 0

    @property
    def mixed_size(self) -> int:
        """Width of what ``mix`` leaves for the output projection."""
        return self.num_heads * self.value_dim

    def cache_spec(self):
        if self.cache_window and self.cache_keep_first:
            return KeptFirstKVCacheSpec(self.num_kv_heads, self.head_dim, self.cache_window, self.value_dim, self.cache_keep_first)
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.cache_window, self.value_dim)

    def tensors(self):
        h = self.hidden_size
        t = {"q": TensorReq((self.nq, h), MATRIX), "o": TensorReq((h, self.mixed_size), MATRIX)}
        if self.own_keys:
            t.update({"k": TensorReq((self.nk, h), MATRIX), "v": TensorReq((self.nv, h), MATRIX)})
        if self.qk_norm:
            t["q.norm"] = TensorReq((self.nq,), NORM)
            if self.own_keys:
                t["k.norm"] = TensorReq((self.nk,), NORM)
        if self.sink:
            t["sink"] = TensorReq((self.num_heads,), VECTOR)
        if self.head_gate:
            t["g"] = TensorReq((self.num_heads, h), MATRIX)
        return t

    def input_rows(self, tensors) -> torch.Tensor:
        """The rows of the product of its input this mixer wants, [q | k | v | gate]; keeps its other tensors."""
        rows = [tensors["q"]] + ([tensors["k"], tensors["v"]] if self.own_keys else []) + ([tensors["g"]] if self.head_gate else [])
        if self.qk_norm:
            self.q_norm = tensors["q.norm"]
            self.k_norm = tensors["k.norm"] if self.own_keys else None
        self.sinks = tensors["sink"] if self.sink else None
        if self.slope_exponent:
            nh = self.num_heads
            self.slopes = torch.tensor([2.0 ** (-self.slope_exponent * (i + 1) / nh) for i in range(nh)], dtype=torch.float64) \
                .to(torch.float32).to(tensors["q"].device)
        return torch.cat(rows, dim=0) if len(rows) > 1 else rows[0]

    def load(self, tensors, dtype, device):
        self.w_in = K.prepare_weight(self.input_rows(tensors).contiguous())
        self.w_o = K.prepare_weight(tensors["o"])

    def mix(self, x, p, off, step, cache, write_cache, out=None, out_scale=1.0):
        """From the product ``p`` of its input ``x`` (its columns start at ``off``) to the heads' outputs side by side
        [T, heads * value_dim], times ``out_scale``, into ``out`` when given."""
        if write_cache != self.own_keys:
            raise PartError("windowed_attention: a layer with key and value projections writes its own cache, one without "
                            "reads another's")
        nh, nkv, hd, vd = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        g = step.kv[cache.group]
        q = K.qkv_prepare(p, off, off + self.nq, off + self.nq + self.nk, self.q_norm, self.k_norm,
                          g.slots if write_cache else None, cache.k, cache.v, nh, nkv, hd, vd, self.norm_eps)
        gate = p[:, off + self.nq + self.nk + self.nv: off + self.nq + self.nk + self.nv + nh] if self.head_gate else None
        if not self.keep_first and self.slopes is None and gate is None and vd == hd and out is None and out_scale == 1.0:
            o = K.attention(q, cache.k, cache.v, g, step, self.window, self.scale, self.score_cap, sink=self.sinks)
            return o.view(o.shape[0], nh * vd)
        return K.attention_masked(q, cache.k, cache.v, g, step, self.window, self.keep_first, self.scale, self.score_cap,
                                  self.slopes, self.sinks, gate, out, out_scale)

    def forward(self, x, step, cache, write_cache=True):
        p = K.linear(x, self.w_in)
        return K.linear(self.mix(x, p, 0, step, cache, write_cache), self.w_o, slices_ok=True)


@dataclasses.dataclass(frozen=True)
class SharedValueKVCacheSpec(KVCacheSpec):
    """Keys and values in pages where several key heads read one value head: ``num_kv_heads`` key heads of ``head_dim``
    and ``num_value_heads`` value heads of ``value_dim`` (key head k goes with value head k mod ``num_value_heads``).
    K ``[pages, key heads, page, head_dim]``, V ``[pages, value heads, value width, page]``."""
    num_value_heads: int = 0

    def bytes_per_token(self, element_size: int) -> int:
        return (self.num_kv_heads * self.head_dim + self.num_value_heads * self.v_dim) * element_size

    def allocate(self, pages, page_size, dtype, device, group):
        from .base import KVLayerCache
        return KVLayerCache(torch.zeros((pages, self.num_kv_heads, page_size, self.head_dim), dtype=dtype, device=device),
                            torch.zeros((pages, self.num_value_heads, self.v_dim, page_size), dtype=dtype, device=device), group)


@register_part("mixer", "differential_attention")
class DifferentialAttention(Mixer):
    """Two attention maps a head over the same values, one taken off the other.  The query projection has
    heads * 2 * head_dim rows and the key projection kv_heads * 2 * head_dim, laid out head by head as [map 1 | map 2];
    the value projection kv_heads * value_dim.  The first ``rotary_dim`` dimensions of every map of every query and key
    head are turned by position, dimension 2i with 2i + 1.  Each map is a softmax attention of its own under the window
    (score = q.k * scale); with a1, a2 their outputs and lambda = exp(lq1.lk1) - exp(lq2.lk2) + ``diff`` (one number a
    layer, from four learned vectors of head_dim), a head's output is u = a1 - lambda a2 over its own
    sqrt(mean(u^2) + eps), times 1 - ``diff``.

    The maps run as 2 * heads query heads over 2 * kv_heads key heads (the projections' rows put map-major when they are
    loaded) whose value head is the key head modulo kv_heads: the values are cached once."""
    LAUNCHES = 5   # merged projection, rotation + cache write, attention, the maps' difference and norm, output projection
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 diff: float, norm_eps: float, window: int = 0, position: Optional[str] = None, rotary_dim: int = 0):
        if num_heads % num_kv_heads:
            raise PartError(f"differential_attention: {num_heads} heads are not a multiple of {num_kv_heads} KV heads")
        if not (1 <= head_dim <= 256 and 1 <= value_dim <= 256):
            raise PartError(f"differential_attention: key width {head_dim} or value width {value_dim} is outside 1..256")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.scale, self.diff = int(head_dim), int(value_dim), float(scale), float(diff)
        self.norm_eps, self.window = float(norm_eps), int(window or 0)
        self.position = position
        self.rotary_dim = int(rotary_dim or 0) if position else 0
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise PartError(f"differential_attention: {self.rotary_dim} rotated dimensions of a map of {self.head_dim}")
        self.rope = None
        self.w_in = self.w_o = None
        self.lam = 0.0

    def cache_spec(self):
        return SharedValueKVCacheSpec(2 * self.num_kv_heads, self.head_dim, self.window, self.value_dim, self.num_kv_heads)

    def bind(self, shared):
        if self.position is not None:
            if self.position not in shared:
                raise PartError(f"differential_attention: the model has no position encoding named {self.position!r}")
            self.rope = shared[self.position]
            if getattr(self.rope, "rotary_dim", None) != self.rotary_dim or not hasattr(self.rope, "inv_freq"):
                raise PartError(f"differential_attention: position encoding {self.position!r} must give the frequencies of "
                                f"{self.rotary_dim} rotated dimensions")

    def tensors(self):
        h, nh, nkv, d, v = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        t = {"q": TensorReq((nh * 2 * d, h), MATRIX), "k": TensorReq((nkv * 2 * d, h), MATRIX),
             "v": TensorReq((nkv * v, h), MATRIX), "o": TensorReq((h, nh * v), MATRIX)}
        t.update({n: TensorReq((d,), VECTOR) for n in ("lq1", "lk1", "lq2", "lk2")})
        return t

    @staticmethod
    def _map_major(w, heads: int, d: int):
        """Rows [head][map][d] -> [map][head][d]."""
        return w.reshape(heads, 2, d, w.shape[1]).transpose(0, 1).reshape(heads * 2 * d, w.shape[1])

    def load(self, tensors, dtype, device):
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        rows = [self._map_major(tensors["q"], nh, d), self._map_major(tensors["k"], nkv, d), tensors["v"]]
        self.w_in = K.prepare_weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = K.prepare_weight(tensors["o"])
        dot = lambda a, b: float((tensors[a].double() * tensors[b].double()).sum().item())
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff

    def forward(self, x, step, cache, write_cache=True):
        if not write_cache:
            raise PartError("differential_attention: reads no other layer's cache")
        nh, nkv, d, v = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        g = step.kv[cache.group]
        p = K.linear(x, self.w_in)
        freq = self.rope.inv_freq if self.rope is not None else None
        nq, nk = 2 * nh * d, 2 * nkv * d
        q = K.qkv_rope_prepare(p, 0, nq, nq + nk, freq, step.positions, g.slots, cache.k, cache.v, 2 * nh, 2 * nkv, nkv, d, v,
                               self.rotary_dim, pairs=True)
        a = K.attention_masked(q, cache.k, cache.v, g, step, self.window, 0, self.scale)
        o = K.diff_combine(a, nh, self.lam, self.norm_eps, 1.0 - self.diff)
        return K.linear(o, self.w_o, slices_ok=True)
