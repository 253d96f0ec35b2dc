"""A decoder assembled from a ``ModelSpec``: embedding, the layers in their run
order, final norm on the wanted rows, output head.

Counterpart of the reference's hand-written model
(crates/prelude-core/src/models/qwen3.rs:534-660: embed, layers carrying
(hidden, residual), final norm of hidden + residual, last-token select, head),
except that the structure is read from data and the head runs only on the rows
whose logits are wanted.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Tuple

import torch

from ..parts import Block, Part, TensorReq, build_part
from ..parts.base import VECTOR, PartError, _REGISTRY
from .spec import ModelSpec, PartSpec


@dataclasses.dataclass
class CacheSlot:
    """What one run of a layer keeps between steps."""
    run: int                    # index in the run order that owns (writes) it
    spec: object                # a PagedCacheSpec (keys and values, or a kind of the mixer's own) | a SlotCacheSpec


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.dtype: Optional[torch.dtype] = None
        self.device: Optional[torch.device] = None
        # (part, its spec) in a fixed order, for tensor requests and loading
        self._parts: List[Tuple[Part, PartSpec]] = []
        self.shared: Dict[str, Part] = {}
        for name, ps in spec.positions.items():
            p = build_part("position", ps.kind, ps.params)
            self.shared[name] = p
            self._parts.append((p, ps))
        self.embedding = self._make("embedding", spec.embedding)
        self.blocks: List[Block] = []
        for ls in spec.layers:
            cls = _REGISTRY.get(("block", ls.block))
            if cls is None:
                raise PartError(f"no block of kind {ls.block!r} is registered")
            subs = {}
            for slot, category in cls.SLOTS.items():
                if slot not in ls.parts:
                    raise PartError(f"block {ls.block!r} needs a part for its slot {slot!r}")
                subs[slot] = self._make(category, ls.parts[slot])
            extra = set(ls.parts) - set(cls.SLOTS)
            if extra:
                raise PartError(f"block {ls.block!r} has no slots {sorted(extra)}")
            self.blocks.append(build_part("block", ls.block, ls.block_params, **subs))
        self.final_norm = self._make("norm", spec.final_norm)
        self.head = self._make("head", spec.head)
        for p, _ in self._parts:
            p.bind(self.shared)

        # caches: one per run that does not read another's; a mixer made of several (``cache_spec()`` a tuple) has one
        # per member that keeps something, and gets them as a tuple in that order
        self.cache_slots: List[Optional[CacheSlot]] = []
        self.run_cache: List[object] = []   # run index -> None | index into cache_slots | tuple of indices
        # an embedding that keeps something per request (the token before, say) has a cache slot of its own, owned by no run
        self.embedding_cache: Optional[int] = None
        ecs = self.embedding.cache_spec() if hasattr(self.embedding, "cache_spec") else None
        if ecs is not None:
            self.embedding_cache = len(self.cache_slots)
            self.cache_slots.append(CacheSlot(-1, ecs))
        self.stream_rows: Optional[torch.Tensor] = None
        for i, r in enumerate(spec.order):
            mixer = getattr(self.blocks[r.layer], "mixer", None)
            cs = mixer.cache_spec() if mixer is not None else None
            several = isinstance(cs, (tuple, list))
            wanted = list(cs) if several else ([cs] if cs is not None else [])
            if r.reads_cache_of is not None:
                src = self.run_cache[r.reads_cache_of]
                have = [] if src is None else [self.cache_slots[j].spec for j in (src if isinstance(src, tuple) else (src,))]
                if not have or have != wanted:
                    raise PartError(f"run {i} cannot read the cache of run {r.reads_cache_of}: "
                                    f"it keeps {have or None}, this layer needs {wanted or None}")
                self.run_cache.append(src)
            elif not wanted:
                self.run_cache.append(None)
            else:
                first = len(self.cache_slots)
                self.cache_slots.extend(CacheSlot(i, w) for w in wanted)
                self.run_cache.append(tuple(range(first, first + len(wanted))) if several else first)

    def _make(self, category: str, ps: PartSpec) -> Part:
        p = build_part(category, ps.kind, ps.params)
        self._parts.append((p, ps))
        return p

    # ---- tensors ---------------------------------------------------------
    def tensor_requests(self) -> Dict[str, TensorReq]:
        """Checkpoint tensor name -> what is required of it, over all parts."""
        out: Dict[str, TensorReq] = {}
        for part, ps in self._parts:
            for local, req in part.tensors().items():
                if local not in ps.weights:
                    raise PartError(f"{ps.kind}: no checkpoint name given for its tensor {local!r}")
                name = ps.weights[local]
                if name in out and out[name] != req:
                    raise PartError(f"tensor {name!r} is asked for as {out[name]} and as {req}")
                out[name] = req
        if self.spec.stream_rows is not None:
            name, rows = self.spec.stream_rows
            out[name] = TensorReq((int(rows), self.spec.hidden_size), VECTOR)
        return out

    def load(self, fetch, dtype: torch.dtype, device: torch.device) -> None:
        """``fetch(checkpoint_name, req)`` returns the tensor on the device in the type its kind asks for."""
        self.dtype, self.device = dtype, device
        for part, ps in self._parts:
            tensors = {local: fetch(ps.weights[local], req) for local, req in part.tensors().items()}
            part.load(tensors, dtype, device)
        if self.spec.stream_rows is not None:
            name, rows = self.spec.stream_rows
            self.stream_rows = fetch(name, TensorReq((int(rows), self.spec.hidden_size), VECTOR)).contiguous()
        for p in self.shared.values():
            p.prepare(device)

    def matrix_elements(self) -> int:
        """Elements of the weight matrices a step multiplies with (the embedding table is only looked up in)."""
        from ..parts.base import MATRIX
        seen, total = set(), 0
        for part, ps in self._parts:
            if part is self.embedding:
                continue
            for local, req in part.tensors().items():
                if req.kind == MATRIX and ps.weights[local] not in seen:
                    seen.add(ps.weights[local])
                    n = 1
                    for d in req.shape:
                        n *= max(int(d), 1)
                    total += n
        return total

    def launches_per_step(self) -> int:
        """Kernel launches of one step, about: every run's block by its parts' own counts, and the embedding, the
        final norm and the head."""
        total = self.embedding.LAUNCHES + self.final_norm.LAUNCHES + self.head.LAUNCHES
        total += sum(1 for r in self.spec.order if r.stream_row is not None)
        for r in self.spec.order:
            b = self.blocks[r.layer]
            total += b.launches() if hasattr(b, "launches") else 1
        return total

    # ---- what the cache manager must provide ------------------------------
    @property
    def needs_state(self) -> bool:
        return any(not getattr(c.spec, "PAGED", False) for c in self.cache_slots)

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step may be captured once and replayed: no part says no."""
        return all(p.GRAPH_SAFE for p, _ in self._parts) and all(b.GRAPH_SAFE for b in self.blocks)

    @property
    def graph_safe_portions(self) -> bool:
        """Whether a step that brings prompt portions may be captured and replayed too: every part says yes."""
        return self.graph_safe and all(p.GRAPH_SAFE_PORTIONS for p, _ in self._parts) and \
            all(b.GRAPH_SAFE_PORTIONS for b in self.blocks)

    @property
    def atomic_prefill(self) -> bool:
        """Whether some mixer cannot continue a prompt from a cut: requests are then fed whole or not at all."""
        return any(getattr(p, "ATOMIC_PREFILL", False) for p, _ in self._parts)

    # ---- forward ------------------------------------------------------------
    def _add_stream_row(self, hidden, residual, row: int):
        """Adds row ``row`` of the model's stream rows to the stream, in 32-bit and in place.  The stream is what a block
        that hands it on left (``hidden`` None, a 32-bit residual), or, in front of the first run, the embedding."""
        from ..ops import kernels as K
        if residual is None:
            hidden = K.as_tensor(hidden)
            stream = hidden if hidden.dtype == torch.float32 else K.to_f32(hidden)
            return K.stream_add_row_(stream, self.stream_rows[row]), None
        if hidden is not None or residual.dtype != torch.float32:
            raise PartError("a row is added to a 32-bit stream that travels alone between blocks")
        K.stream_add_row_(residual, self.stream_rows[row])
        return None, residual

    def forward(self, step, caches) -> torch.Tensor:
        """Runs the step's tokens; returns float32 logits [W, vocab] at ``step.want_rows``.

        ``caches[i]`` is the view of cache slot i (``engine.caches``).
        """
        if getattr(self.embedding, "NEEDS_STEP", False):
            hidden = self.embedding.forward(step.token_ids, step=step,
                                            cache=None if self.embedding_cache is None else caches[self.embedding_cache])
        else:
            hidden = self.embedding.forward(step.token_ids)
        residual = None
        step.compute_dtype = self.dtype
        for i, r in enumerate(self.spec.order):
            if r.stream_row is not None:
                hidden, residual = self._add_stream_row(hidden, residual, r.stream_row)
            ci = self.run_cache[i]
            cache = None if ci is None else (tuple(caches[c] for c in ci) if isinstance(ci, tuple) else caches[ci])
            hidden, residual = self.blocks[r.layer].forward(hidden, residual, step, cache,
                                                            write_cache=r.reads_cache_of is None)
        if step.want_rows.shape[0] == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if self.blocks[self.spec.order[-1].layer].HANDS_ON_STREAM:
            # the last block handed on the stream itself: nothing waits to be added, the norm is of its rows alone
            normed = self.final_norm.forward_rows(None, residual, step.want_rows,
                                                  out_dtype=hidden.dtype if hidden is not None else self.dtype)
            return self.head.forward(normed)
        if not self.final_norm.TAKES_SLICE_SUMS:
            from ..ops import kernels as K
            hidden = K.as_tensor(hidden)
        normed = self.final_norm.forward_rows(hidden, residual, step.want_rows)
        return self.head.forward(normed)
