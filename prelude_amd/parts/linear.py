"""Embedding and output head.

Embedding rows by token id (crates/prelude-core/src/models/commons/embedding.rs:7-36);
head logits = W h with W [vocab, hidden], the embedding matrix itself when tied
(crates/prelude-core/src/models/qwen3.rs:637-660).  Logits leave in float32.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import MATRIX, Part, PartError, StateSpec, TensorReq, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self):
        return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

    def load(self, tensors, dtype, device):
        self.weight = tensors["weight"]

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return K.embed_gather(token_ids, self.weight)


@register_part("embedding", "pair_hash_embedding")
class PairHashEmbedding(Part):
    """x = table[token] * scale + pair[(previous token * mul_prev + token * mul_cur) mod buckets] (the modulus that is
    never negative, whatever the multipliers' signs), taken in 32-bit and
    handed on as the 32-bit stream; a sequence's first token reads row ``buckets`` (the last) of the pair table.  The
    previous token is part of a request's state: an embedding that says ``NEEDS_STEP`` is called with the step and with
    the storage of its ``cache_spec()``, one int32 a request here."""
    GRAPH_SAFE_PORTIONS = True
    NEEDS_STEP = True

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int, scale: float = 1.0):
        if int(buckets) < 1:
            raise PartError(f"pair_hash_embedding: {buckets} buckets")
        self.vocab_size, self.hidden_size, self.buckets = int(vocab_size), int(hidden_size), int(buckets)
        self.mul_prev, self.mul_cur, self.scale = int(mul_prev), int(mul_cur), float(scale)
        self.weight = self.pair = None

    def tensors(self):
        return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX),
                "pair": TensorReq((self.buckets + 1, self.hidden_size), MATRIX)}

    def load(self, tensors, dtype, device):
        self.weight, self.pair = tensors["weight"], tensors["pair"]

    def cache_spec(self):
        return StateSpec((("previous_token", (1,), torch.int32),))

    def forward(self, token_ids: torch.Tensor, step=None, cache=None) -> torch.Tensor:
        if step is None or cache is None:
            raise PartError("pair_hash_embedding: the step and the requests' previous tokens are needed")
        return K.pair_embed(token_ids, step, cache.tensors["previous_token"], self.weight, self.pair, self.buckets,
                            self.mul_prev, self.mul_cur, self.scale)


@register_part("head", "linear_head")
class LinearHead(Part):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, vocab_size: int, hidden_size: int, logit_cap: float = 0.0):
        """``logit_cap`` > 0: the logits leave as cap * tanh(logits / cap)."""
        self.vocab_size, self.hidden_size, self.logit_cap = int(vocab_size), int(hidden_size), float(logit_cap or 0.0)
        if self.logit_cap < 0:
            raise PartError(f"linear_head: a logit cap of {logit_cap} is negative")
        self.LAUNCHES = 2 if self.logit_cap else 1
        self.weight = None

    def tensors(self):
        return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

    def load(self, tensors, dtype, device):
        self.weight = K.prepare_weight(tensors["weight"])

    def forward(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        logits = K.linear(hidden_rows, self.weight, out_dtype=torch.float32)
        return K.cap_logits_(logits, self.logit_cap) if self.logit_cap else logits
