"""Embeddings that are more than one table. The plain table needs no part (``DecoderModel`` looks its rows up
itself); a part registered here replaces that look-up and may keep a little state per request."""
from __future__ import annotations

import torch

from ..native import ops
from .base import EMBEDDINGS, ParamSpec, Part, StateNeed


@EMBEDDINGS.register("hashed_pair")
class HashedPairEmbedding(Part):
    """x_t = table[token_t] + pair[(token_(t-1) * mul_prev + token_t * mul_cur) mod buckets]; the first token of a
    request takes row ``buckets`` (the last) of ``pair``. The rows are added in float and the result is float32 (the
    stream that the layers add to). The token before a portion's first one is kept per request (one int32 in the
    request's state slot), so prompts may be cut anywhere."""

    def __init__(self, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int):
        if buckets <= 0:
            raise ValueError(f"the pair table needs at least one bucket, got {buckets}")
        self.hidden_size, self.buckets, self.mul_prev, self.mul_cur = hidden_size, buckets, mul_prev, mul_cur
        self.pair_weight = None

    def param_specs(self):
        return {"pair.weight": ParamSpec((self.buckets + 1, self.hidden_size))}

    def state_need(self) -> StateNeed:
        return StateNeed({"prev": ((), torch.int32)})

    def forward(self, step, table: torch.Tensor, state: dict) -> torch.Tensor:
        return ops.embed_pair_hash(step.input_ids, table, self.pair_weight, step.attention, step.state_slots,
                                   state["prev"], self.buckets, self.mul_prev, self.mul_cur)


@EMBEDDINGS.register("scaled_float")
class ScaledFloatEmbedding(Part):
    """x_t = table[token_t] * scale as float32: the start of a float32 stream, multiplied and kept unrounded."""

    def __init__(self, scale: float | None = None):
        self.scale = None if scale is None else float(scale)

    def forward(self, step, table: torch.Tensor, state) -> torch.Tensor:
        return ops.embed_float(step.input_ids, table, self.scale)
