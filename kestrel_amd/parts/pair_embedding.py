"""An embedding of token pairs, added to the embedded tokens before the first block."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from .base import PositionEncoding, register_position
from .specs import PairEmbeddingSpec, ParamSpec, StateSpec


class PairEmbedding(PositionEncoding):
    """``x[t] += table[(prev * mul_prev + cur * mul_cur) mod buckets]`` where ``prev`` is the token before ``cur`` in its
    sequence, and ``table[buckets]`` (the last row) for a sequence's first token.

    The token before the first token of a step's portion is per-request state: one int32 per request slot, which the
    kernel reads and then sets to the portion's last token (token ids that sampling left on the device included, so a
    decoded token never has to pass through the host). Places whose embedding is given from outside get nothing added,
    and neither does the token right after such a place."""

    replays_every_step = True

    def __init__(self, spec: PairEmbeddingSpec) -> None:
        super().__init__(spec)
        if spec.buckets <= 0:
            raise ValueError(f"a pair embedding needs a positive number of buckets, got {spec.buckets}")
        self.table: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        return {"table": ParamSpec((self.spec.buckets + 1, self.spec.dim), "matrix", "normal")}

    def state_spec(self) -> StateSpec:
        return StateSpec((1,), "int32")

    def bind(self, tensors, dtype, device) -> None:
        self.table = tensors["table"].to(device).contiguous()

    def add_to_embeddings(self, x, batch, state=None) -> None:
        if state is None:
            raise RuntimeError("the pair embedding needs its per-request state from the cache manager")
        spec = self.spec
        core.pair_embed(self.table, batch.token_ids, batch.positions, batch.token_row, batch.cu_q, batch.row_slot,
                        state.view(-1), spec.buckets, spec.mul_prev, spec.mul_cur, x, spec.vocab_size, batch.pending)


register_position("pair_embedding", PairEmbedding)
