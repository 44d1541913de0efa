"""The token embedding: x = E[token], a row copy widened to the float32 residual stream, no scale
(internal/engine/engine.go:1365, 1375; internal/device/kernels.metal:465-467; the reference's
`GlobalScale` is fixed at 1.0, engine.go:533, 785)."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import EMBEDDINGS, MATRIX, BuildEnv, Embedding, StateNeed, StepContext, TensorSpec


@EMBEDDINGS.register("token_table")
class TokenTable(Embedding):
    graph_safe = True
    # `table` is only ever handed to `kernels.embed`: a model whose head is this table may put the product's
    # form of it (`parts.base.product_weight`) in its place
    table_is_for_kernels = True

    def __init__(self, name: str, vocab_size: int, width: int, scale: float = 1.0) -> None:
        """`scale`: x = scale * E[token] (a model's own constant; the product is taken in 32-bit)."""
        self.name, self.vocab_size, self.width, self.scale = name, int(vocab_size), int(width), float(scale)
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.vocab_size, self.width), kind=MATRIX)]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.table = tensors[self.name].contiguous()

    def forward(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.ws.alloc((ctx.rows, self.width), torch.float32, keep=True)
        if self.scale == 1.0:
            ctx.kernels.embed(self.table, ctx.tokens, x)
        else:
            ctx.kernels.embed(self.table, ctx.tokens, x, scale=self.scale)
        return x


@EMBEDDINGS.register("token_bigram_table")
class TokenBigramTable(TokenTable):
    """x = E[token] + B[row]: a second table, asked with a hash of the token and the one before it in its sequence,
    row = (previous * mul_prev + token * mul_cur) mod buckets; a sequence's first token takes the extra last row
    (number `buckets`).  The previous token is per-sequence state: the last token of every step stays in the
    cache manager's store for the step after it.  The sum is 32-bit."""

    def __init__(self, name: str, vocab_size: int, width: int, bigram_name: str, buckets: int, mul_prev: int,
                 mul_cur: int, scale: float = 1.0) -> None:
        super().__init__(name, vocab_size, width, scale)
        self.bigram_name, self.buckets = bigram_name, int(buckets)
        self.mul_prev, self.mul_cur = int(mul_prev), int(mul_cur)
        if self.buckets < 1:
            raise ValueError("the bigram table needs at least one bucket")
        self.bigram: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return super().tensor_specs() + [TensorSpec(self.bigram_name, (self.buckets + 1, self.width), kind=MATRIX)]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.bigram = tensors[self.bigram_name].contiguous()

    def cache_need(self) -> StateNeed:
        return StateNeed((1,), torch.int32)  # the sequence's last token

    def forward(self, ctx: StepContext, cache=None) -> torch.Tensor:
        if cache is None or getattr(cache, "state", None) is None:
            raise RuntimeError("the bigram embedding needs its store of last tokens")
        x = super().forward(ctx)
        ctx.kernels.bigram_add(x, self.bigram, ctx.tokens, cache.state, self.buckets, self.mul_prev, self.mul_cur,
                               self.vocab_size, ctx.row_pos, ctx.row_seq, ctx.seq_slot, ctx.cu_rows, ctx.batch)
        return x
