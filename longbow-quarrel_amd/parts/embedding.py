"""The token embedding: x = E[token], a row copy widened to the float32 residual stream, no scale
(internal/engine/engine.go:1365, 1375; internal/device/kernels.metal:465-467; the reference's
`GlobalScale` is fixed at 1.0, engine.go:533, 785)."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import EMBEDDINGS, MATRIX, BuildEnv, Embedding, StepContext, TensorSpec


@EMBEDDINGS.register("token_table")
class TokenTable(Embedding):
    graph_safe = True
    # `table` is only ever handed to `kernels.embed`: a model whose head is this table may put the product's
    # form of it (`parts.base.product_weight`) in its place
    table_is_for_kernels = True

    def __init__(self, name: str, vocab_size: int, width: int) -> None:
        self.name, self.vocab_size, self.width = name, int(vocab_size), int(width)
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.vocab_size, self.width), kind=MATRIX)]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.table = tensors[self.name].contiguous()

    def forward(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.ws.alloc((ctx.rows, self.width), torch.float32, keep=True)
        ctx.kernels.embed(self.table, ctx.tokens, x)
        return x
