"""Rewrites of the residual stream between runs.

"embedding_mix": x <- W [x ; x0], one matrix [hidden, 2 hidden] over the stream and the embedding's
output side by side (the stream's columns first).  A model whose layers run several times over uses
it at the start of every pass, so that each pass sees the tokens again.  The two row sets are rounded
to the compute dtype side by side by one small kernel, the product stores 32-bit rows into x.
Parameters: `hidden_size`, `tensor`.

"embedding_add": x <- x + factor x0, no tensor: a pass of a loop sees the tokens again by plain addition
(32-bit).  Parameters: `factor` (default 1).
"""
from __future__ import annotations

from typing import List

from ..kernels import MODE_STORE_F32
from .base import StreamEntry, TensorDecl, register_stream


class EmbeddingMix(StreamEntry):
    graph_safe = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden = int(params["hidden_size"])
        self.name = prefix + params["tensor"]
        self.weight = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.hidden, 2 * self.hidden))]

    def load(self, store, rt) -> None:
        self.weight = rt.k.prepare_weight(store.matrix(self.name))
        store.forget(self.name)

    def forward(self, ctx, x, x0) -> None:
        k = ctx.rt.k
        both = k.concat_round(x, x0, ctx.ws.take((x.shape[0], 2 * self.hidden), ctx.rt.dtype))
        k.gemm(both, self.weight, x, None, MODE_STORE_F32)


class EmbeddingAdd(StreamEntry):
    graph_safe = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.factor = float(params.get("factor", 1.0))

    def forward(self, ctx, x, x0) -> None:
        ctx.rt.k.add_scaled(x, x0, self.factor)


register_stream("embedding_mix", EmbeddingMix)
register_stream("embedding_add", EmbeddingAdd)
