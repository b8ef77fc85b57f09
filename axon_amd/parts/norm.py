"""Norms: rows of the 32-bit residual stream, normalised into the compute dtype (RMSNorm, LayerNorm).

out = (x * 1/sqrt(mean(x^2) + eps)) * gain (src/model.rs:3888-3898).  Parameters: `size`,
`eps`, `tensor` (the gain's name under the part's prefix), `offset` (default 0: the gain is
offset + the stored vector, added once in 32-bit when the weights are loaded; 1 for checkpoints
that store their gains around zero).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .base import FollowingNorm, Norm, PrecedingNorm, TensorDecl, register_norm


class RMSNorm(Norm):
    graph_safe = True
    kind = "rms"         # what a kernel that norms on the way (the sum before a norm, say) is told
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.name = prefix + params.get("tensor", "weight")
        self.offset = float(params.get("offset", 0.0))
        self.gain = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.size,), "gain")]

    def load(self, store, rt) -> None:
        self.gain = store.vector(self.name)
        if self.offset != 0.0:
            self.gain = (self.gain.float() + self.offset).contiguous()      # kept 32-bit: 1 + w has more digits than w

    def forward(self, ctx, x, out=None, rows: Optional["torch.Tensor"] = None):
        """x: float32 [T, size]; `rows` picks rows of x (the wanted positions before the head)."""
        n = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = ctx.ws.take((n, self.size), ctx.rt.dtype)
        return ctx.rt.k.rmsnorm(x, self.gain, self.eps, out, rows)

    def following(self, ctx, n_rows: int) -> Optional[FollowingNorm]:
        """The product before the norm writes the finished rows (where its kernel offers it)."""
        return FollowingNorm(self.gain, self.eps, ctx.ws.take((n_rows, self.size), ctx.rt.dtype))

    def preceding(self, ctx, x) -> Optional[PrecedingNorm]:
        """The product after the norm reads the float32 rows and norms them on the way (where its
        kernel offers it)."""
        return PrecedingNorm(self, x)


class LayerNorm(Norm):
    """out = (x - mean x) / sqrt(var x + eps) * gain, the variance the mean of the squared deviations;
    a gain and no bias.  Parameters: `size`, `eps`, `tensor`.  It offers itself to no product (the
    products' norms are RMS norms): it runs as a pass of its own, or inside the pass of a block that
    norms behind its sums."""
    graph_safe = True
    kind = "layer"

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.name = prefix + params.get("tensor", "weight")
        self.gain = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.size,), "gain")]

    def load(self, store, rt) -> None:
        self.gain = store.vector(self.name)

    def forward(self, ctx, x, out=None, rows: Optional["torch.Tensor"] = None):
        n = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = ctx.ws.take((n, self.size), ctx.rt.dtype)
        return ctx.rt.k.layernorm(x, self.gain, self.eps, out, rows)


register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
