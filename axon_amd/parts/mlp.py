"""The dense SwiGLU feed-forward: down(silu(gate h) * up h), added to the residual stream.

act = (g / (1 + exp(-g))) * u (src/vmath.rs:128-132), no biases (src/model.rs:3043-3055).
gate and up run as one product over a fused [2 ffn, hidden] matrix whose epilogue applies the
activation, so the two halves never travel through memory.  Parameters:
`hidden_size`, `intermediate_size`, `names` (scope "mlp.", gate, up, down, suffix ".weight").
"""
from __future__ import annotations

from typing import List

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE, MODE_STORE_F32, MODE_SWIGLU, PackedMatrix
from .base import FeedForward, PrecedingNorm, TensorDecl, register_feed_forward


class SwiGLUMLP(FeedForward):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden = int(params["hidden_size"])
        self.ffn = int(params["intermediate_size"])
        names = params.get("names", {})
        base = prefix + names.get("scope", "mlp.")
        self.n = {k: base + names.get(k, k + "_proj") + names.get("suffix", ".weight") for k in ("gate", "up", "down")}
        self.w_gate_up = self.w_down = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.n["gate"], (self.ffn, self.hidden)), TensorDecl(self.n["up"], (self.ffn, self.hidden)),
                TensorDecl(self.n["down"], (self.hidden, self.ffn))]

    def load(self, store, rt) -> None:
        self.w_gate_up = rt.k.prepare_weight(store.fused_matrix([self.n["gate"], self.n["up"]]), gated=True)
        self.w_down = rt.k.prepare_weight(store.matrix(self.n["down"]))
        store.forget(self.n["down"])

    def finishes_following_norm(self, ctx) -> bool:
        return isinstance(self.w_down, PackedMatrix) and ctx.rt.k.gemm_then_norm_ok(ctx.n_tokens, self.hidden, self.ffn)

    def applies_preceding_norm(self, ctx) -> bool:
        return (isinstance(self.w_gate_up, PackedMatrix)
                and ctx.rt.k.gemm_normed_ok(ctx.n_tokens, self.ffn, self.hidden, gated=True))

    def forward(self, ctx, h, residual, following=None, accumulate: bool = True) -> None:
        k = ctx.rt.k
        act = ctx.ws.take((h.shape[0], self.ffn), ctx.rt.dtype)
        if isinstance(h, PrecedingNorm) and not k.gemm_normed_ok(h.shape[0], self.ffn, self.hidden, gated=True, gain=h.gain):
            h = h.apply(ctx)
        if isinstance(h, PrecedingNorm):                        # few rows: the norm inside the product
            k.gemm_normed_glu(h.rows, h.gain, h.eps, self.w_gate_up, act)
        else:
            k.gemm(h, self.w_gate_up, act, None, MODE_SWIGLU)   # silu(gate h) * up h, in the product's epilogue
        if not accumulate:          # the output itself, for a block that sums and norms on its own
            k.gemm(act, self.w_down, residual, None, MODE_STORE_F32)
            return
        k.gemm(act, self.w_down, residual, None, MODE_ADD_F32,
               following_norm=None if following is None else following.as_argument())


register_feed_forward("swiglu_mlp", SwiGLUMLP)


class DenseMLP(FeedForward):
    """down(act(up h)): a plain two-matrix feed-forward.  Parameters: `hidden_size`, `ff`,
    `activation` ("gelu_tanh": 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))), or "gelu_erf":
    0.5 z (1 + erf(z / sqrt 2))), `names` (scope "mlp.", up, down)."""
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden, self.ff = int(params["hidden_size"]), int(params["ff"])
        self.activation = params.get("activation", "gelu_tanh")
        if self.activation not in ("gelu_tanh", "gelu_erf"):
            raise ConfigError(f"activation '{self.activation}' is not known (gelu_tanh, gelu_erf)")
        names = params.get("names", {})
        base = prefix + names.get("scope", "mlp.")
        self.n = {k: base + names.get(k, k) for k in ("up", "down")}

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.n["up"], (self.ff, self.hidden)), TensorDecl(self.n["down"], (self.hidden, self.ff))]

    def load(self, store, rt) -> None:
        self.w_up = rt.k.prepare_weight(store.matrix(self.n["up"]))
        self.w_down = rt.k.prepare_weight(store.matrix(self.n["down"]))
        for name in self.n.values():
            store.forget(name)

    def finishes_following_norm(self, ctx) -> bool:
        """In steps of many rows the down projection's last kernel also writes the norm behind it."""
        return isinstance(self.w_down, PackedMatrix) and ctx.rt.k.gemm_then_norm_ok(ctx.n_tokens, self.hidden, self.ff)

    def forward(self, ctx, h, out, following=None, accumulate: bool = True) -> None:
        k = ctx.rt.k
        act = ctx.ws.take((h.shape[0], self.ff), ctx.rt.dtype)
        k.gemm(h, self.w_up, act, None, MODE_STORE)
        k.activation(act, self.activation)
        if following is not None and accumulate:
            k.gemm(act, self.w_down, out, None, MODE_ADD_F32, following_norm=following.as_argument())
        else:
            k.gemm(act, self.w_down, out, None, MODE_ADD_F32 if accumulate else MODE_STORE_F32)


class ClampedGLUMLP(FeedForward):
    """down(g sigmoid(alpha g) (u + 1)) with g = min(gate h, limit), u = clamp(up h, -limit, limit); no
    biases.  Parameters: `hidden_size`, `ff`, `limit`, `alpha` (default 1.702), `names` (scope "mlp.", gate, up, down)."""
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.hidden, self.ff = int(params["hidden_size"]), int(params["ff"])
        self.limit, self.alpha = float(params["limit"]), float(params.get("alpha", 1.702))
        names = params.get("names", {})
        base = prefix + names.get("scope", "mlp.")
        self.n = {k: base + names.get(k, k) for k in ("gate", "up", "down")}

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.n["gate"], (self.ff, self.hidden)), TensorDecl(self.n["up"], (self.ff, self.hidden)),
                TensorDecl(self.n["down"], (self.hidden, self.ff))]

    def load(self, store, rt) -> None:
        self.w_gate_up = rt.k.prepare_weight(store.fused_matrix([self.n["gate"], self.n["up"]]))
        self.w_down = rt.k.prepare_weight(store.matrix(self.n["down"]))
        store.forget(self.n["down"])

    def forward(self, ctx, h, out, accumulate: bool = True) -> None:
        k, T = ctx.rt.k, h.shape[0]
        gate_up = ctx.ws.take((T, 2 * self.ff), ctx.rt.dtype)
        k.gemm(h, self.w_gate_up, gate_up, None, MODE_STORE)
        act = ctx.ws.take((T, self.ff), ctx.rt.dtype)
        k.clamped_glu(gate_up, act, self.limit, self.alpha)
        k.gemm(act, self.w_down, out, None, MODE_ADD_F32 if accumulate else MODE_STORE_F32)


register_feed_forward("dense_mlp", DenseMLP)
register_feed_forward("clamped_glu_mlp", ClampedGLUMLP)
