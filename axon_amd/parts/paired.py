"""Two mixers side by side on the same input: out = mult (rms(left(h)) g_l + rms(right(h)) g_r).

Each side is a mixer of its own (a `PartSpec`), run on the same rows h; its 32-bit output is normed
over the model width (an RMS norm with a plain gain and the layer's eps) and added into the residual
stream times `mult` (a half: the mean of the two), the norm, the factor and the sum in one 32-bit pass a
side.  One side may keep pages (a `CacheSpec`) and one may keep per-request state (a `StateSpec`): the
run's binding serves both; two sides that both want pages, or both want state, are refused.

Parameters: `hidden_size`, `eps`, `left`, `right` (the sides' PartSpecs; their tensors lie under
`<scope>left.` and `<scope>right.`), `mult` (default 0.5), `names` (scope "mix.", left_out "left.out",
right_out "right.out": the gains of the two norms).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.base import ConfigError, PartSpec
from .base import CacheBinding, CacheSpec, Mixer, StateSpec, TensorDecl, build_part, register_mixer


class PairedMixers(Mixer):

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.eps, self.mult = int(p["hidden_size"]), float(p["eps"]), float(p.get("mult", 0.5))
        names = p.get("names", {})
        base = prefix + names.get("scope", "mix.")
        self.gain_names = [base + names.get("left_out", "left.out"), base + names.get("right_out", "right.out")]
        self.sides = [build_part("mixer", s if isinstance(s, PartSpec) else PartSpec(s["kind"], s["params"]), prefix)
                      for s in (p["left"], p["right"])]
        for side in self.sides:
            if not getattr(side, "stores_output", False):
                raise ConfigError(f"a side of a pair of mixers must be able to store its output ({type(side).__name__} cannot)")
        if sum(s.cache_spec() is not None for s in self.sides) > 1 or sum(s.state_spec() is not None for s in self.sides) > 1:
            raise ConfigError("a pair of mixers shares one binding: one side may keep pages, one may keep state")
        self.graph_safe = all(getattr(s, "graph_safe", False) for s in self.sides)
        self.gains = [None, None]

    # what the engine asks a mixer is answered by the side that it concerns
    def _first(self, method: str, *args):
        for side in self.sides:
            got = getattr(side, method)(*args)
            if got is not None:
                return got
        return None

    def cache_spec(self) -> Optional[CacheSpec]:
        return self._first("cache_spec")

    def state_spec(self) -> Optional[StateSpec]:
        return self._first("state_spec")

    def max_context(self) -> Optional[int]:
        limits = [m for m in (s.max_context() for s in self.sides) if m is not None]
        return min(limits) if limits else None

    def decode_shape(self, positions):
        return self._first("decode_shape", positions)

    def decode_input(self, positions):
        return self._first("decode_input", positions)

    def decode_input_capacity(self, max_seqs: int, max_seq_len: int) -> int:
        return max(s.decode_input_capacity(max_seqs, max_seq_len) for s in self.sides)

    def decode_scratch(self, max_seqs: int, max_seq_len: int):
        return self._first("decode_scratch", max_seqs, max_seq_len)

    def tensors(self) -> List[TensorDecl]:
        t = [d for s in self.sides for d in s.tensors()]
        return t + [TensorDecl(name, (self.hidden,), "gain") for name in self.gain_names]

    def load(self, store, rt) -> None:
        for s in self.sides:
            s.load(store, rt)
        self.gains = [store.vector(name) for name in self.gain_names]

    def forward(self, ctx, binding: CacheBinding, h, residual) -> None:
        k = ctx.rt.k
        y = ctx.ws.take(tuple(residual.shape), torch.float32)
        for side, gain in zip(self.sides, self.gains):
            side.forward(ctx, binding, h, y, accumulate=False)
            k.norm_add(y, gain, self.eps, self.mult, residual)


register_mixer("paired_mixers", PairedMixers)
