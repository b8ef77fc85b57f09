"""A mixture of experts: each token goes through the `top` experts its router ranks first; a shared
expert, if any, sees every token.  Two routers: "softmax" (the default): the largest logits, weighted by
the softmax over those logits alone; "sigmoid": scores s = sigmoid(logits) that do not compete, the
choice made by s + a stored correction among the experts of the `keep` best of `groups` equal groups of
neighbours (a group's score: the sum of its two largest choice scores), weighted by s over the sum of
the chosen s, times `scale` (with `normalize` false: the chosen s themselves, times `scale`).  A weight
multiplies its expert's output, or with `weight_on` = "input" the expert's input: sum_e expert_e(w_e h),
which differs since an expert is not linear (the products being linear, the factor is applied to their sums
in 32-bit, before the unit).

Router logits are 32-bit (Wr h with h in the compute dtype).  An expert is a gated unit with
clamps: g = min(Wgate h, limit), u = clamp(Wup h, -limit, limit), out = Wdown (g sigmoid(alpha g)
(u + 1)), without biases.  The (token, chosen expert) pairs are listed expert by expert on the
device and two grouped products (gate|up with the activation in its epilogue, then down) run
over the list; a token's rows are then added in the order of its router's ranking.  With many rows
an expert (a long prompt) the list is made in tiles of 64 rows, which the grouped product takes
through LDS: the same chains and bits as the tiles of 16 of a short step.

Parameters: `hidden_size`, `experts`, `top`, `ff`, `limit` (None: no clamps), `alpha` (default 1.702),
`shift` (default 1: the unit is g sigmoid(alpha g) (u + shift); no clamps, alpha 1 and shift 0 make it
silu(gate) up), `router` (None, or {"scores": "sigmoid", "correction": bool, "groups", "keep", "scale",
"normalize"}), `weight_on` ("output", the default, or "input"), `shared` (None, or {"ff", "limit"}: the clamped
unit; {"ff", "unit": "gated"}: silu(gate) up without clamps; with "gate": name, the shared expert's output is
multiplied by sigmoid(w . h), w the tensor [1, hidden] of that name in the shared expert's scope, whose logit
is one more row of the router's product), `names` (scope "mlp.", router, correction, expert "e{}.", shared
"shared.").
"""
from __future__ import annotations

import math
from typing import List

import torch

from ..config.base import ConfigError, PartSpec
from ..kernels import MODE_STORE_F32
from .base import FeedForward, TensorDecl, build_part, register_feed_forward


class RoutedExperts(FeedForward):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.n_experts, self.top = int(p["hidden_size"]), int(p["experts"]), int(p["top"])
        self.ff, self.alpha, self.shift = int(p["ff"]), float(p.get("alpha", 1.702)), float(p.get("shift", 1.0))
        self.limit = math.inf if p.get("limit") is None else float(p["limit"])
        if not 1 <= self.top <= self.n_experts:
            raise ConfigError(f"{self.top} of {self.n_experts} experts a token")
        names = p.get("names", {})
        self.base = prefix + names.get("scope", "mlp.")
        self.router_name = self.base + names.get("router", "router")
        router = dict(p.get("router") or {})
        self.scores = router.get("scores", "softmax")
        if self.scores not in ("softmax", "sigmoid"):
            raise ConfigError(f"a router with '{self.scores}' scores is not known (softmax, sigmoid)")
        self.groups, self.keep = int(router.get("groups", 1)), int(router.get("keep", 1))
        self.route_scale = float(router.get("scale", 1.0))
        self.normalize = bool(router.get("normalize", True))
        self.weight_on = p.get("weight_on", "output")
        if self.weight_on not in ("output", "input"):
            raise ConfigError(f"a router's weight on '{self.weight_on}' is not known (output, input)")
        self.correction_name = self.base + names.get("correction", "correction") if router.get("correction") else None
        self.correction = None
        if self.scores == "sigmoid":
            if self.n_experts > 1024 or self.top > 64 or self.groups > 64:
                raise ConfigError(f"the sigmoid router takes up to 1024 experts in up to 64 groups and up to 64 a token, "
                                  f"not {self.top} of {self.n_experts} in {self.groups}")
            if self.groups < 1 or self.n_experts % self.groups or not 1 <= self.keep <= self.groups \
                    or self.keep * (self.n_experts // self.groups) < self.top:
                raise ConfigError(f"{self.keep} of {self.groups} groups of {self.n_experts} experts cannot give {self.top} a token")
        elif router:
            raise ConfigError("groups, a correction and a scale belong to the router with sigmoid scores")
        self.expert_scope = names.get("expert", "e{}.")
        self.shared = None
        self.shared_gate_name = None
        if p.get("shared"):
            sh = p["shared"]
            scope = names.get("scope", "mlp.") + names.get("shared", "shared.")
            if sh.get("unit", "clamped") == "gated":
                self.shared = build_part("feed_forward", PartSpec("swiglu_mlp", {
                    "hidden_size": self.hidden, "intermediate_size": int(sh["ff"]),
                    "names": {"scope": scope, "gate": "gate", "up": "up", "down": "down", "suffix": ""}}), prefix)
            elif sh.get("unit", "clamped") == "clamped":
                self.shared = build_part("feed_forward", PartSpec("clamped_glu_mlp", {
                    "hidden_size": self.hidden, "ff": int(sh["ff"]), "limit": float(sh["limit"]),
                    "alpha": float(sh.get("alpha", self.alpha)), "names": {"scope": scope}}), prefix)
            else:
                raise ConfigError(f"a shared expert's unit '{sh.get('unit')}' is not known (clamped, gated)")
            if sh.get("gate"):
                if self.scores != "sigmoid":
                    raise ConfigError("a gate on the shared expert comes with the router of sigmoid scores (its logit is a row of that product)")
                self.shared_gate_name = prefix + scope + str(sh["gate"])

    def _expert(self, e: int, which: str) -> str:
        return self.base + self.expert_scope.format(e) + which

    def tensors(self) -> List[TensorDecl]:
        t = [TensorDecl(self.router_name, (self.n_experts, self.hidden))]
        if self.correction_name is not None:
            t.append(TensorDecl(self.correction_name, (self.n_experts,), "bias"))
        for e in range(self.n_experts):
            t += [TensorDecl(self._expert(e, "gate"), (self.ff, self.hidden)), TensorDecl(self._expert(e, "up"), (self.ff, self.hidden)),
                  TensorDecl(self._expert(e, "down"), (self.hidden, self.ff))]
        if self.shared_gate_name is not None:
            t.append(TensorDecl(self.shared_gate_name, (1, self.hidden)))
        return t + (self.shared.tensors() if self.shared is not None else [])

    def load(self, store, rt) -> None:
        if self.shared_gate_name is not None:       # the shared expert's gate logit: one more row of the router's product
            self.w_router = rt.k.prepare_weight(store.fused_matrix([self.router_name, self.shared_gate_name]))
        else:
            self.w_router = rt.k.prepare_weight(store.matrix(self.router_name))
        if self.correction_name is not None:
            self.correction = store.vector(self.correction_name).float().contiguous()
        E = self.n_experts
        # every expert's gate rows, then its up rows: [experts, 2 ff, hidden]; and [experts, hidden, ff]
        self.w_gate_up = torch.empty((E, 2 * self.ff, self.hidden), dtype=rt.dtype, device=rt.device)
        self.w_down = torch.empty((E, self.hidden, self.ff), dtype=rt.dtype, device=rt.device)
        for e in range(E):
            self.w_gate_up[e, :self.ff].copy_(store.matrix(self._expert(e, "gate")))
            self.w_gate_up[e, self.ff:].copy_(store.matrix(self._expert(e, "up")))
            self.w_down[e].copy_(store.matrix(self._expert(e, "down")))
            for which in ("gate", "up", "down"):
                store.forget(self._expert(e, which))
        if self.shared is not None:
            self.shared.load(store, rt)

    def forward(self, ctx, h, out, accumulate: bool = True) -> None:
        k, T, E, top = ctx.rt.k, h.shape[0], self.n_experts, self.top
        i32 = torch.int32
        gated_shared = self.shared_gate_name is not None
        logits = ctx.ws.take((T, E + 1 if gated_shared else E), torch.float32)
        k.gemm(h, self.w_router, logits, None, MODE_STORE_F32)
        chosen, weights = ctx.ws.take((T, top), i32), ctx.ws.take((T, top), torch.float32)
        if self.scores == "sigmoid" and (gated_shared or not self.normalize):
            k.route_scored(logits, self.correction, top, self.groups, self.keep, self.route_scale, chosen, weights,
                           normalize=self.normalize, n_experts=E)
        elif self.scores == "sigmoid":
            k.route_scored(logits, self.correction, top, self.groups, self.keep, self.route_scale, chosen, weights)
        else:
            k.route_topk(logits, top, chosen, weights)
        P = T * top
        tile_rows = 64 if P >= 32 * E else 16          # many rows an expert: tiles of 64 rows through LDS (the same bits)
        max_tiles = k.route_max_tiles(P, E, tile_rows)
        pairs, tokens = ctx.ws.take((P,), i32), ctx.ws.take((P,), i32)
        tiles, n_tiles = ctx.ws.take((3 * max_tiles,), i32), ctx.ws.take((1,), i32)
        k.route_sort(chosen, E, pairs, tokens, tiles, n_tiles, tile_rows=tile_rows)
        act = ctx.ws.take((P, self.ff), ctx.rt.dtype)
        on_input = self.weight_on == "input"        # act row p is the unit of (weight of pair p) x (the token's row)
        k.grouped_gemm(h, self.w_gate_up, act, x_group_stride=0, out_group_stride=0, glu=(self.limit, self.alpha, self.shift),
                       routed=(tiles, n_tiles, max_tiles, tokens, pairs, tile_rows), rows=P,
                       row_scale=weights.view(-1) if on_input else None)
        rows = ctx.ws.take((P, self.hidden), torch.float32)
        k.grouped_gemm(act, self.w_down, rows, x_group_stride=0, out_group_stride=0,
                       routed=(tiles, n_tiles, max_tiles, pairs, pairs, tile_rows), rows=P)
        if gated_shared:
            extra = ctx.ws.take((T, self.hidden), torch.float32)
            self.shared.forward(ctx, h, extra, accumulate=False)
            k.route_combine(rows, None if on_input else weights, out, accumulate, top=top, extra=extra, extra_gate=logits[:, E:])
            return
        k.route_combine(rows, None if on_input else weights, out, accumulate, top=top)
        if self.shared is not None:
            self.shared.forward(ctx, h, out)


register_feed_forward("routed_experts", RoutedExperts)
