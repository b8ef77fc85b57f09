"""Attention whose keys and values go through a shared latent (multi-head latent attention).

From the input h: the query latent c_q = rmsnorm(Wdq h), q = Wuq c_q, laid out head by head as
[dim unrotated, rot_dim rotated]; Wdkv h gives kv_rank rows that, RMS-normed, are the latent c,
and rot_dim more that are one rotated key part shared by all heads.  A head's unrotated key is
Wuk c and its value Wuv c; the score is (q_unrot . k_unrot + q_rot . k_rot) * scale over a
causal window; the concatenated heads are multiplied by sigmoid(Wg h) and projected by Wo.

Only c and the rotated key part are cached, and the keys and values are never built (a position
takes 2 kv_rank + rot_dim elements of its page: the row the scores read, and the latent once more
with the positions of one dim side by side, as the matrix cores want the weighted sum's operand): the unrotated query is carried into the latent space
(q_lat = Wuk^T q_unrot, a per-head product), attention runs there, and the head's output is
Wuv (sum_j p_j c_j), a second per-head product.

Variations, all parameters: no query latent (`q_rank` 0: q = Wq h, one matrix); a sink (`sink`: a learned
number a head whose exponential the softmax's denominator also holds, once, with no key and no value);
the gate one number a head (`gate` "heads": sigmoid(Wg h)_head, Wg [heads, hidden]) instead of one an
output element (`gate` "elements"); the rotation's pairs, frequencies and magnitude are the position
encoding's (`pairing`, `scaling`).

Parameters: `hidden_size`, `heads`, `dim`, `rot_dim`, `vdim`, `kv_rank`, `q_rank`, `scale`,
`window` (0: all earlier positions), `eps` (of the latents' norms), `gated` (the sigmoid gate) or
`gate` (None, "elements", "heads"), `sink`, `position` (a PartSpec of the rotation), `names`.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE_F32
from .base import CacheBinding, CacheSpec, Mixer, TensorDecl, build_part, register_mixer


class LatentAttention(Mixer):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.heads = int(p["hidden_size"]), int(p["heads"])
        self.dim, self.rot, self.vdim = int(p["dim"]), int(p["rot_dim"]), int(p["vdim"])
        self.kv_rank, self.q_rank = int(p["kv_rank"]), int(p["q_rank"])
        self.scale, self.window, self.eps = float(p["scale"]), int(p.get("window", 0)), float(p["eps"])
        self.gate = p["gate"] if "gate" in p else ("elements" if p.get("gated", True) else None)
        if self.gate not in (None, "elements", "heads"):
            raise ConfigError(f"a gate '{self.gate}' is not known (elements, heads)")
        self.gated = self.gate is not None
        self.has_sink = bool(p.get("sink", False))
        self.position = build_part("position", p["position"]) if p.get("position") is not None and self.rot > 0 else None
        self.rot_dims = self.position.rotary_dim if self.position is not None else 0
        if self.rot_dims > self.rot:
            raise ConfigError(f"{self.rot_dims} rotated dims in a rotated part of {self.rot}")
        if self.kv_rank > 1024:
            raise ConfigError(f"a key/value latent of {self.kv_rank} is more than the attention kernel's 1024")
        names = p.get("names", {})
        base = prefix + names.get("scope", "mix.")
        self.n = {k: base + names.get(k, k) for k in ("q", "dq", "uq", "dkv", "uk", "uv", "g", "o", "sink")}
        self.neighbours = self.position is not None and self.position.pairing == "neighbours"
        self.magnitude = self.position.magnitude if self.position is not None else 1.0
        self.n_gate = 0 if not self.gated else (self.heads if self.gate == "heads" else self.heads * self.vdim)

    def tensors(self) -> List[TensorDecl]:
        n, H = self.n, self.heads
        if self.q_rank:
            t = [TensorDecl(n["dq"], (self.q_rank, self.hidden)), TensorDecl(n["dq"] + ".norm", (self.q_rank,), "gain"),
                 TensorDecl(n["uq"], (H * (self.dim + self.rot), self.q_rank))]
        else:
            t = [TensorDecl(n["q"], (H * (self.dim + self.rot), self.hidden))]
        t += [TensorDecl(n["dkv"], (self.kv_rank + self.rot, self.hidden)), TensorDecl(n["dkv"] + ".norm", (self.kv_rank,), "gain"),
             TensorDecl(n["uk"], (H * self.dim, self.kv_rank)), TensorDecl(n["uv"], (H * self.vdim, self.kv_rank)),
             TensorDecl(n["o"], (self.hidden, H * self.vdim))]
        if self.gated:
            t.append(TensorDecl(n["g"], (self.n_gate, self.hidden)))
        if self.has_sink:
            t.append(TensorDecl(n["sink"], (H,), "bias"))
        return t

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(entries=1, heads=1, head_dim=2 * self.kv_rank + self.rot, window=self.window)

    def load(self, store, rt) -> None:
        n, H = self.n, self.heads
        # every product of the input as one matrix: [the query latent's, or the queries'; the key/value latent's; the gate's]
        down = [n["dq"] if self.q_rank else n["q"], n["dkv"]] + ([n["g"]] if self.gated else [])
        self.w_down = rt.k.prepare_weight(store.fused_matrix(down))
        self.kv_gain = store.vector(n["dkv"] + ".norm")
        self.q_gain = store.vector(n["dq"] + ".norm") if self.q_rank else None
        self.w_uq = rt.k.prepare_weight(store.matrix(n["uq"])) if self.q_rank else None
        self.sink = store.vector(n["sink"]).float().contiguous() if self.has_sink else None
        # per head: Wuk^T [kv_rank, dim] carries a query into the latent space, Wuv [vdim, kv_rank] a latent out of it
        self.w_uk_t = store.matrix(n["uk"]).view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = store.matrix(n["uv"]).view(H, self.vdim, self.kv_rank).contiguous()
        self.w_o = rt.k.prepare_weight(store.matrix(n["o"]))
        for name in ([n["uq"]] if self.q_rank else []) + [n["uk"], n["o"]]:
            store.forget(name)
        if self.position is not None:
            self.position.load(store, rt)

    SPAN_STEP = 512      # the positions a decoding step's longest row sees, rounded up to this: part of the step's shape

    def decode_shape(self, positions):
        """Without a window the blocks of positions that run side by side depend on how long the
        contexts are: a captured graph is replayed for steps whose longest row sees as many."""
        if self.window > 0:
            return None
        return ("latent_span", -(-(max(positions) + 1) // self.SPAN_STEP) * self.SPAN_STEP)

    def forward(self, ctx, binding: CacheBinding, h, out, accumulate: bool = True) -> None:
        k, T, H = ctx.rt.k, h.shape[0], self.heads
        group = ctx.cache.group(binding.group)
        (cache,) = group.layer(binding.index)
        n_q = self.q_rank if self.q_rank else H * (self.dim + self.rot)        # the first columns of the fused product
        down = ctx.ws.take((T, n_q + self.kv_rank + self.rot + self.n_gate), torch.float32)
        k.gemm(h, self.w_down, down, None, MODE_STORE_F32)
        table = self.position.tables(ctx) if self.position is not None else ctx.no_rotation()
        cq = ctx.ws.take((T, self.q_rank), ctx.rt.dtype) if self.q_rank else None
        k.latent_prepare(down, 0, self.q_rank, n_q, self.kv_rank, self.rot, self.rot_dims, self.q_gain, self.kv_gain,
                         self.eps, table, ctx.positions, ctx.seq_rows, group.block_table, cache, group.page_size, cq,
                         binding.writes, neighbours=self.neighbours, magnitude=self.magnitude)
        if self.q_rank:
            q = ctx.ws.take((T, H * (self.dim + self.rot)), torch.float32)
            k.gemm(cq, self.w_uq, q, None, MODE_STORE_F32)
        else:
            q = down[:, :n_q]
        width = self.kv_rank + self.rot
        q_full = ctx.ws.take((T, H * width), torch.float32)
        k.latent_query_rope(q, self.dim, self.rot, self.rot_dims, table, q_full, self.kv_rank, H, neighbours=self.neighbours,
                            magnitude=self.magnitude)
        k.grouped_gemm(q, self.w_uk_t, q_full, x_group_stride=self.dim + self.rot, out_group_stride=width)
        o_lat = ctx.ws.take((T, H * self.kv_rank), torch.float32)
        if ctx.decode_only:
            span = ctx.decode_shapes.get("latent_span", 0)
        else:
            span = max(s.start_pos + s.q_len for s in ctx.spans)
        k.latent_attention(q_full, cache, group.block_table, ctx.positions, ctx.seq_rows, o_lat, H, self.kv_rank, self.rot,
                           group.page_size, self.window, self.scale, sink=self.sink, span=span)
        att = ctx.ws.take((T, H * self.vdim), ctx.rt.dtype)
        gate = down[:, n_q + self.kv_rank + self.rot:] if self.gated else None
        k.grouped_gemm(o_lat, self.w_uv, att, x_group_stride=self.kv_rank, out_group_stride=self.vdim, gate=gate,
                       gate_per_group=self.gate == "heads")
        k.gemm(att, self.w_o, out, None, MODE_ADD_F32 if accumulate else MODE_STORE_F32)


register_mixer("latent_attention", LatentAttention)
