"""Grouped-query attention whose variations are parameters: score maps, norms, masks, bent scores, a gate.

q = Wq h (+ bq), k = Wk h (+ bk), laid out head by head; query head i reads key/value head
i // (heads / kv_heads).  What a configuration may turn on, each on its own:

* `maps` = 2, differential attention: a head's query and key hold two maps side by side,
  [map 1 | map 2] of `dim` each; each map is an attention of its own over the same values,
  a_1 and a_2, and the head's output is rms(a_1 - lam a_2) (1 - diff) with
  lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number a layer (vectors `lq1` .. `lk2` of
  `dim`), and rms(o) = o / sqrt(mean(o^2) + eps) over the head's `vdim` outputs, no gain;
* `values` = "keys": there is no Wv, the values are the keys as projected (before norm and
  rotation), so `vdim` = `dim`; "projected": v = Wv h (+ bv) of `vdim` a kv head;
* `qk_norm`: per head, q and k go through an RMS norm over `dim` with a gain of `dim` shared by
  all heads (`q.norm`, `k.norm`), before the rotation;
* `position`: a rotary encoding (its `pairing`, scaling and magnitude are the encoding's own);
* `mask`: {"kind": "causal"}, {"kind": "window", "size": n} (position i sees 0 <= i - j < n) or
  {"kind": "chunk", "size": n} (j <= i in the same chunk, floor(i / n) = floor(j / n), counted
  from position 0 of the request);
* `softcap` c > 0: score <- c tanh(score / c), after the scale;
* `sink` (a number): every softmax has one more key of that score, which has no value:
  p_j = exp(s_j) / (exp(sink) + sum exp(s_j')); 0 adds one to the denominator;
* `q_temp` = {"coef": c, "every": n}: the query at position p is multiplied by
  1 + c ln(floor((p + 1) / n) + 1), in 32-bit, behind norm and rotation;
* `gate`: the concatenated heads are multiplied by sigmoid(Wg h) before the output projection, a number
  an element (true, or "elements": Wg has heads vdim rows) or a number a head ("heads": Wg has heads rows).

All projections of h are one product into 32-bit rows; one kernel norms, rotates and stores
(queries for the attention kernel, keys and values into the request's page, whose row holds a
position's keys of all kv heads and maps and, position-contiguous, its values); one kernel does
the attention of all maps, their combination, the norm and the gate; the output projection adds
into the residual stream.  With a window or chunks only the last `size` positions are ever read,
so the cache manager may take back earlier pages.

Parameters: `hidden_size`, `heads`, `kv_heads`, `dim`, `vdim`, `maps`, `diff`, `values`, `bias`,
`qk_norm`, `eps`, `scale`, `softcap`, `sink`, `q_temp`, `mask`, `gate`, `position` (a PartSpec), `names`.
`forward(..., accumulate=False)` stores the 32-bit output instead of adding it (for a part that combines
several mixers' outputs itself).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE_F32, PackedMatrix
from .base import CacheBinding, CacheSpec, Mixer, TensorDecl, build_part, register_mixer

TILE_TOKENS = 16        # tokens of one request a tile of the matrix-core kernel holds


def first_seen(pos: int, mask: str, size: int) -> int:
    """The first position that position `pos` sees under a mask."""
    if mask == "window":
        return max(0, pos + 1 - size)
    if mask == "chunk":
        return pos // size * size
    return 0


def attention_tiles(ctx, mask: str, size: int) -> Optional[torch.Tensor]:
    """The step's tokens in tiles of up to 16 consecutive tokens of one request, int32 [n, 2] (first
    token, count) on the device, those that see the most positions first (they run longest, and a
    kernel ends with its last block); made once a step and mask.  None in a step of single tokens that
    may be replayed from a graph: every token is then a tile of its own, which the kernel knows without a list."""
    if ctx.decode_only:
        return None
    key = ("masked_attention_tiles", mask, size)
    tiles = ctx.shared.get(key)
    if tiles is None:
        rows = []
        for s in ctx.spans:
            for at in range(0, s.q_len, TILE_TOKENS):
                n = min(TILE_TOKENS, s.q_len - at)
                first = s.start_pos + at
                rows.append((first + n - first_seen(first, mask, size), s.q_start + at, n))
        if any(a < 0 or n < 1 or a + n > ctx.n_tokens for _, a, n in rows):
            raise ValueError("attention tiles: a span lies outside the tokens of the step")
        rows.sort(key=lambda r: -r[0])
        tiles = ctx.shared[key] = torch.tensor([(a, n) for _, a, n in rows], dtype=torch.int32).to(ctx.rt.device)
    return tiles


class MaskedAttention(Mixer):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.heads, self.kv_heads = int(p["hidden_size"]), int(p["heads"]), int(p["kv_heads"])
        self.dim, self.vdim, self.maps = int(p["dim"]), int(p["vdim"]), int(p.get("maps", 1))
        self.values = p.get("values", "projected")
        self.bias, self.qk_norm, self.gate = bool(p.get("bias", False)), bool(p.get("qk_norm", False)), bool(p.get("gate", False))
        if p.get("gate") not in (None, False, True, "elements", "heads"):
            raise ConfigError(f"gate {p.get('gate')!r} is not known (elements, heads)")
        self.gate_per_head = p.get("gate") == "heads"
        self.sink = None if p.get("sink") is None else float(p["sink"])
        temp = p.get("q_temp")
        self.q_temp = None if not temp else (float(temp["coef"]), int(temp["every"]))
        if self.q_temp is not None and self.q_temp[1] < 1:
            raise ConfigError(f"a query temperature every {self.q_temp[1]} positions")
        self.eps, self.scale = float(p.get("eps", 0.0)), float(p["scale"])
        self.softcap, self.diff = float(p.get("softcap") or 0.0), float(p.get("diff", 0.0))
        mask = p.get("mask") or {"kind": "causal"}
        self.mask, self.mask_size = mask.get("kind", "causal"), int(mask.get("size", 0))
        if self.heads % self.kv_heads:
            raise ConfigError(f"{self.heads} query heads are not a multiple of {self.kv_heads} key/value heads")
        if self.maps not in (1, 2):
            raise ConfigError(f"{self.maps} score maps a head: one, or two (differential attention)")
        if self.values not in ("projected", "keys"):
            raise ConfigError(f"values '{self.values}' are not known (projected, keys)")
        if self.values == "keys" and self.vdim != self.maps * self.dim:
            raise ConfigError(f"values that are the keys have their size: vdim {self.vdim}, keys of {self.maps * self.dim}")
        if self.mask not in ("causal", "window", "chunk") or (self.mask != "causal" and self.mask_size < 1):
            raise ConfigError(f"mask {mask!r} is not causal, a window or chunks of a size")
        if self.vdim > 512:
            raise ConfigError(f"values of {self.vdim} dims are more than the attention kernel's 512")
        self.position = build_part("position", p["position"]) if p.get("position") is not None else None
        self.rot = self.position.rotary_dim if self.position is not None else 0
        if self.rot > self.dim:
            raise ConfigError(f"{self.rot} rotated dims in keys of {self.dim}")
        names = p.get("names", {})
        base = prefix + names.get("scope", "mix.")
        self.n = {k: base + names.get(k, k) for k in ("q", "k", "v", "g", "o", "lq1", "lk1", "lq2", "lk2")}
        self.n_q, self.n_k = self.heads * self.maps, self.kv_heads * self.maps
        self.q_width, self.k_width, self.v_width = self.n_q * self.dim, self.n_k * self.dim, self.kv_heads * self.vdim
        self.o_width = self.heads * self.vdim
        # the columns of the fused projection: q, k, then v (unless the values are the keys), then the gate
        self.k_at = self.q_width
        self.v_at = self.k_at if self.values == "keys" else self.k_at + self.k_width
        self.g_at = self.k_at + self.k_width + (0 if self.values == "keys" else self.v_width)
        self.g_width = 0 if not self.gate else self.heads if self.gate_per_head else self.o_width
        self.proj_width = self.g_at + self.g_width
        self.lam = 0.0
        self.q_gain = self.k_gain = self.b_proj = None

    # ------------------------------------------------------------------ declarations
    def _projections(self) -> List[str]:
        return ["q", "k"] + (["v"] if self.values == "projected" else []) + (["g"] if self.gate else [])

    def tensors(self) -> List[TensorDecl]:
        n = self.n
        rows = {"q": self.q_width, "k": self.k_width, "v": self.v_width, "g": self.g_width}
        t = [TensorDecl(n[k], (rows[k], self.hidden)) for k in self._projections()]
        if self.bias:
            t += [TensorDecl(n[k] + ".b", (rows[k],), "bias") for k in self._projections() if k != "g"]
        if self.qk_norm:
            t += [TensorDecl(n["q"] + ".norm", (self.dim,), "gain"), TensorDecl(n["k"] + ".norm", (self.dim,), "gain")]
        if self.maps == 2:
            t += [TensorDecl(n[k], (self.dim,), "bias") for k in ("lq1", "lk1", "lq2", "lk2")]
        t.append(TensorDecl(n["o"], (self.hidden, self.o_width)))
        return t

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(entries=1, heads=1, head_dim=self.k_width + self.v_width,
                         window=self.mask_size if self.mask != "causal" else 0)

    def load(self, store, rt) -> None:
        n = self.n
        names = self._projections()
        self.w_proj = rt.k.prepare_weight(store.fused_matrix([n[k] for k in names]))
        if self.bias:
            parts = [store.vector(n[k] + ".b").float() if k != "g" else torch.zeros(self.g_width, device=rt.device) for k in names]
            self.b_proj = torch.cat(parts).contiguous()
        if self.qk_norm:
            self.q_gain, self.k_gain = store.vector(n["q"] + ".norm"), store.vector(n["k"] + ".norm")
        if self.maps == 2:
            lq1, lk1, lq2, lk2 = (store.vector(n[k]).float() for k in ("lq1", "lk1", "lq2", "lk2"))
            # one number a layer, in 32-bit, once
            self.lam = float((torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())).item()) + self.diff
        self.w_o = rt.k.prepare_weight(store.matrix(n["o"]))
        store.forget(n["o"])
        if self.position is not None:
            self.position.load(store, rt)

    SPAN_STEP = 512      # the positions a decoding step's longest row sees, rounded up to this: part of the step's shape

    def decode_shape(self, positions):
        """Without a window or chunks the blocks of positions that run side by side in a step of few tokens
        depend on how long the contexts are: a captured graph is replayed for steps whose longest row sees as many."""
        if self.mask != "causal":
            return None
        return ("masked_attention_span", -(-(max(positions) + 1) // self.SPAN_STEP) * self.SPAN_STEP)

    # ------------------------------------------------------------------ the step
    def finishes_following_norm(self, ctx) -> bool:
        """In steps of many rows the output projection's last kernel also writes the norm behind it."""
        return isinstance(self.w_o, PackedMatrix) and ctx.rt.k.gemm_then_norm_ok(ctx.n_tokens, self.hidden, self.o_width)

    def forward(self, ctx, binding: CacheBinding, h, residual, following=None, accumulate: bool = True) -> None:
        k, T = ctx.rt.k, h.shape[0]
        group = ctx.cache.group(binding.group)
        (cache,) = group.layer(binding.index)
        proj = ctx.ws.take((T, self.proj_width), torch.float32)
        k.gemm(h, self.w_proj, proj, self.b_proj, MODE_STORE_F32)
        if self.position is not None:
            table, neighbours, magnitude = self.position.tables(ctx), self.position.pairing == "neighbours", self.position.magnitude
        else:
            table, neighbours, magnitude = ctx.no_rotation(), False, 1.0
        q = ctx.ws.take((T, self.q_width), ctx.rt.dtype)
        k.heads_prepare(proj, 0, self.n_q, self.k_at, self.n_k, self.v_at, self.v_width, self.dim, self.q_gain, self.k_gain,
                        self.eps, self.rot, neighbours, magnitude, table, ctx.positions, ctx.seq_rows, group.block_table, cache,
                        group.page_size, q, binding.writes, q_temp=self.q_temp)
        att = ctx.ws.take((T, self.o_width), ctx.rt.dtype)
        tiles = None
        if k.masked_attention_uses_mfma(self.heads, self.kv_heads, self.maps, self.dim, self.vdim, group.page_size):
            tiles = attention_tiles(ctx, self.mask, self.mask_size)
        span = 0
        if self.mask == "causal":
            span = ctx.decode_shapes.get("masked_attention_span", 0) if ctx.decode_only else max(s.start_pos + s.q_len for s in ctx.spans)
        k.masked_attention(q, cache, group.block_table, ctx.positions, ctx.seq_rows, att, self.heads, self.kv_heads, self.maps,
                           self.dim, self.vdim, group.page_size, self.mask, self.mask_size, self.scale, self.softcap, self.lam,
                           1.0 - self.diff, self.eps, gate=proj[:, self.g_at:] if self.gate else None, tiles=tiles,
                           sink=self.sink, gate_per_head=self.gate_per_head, span=span)
        if not accumulate:          # the output itself, for a part that sums and norms on its own
            k.gemm(att, self.w_o, residual, None, MODE_STORE_F32)
            return
        k.gemm(att, self.w_o, residual, None, MODE_ADD_F32,
               following_norm=None if following is None else following.as_argument())


register_mixer("masked_attention", MaskedAttention)
