"""A selective state-space mixer in its recurrent form (the "state-space duality" layer of Mamba-2-like
models), with its state in the cache manager's state slots.

From the input h one product gives [z | x | B | C | dt] with inner = heads * vdim columns of z and of x,
groups * state of B and of C, and heads of dt.  x, B and C together pass a causal convolution of `conv`
taps per channel with a bias, then silu.  Per head a (head a reads B and C of group a // (heads / groups)):

    dt_t = softplus(dt_t + dt_bias_a),  S_t = exp(-exp(A_log_a) dt_t) S_(t-1) + dt_t B_t x_t^T,
    y_t = S_t^T C_t + D_a x_t                      (S: state x vdim, zero before the first token)

and the output is Wo (rms in `norm_groups` equal parts of (y silu(z)) * gain).  The product's rows, the
convolution's result, dt, the decays, the state and the norm are 32-bit; a request's state row holds S
and the convolution's last conv - 1 inputs, twice: the state behind position p in copy p & 1, so that a
decoding step reads one copy and writes the other and may be run again (the engine runs a step once
before it captures it into a graph) with the same result.  Where the walk of one chain a request would leave most of the chip idle, a long
stretch of a request's tokens in one step runs in segments side by side, each from a zero state but the first,
whose end states are then folded in order and whose carried-in states' share is added to the outputs: the same
sums in another order.

Parameters: `hidden_size`, `heads`, `vdim`, `state`, `groups`, `conv`, `norm_groups`, `eps`, `names` (the
tensors' names under the prefix: scope "mix.", in, conv, dt_bias, A_log, D, norm, o; the convolution's
bias is the name + ".b").  `forward(..., accumulate=False)` stores the 32-bit output instead of adding it.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE_F32
from .base import CacheBinding, Mixer, StateSpec, TensorDecl, register_mixer
from .recurrent import step_spans

SEGMENT = 128           # the fewest tokens a segment of a long stretch (a request's tokens of one step) holds
TARGET_BLOCKS = 2048    # blocks the segmented scan launches: eight a compute unit
FEW_BLOCKS = 256        # a walk of one chain a request that launches more blocks than this is left as it is


def step_segments(ctx, blocks_a_stretch: int):
    """The stretches of a step cut into segments, for the scan that runs a long stretch's segments side by side:
    (segs int32 [n, 4] = (slot, first token, tokens, whether the request's first), spans5 int32 [requests, 5] =
    (slot, first token, tokens, first segment, segments), the longest segment's tokens) on the device, made once a step and scan shape.  A walk
    of one chain a stretch launches `blocks_a_stretch` blocks a stretch; stretches are cut into as many equal
    segments (of SEGMENT tokens at least) as brings the launch to TARGET_BLOCKS.  None where that is one segment
    a stretch, where the walk of one chain a request fills the chip by itself (measured: 512 blocks walk 2,048
    tokens in 556 us, in four segments each they take 611 with the two further launches; 256 blocks take 533 us
    and, in eight segments, 337), and in steps of single tokens: one walk a request then, whose sums do not depend
    on the cuts."""
    if ctx.decode_only or blocks_a_stretch * len(ctx.spans) > FEW_BLOCKS:
        return None
    most = TARGET_BLOCKS // max(1, blocks_a_stretch * len(ctx.spans))
    if most < 2 or all(s.q_len < 2 * SEGMENT for s in ctx.spans):
        return None
    key = ("state_space_segments", most)
    made = ctx.shared.get(key)
    if made is None:
        segs, spans5 = [], []
        for s in ctx.spans:
            n = max(1, min(most, s.q_len // SEGMENT))
            size = -(-s.q_len // n)
            spans5.append([s.slot, s.q_start, s.q_len, len(segs), -(-s.q_len // size)])
            for at in range(0, s.q_len, size):
                segs.append([s.slot, s.q_start + at, min(size, s.q_len - at), 1 if at == 0 else 0])
        made = ctx.shared[key] = (torch.tensor(segs, dtype=torch.int32).to(ctx.rt.device),
                                  torch.tensor(spans5, dtype=torch.int32).to(ctx.rt.device), max(r[2] for r in segs))
    return made


class SelectiveStateSpace(Mixer):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.heads, self.vdim = int(p["hidden_size"]), int(p["heads"]), int(p["vdim"])
        self.n_state, self.groups, self.taps = int(p["state"]), int(p["groups"]), int(p["conv"])
        self.norm_groups, self.eps = int(p.get("norm_groups", 1)), float(p["eps"])
        if self.groups < 1 or self.heads % self.groups:
            raise ConfigError(f"{self.heads} heads do not share {self.groups} groups of B and C equally")
        if self.taps < 1:
            raise ConfigError(f"a convolution of {self.taps} taps")
        if not 1 <= self.n_state <= 256:
            raise ConfigError(f"a state of {self.n_state} rows a head: the scan's kernel takes 1 to 256")
        self.inner = self.heads * self.vdim
        if self.norm_groups < 1 or self.inner % self.norm_groups:
            raise ConfigError(f"{self.inner} channels are not normed in {self.norm_groups} equal parts")
        self.bc = self.groups * self.n_state
        self.channels = self.inner + 2 * self.bc                   # what the convolution sees: x, B, C
        self.proj_width = 2 * self.inner + 2 * self.bc + self.heads
        self.tail_at = self.heads * self.n_state * self.vdim       # a copy of the state: S, then the kept inputs
        self.copy_elems = self.tail_at + (self.taps - 1) * self.channels
        names = p.get("names", {})
        base = prefix + names.get("scope", "mix.")
        self.n = {k: base + names.get(k, k) for k in ("in", "conv", "dt_bias", "A_log", "D", "norm", "o")}

    def tensors(self) -> List[TensorDecl]:
        n = self.n
        return [TensorDecl(n["in"], (self.proj_width, self.hidden)),
                TensorDecl(n["conv"], (self.channels, self.taps)), TensorDecl(n["conv"] + ".b", (self.channels,), "bias"),
                TensorDecl(n["dt_bias"], (self.heads,), "bias"), TensorDecl(n["A_log"], (self.heads,), "bias"),
                TensorDecl(n["D"], (self.heads,), "bias"), TensorDecl(n["norm"], (self.inner,), "gain"),
                TensorDecl(n["o"], (self.hidden, self.inner))]

    def state_spec(self) -> StateSpec:
        return StateSpec(2 * self.copy_elems)

    def load(self, store, rt) -> None:
        n = self.n
        self.w_in = rt.k.prepare_weight(store.matrix(n["in"]))
        store.forget(n["in"])
        self.conv_w, self.conv_b = store.matrix(n["conv"]), store.vector(n["conv"] + ".b")
        self.dt_bias, self.a_log, self.d_skip = store.vector(n["dt_bias"]), store.vector(n["A_log"]), store.vector(n["D"])
        self.gain = store.vector(n["norm"])
        self.w_o = rt.k.prepare_weight(store.matrix(n["o"]))
        store.forget(n["o"])

    def forward(self, ctx, binding: CacheBinding, h, out, accumulate: bool = True) -> None:
        k, T = ctx.rt.k, h.shape[0]
        state = ctx.cache.state(binding.state_index)
        f32 = torch.float32
        proj = ctx.ws.take((T, self.proj_width), f32)
        k.gemm(h, self.w_in, proj, None, MODE_STORE_F32)
        z, xbc, raw = proj[:, :self.inner], proj[:, self.inner:self.inner + self.channels], proj[:, self.inner + self.channels:]
        u, terms = ctx.ws.take((T, self.channels), f32), ctx.ws.take((T, self.heads, 2), f32)
        k.state_conv(xbc, self.conv_w, self.conv_b, state, self.copy_elems, self.tail_at, ctx.positions, ctx.seq_rows, u,
                     silu=True, raw=raw, dt_bias=self.dt_bias, a_log=self.a_log, terms=terms)
        y = ctx.ws.take((T, self.inner), f32)
        k.state_space_scan(u, terms, self.d_skip, state, self.copy_elems, self.tail_at, step_spans(ctx), ctx.positions,
                           ctx.seq_rows, xbc, y, self.heads, self.groups, self.vdim, self.n_state, self.taps,
                           segments=step_segments(ctx, self.heads * -(-self.vdim // 8)))
        normed = ctx.ws.take((T, self.inner), ctx.rt.dtype)
        k.gated_group_norm(y, z, self.gain, self.eps, normed, self.norm_groups)
        k.gemm(normed, self.w_o, out, None, MODE_ADD_F32 if accumulate else MODE_STORE_F32)


register_mixer("selective_state_space", SelectiveStateSpace)
