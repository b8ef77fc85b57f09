"""Small Zugutar configurations and weights for the tests: sizes that differ between the models and
between the layers of a model (query/key size against value size, heads of the two sides of a pair,
state against value size), values of 1 (one head, one expert a token, one group, one tap, a loop that
runs once), every expert chosen, no shared expert, no feed-forward, fewer rotated places than a head
holds, widths that no matrix-core product takes and sizes that the matrix-core attention takes, states of
more rows than a lane holds at once, loops that start at the first layer or end at the last, and
weights drawn so that the mechanisms matter: decays from a step to hundreds of steps, scores of the
size of the sink's, routers whose scores spread over (0, 1)."""
import json
import os

import torch


def left(heads, kv_heads, dim, vdim, dims=None, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale else dim ** -0.5}
    if dims != 0:
        m["rot"] = {"base": base, "dims": dim if dims is None else dims}
    return m


def right(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def pair(l, r):
    return {"type": "parallel", "mixer": {"left": l, "right": r}}


def att(heads, kv_heads, dim, vdim, temp=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale else dim ** -0.5}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, loop=None, eps=1e-5, logit_scale=None):
    cfg = {"architecture": "Zugutar", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


MODELS = {
    # nothing a multiple of 16: three heads on one key/value head beside three state-space heads of five dims and a
    # state of seven rows, four of ten places rotated, pages of 8; a loop from the first layer on, three passes; a
    # layer without a feed-forward; two of five experts; a temperature every five positions
    "A": dict(cfg=config(40, 131, [
        layer(pair(left(3, 1, 10, 6, dims=4, base=100.0), right(3, 5, 7, groups=1, conv=3, norm_groups=3)), moe(5, 2, 24, shared=16)),
        layer(att(4, 2, 6, 10, temp=(0.7, 5)), None),
        layer(pair(left(2, 2, 12, 4, dims=12, base=30.0), right(4, 3, 5, groups=2, conv=2, norm_groups=1)), moe(3, 1, 8))],
        loop=(0, 2, 3), eps=1e-5, logit_scale=0.5), page=8, seed=3),
    # what the matrix cores take: heads in groups on pages of 64, keys of 32 and 64, a state of 64 rows in two
    # groups; every expert chosen; a loop of one layer in the middle, twice; no logit scale
    "B": dict(cfg=config(128, 300, [
        layer(pair(left(8, 2, 32, 32, base=1000000.0), right(4, 32, 64, groups=2, conv=4, norm_groups=4)), moe(4, 4, 64, shared=96)),
        layer(att(16, 16, 64, 16, temp=(0.5, 64)), moe(8, 2, 32, shared=32)),
        layer(pair(left(4, 4, 64, 48, dims=32), right(8, 16, 32, groups=8, conv=4, norm_groups=2)), moe(4, 1, 64))],
        loop=(1, 2, 2), eps=1e-6), page=64, seed=8),
    # a state of more rows than sixteen lanes hold at eight each, two taps, as many groups as heads, one expert a
    # token, no loop, the attention layer first, a temperature at every position, pages of 16
    "C": dict(cfg=config(64, 257, [
        layer(att(2, 1, 24, 40, temp=(0.25, 1)), moe(6, 1, 32, shared=8)),
        layer(pair(left(4, 4, 16, 16, dims=8, base=500.0), right(2, 24, 130, groups=2, conv=2, norm_groups=2)), moe(5, 3, 16, shared=24)),
        layer(att(5, 5, 8, 8), None)],
        eps=1e-4, logit_scale=2.0), page=16, seed=5),
    # one head each, one tap (no convolution to remember), a loop that ends with the last layer and runs once
    # more than once only in name (times 1), no rotation on the left side, no temperature
    "D": dict(cfg=config(80, 140, [
        layer(pair(left(1, 1, 24, 40, dims=0), right(1, 40, 16, groups=1, conv=1, norm_groups=1)), moe(8, 3, 24)),
        layer(pair(left(5, 1, 8, 16, dims=2, base=7.0), right(5, 8, 24, groups=1, conv=5, norm_groups=5)), moe(2, 2, 40, shared=40))],
        loop=(1, 2, 1), eps=1e-6, logit_scale=0.25), page=16, seed=12),
}


def draw_weights(cfg, seed):
    """name -> float32 tensor of values that bfloat16 holds exactly (both compute dtypes and the
    plain implementation then start from the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def matrix(name, *shape, gain=1.0):
        W[name] = torch.randn(*shape, generator=g) * (gain / shape[-1] ** 0.5)

    def vector(name, *shape, mean=0.0, std=0.1):
        W[name] = torch.randn(*shape, generator=g) * std + mean

    def heads_attention(p, m, gate_rows):
        H, G = m["heads"], m["kv_heads"]
        matrix(p + "q", H * m["dim"], width, gain=1.5)
        matrix(p + "k", G * m["dim"], width, gain=1.5)
        matrix(p + "v", G * m["vdim"], width)
        matrix(p + "g", gate_rows, width, gain=2.0)
        matrix(p + "o", width, H * m["vdim"])

    width = cfg["width"]
    # small against what the layers add: the next token then depends on the earlier ones, not on the last alone
    W["embed"] = torch.randn(cfg["vocab"], width, generator=g) * 0.3
    vector("final.norm", width)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vector(p + "norm1", width)
        if L["type"] == "attention":
            heads_attention(p + "mix.", m, m["heads"] * m["vdim"])
        else:
            l, r = m["left"], m["right"]
            heads_attention(p + "mix.left.", l, l["heads"])
            vector(p + "mix.left.q.norm", l["dim"], mean=1.0, std=0.2)
            vector(p + "mix.left.k.norm", l["dim"], mean=1.0, std=0.2)
            inner, bc = r["heads"] * r["vdim"], r["groups"] * r["state"]
            matrix(p + "mix.right.in", 2 * inner + 2 * bc + r["heads"], width, gain=1.5)
            W[p + "mix.right.conv"] = torch.randn(inner + 2 * bc, r["conv"], generator=g) * 0.5
            vector(p + "mix.right.conv.b", inner + 2 * bc, std=0.2)
            vector(p + "mix.right.dt_bias", r["heads"], mean=-1.0, std=1.0)
            # decays from a step (A_log near 0.5) to hundreds of steps (near -5)
            W[p + "mix.right.A_log"] = torch.rand(r["heads"], generator=g) * 5.5 - 5.0
            vector(p + "mix.right.D", r["heads"], mean=1.0, std=0.3)
            vector(p + "mix.right.norm", inner, mean=1.0)
            matrix(p + "mix.right.o", width, inner)
            vector(p + "mix.left.out", width, mean=1.0)
            vector(p + "mix.right.out", width, mean=1.0)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        E = mlp["router"]["experts"]
        matrix(p + "mlp.router", E, width, gain=2.0)
        units = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(E)]
        if mlp.get("shared"):
            units.append(("shared.", mlp["shared"]["ff"]))
            matrix(p + "mlp.shared.sg", 1, width, gain=2.0)
        for scope, ff in units:
            matrix(p + "mlp." + scope + "gate", ff, width, gain=2.0)
            matrix(p + "mlp." + scope + "up", ff, width, gain=2.0)
            matrix(p + "mlp." + scope + "down", width, ff)
    return {k: v.to(torch.bfloat16).float() for k, v in W.items()}


def write_model(path, cfg, W):
    from axon_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path, exist_ok=True)
    write_safetensors(os.path.join(path, "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in W.items()], {"format": "pt"})
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return path


def make(path, name):
    m = MODELS[name]
    return write_model(path, m["cfg"], draw_weights(m["cfg"], m["seed"]))
