"""Small Napizen configurations and weights for the tests: sizes that differ between the models and
between the layers of a model (query/key size against value size, latent against width), values of 1
(one head, one expert a token, groups of one expert, no stretch of the stream, no scale), widths that
no matrix-core product takes and heads in sixteens that the matrix-core attention takes, fewer rotated
dims than the rotated part holds, frequencies ramped and not, and weights drawn so that the mechanisms
matter: sinks of the size of the scores, corrections large enough to turn a choice score negative.  The
attention's `scale` keeps a score's spread near 3 under these weights: 16 bits of cache cannot carry
weights much sharper."""
import json
import os

import torch


def att(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, scale=0.5, dims=None, scaling=None):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot, "scale": scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, scale=1.0):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config(width, vocab, layers, eps=1e-6, alpha=1.5, scale=4.0, softcap=30.0):
    cfg = {"architecture": "Napizen", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps},
           "postln_alpha": alpha, "vocab": vocab, "width": width}
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


MODELS = {
    # nothing a multiple of 16: three heads, a latent of 20, pages of 8; three groups of two experts of which
    # two stay; ramped frequencies; a layer without a feed-forward
    "A": dict(cfg=config(48, 131, [
        layer(att(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, base=100.0, scaling=(4.0, 16, 8.0, 1.0)), moe(6, 2, 24, (3, 2), 2.5)),
        layer(att(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, base=100.0, scaling=(4.0, 16, 8.0, 1.0)), dense(80)),
        layer(att(heads=2, dim=12, rot_dim=6, vdim=4, kv_rank=16, base=30.0, scale=0.3), None)],
        eps=1e-5, alpha=1.7, scale=3.0, softcap=8.0), page=8, seed=3),
    # what the matrix-core attention takes: sixteen heads, latents in sixteens, key rows in chunks of 32, pages
    # of 64; every expert chosen (no groups); no stretch, no scale, no bend
    "B": dict(cfg=config(128, 300, [
        layer(att(heads=16, dim=32, rot_dim=32, vdim=16, kv_rank=96, base=1000000.0, scaling=(8.0, 64, 32.0, 1.0), scale=0.2), moe(4, 4, 64)),
        layer(att(heads=16, dim=32, rot_dim=32, vdim=16, kv_rank=96, base=1000000.0, scaling=(8.0, 64, 32.0, 1.0), scale=0.2), dense(256))],
        eps=1e-6, alpha=1.0, scale=1.0, softcap=0), page=64, seed=8),
    # two attention layers of other sizes (two page pools): thirty-two heads over a small latent, sixteen over
    # a large one; groups of one expert each; one expert a token; fewer rotated dims than the rotated part holds
    "C": dict(cfg=config(64, 257, [
        layer(att(heads=32, dim=8, rot_dim=32, vdim=8, kv_rank=32, dims=16, base=500.0, scale=0.4), moe(8, 2, 32, (8, 3), 1.0)),
        layer(att(heads=16, dim=16, rot_dim=64, vdim=24, kv_rank=192, base=10000.0, scaling=(2.0, 32, 4.0, 0.5), scale=0.25), moe(5, 1, 16, (1, 1), 0.5))],
        eps=1e-4, alpha=2.2, scale=9.0, softcap=50.0), page=64, seed=5),
    # one head, a rotated part of two dims, pages of 16, two groups of which one stays, three of its four experts
    "D": dict(cfg=config(80, 140, [
        layer(att(heads=1, dim=24, rot_dim=2, vdim=40, kv_rank=24, base=7.0, scale=0.25), moe(8, 3, 24, (2, 1), 1.25)),
        layer(att(heads=5, dim=8, rot_dim=8, vdim=16, kv_rank=12, base=10000.0, scaling=(16.0, 8, 2.0, 1.0), scale=0.35), dense(96)),
        layer(att(heads=1, dim=24, rot_dim=2, vdim=40, kv_rank=24, base=7.0, scale=0.25), moe(8, 3, 24, (2, 1), 1.25))],
        eps=1e-6, alpha=0.8, scale=2.0, softcap=12.0), page=16, seed=12),
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

    width = cfg["width"]
    W["embed"] = torch.randn(cfg["vocab"], width, generator=g)
    vector("final.norm", width, mean=1.0)
    matrix("head", cfg["vocab"], width, gain=2.0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H = m["heads"]
        vector(p + "norm1", width, mean=1.0)
        matrix(p + "mix.q", H * (m["dim"] + m["rot_dim"]), width, gain=1.5)
        matrix(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], width)
        vector(p + "mix.dkv.norm", m["kv_rank"], mean=1.0)
        matrix(p + "mix.uk", H * m["dim"], m["kv_rank"], gain=1.5)
        matrix(p + "mix.uv", H * m["vdim"], m["kv_rank"])
        vector(p + "mix.sink", H, mean=0.5, std=1.0)              # of the size of the scores: leaving it out shows
        matrix(p + "mix.g", H, width, gain=2.0)
        matrix(p + "mix.o", width, H * m["vdim"])
        mlp = L.get("mlp")
        if mlp is None:
            continue
        vector(p + "norm2", width, mean=1.0)
        if mlp["kind"] == "dense":
            units = [("", mlp["ff"])]
        else:
            E = mlp["router"]["experts"]
            matrix(p + "mlp.router", E, width, gain=2.0)
            vector(p + "mlp.correction", E, std=0.7)              # some choice scores go below zero
            units = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(E)]
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
