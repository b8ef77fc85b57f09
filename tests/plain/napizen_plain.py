"""The Napizen decoder, slowly and plainly: whole sequences, no cache, float64.

One function per mechanism, written from the design's equations and sharing nothing with the
engine.  A model is (cfg, W): config.json as a dict and the tensors by name as float64.

Notation: h is a [T, width] input, positions are 0 .. T - 1, sigma is the logistic function.

    ln(x, g)         = (x - mean x) / sqrt(var x + eps) * g          (var: mean of squared deviations)
    rms(x, g)        = x / sqrt(mean(x^2) + eps) * g
    layer            : x <- ln(alpha x + mixer(x), g1);  x <- ln(alpha x + ff(x), g2)
    latent attention : q = Wq h = per head [qn | qr];  [c_raw | kr] = Wdkv h;  c = rms(c_raw, gkv)
                       kn = Wuk c; v = Wuv c (per head);  qr, kr turned by position in pairs (2k, 2k + 1)
                       score(i, j) = (qn_i . kn_j + qr_i . kr_j) scale, j <= i
                       p_ij = exp(score_ij) / (exp(sink) + sum_j' exp(score_ij'))     (sink: a number a head)
                       out = Wo [head a: sigma(Wg h)_a sum_j p_ij v_j]
    gated unit       : Wd (silu(Wg h) * (Wu h))
    experts          : s = sigma(Wr h); choice = s + correction; groups of neighbours ranked by the sum of
                       their two largest choices, `keep` groups stay; the `top` largest choices among them;
                       weights s_e / (sum of the chosen s + 1e-20) * router scale
    output           : z = head ln(x, g_final);  logits = cap tanh(z / cap)
"""
import json
import math
import os

import torch


def load_plain(model_dir):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    W = {k: v.double() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, W


# --------------------------------------------------------------------------- small pieces
def layer_norm(x, gain, eps):
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * gain


def rms(x, gain, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


def sigma(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigma(z)


# --------------------------------------------------------------------------- rotation
def pair_frequencies(rot):
    """The frequency of every pair, with the ramp between divided and kept frequencies, and the factor
    on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * k / dims) for k in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = sc["factor"], sc["original"]

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    out = []
    for k, fk in enumerate(f):
        ramp = min(max((k - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fk / factor * ramp + fk * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_neighbours(v, positions, rot):
    """Places (2k, 2k + 1) of the first rot['dims'] places of v [T, ..., n] turned by position * f_k;
    the rest pass."""
    f, mag = pair_frequencies(rot)
    out = v.clone()
    shape = [-1] + [1] * (v.dim() - 2)
    for k, fk in enumerate(f):
        angle = positions.double() * fk
        c, s = (torch.cos(angle) * mag).view(shape), (torch.sin(angle) * mag).view(shape)
        a, b = v[..., 2 * k], v[..., 2 * k + 1]
        out[..., 2 * k] = a * c - b * s
        out[..., 2 * k + 1] = b * c + a * s
    return out


# --------------------------------------------------------------------------- latent attention
def latent_attention(W, p, c, h, eps, first_position=0):
    T, H = h.shape[0], c["heads"]
    dim, rot, vdim, rank = c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    pos = torch.arange(T) + first_position
    q = (h @ W[p + "q"].T).view(T, H, dim + rot)
    down = h @ W[p + "dkv"].T
    latent = rms(down[:, :rank], W[p + "dkv.norm"], eps)
    shared_key = down[:, rank:]
    q_plain, q_turned = q[..., :dim], q[..., dim:]
    if rot:
        q_turned = rotate_neighbours(q_turned, pos, c["rot"])
        shared_key = rotate_neighbours(shared_key, pos, c["rot"])
    keys = (latent @ W[p + "uk"].T).view(T, H, dim)
    values = (latent @ W[p + "uv"].T).view(T, H, vdim)
    gate = sigma(h @ W[p + "g"].T)                       # [T, H]
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for i in range(T):
        for a in range(H):
            s = (keys[:i + 1, a] @ q_plain[i, a] + shared_key[:i + 1] @ q_turned[i, a]) * c["scale"]
            sink = W[p + "sink"][a]
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            out[i, a] = (e @ values[:i + 1, a]) / (e.sum() + torch.exp(sink - m)) * gate[i, a]
    return out.reshape(T, H * vdim) @ W[p + "o"].T


# --------------------------------------------------------------------------- feed-forwards
def gated_unit(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def choose_experts(scores, correction, top, groups, keep):
    """scores [E] -> the chosen experts of one token."""
    E = scores.numel()
    choice = (scores + correction).tolist()
    size = E // groups
    ranked = []
    for g in range(groups):
        members = sorted(choice[g * size:(g + 1) * size], reverse=True)
        ranked.append((-sum(members[:2]), g))
    kept = {g for _, g in sorted(ranked)[:keep]}
    allowed = [e for e in range(E) if e // size in kept]
    return sorted(allowed, key=lambda e: (-choice[e], e))[:top]


def routed_ff(W, p, c, h, forced=None, slack=0.0):
    """forced: for every token the experts another implementation chose.  They are taken instead of this
    one's own choice, after a check that they are a choice one may arrive at: the one made when each
    of them scores `slack` higher (a close call that rounding decides the other way)."""
    r = c["router"]
    s = sigma(h @ W[p + "router"].T)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = choose_experts(s[t], W[p + "correction"], r["top"], groups["count"], groups["keep"])
        if forced is not None and sorted(forced[t]) != sorted(chosen):
            lifted = s[t].clone()
            lifted[list(forced[t])] += slack
            close = choose_experts(lifted, W[p + "correction"], r["top"], groups["count"], groups["keep"])
            assert sorted(close) == sorted(forced[t]), f"{p} token {t}: {forced[t]} is no close call of {chosen}"
            chosen = list(forced[t])
        total = sum(s[t, e] for e in chosen) + 1e-20
        for e in chosen:
            out[t] += s[t, e] / total * r["scale"] * gated_unit(W, f"{p}e{e}.", h[t:t + 1])[0]
    return out


def feed_forward(W, p, c, h, forced=None, slack=0.0):
    return gated_unit(W, p, h) if c["kind"] == "dense" else routed_ff(W, p, c, h, forced, slack)


# --------------------------------------------------------------------------- the model
def residual_stream(cfg, W, tokens, after_every_layer=None, forced=None, slack=0.0):
    """forced: {layer: the experts chosen for every token} for layers with experts (see routed_ff)."""
    eps, alpha = cfg["norm"]["eps"], cfg.get("postln_alpha", 1.0)
    x = W["embed"][torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = layer_norm(alpha * x + latent_attention(W, p + "mix.", layer["mixer"], x, eps), W[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = layer_norm(alpha * x + feed_forward(W, p + "mlp.", layer["mlp"], x, (forced or {}).get(i), slack), W[p + "norm2"], eps)
        if after_every_layer is not None:
            after_every_layer.append(x.clone())
    return x


def forward_logits(cfg, W, tokens, forced=None, slack=0.0):
    x = residual_stream(cfg, W, tokens, None, forced, slack)
    z = layer_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


def greedy_generate(cfg, W, prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        row = forward_logits(cfg, W, seq)[-1].float()
        best = max(range(row.numel()), key=lambda v: (float(row[v]), v))
        out.append(best)
        seq.append(best)
    return out
