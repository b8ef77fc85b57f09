"""The Zugutar decoder, slowly and plainly: whole sequences, no cache, float64.

One function per mechanism, written from the design's equations and sharing nothing with the
engine.  A model is (cfg, W): config.json as a dict and the tensors by name as float64.

Notation: h is a [T, width] input, positions are 0 .. T - 1, sigma is the logistic function,
rms(x) = x / sqrt(mean(x^2) + eps).

    layer            : h = rms(x) (1 + g1);  x <- x + mixer(h) + ff(h)       (both sublayers read h)
    loop             : layers start .. stop - 1 run `times` times; before every pass but the first
                       x <- x + x0 (x0 the embedding's rows)
    attention        : q, k, v = Wq h, Wk h, Wv h; query head a reads key/value head a // (H / G);
                       q_i <- q_i (1 + coef ln(floor((i + 1) / every) + 1));  s_ij = q_i . k_j scale, j <= i;
                       softmax; the heads side by side times sigma(Wg h); Wo
    paired mixer     : (rms(left(h)) gl + rms(right(h)) gr) / 2
      left           : q, k per head rms-normed with a gain shared by the heads, the first `dims` places
                       turned by position in pairs (i, i + dims / 2); p_ij = exp(s_ij) / (1 + sum_j' exp(s_ij'));
                       head a times sigma(Wg h)_a; Wo
      right          : [z | x | B | C | dt] = Win h; (x, B, C) <- silu(causal conv + bias);
                       dt <- softplus(dt + dt_bias);  S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T;
                       y_t = S_t^T C_t + D x_t;  rms in equal parts of (y silu(z)) times a gain; Wo
    experts          : s = sigma(Wr h); the `top` largest; out = sum_e expert_e(s_e h) + sigma(w_sg . h) shared(h)
    output           : logits = embed rms(x) (1 + g) logit_scale
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
def unit(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigma(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigma(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- rotation
def rotate_halves(v, positions, rot):
    """v [T, heads, dim]: the first rot.dims places of every head turn, place i with place i + dims / 2."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    out = v.clone()
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a = positions.double() * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, w = v[..., i], v[..., i + half]
        out[..., i] = u * c - w * s
        out[..., i + half] = w * c + u * s
    return out


# --------------------------------------------------------------------------- attention
def heads_attention(q, k, v, scale, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; causal; `sink`: one is added to the softmax's
    denominator (a key of score 0 that has no value)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=torch.float64)
    for a in range(H):
        g = a // (H // G)
        for i in range(T):
            s = (k[:i + 1, g] @ q[i, a]) * scale
            m = max(float(s.max()), 0.0) if sink else float(s.max())
            e = torch.exp(s - m)
            den = e.sum() + (math.exp(-m) if sink else 0.0)
            out[i, a] = (e / den) @ v[:i + 1, g]
    return out


def plain_attention(W, p, c, h, first_position=0):
    """The mixer 'attention': no rotation, a query temperature by position, a gate on every element."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, G, d)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    temp = c.get("q_temp")
    if temp:
        pos = torch.arange(first_position, first_position + T)
        steps = torch.div(pos + 1, int(temp["every"]), rounding_mode="floor").double()
        q = q * (1.0 + float(temp["coef"]) * torch.log(steps + 1.0))[:, None, None]
    o = heads_attention(q, k, v, float(c["scale"]), sink=False).reshape(T, H * dv)
    return (o * sigma(h @ W[p + "g"].T)) @ W[p + "o"].T


def left_attention(W, p, c, h, eps, first_position=0):
    """The paired mixer's left side: normed and turned queries and keys, a sink, a gate a head."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    pos = torch.arange(first_position, first_position + T)
    q = unit((h @ W[p + "q"].T).view(T, H, d), eps) * W[p + "q.norm"]
    k = unit((h @ W[p + "k"].T).view(T, G, d), eps) * W[p + "k.norm"]
    v = (h @ W[p + "v"].T).view(T, G, dv)
    rot = c.get("rot")
    if rot and int(rot["dims"]) > 0:
        q, k = rotate_halves(q, pos, rot), rotate_halves(k, pos, rot)
    o = heads_attention(q, k, v, float(c["scale"]), sink=True)
    o = o * sigma(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T


# --------------------------------------------------------------------------- the state-space side
def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x])
    out = b.expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * w[:, j]
    return out


def state_space(W, p, c, h, eps):
    T = h.shape[0]
    H, P, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
    inner = H * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * dt)             # [T, H]
    y = torch.zeros(T, H, P, dtype=torch.float64)
    for a in range(H):
        g = a // (H // G)
        S = torch.zeros(N, P, dtype=torch.float64)
        for t in range(T):
            S = decay[t, a] * S + dt[t, a] * torch.outer(B[t, g], x[t, a])
            y[t, a] = S.T @ C[t, g] + W[p + "D"][a] * x[t, a]
    y = y.reshape(T, inner) * silu(z)
    parts = int(c["norm_groups"])
    y = unit(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def paired_mixer(W, p, c, h, eps):
    left = unit(left_attention(W, p + "left.", c["left"], h, eps), eps) * W[p + "left.out"]
    right = unit(state_space(W, p + "right.", c["right"], h, eps), eps) * W[p + "right.out"]
    return 0.5 * (left + right)


# --------------------------------------------------------------------------- feed-forward
def gated_unit(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def router_scores(W, p, h):
    return sigma(h @ W[p + "router"].T)


def choose_experts(scores, top):
    """The `top` largest scores of every row, of equal ones the lower expert: [T, top]."""
    rows = []
    for s in scores.tolist():
        order = sorted(range(len(s)), key=lambda e: (-s[e], e))
        rows.append(order[:top])
    return rows


def experts_ff(W, p, c, h, forced=None, slack=0.0):
    """`forced`: per position the experts another implementation chose; they are taken if each of them
    would be among the chosen with `slack` added to its score (a close call), else the run fails."""
    scores = router_scores(W, p, h)
    top = int(c["router"]["top"])
    chosen = choose_experts(scores, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        mine = chosen[t]
        if forced is not None and sorted(forced[t]) != sorted(mine):
            floor = min(float(scores[t, e]) for e in mine)
            if any(float(scores[t, e]) + slack < floor for e in forced[t]):
                raise AssertionError(f"{p} position {t}: experts {forced[t]} are no close call of {mine}")
            mine = forced[t]
        for e in mine:
            out[t] += gated_unit(W, f"{p}e{e}.", (scores[t, e] * h[t])[None])[0]
    if c.get("shared"):
        out = out + sigma(h @ W[p + "shared.sg"].T) * gated_unit(W, p + "shared.", h)
    return out


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    """(layer, whether a pass of the loop other than the first begins here)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for k in range(times):
        order += [(i, k > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def residual_stream(cfg, W, tokens, after_every_layer=None, forced=None, slack=0.0):
    eps = float(cfg["norm"]["eps"])
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    for run, (i, again) in enumerate(run_order(cfg)):
        L, p = cfg["layers"][i], f"l{i}."
        if again:
            x = x + x0
        h = unit(x, eps) * (1.0 + W[p + "norm1"])
        if L["type"] == "parallel":
            y = paired_mixer(W, p + "mix.", L["mixer"], h, eps)
        elif L["type"] == "attention":
            y = plain_attention(W, p + "mix.", L["mixer"], h)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            y = y + experts_ff(W, p + "mlp.", L["mlp"], h, None if forced is None else forced.get(run), slack)
        x = x + y
        if after_every_layer is not None:
            after_every_layer.append(x.clone())
    return x


def forward_logits(cfg, W, tokens, forced=None, slack=0.0):
    x = residual_stream(cfg, W, tokens, forced=forced, slack=slack)
    eps = float(cfg["norm"]["eps"])
    h = unit(x, eps) * (1.0 + W["final.norm"])
    return (h @ W["embed"].T) * float(cfg.get("logit_scale", 1.0))


def greedy_generate(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward_logits(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]
