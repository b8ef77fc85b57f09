"""The Zugutar configuration reader and the model it describes (CPU): every size and constant of
config.json reaches the parts, the tensors declared are the checkpoint's, runs and their caches and states
follow the loop, what the design does not have is refused; and the plain implementation's pieces against
special cases that reduce to library routines."""
import math

import pytest
import torch

from axon_amd.config import ConfigError, config_from_dict
from axon_amd.models.decoder import DecoderModel
from plain import zugutar_plain as P
from zugutar_models import MODELS, att, config, draw_weights, layer, left, moe, pair, right


@pytest.mark.parametrize("name", sorted(MODELS))
def test_the_declared_tensors_are_the_checkpoints(name):
    m = MODELS[name]
    W = draw_weights(m["cfg"], m["seed"])
    model = DecoderModel(config_from_dict(m["cfg"]))
    decl = {d.name: tuple(d.shape) for d in model.tensors()}
    optional = {d.name for d in model.tensors() if d.optional}
    assert optional == {"head"}                       # the head is the embedding's matrix
    assert set(decl) - optional == set(W)
    assert all(tuple(W[k].shape) == decl[k] for k in W)


def test_every_constant_reaches_its_part():
    cfg = config(96, 50, [layer(pair(left(6, 2, 12, 20, dims=8, base=777.0, scale=0.31), right(3, 10, 9, groups=3, conv=5, norm_groups=2)),
                                moe(7, 3, 11, shared=13)),
                          layer(att(4, 4, 10, 6, temp=(0.125, 37), scale=0.77), None)], loop=(1, 2, 3), eps=3e-4, logit_scale=0.3)
    spec = config_from_dict(cfg).model_spec()
    assert spec.hidden_size == 96 and spec.vocab_size == 50 and spec.head.params["scale"] == 0.3 and spec.head.params["tied"]
    assert spec.final_norm.params == {"size": 96, "eps": 3e-4, "tensor": "final.norm", "offset": 1.0}
    first, second = spec.layers
    assert first.block == second.block == "parallel" and first.norm.params["offset"] == 1.0 and first.norm.params["eps"] == 3e-4
    l, r = first.mixer.params["left"].params, first.mixer.params["right"].params
    assert first.mixer.kind == "paired_mixers" and first.mixer.params["mult"] == 0.5 and first.mixer.params["eps"] == 3e-4
    assert (l["heads"], l["kv_heads"], l["dim"], l["vdim"], l["scale"], l["sink"], l["gate"], l["qk_norm"]) == (6, 2, 12, 20, 0.31, 0.0, "heads", True)
    assert l["position"].params == {"head_dim": 12, "rotary_dim": 8, "theta": 777.0, "pairing": "halves"}
    assert (r["heads"], r["vdim"], r["state"], r["groups"], r["conv"], r["norm_groups"], r["eps"]) == (3, 10, 9, 3, 5, 2, 3e-4)
    f = first.feed_forward.params
    assert (f["experts"], f["top"], f["ff"], f["weight_on"], f["router"], f["shared"]) == (
        7, 3, 11, "input", {"scores": "sigmoid", "normalize": False}, {"ff": 13, "unit": "gated", "gate": "sg"})
    a = second.mixer.params
    assert second.mixer.kind == "masked_attention" and second.feed_forward is None
    assert (a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["scale"], a["q_temp"], a["gate"], a["position"]) == (
        4, 4, 10, 6, 0.77, {"coef": 0.125, "every": 37}, "elements", None)
    assert a.get("sink") is None
    # layer 1 three times, a cache and a state a run, the embedding added before the second and third pass
    assert [(r.layer, r.cache, r.enter) for r in spec.order] == [(0, 0, None), (1, 1, None), (1, 2, 0), (1, 3, 0)]
    assert [e.kind for e in spec.entries] == ["embedding_add"]


def test_runs_get_caches_and_states_of_their_own():
    m = MODELS["A"]
    model = DecoderModel(config_from_dict(m["cfg"]))
    plan = model.cache_plan
    assert [r.layer for r in model.order] == [0, 1, 0, 1, 0, 1, 2]
    pairs = [b for b, r in zip(plan.bindings, model.order) if r.layer != 1]
    assert sorted(b.state_index for b in pairs) == [0, 1, 2, 3] and all(b.state_index == -1 for b, r in zip(plan.bindings, model.order) if r.layer == 1)
    assert len({(b.group, b.index) for b in plan.bindings}) == 7
    # a copy of a pair's state: the heads' states, then the convolution's kept inputs; two copies a row
    c = m["cfg"]["layers"][0]["mixer"]["right"]
    channels = c["heads"] * c["vdim"] + 2 * c["groups"] * c["state"]
    assert plan.state_elems[0] == (2 * (c["heads"] * c["state"] * c["vdim"] + (c["conv"] - 1) * channels), "float32")
    no_loop = DecoderModel(config_from_dict(MODELS["C"]["cfg"]))
    assert not no_loop.entries and [r.enter for r in no_loop.order] == [None] * 3
    once = DecoderModel(config_from_dict(MODELS["D"]["cfg"]))
    assert not once.entries and [r.layer for r in once.order] == [0, 1]


def test_what_the_design_does_not_have_is_refused():
    good = MODELS["A"]["cfg"]
    def changed(path, value):
        import copy
        cfg = copy.deepcopy(good)
        at = cfg
        for k in path[:-1]:
            at = at[k]
        if value is None:
            at.pop(path[-1])
        else:
            at[path[-1]] = value
        return cfg
    for path, value in [(("layers", 0, "type"), "recurrent"), (("layers", 0, "mlp", "kind"), "dense"), (("width",), None),
                        (("norm",), None), (("layers", 1, "mixer", "scale"), None), (("layers", 0, "mixer", "right", "state"), 0),
                        (("loop", "stop"), 9), (("layers", 0, "mixer", "left", "rot", "dims"), 3), (("layers",), [])]:
        with pytest.raises(ConfigError):
            DecoderModel(config_from_dict(changed(path, value)))
    with pytest.raises(ConfigError):
        DecoderModel(config_from_dict(changed(("layers", 0, "mixer", "left", "kv_heads"), 2)))        # three heads on two
    with pytest.raises(ConfigError):
        DecoderModel(config_from_dict(changed(("layers", 0, "mixer", "right", "groups"), 2)))          # three heads in two groups
    with pytest.raises(ConfigError):
        DecoderModel(config_from_dict(changed(("layers", 0, "mlp", "router", "top"), 6)))              # six of five experts


# --------------------------------------------------------------------------- the plain implementation's pieces
def test_plain_attention_reduces_to_a_library_softmax():
    g = torch.Generator().manual_seed(1)
    T, H, G, d, dv = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(T, n, s, generator=g, dtype=torch.float64) for n, s in ((H, d), (G, d), (G, dv)))
    got = P.heads_attention(q, k, v, 0.4, sink=False)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for a in range(H):
        s = (q[:, a] @ k[:, a // 2].T * 0.4).masked_fill(~mask, -math.inf)
        assert torch.allclose(got[:, a], torch.softmax(s, -1) @ v[:, a // 2], atol=1e-12)
        # a sink of score 0: one more key of score 0 whose value is nothing
        with_zero = torch.cat([torch.zeros(T, 1, dtype=torch.float64), s], 1)
        sunk = torch.softmax(with_zero, -1)[:, 1:] @ v[:, a // 2]
        assert torch.allclose(P.heads_attention(q, k, v, 0.4, sink=True)[:, a], sunk, atol=1e-12)


def test_plain_rotation_is_a_complex_product_on_the_leading_places():
    g = torch.Generator().manual_seed(2)
    v = torch.randn(7, 2, 10, generator=g, dtype=torch.float64)
    pos = torch.arange(3, 10)
    out = P.rotate_halves(v, pos, {"dims": 6, "base": 50.0})
    assert torch.equal(out[..., 6:], v[..., 6:])
    for i in range(3):
        z = torch.complex(v[..., i], v[..., i + 3]) * torch.polar(torch.ones(7, dtype=torch.float64), pos.double() * 50.0 ** (-2 * i / 6))[:, None]
        assert torch.allclose(out[..., i], z.real, atol=1e-12) and torch.allclose(out[..., i + 3], z.imag, atol=1e-12)


def test_plain_state_space_is_its_unrolled_sum():
    """y_t = sum_(s <= t) (prod_(s < r <= t) a_r) dt_s (C_t . B_s) x_s + D x_t, one head, written out."""
    g = torch.Generator().manual_seed(3)
    cfg = config(16, 8, [layer(pair(left(1, 1, 4, 4), right(1, 3, 4, conv=1)), None)])
    W = {k: v.double() for k, v in draw_weights(cfg, 5).items()}
    W["l0.mix.right.norm"] = torch.ones(3, dtype=torch.float64)
    W["l0.mix.right.o"] = torch.eye(16, 3, dtype=torch.float64)
    c, p = cfg["layers"][0]["mixer"]["right"], "l0.mix.right."
    h = torch.randn(6, 16, generator=g, dtype=torch.float64)
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :3], P.silu(proj[:, 3:14] * W[p + "conv"][:, 0] + W[p + "conv.b"]), torch.nn.functional.softplus(proj[:, 14] + W[p + "dt_bias"][0])
    x, B, C = xbc[:, :3], xbc[:, 3:7], xbc[:, 7:]
    a = torch.exp(-torch.exp(W[p + "A_log"][0]) * dt)
    y = torch.stack([sum(torch.prod(a[s + 1:t + 1]) * dt[s] * (C[t] @ B[s]) * x[s] for s in range(t + 1)) + W[p + "D"][0] * x[t] for t in range(6)])
    want = P.unit(y * P.silu(z), 1e-5)
    assert torch.allclose(P.state_space(W, p, c, h, 1e-5)[:, :3], want, atol=1e-10)


def test_plain_conv_reads_zeros_before_the_start_and_its_last_column_now():
    x = torch.arange(1.0, 6.0, dtype=torch.float64)[:, None]
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)
    assert P.causal_conv(x, w, torch.zeros(1, dtype=torch.float64))[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0, 345.0]


def test_plain_experts_take_the_largest_scores_and_the_lower_of_equals():
    assert P.choose_experts(torch.tensor([[0.2, 0.9, 0.9, 0.1], [0.5, 0.5, 0.5, 0.5]]), 2) == [[1, 2], [0, 1]]
