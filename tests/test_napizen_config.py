"""The Napizen configuration as data (no GPU): which class config.json selects, the parts and tensors
the model declares, what is refused; and pins of the plain implementation's pieces against library
routines and against what the design says of them."""
import copy
import math

import pytest
import torch

from axon_amd.config import ConfigError, NapizenConfig, config_from_dict
from axon_amd.config.base import PartSpec
from axon_amd.models import build_model_description
from axon_amd.parts import build_part
from napizen_models import MODELS, att, config, dense, draw_weights, layer, moe
from plain import napizen_plain as P


def test_config_json_selects_the_class_and_describes_the_layers():
    cfg = MODELS["A"]["cfg"]
    c = config_from_dict(cfg)
    assert isinstance(c, NapizenConfig) and c.to_dict() == cfg
    spec = c.model_spec()
    assert [l.prefix for l in spec.layers] == ["l0.", "l1.", "l2."] and [(r.layer, r.cache) for r in spec.order] == [(0, 0), (1, 1), (2, 2)]
    assert [l.block for l in spec.layers] == ["postnorm"] * 3 and spec.layers[0].norm.kind == "layernorm"
    assert spec.layers[0].norm.params["stream_alpha"] == 1.7 and spec.embedding.params["scale"] == 3.0
    assert spec.final_norm.kind == "layernorm" and spec.head.params["softcap"] == 8.0
    m = spec.layers[0].mixer.params
    assert (m["q_rank"], m["window"], m["gate"], m["sink"], m["kv_rank"], m["rot_dim"]) == (0, 0, "heads", True, 20, 4)
    pos = m["position"].params
    assert pos["pairing"] == "neighbours" and pos["theta"] == 100.0 and pos["scaling"]["kind"] == "ramp" and pos["scaling"]["factor"] == 4.0
    assert "scaling" not in spec.layers[2].mixer.params["position"].params
    f = spec.layers[0].feed_forward.params
    assert (f["experts"], f["top"], f["limit"], f["alpha"], f["shift"]) == (6, 2, None, 1.0, 0.0)
    assert f["router"] == {"scores": "sigmoid", "correction": True, "groups": 3, "keep": 2, "scale": 2.5}
    assert spec.layers[1].feed_forward.kind == "swiglu_mlp" and spec.layers[2].feed_forward is None
    model = build_model_description(c)
    plan = model.cache_plan
    # the first two layers share a pool, the third has sizes (and so a pool) of its own; no state
    assert [(s.entries, s.heads, s.head_dim, s.window, n) for s, n in zip(plan.group_specs, plan.group_layers)] == \
        [(1, 1, 44, 0, 2), (1, 1, 38, 0, 1)]
    assert plan.state_elems == [] and model.blocks[2].norm2 is None


@pytest.mark.parametrize("name", sorted(MODELS))
def test_the_declared_tensors_are_the_checkpoints(name):
    cfg = MODELS[name]["cfg"]
    declared = {d.name: tuple(d.shape) for d in build_model_description(config_from_dict(cfg)).tensors()}
    assert declared == {k: tuple(v.shape) for k, v in draw_weights(cfg, 0).items()}


def test_defaults_where_config_json_is_silent():
    cfg = config(32, 50, [layer(att(2, 4, 4, 4, 8), moe(4, 2, 8))])
    del cfg["embedding"], cfg["postln_alpha"], cfg["logit_softcap"]
    c = config_from_dict(cfg)
    assert c.embedding_scale == 1.0 and c.alpha == 1.0 and c.softcap == 0.0
    spec = c.model_spec()
    assert spec.layers[0].feed_forward.params["router"]["groups"] == 1 and spec.layers[0].feed_forward.params["router"]["keep"] == 1


@pytest.mark.parametrize("breaker,message", [
    (lambda c: c["layers"][0].update(type="rglru"), "is not a mixer of this design"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "is not a feed-forward of this design"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "cannot give 5 a token"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "cannot give"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=4), "cannot give"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=6), "rotary_dim 6 must be even and at most head_dim 4"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "must be even"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "missing kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("fast"), "missing fast"),
    (lambda c: c.pop("vocab"), "missing vocab"),
    (lambda c: c["norm"].pop("eps"), "missing eps"),
    (lambda c: c.update(logit_softcap=-1.0), "must not be below 0"),
])
def test_what_cannot_run_is_refused_with_its_key(breaker, message):
    cfg = copy.deepcopy(MODELS["A"]["cfg"])
    breaker(cfg)
    with pytest.raises(ConfigError, match=message):
        build_model_description(config_from_dict(cfg))


def test_the_encodings_frequencies_are_the_plain_ones():
    for name in sorted(MODELS):
        for L in MODELS[name]["cfg"]["layers"]:
            rot = L["mixer"]["rot"]
            spec = config_from_dict(config(16, 16, [layer(dict(L, mlp=None), None)])).model_spec().layers[0].mixer.params["position"]
            enc = build_part("position", spec)
            f, mag = P.pair_frequencies(rot)
            assert torch.allclose(enc.frequencies(), torch.tensor(f, dtype=torch.float64), rtol=1e-14, atol=0)
            assert enc.magnitude == pytest.approx(mag, rel=1e-15) and enc.pairing == "neighbours"


# --------------------------------------------------------------------------- pins of the plain implementation
def test_plain_pieces_reduce_to_library_routines():
    g = torch.Generator().manual_seed(0)
    z = torch.randn(50, generator=g, dtype=torch.float64) * 3
    assert torch.allclose(P.silu(z), torch.nn.functional.silu(z), atol=1e-12)
    assert torch.allclose(P.sigma(z), torch.sigmoid(z), atol=1e-12)
    x = torch.randn(4, 10, generator=g, dtype=torch.float64) + 2.0
    gain = torch.randn(10, generator=g, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, gain, 1e-3), torch.nn.functional.layer_norm(x, (10,), gain, None, 1e-3), atol=1e-12)
    assert torch.allclose(P.rms(x, torch.ones(10, dtype=torch.float64), 0.0).pow(2).mean(-1), torch.ones(4, dtype=torch.float64))
    # the rotation of pair (2k, 2k + 1) is a complex product by mag exp(i p f_k); the places behind `dims` pass
    rot = {"base": 50.0, "dims": 6, "scaling": {"factor": 3.0, "original": 20, "fast": 4.0, "slow": 0.5}}
    f, mag = P.pair_frequencies(rot)
    assert mag == pytest.approx(0.1 * math.log(3.0) + 1.0)
    v = torch.randn(6, 3, 8, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 7, 100, 1000])
    got = P.rotate_neighbours(v, pos, rot)
    turn = torch.polar(torch.full((6, 3), mag, dtype=torch.float64), pos[:, None].double() * torch.tensor(f, dtype=torch.float64))[:, None, :]
    turned = torch.complex(v[..., 0:6:2], v[..., 1:6:2]) * turn
    assert torch.allclose(got[..., 0:6:2], turned.real) and torch.allclose(got[..., 1:6:2], turned.imag)
    assert torch.equal(got[..., 6:], v[..., 6:])
    # the ramp: pairs before `lo` keep their frequency, pairs from `hi` on are divided by the factor
    plain_f = [50.0 ** (-2.0 * k / 6) for k in range(3)]
    pair_of = lambda t: 6 * math.log(20 / (2 * math.pi * t)) / (2 * math.log(50.0))
    lo, hi = max(math.floor(pair_of(4.0)), 0), min(math.ceil(pair_of(0.5)), 5)
    for k in range(3):
        r = min(max((k - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        assert f[k] == pytest.approx(plain_f[k] * (r / 3.0 + 1.0 - r))
    assert P.pair_frequencies({"base": 50.0, "dims": 6}) == (plain_f, 1.0)


def test_plain_attention_behaves_as_the_design_says():
    cfg = config(16, 20, [layer(att(heads=2, dim=4, rot_dim=4, vdim=6, kv_rank=8), dense(12))])
    W = {k: v.double() for k, v in draw_weights(cfg, 1).items()}
    g = torch.Generator().manual_seed(1)
    h = torch.randn(12, 16, generator=g, dtype=torch.float64)
    c = cfg["layers"][0]["mixer"]
    full = P.latent_attention(W, "l0.mix.", c, h, 1e-6)
    # causal: a later token moves no earlier row; every earlier token moves the last row
    later = h.clone()
    later[9] += 1.0
    assert torch.allclose(P.latent_attention(W, "l0.mix.", c, later, 1e-6)[:9], full[:9])
    first = h.clone()
    first[0] += 1.0
    assert not torch.allclose(P.latent_attention(W, "l0.mix.", c, first, 1e-6)[-1], full[-1])
    # a sink far below every score is no sink: the library's softmax attention over keys and values built in full
    Wn = dict(W)
    Wn["l0.mix.sink"] = torch.full((2,), -1e9, dtype=torch.float64)
    T, H = 12, 2
    q = (h @ W["l0.mix.q"].T).view(T, H, 8)
    down = h @ W["l0.mix.dkv"].T
    lat = P.rms(down[:, :8], W["l0.mix.dkv.norm"], 1e-6)
    pos = torch.arange(T)
    qf = torch.cat([q[..., :4], P.rotate_neighbours(q[..., 4:], pos, c["rot"])], -1)
    kf = torch.cat([(lat @ W["l0.mix.uk"].T).view(T, H, 4), P.rotate_neighbours(down[:, 8:], pos, c["rot"])[:, None, :].expand(T, H, 4)], -1)
    vals = (lat @ W["l0.mix.uv"].T).view(T, H, 6)
    lib = torch.nn.functional.scaled_dot_product_attention(qf.transpose(0, 1), kf.transpose(0, 1), vals.transpose(0, 1), is_causal=True,
                                                           scale=c["scale"]).transpose(0, 1)
    want = (lib * P.sigma(h @ W["l0.mix.g"].T)[:, :, None]).reshape(T, H * 6) @ W["l0.mix.o"].T
    assert torch.allclose(P.latent_attention(Wn, "l0.mix.", c, h, 1e-6), want, atol=1e-10)
    # with the sink a head's weights sum to less than one: the first row's is exp(s) / (exp(s) + exp(sink))
    s0 = (qf[0, 0] @ kf[0, 0]) * c["scale"]
    share = torch.exp(s0) / (torch.exp(s0) + torch.exp(W["l0.mix.sink"][0]))
    Wo = dict(W)
    Wo["l0.mix.o"] = torch.eye(16, 12, dtype=torch.float64)
    head0 = P.latent_attention(Wo, "l0.mix.", c, h, 1e-6)[0, :6]
    assert torch.allclose(head0, share * vals[0, 0] * P.sigma(h[0] @ W["l0.mix.g"][0]), atol=1e-12)
    # positions shifted together: scores depend on differences of positions alone
    assert torch.allclose(P.latent_attention(W, "l0.mix.", c, h, 1e-6, first_position=37), full, atol=1e-9)


def test_plain_routing_behaves_as_the_design_says():
    corr = torch.zeros(6, dtype=torch.float64)
    s = torch.tensor([0.9, 0.1, 0.5, 0.6, 0.2, 0.8], dtype=torch.float64)
    assert P.choose_experts(s, corr, 3, 1, 1) == [0, 5, 3]                       # no groups: the largest scores
    # three groups of two: sums 1.0, 1.1, 1.0; the best and, of equal ones, the lower stay
    assert P.choose_experts(s, corr, 3, 3, 2) == [0, 3, 2]
    assert P.choose_experts(s, corr, 2, 3, 1) == [3, 2]
    # the correction decides the choice
    assert P.choose_experts(s, torch.tensor([0, 0, 0, 0, 1.0, 0], dtype=torch.float64), 2, 1, 1) == [4, 0]
    # negative choice scores: the experts of a group that is left out are no candidates, not zeros
    low = torch.tensor([-1.5] * 3 + [-2.0] * 3, dtype=torch.float64)
    assert P.choose_experts(s, low, 2, 2, 1) == [0, 2]
    # the weights come from the scores without the correction, over their sum, times the scale
    cfg = config(16, 20, [layer(att(2, 4, 4, 6, 8), moe(6, 2, 8, (3, 2), 2.5))])
    W = {k: v.double() for k, v in draw_weights(cfg, 2).items()}
    h = torch.randn(5, 16, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    m = cfg["layers"][0]["mlp"]
    got = P.routed_ff(W, "l0.mlp.", m, h)
    sc = P.sigma(h @ W["l0.mlp.router"].T)
    for t in range(5):
        chosen = P.choose_experts(sc[t], W["l0.mlp.correction"], 2, 3, 2)
        a, b = chosen
        want = 2.5 * (sc[t, a] * P.gated_unit(W, f"l0.mlp.e{a}.", h[t:t + 1])[0] + sc[t, b] * P.gated_unit(W, f"l0.mlp.e{b}.", h[t:t + 1])[0]) / (sc[t, a] + sc[t, b])
        assert torch.allclose(got[t], want, atol=1e-12)
    assert torch.allclose(P.gated_unit(W, "l0.mlp.e0.", h),
                          (torch.nn.functional.silu(h @ W["l0.mlp.e0.gate"].T) * (h @ W["l0.mlp.e0.up"].T)) @ W["l0.mlp.e0.down"].T)


def test_the_arrangement_of_a_layer_and_the_output():
    cfg = config(16, 20, [layer(att(2, 4, 4, 6, 8), dense(12)), layer(att(2, 4, 4, 6, 8), None)], alpha=1.7, scale=3.0, softcap=5.0)
    W = {k: v.double() for k, v in draw_weights(cfg, 3).items()}
    toks = [3, 7, 7, 1, 19, 0]
    seen = []
    x = P.residual_stream(cfg, W, toks, seen)
    x0 = W["embed"][torch.tensor(toks)] * 3.0
    ln = lambda v, gname: torch.nn.functional.layer_norm(v, (16,), W[gname], None, 1e-6)
    a = ln(1.7 * x0 + P.latent_attention(W, "l0.mix.", cfg["layers"][0]["mixer"], x0, 1e-6), "l0.norm1")
    b = ln(1.7 * a + P.gated_unit(W, "l0.mlp.", a), "l0.norm2")
    c = ln(1.7 * b + P.latent_attention(W, "l1.mix.", cfg["layers"][1]["mixer"], b, 1e-6), "l1.norm1")
    assert torch.allclose(seen[0], b) and torch.allclose(seen[1], c) and torch.allclose(x, c)
    z = ln(c, "final.norm") @ W["head"].T
    logits = P.forward_logits(cfg, W, toks)
    assert torch.allclose(logits, 5.0 * torch.tanh(z / 5.0)) and float(logits.abs().max()) < 5.0
    # variants that must differ: a norm before the sublayer, the stream not stretched
    pre = x0 + P.latent_attention(W, "l0.mix.", cfg["layers"][0]["mixer"], ln(x0, "l0.norm1"), 1e-6)
    assert not torch.allclose(pre, a, atol=1e-3)
    assert not torch.allclose(ln(x0 + P.latent_attention(W, "l0.mix.", cfg["layers"][0]["mixer"], x0, 1e-6), "l0.norm1"), a, atol=1e-3)


def test_the_command_line_writes_and_describes_a_model_of_the_design(tmp_path, capsys):
    import json
    from axon_amd.cli import main
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(MODELS["D"]["cfg"]))
    out = tmp_path / "model"
    assert main(["random-weights", str(cfg_path), str(out), "--seed", "3"]) == 0
    assert main(["info", str(out)]) == 0
    text = capsys.readouterr().out
    assert "architecture: Napizen" in text and "cache group: 2 layers x 1 x 1 heads x 50" in text
    from safetensors.torch import load_file
    names = set(load_file(str(out / "model.safetensors")))
    assert names == set(draw_weights(MODELS["D"]["cfg"], 0))
