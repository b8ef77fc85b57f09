"""The Napizen decoder through the engine against the plain implementation (tests/plain/napizen_plain.py):
whole prompts, decoding token by token, portions down to two tokens, unequal requests side by side with
pages and slots that come round again, long decoding across pages, generation through the engine's own
entry point, the trace replay program, and every mechanism alone with weights or inputs made so that a
fault shows (a sink left out, a far key lost, a pairing of halves, a correction in the weights, a group
that is left out counted as zeros: each differs from the plain implementation by far more than the
tolerance)."""
import math

import pytest
import torch

import axon_amd
from axon_amd.config import config_from_dict
from axon_amd.config.base import PartSpec
from axon_amd.engine import StepEntry
from axon_amd.parts import CacheBinding, CacheSpec, build_part
from axon_amd.weights import WeightStore
from gpu_helpers import DTYPES, DictSource, PartHarness
from helpers import TraceBuilder, engine_for, run_trace, tolerance
from napizen_models import MODELS, att, config, dense, draw_weights, layer, make, moe
from plain import napizen_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = make(str(tmp_path_factory.mktemp("napizen_" + name)), name)
        return made[name]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    """The plain implementation's logits of a model's test sequences.  float32: its own choice of experts
    (worked out once a sequence).  bfloat16: with the experts the engine chose where these are a close
    call of its own choice (16 bits decide a close call either way, and every later row sees it)."""
    kept, models = {}, {}

    def get(name, seq, dtype="float32", forced=None):
        if name not in models:
            models[name] = P.load_plain(folders(name))
        cfg, W = models[name]
        if dtype == "bfloat16":
            return P.forward_logits(cfg, W, seq, forced, SLACK).float()
        key = (name, tuple(seq))
        if key not in kept:
            kept[key] = P.forward_logits(cfg, W, seq).float()
        return kept[key]
    return get


SLACK = 0.05          # how far 16 bits of stream may move a router's score


def sequences(name, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, MODELS[name]["cfg"]["vocab"], (n,), generator=g).tolist() for n in lengths]


def assert_close(got, ref, dtype, what):
    """Rows of logits against the plain implementation's, every row."""
    err = (got - ref).abs().max(dim=-1).values
    # a norm behind every sum passes each rounding on at full size: twice (32-bit) and three times (16 bits)
    # what the engine's other designs are held to
    limit = tolerance(dtype, ref) * (2.0 if dtype == "float32" else 3.0)
    assert float(err.max()) <= limit, f"{what}: {float(err.max())} > {limit} at row {int(err.argmax())}"


class RouterLog:
    """What the engine's router chose, launch by launch: the kernels' entry is wrapped while a schedule runs."""

    def __init__(self, eng):
        self.k, self.calls = eng.rt.k, []

    def __enter__(self):
        inner = self.k.route_scored

        def logged(logits, correction, top, groups, keep, scale, chosen, weights):
            inner(logits, correction, top, groups, keep, scale, chosen, weights)
            self.calls.append(chosen.cpu().tolist())
        self.k.route_scored = logged
        return self

    def __exit__(self, *exc):
        del self.k.route_scored


def run_schedule(eng, name, seqs, schedule):
    """schedule: steps of [(request, tokens)]; every position's logits are asked for.  A request
    ends with its last token.  `name`: one of MODELS, or a configuration.  Returns ({request: [len, vocab]},
    {request: {layer: chosen experts by position}})."""
    cfg = MODELS[name]["cfg"] if isinstance(name, str) else name
    routed = [i for i, L in enumerate(cfg["layers"]) if L.get("mlp") and L["mlp"]["kind"] == "moe"]
    at = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    chose = {r: {i: [] for i in routed} for r in seqs}
    with RouterLog(eng) as log:
        for step in schedule:
            entries, ends = [], []
            for rid, n in step:
                toks = seqs[rid][at[rid]:at[rid] + n]
                entries.append(StepEntry(rid, toks, list(range(len(toks)))))
                at[rid] += len(toks)
                if at[rid] == len(seqs[rid]):
                    ends.append(rid)
            del log.calls[:]
            out = eng.step(entries, ends).cpu()
            assert len(log.calls) == len(routed)
            row = 0
            for e in entries:
                got[e.id].append(out[row:row + len(e.tokens)].clone())
                for i, call in zip(routed, log.calls):
                    chose[e.id][i] += call[row:row + len(e.tokens)]
                row += len(e.tokens)
    assert all(at[r] == len(seqs[r]) for r in seqs)
    return {r: torch.cat(v) for r, v in got.items()}, chose


def pages_for(name, tokens):
    return -(-tokens // MODELS[name]["page"]) + 2


# --------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_whole_prompts_and_decoding_token_by_token(folders, plain_logits, name, dtype):
    n = 150 if name in "BC" else 70
    (seq,) = sequences(name, [n], seed=1)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    got, chose = run_schedule(eng, name, {"a": seq}, [[("a", n)]])
    ref = plain_logits(name, seq, dtype, chose["a"])
    whole = got["a"]
    assert_close(whole, ref, dtype, "whole prompt")
    # from the first token on, one token a step: the first tokens of a sequence, every page's edge
    got, chose = run_schedule(eng, name, {"b": seq}, [[("b", 1)] for _ in range(n)])
    single = got["b"]
    assert_close(single, plain_logits(name, seq, dtype, chose["b"]), dtype, "token by token")
    # most of it at once, the rest decoded
    got, chose = run_schedule(eng, name, {"c": seq}, [[("c", n - 45)]] + [[("c", 1)] for _ in range(45)])
    assert_close(got["c"], plain_logits(name, seq, dtype, chose["c"]), dtype, "prompt then decoding")
    if dtype == "float32":
        assert float((single - whole).abs().max()) <= 2 * tolerance(dtype, ref)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_portions_of_many_sizes_down_to_two_tokens(folders, plain_logits, name, dtype):
    n = 200 if name in "BC" else 90
    (seq,) = sequences(name, [n], seed=2)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    for cuts in ([2, 2, 3, 1, 2, 7, 1, 1, 5, 64, 2], [63, 2, 1, 64, 9], [8, 8, 1, 16, 2]):
        sched, left, i = [], n, 0
        while left:
            take = min(cuts[i % len(cuts)], left)
            sched.append([("a", take)])
            left -= take
            i += 1
        got, chose = run_schedule(eng, name, {"a": seq}, sched)
        assert_close(got["a"], plain_logits(name, seq, dtype, chose["a"]), dtype, f"portions {cuts}")
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(folders, plain_logits, name, dtype):
    lengths = [57, 5, 120, 33, 1, 76]
    seqs = dict(enumerate(sequences(name, lengths, seed=3)))
    page = MODELS[name]["page"]
    # three slots and a pool for the three longest live at once: later requests get the pages and
    # the slots of finished ones
    eng = engine_for(folders(name), dtype, page, 3 * (-(-120 // page)) + 1, max_seqs=3, max_seq_len=128, shuffle_pages_seed=5)
    cuts = {0: [9, 1, 1, 2, 30, 1], 1: [2, 1, 1, 1], 2: [1, 40, 1, 1, 3, 64, 1], 3: [33], 4: [1], 5: [2, 1, 50, 1, 1, 1]}
    at = {r: 0 for r in seqs}
    waiting, live, sched, turn = [0, 1, 2, 3, 4, 5], [], [], 0
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        step = []
        for r in list(live):
            if (turn + r) % 4 == 3 and len(live) > 1:
                continue                                  # left out of this step, goes on later
            n = min(cuts[r][(turn // 2) % len(cuts[r])], lengths[r] - at[r])
            step.append((r, n))
            at[r] += n
            if at[r] == lengths[r]:
                live.remove(r)
        if step:
            sched.append(step)
        turn += 1
    got, chose = run_schedule(eng, name, seqs, sched)
    for r in seqs:
        assert_close(got[r], plain_logits(name, seqs[r], dtype, chose[r]), dtype, f"request {r} in the mixed schedule")
    eng.cache.check()
    assert not eng.live
    for g in range(len(eng.cache.groups)):
        assert eng.cache.free_pages(g) == eng.cache.groups[g].n_pages
    if dtype == "float32":
        # each request alone gives the same rows as side by side, to rounding
        alone, _ = run_schedule(eng, name, {2: seqs[2]}, [[(2, lengths[2])]])
        assert float((alone[2] - got[2]).abs().max()) <= 2 * tolerance(dtype, plain_logits(name, seqs[2]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_portions_of_several_requests_in_one_step(folders, plain_logits, name, dtype):
    """Hundreds of tokens a step with heads in sixteens: the attention takes four neighbouring tokens a block
    and stages their pages once where they are one request's; blocks that hold the end of one request and
    the start of the next, or decoded rows of several, let every token read its own pages."""
    lengths = [150, 131, 97, 64]
    seqs = dict(enumerate(sequences(name, lengths, seed=11)))
    eng = engine_for(folders(name), dtype, 64, 9, max_seqs=4, max_seq_len=192, max_batch_tokens=512, shuffle_pages_seed=3)
    sched = [[(0, 101), (1, 99), (2, 95), (3, 1)], [(0, 47), (1, 30), (2, 1), (3, 62)], [(0, 2), (1, 2), (2, 1), (3, 1)]]
    got, chose = run_schedule(eng, name, seqs, sched)
    for r in seqs:
        assert_close(got[r], plain_logits(name, seqs[r], dtype, chose[r]), dtype, f"request {r}")
    eng.cache.check()


@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding_across_many_pages(folders, plain_logits, name):
    n = 250
    (seq,) = sequences(name, [n], seed=4)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), "float32", MODELS[name]["page"], pages_for(name, n), max_seqs=1, max_seq_len=256)
    got, _ = run_schedule(eng, name, {"a": seq}, [[("a", 3)]] + [[("a", 1)] for _ in range(n - 3)])
    assert_close(got["a"], ref, "float32", "long decoding")


@pytest.mark.parametrize("name", sorted(MODELS))
def test_greedy_generation_through_the_entry_point(folders, name):
    cfg, W = P.load_plain(folders(name))
    prompts = sequences(name, [11, 3, 30], seed=6)
    want = [P.greedy_generate(cfg, W, p, 10) for p in prompts]
    page = MODELS[name]["page"]
    pages = 3 * (-(-128 // page))
    llm = axon_amd.load(folders(name), dtype="float32", page_size=page, num_pages=pages, max_seqs=3, max_seq_len=128)
    assert llm.generate(prompts, max_new_tokens=10) == want                       # decoding steps replay graphs
    assert llm.engine.graphs_ok and all(c for c, _, _ in llm.engine._segments)
    assert llm.generate(prompts[:1], max_new_tokens=10) == want[:1]               # alone, in a slot used before
    eager = axon_amd.load(folders(name), dtype="float32", page_size=page, num_pages=pages, max_seqs=3, max_seq_len=128,
                          use_graphs=False)
    assert eager.generate(prompts, max_new_tokens=10) == want
    # 16 bits: the tokens that come out of the scheduler's steps and the graphs are the best of the engine's own
    # logits of prompt and tokens in one step (what those logits are worth is the matter of the tests above)
    half = axon_amd.load(folders(name), dtype="bfloat16", page_size=page, num_pages=pages, max_seqs=3, max_seq_len=128)
    for p, o in zip(prompts, half.generate(prompts, max_new_tokens=10)):
        logits = half.logits(p + o, all_positions=True).float().cpu()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 0.1 * tolerance("bfloat16", logits)


def test_the_command_line_generates_with_the_design(folders):
    import os
    import subprocess
    import sys
    from helpers import ROOT
    name = "D"
    cfg, W = P.load_plain(folders(name))
    p, q = sequences(name, [9, 14], seed=9)
    axon = [sys.executable, os.path.join(ROOT, "bin", "axon")]
    ids = lambda seq: " ".join(map(str, seq))
    r = subprocess.run(axon + ["gen", folders(name), ids(p), ids(q), "-n", "8", "--dtype", "float32", "--page-size", "64"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [[int(t) for t in line.split()] for line in r.stdout.splitlines()] == [
        P.greedy_generate(cfg, W, p, 8), P.greedy_generate(cfg, W, q, 8)]
    r = subprocess.run(axon + ["logits", folders(name), ids(p), "-k", "3", "--dtype", "float32"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    top = torch.topk(P.forward_logits(cfg, W, p)[-1].float(), 3)
    lines = [l.split() for l in r.stdout.splitlines() if "logit" in l]
    assert [int(l[0]) for l in lines] == top.indices.tolist()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_replay_program_runs_the_design(folders, plain_logits, tmp_path, dtype):
    name = "C"
    seqs = sequences(name, [40, 17, 64], seed=7)
    refs = [plain_logits(name, s) for s in seqs]
    tb = TraceBuilder()
    tb.step([("a", seqs[0][:30], [0, 29]), ("b", seqs[1][:2], [1])])
    tb.step([("a", seqs[0][30:31], [0]), ("b", seqs[1][2:], [0, 14]), ("c", seqs[2][:7], [])], end=["b"])
    tb.step([("a", seqs[0][31:], [8]), ("c", seqs[2][7:], [0, 56])], end=["a", "c"])
    rows = tb.collect(run_trace(folders(name), dtype, tb.steps, str(tmp_path), max_tokens=192))
    for (rid, pos), row in rows.items():
        ref = refs["abc".index(rid)]
        assert float((torch.from_numpy(row) - ref[pos]).abs().max()) <= 3 * tolerance(dtype, ref)


# --------------------------------------------------------------------------- the mechanisms alone
def rows_in(T, width, seed, dtype, scale=1.0):
    """Random rows; for the 16-bit run, rows that 16 bits hold exactly (the plain run starts from the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, width, generator=g) * scale
    return h.to(torch.bfloat16).float() if dtype == "bfloat16" else h


def part_tol(dtype, ref):
    return (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))


def mixer_of(cfg, i, prefix):
    """The design's mixer of layer i as the configuration reader describes it."""
    return build_part("mixer", config_from_dict(cfg).layers[i]["mixer"], prefix)


def run_mixer(part, harness, h, cuts, width):
    """The mixer's 32-bit output for rows h, fed in portions of the given sizes."""
    outs, at = [], 0
    for n in cuts:
        ctx = harness.ctx([0] * n)
        x = h[at:at + n].to(harness.rt.dtype).cuda()
        out = torch.full((n, width), float("nan"), dtype=torch.float32, device="cuda")
        part.forward(ctx, CacheBinding(group=0, index=0, writes=True, state_index=0), x, out, accumulate=False)
        outs.append(out.cpu())
        at += n
    assert at == h.shape[0]
    return torch.cat(outs)


def check_latent_attention(cfg, W, page, dtype, T, cut_sets):
    c = cfg["layers"][0]["mixer"]
    part = mixer_of(cfg, 0, "l0.")
    # sinks of the size of the scores (a score's spread under the drawn weights), from head to head half as much again
    W = dict(W, **{"l0.mix.sink": c["scale"] * 2.25 * c["dim"] ** 0.5 * (1.0 + 0.5 * torch.arange(c["heads"]) / c["heads"])})
    h = rows_in(T, cfg["width"], 13, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    ref = P.latent_attention(Wd, "l0.mix.", c, h.double(), eps).float()
    for cuts in cut_sets:
        hs = PartHarness(dtype, part.cache_spec(), page_size=page, n_pages=-(-T // page) + 3, max_seq_len=1024)
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, cfg["width"])
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    # what the test would catch: the sink left out, the sink taken times the scale, a pairing of halves,
    # cos and sin without their factor, the gate left out
    loud = 20 * part_tol("float32", ref)
    no_sink = dict(Wd, **{"l0.mix.sink": torch.full_like(Wd["l0.mix.sink"], -1e9)})
    assert float((P.latent_attention(no_sink, "l0.mix.", c, h.double(), eps).float() - ref).abs().max()) > loud
    scaled = dict(Wd, **{"l0.mix.sink": Wd["l0.mix.sink"] * c["scale"]})
    assert float((P.latent_attention(scaled, "l0.mix.", c, h.double(), eps).float() - ref).abs().max()) > loud
    if c["rot"]["dims"] >= 4:
        # pairs (i, i + n / 2) on the same weights: the plain rotation of neighbours on weights whose rotated rows
        # are laid out [0, n / 2, 1, n / 2 + 1, ...] (queries and the shared key alike, so only the pairing differs)
        n = c["rot"]["dims"]
        as_halves = torch.cat([torch.stack([torch.arange(0, n // 2), torch.arange(n // 2, n)], 1).reshape(-1), torch.arange(n, c["rot_dim"])])
        Wh = dict(Wd)
        q = Wd["l0.mix.q"].view(c["heads"], c["dim"] + c["rot_dim"], -1).clone()
        q[:, c["dim"]:] = q[:, c["dim"]:][:, as_halves]
        Wh["l0.mix.q"] = q.reshape(Wd["l0.mix.q"].shape)
        Wh["l0.mix.dkv"] = torch.cat([Wd["l0.mix.dkv"][:c["kv_rank"]], Wd["l0.mix.dkv"][c["kv_rank"]:][as_halves]])
        assert float((P.latent_attention(Wh, "l0.mix.", c, h.double(), eps).float() - ref).abs().max()) > loud
    if c["rot"].get("scaling"):
        flat = dict(c, rot={k: v for k, v in c["rot"].items() if k != "scaling"})
        assert float((P.latent_attention(Wd, "l0.mix.", flat, h.double(), eps).float() - ref).abs().max()) > loud
    open_gate = dict(Wd, **{"l0.mix.g": torch.zeros_like(Wd["l0.mix.g"])})
    assert float((P.latent_attention(open_gate, "l0.mix.", c, h.double(), eps).float() - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer_i,page", [("A", 0, 8), ("A", 2, 4), ("D", 0, 16), ("D", 1, 32), ("C", 1, 64)])
def test_latent_attention_with_a_sink_and_a_gate_a_head(name, layer_i, page, dtype):
    m = MODELS[name]
    cfg = config(m["cfg"]["width"], 16, [layer({k: v for k, v in m["cfg"]["layers"][layer_i].items() if k != "mlp"}, None)],
                 eps=m["cfg"]["norm"]["eps"])
    W = {k: v for k, v in draw_weights(cfg, 31 + layer_i).items() if k.startswith("l0.")}
    T = 200
    check_latent_attention(cfg, W, page, dtype, T,
                           [[T], [page - 1] + [1] * 8 + [T - page - 7], [2, 1, 1, 3] + [1] * 30 + [64, 2, T - 103]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,vdim,rank,page", [(16, 16, 32, 16, 32, 64), (32, 8, 32, 24, 96, 128), (16, 32, 64, 8, 256, 64),
                                                          (48, 16, 16, 16, 64, 64)])
def test_latent_attention_with_heads_in_sixteens(heads, dim, rot, vdim, rank, page, dtype):
    """Sizes that the matrix-core form takes in 16 bits (heads in sixteens, latents in sixteens, key rows
    in chunks of 32, pages of 64 or 128), with the sink in its softmax: few tokens (a token's blocks of
    positions side by side and folded) and many (a wave walks them)."""
    cfg = config(64, 16, [layer(att(heads, dim, rot, vdim, rank, base=10000.0, scaling=(4.0, 64, 16.0, 1.0), scale=0.3), None)])
    W = {k: v for k, v in draw_weights(cfg, 37).items() if k.startswith("l0.")}
    T = 330
    check_latent_attention(cfg, W, page, dtype, T, [[T], [300] + [1] * 30, [2, 5, 1, 1, 64, 129, 1, 1, 1, 125]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads", [2, 16])
def test_a_key_hundreds_of_positions_back_decides_a_row_against_the_sink(heads, dtype):
    """Weights set by hand: the latent's first half is what keys and queries compare, its second half
    what values carry; the rotated part is silent.  Positions 150 and 880 share the first half (a loud
    match), every other key is faint, and the sink is as loud as the match: row 880 is then a third
    each of the values at 150 and 880, in a prompt and decoded, 730 positions and eleven pages back."""
    width, H, half, rot = 64, heads, 16, (32 if heads == 16 else 4)      # sixteen heads, key rows of 64: the matrix-core form
    eye = torch.eye(half)
    c = att(H, half, rot, half, 2 * half, scale=1.0)["mixer"]
    cfg = config(width, 16, [layer(att(H, half, rot, half, 2 * half, scale=1.0), None)])
    W = {"l0.mix.dkv": torch.cat([torch.eye(2 * half, width), torch.zeros(rot, width)]), "l0.mix.dkv.norm": torch.ones(2 * half),
         "l0.mix.q": torch.cat([torch.cat([torch.eye(half, width), torch.zeros(rot, width)])] * H),
         "l0.mix.uk": torch.cat([torch.cat([eye, 0 * eye], 1)] * H), "l0.mix.uv": torch.cat([torch.cat([0 * eye, eye], 1)] * H),
         "l0.mix.g": torch.zeros(H, width),
         "l0.mix.o": torch.randn(width, H * half, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).float()}
    T = 900
    h = rows_in(T, width, 17, dtype)
    h[:, :half] *= 0.1                                   # faint keys
    h[150, :half] = h[880, :half] = rows_in(1, half, 18, dtype)[0]
    Wd = {k: v.double() for k, v in W.items()}
    # the loud score: q . k of position 880 with itself
    lat = P.rms(h[880:881, :2 * half].double(), torch.ones(2 * half, dtype=torch.float64), 1e-6)[0]
    loud = float(h[880, :half].double() @ lat[:half])
    W["l0.mix.sink"] = torch.full((H,), loud).to(torch.bfloat16).float()
    Wd["l0.mix.sink"] = W["l0.mix.sink"].double()
    ref = P.latent_attention(Wd, "l0.mix.", c, h.double(), 1e-6).float()
    big = 0.05 * float(ref.abs().max())
    no_sink = dict(Wd, **{"l0.mix.sink": torch.full((H,), -1e9, dtype=torch.float64)})
    assert float((P.latent_attention(no_sink, "l0.mix.", c, h.double(), 1e-6).float() - ref)[880].abs().max()) > big
    twice = dict(Wd, **{"l0.mix.sink": Wd["l0.mix.sink"] + math.log(2.0)})          # a sink that counts twice
    assert float((P.latent_attention(twice, "l0.mix.", c, h.double(), 1e-6).float() - ref)[880].abs().max()) > big
    lost = h.clone()
    lost[150, :half] *= 0.1                                                          # the far key not seen
    assert float((P.latent_attention(Wd, "l0.mix.", c, lost.double(), 1e-6).float() - ref)[880].abs().max()) > big
    part = mixer_of(cfg, 0, "l0.")
    for cuts in ([T], [870] + [1] * 30, [149, 2, 700, 19, 2, 28]):
        hs = PartHarness(dtype, part.cache_spec(), page_size=64, n_pages=16, max_seq_len=1024)
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, width)
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts


def test_the_router_with_sigmoid_scores_in_groups():
    from axon_amd.kernels import kernels
    k = kernels("float32")
    g = torch.Generator().manual_seed(5)
    cases = [(6, 2, 3, 2, 2.5, 0.7), (16, 3, 4, 2, 1.25, 0.3), (64, 6, 8, 4, 1.0, 0.5), (256, 8, 8, 4, 2.0, 0.2), (5, 1, 1, 1, 0.5, 0.7),
             (8, 2, 8, 3, 1.0, 0.7), (8, 8, 1, 1, 1.0, 0.0), (12, 4, 3, 1, 1.0, -3.0), (1000, 7, 10, 3, 1.0, 0.4), (70, 64, 1, 1, 1.0, 0.1)]
    for E, top, groups, keep, scale, spread in cases:
        T = 37
        z = torch.randn(T, E, generator=g) * 2
        # a negative spread: every choice score below zero (an expert of a group that is left out, counted as
        # zero, would then win)
        corr = torch.randn(E, generator=g) * spread if spread >= 0 else torch.full((E,), spread)
        chosen = torch.zeros(T, top, dtype=torch.int32, device="cuda")
        weights = torch.zeros(T, top, dtype=torch.float32, device="cuda")
        k.route_scored(z.cuda(), corr.cuda(), top, groups, keep, scale, chosen, weights)
        s = P.sigma(z.double())
        for t in range(T):
            want = P.choose_experts(s[t], corr.double(), top, groups, keep)
            assert chosen[t].tolist() == want, (E, top, groups, keep, t)
            share = torch.stack([s[t, e] for e in want])
            assert torch.allclose(weights[t].cpu().double(), share / (share.sum() + 1e-20) * scale, rtol=1e-5, atol=1e-7)
        if groups > keep:
            sizes = {len({e // (E // groups) for e in chosen[t].tolist()}) for t in range(T)}
            assert max(sizes) <= keep
    # no correction at all
    z = torch.randn(9, 10, generator=g)
    chosen, weights = torch.zeros(9, 3, dtype=torch.int32, device="cuda"), torch.zeros(9, 3, dtype=torch.float32, device="cuda")
    k.route_scored(z.cuda(), None, 3, 1, 1, 1.0, chosen, weights)
    assert torch.equal(chosen.cpu().long(), torch.topk(z, 3, dim=-1).indices)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer_i", [("A", 0), ("A", 1), ("B", 0), ("C", 0), ("C", 1), ("D", 0), ("D", 1)])
def test_feed_forwards_alone(name, layer_i, dtype):
    m = MODELS[name]
    cfg = m["cfg"]
    W = {k: v for k, v in draw_weights(cfg, m["seed"]).items() if k.startswith(f"l{layer_i}.mlp.")}
    mlp = cfg["layers"][layer_i]["mlp"]
    prefix = f"l{layer_i}."
    part = build_part("feed_forward", config_from_dict(cfg).layers[layer_i]["mlp"], prefix)
    hs = PartHarness(dtype, CacheSpec(entries=1, heads=1, head_dim=8), page_size=64, n_pages=16, max_seq_len=1024)
    part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
    Wd = {k: v.double() for k, v in W.items()}
    for T in (1, 5, 70, 400):            # 400 rows: many rows an expert, the tiles through LDS
        h = rows_in(T, cfg["width"], 19 + T, dtype, 1.5)
        ref = P.feed_forward(Wd, prefix + "mlp.", mlp, h.double()).float()
        ctx = hs.ctx([0] * T)
        out = torch.full((T, cfg["width"]), float("nan"), dtype=torch.float32, device="cuda")
        if getattr(part, "stores_output", False):
            part.forward(ctx, h.to(hs.rt.dtype).cuda(), out, accumulate=False)
        else:
            out.zero_()
            part.forward(ctx, h.to(hs.rt.dtype).cuda(), out)
        err = (out.cpu() - ref).abs().max(dim=-1).values
        if mlp["kind"] == "moe":
            # a row whose choice is a close call may go either way: not this test's matter.  Firm rows keep their
            # choice when every score is moved by up to 1e-4
            r = mlp["router"]
            groups = r.get("groups") or {"count": 1, "keep": 1}
            s = P.sigma(h.double() @ Wd[prefix + "mlp.router"].T)
            noise = torch.Generator().manual_seed(T)
            firm = []
            for t in range(T):
                picks = {tuple(P.choose_experts(s[t] + 1e-4 * torch.sign(torch.randn(s.shape[1], generator=noise, dtype=torch.float64)) * i,
                                                Wd[prefix + "mlp.correction"], r["top"], groups["count"], groups["keep"])) for i in (0, 1, 1, 1)}
                firm.append(len(picks) == 1)
            assert sum(firm) >= 0.9 * T
            err = err[torch.tensor(firm)]
        assert float(err.max()) <= part_tol(dtype, ref), (T, int(err.argmax()))
    if mlp["kind"] == "moe":
        # what the test would catch: weights from the choice scores, weights not divided by their sum, one expert fewer
        h = rows_in(70, cfg["width"], 89, dtype, 1.5)
        ref = P.feed_forward(Wd, prefix + "mlp.", mlp, h.double()).float()
        loud = 20 * part_tol("float32", ref)
        r = mlp["router"]
        if r["top"] > 1:
            fewer = dict(mlp, router=dict(r, top=r["top"] - 1))
            assert float((P.feed_forward(Wd, prefix + "mlp.", fewer, h.double()).float() - ref).abs().max()) > loud
        if r["top"] < r["experts"]:
            plain_choice = dict(Wd, **{prefix + "mlp.correction": torch.zeros_like(Wd[prefix + "mlp.correction"])})
            assert float((P.feed_forward(plain_choice, prefix + "mlp.", mlp, h.double()).float() - ref).abs().max()) > loud
        if r["scale"] != 1.0:
            assert float((P.feed_forward(Wd, prefix + "mlp.", dict(mlp, router=dict(r, scale=1.0)), h.double()).float() - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_norm_behind_the_sum_and_the_bent_logits(dtype):
    from axon_amd.kernels import kernels
    k = kernels(dtype)
    g = torch.Generator().manual_seed(2)
    for T, width in ((1, 48), (9, 250), (3, 1030), (70, 4096)):
        y, x = torch.randn(T, width, generator=g) * 3, torch.randn(T, width, generator=g) + 0.5
        gain = 1 + 0.1 * torch.randn(width, generator=g)
        for kind, plain in (("layer", P.layer_norm), ("rms", P.rms)):
            ref = plain(1.7 * x.double() + y.double(), gain.double(), 1e-5)
            xd = x.clone().cuda()
            rounded = torch.zeros(T, width, dtype=k.dtype, device="cuda")
            k.sum_norm(y.cuda(), 1.7, gain.cuda(), 1e-5, kind, xd, rounded)
            assert float((xd.cpu() - ref.float()).abs().max()) <= 2e-5
            assert torch.equal(rounded.cpu(), xd.cpu().to(k.dtype))
            again = x.clone().cuda()
            k.sum_norm(y.cuda(), 1.7, gain.cuda(), 1e-5, kind, again)
            assert torch.equal(again, xd)
        # a layer norm is no RMS norm for rows whose mean is not zero, and alpha stretches the stream
        assert float((P.rms(1.7 * x.double() + y.double(), gain.double(), 1e-5) - P.layer_norm(1.7 * x.double() + y.double(), gain.double(), 1e-5)).abs().max()) > 0.01
        out = torch.zeros(T, width, dtype=k.dtype, device="cuda")
        k.layernorm(x.cuda(), gain.cuda(), 1e-5, out)
        ref = P.layer_norm(x.double(), gain.double(), 1e-5).float()
        assert float((out.float().cpu() - ref).abs().max()) <= (2e-5 if dtype == "float32" else 2e-2) * float(ref.abs().max())
        rows = torch.tensor([T - 1, 0], dtype=torch.int32).cuda()
        picked = torch.zeros(2, width, dtype=k.dtype, device="cuda")
        k.layernorm(x.cuda(), gain.cuda(), 1e-5, picked, rows)
        assert torch.equal(picked, out[[T - 1, 0]])
        # rows far from zero: the variance is taken of the deviations, not as mean(x^2) - mean^2
        far = (torch.randn(T, width, generator=g) * 0.01 + 300.0)
        k.layernorm(far.cuda(), gain.cuda(), 1e-7, out)
        ref = P.layer_norm(far.double(), gain.double(), 1e-7).float()
        assert float((out.float().cpu() - ref).abs().max()) <= (2e-3 if dtype == "float32" else 3e-2) * float(ref.abs().max())
    z = (torch.randn(5, 777, generator=g) * 40).cuda()
    wide = torch.zeros(5, 800, device="cuda")
    wide[:, :777] = z
    k.softcap(wide[:, :777], 11.0)
    assert float((wide[:, :777].cpu() - 11.0 * torch.tanh(z.cpu().double() / 11.0).float()).abs().max()) <= 1e-5
    assert float(wide[:, 777:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_rotation_in_neighbouring_pairs_with_ramped_frequencies(dtype):
    """The query's rotated part through the kernel that lays queries out for the attention, against the
    plain rotation: pairs (2k, 2k + 1), frequencies ramped by pair index, cos and sin times their factor,
    the places behind the rotated dims passed on; positions up to far beyond the original context."""
    from axon_amd.kernels import kernels
    k = kernels(dtype)
    g = torch.Generator().manual_seed(4)
    for dim, rot_dim, dims, base, scaling in ((8, 4, 4, 100.0, (4.0, 16, 8.0, 1.0)), (40, 16, 16, 5e5, (6.0, 256, 24.0, 1.0)),
                                              (8, 32, 16, 500.0, None), (16, 64, 64, 1e4, (2.0, 32, 4.0, 0.5)), (24, 2, 2, 7.0, None)):
        rot = {"base": base, "dims": dims}
        if scaling:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        enc = build_part("position", PartSpec("rope", {"head_dim": rot_dim, "rotary_dim": dims, "theta": base, "pairing": "neighbours",
                                                       **({"scaling": dict(rot["scaling"], kind="ramp")} if scaling else {})}))
        H, rank = 3, 8
        pos = torch.tensor([0, 1, 2, 3, 63, 64, 511, 512, 5000, 100000], dtype=torch.int32)
        T = pos.numel()
        q = torch.randn(T, H * (dim + rot_dim), generator=g)
        table = torch.zeros(T, dims // 2, 2, dtype=torch.float32, device="cuda")
        k.rope_table(pos.cuda(), enc.frequencies().cuda(), table)
        q_full = torch.zeros(T, H * (rank + rot_dim), dtype=torch.float32, device="cuda")
        k.latent_query_rope(q.cuda(), dim, rot_dim, dims, table, q_full, rank, H, neighbours=True, magnitude=enc.magnitude)
        want = P.rotate_neighbours(q.double().view(T, H, dim + rot_dim)[..., dim:], pos.long(), rot).float()
        got = q_full.cpu().view(T, H, rank + rot_dim)[..., rank:]
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max()), (dim, rot_dim, dims)
