"""The Zugutar decoder through the engine against the plain implementation (tests/plain/zugutar_plain.py):
whole prompts, decoding token by token from the first token on, portions down to two tokens, unequal
requests side by side with pages and slots that come round again, long decoding across pages, generation
through the engine's own entry point, the command line, the trace replay program, and every mechanism alone
with weights or inputs made so that a fault shows (a sink left out, a far key lost, a state not carried
across a cut, a temperature one position off, a router's weight on the wrong side of its expert: each
differs from the plain implementation by far more than the tolerance)."""
import math

import pytest
import torch

import axon_amd
from axon_amd.config import config_from_dict
from axon_amd.engine import StepEntry
from axon_amd.parts import CacheBinding, build_part
from axon_amd.weights import WeightStore
from gpu_helpers import DTYPES, DictSource, PartHarness
from helpers import TraceBuilder, engine_for, run_trace, tolerance
from plain import zugutar_plain as P
from zugutar_models import MODELS, att, config, draw_weights, layer, left, make, moe, pair, right

pytestmark = pytest.mark.gpu

SLACK = 0.05          # how far 16 bits of stream may move a router's score


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = make(str(tmp_path_factory.mktemp("zugutar_" + name)), name)
        return made[name]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    """The plain implementation's logits of a model's test sequences.  float32: its own choice of experts.
    bfloat16: with the experts the engine chose where these are a close call of its own choice (16 bits
    decide a close call either way, and every later row sees it)."""
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


def sequences(name, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, MODELS[name]["cfg"]["vocab"], (n,), generator=g).tolist() for n in lengths]


def assert_close(got, ref, dtype, what):
    """Rows of logits against the plain implementation's, every row.  32-bit: every row within rounding.  16 bits:
    the design norms a side's gated output in parts of few values, and a row whose part happens to be small passes
    its rounding on many times enlarged (measured: a row of a model here whose layer, given the engine's own input,
    is right to 0.05, leaves that layer 0.8 off); so one row in a hundred may reach twice the limit of the others."""
    err = (got - ref).abs().max(dim=-1).values
    limit = tolerance(dtype, ref) * (2.0 if dtype == "float32" else 3.0)
    if dtype == "float32":
        assert float(err.max()) <= limit, f"{what}: {float(err.max())} > {limit} at row {int(err.argmax())}"
        return
    over = int((err > limit).sum())
    assert over <= max(1, len(err) // 100) and float(err.max()) <= 2 * limit, \
        f"{what}: {over} of {len(err)} rows over {limit}, the worst {float(err.max())} at row {int(err.argmax())}"


class RouterLog:
    """What the engine's router chose, launch by launch: the kernels' entry is wrapped while a schedule runs."""

    def __init__(self, eng):
        self.k, self.calls = eng.rt.k, []

    def __enter__(self):
        inner = self.k.route_scored

        def logged(logits, correction, top, groups, keep, scale, chosen, weights, **kw):
            inner(logits, correction, top, groups, keep, scale, chosen, weights, **kw)
            self.calls.append(chosen.cpu().tolist())
        self.k.route_scored = logged
        return self

    def __exit__(self, *exc):
        del self.k.route_scored


def run_schedule(eng, name, seqs, schedule):
    """schedule: steps of [(request, tokens)]; every position's logits are asked for.  A request ends with
    its last token.  Returns ({request: [len, vocab]}, {request: {layer run: chosen experts by position}})."""
    cfg = MODELS[name]["cfg"] if isinstance(name, str) else name
    routed = [run for run, (i, _) in enumerate(P.run_order(cfg)) if cfg["layers"][i].get("mlp")]
    at = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    chose = {r: {run: [] for run in routed} for r in seqs}
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
                for run, call in zip(routed, log.calls):
                    chose[e.id][run] += call[row:row + len(e.tokens)]
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
    # from the first token on, one token a step: the first tokens of a sequence (a state and a convolution that
    # start from nothing), every page's edge, every edge of the query temperature
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
        sched, rest, i = [], n, 0
        while rest:
            take = min(cuts[i % len(cuts)], rest)
            sched.append([("a", take)])
            rest -= take
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
    # three slots and a pool for the three longest live at once: later requests get the pages, the slots and
    # the state rows of finished ones
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
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_long_stretches_run_the_scan_in_segments(folders, plain_logits, name, dtype):
    """Hundreds of tokens of a request in one step: the scan cuts the stretch into segments that run side by side,
    folds their end states and adds the carried-in states' share; the state it leaves is what later portions and
    decoded tokens go on from.  Beside a short request in the same step, whose stretch is one segment."""
    n = 420
    long, short = sequences(name, [n, 9], seed=5)
    page = MODELS[name]["page"]
    eng = engine_for(folders(name), dtype, page, -(-n // page) + 4, max_seqs=2, max_seq_len=448, max_batch_tokens=512)
    seen = []
    inner = eng.rt.k.state_space_scan

    def logged(*a, segments=None, **kw):
        seen.append(None if segments is None else segments[0].shape[0])
        return inner(*a, segments=segments, **kw)
    eng.rt.k.state_space_scan = logged
    try:
        got, chose = run_schedule(eng, name, {"a": long, "b": short}, [[("a", 300), ("b", 4)], [("a", 1), ("b", 5)], [("a", 2)], [("a", 117)]])
    finally:
        del eng.rt.k.state_space_scan
    assert any(k is not None and k > 2 for k in seen) and any(k is None for k in seen)
    assert_close(got["a"], plain_logits(name, long, dtype, chose["a"]), dtype, "the long request")
    assert_close(got["b"], plain_logits(name, short, dtype, chose["b"]), dtype, "the short request beside it")
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
    name = "C"
    cfg, W = P.load_plain(folders(name))
    p, q = sequences(name, [9, 14], seed=9)
    axon = [sys.executable, os.path.join(ROOT, "bin", "axon")]
    ids = lambda seq: " ".join(map(str, seq))
    r = subprocess.run(axon + ["gen", folders(name), ids(p), ids(q), "-n", "8", "--dtype", "float32", "--page-size", "64"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [[int(t) for t in line.split()] for line in r.stdout.splitlines()] == [
        P.greedy_generate(cfg, W, p, 8), P.greedy_generate(cfg, W, q, 8)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_replay_program_runs_the_design(folders, plain_logits, tmp_path, dtype):
    name = "B"
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


def one_layer(width, mixer, mlp=None, eps=1e-5):
    return config(width, 16, [layer(mixer, mlp)], eps=eps)


def side_spec(cfg, side=None):
    """The design's mixer of layer 0 as the configuration reader describes it (a side of a pair, if named)."""
    spec = config_from_dict(cfg).layers[0]["mixer"]
    return spec if side is None else spec.params[side]


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


def loaded(part, W, harness):
    part.load(WeightStore(DictSource(W), harness.rt.device, harness.rt.dtype), harness.rt)
    return part


CUTS = lambda T, page: [[T], [page - 1] + [1] * 8 + [T - page - 7], [2, 1, 1, 3] + [1] * 30 + [64, 2, T - 103], [1] * T]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,vdim,state,groups,conv,norm_groups", [(3, 5, 7, 1, 3, 3), (4, 32, 64, 2, 4, 2), (2, 24, 130, 2, 2, 1),
                                                                      (1, 40, 16, 1, 1, 1), (6, 16, 200, 3, 5, 6), (8, 64, 128, 2, 4, 2)])
def test_the_state_space_side_alone_in_portions(heads, vdim, state, groups, conv, norm_groups, dtype):
    """The scan with its state and the convolution's kept inputs carried across cuts of every kind: whole, a
    token at a time from the first token on (a state that starts from nothing), portions that end inside the
    convolution's reach.  Decays from a step to hundreds of steps."""
    width, T = 48, 140
    cfg = one_layer(width, pair(left(1, 1, 8, 8), right(heads, vdim, state, groups, conv, norm_groups)))
    W = {k: v for k, v in draw_weights(cfg, 41).items() if k.startswith("l0.mix.right.")}
    c = cfg["layers"][0]["mixer"]["right"]
    h = rows_in(T, width, 13, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.state_space(Wd, "l0.mix.right.", c, h.double(), 1e-5).float()
    for cuts in CUTS(T, 16):
        part = build_part("mixer", side_spec(cfg, "right"), "l0.")
        ss = part.state_spec()
        hs = PartHarness(dtype, None, state_elems=[(ss.elems, ss.dtype)])
        got = run_mixer(loaded(part, W, hs), hs, h, cuts, width)
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    # what the test would catch: a state that starts anew at a cut, a convolution that forgets its inputs there
    loud = 20 * part_tol("float32", ref)
    cut = 100
    anew = torch.cat([P.state_space(Wd, "l0.mix.right.", c, h[:cut].double(), 1e-5), P.state_space(Wd, "l0.mix.right.", c, h[cut:].double(), 1e-5)])
    assert float((anew.float() - ref)[cut + 8:].abs().max()) > loud
    no_gate = dict(Wd, **{"l0.mix.right.in": Wd["l0.mix.right.in"].clone()})
    no_gate["l0.mix.right.in"][:heads * vdim] = 0
    assert float((P.state_space(no_gate, "l0.mix.right.", c, h.double(), 1e-5).float() - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slow_state_remembers_an_input_hundreds_of_positions_back(dtype):
    """One head whose decay is set by hand to 0.999 a step, fed a loud row at position 3 and faint rows after
    it: 600 positions on, the output is still that row's doing, in a prompt and decoded one token at a time."""
    width, T = 32, 640
    cfg = one_layer(width, pair(left(1, 1, 8, 8), right(1, 16, 8, 1, 2, 1)))
    W = {k: v for k, v in draw_weights(cfg, 43).items() if k.startswith("l0.mix.right.")}
    W["l0.mix.right.A_log"] = torch.tensor([math.log(0.001)])
    W["l0.mix.right.dt_bias"] = torch.tensor([0.5413])              # softplus gives 1: a = exp(-0.001)
    W["l0.mix.right.in"][-1] = 0                                    # dt does not depend on the input
    W["l0.mix.right.D"] = torch.zeros(1)
    W["l0.mix.right.conv.b"] = torch.zeros_like(W["l0.mix.right.conv.b"])      # faint rows leave faint traces
    W = {k: v.to(torch.bfloat16).float() for k, v in W.items()}
    c = cfg["layers"][0]["mixer"]["right"]
    h = rows_in(T, width, 15, dtype, scale=0.02)
    h[3] = rows_in(1, width, 16, dtype, scale=3.0)[0]
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.state_space(Wd, "l0.mix.right.", c, h.double(), 1e-5).float()
    quiet = h.clone()
    quiet[3] = h[4]
    assert float((P.state_space(Wd, "l0.mix.right.", c, quiet.double(), 1e-5).float() - ref)[600:].abs().max()) > 0.2 * float(ref[600:].abs().max())
    for cuts in ([T], [600] + [1] * 40, [2, 3, 64, 129, 1, 1, 400, 38, 2]):
        part = build_part("mixer", side_spec(cfg, "right"), "l0.")
        ss = part.state_spec()
        hs = PartHarness(dtype, None, state_elems=[(ss.elems, ss.dtype)], max_seq_len=1024)
        got = run_mixer(loaded(part, W, hs), hs, h, cuts, width)
        assert float((got - ref)[600:].abs().max()) <= part_tol(dtype, ref), cuts


def check_attention(cfg, W, scope, plain, page, dtype, T, cut_sets, side=None):
    part_spec = side_spec(cfg, side)
    h = rows_in(T, cfg["width"], 13, dtype)
    ref = plain(W, h).float()
    for cuts in cut_sets:
        part = build_part("mixer", part_spec, "l0.")
        hs = PartHarness(dtype, part.cache_spec(), page_size=page, n_pages=-(-T // page) + 3, max_seq_len=1024)
        got = run_mixer(loaded(part, W, hs), hs, h, cuts, cfg["width"])
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    return h, ref


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,dims,page", [(3, 1, 10, 6, 4, 8), (8, 2, 32, 32, 32, 64), (4, 4, 64, 48, 32, 64),
                                                               (1, 1, 24, 40, 0, 16), (6, 3, 48, 16, 48, 128), (8, 2, 128, 128, 64, 64),
                                                               (32, 2, 64, 64, 64, 64), (4, 1, 256, 192, 128, 64)])
def test_the_attention_side_with_a_sink_and_a_gate_a_head(heads, kv_heads, dim, vdim, dims, page, dtype):
    cfg = one_layer(64, pair(left(heads, kv_heads, dim, vdim, dims=dims, base=100.0), right(1, 8, 8)))
    W = {k: v for k, v in draw_weights(cfg, 31).items() if k.startswith("l0.mix.left.")}
    c = cfg["layers"][0]["mixer"]["left"]
    plain = lambda W, h, c=c: P.left_attention({k: v.double() for k, v in W.items()}, "l0.mix.left.", c, h.double(), 1e-5)
    T = 200
    h, ref = check_attention(cfg, W, "l0.mix.left.", plain, page, dtype, T, CUTS(T, page)[:3], side="left")
    # what the test would catch: the sink left out, the gate left out, the norm's gain left out, all places rotated
    loud = 20 * part_tol("float32", ref)
    Wd = {k: v.double() for k, v in W.items()}
    no_sink = P.heads_attention
    try:
        P.heads_attention = lambda q, k, v, scale, sink: no_sink(q, k, v, scale, False)
        assert float((plain(W, h).float() - ref).abs().max()) > loud
    finally:
        P.heads_attention = no_sink
    assert float((plain(dict(W, **{"l0.mix.left.g": torch.zeros_like(W["l0.mix.left.g"])}), h).float() - ref).abs().max()) > loud
    assert float((plain(dict(W, **{"l0.mix.left.k.norm": torch.ones(dim)}), h).float() - ref).abs().max()) > loud
    if 0 < dims < dim:
        everywhere = dict(c, rot=dict(c["rot"], dims=dim if dim % 2 == 0 else dim - 1))
        assert float((plain(W, h, everywhere).float() - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,temp,page", [(4, 2, 6, 10, (0.7, 5), 8), (16, 16, 64, 16, (0.5, 64), 64),
                                                               (2, 1, 24, 40, (0.25, 1), 16), (5, 5, 8, 8, None, 16), (8, 2, 32, 64, (1.0, 63), 64),
                                                               (8, 2, 128, 128, (0.1, 128), 64), (40, 2, 64, 128, (0.5, 100), 64)])
def test_attention_with_a_temperature_by_position_and_a_gate_an_element(heads, kv_heads, dim, vdim, temp, page, dtype):
    """Positions on both sides of every multiple of `every` (and of every - 1: the count goes by p + 1), in
    prompts and decoded."""
    cfg = one_layer(64, att(heads, kv_heads, dim, vdim, temp=temp))
    W = {k: v for k, v in draw_weights(cfg, 33).items() if k.startswith("l0.mix.")}
    c = cfg["layers"][0]["mixer"]
    plain = lambda W, h, c=c: P.plain_attention({k: v.double() for k, v in W.items()}, "l0.mix.", c, h.double())
    T = 200
    h, ref = check_attention(cfg, W, "l0.mix.", plain, page, dtype, T, CUTS(T, page)[:3] + [[60] + [1] * 10 + [56] + [1] * 74])
    loud = 20 * part_tol("float32", ref)
    if temp is not None:
        # a temperature counted from p instead of p + 1 moves every edge by one position
        late = P.plain_attention({k: v.double() for k, v in W.items()}, "l0.mix.", c, h.double(), first_position=-1).float()
        assert float((late - ref).abs().max()) > loud
        assert float((plain(W, h, dict(c, q_temp=None)).float() - ref).abs().max()) > loud
    assert float((plain(dict(W, **{"l0.mix.g": torch.zeros_like(W["l0.mix.g"])}), h).float() - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,heads,kv_heads,page", [("left", 2, 1, 8), ("left", 8, 2, 64), ("attention", 3, 3, 16), ("attention", 16, 4, 64)])
def test_a_key_hundreds_of_positions_back_decides_a_row(kind, heads, kv_heads, page, dtype):
    """Weights set by hand: queries and keys read the same places of the input, values others.  Positions 150
    and 880 hold the same loud row, every other row is faint there: row 880 is then mostly the values at 150
    and at 880 (and, on the side with a sink, the sink's share of nothing), in a prompt and decoded, 730
    positions and many pages back."""
    width, dim, T = 64, 16, 900
    if kind == "left":
        cfg = one_layer(width, pair(left(heads, kv_heads, dim, dim, dims=0, scale=1.0), right(1, 8, 8)))
        scope, c, side = "l0.mix.left.", cfg["layers"][0]["mixer"]["left"], "left"
    else:
        cfg = one_layer(width, att(heads, kv_heads, dim, dim, temp=(0.1, 128), scale=0.4))
        scope, c, side = "l0.mix.", cfg["layers"][0]["mixer"], None
    g = torch.Generator().manual_seed(3)
    W = {scope + "q": torch.cat([torch.eye(dim, width)] * heads), scope + "k": torch.cat([torch.eye(dim, width)] * kv_heads),
         scope + "v": torch.cat([torch.cat([torch.zeros(dim, dim), torch.eye(dim, width - dim)], 1)] * kv_heads),
         scope + "g": torch.zeros(heads if kind == "left" else heads * dim, width),
         scope + "o": torch.randn(width, heads * dim, generator=g).to(torch.bfloat16).float()}
    if kind == "left":
        W[scope + "q.norm"] = W[scope + "k.norm"] = torch.ones(dim)
    h = rows_in(T, width, 17, dtype)
    h[150, :dim] = h[880, :dim] = rows_in(1, dim, 18, dtype)[0] * (1.0 if kind == "left" else 1.5)
    if kind == "attention":         # (on the other side keys are normed, all as long: there the others point elsewhere)
        h[:, :dim] *= torch.where((torch.arange(T) == 150) | (torch.arange(T) == 880), 1.0, 0.1)[:, None]
    Wd = {k: v.double() for k, v in W.items()}
    plain = (lambda hh: P.left_attention(Wd, scope, c, hh.double(), 1e-5)) if kind == "left" else (lambda hh: P.plain_attention(Wd, scope, c, hh.double()))
    ref = plain(h).float()
    lost = h.clone()
    lost[150, dim:] = 0                                     # the far key's values gone: row 880 must show it
    assert float((plain(lost).float() - ref)[880].abs().max()) > 0.1 * float(ref[880].abs().max())
    part_spec = side_spec(cfg, side)
    for cuts in ([T], [870] + [1] * 30, [2, 147, 1, 1, 64, 600, 60, 5] + [1] * 20):
        part = build_part("mixer", part_spec, "l0.")
        hs = PartHarness(dtype, part.cache_spec(), page_size=page, n_pages=-(-T // page) + 3, max_seq_len=1024)
        got = run_mixer(loaded(part, W, hs), hs, h, cuts, width)
        assert float((got - ref)[870:].abs().max()) <= part_tol(dtype, ref), cuts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,ff,shared", [(5, 2, 24, 16), (4, 4, 64, 96), (6, 1, 32, None), (8, 3, 48, 8), (40, 6, 32, 64)])
def test_experts_fed_their_score_times_the_input(experts, top, ff, shared, dtype):
    width, T = 64, 70
    cfg = one_layer(width, att(1, 1, 8, 8), moe(experts, top, ff, shared))
    W = {k: v for k, v in draw_weights(cfg, 35).items() if k.startswith("l0.mlp.")}
    c = cfg["layers"][0]["mlp"]
    part = build_part("feed_forward", config_from_dict(cfg).layers[0]["mlp"], "l0.")
    hs = PartHarness(dtype)
    loaded(part, W, hs)
    h = rows_in(T, width, 19, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    chosen = []
    inner = hs.rt.k.route_scored

    def logged(logits, correction, top_, groups, keep, scale, ch, weights, **kw):
        inner(logits, correction, top_, groups, keep, scale, ch, weights, **kw)
        chosen.append(ch.cpu().tolist())
    hs.rt.k.route_scored = logged
    try:
        out = torch.full((T, width), 1.0, dtype=torch.float32, device="cuda")
        part.forward(hs.ctx([0] * T), h.to(hs.rt.dtype).cuda(), out)                    # adds into what is there
        stored = torch.full((T, width), float("nan"), dtype=torch.float32, device="cuda")
        part.forward(hs.ctx([0] * T), h.to(hs.rt.dtype).cuda(), stored, accumulate=False)
    finally:
        del hs.rt.k.route_scored
    ref = P.experts_ff(Wd, "l0.mlp.", c, h.double(), chosen[0] if dtype == "bfloat16" else None, SLACK).float()
    assert float((stored.cpu() - ref).abs().max()) <= part_tol(dtype, ref)
    assert float((out.cpu() - 1.0 - ref).abs().max()) <= part_tol(dtype, ref)
    # what the test would catch: the score on the expert's output, scores renormalised, the shared expert's gate left out
    loud = 20 * part_tol("float32", ref)
    scores = P.router_scores(Wd, "l0.mlp.", h.double())
    picks = P.choose_experts(scores, top)
    behind = torch.zeros(T, width, dtype=torch.float64)
    over_sum = torch.zeros(T, width, dtype=torch.float64)
    for t in range(T):
        total = sum(scores[t, e] for e in picks[t])
        for e in picks[t]:
            behind[t] += scores[t, e] * P.gated_unit(Wd, f"l0.mlp.e{e}.", h[t].double()[None])[0]
            over_sum[t] += P.gated_unit(Wd, f"l0.mlp.e{e}.", (scores[t, e] / total * h[t].double())[None])[0]
    share = P.sigma(h.double() @ Wd["l0.mlp.shared.sg"].T) * P.gated_unit(Wd, "l0.mlp.shared.", h.double()) if shared else 0.0
    assert float((behind + share - ref).abs().max()) > loud
    assert float((over_sum + share - ref).abs().max()) > loud
    if shared:
        assert float((ref - share + P.gated_unit(Wd, "l0.mlp.shared.", h.double()) - ref).abs().max()) > loud


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_embedding_comes_back_before_a_loops_later_passes_only(folders, plain_logits, dtype):
    """The plain implementation's order of runs and where it adds the embedding's rows is what the engine does:
    a model whose loop adds them before every pass, or never, gives other logits by far."""
    name = "A"
    (seq,) = sequences(name, [40], seed=21)
    cfg, W = P.load_plain(folders(name))
    ref = P.forward_logits(cfg, W, seq).float()
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, 40), max_seqs=1, max_seq_len=64)
    got, chose = run_schedule(eng, name, {"a": seq}, [[("a", 40)]])
    assert_close(got["a"], plain_logits(name, seq, dtype, chose["a"]), dtype, "the looped model")
    order = P.run_order
    try:
        P.run_order = lambda c: [(i, False) for i, _ in order(c)]
        never = P.forward_logits(cfg, W, seq).float()
        P.run_order = lambda c: [(i, i == c["loop"]["start"]) for i, _ in order(c)]
        always = P.forward_logits(cfg, W, seq).float()
    finally:
        P.run_order = order
    loud = 20 * tolerance("float32", ref)
    assert float((never - ref).abs().max()) > loud and float((always - ref).abs().max()) > loud
    assert [i for i, _ in order(cfg)] == [0, 1, 0, 1, 0, 1, 2] and [a for _, a in order(cfg)] == [False, False, True, False, True, False, False]
