"""Random Napizen configurations through the engine against the plain implementation: layer counts and
orders of feed-forwards (gated, experts, none), head counts in and out of the matrix cores' tiles, query,
rotated, value and latent sizes that differ from layer to layer, frequencies ramped or not, experts in
groups of every shape, stretches of the stream, scales and bends; three unequal requests side by side in
random portions with shuffled pages, and the longest alone."""
import random

import pytest
import torch

from helpers import engine_for, tolerance
from napizen_models import att, config, dense, draw_weights, layer, moe, write_model
from plain import napizen_plain as P
from test_napizen_gpu import SLACK, run_schedule

pytestmark = pytest.mark.gpu


def random_config(rng):
    width = rng.choice([48, 64, 96, 128, 256])
    layers = []
    for _ in range(rng.randint(2, 5)):
        heads = rng.choice([1, 2, 3, 4, 5, 8, 16, 16, 32])
        dim = rng.choice([8, 16, 24, 32, 64])
        rot_dim = rng.choice([2, 4, 8, 16, 32, 64])
        rank = rng.choice([12, 16, 32, 64, 96, 128, 192])
        # a score's spread near 2.5 under the drawn weights, whatever the sizes
        scale = 2.5 / (2.25 * dim ** 0.5 + 1.5 * rot_dim ** 0.5)
        mixer = att(heads, dim, rot_dim, rng.choice([8, 16, 24, 48, 64]), rank, base=rng.choice([50.0, 10000.0, 1e6]), scale=scale,
                    scaling=rng.choice([None, (4.0, 16, 8.0, 1.0), (6.0, 256, 24.0, 2.0), (2.0, 64, 4.0, 0.5)]))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = dense(rng.choice([40, 64, 200, 320]))
        else:
            count = rng.choice([1, 2, 3, 4, 8])
            size = rng.choice([1, 2, 3, 4, 8])
            keep = rng.randint(1, count)
            top = rng.randint(1, min(keep * size, 8))
            mlp = moe(count * size, top, rng.choice([8, 24, 64]), rng.choice([(count, keep), None]) if keep == count == 1 else (count, keep),
                      rng.choice([1.0, 1.5, 2.5]))
        layers.append(layer(mixer, mlp))
    return config(width, rng.choice([97, 256, 1000]), layers, eps=rng.choice([1e-5, 1e-6]), alpha=rng.choice([0.7, 1.0, 1.6, 2.5]),
                  scale=rng.choice([1.0, 3.0, width ** 0.5]), softcap=rng.choice([0, 8.0, 30.0]))


@pytest.mark.parametrize("seed", range(10))
def test_a_random_configuration_in_a_random_schedule(seed, tmp_path):
    rng = random.Random(2000 + seed)
    cfg = random_config(rng)
    W = draw_weights(cfg, seed)
    folder = write_model(str(tmp_path / "model"), cfg, W)
    g = torch.Generator().manual_seed(seed)
    lengths = [rng.randint(1, 40), rng.randint(100, 300), rng.randint(40, 150)]
    seqs = {i: torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
    Wd = {k: v.double() for k, v in W.items()}
    refs = {i: P.forward_logits(cfg, Wd, s).float() for i, s in seqs.items()}
    at, sched = {i: 0 for i in seqs}, []
    while any(at[i] < lengths[i] for i in seqs):
        step = []
        for i in seqs:
            if at[i] < lengths[i] and rng.random() < 0.8:
                n = min(rng.choice([1, 1, 2, 5, 16, 17, 33, 64, 100]), lengths[i] - at[i])
                step.append((i, n))
                at[i] += n
        if step:
            sched.append(step)
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folder, dtype, 64, 3 * 5 + 2, max_seqs=3, max_seq_len=320, shuffle_pages_seed=seed)
        got, chose = run_schedule(eng, cfg, seqs, sched)
        alone, chose_alone = run_schedule(eng, cfg, {1: seqs[1]}, [[(1, lengths[1])]])
        got["alone"], chose["alone"] = alone[1], chose_alone[1]
        for i, rows in got.items():
            r = 1 if i == "alone" else i
            # 16 bits: the plain run takes the engine's experts where these are a close call of its own choice
            ref = refs[r] if dtype == "float32" else P.forward_logits(cfg, Wd, seqs[r], chose[i], SLACK).float()
            err = (rows - ref).abs().max(dim=-1).values / tolerance(dtype, ref)
            if dtype == "float32":
                assert float(err.max()) <= 2.0, (i, float(err.max()), cfg)
            else:
                # 16 bits: a norm behind every sum passes each rounding on; single rows of deep random models lie at a few
                # per cent of the logits' range, the typical row well inside
                assert float(err.max()) <= 6.0 and float(err.median()) <= 2.0, (i, float(err.max()), float(err.median()), cfg)
        eng.cache.check()
        assert not eng.live
