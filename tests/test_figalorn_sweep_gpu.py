"""Random Figalorn configurations through the engine against the plain implementation: layer orders, loops,
head counts and groups, key and value sizes in and out of the matrix cores' tiles, rotated dims, windows and
chunks from one position to several pages, with and without bend, scaling and feed-forward; three unequal
requests side by side in random portions with shuffled pages, and the longest alone."""
import random

import pytest
import torch

from figalorn_models import config, diff, draw_weights, keyed, layer, write_model
from helpers import engine_for, tolerance
from plain import figalorn_plain as P
from test_figalorn_gpu import run_schedule

pytestmark = pytest.mark.gpu


def random_config(rng):
    width = rng.choice([64, 96, 128, 192, 320])
    layers = []
    for _ in range(rng.randint(2, 5)):
        heads = rng.choice([1, 2, 3, 4, 6, 8, 12])
        kv = rng.choice([k for k in (1, 2, 3, 4, 6, 8, 12) if heads % k == 0])
        ff = rng.choice([None, 64, 96, 200, 384])
        if rng.random() < 0.5:
            dim = rng.choice([8, 12, 16, 24, 32, 40, 48, 64, 96, 128])
            rot = rng.choice([r for r in (2, 4, 8, 12, 16, 32, 64, dim) if r <= dim and r % 2 == 0])
            layers.append(layer(keyed(heads, kv, dim, window=rng.choice([1, 2, 17, 63, 64, 65, 128, 200, 300]), rot_dims=rot,
                                      softcap=rng.choice([0, 5.0, 30.0, 50.0]),
                                      scaling=rng.choice([None, (4.0, 128, 32.0, 1.0), (8.0, 64, 16.0, 2.0)])), ff))
        else:
            dim = rng.choice([8, 16, 20, 24, 32, 48, 64, 96])
            vdim = rng.choice([16, 24, 32, 48, 64, 96, 128, 160, 256])
            rot = rng.choice([r for r in (2, 4, 8, 12, 16, 32, 64, dim) if r <= dim and r % 2 == 0])
            layers.append(layer(diff(heads, kv, dim, vdim, chunk=rng.choice([1, 3, 40, 64, 100, 128, 256]), rot_dims=rot,
                                     d=rng.choice([0.0, 0.1, 0.3, 0.5]),
                                     scaling=rng.choice([None, (8.0, 1.0, 4.0, 64), (2.0, 1.0, 2.0, 32)])), ff))
    loop = None
    if rng.random() < 0.7:
        a = rng.randint(0, len(layers) - 1)
        loop = (a, rng.randint(a + 1, len(layers)), rng.randint(1, 3))
    return config(width, rng.choice([97, 256, 1000]), layers, loop=loop, eps=rng.choice([1e-5, 1e-6]))


@pytest.mark.parametrize("seed", range(12))
def test_a_random_configuration_in_a_random_schedule(seed, tmp_path):
    rng = random.Random(1000 + seed)
    cfg = random_config(rng)
    W = draw_weights(cfg, seed)
    folder = write_model(str(tmp_path / "model"), cfg, W)
    g = torch.Generator().manual_seed(seed)
    lengths = [rng.randint(1, 40), rng.randint(100, 330), rng.randint(40, 150)]
    seqs = {i: torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
    Wd = {k: v.double() for k, v in W.items()}
    refs = {i: P.forward(cfg, Wd, s).float() for i, s in seqs.items()}
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
        eng = engine_for(folder, dtype, 64, 3 * 6 + 2, max_seqs=3, max_seq_len=384, shuffle_pages_seed=seed)
        got = run_schedule(eng, seqs, sched)
        got["alone"] = run_schedule(eng, {1: seqs[1]}, [[(1, lengths[1])]])[1]
        for i, rows in got.items():
            ref = refs[1 if i == "alone" else i]
            err = (rows - ref).abs().max(dim=-1).values / tolerance(dtype, ref)
            if dtype == "float32":
                assert float(err.max()) <= 1.0, (i, cfg)
            else:
                # 16 bits: deep random models with sharp scores put single rows at 2.5 % of the logits' range, whichever
                # kernel runs; the typical row stays well inside 1 %
                assert float(err.max()) <= 4.0 and float(err.median()) <= 1.0, (i, float(err.max()), cfg)
        eng.cache.check()
        assert not eng.live
