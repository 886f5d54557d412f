"""Sefevik configurations drawn at random, each replayed in portions and mixed against the plain implementation: any
order of the two mixers, layers that read an earlier layer's rows with a window of their own, layers without a
feed-forward, with and without a pair table, sizes that are odd, multiples of 8 (the MFMA attention) or of 128 (the
tiled products), pages of 8 to 64 tokens.  Every logit is compared.

Tolerances: float32 2e-4 (times the logits' rms beyond 1).  bfloat16: how far the rounding of activations moves a logit
depends on the configuration drawn (recurrences in a row and the activation's quadratic branch amplify it; the plain
attention kernel and the MFMA one give the same errors at the same positions), so a position's largest error is held
to 0.3 of the logits' rms, where a wrong page, a dropped key or a lost state moves logits by their own size, and nine
positions in ten to 0.1 of it."""
import random

import pytest
import torch

from tests import replay_cases as rc
from tests import sefevik_cases as sc
from tests.gpu_util import require_gpu

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(7000 + seed)
    tiled = seed % 3 == 0
    width = rng.choice([128, 256]) if tiled else rng.choice([24, 40, 56, 72, 90, 100])
    layers, sources = [], []
    for i in range(rng.randint(1, 5)):
        ff = None if rng.random() < 0.2 else (rng.choice([128, 256, 384]) if tiled else rng.randint(20, 150))
        if rng.random() < 0.4:
            layers.append(sc._layer("mingru", dict(width=rng.choice([128, 256]) if tiled else rng.randint(9, 90)), ff))
            continue
        window = rng.choice([None, 1, 3, 17, 40, 64, 100])
        if sources and rng.random() < 0.4:
            src = rng.choice(sources)
            m = dict(layers[src]["mixer"])
            m.pop("mask", None)
            m.pop("kv_from", None)
            m.update(heads=rng.randint(1, 6), dim=rng.choice([4, 8, 16, 24]), vdim=rng.choice([4, 8, 12, 16, 32]), scale=rng.choice([0.2, 0.5, 1.0]),
                     kv_from=src)
            if window is not None:
                m["mask"] = dict(size=window)
        else:
            aligned = rng.random() < 0.6
            rot_dim = rng.choice([8, 16, 32]) if aligned else rng.choice([2, 6, 10])
            rank = rng.choice([8, 24, 64, 112]) if aligned else rng.choice([5, 12, 30])
            scaling = None if rng.random() < 0.3 else dict(factor=rng.choice([2.0, 8.0, 16.0]), original=rng.choice([16, 64, 256]),
                                                           fast=rng.choice([4.0, 16.0]), slow=rng.choice([1.0, 2.0]))
            m = sc._latent(rng.randint(1, 6), rng.choice([4, 8, 16, 24]), rot_dim, rng.choice([4, 8, 12, 16, 32]), rank, rng.choice([0.2, 0.5, 1.0]),
                           window=window, base=rng.choice([100.0, 1e4, 5e5]), dims=rng.choice([rot_dim, rot_dim, max(2, rot_dim - 2 - rot_dim % 2)]),
                           scaling=scaling)
            sources.append(i)
        layers.append(sc._layer("latent_attention", m, ff))
    cfg = dict(architecture="Sefevik", vocab=rng.randint(50, 600), width=width, norm=dict(eps=rng.choice([1e-6, 3e-6, 2e-5])), layers=layers)
    if rng.random() < 0.7:
        cfg["embedding"] = dict(bigram=dict(buckets=rng.randint(3, 300), mul_prev=rng.randint(1, 50), mul_cur=rng.randint(1, 50)))
    return cfg, rng.choice([8, 16, 32, 64])


@pytest.mark.parametrize("seed", range(30))
def test_random_configuration(seed, tmp_path):
    require_gpu()
    cfg, page = draw_config(seed)
    what = "seed %d: width %d, page %d, layers %s" % (seed, cfg["width"], page, [(l["type"], l["mixer"], l["mlp"]) for l in cfg["layers"]])
    print(what, flush=True)
    folder = sc.write_model(str(tmp_path / "m"), cfg, 500 + seed)
    rng = random.Random(seed)
    reqs = rc.random_requests(cfg["vocab"], [rng.randint(1, 150) for _ in range(5)] + [140], seed=seed)
    ref = sc.plain_logits(folder, reqs)
    rms = float(torch.cat(list(ref.values())).pow(2).mean().sqrt())
    for dtype in ("float32", "bfloat16"):
        tol = dict(atol=2e-4 * max(1.0, rms), rtol=2e-4)
        for mode, steps in (("portions", rc.portions(reqs)), ("mixed", rc.mixed(reqs, seed=seed))):
            out = tmp_path / ("%s_%s" % (dtype, mode))
            rc.run_replay_inprocess(folder, dtype, str(out), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page), "--poison-cache"])
            got = rc.collect(str(out), steps, cfg["vocab"])
            if dtype == "float32":
                rc.compare(got, ref, what="%s / %s / %s" % (what, dtype, mode), **tol)
                continue
            errs = sorted(float((torch.from_numpy(row).double() - ref[rid][pos].double()).abs().max()) for (rid, pos), row in got.items())
            assert all(e == e for e in errs), "%s / %s: a logit is not a number" % (what, mode)
            assert errs[-1] <= 0.3 * max(1.0, rms) and errs[int(0.9 * len(errs))] <= 0.1 * max(1.0, rms), \
                "%s / bfloat16 / %s: largest error %.3f, 90th centile %.3f at logits of rms %.2f" % (what, mode, errs[-1], errs[int(0.9 * len(errs))], rms)
