"""Pins the quality of the heuristic planner: on a seeded set of 24 tensors (ranks 2-7, 4- and
8-byte elements, about 5e7 elements) the plan cuttPlan picks from its cost model must stay close to
the plan cuttPlanMeasure finds by timing the candidates (the acceptance idea of the reference's
findMispredictionBest, src/cutt.cpp:264).  The cost model's constants are fitted to measurements;
this test is what notices when a change to them makes the choices worse."""
import sys

import numpy as np
import pytest

import baseline_configs as bc

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def quality_set(count=24, seed=4242, elems=5.0e7):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        i = len(out)
        rank = 2 + i % 6
        if (i // 6) % 2 == 0:   # uneven extents
            dim = bc.random_dims(rng, rank, target=elems, tol=0.05)
        else:                   # extents within a factor of ten of each other, shuffled
            f = 1.0 + np.arange(rank) * 9.0 / max(rank - 1, 1)
            scale = (elems * rng.uniform(0.7, 1.3) / np.prod(f)) ** (1.0 / rank)
            dim = [int(d) for d in np.maximum(2, np.round(f * scale))]
            rng.shuffle(dim)
            dim = [int(d) for d in dim]
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)):
            continue
        out.append(dict(name="Q%02d" % i, dim=tuple(dim), perm=tuple(perm), es=8 if i % 2 == 0 else 4))
    return out


def test_heuristic_plans_are_close_to_measured_plans():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    import cutt_amd
    import sweep_runner
    cutt_amd.lib()
    cutt_amd.set_method_override(0)
    ratios = []
    for cfg in quality_set():
        r = sweep_runner.run_tensor(cfg, reps=5)
        assert r["plan"]["exact"] and r["measure"]["exact"], cfg
        q = r["measure"]["ms"] / r["plan"]["ms"]   # throughput of the heuristic plan / of the measured plan
        ratios.append(q)
        say("%s dim=%s perm=%s es=%d: heuristic %s %.0f GB/s, measured %s %.0f GB/s, ratio %.3f" %
            (cfg["name"], cfg["dim"], cfg["perm"], cfg["es"], r["plan"]["method"], r["plan"]["gbs"],
             r["measure"]["method"], r["measure"]["gbs"], q))
    ratios = np.array(ratios)
    say("heuristic / measured throughput: median %.3f mean %.3f min %.3f" % (np.median(ratios), ratios.mean(), ratios.min()))
    # this build: median 0.943-0.945, mean 0.935-0.94; the minimum moves with the machine (0.85 on one MI355X,
    # 0.78 on another, both from 4-byte PackedSplit plans whose two best candidates the model rates equal), so one
    # outlier is allowed for and the rest is held to the tighter bound.  (The measured plan also profits from
    # timing noise in its favour.)
    ordered = np.sort(ratios)
    assert np.median(ratios) >= 0.92
    assert ratios.mean() >= 0.915
    assert ordered[1] >= 0.80
    assert ordered[0] >= 0.70
