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
    # this build: median 0.99, mean 0.972-0.977, lowest 0.83-0.875 (tiles over fused rank sets and their pricing
    # brought the mean up from 0.935-0.94).  The two lowest move with the machine and the run: the same two plans,
    # (932,93,512)/(1,2,0) and (8,27,84,46,65)/(2,1,0,4,3) with 4-byte elements, read 0.875 / 0.91 in one run and
    # 0.83 / 0.84 in another, because these tensors fit the memory-side cache and the measured plan also profits
    # from timing noise in its favour - so median and mean carry the check and the tail gets a wide bound.
    ordered = np.sort(ratios)
    assert np.median(ratios) >= 0.95
    assert ratios.mean() >= 0.945
    assert ordered[1] >= 0.80
    assert ordered[0] >= 0.75


def aligned_set(seed=77):
    """Twelve seeded tensors of about 2e8 elements whose rows start on 128-byte lines on both sides, the class in
    which the cost model's line counts are the same for nearly all candidates and what decides is which
    addresses are in flight at one time: four batched transposes (2^a, 2^j, 2^b, 3) -> (2^b, 2^j, 2^a, 3), four
    tensors of ranks 3-6 whose extents are powers of two (one of them times three), four whose extents are
    multiples of 32; 8- and 4-byte elements alternating."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < 4:
        a, b = int(rng.integers(8, 13)), int(rng.integers(8, 13))
        j = 26 - a - b
        if j < 1:
            continue
        out.append(dict(dim=(2 ** a, 2 ** j, 2 ** b, 3), perm=(2, 1, 0, 3)))
    while len(out) < 8:
        rank = 3 + len(out) % 4
        cuts = np.sort(rng.choice(np.arange(1, 26), size=rank - 1, replace=False))
        bits = np.diff(np.concatenate(([0], cuts, [26])))
        dim = [int(2 ** e) for e in bits]
        dim[int(rng.integers(rank))] *= 3
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)) or perm[0] == 0:
            continue
        out.append(dict(dim=tuple(dim), perm=tuple(perm)))
    while len(out) < 12:
        rank = 3 + len(out) % 3
        dim = bc.random_dims(rng, rank, target=2.0e8 / 32 ** 2, tol=0.05)
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)) or perm[0] == 0:
            continue
        dim = list(dim)
        dim[0] *= 32            # the rank that leads the input
        dim[perm[0]] *= 32      # the rank that leads the output
        out.append(dict(dim=tuple(int(d) for d in dim), perm=tuple(perm)))
    for i, c in enumerate(out):
        c["name"] = "A%02d" % i
        c["es"] = 8 if i % 2 == 0 else 4
    return out


def test_heuristic_plans_on_line_aligned_tensors():
    """The second set: tensors on the line grid (powers of two above all), where cuttPlan used to reach 0.90 of
    the measured plan's rate in the mean and 0.61 at worst."""
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    import cutt_amd
    import sweep_runner
    cutt_amd.lib()
    cutt_amd.set_method_override(0)
    ratios = []
    for cfg in aligned_set():
        r = sweep_runner.run_tensor(cfg, reps=5)
        assert r["plan"]["exact"] and r["measure"]["exact"], cfg
        q = r["measure"]["ms"] / r["plan"]["ms"]
        ratios.append(q)
        say("%s dim=%s perm=%s es=%d: heuristic %s %.0f GB/s, measured %s %.0f GB/s, ratio %.3f" %
            (cfg["name"], cfg["dim"], cfg["perm"], cfg["es"], r["plan"]["method"], r["plan"]["gbs"],
             r["measure"]["method"], r["measure"]["gbs"], q))
    ratios = np.array(ratios)
    say("line-aligned set, heuristic / measured throughput: median %.3f mean %.3f min %.3f" %
        (np.median(ratios), ratios.mean(), ratios.min()))
    # this build: median 0.961, mean 0.951, lowest 0.868
    assert ratios.mean() >= 0.925
    assert ratios.min() >= 0.80
