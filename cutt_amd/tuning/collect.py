"""Times every candidate plan of random tensors on the current GPU (CUTT_MEASURE_ALL=1) and writes,
per candidate, what the cost model knew (its counters and prediction) beside the measured time.

  python -m cutt_amd.tuning.collect --out samples.json [--seed 1] [--count 200] [--elems 2e8]

Tensors: ranks 2-7, 4- and 8-byte elements alternating, three shape generators in turn - extents
that grow linearly up to ten times the smallest and are then shuffled (the reference's bench 5,
src/cutt_bench.cpp:455-546), extents drawn freely around the geometric mean (its bench 3,
:414-431), and a Dirichlet split of the volume (very uneven extents) - each with a random
non-identity permutation."""
import argparse
import json
import os
import sys

import numpy as np


def shape_ratio(rng, rank, vol, ratio=10):
    f = 1.0 + np.arange(rank) * (ratio - 1.0) / max(rank - 1, 1)
    scale = (vol / np.prod(f)) ** (1.0 / rank)
    dim = np.maximum(2, np.round(f * scale)).astype(np.int64)
    rng.shuffle(dim)
    return [int(d) for d in dim]


def shape_free(rng, rank, vol):
    mean = vol ** (1.0 / rank)
    f = np.maximum(1.0, mean + (2.0 * rng.random(rank) - 1.0) * (mean - 2.0))
    f *= (vol / np.prod(f)) ** (1.0 / rank)
    return [int(max(2, round(x))) for x in f]


def shape_uneven(rng, rank, vol):
    w = rng.dirichlet(np.ones(rank) * 2.0)
    dim = np.maximum(2, np.round(np.exp(w * np.log(vol)))).astype(np.int64)
    i = int(np.argmax(dim))
    rest = int(np.prod(np.delete(dim, i), dtype=np.int64))
    dim[i] = max(2, int(round(vol / rest)))
    return [int(d) for d in dim]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", required=True)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--count", type=int, default=200)
    ap.add_argument("--elems", type=float, default=2e8)
    ap.add_argument("--elemsize", type=int, default=0, help="4 or 8; 0 = alternate")
    args = ap.parse_args()
    import torch
    import cutt_amd as cutt
    cutt.lib()
    os.environ["CUTT_MEASURE_ALL"] = "1"
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(args.seed)
    gens = [shape_ratio, shape_free, shape_uneven]
    out = []
    n = 0
    while len(out) < args.count:
        n += 1
        rank = 2 + n % 6
        es = args.elemsize or (8 if (n // 6) % 2 == 0 else 4)
        vol = args.elems * float(np.clip(rng.normal(1.0, 0.2), 0.3, 1.25))
        dim = gens[(n // 12) % 3](rng, rank, vol)
        perm = [int(p) for p in rng.permutation(rank)]
        v = int(np.prod(dim, dtype=np.int64))
        if perm == list(range(rank)) or v > 2.6e8 or v < 1e6:
            continue
        a = torch.arange(v, dtype=torch.int64 if es == 8 else torch.int32, device="cuda")
        b = torch.empty_like(a)
        rc, h = cutt.cuttPlanMeasure(rank, dim, perm, es, st, a.data_ptr(), b.data_ptr())
        if rc != cutt.CUTT_SUCCESS:
            raise SystemExit("cuttPlanMeasure failed with %d for %s %s" % (rc, dim, perm))
        cutt.cuttDestroy(h)
        cands = [c.as_dict() for c in cutt.get_last_measurement()]
        out.append(dict(dim=dim, perm=perm, es=es, cands=cands))
        print("%d %s %s es%d: %d candidates" % (len(out), dim, perm, es, len(cands)), file=sys.stderr, flush=True)
        del a, b
    with open(args.out, "w") as f:
        json.dump(out, f)


if __name__ == "__main__":
    main()
