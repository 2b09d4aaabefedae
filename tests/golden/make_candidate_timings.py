"""Writes tests/golden/candidate_timings.json from files made by `python -m cutt_amd.tuning.collect`
(every candidate plan of a tensor timed on an MI355X by cuttPlanMeasure with CUTT_MEASURE_ALL=1):

  python tests/golden/make_candidate_timings.py worst.json random.json

Keeps, per tensor, the measured microseconds of every candidate under a key that names the
candidate's index sets (method, fused problem or not, numMm, numMk, split ranks and slab counts).
tests/test_heuristic_regret.py replays the planner's choice against these timings without a GPU."""
import json
import os
import sys


def key(c):
    return "%d/%d/%d/%d/%d/%d/%d/%d" % (c["method"], c["fromReduced"], c["numMm"], c["numMk"], c["splitRank"],
                                        c["numSplit"], c["splitRank2"], c["numSplit2"])


def main():
    out = []
    for path, take in zip(sys.argv[1:], (24, 36)):
        rows = json.load(open(path))
        step = max(1, len(rows) // take)
        for r in rows[::step][:take]:
            times = {}
            for c in r["cands"]:
                if c["usMeasured"] > 0 and c["numBlocks"] * c["numThreads"] < 2 ** 32:
                    k = key(c)
                    times[k] = round(min(times.get(k, 1e30), c["usMeasured"]), 1)
            out.append(dict(dim=r["dim"], perm=r["perm"], es=r["es"], us=times))
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "candidate_timings.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(len(out), "tensors")


if __name__ == "__main__":
    main()
