#!/usr/bin/env python3
"""Writes tests/golden/counter_goldens.json from the known-answer tables that the reference's own
counter self-test holds (testCounters, reference src/cuttGpuModel.cpp:901-1100).

The reference file is read as text only: the script picks out the numeric initialisers of the arrays
posData, arrayResultsDouble, arrayResultsFloat, contResultsDouble, contResultsFloat and shTestData.
These are data (inputs and expected outputs), not code.  Run in the build container:

    python tests/golden/make_counter_goldens.py /root/reference/src/cuttGpuModel.cpp
"""
import json
import os
import re
import sys


def array_numbers(text, name):
    m = re.search(r"\b" + re.escape(name) + r"\s*(\[[^\]]*\])+\s*=\s*\{", text)
    if not m:
        raise SystemExit("array %s not found" % name)
    i = m.end() - 1
    depth = 0
    j = i
    while True:
        ch = text[j]
        if ch == "{":
            depth += 1
        elif ch == "}":
            depth -= 1
            if depth == 0:
                break
        j += 1
    return [int(x) for x in re.findall(r"-?\d+", text[i:j + 1])]


def main():
    src = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/src/cuttGpuModel.cpp"
    text = open(src).read()
    pos = array_numbers(text, "posData")
    out = {
        "source": "reference src/cuttGpuModel.cpp:907-1100 (testCounters known-answer tables)",
        "warpSize": 32,
        "posData": [pos[i * 32:(i + 1) * 32] for i in range(10)],
        "arrayResultsDouble": array_numbers(text, "arrayResultsDouble"),   # 10 x (tran, cl_full, cl_part), accWidth 16, cacheWidth 4
        "arrayResultsFloat": array_numbers(text, "arrayResultsFloat"),     # accWidth 32, cacheWidth 8
        "contResultsDouble": array_numbers(text, "contResultsDouble"),     # 16 offsets x 33 lengths x 3
        "contResultsFloat": array_numbers(text, "contResultsFloat"),       # 32 offsets x 33 lengths x 3
        "shTestData": array_numbers(text, "shTestData"),                   # 138 triples
    }
    assert len(pos) == 320 and len(out["arrayResultsDouble"]) == 30 and len(out["arrayResultsFloat"]) == 30
    assert len(out["contResultsDouble"]) == 16 * 33 * 3 and len(out["contResultsFloat"]) == 32 * 33 * 3
    assert len(out["shTestData"]) == 138 * 3
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "counter_goldens.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
