"""The seeded benchmark inputs are what the configuration list says they are (CPU)."""
import numpy as np

import baseline_configs as bc


def test_fixed_configs():
    vols = {c["name"]: int(np.prod(c["dim"], dtype=np.int64)) for c in bc.FIXED}
    assert vols == {"C1": 67108864, "C2": 201326592, "C3": 92997905, "C4": 200000000}


def test_sweep_properties():
    s = bc.sweep()
    assert len(s) == 50
    assert s == bc.sweep()  # seeded: reproducible
    ranks = set()
    for c in s:
        vol = int(np.prod(c["dim"], dtype=np.int64))
        assert abs(vol - 2.0e8) <= 0.01 * 2.0e8
        assert min(c["dim"]) >= 2 and vol < 2 ** 31
        assert sorted(c["perm"]) == list(range(len(c["dim"]))) and list(c["perm"]) != list(range(len(c["dim"])))
        ranks.add(len(c["dim"]))
    assert ranks == {2, 3, 4, 5, 6, 7}
    assert {c["es"] for c in s} == {4, 8}


def test_small_inputs_are_seeded():
    cfg = dict(name="C3", dim=(5, 7, 11), perm=(2, 0, 1), es=4)
    a, b = bc.make_input(cfg), bc.make_input(cfg)
    assert a.dtype == np.uint32 and np.array_equal(a, b)
    c2 = bc.make_input(dict(name="C2", dim=(4, 3), perm=(1, 0), es=8))
    assert c2.view(np.float64).tolist() == [float(i) for i in range(12)]
