"""The benchmark configurations as concrete, seeded inputs (shared by tests and bench.py).

C1-C4 are fixed; C5 is a seeded sweep of random tensors of about 2e8 elements:
ranks 2-7, every dim >= 2, product within 1 % of 2e8, a random non-identity
permutation, alternating 8- and 4-byte elements.
"""
import numpy as np

C1 = dict(name="C1", dim=(8192, 8192), perm=(1, 0), es=4)
C2 = dict(name="C2", dim=(1024, 64, 1024, 3), perm=(2, 1, 0, 3), es=8)
C3 = dict(name="C3", dim=(5, 7, 11, 13, 17, 1093), perm=(4, 2, 0, 5, 1, 3), es=4)
C4 = dict(name="C4", dim=(200000, 2, 500), perm=(2, 1, 0), es=8)
FIXED = [C1, C2, C3, C4]


def make_input(cfg, seed=1234):
    """Flat numpy array of unsigned words holding the configuration's input bits."""
    vol = int(np.prod(cfg["dim"], dtype=np.int64))
    rng = np.random.default_rng(seed)
    name = cfg["name"]
    if name == "C1":    # uniform random floats from a fixed seed
        return rng.random(vol, dtype=np.float32).view(np.uint32)
    if name == "C2":    # value = element linear index as double
        return np.arange(vol, dtype=np.float64).view(np.uint64)
    if name == "C3":    # random 32-bit patterns reinterpreted as fp32 (NaNs included)
        return rng.integers(0, 2 ** 32 - 1, size=vol, dtype=np.uint32, endpoint=True)
    if name == "C4":    # doubles in [-1, 1)
        return (rng.random(vol, dtype=np.float64) * 2.0 - 1.0).view(np.uint64)
    if cfg["es"] == 8:
        return rng.integers(0, 2 ** 64 - 1, size=vol, dtype=np.uint64, endpoint=True)
    return rng.integers(0, 2 ** 32 - 1, size=vol, dtype=np.uint32, endpoint=True)


def random_dims(rng, rank, target=2.0e8, tol=0.01, min_dim=2):
    """Integer dims >= min_dim whose product is within tol of target."""
    for _ in range(10000):
        # random split of log(target) over the ranks
        w = rng.dirichlet(np.ones(rank) * 2.0)
        dims = np.maximum(min_dim, np.round(np.exp(w * np.log(target)))).astype(np.int64)
        # repair the product by adjusting the largest dim
        i = int(np.argmax(dims))
        rest = int(np.prod(np.delete(dims, i), dtype=np.int64))
        dims[i] = max(min_dim, int(round(target / rest)))
        vol = int(np.prod(dims, dtype=np.int64))
        if abs(vol - target) <= tol * target and vol < 2 ** 31 and dims.min() >= min_dim:
            return [int(d) for d in dims]
    raise RuntimeError("no dims found")


def sweep(count=50, seed=20240601):
    """The C5 sweep: list of dict(name, dim, perm, es)."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        rank = 2 + i % 6
        dim = random_dims(rng, rank)
        while True:
            perm = [int(p) for p in rng.permutation(rank)]
            if perm != list(range(rank)):
                break
        out.append(dict(name="C5-%02d" % i, dim=tuple(dim), perm=tuple(perm), es=8 if i % 2 == 0 else 4))
    return out
