"""Tensors that one launch cannot address are transposed piece by piece (no GPU needed here).

The library cuts a tensor whose input or output spans more elements than the kernels' 32-bit
offsets reach into pieces, each a transpose problem with the large tensor's strides.  With a small
span limit the same code cuts small tensors, which numpy can check exhaustively: the pieces must
tile the tensor exactly, stay within the limit, and every candidate plan of every piece shape -
replayed address by address - must move exactly that piece's elements to where the CPU oracle
puts them.
"""
import numpy as np
import pytest

from plan_emulator import emulate


def piece_offsets(shape):
    """Element offsets (input side, output side) of a piece relative to its bases, as flat arrays."""
    idx = np.indices(shape["dim"][::-1]).reshape(len(shape["dim"]), -1)[::-1]  # idx[r] = index along rank r
    rel_in = sum(idx[r].astype(np.int64) * shape["stride_in"][r] for r in range(len(shape["dim"])))
    rel_out = sum(idx[r].astype(np.int64) * shape["stride_out"][r] for r in range(len(shape["dim"])))
    return rel_in, rel_out


def random_problem(rng, max_vol):
    while True:
        rank = int(rng.integers(2, 7))
        dim = [int(d) for d in rng.integers(2, 12, size=rank)]
        if int(np.prod(dim)) <= max_vol:
            return dim, [int(p) for p in rng.permutation(rank)]


def test_pieces_tile_the_tensor_and_stay_within_the_limit(cutt, oracle_mod):
    rng = np.random.default_rng(11)
    cut = 0
    for _ in range(300):
        dim, perm = random_problem(rng, 30000)
        vol = int(np.prod(dim))
        limit = int(rng.integers(max(8, vol // 50), max(10, vol + 2)))
        dec = cutt.slab_decomposition(dim, perm, 4, limit)
        if dec is None:
            continue  # only when a piece's leading rank could not keep stride 1
        shapes, pieces = dec
        assert 1 <= len(shapes) <= 4
        cut += len(pieces) > 1
        data = np.arange(vol, dtype=np.uint32)
        expect = oracle_mod.transpose(dim, perm, data)
        out = np.zeros(vol, dtype=np.uint32)
        hits = np.zeros(vol, dtype=np.int32)
        offs = [piece_offsets(s) for s in shapes]
        for s, (rel_in, rel_out) in zip(shapes, offs):
            assert rel_in.max() < limit and rel_out.max() < limit, (dim, perm, limit, s)
            assert s["stride_in"][0] == 1 and s["stride_out"][s["perm"][0]] == 1
            assert sorted(s["perm"]) == list(range(len(s["dim"])))
        for shape, base_in, base_out in pieces:
            rel_in, rel_out = offs[shape]
            out[base_out + rel_out] = data[base_in + rel_in]
            np.add.at(hits, base_out + rel_out, 1)
        assert np.all(hits == 1), (dim, perm, limit)
        assert np.array_equal(out, expect), (dim, perm, limit)
    assert cut > 150


def test_a_tensor_within_the_limit_is_one_piece(cutt):
    shapes, pieces = cutt.slab_decomposition([7, 5, 3], [2, 1, 0], 8, 0)
    assert pieces == [(0, 0, 0)] and shapes[0]["dim"] == [7, 5, 3] and shapes[0]["stride_in"] == [1, 7, 35]
    # ranks that stay adjacent are fused before the tensor is cut
    shapes, pieces = cutt.slab_decomposition([7, 5, 3], [2, 0, 1], 8, 0)
    assert pieces == [(0, 0, 0)] and shapes[0]["dim"] == [35, 3] and shapes[0]["stride_out"] == [3, 1]


def test_a_tensor_of_2_to_the_33_elements(cutt):
    """Index arithmetic only: 8192 x 1024 x 1024 (2^33 elements), reversed."""
    dim, perm = [8192, 1024, 1024], [2, 1, 0]
    shapes, pieces = cutt.slab_decomposition(dim, perm, 4, 0)
    total = 0
    for shape, base_in, base_out in pieces:
        s = shapes[shape]
        span_in = 1 + sum((d - 1) * st for d, st in zip(s["dim"], s["stride_in"]))
        span_out = 1 + sum((d - 1) * st for d, st in zip(s["dim"], s["stride_out"]))
        assert span_in < 2 ** 32 and span_out < 2 ** 32
        assert base_in + span_in <= 2 ** 33 and base_out + span_out <= 2 ** 33
        total += int(np.prod(s["dim"], dtype=np.int64))
    assert total == 2 ** 33
    assert len(pieces) <= 16


def test_ranks_beyond_32(cutt):
    """34 ranks of extent 2, the first 30 reversed and the last four swapped in pairs: the pieces have
    at most 32 ranks and cover 2^34 elements."""
    dim, perm = [2] * 34, list(range(29, -1, -1)) + [31, 30, 33, 32]
    shapes, pieces = cutt.slab_decomposition(dim, perm, 4, 0)
    assert all(len(s["dim"]) <= 32 for s in shapes)
    assert sum(int(np.prod(shapes[p[0]]["dim"], dtype=np.int64)) for p in pieces) == 2 ** 34
    assert len({p[1] for p in pieces}) == len(pieces) and len({p[2] for p in pieces}) == len(pieces)


def _check_cover(shapes, pieces, total, limit=2 ** 32):
    seen = 0
    for shape, base_in, base_out in pieces:
        s = shapes[shape]
        assert s["stride_in"][0] == 1 and 1 in s["stride_out"], s      # contiguous rows on both sides
        span_in = 1 + sum((d - 1) * st for d, st in zip(s["dim"], s["stride_in"]))
        span_out = 1 + sum((d - 1) * st for d, st in zip(s["dim"], s["stride_out"]))
        assert span_in < limit and span_out < limit
        assert base_in + span_in <= total and base_out + span_out <= total
        seen += int(np.prod(s["dim"], dtype=np.int64))
    assert seen == total


def test_a_short_leading_rank_that_moves_to_the_back(cutt):
    """Arrays of structures turned into structures of arrays: the short leading rank of the input is the
    slowest of the output.  Cutting that rank into 2 + 1 would leave a piece without contiguous input
    rows; it stays whole and the two long ranks are cut instead."""
    shapes, pieces = cutt.slab_decomposition([3, 40000, 40000], [2, 1, 0], 4, 0)
    assert len(pieces) == 4 and len(shapes) == 1 and shapes[0]["dim"] == [3, 20000, 20000]
    _check_cover(shapes, pieces, 3 * 40000 * 40000)
    # the same with the short rank leading the output, and with a limit that small tensors reach
    shapes, pieces = cutt.slab_decomposition([40000, 40000, 3], [2, 1, 0], 8, 0)
    _check_cover(shapes, pieces, 3 * 40000 * 40000)
    # (the limit leaves room for all entries of the short rank, which lie far apart on the other side)
    for dim, perm, limit in [([3, 40, 50], [2, 1, 0], 4500), ([40, 50, 3], [2, 0, 1], 4500), ([5, 4, 60, 70], [3, 2, 1, 0], 70000),
                             ([2, 90, 80], [1, 2, 0], 8000)]:
        got = cutt.slab_decomposition(dim, perm, 4, limit)
        assert got is not None, (dim, perm)
        assert len(got[1]) > 1
        _check_cover(got[0], got[1], int(np.prod(dim)), limit=limit + 1)


def test_shapes_that_cannot_be_cut_are_refused(cutt):
    # the fastest rank of the input (2 entries) lies 4.9e9 elements apart in the output: no piece within
    # 32-bit offsets holds two neighbouring input elements
    assert cutt.slab_decomposition([2, 70000, 70000], [1, 2, 0], 4, 0) is None
    # ... and the same seen from the output
    assert cutt.slab_decomposition([70000, 70000, 2], [2, 0, 1], 4, 0) is None
    # a rank of 2^31 - 1 entries beside one of 3: the piece that fits 32-bit offsets on both sides would
    # have to fix the short rank, and the long one then has stride 3 on one side
    assert cutt.slab_decomposition([3, 2 ** 31 - 1], [1, 0], 4, 0) is None
    # 34 ranks of extent 2 reversed: the fastest rank of the input is the slowest of the output, 2^33
    # elements apart, so no piece within 32-bit offsets holds two neighbouring input elements
    assert cutt.slab_decomposition([2] * 34, list(range(33, -1, -1)), 4, 0) is None


@pytest.mark.parametrize("es", [4, 8])
def test_every_candidate_of_every_piece_shape(cutt, oracle_mod, es):
    rng = np.random.default_rng(5 + es)
    dtype = np.uint32 if es == 4 else np.uint64
    checked = strided = 0
    methods = set()
    for _ in range(250):
        dim, perm = random_problem(rng, 12000)
        vol = int(np.prod(dim))
        limit = int(rng.integers(max(16, vol // 12), max(17, vol // 2)))
        dec = cutt.slab_decomposition(dim, perm, es, limit)
        if dec is None:
            continue
        shapes, pieces = dec
        data = (np.arange(vol, dtype=np.uint64) * 2654435761 % (2 ** 31)).astype(dtype)
        expect = oracle_mod.transpose(dim, perm, data)
        for si, s in enumerate(shapes):
            if len(s["dim"]) < 2 and s["dim"][0] < 2:
                continue  # a single element
            _, base_in, base_out = next(p for p in pieces if p[0] == si)
            rel_in, rel_out = piece_offsets(s)
            # the piece's buffers as the kernel sees them: they start at the piece's bases
            padded = np.concatenate([data, np.zeros(vol, dtype=dtype)])
            src = padded[base_in: base_in + vol]
            if len(s["dim"]) < 2:
                continue  # one contiguous rank: a plain copy, no candidate list to replay
            with cutt.Candidates(s["dim"], s["perm"], es, int(rng.choice([0, 1024, 2048, 4096])),
                                 stride_in=s["stride_in"], stride_out=s["stride_out"]) as c:
                assert len(c) >= 1
                for i in range(len(c)):
                    info = c.info(i)
                    methods.add(info.method_name)
                    out, count = emulate(c, i, src)
                    want_hits = np.zeros(vol, dtype=np.int32)
                    want_hits[rel_out] = 1
                    assert np.array_equal(count, want_hits), (dim, perm, limit, s, info.method_name)
                    assert np.array_equal(out[rel_out], expect[base_out + rel_out]), (dim, perm, limit, s, info.method_name)
                    checked += 1
                    strided += any(a * d != b for a, d, b in zip(s["stride_in"], s["dim"], s["stride_in"][1:]))
    assert checked > 300 and strided > 100
    assert {"Tiled", "TiledCopy", "Packed", "PackedSplit"} <= methods


def test_a_small_piece_that_reaches_far_gets_64_bit_addresses(cutt):
    """The packed kernel keeps 32-bit byte offsets only while everything it can reach lies within
    4 GB of its base pointers; for a piece of a larger tensor that is its span, not its volume."""
    far = dict(stride_in=[1, 64, 2 ** 24], stride_out=[2 ** 26, 64, 1])   # 16 x 8 x 16 elements that reach 8 GB
    near = dict(stride_in=[1, 64, 2 ** 12], stride_out=[2 ** 13, 64, 1])
    for strides, wide in ((far, 1), (near, 0)):
        with cutt.Candidates([16, 8, 16], [2, 1, 0], 8, **strides) as c:
            packed = [c.info(i) for i in range(len(c)) if c.info(i).method_name in ("Packed", "PackedSplit")]
            assert packed and all(i.wideOffsets == wide for i in packed)
