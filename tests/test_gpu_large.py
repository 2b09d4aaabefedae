"""Tensors that are transposed piece by piece, on the GPU.

A tensor of 2^32 elements and more (or of more than 32 ranks) is beyond the kernels' 32-bit element
offsets; the library cuts it into pieces and launches one kernel per piece.  Small tensors go
through the same code when CUTT_SPAN_LIMIT lowers the limit, and are compared with the CPU oracle;
tensors of 4.3e9 to 1.7e10 elements are checked on the device against a closed form, chunk by chunk,
with a value pattern that does not repeat every 2^32 elements (so a base offset that lost its high
bits cannot pass).
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

MULT = 2654435761


def stream():
    return torch.cuda.current_stream().cuda_stream


def pattern(idx):
    """32-bit value of the element with linear input index idx (int64 tensor); differs between
    indices 2^32 apart."""
    v = (idx * MULT + (idx >> 32) * 40503 + (idx >> 31)) & 0xFFFFFFFF
    return torch.where(v >= 2 ** 31, v - 2 ** 32, v).to(torch.int32)


def fill_pattern(vol, words_per_elem, chunk=1 << 27):
    buf = torch.empty(vol * words_per_elem, dtype=torch.int32, device="cuda")
    for s in range(0, vol, chunk):
        idx = torch.arange(s, min(vol, s + chunk), dtype=torch.int64, device="cuda")
        v = pattern(idx)
        if words_per_elem == 1:
            buf[s: s + idx.numel()] = v
        else:  # an 8-byte element: the pattern and its complement
            w = buf[2 * s: 2 * (s + idx.numel())].view(-1, 2)
            w[:, 0] = v
            w[:, 1] = ~v
    return buf


def count_wrong(out, dim, perm, words_per_elem, chunk=1 << 27):
    """Compares the transposed buffer with the closed form: output position o holds the element
    whose input index follows from o's mixed-radix digits."""
    vol = int(np.prod(dim, dtype=np.int64))
    in_stride = np.cumprod([1] + list(dim[:-1]), dtype=np.int64)
    wrong = 0
    for s in range(0, vol, chunk):
        o = torch.arange(s, min(vol, s + chunk), dtype=torch.int64, device="cuda")
        rest, idx = o, torch.zeros_like(o)
        for j in range(len(dim)):
            d = int(dim[perm[j]])
            q = rest // d
            idx += (rest - q * d) * int(in_stride[perm[j]])
            rest = q
        v = pattern(idx)
        if words_per_elem == 1:
            wrong += int((out[s: s + o.numel()] != v).sum())
        else:
            w = out[2 * s: 2 * (s + o.numel())].view(-1, 2)
            wrong += int(((w[:, 0] != v) | (w[:, 1] != ~v)).sum())
    return wrong


@pytest.fixture
def span_limit():
    saved = os.environ.get("CUTT_SPAN_LIMIT")

    def set_limit(v):
        os.environ["CUTT_SPAN_LIMIT"] = str(int(v))
    yield set_limit
    if saved is None:
        os.environ.pop("CUTT_SPAN_LIMIT", None)
    else:
        os.environ["CUTT_SPAN_LIMIT"] = saved


def test_small_tensors_cut_into_pieces_match_the_oracle(cutt, oracle_mod, span_limit):
    rng = np.random.default_rng(21)
    pieces_seen, shapes_seen, methods = 0, 0, set()
    for case in range(24):
        es = 4 if case % 2 else 8
        while True:
            rank = int(rng.integers(2, 7))
            dim = [int(d) for d in rng.integers(2, 60, size=rank)]
            vol = int(np.prod(dim))
            if 200_000 <= vol <= 3_000_000:
                break
        perm = [int(p) for p in rng.permutation(rank)]
        limit = int(rng.integers(vol // 9, vol // 2))
        if cutt.slab_decomposition(dim, perm, es, limit) is None:
            continue
        span_limit(limit)
        dtype = np.uint32 if es == 4 else np.uint64
        data = rng.integers(0, 2 ** 32, size=vol, dtype=np.uint64).astype(dtype)
        expect = oracle_mod.transpose(dim, perm, data)
        a = torch.from_numpy(data.view(np.int32 if es == 4 else np.int64)).cuda()
        for how in ("plan", "measure", "tiled", "packed", "packedsplit"):
            b = torch.full_like(a, -1)
            force = {"tiled": cutt.METHOD_TILED, "packed": cutt.METHOD_PACKED, "packedsplit": cutt.METHOD_PACKEDSPLIT}.get(how, 0)
            cutt.set_method_override(force)
            try:
                if how == "measure":
                    rc, h = cutt.cuttPlanMeasure(rank, dim, perm, es, stream(), a.data_ptr(), b.data_ptr())
                else:
                    rc, h = cutt.cuttPlan(rank, dim, perm, es, stream())
            finally:
                cutt.set_method_override(0)
            if force and rc != cutt.CUTT_SUCCESS:
                continue  # the forced method has no candidate for some piece
            assert rc == cutt.CUTT_SUCCESS, (dim, perm, es, limit, how)
            info = cutt.get_plan_info(h)
            assert info.numPieces > 1 and 1 <= info.numShapes <= 4
            pieces_seen += info.numPieces
            shapes_seen = max(shapes_seen, info.numShapes)
            methods.add(info.method_name)
            b.fill_(-1)
            assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_SUCCESS
            torch.cuda.synchronize()
            got = b.cpu().numpy().view(dtype)
            assert np.array_equal(got, expect), (dim, perm, es, limit, how, info.method_name)
            assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    assert pieces_seen > 200 and shapes_seen >= 2
    assert {"Tiled", "Packed", "PackedSplit"} & methods


def test_entry_points_that_do_not_cut_refuse(cutt, span_limit):
    span_limit(1000)
    a = torch.zeros(64 * 64, dtype=torch.int32, device="cuda")
    b = torch.zeros_like(a)
    assert cutt.cuttExecuteNoAlloc(2, [64, 64], [1, 0], 4, stream(), a.data_ptr(), b.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    with pytest.raises(ValueError):
        cutt.Candidates([64, 64], [1, 0], 4)


@pytest.mark.parametrize("dim,perm,es,how", [
    ((65552, 65536), (1, 0), 4, "plan"),          # 4.296e9 elements, 17 GB per buffer
    ((4100, 1024, 1024), (2, 0, 1), 8, "measure"),  # 4.299e9 elements, 34 GB per buffer
    ((3, 1499, 997, 1009), (3, 2, 0, 1), 4, "plan"),  # 4.5e9 elements, last pieces shorter on both sides: 4 shapes
])
def test_more_than_2_to_the_32_elements(cutt, dim, perm, es, how):
    dim, perm = list(dim), list(perm)
    vol = int(np.prod(dim, dtype=np.int64))
    assert vol >= 2 ** 32
    words = es // 4
    a = fill_pattern(vol, words)
    b = torch.full((vol * words,), -1, dtype=torch.int32, device="cuda")
    print("planning", dim, perm, es, how, flush=True)
    if how == "measure":
        rc, h = cutt.cuttPlanMeasure(len(dim), dim, perm, es, stream(), a.data_ptr(), b.data_ptr())
    else:
        rc, h = cutt.cuttPlan(len(dim), dim, perm, es, stream())
    assert rc == cutt.CUTT_SUCCESS
    info = cutt.get_plan_info(h)
    print("pieces", info.numPieces, "shapes", info.numShapes, info.method_name, flush=True)
    assert info.numPieces >= 2
    b.fill_(-1)
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_SUCCESS
    t1.record()
    torch.cuda.synchronize()
    print("GB/s %.0f" % (2.0 * vol * es / (t0.elapsed_time(t1) * 1e-3) / 1e9), flush=True)
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    assert count_wrong(b, dim, perm, words) == 0


def test_rank_34(cutt):
    """34 ranks of extent 2 (1.7e10 four-byte elements, 69 GB per buffer).  The permutation leaves pieces
    of 2^29 elements (2 GB) that reach 2^31 elements (8 GB) from their base on both sides: the kernel
    instance with 64-bit addresses has to be chosen by reach, not by volume."""
    dim = [2] * 34
    perm = [30, 29, 28, 27, 26, 25, 24, 23, 22, 21, 19, 18, 17, 16, 15, 14, 13, 12, 9, 8, 7, 6, 5, 4, 3, 2, 1, 0,
            31, 32, 33, 20, 10, 11]
    vol = 2 ** 34
    a = fill_pattern(vol, 1)
    b = torch.full((vol,), -1, dtype=torch.int32, device="cuda")
    print("planning", flush=True)
    rc, h = cutt.cuttPlan(34, dim, perm, 4, stream())
    assert rc == cutt.CUTT_SUCCESS
    info = cutt.get_plan_info(h)
    print("pieces", info.numPieces, "shapes", info.numShapes, info.method_name, "wide", info.wideOffsets, flush=True)
    assert info.numPieces == 32
    assert info.method_name not in ("Packed", "PackedSplit") or info.wideOffsets == 1
    assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_SUCCESS
    torch.cuda.synchronize()
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    print("checking", flush=True)
    assert count_wrong(b, dim, perm, 1) == 0
    # ranks beyond 64, and shapes whose leading ranks cannot stay contiguous inside 32-bit offsets, are refused
    assert cutt.cuttPlan(65, [2] * 65, list(range(64, -1, -1)), 4, stream())[0] == cutt.CUTT_INVALID_PARAMETER
    assert cutt.cuttPlan(34, [2] * 34, list(range(33, -1, -1)), 4, stream())[0] == cutt.CUTT_INVALID_PARAMETER
