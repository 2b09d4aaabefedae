"""The cost model's walk of a plan's address stream against kernels that replay the stream on the
GPU (same workgroup numbering, index arithmetic and tables as the transpose kernels, counted with
64-lane ballots): instructions, 128-byte lines, 32-byte sectors, partly written lines and LDS
gather cycles must agree exactly when the model walks every work item, and within sampling error
when it samples ten.  Shapes: the reference's hand-picked test tensors (src/cutt_test.cpp:245-366)
and the benchmark configurations, with every method that applies."""
import sys

import pytest

import baseline_configs as bc

pytestmark = pytest.mark.gpu

TEST3 = [((43, 67), (1, 0)), ((65536, 2), (1, 0)), ((1305, 599, 88), (0, 2, 1)), ((24, 330, 64, 147), (1, 0, 2, 3)),
         ((5, 42, 75, 86, 57), (1, 3, 4, 2, 0)), ((5, 3, 2, 9, 14), (0, 1, 3, 2, 4))]
EXACT = ("rdInstr", "wrInstr", "rdLines", "wrLines", "rdSectors", "wrSectors", "wrPartialLines")


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def plans_for(cutt, dim, perm, es, st):
    """(label, handle) for the planner's choice and for every method that has a candidate."""
    for method in (0, cutt.METHOD_TILED, cutt.METHOD_TILEDCOPY, cutt.METHOD_PACKED, cutt.METHOD_PACKEDSPLIT):
        cutt.set_method_override(method)
        try:
            rc, h = cutt.cuttPlan(len(dim), list(dim), list(perm), es, st)
        finally:
            cutt.set_method_override(0)
        if rc == cutt.CUTT_SUCCESS:
            yield method, h


def check(cutt, h, label, samples, es):
    info = cutt.get_plan_info(h)
    dev, mod = cutt.count_address_stream(h, samples)
    d, m = dev.as_dict(), mod.as_dict()
    say("  %s %s samples=%d: device %s" % (label, info.method_name, samples, {k: int(v) for k, v in d.items()}))
    packed = info.method_name in ("Packed", "PackedSplit")
    names = EXACT + (("ldsCycles",) if packed else ())
    if samples == 0:
        for k in names:
            assert d[k] == m[k], (label, info.method_name, k, d[k], m[k])
    else:
        for k in names:
            assert abs(d[k] - m[k]) <= 0.08 * max(d[k], 1.0), (label, info.method_name, k, d[k], m[k])
    if info.method_name == "Tiled":
        # the padded tile is free of bank conflicts: one lane per 4-byte bank; an 8-byte word is
        # counted on its first bank, so 64 lanes meet two by two (the hardware serves them in two
        # passes of 32 lanes)
        assert dev.ldsMaxDegree == (1 if es == 4 else 2), (label, dev.ldsMaxDegree)


def test_counts_agree_on_the_reference_test_shapes():
    import torch
    import cutt_amd as cutt
    assert torch.cuda.is_available()
    cutt.lib()
    st = torch.cuda.current_stream().cuda_stream
    for dim, perm in TEST3:
        for es in (4, 8):
            say("dim=%s perm=%s es=%d" % (dim, perm, es))
            for method, h in plans_for(cutt, dim, perm, es, st):
                check(cutt, h, "forced %d" % method, 0, es)
                cutt.cuttDestroy(h)


@pytest.mark.parametrize("cfg", bc.FIXED, ids=[c["name"] for c in bc.FIXED])
def test_counts_agree_on_the_benchmark_configurations(cfg):
    import torch
    import cutt_amd as cutt
    cutt.lib()
    st = torch.cuda.current_stream().cuda_stream
    dim, perm, es = cfg["dim"], cfg["perm"], cfg["es"]
    say("%s dim=%s perm=%s es=%d" % (cfg["name"], dim, perm, es))
    for method, h in plans_for(cutt, dim, perm, es, st):
        info = cutt.get_plan_info(h)
        # every work item on the host takes a while for the 2e8-element tensors: the planner's own
        # choice is walked completely, the forced methods with the ten samples cuttPlan uses
        check(cutt, h, "forced %d" % method, 0 if method == 0 else 10, es)
        cutt.cuttDestroy(h)


def test_refusals():
    import torch
    import cutt_amd as cutt
    st = torch.cuda.current_stream().cuda_stream
    rc, h = cutt.cuttPlan(3, [4, 5, 6], [0, 1, 2], 8, st)
    assert rc == cutt.CUTT_SUCCESS
    with pytest.raises(cutt.CuttError):
        cutt.count_address_stream(h, 0)   # a plain copy
    cutt.cuttDestroy(h)
    with pytest.raises(cutt.CuttError):
        cutt.count_address_stream(123456, 0)


def test_counts_agree_for_every_work_item_order(monkeypatch):
    """The packed kernel's three ways of handing out work items (neighbouring slabs, own slabs over Mbar
    positions, every B-th item of the XCD's chunk): the counting kernel takes its items from the function the
    transpose kernel uses, so the totals must equal the host model's for each of them."""
    import torch
    import cutt_amd as cutt
    cutt.lib()
    st = torch.cuda.current_stream().cuda_stream
    for dim, perm, es in [((331, 7, 257, 3), (2, 1, 0, 3), 4), ((20000, 2, 50), (2, 1, 0), 8), ((5, 7, 11, 13, 17), (4, 2, 0, 1, 3), 4)]:
        for order in (0, 1, 2):
            monkeypatch.setenv("CUTT_ITEM_ORDER", str(order))
            monkeypatch.setenv("CUTT_MAX_ITEMS", "4")
            for method in (cutt.METHOD_PACKED, cutt.METHOD_PACKEDSPLIT):
                cutt.set_method_override(method)
                try:
                    rc, h = cutt.cuttPlan(len(dim), list(dim), list(perm), es, st)
                finally:
                    cutt.set_method_override(0)
                if rc != cutt.CUTT_SUCCESS:
                    continue
                say("dim=%s perm=%s es=%d item order %d method %d" % (dim, perm, es, order, method))
                check(cutt, h, "item order %d" % order, 0, es)
                cutt.cuttDestroy(h)
