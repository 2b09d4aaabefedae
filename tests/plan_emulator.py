"""Host-side replay of a candidate's address stream (numpy).

Reads the index data that the planner would hand to the kernels
(cuttCandidatesData) and applies exactly the arithmetic of the kernels in
cutt_amd/csrc/kernels.hip - same work-item numbering, same row/column split
with the multiply-high division, same LDS slot skew - to move a flat numpy
array.  It is a test tool: it validates tables and launch geometry on a
machine without a GPU, including that no offset leaves the tensor and that
every output element is written exactly once.
"""
import numpy as np


def _mbar_offsets(tab, vol_mbar):
    m = np.arange(vol_mbar, dtype=np.int64)
    off_in = np.zeros(vol_mbar, dtype=np.int64)
    off_out = np.zeros(vol_mbar, dtype=np.int64)
    rem = m.copy()
    for k in range(len(tab) // 3):
        e, si, so = int(tab[3 * k]), int(tab[3 * k + 1]), int(tab[3 * k + 2])
        i = rem % e
        rem //= e
        off_in += i * si
        off_out += i * so
    return off_in, off_out


def _check_tile_decode(num_blocks, order, tiles_m, tiles_k, vol_mbar, xcd_chunk, sup_m, sup_k, digits=()):
    """The kernels' workgroup-index decoding visits every (tile, Mbar position) exactly once."""
    b = np.arange(num_blocks, dtype=np.int64)
    if xcd_chunk:
        assert num_blocks == 8 * xcd_chunk
        l = (b % 8) * xcd_chunk + b // 8
    else:
        l = b
    if order == 7:
        # mixed-radix number, fastest digit first; every digit belongs to one coordinate
        n = len(digits) // 3
        assert 1 <= n <= 16
        coord = [np.zeros_like(l), np.zeros_like(l), np.zeros_like(l)]
        rest = l.copy()
        for i in range(n):
            which, radix, weight = int(digits[3 * i]), int(digits[3 * i + 1]), int(digits[3 * i + 2])
            assert which in (0, 1, 2) and radix >= 1 and weight >= 1
            v = rest % radix if i + 1 < n else rest
            rest = rest // radix
            coord[which] = coord[which] + v * weight
        tm, tk, m = coord
        ok = (tm < tiles_m) & (tk < tiles_k) & (m < vol_mbar)
    elif order == 0:
        t, m = l // vol_mbar, l % vol_mbar
        tk, tm = t // tiles_m, t % tiles_m
        ok = tk < tiles_k
    elif order == 1:
        t, tm = l // tiles_m, l % tiles_m
        m, tk = t // tiles_k, t % tiles_k
        ok = m < vol_mbar
    elif order == 2:
        t, tk = l // tiles_k, l % tiles_k
        m, tm = t // tiles_m, t % tiles_m
        ok = m < vol_mbar
    else:
        assert order in (3, 4, 5, 6) and sup_m >= 1 and sup_k >= 1
        n_sm, n_sk = -(-tiles_m // sup_m), -(-tiles_k // sup_k)
        per = sup_m * sup_k
        w, t = l % per, l // per
        if order >= 5:
            st, m = t // vol_mbar, t % vol_mbar
        else:
            st, m = t % (n_sm * n_sk), t // (n_sm * n_sk)
        if order == 6:
            mi = st // n_sk
            tm = mi * sup_m + w % sup_m
            tk = ((st % n_sk + mi) % n_sk) * sup_k + w // sup_m
        elif order != 4:
            tm = (st % n_sm) * sup_m + w % sup_m
            tk = (st // n_sm) * sup_k + w // sup_m
        else:
            tk = (st % n_sk) * sup_k + w % sup_k
            tm = (st // n_sk) * sup_m + w // sup_k
        ok = (m < vol_mbar) & (st < n_sm * n_sk) & (tm < tiles_m) & (tk < tiles_k)
    key = (m[ok] * tiles_k + tk[ok]) * tiles_m + tm[ok]
    assert key.size == tiles_m * tiles_k * vol_mbar, "tile decode misses or repeats tiles"
    assert np.array_equal(np.sort(key), np.arange(key.size))


def emulate(cands, idx, data):
    """Return (out, write_count) for candidate idx applied to the flat array data."""
    info = cands.info(idx)
    vol = data.size
    out = np.zeros_like(data)
    count = np.zeros(vol, dtype=np.int32)
    name = info.method_name

    def scatter(dst_idx, src_idx):
        assert dst_idx.min() >= 0 and dst_idx.max() < vol, "output offset out of range"
        assert src_idx.min() >= 0 and src_idx.max() < vol, "input offset out of range"
        out[dst_idx] = data[src_idx]
        np.add.at(count, dst_idx, 1)

    if name == "Trivial":
        out[:] = data
        count[:] = 1
        return out, count

    mbar = cands.data(idx, 0)
    if name in ("Tiled", "TiledCopy"):
        vol_mm, vol_mk, s_in_k, s_out, tiles_m, tiles_k, vol_mbar, order, xcd_chunk, sup_m, sup_k = [int(v) for v in cands.data(idx, 1)]
        assert tiles_m == -(-vol_mm // 64) and tiles_k == -(-vol_mk // 64)
        _check_tile_decode(info.numBlocks, order, tiles_m, tiles_k, vol_mbar, xcd_chunk, sup_m, sup_k,
                           cands.data(idx, 8) if order == 7 else ())
        off_in, off_out = _mbar_offsets(mbar, vol_mbar)
        x = np.arange(vol_mm, dtype=np.int64)
        k = np.arange(vol_mk, dtype=np.int64)

        def row_offsets(i, radix, stride):
            """Offsets of the rows of a tile axis: i * stride, or the mixed-radix sum over a fused rank set."""
            if len(radix) == 0:
                return i * stride
            n = len(radix) // 2
            assert n <= 4 and int(np.prod([int(radix[2 * j]) for j in range(n)])) == i.size
            off = np.zeros_like(i)
            rest = i.copy()
            for j in range(n):
                e, st = int(radix[2 * j]), int(radix[2 * j + 1])
                off += (rest % e if j + 1 < n else rest) * st
                rest //= e
            return off

        rows_k = cands.data(idx, 7, 0) if name == "Tiled" else ()
        rows_m = cands.data(idx, 7, 1) if name == "Tiled" else ()
        xx, kk = np.meshgrid(x, k, indexing="ij")
        in_k = row_offsets(k, rows_k, s_in_k)
        src = (xx + in_k[None, :]).ravel()
        if name == "Tiled":
            out_m = row_offsets(x, rows_m, s_out)
            dst = (kk + out_m[:, None]).ravel()
        else:
            dst = (xx + kk * s_out).ravel()
        for m in range(vol_mbar):
            scatter(off_out[m] + dst, off_in[m] + src)
        return out, count

    # Packed / PackedSplit
    sc = [int(v) for v in cands.data(idx, 2)]
    num_threads, vol_mbar, items_per_block, pad_shift, lds_elems, xcd_chunk, elems_per_thread, item_order = sc[:8]
    splits = [sc[8:13], sc[13:18]]  # numSplit, slabFloor, slabRem, strideIn, strideOut
    assert num_threads % 64 == 0 and 64 <= num_threads <= 1024
    # 16 elements per lane exist for 4-byte elements only
    assert elems_per_thread in (1, 2, 4, 8) or (elems_per_thread == 16 and data.dtype.itemsize == 4)
    off_in, off_out = _mbar_offsets(mbar, vol_mbar)
    ns0, ns1 = splits[0][0], splits[1][0]
    total_items = vol_mbar * ns0 * ns1
    assert item_order in (0, 1, 2)
    numbers = total_items if item_order != 1 else -(-vol_mbar // items_per_block) * ns0 * ns1 * items_per_block
    logical_blocks = -(-numbers // items_per_block)
    if xcd_chunk:
        # workgroup b handles logical block (b % 8) * xcd_chunk + b // 8: every logical block once
        assert info.numBlocks == 8 * xcd_chunk and 8 * xcd_chunk >= logical_blocks
        b = np.arange(info.numBlocks, dtype=np.int64)
        lb = (b % 8) * xcd_chunk + b // 8
        assert np.array_equal(np.sort(lb), b)
    else:
        assert info.numBlocks == logical_blocks
    if item_order == 2:
        # the numbers are those of order 0, handed out round by round inside each chunk of workgroups:
        # every number must belong to exactly one workgroup, and to none more than items_per_block
        chunk_blocks = xcd_chunk if xcd_chunk else info.numBlocks
        lb = np.arange(info.numBlocks, dtype=np.int64)
        x, q = lb // chunk_blocks, lb % chunk_blocks
        start = x * chunk_blocks * items_per_block
        end = np.minimum(start + chunk_blocks * items_per_block, numbers)
        taken = []
        for i in range(items_per_block):
            w = start + q + i * chunk_blocks
            taken.append(w[w < end])
        taken = np.concatenate(taken)
        assert np.array_equal(np.sort(taken), np.arange(numbers)), "order 2 misses or repeats work items"
    classes = {}
    for c in range(4):
        if ((c & 1) and splits[0][2] == 0) or ((c & 2) and splits[1][2] == 0):
            continue
        cvol, in_cont, out_cont = [int(v) for v in cands.data(idx, 3, c)]
        row_in, row_out, sh = cands.data(idx, 4, c), cands.data(idx, 5, c), cands.data(idx, 6, c)
        assert cvol % in_cont == 0 and cvol % out_cont == 0
        assert len(row_in) == cvol // in_cont and len(row_out) == cvol // out_cont and len(sh) == cvol
        assert cvol <= num_threads * elems_per_thread, "a lane would need more table registers"
        p = np.arange(cvol, dtype=np.int64)
        # per-element offsets as the kernel derives them: run offset + position inside the run
        in_off = row_in[p // in_cont] + p % in_cont
        out_off = row_out[p // out_cont] + p % out_cont
        slot = p + (p >> pad_shift)
        assert slot.max() < lds_elems, "LDS slot outside the buffer"
        assert len(np.unique(slot)) == cvol
        assert sh.min() >= 0 and sh.max() < lds_elems
        # LDS content after the load phase, as "which input-compact element sits in slot"
        which = np.full(lds_elems, -1, dtype=np.int64)
        which[slot] = p
        src_p = which[sh]
        assert src_p.min() >= 0, "gather reads an LDS slot that was never written"
        classes[c] = (in_off[src_p], out_off)
    seen = 0
    for w in range(numbers):
        if item_order != 1:
            t, s0 = divmod(w, ns0)
            m, s1 = divmod(t, ns1)
        else:  # the workgroup keeps its slabs and walks items_per_block Mbar positions
            slab, mi = divmod(w, items_per_block)
            t, s0 = divmod(slab, ns0)
            mb, s1 = divmod(t, ns1)
            m = mb * items_per_block + mi
            if m >= vol_mbar:
                continue
        seen += 1
        c = (1 if s0 < splits[0][2] else 0) + (2 if s1 < splits[1][2] else 0)
        p0 = s0 * splits[0][1] + min(s0, splits[0][2])
        p1 = s1 * splits[1][1] + min(s1, splits[1][2])
        src_rel, dst_rel = classes[c]
        scatter(off_out[m] + p0 * splits[0][4] + p1 * splits[1][4] + dst_rel,
                off_in[m] + p0 * splits[0][3] + p1 * splits[1][3] + src_rel)
    assert seen == total_items
    return out, count
