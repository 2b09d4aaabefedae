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
        vol_mm, vol_mk, s_in_k, s_out, tiles_m, tiles_k, vol_mbar, order = [int(v) for v in cands.data(idx, 1)]
        assert tiles_m == -(-vol_mm // 64) and tiles_k == -(-vol_mk // 64)
        assert info.numBlocks == tiles_m * tiles_k * vol_mbar
        off_in, off_out = _mbar_offsets(mbar, vol_mbar)
        x = np.arange(vol_mm, dtype=np.int64)
        k = np.arange(vol_mk, dtype=np.int64)
        xx, kk = np.meshgrid(x, k, indexing="ij")
        src = (xx + kk * s_in_k).ravel()
        if name == "Tiled":
            dst = (kk + xx * s_out).ravel()
        else:
            dst = (xx + kk * s_out).ravel()
        for m in range(vol_mbar):
            scatter(off_out[m] + dst, off_in[m] + src)
        return out, count

    # Packed / PackedSplit
    (num_threads, vol_mbar, num_split, slab_floor, slab_rem, split_in, split_out, items_per_block,
     pad_shift, lds_elems) = [int(v) for v in cands.data(idx, 2)]
    assert num_threads % 64 == 0 and 64 <= num_threads <= 1024
    off_in, off_out = _mbar_offsets(mbar, vol_mbar)
    total_items = vol_mbar * num_split
    assert info.numBlocks == -(-total_items // items_per_block)
    classes = {}
    for c in ([0, 1] if slab_rem > 0 else [0]):
        cvol, in_cont, out_cont, in_magic, out_magic, n_rows_in, n_rows_out = [int(v) for v in cands.data(idx, 3, c)]
        row_in, row_out, sh = cands.data(idx, 4, c), cands.data(idx, 5, c), cands.data(idx, 6, c)
        assert len(row_in) == n_rows_in and len(row_out) == n_rows_out and len(sh) == cvol
        assert n_rows_in * in_cont == cvol and n_rows_out * out_cont == cvol
        assert cvol <= 65536
        p = np.arange(cvol, dtype=np.uint64)
        # the kernel's division: mulhi(p, magic), or p itself when the divisor is 1
        row_p = (p * np.uint64(in_magic)) >> np.uint64(32) if in_cont > 1 else p
        row_q = (p * np.uint64(out_magic)) >> np.uint64(32) if out_cont > 1 else p
        assert np.array_equal(row_p, p // np.uint64(in_cont)), "input magic division is wrong"
        assert np.array_equal(row_q, p // np.uint64(out_cont)), "output magic division is wrong"
        p = p.astype(np.int64)
        row_p = row_p.astype(np.int64)
        row_q = row_q.astype(np.int64)
        in_off = row_in[row_p] + (p - row_p * in_cont)
        out_off = row_out[row_q] + (p - row_q * out_cont)
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
    for w in range(total_items):
        m, s = divmod(w, num_split)
        c = 1 if s < slab_rem else 0
        p0 = s * slab_floor + min(s, slab_rem)
        src_rel, dst_rel = classes[c]
        scatter(off_out[m] + p0 * split_out + dst_rel, off_in[m] + p0 * split_in + src_rel)
    return out, count
