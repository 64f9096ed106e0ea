"""Properties of the tables behind the hub pass of the SpMM, read back from the plan: every entry of every hub row sits
in exactly one stream exactly once, under the slot of its own row and part, in the window and column range the stream says;
window marks, padding and the split of a row's entries over its parts are what the kernel assumes.  The pass itself is
checked against the oracle elsewhere; this pins the construction it relies on."""
import numpy as np
import pytest
import torch

from plexus_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
WAVES_PER_RANGE = 256
RANGES = 8


def say(msg):
    print("[case] " + msg, flush=True)


def hub_tables(a, wide):
    lib = _lib.load()
    info = lambda what: int(lib.plx_spmm_plan_hub_info(a._plan, int(wide), what))
    n_rows, n_slots, entries, stored, window, n_windows, wpr, rpw, cap, streams = (info(i) for i in range(10))
    t = {"n_rows": n_rows, "n_slots": n_slots, "entries": entries, "stored": stored, "window": window, "n_windows": n_windows, "wpr": wpr,
         "rpw": rpw, "cap": cap, "streams": streams}
    t["hub_row"] = np.empty(cap, np.int32)
    t["rows"] = np.empty(n_rows, np.int32)
    t["row_slot_first"] = np.empty(n_rows + 1, np.int32)
    t["row_slots"] = np.empty(n_slots, np.int32)
    t["stream_first"] = np.empty(streams, np.int64)
    t["stream_total"] = np.empty(streams, np.int32)
    t["stream_pos"] = np.empty(stored, np.int32)
    t["stream_run"] = np.empty(stored, np.uint8)
    t["stream_mark"] = np.empty((streams, wpr), np.int32)
    ptr = lambda x: x.ctypes.data
    _lib.check(lib.plx_spmm_plan_hub_tables_host(a._plan, int(wide), ptr(t["hub_row"]), ptr(t["rows"]), ptr(t["row_slot_first"]), ptr(t["row_slots"]),
                                                 ptr(t["stream_first"]), ptr(t["stream_total"]), ptr(t["stream_pos"]), ptr(t["stream_run"]),
                                                 ptr(t["stream_mark"])), "plx_spmm_plan_hub_tables_host")
    return t


def check_tables(rowptr, col, k, seg_len, t, part_factor):
    rowptr = rowptr.astype(np.int64)
    col = col.astype(np.int64)
    rpw, cap, wpr, window = t["rpw"], t["cap"], t["wpr"], t["window"]
    assert t["streams"] == RANGES * WAVES_PER_RANGE and cap == WAVES_PER_RANGE * rpw
    assert wpr == -(-(-(-k // RANGES)) // window) and t["n_windows"] == wpr * RANGES
    rows = t["rows"].astype(np.int64)
    lens = rowptr[rows + 1] - rowptr[rows]
    # the hub rows: split rows, distinct, longest first; their slots: one per part of at most part_factor * seg_len entries
    assert len(set(rows.tolist())) == len(rows) and (lens > seg_len).all() and (np.diff(lens) <= 0).all()
    parts = -(-lens // (part_factor * seg_len))
    assert (np.diff(t["row_slot_first"]) == parts).all() and t["row_slot_first"][0] == 0 and t["row_slot_first"][-1] == t["n_slots"]
    assert t["entries"] == int(lens.sum())
    used = t["row_slots"].astype(np.int64)
    assert len(set(used.tolist())) == len(used) and (used >= 0).all() and (used < cap).all()
    slot_row = np.full(cap, -1, np.int64)
    slot_part = np.zeros(cap, np.int64)
    slot_parts = np.ones(cap, np.int64)
    for q, r in enumerate(rows):
        for p_, s_ in enumerate(used[t["row_slot_first"][q]:t["row_slot_first"][q + 1]]):
            slot_row[s_], slot_part[s_], slot_parts[s_] = r, p_, parts[q]
    assert (t["hub_row"].astype(np.int64) == slot_row).all()  # unused slots say -1
    # the streams
    first, total = t["stream_first"], t["stream_total"].astype(np.int64)
    padded = -(-total // 64) * 64
    assert first[0] == 0 and (first[1:] == np.cumsum(padded)[:-1]).all() and int(padded.sum()) == t["stored"]
    assert int(total.sum()) == t["entries"]
    seen = []
    for s_ in range(t["streams"]):
        rng, wave = divmod(s_, WAVES_PER_RANGE)
        lo, n, npad = int(first[s_]), int(total[s_]), int(padded[s_])
        pos = t["stream_pos"][lo:lo + n].astype(np.int64)
        run = t["stream_run"][lo:lo + n].astype(np.int64)
        # padding: slot 255, a valid position
        assert (t["stream_run"][lo + n:lo + npad] == 255).all() and (t["stream_pos"][lo + n:lo + npad] == 0).all()
        marks = t["stream_mark"][s_].astype(np.int64)
        w_begin = rng * wpr
        n_w = max(0, min(wpr, -(-k // window) - w_begin))  # windows of this range that hold columns at all
        live = marks[:min(wpr, t["n_windows"] - w_begin)]
        assert (np.diff(live) >= 0).all()
        if n == 0:
            assert (live == 0).all()
            continue
        assert (run < rpw).all()
        slot = wave * rpw + run
        r = slot_row[slot]
        assert (r >= 0).all() and (pos >= rowptr[r]).all() and (pos < rowptr[r + 1]).all()  # under the slot of its own row
        w = col[pos] // window
        assert (w >= w_begin).all() and (w < w_begin + wpr).all()  # inside the stream's column range
        assert (np.diff(w) >= 0).all()  # window after window
        # the batch in which each window begins: entries of the windows before it, in batches of 64
        before = np.searchsorted(w, np.arange(w_begin, w_begin + len(live)), side="left")
        assert (live == before // 64).all(), (s_, live[:8], before[:8])
        assert n_w <= len(live)
        # inside a window: the runs of the wavefront's slots one after the other, each a contiguous stretch of the CSR arrays
        key = w * rpw + run
        assert (np.diff(key) >= 0).all()
        same = np.diff(key) == 0
        assert (np.diff(pos)[same] == 1).all()
        # part p of P takes the p-th P-th of the row's entries inside the window
        row_lo = rowptr[r]
        row_cols_before = np.empty(n, np.int64)  # position of the first entry of the row that lies in the window
        for rr in np.unique(r):
            m_ = r == rr
            seg = col[rowptr[rr]:rowptr[rr + 1]]
            assert (np.diff(seg) >= 0).all()
            w_first = np.searchsorted(seg, w[m_] * window, side="left")
            w_last = np.searchsorted(seg, (w[m_] + 1) * window, side="left")
            j = pos[m_] - row_lo[m_] - w_first
            n_in = w_last - w_first
            p_, P = slot_part[slot[m_]], slot_parts[slot[m_]]
            assert (j >= n_in * p_ // P).all() and (j < n_in * (p_ + 1) // P).all()
        seen.append(pos)
    seen = np.sort(np.concatenate(seen)) if seen else np.empty(0, np.int64)
    want = np.sort(np.concatenate([np.arange(rowptr[r], rowptr[r + 1]) for r in rows])) if len(rows) else np.empty(0, np.int64)
    assert len(seen) == len(want) and (seen == want).all()  # every entry of every hub row exactly once


def random_matrix(seed):
    gen = torch.Generator().manual_seed(100 + seed)
    m = int(torch.randint(50, 4000, (1,), generator=gen))
    k = int(torch.randint(9, 30000, (1,), generator=gen))
    seg_len = [2, 8, 64, 256][seed % 4]
    lens = torch.randint(0, 6, (m,), generator=gen)
    long_rows = torch.randperm(m, generator=gen)[: max(3, m // 20)]
    lens[long_rows] = torch.randint(seg_len + 1, max(seg_len + 2, min(k, 40 * seg_len)), (long_rows.numel(),), generator=gen)
    lens[long_rows[0]] = k
    lens = lens.clamp(max=k)
    cols = [torch.randperm(k, generator=gen)[: int(n)].sort().values for n in lens]
    rowptr = torch.zeros(m + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(lens, 0)
    return m, k, seg_len, rowptr.to(torch.int32), torch.cat(cols).to(torch.int32)


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7])
def test_hub_tables_hold_every_entry_once_in_the_window_and_slot_they_say(seed):
    say("hub tables of random shape %d, both layouts" % seed)
    if seed == 7:  # a rectangular block with many more columns than rows and rows far beyond one part
        gen = torch.Generator().manual_seed(7)
        m, k, seg_len = 300, 70000, 32
        lens = torch.randint(0, 40, (m,), generator=gen)
        lens[::7] = torch.randint(600, 9000, (len(lens[::7]),), generator=gen)
        cols = [torch.randperm(k, generator=gen)[: int(n)].sort().values for n in lens]
        rowptr = torch.zeros(m + 1, dtype=torch.int64)
        rowptr[1:] = torch.cumsum(lens, 0)
        rowptr, col = rowptr.to(torch.int32), torch.cat(cols).to(torch.int32)
    else:
        m, k, seg_len, rowptr, col = random_matrix(seed)
    val = torch.ones(col.numel())
    a = ops.CsrMatrix(rowptr.to(DEV), col.to(DEV), val.to(DEV), (m, k), seg_len)
    a.build_hub()
    a.build_hub_wide()
    for wide, factor in ((False, 16), (True, 32)):
        t = hub_tables(a, wide)
        assert t["n_rows"] > 0 and t["rpw"] == (18 if wide else 36)
        check_tables(rowptr.numpy(), col.numpy(), k, seg_len, t, factor)
