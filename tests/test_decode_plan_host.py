"""CPU tests of the decode planner (the replacement of BlitzBatchDecodeHandler::plan,
src/kernel/flashinfer_types.cu:52-80): the schedule is pure integer work on the host copies of indptr /
last_page_len, so its invariants are checked here without a GPU through bz_decode_plan_workspace (which
builds the same schedule for a stated number of compute units) and bz_decode_plan_host_schedule.

What must hold for the kernels to be right: every 32-token tile of every (sequence, kv head) appears in
exactly one record, in order inside its piece; the records point at the pages that hold the tile; the
wave slots cover the records without gaps and evenly; a (sequence, kv head) cut into several pieces, or
longer than split_tokens, gets distinct partial slots and one combine entry; the general kernel's
segments tile every sequence's pages exactly once."""
import numpy as np
import pytest

from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl

CUS = 256


def schedule(lens, Hq, Hkv, D, P, split_tokens=0, cus=CUS):
    rng = np.random.default_rng(1)
    lens = np.asarray(lens, np.int64)
    need = int(((lens + P - 1) // P).sum())
    indices, indptr, lpl = wl.page_table_for(lens, P, max(1, 2 * need), rng)
    h = K.BlitzBatchDecodeHandler()
    fb, ib = h.workspace(indptr, lpl, len(lens), Hq, Hkv, D, P, split_tokens=split_tokens, num_compute_units=cus)
    names = ["segments", "combos", "empty", "tiles", "slot_ptr", "pieces", "mcombos", "units"]
    s = {n: h.host_schedule(i) for i, n in enumerate(names)}
    s.update(indptr=np.asarray(indptr), lens=lens, float_bytes=fb, int_bytes=ib)
    return s


def check_mfma_schedule(s, Hkv, P, split_tokens):
    lens, indptr = s["lens"], s["indptr"]
    tiles, pieces, slot_ptr, mc = s["tiles"], s["pieces"], s["slot_ptr"][:, 0], s["mcombos"]
    cap = 0x7FFFFFFF if split_tokens == 0xFFFFFFFF else max(1, (split_tokens or 2048) // 32)
    # every tile exactly once, pointing at its pages
    seen = set()
    for idx0, idx1, t, pc in tiles:
        seq, kvh, t0, t1 = pieces[pc][:4]
        assert t0 <= t < t1
        key = (seq, kvh, t)
        assert key not in seen
        seen.add(key)
        npg = indptr[seq + 1] - indptr[seq]
        assert idx0 == indptr[seq] + min((32 * t) // P, npg - 1)
        assert idx1 == indptr[seq] + min((32 * t + 16) // P, npg - 1)
    want = {(b, h, t) for b in range(len(lens)) for h in range(Hkv) for t in range((int(lens[b]) + 31) // 32)}
    assert seen == want
    # records of a piece are consecutive and ascending; pieces are in record order
    pos = 0
    for i, pc in enumerate(pieces):
        seq, kvh, t0, t1, partial, combo, count, first, ip0, npg, seq_len = pc[:11]
        assert t1 - t0 <= cap and t1 > t0
        assert (ip0, npg, seq_len) == (indptr[seq], indptr[seq + 1] - indptr[seq], lens[seq])
        block = tiles[pos:pos + (t1 - t0)]
        assert (block[:, 3] == i).all() and (block[:, 2] == np.arange(t0, t1)).all()
        pos += t1 - t0
    assert pos == len(tiles)
    # wave slots: monotone cover, no more than 8 per compute unit, even shares (within the odd/even skew + 1)
    assert slot_ptr[0] == 0 and slot_ptr[-1] == len(tiles) and (np.diff(slot_ptr) >= 0).all()
    shares = np.diff(slot_ptr)
    assert len(shares) <= CUS * 8
    if split_tokens != 0xFFFFFFFF and len(tiles) >= CUS * 8:
        assert shares.min() >= 1 and shares.max() <= np.ceil(shares.mean() * 1.06) + 1
    # partial slots and combine entries
    by_unit = {}
    for i, pc in enumerate(pieces):
        by_unit.setdefault((pc[0], pc[1]), []).append(pc)
    used = []
    for (seq, kvh), pcs in by_unit.items():
        assert [p[2] for p in pcs] == sorted(p[2] for p in pcs) and pcs[0][2] == 0
        assert all(a[3] == b[2] for a, b in zip(pcs, pcs[1:])) and pcs[-1][3] == (int(lens[seq]) + 31) // 32
        if len(pcs) == 1:
            assert pcs[0][4] == -1
        else:
            first = pcs[0][7]
            assert [p[4] for p in pcs] == list(range(first, first + len(pcs)))
            assert all(p[6] == len(pcs) and p[7] == first for p in pcs)
            c = mc[pcs[0][5]]
            assert tuple(c) == (seq, kvh, first, len(pcs))
            used.extend(p[4] for p in pcs)
    assert sorted(used) == list(range(len(used))) and len(mc) == sum(len(v) > 1 for v in by_unit.values())


def check_general_schedule(s, P):
    lens, indptr = s["lens"], s["indptr"]
    segs, combos, empty = s["segments"], s["combos"], s["empty"][:, 0]
    assert sorted(empty) == [b for b in range(len(lens)) if lens[b] == 0]
    cover = {}
    for seq, lo, hi, partial in segs:
        assert 0 <= lo < hi <= indptr[seq + 1] - indptr[seq]
        cover.setdefault(seq, []).append((lo, hi, partial))
    sizes = (segs[:, 2] - segs[:, 1])
    assert (np.diff(sizes) <= 0).all()  # longest first
    n_partials = 0
    for seq, lst in cover.items():
        lst.sort()
        assert lst[0][0] == 0 and lst[-1][1] == indptr[seq + 1] - indptr[seq]
        assert all(a[1] == b[0] for a, b in zip(lst, lst[1:]))
        if len(lst) == 1:
            assert lst[0][2] == -1
        else:
            c = [c for c in combos if c[0] == seq]
            assert len(c) == 1 and c[0][2] == len(lst)
            assert [x[2] for x in lst] == list(range(c[0][1], c[0][1] + len(lst)))
            n_partials += len(lst)
    assert set(cover) == {b for b in range(len(lens)) if lens[b] > 0}
    assert len(combos) == sum(len(v) > 1 for v in cover.values())
    return n_partials


@pytest.mark.parametrize("name,lens,Hq,Hkv,P,split", [
    ("headline", None, 32, 8, 16, 2048),                       # config 3: lognormal contexts, batch 128
    ("page64", None, 32, 8, 64, 2048),
    ("small_batch", [1024] * 8, 32, 8, 16, 2048),              # fewer tiles than wave slots
    ("ragged", [0, 1, 31, 32, 33, 4097, 0, 700, 16, 17], 16, 2, 16, 256),
    ("never_split", [5000, 40, 900], 8, 8, 16, 0xFFFFFFFF),
    ("one_token", [1], 8, 1, 16, 0),
    ("page48", [100, 1000, 47, 48, 49], 32, 8, 48, 512),      # page size not a power of two
    ("group32", [700, 64, 3000], 32, 1, 16, 2048),             # 32 q heads on one kv head: two parts of 16
    ("group24", [700, 64, 3000], 48, 2, 16, 2048),             # 24 per kv head: two parts of 12
])
def test_matrix_core_schedule_invariants(name, lens, Hq, Hkv, P, split):
    if lens is None:
        lens = wl.lognormal_ctx(np.random.default_rng(0x5EED), 128, 1024, 1.0, 64, 8192)
    s = schedule(lens, Hq, Hkv, 128, P, split)
    # a kv head with more than 16 q heads is scheduled as equal parts, each a unit of its own
    G = Hq // Hkv
    parts = next(p for p in range((G + 15) // 16, G + 1) if G % p == 0)
    units = Hkv * parts
    assert len(s["tiles"]) == sum((int(l) + 31) // 32 for l in lens) * units
    check_mfma_schedule(s, units, P, split)
    assert (s["pieces"][:, 11] == s["pieces"][:, 1] // parts).all()  # the kv head whose K/V a piece reads
    n_partials = check_general_schedule(s, P)
    # reported workspace: the sections the kernels read, 256-byte aligned
    al = lambda x: (x + 255) // 256 * 256
    n_mp = int(s["mcombos"][:, 3].sum()) if len(s["mcombos"]) else 0  # partial slots of the matrix-core path
    assert s["int_bytes"] == (al(len(s["segments"]) * 16) + al(len(s["combos"]) * 16) + al(len(s["empty"]) * 4) +
                              al(len(s["pieces"]) * 64) + al((len(s["slot_ptr"]) - 1) * 64) +
                              al(len(s["mcombos"]) * 16) + al(len(s["tiles"]) * 16) + al(len(s["units"]) * 32))
    # (the one-call decode step keeps one partial per piece, split or not)
    assert s["float_bytes"] == max(al(n_partials * Hq * 128 * 4) + al(n_partials * Hq * 4),
                                   al(n_mp * 16 * 128 * 4) + al(n_mp * 16 * 4),
                                   al(len(s["pieces"]) * 16 * 128 * 4) + al(len(s["pieces"]) * 16 * 4))
    # every (sequence with pages, unit) is listed once with its consecutive run of pieces
    un = s["units"]
    live = [b for b, l in enumerate(lens) if l > 0]
    assert [tuple(r[:2]) for r in un] == [(b, h) for b in live for h in range(units)]
    assert (un[:, 3] >= 1).all() and (un[1:, 2] == un[:-1, 2] + un[:-1, 3]).all() and un[0, 2] == 0
    assert un[-1, 2] + un[-1, 3] == len(s["pieces"])
    for b, h, first, cnt, ip0, ntok in un[:: max(1, len(un) // 50), :6]:
        pc = s["pieces"][first:first + cnt]
        assert (pc[:, 0] == b).all() and (pc[:, 1] == h).all()
        assert ip0 == s["indptr"][b] and ntok == lens[b]


def test_shapes_outside_the_matrix_core_kernel_get_segments_only():
    # config 1 of the baseline (head_dim 64): hand-checked segments; 4 sequences of 2, 4, 9, 16 pages
    s = schedule([17, 64, 130, 255], 4, 4, 64, 16, split_tokens=0)
    assert len(s["tiles"]) == 0 and len(s["pieces"]) == 0
    check_general_schedule(s, 16)
    # 31 pages over 4 sequences is far fewer items than 4 per compute unit: pieces shrink to 256 tokens = 16 pages,
    # so nothing is cut here
    assert sorted(map(tuple, s["segments"][:, :3])) == [(0, 0, 2), (1, 0, 4), (2, 0, 9), (3, 0, 16)]
    assert (s["segments"][:, 3] == -1).all() and s["float_bytes"] == 0
    # a long sequence at the same shape is cut into equal page-aligned pieces with one combine entry
    s = schedule([4096], 4, 4, 64, 16, split_tokens=1024)
    segs = s["segments"]
    assert len(segs) == 16 and (segs[:, 2] - segs[:, 1] == 16).all() and sorted(segs[:, 3]) == list(range(16))
    assert [tuple(c) for c in s["combos"]] == [(0, 0, 16, 0)]


def test_fewer_compute_units_mean_fewer_longer_shares():
    lens = [2048] * 64
    a = schedule(lens, 32, 8, 128, 16, 2048, cus=256)
    b = schedule(lens, 32, 8, 128, 16, 2048, cus=64)
    assert len(a["slot_ptr"]) - 1 == 2048 and len(b["slot_ptr"]) - 1 == 512
    assert np.diff(b["slot_ptr"][:, 0]).mean() == pytest.approx(4 * np.diff(a["slot_ptr"][:, 0]).mean())


@pytest.mark.parametrize("lens,Hq,Hkv", [
    ([20, 37], 4, 2),
    ([128, 129, 1, 4096, 0, 640], 8, 8),
    (None, 40, 40),  # config 4: 16 prompts U[128, 4096], 40 heads
    ([512, 300, 2048, 77], 32, 8),  # grouped-query attention with enough units: whole groups stay together
    ([4096], 32, 4),                # ... and with too few: the group of 8 is cut into parts
    ([700, 300, 300, 1200, 129, 128, 127], 16, 8),  # seven units per column, groups of two
])
def test_prefill_job_list_invariants(lens, Hq, Hkv):
    """The prefill plan (replacement of BatchPrefillRaggedHandler::plan, src/kernel/flashinfer_types.cu:24-49):
    one job per (request, q head, 128-row q tile), each exactly once; the jobs of a (request, kv head) unit
    sit in one column of the 8-wide launch order (one XCD, consecutive there), the q heads of the group side
    by side, tiles from the last to the first -- or, for every second unit of a column of six or more units,
    its last two excepted, from the first to the last; longer requests come first; padding entries have
    length 0."""
    if lens is None:
        lens = np.random.default_rng(0x5EED).integers(128, 4097, 16)
    lens = np.asarray(lens, np.int64)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    h = K.BatchPrefillRaggedHandler()
    fb, ib = h.workspace(indptr, indptr, len(lens), Hq, Hkv, 128)
    items = h.host_schedule()
    assert items.shape[1] == 8 and np.array_equal(items[:, 4:6], items[:, 0:2]) and not items[:, 6:].any()  # K/V range = q range here
    items = items[:, :4]
    # float workspace: the angle table of the q rotation, 512 bytes per position of the longest request
    assert fb == 512 * max(lens) and ib == (len(items) * 32 + 255) // 256 * 256 and len(items) % 8 == 0
    tok0_to_req = {int(indptr[b]): b for b in range(len(lens)) if lens[b] > 0}
    seen, column, q0s = set(), {}, {}
    first_seen_len = []
    for i, (tok0, ln, q0, head) in enumerate(items):
        if ln == 0:
            continue
        b = tok0_to_req[int(tok0)]
        assert ln == lens[b] and q0 % 128 == 0 and 0 <= q0 < ln and 0 <= head < Hq
        key = (b, int(head), int(q0))
        assert key not in seen
        seen.add(key)
        pair = (b, int(head))
        assert column.setdefault(pair, i % 8) == i % 8
        if pair not in q0s:
            first_seen_len.append(int(ln))
        q0s.setdefault(pair, []).append(int(q0))
    want = {(b, hd, q0) for b in range(len(lens)) for hd in range(Hq) for q0 in range(0, int(lens[b]), 128)}
    assert seen == want
    # a unit's tiles are consecutive in its column: most keys first, or fewest keys first for the units named above
    G = Hq // Hkv
    live = int((lens > 0).sum())
    parts = next(p for p in range(1, G + 1) if G % p == 0 and (live * Hkv * p >= 16 or p == G))
    per_part = G // parts
    units_per_col = live * Hkv * parts // 8
    nth_in_col, n_ascending = {}, 0
    for (b, hd), seq in q0s.items():  # (in order of first appearance)
        unit = (b, hd - hd % per_part)
        if unit not in nth_in_col:
            nth_in_col[unit] = sum(1 for u in nth_in_col if column[u] == column[unit])
        nth = nth_in_col[unit]
        down = list(range((int(lens[b]) - 1) // 128 * 128, -1, -128))
        ascending = nth % 2 == 1 and units_per_col >= 6 and nth + 2 < units_per_col
        assert seq == (down[::-1] if ascending else down)
        n_ascending += ascending
    assert (n_ascending > 0) == (units_per_col >= 6)
    # pairs are dealt to the columns in turn, longest requests first: within one column lengths never grow
    for c in range(8):
        col = [int(ln) for (tok0, ln, q0, head) in items[c::8] if ln > 0]
        assert all(a >= b for a, b in zip(col, col[1:]))
    # grouped-query attention: the q heads of a kv head travel together (same column, same tile side by side)
    # unless that would leave fewer than two units per column, in which case the group is cut into equal parts
    for (b, hd), c in column.items():
        assert c == column[(b, hd - hd % per_part)]
    # no column holds more than its share of units + 1
    per_col = np.bincount([c for (b, hd), c in column.items() if hd % per_part == 0], minlength=8)
    assert per_col.max() - per_col.min() <= 1
    # a head size the kernel does not cover is refused on the host
    with pytest.raises(K.BzError):
        h.workspace(indptr, indptr, len(lens), Hq, Hkv, 64)


def test_prefill_job_list_with_distinct_q_and_kv_lengths():
    """qo_indptr != kv_indptr: a job covers 128 q rows of the request's last qo_len tokens and carries the request's
    K/V range; requests are ordered by their K/V length (what a tile's work goes with); no q rows, no jobs."""
    kv_lens = np.array([300, 64, 1000, 40], np.int64)
    q_lens = np.array([130, 64, 0, 1], np.int64)
    qo = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    kv = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int32)
    h = K.BatchPrefillRaggedHandler()
    fb, ib = h.workspace(qo, kv, 4, 8, 2, 128)
    items = h.host_schedule()
    assert fb == 512 * 1000  # the angle table covers the longest K/V length
    live = items[items[:, 1] > 0]
    want = {(b, hd, q0) for b in range(4) for hd in range(8) for q0 in range(0, int(q_lens[b]), 128)}
    seen = set()
    for tok0, ln, q0, head, kv0, kv_len, _, _ in live:
        b = int(np.searchsorted(qo[1:], tok0, side="right"))
        while q_lens[b] == 0:
            b += 1
        assert tok0 == qo[b] and ln == q_lens[b] and kv0 == kv[b] and kv_len == kv_lens[b]
        seen.add((b, int(head), int(q0)))
    assert seen == want and len(live) == len(want)
    first = [int(r[5]) for r in live[::1] if r[2] == (r[1] - 1) // 128 * 128 and r[3] == 0]
    assert first[0] == 300  # among the requests with q rows, the longest K/V range is dealt first
    with pytest.raises(K.BzError):
        h.workspace(kv, qo, 4, 8, 2, 128)  # fewer K/V rows than q rows
