"""GPU parity of the device-side re-placement kernels (rank select, membership bitmap, ordered bitmap compaction)
against numpy: a full sort for the rank threshold, flatnonzero for the compactions."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import PinnedArray, dev_bytes, dev_zeros_u32, ptr, status_value, sync, to_dev, to_np
from ugache_amd import hip

pytestmark = pytest.mark.gpu


def ranks_of(counts):
    """observed rows by (count << 32 | row), never-observed rows behind them in ascending row order
    (freq_recorder.cc:275-281 for the observed ones)"""
    rows = np.arange(len(counts), dtype=np.uint64)
    c = counts.astype(np.uint64)
    return np.where(c > 0, (c << np.uint64(32)) | rows, np.uint64(0xFFFFFFFF) - rows)


def _counts(rng, n, kind):
    if kind == "zipf":  # most rows never observed, a few hot
        c = np.zeros(n, np.uint32)
        hit = rng.zipf(1.2, size=max(n // 2, 1)) % n
        np.add.at(c, hit, 1)
        return c
    if kind == "ties":  # few distinct values: the row number decides
        return rng.integers(0, 3, size=n).astype(np.uint32)
    if kind == "huge":  # counts in every digit of the 32 bits
        return (rng.integers(0, 1 << 32, size=n, dtype=np.uint64) * (rng.random(n) < 0.7)).astype(np.uint32)
    if kind == "zero":
        return np.zeros(n, np.uint32)
    if kind == "saturated":  # the k-th best count lies at or beyond the 2047 the first histogram pass tells apart
        return rng.integers(2040, 2060, size=n).astype(np.uint32) * (rng.random(n) < 0.9)
    raise AssertionError(kind)


def _place(counts, k, reset, with_observed=False, keep=None, ws=None):
    """-> membership bits of the k best rows, the rank threshold, the counters afterwards.
    keep (bool per row, optional): rows that win ties at the k-th count (ugk_rank_place_keep);
    ws (optional): a workspace that earlier placements have used"""
    n = len(counts)
    words = (n + 63) // 64
    d_counts = to_dev(counts)
    if ws is None:
        ws = dev_bytes(hip.lib().ugk_rank_workspace_bytes())
    bitmap = dev_bytes(words * 8, fill=0xA5)
    scratch = dev_bytes(words * 8, fill=0x5A)
    observed = None
    if with_observed:  # the bitmap ugk_record_* would have kept: counter above zero
        pad = np.zeros(words * 64, bool)
        pad[:n] = counts > 0
        observed = to_dev(np.packbits(pad, bitorder="little").view(np.uint64))
    if keep is None:
        hip.call("ugk_rank_place", ptr(d_counts), n, k, ptr(ws), ptr(bitmap), ptr(scratch), ptr(observed), reset, None)
    else:
        pad = np.zeros(words * 64, bool)
        pad[:n] = keep
        d_keep = to_dev(np.packbits(pad, bitorder="little").view(np.uint64))
        hip.call("ugk_rank_place_keep", ptr(d_counts), n, k, ptr(ws), ptr(bitmap), ptr(scratch), ptr(observed),
                 ptr(d_keep), reset, None)
        assert np.array_equal(to_np(d_keep, np.uint8)[: words * 8], np.packbits(pad, bitorder="little"))  # read only
    th = C.c_uint64(0)
    hip.call("ugk_rank_threshold", ptr(ws), C.byref(th), None)
    bits = np.unpackbits(to_np(bitmap)[: words * 8], bitorder="little")
    assert not bits[n:].any()  # the tail of the last word is clear
    if with_observed:
        left = np.unpackbits(to_np(observed, np.uint8)[: words * 8], bitorder="little")[:n].astype(bool)
        assert np.array_equal(left, (counts > 0) & (reset == 0))  # cleared together with the counters
    return bits[:n].astype(bool), th.value, to_np(d_counts, np.uint32)[:n]


@pytest.mark.parametrize("kind", ["zipf", "ties", "huge", "zero", "saturated"])
@pytest.mark.parametrize("n", [1, 3, 63, 64, 65, 1000, 100_003, 2_000_001])
def test_rank_place_matches_a_full_sort(kind, n):
    rng = np.random.default_rng(n * 7 + len(kind))
    counts = _counts(rng, n, kind)
    ranks = ranks_of(counts)
    order = np.sort(ranks)[::-1]
    observed = int((counts > 0).sum())
    ks = sorted({0, 1, n // 3, max(observed - 1, 0), observed, min(observed + 1, n), n - 1, n, n + 5})
    for k in ks:
        if k == 0:
            want = np.zeros(n, bool)
        elif k >= n:
            want = np.ones(n, bool)
        else:
            want = ranks >= order[k - 1]
        assert int(want.sum()) == min(k, n)
        for reset, with_observed in ((0, False), (1, False), (0, True), (1, True)):
            got, th, left = _place(counts, k, reset, with_observed)
            if 0 < k < n:
                assert th == int(order[k - 1]), (kind, n, k, with_observed)
            assert np.array_equal(got, want), (kind, n, k, reset, with_observed)
            assert np.array_equal(left, counts if reset == 0 else np.zeros(n, np.uint32))


@pytest.mark.parametrize("kind", ["zipf", "ties", "saturated"])
@pytest.mark.parametrize("n", [65, 1000, 100_003, 2_000_001])
def test_placements_that_share_a_workspace(kind, n):
    """With the counters kept, the first pass over them splits by the threshold count of the placement before (left in
    the workspace) and the second pass is skipped when that guess holds.  A sequence of placements in one workspace -
    the same one again (guess right), counters grown a little (mostly right), another k (wrong), counters grown a lot
    (wrong), a placement with a reset in between (two passes, as before) - gives what a full sort gives every time."""
    rng = np.random.default_rng(n * 3 + len(kind))
    counts = _counts(rng, n, kind)
    ws = dev_bytes(hip.lib().ugk_rank_workspace_bytes(), fill=0xC3)  # whatever the memory held: a guess like any other
    observed = int((counts > 0).sum())
    k0 = max(1, min(observed // 2, n - 1))
    steps = [("same", k0), ("same", k0), ("grow_a_little", k0), ("same", max(1, k0 // 3)), ("grow_a_lot", k0),
             ("reset", k0), ("same", k0), ("same", min(n - 1, max(1, observed + 1)))]
    for what, k in steps:
        if what == "grow_a_little":
            counts = counts.copy()
            counts[rng.integers(0, n, size=max(n // 200, 1))] += 1
        elif what == "grow_a_lot":
            counts = (counts + rng.integers(0, 4, size=n)).astype(np.uint32)
        ranks = ranks_of(counts)
        order = np.sort(ranks)[::-1]
        want = ranks >= order[k - 1]
        for keep in (None, rng.random(n) < 0.5):
            if keep is not None:
                rows = np.arange(n, dtype=np.int64)
                best = np.lexsort((np.where(counts > 0, rows, -rows), keep, counts))[::-1]
                want_k = np.zeros(n, bool)
                want_k[best[:k]] = True
            got, th, left = _place(counts, k, 1 if what == "reset" else 0, with_observed=(n % 2 == 1), keep=keep, ws=ws)
            assert np.array_equal(got, want if keep is None else want_k), (kind, n, what, k, keep is not None)
            if keep is None:
                assert th == int(order[k - 1])
            assert np.array_equal(left, np.zeros(n, np.uint32) if what == "reset" else counts)


def test_rank_place_picks_the_hotter_rows_and_breaks_ties_towards_larger_rows():
    # hand-worked: counts 0 5 5 0 9 1 0 -> order 4, 2, 1, 5, then the never-observed rows 0, 3, 6
    counts = np.array([0, 5, 5, 0, 9, 1, 0], np.uint32)
    for k, want_rows in [(1, [4]), (2, [4, 2]), (3, [4, 2, 1]), (4, [4, 2, 1, 5]), (5, [4, 2, 1, 5, 0]),
                         (6, [4, 2, 1, 5, 0, 3])]:
        got, _, _ = _place(counts, k, 0)
        assert sorted(np.flatnonzero(got).tolist()) == sorted(want_rows)


@pytest.mark.parametrize("kind", ["zipf", "ties", "zero", "saturated", "huge"])
@pytest.mark.parametrize("n", [1, 64, 65, 1000, 100_003, 2_000_001])
def test_rank_place_with_kept_rows_winning_ties(kind, n):
    """rows ordered by (count, kept, row for counted rows / -row for the others), every key distinct: the k best by a
    full lexicographic sort"""
    rng = np.random.default_rng(n * 11 + len(kind))
    counts = _counts(rng, n, kind)
    rows = np.arange(n, dtype=np.int64)
    tie = np.where(counts > 0, rows, -rows)
    observed = int((counts > 0).sum())
    for keep_share in (0.0, 0.2, 0.9, 1.0):
        keep = rng.random(n) < keep_share
        order = np.lexsort((tie, keep, counts))[::-1]  # best first; the last key of lexsort is the primary one
        n_kept_zero = int((keep & (counts == 0)).sum())
        ks = sorted({1, n // 3, observed, min(observed + max(n_kept_zero - 1, 0), n), min(observed + n_kept_zero, n),
                     min(observed + n_kept_zero + 1, n), n - 1} - {0})
        for k in ks:
            if k >= n:
                continue
            want = np.zeros(n, bool)
            want[order[:k]] = True
            for reset, with_observed in ((0, False), (1, True), (0, True)):
                got, th, left = _place(counts, k, reset, with_observed, keep=keep)
                assert np.array_equal(got, want), (kind, n, k, keep_share, reset, with_observed)
                last = order[k - 1]
                want_th = (int(counts[last]) << 32) | int(last) if counts[last] else 0xFFFFFFFF - int(last)
                assert th == want_th
                assert np.array_equal(left, counts if reset == 0 else np.zeros(n, np.uint32))
            if keep_share == 0.0:  # nothing kept: the plain placement
                plain, _, _ = _place(counts, k, 0)
                assert np.array_equal(plain, want)


def test_rank_place_keeps_cached_rows_the_counters_do_not_tell_apart():
    # hand-worked: counts 0 5 5 0 9 1 0 0, rows 3 and 7 kept.  Counted rows first: 4, 2, 1, 5; then the kept
    # never-counted rows 3, 7 (ascending), then 0, 6.  With k = 2 the tie of rows 1 and 2 goes to the kept one.
    counts = np.array([0, 5, 5, 0, 9, 1, 0, 0], np.uint32)
    keep = np.zeros(8, bool)
    keep[[3, 7]] = True
    for k, want_rows in [(4, [4, 2, 1, 5]), (5, [4, 2, 1, 5, 3]), (6, [4, 2, 1, 5, 3, 7]), (7, [4, 2, 1, 5, 3, 7, 0])]:
        got, _, _ = _place(counts, k, 0, keep=keep)
        assert sorted(np.flatnonzero(got).tolist()) == sorted(want_rows), k
    keep[:] = False
    keep[1] = True
    got, _, _ = _place(counts, 2, 0, keep=keep)
    assert sorted(np.flatnonzero(got).tolist()) == [1, 4]
    got, _, _ = _place(counts, 2, 0)
    assert sorted(np.flatnonzero(got).tolist()) == [2, 4]


def test_rank_place_on_the_committed_golden_case():
    """tests/golden/extract_small.json: the record stream counted per row, the 16 best rows placed on the device are
    the fixture's cached set (written by brute-force loops, not by the oracle)"""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "extract_small.json")) as f:
        fx = json.load(f)
    counts = np.bincount(np.array(fx["record_stream"]), minlength=fx["n_item"]).astype(np.uint32)
    k = int(fx["n_item"] * fx["cache_percentage"])
    got, th, _ = _place(counts, k, 0)
    assert np.flatnonzero(got).tolist() == fx["cached_keys"]
    last = fx["rank_keys_observed"][k - 1]
    assert th == (fx["rank_counts_observed"][k - 1] << 32) | last


def _place_observed(counts, k, reset, cached=None):
    """ugk_rank_place_observed -> (membership bits or None when the promise was refused, status word, counters afterwards,
    lists of the rows that leave and come in when `cached` is given, the observed count the host was told)"""
    n = len(counts)
    words = (n + 63) // 64
    d_counts = to_dev(counts)
    ws = dev_bytes(hip.lib().ugk_rank_workspace_bytes())
    bitmap = dev_bytes(words * 8, fill=0xA5)
    pad = np.zeros(words * 64, bool)
    pad[:n] = counts > 0
    observed = to_dev(np.packbits(pad, bitorder="little").view(np.uint64))
    st = dev_zeros_u32(1)
    totals = PinnedArray((4,), np.uint32)
    try:
        totals.array[...] = 0xFFFFFFFF
        d_cached = ws_out = ws_in = None
        if cached is not None:
            cpad = np.zeros(words * 64, bool)
            cpad[:n] = cached
            d_cached = to_dev(np.packbits(cpad, bitorder="little").view(np.uint64))
            ws_out = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
            ws_in = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
        hip.call("ugk_rank_place_observed", ptr(d_counts), n, k, ptr(ws), ptr(bitmap), ptr(observed), reset,
                 ptr(d_cached), ptr(ws_out), ptr(ws_in), totals.ptr, ptr(st), None)
        status = status_value(st)
        seen = int(totals.array[2])
        if status & hip.ST_PLACE_PROMISE:
            assert np.array_equal(to_np(bitmap)[: words * 8], np.full(words * 8, 0xA5, np.uint8))  # left as it was
            return None, status, to_np(d_counts, np.uint32)[:n], None, None, seen
        th = C.c_uint64(0)
        hip.call("ugk_rank_threshold", ptr(ws), C.byref(th), None)
        bits = np.unpackbits(to_np(bitmap)[: words * 8], bitorder="little")
        assert not bits[n:].any()
        left = np.unpackbits(to_np(observed, np.uint8)[: words * 8], bitorder="little")[:n].astype(bool)
        assert np.array_equal(left, (counts > 0) & (reset == 0))
        leaving = coming = None
        if cached is not None:
            n_out, n_in = int(totals.array[0]), int(totals.array[1])
            out_l, in_l = dev_zeros_u32(max(n_out, 1)), dev_zeros_u32(max(n_in, 1))
            hip.call("ugk_bitmap_emit", ptr(d_cached), ptr(bitmap), 0, n, ptr(ws_out), ptr(out_l), n_out, None)
            hip.call("ugk_bitmap_emit", ptr(bitmap), ptr(d_cached), 0, n, ptr(ws_in), ptr(in_l), n_in, None)
            sync()
            leaving, coming = to_np(out_l, np.uint32)[:n_out], to_np(in_l, np.uint32)[:n_in]
            # both lists in one launch from the same two workspaces
            out_2, in_2 = dev_zeros_u32(max(n_out, 1)), dev_zeros_u32(max(n_in, 1))
            hip.call("ugk_bitmap_emit_diff", ptr(d_cached), ptr(bitmap), n, ptr(ws_out), ptr(ws_in), ptr(out_2), n_out,
                     ptr(in_2), n_in, None)
            sync()
            assert np.array_equal(to_np(out_2, np.uint32)[:n_out], leaving)
            assert np.array_equal(to_np(in_2, np.uint32)[:n_in], coming)
        return bits[:n].astype(bool), (status, th.value), to_np(d_counts, np.uint32)[:n], leaving, coming, seen
    finally:
        totals.free()


@pytest.mark.parametrize("kind", ["zipf", "zero", "ties"])
@pytest.mark.parametrize("n", [2, 3, 63, 64, 65, 1000, 100_003, 2_000_001, 40_000_000])
def test_rank_place_observed_is_rank_place_where_few_rows_were_observed(kind, n):
    """every observed row and the lowest never-observed ones, as ugk_rank_place and a full sort give them; the rows
    that leave and come in against a cached set, counted on the way, as flatnonzero gives them; k at or below the
    number of observed rows is refused"""
    rng = np.random.default_rng(n * 13 + len(kind))
    if n < 40_000_000:
        counts = _counts(rng, n, kind)
    else:  # sparse: whole chunks and blocks without an observed row
        counts = np.zeros(n, np.uint32)
        counts[rng.integers(0, n, size=300_000)] = 3
        counts[n // 2: n // 2 + 100_000] = 1
    ranks = ranks_of(counts)
    order = np.sort(ranks)[::-1]
    observed = int((counts > 0).sum())
    ks = sorted({observed + 1, observed + 2, (observed + n) // 2, n - 1} - {0, n})
    ks = [k for k in ks if observed < k < n]
    for k in ks:
        want = ranks >= order[k - 1]
        cached = np.zeros(n, bool)
        cached[rng.permutation(n)[: max(k - 1, 0)] if n < 3_000_000 else slice(0, k - 1)] = True
        for reset in (0, 1):
            got, (status, th), left, leaving, coming, seen = _place_observed(counts, k, reset, cached)
            assert status == 0 and seen == observed
            assert th == int(order[k - 1]), (kind, n, k)
            assert np.array_equal(got, want), (kind, n, k, reset)
            assert np.array_equal(left, counts if reset == 0 else np.zeros(n, np.uint32))
            assert np.array_equal(leaving, np.flatnonzero(cached & ~want).astype(np.uint32))
            assert np.array_equal(coming, np.flatnonzero(want & ~cached).astype(np.uint32))
        if n <= 100_003:
            plain, _, _ = _place(counts, k, 0, with_observed=True)
            assert np.array_equal(plain, want)
            got, (status, _), _, leaving, coming, _ = _place_observed(counts, k, 0, None)  # no diff asked for
            assert status == 0 and np.array_equal(got, want) and leaving is None
    for k in sorted({1, observed // 2, observed} - {0}):
        if k >= n or k > observed:
            continue
        got, status, left, _, _, seen = _place_observed(counts, k, 1, np.zeros(n, bool))
        assert got is None and status == hip.ST_PLACE_PROMISE and seen == observed
        assert np.array_equal(left, counts)  # nothing was reset either


def _bits(rng, nbits, density):
    words = (nbits + 63) // 64
    b = rng.random(words * 64) < density
    return np.packbits(b, bitorder="little").view(np.uint64), b


@pytest.mark.parametrize("nbits", [1, 64, 65, 4097, 1_000_003, 40_000_000])
@pytest.mark.parametrize("mode", ["a", "not_a", "a_and_not_b", "not_a_and_not_b"])
def test_bitmap_compaction_matches_flatnonzero(nbits, mode):
    rng = np.random.default_rng(nbits % 1000 + len(mode))
    a_w, a = _bits(rng, nbits, 0.02 if nbits > 10_000_000 else 0.3)
    b_w, b = _bits(rng, nbits, 0.5)
    m = a.copy()
    if mode.startswith("not_a"):
        m = ~m
    use_b = mode.endswith("not_b")
    if use_b:
        m &= ~b
    m[nbits:] = False
    want = np.flatnonzero(m).astype(np.uint32)
    d_a, d_b = to_dev(a_w), to_dev(b_w)
    ws = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
    total = PinnedArray((4,), np.uint32)
    try:
        total.array[...] = 0xFFFFFFFF
        inv = 1 if mode.startswith("not_a") else 0
        hip.call("ugk_bitmap_count", ptr(d_a), ptr(d_b) if use_b else None, inv, nbits, ptr(ws), total.ptr, None)
        sync()
        assert int(total.array[0]) == len(want)
        for max_out in sorted({len(want), len(want) // 2, 1}):
            out = dev_zeros_u32(max(len(want), 1) + 8)
            out.fill_(-1)
            hip.call("ugk_bitmap_emit", ptr(d_a), ptr(d_b) if use_b else None, inv, nbits, ptr(ws), ptr(out), max_out,
                     None)
            sync()
            got = to_np(out, np.uint32)
            lim = min(max_out, len(want))
            assert np.array_equal(got[:lim], want[:lim])
            assert (got[lim: lim + 8] == 0xFFFFFFFF).all()  # nothing written beyond the limit
    finally:
        sync()
        total.free()


@pytest.mark.parametrize("nbits", [1, 64, 65, 4097, 1_000_003, 40_000_000])
@pytest.mark.parametrize("shape", ["dense", "sparse", "run", "same"])
def test_bitmap_emit_diff_writes_both_lists_as_two_emits_would(nbits, shape):
    """a & ~b and b & ~a from one launch = flatnonzero of each, for bitmaps that differ everywhere, in a few places, in
    one contiguous run (what a refresh of never-observed filler rows looks like) and nowhere; limits below the sizes
    cut the lists and nothing is written behind them; a limit of 0 with a null list skips that side"""
    rng = np.random.default_rng(nbits % 977 + len(shape))
    a_w, a = _bits(rng, nbits, 0.3)
    if shape == "dense":
        b_w, b = _bits(rng, nbits, 0.5)
    else:
        b = a.copy()
        if shape == "sparse":
            flip = rng.integers(0, nbits, size=max(nbits // 1000, 1))
            b[flip] = ~b[flip]
        elif shape == "run":
            lo = nbits // 3
            b[lo: lo + max(nbits // 50, 1)] = True
            a[lo: lo + max(nbits // 50, 1)] = False
            a[-(nbits // 7 + 1):] = True
            b[-(nbits // 7 + 1):] = False
            a_w = np.packbits(a, bitorder="little").view(np.uint64)
        b_w = np.packbits(b, bitorder="little").view(np.uint64)
    valid = np.zeros(len(a), bool)
    valid[:nbits] = True
    want_ab = np.flatnonzero(a & ~b & valid).astype(np.uint32)
    want_ba = np.flatnonzero(b & ~a & valid).astype(np.uint32)
    d_a, d_b = to_dev(a_w), to_dev(b_w)
    ws_ab = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
    ws_ba = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
    total = PinnedArray((4,), np.uint32)
    try:
        total.array[...] = 0xFFFFFFFF
        if shape in ("dense", "run"):  # both counts from one pass over the two bitmaps, or one pass each
            hip.call("ugk_bitmap_count_diff", ptr(d_a), ptr(d_b), nbits, ptr(ws_ab), ptr(ws_ba), total.ptr, None)
        else:
            hip.call("ugk_bitmap_count", ptr(d_a), ptr(d_b), 0, nbits, ptr(ws_ab), total.ptr, None)
            hip.call("ugk_bitmap_count", ptr(d_b), ptr(d_a), 0, nbits, ptr(ws_ba), total.ptr + 4, None)
        sync()
        assert (int(total.array[0]), int(total.array[1])) == (len(want_ab), len(want_ba))
        for cut_ab, cut_ba in ((1.0, 1.0), (0.5, 1.0), (1.0, 0.0), (0.0, 0.3)):
            max_ab, max_ba = int(len(want_ab) * cut_ab), int(len(want_ba) * cut_ba)
            out_ab, out_ba = dev_zeros_u32(len(want_ab) + 8), dev_zeros_u32(len(want_ba) + 8)
            out_ab.fill_(-1)
            out_ba.fill_(-1)
            hip.call("ugk_bitmap_emit_diff", ptr(d_a), ptr(d_b), nbits, ptr(ws_ab), ptr(ws_ba),
                     ptr(out_ab) if max_ab else None, max_ab, ptr(out_ba) if max_ba else None, max_ba, None)
            sync()
            got_ab, got_ba = to_np(out_ab, np.uint32), to_np(out_ba, np.uint32)
            assert np.array_equal(got_ab[:max_ab], want_ab[:max_ab]), (nbits, shape, cut_ab)
            assert np.array_equal(got_ba[:max_ba], want_ba[:max_ba]), (nbits, shape, cut_ba)
            assert (got_ab[max_ab: max_ab + 8] == 0xFFFFFFFF).all() and (got_ba[max_ba: max_ba + 8] == 0xFFFFFFFF).all()
    finally:
        sync()
        total.free()


def test_bitmap_compaction_of_an_empty_and_a_full_set():
    nbits = 70_000
    ws = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
    total = PinnedArray((4,), np.uint32)
    try:
        zero = to_dev(np.zeros((nbits + 63) // 64, np.uint64))
        hip.call("ugk_bitmap_count", ptr(zero), None, 0, nbits, ptr(ws), total.ptr, None)
        sync()
        assert total.array[0] == 0
        hip.call("ugk_bitmap_count", ptr(zero), None, 1, nbits, ptr(ws), total.ptr, None)
        out = dev_zeros_u32(nbits)
        hip.call("ugk_bitmap_emit", ptr(zero), None, 1, nbits, ptr(ws), ptr(out), nbits, None)
        sync()
        assert total.array[0] == nbits
        assert np.array_equal(to_np(out, np.uint32)[:nbits], np.arange(nbits, dtype=np.uint32))
    finally:
        sync()
        total.free()


def test_bitmap_update_sets_and_clears_listed_bits():
    rng = np.random.default_rng(5)
    nbits = 123_457
    w, b = _bits(rng, nbits, 0.4)
    d = to_dev(w)
    st = dev_zeros_u32(1)
    on = rng.choice(nbits, 5000, replace=False).astype(np.uint32)
    off = rng.choice(nbits, 7000, replace=False).astype(np.uint32)
    d_on, d_off = to_dev(on), to_dev(off)
    hip.call("ugk_bitmap_update", ptr(d), nbits, ptr(d_on), len(on), 1, ptr(st), None)
    hip.call("ugk_bitmap_update", ptr(d), nbits, ptr(d_off), len(off), 0, ptr(st), None)
    assert status_value(st) == 0
    b[on] = True
    b[off] = False
    got = np.unpackbits(to_np(d, np.uint8)[: len(w) * 8], bitorder="little").astype(bool)
    assert np.array_equal(got, b)
    bad = to_dev(np.array([3, nbits], np.uint32))
    hip.call("ugk_bitmap_update", ptr(d), nbits, ptr(bad), 2, 1, ptr(st), None)
    assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE


def test_rows_to_keys_is_the_forward_id_map():
    rng = np.random.default_rng(9)
    bits, mul = 40, 0x9E3779B97F4A7C15 | 1
    rows = rng.integers(0, 1 << 31, size=10_001).astype(np.uint32)
    d_rows = to_dev(rows)
    out = dev_bytes(len(rows) * 8)
    hip.call("ugk_rows_to_keys", ptr(d_rows), len(rows), mul, (1 << bits) - 1, ptr(out), None)
    sync()
    want = np.array([(int(r) * mul) & ((1 << bits) - 1) for r in rows], np.int64)
    assert np.array_equal(to_np(out, np.int64)[: len(rows)], want)


@pytest.mark.parametrize("nbits", [1, 63, 64, 65, 1000, 100_003])
def test_bitmap_set_through_fills_the_low_bits(nbits):
    """ugk_bitmap_set_through: every bit up to and including the position read from the device is set, bits above it
    are left as they were; a position outside the bitmap is refused and changes nothing"""
    rng = np.random.default_rng(nbits)
    words = (nbits + 63) // 64
    st = dev_zeros_u32(1)
    for last in sorted({0, nbits // 2, nbits - 1}):
        bits = rng.integers(0, 2, size=words * 64).astype(bool)
        bm = to_dev(np.packbits(bits, bitorder="little").view(np.uint64))
        pos = to_dev(np.array([7, last, 9], np.uint32))
        hip.call("ugk_bitmap_set_through", ptr(bm), nbits, ptr(pos) + 4, ptr(st), None)
        assert status_value(st) == 0
        want = bits.copy()
        want[: last + 1] = True
        got = np.unpackbits(to_np(bm, np.uint64)[:words].view(np.uint8), bitorder="little").astype(bool)
        assert np.array_equal(got, want), (nbits, last)
    bm = to_dev(np.zeros(words, np.uint64))
    pos = to_dev(np.array([nbits], np.uint32))
    hip.call("ugk_bitmap_set_through", ptr(bm), nbits, ptr(pos), ptr(st), None)
    assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE
    assert not to_np(bm, np.uint64)[:words].any()


@pytest.mark.parametrize("kind", ["flat", "hash"])
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
def test_evict_that_releases_the_slots(kind, kdtype):
    """ugk_table_evict_release_*: the keys leave the table exactly as with ugk_table_evict_*, and the bit of the slot
    each of them held is cleared in the slot bitmap; the bits of the keys that stay are untouched; an absent key is
    flagged and releases nothing"""
    rng = np.random.default_rng(5)
    nkeys, n, nslots = 50_000, 20_000, 30_000
    keys = rng.choice(nkeys, n, replace=False).astype(kdtype)
    slots = rng.choice(nslots, n, replace=False).astype(np.uint32)
    if kind == "flat":
        mem = dev_zeros_u32(nkeys)
        hip.call("ugk_fill_u32", ptr(mem), hip.EMPTY_U32, nkeys, None)
        tb = hip.table(hip.TABLE_FLAT, ptr(mem), nkeys)
    else:
        nb = hip.lib().ugk_hash_buckets_for(n, 0.7)
        mem = dev_bytes(nb * 16 + 128)
        base = (ptr(mem) + 127) // 128 * 128
        hip.call("ugk_hash_init", base, nb, None)
        tb = hip.table(hip.TABLE_HASH, base, nb)
    st = dev_zeros_u32(1)
    ins = "ugk_table_insert_i64" if kdtype == np.int64 else "ugk_table_insert_u32"
    d_keys, d_slots = to_dev(keys), to_dev(slots)
    hip.call(ins, tb, ptr(d_keys), ptr(d_slots), 0, 0, n, ptr(st), None)
    assert status_value(st) == 0
    used = np.zeros((nslots + 63) // 64 * 64, bool)
    used[slots] = True
    used[rng.choice(np.flatnonzero(~used[:nslots]), 500, replace=False)] = True  # slots of nobody in particular
    bm = to_dev(np.packbits(used, bitorder="little").view(np.uint64))
    gone = rng.choice(n, n // 3, replace=False)
    d_gone = to_dev(keys[gone])
    fn = "ugk_table_evict_release_i64" if kdtype == np.int64 else "ugk_table_evict_release_u32"
    hip.call(fn, tb, ptr(d_gone), len(gone), ptr(bm), nslots, ptr(st), None)
    assert status_value(st) == 0
    want = used.copy()
    want[slots[gone]] = False
    got = np.unpackbits(to_np(bm, np.uint64)[: len(used) // 64].view(np.uint8), bitorder="little").astype(bool)
    assert np.array_equal(got, want)
    loc, off = dev_zeros_u32(n), dev_zeros_u32(n)
    lk = "ugk_table_lookup_i64" if kdtype == np.int64 else "ugk_table_lookup_u32"
    hip.call(lk, tb, ptr(d_keys), n, 9, ptr(loc), ptr(off), None)
    stays = np.ones(n, bool)
    stays[gone] = False
    got_loc, got_off = to_np(loc, np.uint32)[:n], to_np(off, np.uint32)[:n]
    assert (got_loc[stays] == 0).all() and np.array_equal(got_off[stays], slots[stays]) and (got_loc[~stays] == 9).all()
    # evicting them again: absent, and no bit moves
    hip.call(fn, tb, ptr(d_gone), len(gone), ptr(bm), nslots, ptr(st), None)
    assert status_value(st) & hip.ST_EVICT_ABSENT
    got = np.unpackbits(to_np(bm, np.uint64)[: len(used) // 64].view(np.uint8), bitorder="little").astype(bool)
    assert np.array_equal(got, want)
