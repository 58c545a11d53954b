"""GPU parity tests of the HIP kernels, called through the C-ABI of libugache_hip.so and checked bit-for-bit
against the CPU oracle (and against closed forms at full size)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle_lib import IDX_DTYPE, Oracle  # noqa: E402
from ugache_amd import hip  # noqa: E402

if torch.cuda.is_available():
    from gpu_util import (PinnedArray, dev_bytes, dev_zeros_u32, pinned_from, ptr, status_value, sync, to_dev,
                          to_np)

ORC = Oracle()


def _rand_table(rng, rows, row_bytes):
    return rng.integers(0, 256, size=(rows, row_bytes), dtype=np.uint8)


def _gather_direct(table_np, keys_np, max_blocks=0):
    rows, rb = table_np.shape
    tbl = to_dev(table_np)
    keys = to_dev(keys_np)
    out = dev_bytes(len(keys_np) * rb, fill=0xEE)
    st = dev_zeros_u32(1)
    fn = "ugk_gather_direct_i64" if keys_np.dtype == np.int64 else "ugk_gather_direct_u32"
    hip.call(fn, ptr(tbl), rows, ptr(keys), len(keys_np), ptr(out), rb, max_blocks, ptr(st), None, None)
    return to_np(out)[: len(keys_np) * rb].reshape(len(keys_np), rb), status_value(st)


# ------------------------------------------------------------------------------------------------------
# direct gather (IsDirectMapping fast path)
# ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("row_bytes", [512, 128, 16, 32, 400, 2048, 4096 + 16, 8, 24, 4, 12, 2, 6, 1, 3])
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
def test_gather_direct_matches_oracle(row_bytes, kdtype):
    rng = np.random.default_rng(row_bytes)
    rows = 3001
    table = _rand_table(rng, rows, row_bytes)
    for n in (1, 63, 4099):
        keys = rng.integers(0, rows, size=n).astype(kdtype)
        got, st = _gather_direct(table, keys)
        assert st == 0
        assert got.tobytes() == ORC.gather(table, keys).tobytes(), (row_bytes, n)


def test_gather_direct_empty_and_capped_grid():
    rng = np.random.default_rng(1)
    table = _rand_table(rng, 100, 512)
    got, st = _gather_direct(table, np.zeros(0, np.uint32))
    assert got.shape == (0, 512) and st == 0
    keys = rng.integers(0, 100, size=20000).astype(np.uint32)
    for cap in (1, 3, 16):
        got, st = _gather_direct(table, keys, max_blocks=cap)
        assert st == 0 and got.tobytes() == table[keys].tobytes()


def test_gather_out_of_range_key_sets_status_and_skips_row():
    rng = np.random.default_rng(2)
    table = _rand_table(rng, 50, 128)
    keys = np.array([1, 50, 2, 0xFFFFFFFF, 49], np.uint32)
    got, st = _gather_direct(table, keys)
    assert st & hip.ST_KEY_OUT_OF_RANGE
    assert (got[[1, 3]] == 0xEE).all()
    assert got[[0, 2, 4]].tobytes() == table[[1, 2, 49]].tobytes()
    keys64 = np.array([3, -1, 1 << 40], np.int64)
    got, st = _gather_direct(table, keys64)
    assert st & hip.ST_KEY_OUT_OF_RANGE and got[0].tobytes() == table[3].tobytes() and (got[1:] == 0xEE).all()


@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
def test_gather_scatter(kdtype):
    rng = np.random.default_rng(3)
    table = _rand_table(rng, 500, 512)
    n = 300
    keys = rng.integers(0, 500, size=n).astype(kdtype)
    dst = rng.permutation(400)[:n].astype(np.uint32)
    out = dev_bytes(400 * 512, fill=0)
    st = dev_zeros_u32(1)
    fn = "ugk_gather_scatter_i64" if kdtype == np.int64 else "ugk_gather_scatter_u32"
    d_table, d_keys, d_dst = to_dev(table), to_dev(keys), to_dev(dst)
    hip.call(fn, ptr(d_table), 500, ptr(d_keys), ptr(d_dst), n, ptr(out), 400, 512, 0, ptr(st), None, None)
    want = np.zeros((400, 512), np.uint8)
    want[dst] = table[keys.astype(np.int64)]
    assert status_value(st) == 0 and to_np(out).reshape(400, 512).tobytes() == want.tobytes()
    # destination beyond the output is refused
    bad = dst.copy()
    bad[0] = 400
    d_bad = to_dev(bad)
    hip.call(fn, ptr(d_table), 500, ptr(d_keys), ptr(d_bad), n, ptr(out), 400, 512, 0, ptr(st), None, None)
    assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE


def test_gather_from_pinned_host_memory():
    rng = np.random.default_rng(4)
    table = _rand_table(rng, 2000, 512)
    pin = pinned_from(table)
    try:
        keys = rng.integers(0, 2000, size=5000).astype(np.uint32)
        out = dev_bytes(5000 * 512)
        st = dev_zeros_u32(1)
        d_keys = to_dev(keys)
        hip.call("ugk_gather_direct_u32", pin.ptr, 2000, ptr(d_keys), 5000, ptr(out), 512, 8, ptr(st), None, None)
        assert status_value(st) == 0
        assert to_np(out).reshape(5000, 512).tobytes() == table[keys].tobytes()
        kind = C.c_int(-1)
        hip.call("ugk_pointer_kind", pin.ptr, C.byref(kind))
        assert kind.value == 1
        hip.call("ugk_pointer_kind", ptr(out), C.byref(kind))
        assert kind.value == 2
        plain = np.zeros(64, np.uint8)
        hip.call("ugk_pointer_kind", plain.ctypes.data, C.byref(kind))
        assert kind.value == 0
    finally:
        sync()
        pin.free()


@pytest.mark.parametrize("spin_us", [0, 1, 1_000_000])
def test_wait_on_a_ticket_behind_the_launch(spin_us):
    """ugk_stream_sync_ticket: the ticket kernel runs behind what was enqueued, so once the call returns - having seen
    the ticket, or having fallen back to waiting for the stream when the poll budget ran out first - the gather in
    front of it is complete and the word holds the ticket"""
    rng = np.random.default_rng(7)
    table = _rand_table(rng, 20_000, 512)
    keys = rng.integers(0, 20_000, size=300_000).astype(np.uint32)
    d_table, d_keys = to_dev(table), to_dev(keys)
    out = dev_bytes(len(keys) * 512, fill=0)
    st = dev_zeros_u32(1)
    word = PinnedArray((16,), np.uint32)
    try:
        word.array[...] = 0
        stream = C.c_void_p()
        hip.call("ugk_stream_create", C.byref(stream))
        sync()
        for ticket in (1, 2, 0xFFFFFFFF):
            out.zero_()
            sync()
            hip.call("ugk_gather_direct_u32", ptr(d_table), 20_000, ptr(d_keys), len(keys), ptr(out), 512, 4, ptr(st), None,
                     stream)  # 4 workgroups: a launch of a few hundred microseconds
            hip.call("ugk_stream_sync_ticket", stream, word.ptr, ticket, spin_us)
            assert int(word.array[0]) == ticket
            got = out.cpu().numpy()  # a copy on another stream: complete only if the gather was
            assert got.tobytes() == table[keys].tobytes()
        hip.call("ugk_stream_destroy", stream)
    finally:
        sync()
        word.free()


def test_preload_launches_an_empty_kernel_of_every_source_file():
    """ugk_preload_kernels: returns once its empty launches have run; any number of times, beside other work"""
    d = to_dev(np.arange(1000, dtype=np.uint32))
    for _ in range(3):
        hip.call("ugk_preload_kernels")
    sync()
    assert np.array_equal(to_np(d, np.uint32)[:1000], np.arange(1000, dtype=np.uint32))


@pytest.mark.parametrize("spin_us", [0, 1, 1_000_000])
def test_words_brought_to_the_host_with_the_ticket(spin_us):
    """ugk_words_to_host_ticket: device words written by a launch in front of it arrive with the ticket, whichever way
    the wait ends; either source may be absent"""
    rng = np.random.default_rng(11)
    table = _rand_table(rng, 20_000, 512)
    keys = rng.integers(0, 20_000, size=300_000).astype(np.uint32)
    d_table, d_keys = to_dev(table), to_dev(keys)
    out = dev_bytes(len(keys) * 512, fill=0)
    st = dev_zeros_u32(1)
    extra = to_dev(np.arange(100, 130, dtype=np.uint32))
    dst = PinnedArray((64,), np.uint32)
    try:
        dst.array[...] = 0
        stream = C.c_void_p()
        hip.call("ugk_stream_create", C.byref(stream))
        sync()
        bad = keys.copy()
        bad[12345] = 20_000  # a key outside the table: the gather flags it in its status word
        d_bad = to_dev(bad)
        for ticket, (k_dev, n_b) in zip((1, 2, 0xFFFFFFFF), ((d_keys, 30), (d_bad, 7), (d_keys, 0))):
            st.zero_()
            sync()
            hip.call("ugk_gather_direct_u32", ptr(d_table), 20_000, ptr(k_dev), len(keys), ptr(out), 512, 4, ptr(st), None,
                     stream)  # 4 workgroups: a launch of a few hundred microseconds
            hip.call("ugk_words_to_host_ticket", ptr(st), 1, ptr(extra) if n_b else None, n_b, dst.ptr, ticket, spin_us,
                     stream)
            assert int(dst.array[0]) == ticket
            assert int(dst.array[1]) == (hip.ST_KEY_OUT_OF_RANGE if k_dev is d_bad else 0)
            assert dst.array[2: 2 + n_b].tolist() == list(range(100, 100 + n_b))
        hip.call("ugk_words_to_host_ticket", None, 0, ptr(extra), 3, dst.ptr, 77, spin_us, stream)
        assert dst.array[:4].tolist() == [77, 100, 101, 102]
        with pytest.raises(hip.UgkError):
            hip.call("ugk_words_to_host_ticket", ptr(st), 34, ptr(extra), 30, dst.ptr, 78, spin_us, stream)
        hip.call("ugk_stream_destroy", stream)
    finally:
        sync()
        dst.free()


def test_gather_full_size_all_hit_closed_form():
    """10M x 128 fp32 table resident in HBM, 262144 uniform uint32 keys (the all-hit configuration).
    table[r, c] is a closed form of (r, c), so out[i, c] can be checked without a host copy of the table."""
    rows, dim, n = 10_000_000, 128, 262_144
    r = torch.arange(rows, device="cuda", dtype=torch.int32).unsqueeze(1)
    c = torch.arange(dim, device="cuda", dtype=torch.int32).unsqueeze(0)
    table = (r * 131 + c * 7919) ^ (r >> 3)  # int32 bit pattern, 4 bytes per element like fp32
    del r
    g = torch.Generator(device="cuda").manual_seed(4)
    keys = torch.randint(0, rows, (n,), generator=g, device="cuda", dtype=torch.int32)
    out = torch.empty((n, dim), dtype=torch.int32, device="cuda")
    st = dev_zeros_u32(1)
    hip.call("ugk_gather_direct_u32", table.data_ptr(), rows, keys.data_ptr(), n, out.data_ptr(), dim * 4, 0, ptr(st),
             None, None)
    assert status_value(st) == 0
    k = keys.unsqueeze(1)
    want = (k * 131 + c * 7919) ^ (k >> 3)
    assert torch.equal(out, want)
    # and a sample of rows against the oracle on the host
    sample = keys[:4096].cpu().numpy().astype(np.uint32)
    sub = table[keys[:4096].long()].cpu().numpy()
    assert ORC.gather(sub, np.arange(4096, dtype=np.uint32)).tobytes() == out[:4096].cpu().numpy().tobytes()
    assert sample.max() < rows


# ------------------------------------------------------------------------------------------------------
# lookup tables
# ------------------------------------------------------------------------------------------------------
def _make_flat(nkeys):
    t = dev_zeros_u32(nkeys)
    hip.call("ugk_fill_u32", ptr(t), hip.EMPTY_U32, nkeys, None)
    return t, hip.table(hip.TABLE_FLAT, ptr(t), nkeys)


def _make_hash(n_entries, load=0.7):
    nb = hip.lib().ugk_hash_buckets_for(n_entries, load)
    t = dev_bytes(nb * 16 + 128)
    base = (ptr(t) + 127) // 128 * 128
    hip.call("ugk_hash_init", base, nb, None)
    return t, hip.table(hip.TABLE_HASH, base, nb), nb


def _make_hash32(n_entries, load=0.7, fb_mul=0, fb_mask=0):
    """the compact hash table (kind 3): 8-byte entries, sixteen to a 128-byte line, keyed by the row a key stands for"""
    ne = hip.lib().ugk_hash32_entries_for(n_entries, load)
    assert ne % 16 == 0
    t = dev_bytes(ne * 8 + 128)
    base = (ptr(t) + 127) // 128 * 128
    tb = hip.table(hip.TABLE_HASH32, base, ne, fb_mul, fb_mask)
    hip.call("ugk_table_init", tb, None)
    return t, tb, ne


def _lookup(tb, keys_np, fallback=1):
    n = len(keys_np)
    loc = dev_zeros_u32(n)
    off = dev_zeros_u32(n)
    fn = "ugk_table_lookup_i64" if keys_np.dtype == np.int64 else "ugk_table_lookup_u32"
    d_keys = to_dev(keys_np)
    hip.call(fn, tb, ptr(d_keys), n, fallback, ptr(loc), ptr(off), None)
    sync()
    return to_np(loc, np.uint32)[:n], to_np(off, np.uint32)[:n]


def _insert(tb, keys_np, offs_np=None, seq_base=0, loc=0):
    st = dev_zeros_u32(1)
    fn = "ugk_table_insert_i64" if keys_np.dtype == np.int64 else "ugk_table_insert_u32"
    offs = None if offs_np is None else to_dev(offs_np)
    d_keys = to_dev(keys_np)
    hip.call(fn, tb, ptr(d_keys), ptr(offs), seq_base, loc, len(keys_np), ptr(st), None)
    return status_value(st)


def _evict(tb, keys_np):
    st = dev_zeros_u32(1)
    fn = "ugk_table_evict_i64" if keys_np.dtype == np.int64 else "ugk_table_evict_u32"
    d_keys = to_dev(keys_np)
    hip.call(fn, tb, ptr(d_keys), len(keys_np), ptr(st), None)
    return status_value(st)


def test_flat_table_matches_oracle_rule():
    rng = np.random.default_rng(5)
    nkeys = 200_000
    cached = rng.choice(nkeys, 50_000, replace=False).astype(np.uint32)
    mem, tb = _make_flat(nkeys)
    assert _insert(tb, cached) == 0  # sequential slots, location 0 (InsertSeqOffWithLoc)
    oflat = ORC.flat_table(nkeys)
    ORC.lib.orc_flat_insert(oflat, cached, np.arange(len(cached), dtype=np.uint32), len(cached))
    q = rng.integers(0, nkeys, size=100_003).astype(np.uint32)
    loc, off = _lookup(tb, q)
    want = ORC.lookup_src_dst(q, flat=oflat, fallback_loc=1)
    assert np.array_equal(loc, want["src"] >> 28) and np.array_equal(off, want["src"] & 0x0FFFFFFF)
    assert np.array_equal(to_np(mem, np.uint32)[:nkeys], oflat)
    # evict
    ev = cached[:10_000]
    assert _evict(tb, ev) == 0
    ORC.lib.orc_flat_evict(oflat, ev, len(ev))
    assert np.array_equal(to_np(mem, np.uint32)[:nkeys], oflat)
    assert _evict(tb, ev[:5]) & hip.ST_EVICT_ABSENT
    assert _insert(tb, cached[10_000:10_001]) & hip.ST_DUP_KEY
    assert _insert(tb, np.array([nkeys], np.uint32)) & hip.ST_KEY_OUT_OF_RANGE


# uint32 keys stay below 2^28: the reference packs a missed key into the 28-bit offset field
@pytest.mark.parametrize("kdtype,space", [(np.uint32, 1 << 28), (np.int64, 1 << 40)])
@pytest.mark.parametrize("n", [10, 1000, 200_000])
def test_hash_table_against_dict_and_oracle_table(kdtype, space, n):
    rng = np.random.default_rng(n)
    keys = np.unique(rng.integers(0, space, size=n * 2))[:n]
    rng.shuffle(keys)
    keys = keys.astype(kdtype)
    n = len(keys)
    offs = rng.integers(0, 1 << 28, size=n).astype(np.uint32)
    mem, tb, nb = _make_hash(n)
    assert _insert(tb, keys, offs, loc=0) == 0
    absent = np.setdiff1d(rng.integers(0, space, size=n).astype(kdtype), keys)
    q = np.concatenate([keys, absent, keys[::-1][: n // 2]])
    loc, off = _lookup(tb, q)
    model = dict(zip(keys.tolist(), offs.tolist()))
    want_loc = np.array([0 if int(k) in model else 1 for k in q], np.uint32)
    want_off = np.array([model.get(int(k), int(k) & 0xFFFFFFFF) for k in q], np.uint32)
    assert np.array_equal(loc, want_loc) and np.array_equal(off, want_off)
    if kdtype == np.uint32:
        # same answers as the reference's simple table restated in the oracle
        ot = ORC.simple_table(n)
        ORC.simple_insert(ot, keys, offs)  # loc 0 => packed value == off
        want = ORC.lookup_src_dst(q.astype(np.uint32), simple=ot, fallback_loc=1)
        assert np.array_equal(loc, want["src"] >> 28) and np.array_equal(off, want["src"] & 0x0FFFFFFF)
    # census: occupied / tombstones / never used
    cen = torch.zeros(3, dtype=torch.int64, device="cuda")
    hip.call("ugk_hash_census", tb.table, nb, cen.data_ptr(), None)
    sync()
    assert cen.cpu().tolist() == [n, 0, nb - n]
    # evict half: they miss, the rest still hit; tombstones appear
    ev = keys[: n // 2]
    assert _evict(tb, ev) == 0
    loc, off = _lookup(tb, keys)
    assert (loc[: n // 2] == 1).all() and (loc[n // 2:] == 0).all()
    assert np.array_equal(off[n // 2:], offs[n // 2:])
    hip.call("ugk_hash_census", tb.table, nb, cen.data_ptr(), None)
    sync()
    assert cen.cpu().tolist() == [n - n // 2, n // 2, nb - n]
    assert _evict(tb, ev[:1]) & hip.ST_EVICT_ABSENT
    # re-insert with new offsets
    new_offs = (offs[: n // 2] ^ 0x5555).astype(np.uint32)
    assert _insert(tb, ev, new_offs) == 0
    loc, off = _lookup(tb, keys)
    assert (loc == 0).all() and np.array_equal(off[: n // 2], new_offs)
    assert _insert(tb, keys[:1], offs[:1]) & hip.ST_DUP_KEY
    hip.call("ugk_hash_census", tb.table, nb, cen.data_ptr(), None)
    sync()
    occ, tomb, empty = cen.cpu().tolist()
    assert occ == n and occ + tomb + empty == nb


@pytest.mark.parametrize("load", [0.5, 0.7, 0.9])
def test_hash_table_under_churn_follows_a_dict(load):
    """refresh-like churn: rounds of evicting a tenth of the keys and inserting as many new ones, tombstones piling
    up in between; after every round each present key returns its latest value, every evicted or never-inserted key
    misses, and occupied + tombstoned + never used == buckets"""
    rng = np.random.default_rng(int(load * 10))
    n = 40_000
    mem, tb, nb = _make_hash(n, load=load)
    model = {}
    keys = np.unique(rng.integers(0, 1 << 40, size=2 * n))[:n].astype(np.int64)
    offs = rng.integers(0, 1 << 31, size=n).astype(np.uint32)
    assert _insert(tb, keys, offs) == 0
    model.update(zip(keys.tolist(), offs.tolist()))
    gone = set()
    cen = torch.zeros(3, dtype=torch.int64, device="cuda")
    for rnd in range(12):
        present = np.fromiter(model.keys(), np.int64, len(model))
        ev = rng.choice(present, n // 10, replace=False)
        assert _evict(tb, ev) == 0
        for k in ev.tolist():
            del model[k]
            gone.add(k)
        fresh = np.setdiff1d(np.unique(rng.integers(0, 1 << 40, size=n // 5)).astype(np.int64), present)[: n // 10]
        back = np.array(list(gone)[: n // 50], np.int64)  # some evicted keys come back
        ins = np.unique(np.concatenate([back, fresh]))
        ins = rng.permutation(ins)[: n // 10]  # as many in as out: the table keeps its load
        ins_off = rng.integers(0, 1 << 31, size=len(ins)).astype(np.uint32)
        st = _insert(tb, ins, ins_off)
        assert st == 0, (rnd, st)
        for k, o in zip(ins.tolist(), ins_off.tolist()):
            model[k] = o
            gone.discard(k)
        present = np.fromiter(model.keys(), np.int64, len(model))
        absent = np.array(list(gone)[:5000] + rng.integers(1 << 41, 1 << 42, size=1000).tolist(), np.int64)
        loc, off = _lookup(tb, np.concatenate([present, absent]), fallback=1)
        assert (loc[: len(present)] == 0).all() and (loc[len(present):] == 1).all(), rnd
        assert np.array_equal(off[: len(present)], np.array([model[k] for k in present.tolist()], np.uint32)), rnd
        hip.call("ugk_hash_census", tb.table, nb, cen.data_ptr(), None)
        sync()
        occ, tomb, empty = cen.cpu().tolist()
        assert occ == len(model) and occ + tomb + empty == nb, rnd


def test_hash_table_dense_collisions_and_host_entries():
    """Load factor 0.9 with sequential keys forces long probe runs; host-located entries carry explicit rows."""
    n = 50_000
    keys = (np.arange(n, dtype=np.int64) * 7 + 3)
    mem, tb, nb = _make_hash(n, load=0.9)
    locs_half = n // 2
    assert _insert(tb, keys[:locs_half], seq_base=100, loc=hip.LOC_LOCAL) == 0
    assert _insert(tb, keys[locs_half:], seq_base=0, loc=hip.LOC_HOST) == 0
    loc, off = _lookup(tb, keys, fallback=9)
    assert (loc[:locs_half] == 0).all() and (loc[locs_half:] == 1).all()
    assert np.array_equal(off[:locs_half], 100 + np.arange(locs_half, dtype=np.uint32))
    assert np.array_equal(off[locs_half:], np.arange(n - locs_half, dtype=np.uint32))
    loc, off = _lookup(tb, keys + 1, fallback=9)
    assert (loc == 9).all()
    # table full
    mem2, tb2, nb2 = _make_hash(10, load=0.9)
    many = np.arange(nb2 + 5, dtype=np.int64)
    assert _insert(tb2, many) & hip.ST_TABLE_FULL
    loc, off = _lookup(tb2, np.array([10_000_000], np.int64), fallback=1)  # full lap without a free bucket ends
    assert loc[0] == 1


# ---- the compact hash table (kind 3): keyed by the row a key stands for --------------------------------------------
def _census(tb):
    cen = torch.zeros(3, dtype=torch.int64, device="cuda")
    hip.call("ugk_table_census", tb, cen.data_ptr(), None)
    sync()
    return cen.cpu().tolist()


def _sparse_map(bits=40):
    """an odd multiplier and its inverse modulo 2^bits: ids = (rows * mul) & mask, rows = (ids * inv) & mask"""
    mask = (1 << bits) - 1
    mul = (0x9E3779B97F4A7C15 | 1) & mask
    return mul, pow(mul, -1, 1 << bits), mask


@pytest.mark.parametrize("keys_are", ["u32", "i64_rows", "i64_sparse_ids"])
@pytest.mark.parametrize("n", [10, 1000, 200_000])
def test_compact_hash_table_against_dict_and_oracle_table(keys_are, n):
    rng = np.random.default_rng(n + len(keys_are))
    kdtype = np.uint32 if keys_are == "u32" else np.int64
    row_space = 1 << 28 if keys_are == "u32" else 0xFFFFFFFE  # rows the table can hold: all below the tombstone mark
    rows = np.unique(np.concatenate([rng.integers(0, row_space, size=n * 2), [row_space - 1, 0]]))
    rng.shuffle(rows)
    rows = rows[:n].astype(np.uint64)
    n = len(rows)
    fb_mul = inv = fb_mask = 0
    if keys_are == "i64_sparse_ids":
        mul, inv, fb_mask = _sparse_map()
        fb_mul = inv  # the table turns an id back into its row
        keys = ((rows * np.uint64(mul)) & np.uint64(fb_mask)).astype(np.int64)
    else:
        keys = rows.astype(kdtype)
    offs = rng.integers(0, 1 << 28, size=n).astype(np.uint32)
    mem, tb, ne = _make_hash32(n, fb_mul=fb_mul, fb_mask=fb_mask)
    assert _census(tb) == [0, 0, ne]
    assert _insert(tb, keys, offs, loc=0) == 0
    absent_rows = np.setdiff1d(rng.integers(0, row_space, size=n).astype(np.uint64), rows)
    absent = (((absent_rows * np.uint64(mul)) & np.uint64(fb_mask)).astype(np.int64)
              if keys_are == "i64_sparse_ids" else absent_rows.astype(kdtype))
    q = np.concatenate([keys, absent, keys[::-1][: n // 2]])
    q_rows = np.concatenate([rows, absent_rows, rows[::-1][: n // 2]])
    loc, off = _lookup(tb, q)
    model = dict(zip(keys.tolist(), offs.tolist()))
    want_loc = np.array([0 if int(k) in model else 1 for k in q], np.uint32)
    want_off = np.array([model.get(int(k), int(r) & 0xFFFFFFFF) for k, r in zip(q, q_rows)], np.uint32)
    assert np.array_equal(loc, want_loc) and np.array_equal(off, want_off)
    if keys_are == "u32":
        ot = ORC.simple_table(n)
        ORC.simple_insert(ot, keys, offs)
        want = ORC.lookup_src_dst(q.astype(np.uint32), simple=ot, fallback_loc=1)
        assert np.array_equal(loc, want["src"] >> 28) and np.array_equal(off, want["src"] & 0x0FFFFFFF)
    assert _census(tb) == [n, 0, ne - n]
    ev = keys[: n // 2]
    assert _evict(tb, ev) == 0
    loc, off = _lookup(tb, keys)
    assert (loc[: n // 2] == 1).all() and (loc[n // 2:] == 0).all()
    assert np.array_equal(off[n // 2:], offs[n // 2:])
    assert _census(tb) == [n - n // 2, n // 2, ne - n]
    assert _evict(tb, ev[:1]) & hip.ST_EVICT_ABSENT
    new_offs = (offs[: n // 2] ^ 0x5555).astype(np.uint32)
    assert _insert(tb, ev, new_offs) == 0
    loc, off = _lookup(tb, keys)
    assert (loc == 0).all() and np.array_equal(off[: n // 2], new_offs)
    assert _insert(tb, keys[:1], offs[:1]) & hip.ST_DUP_KEY
    occ, tomb, empty = _census(tb)
    assert occ == n and occ + tomb + empty == ne


def test_compact_hash_table_refuses_what_its_entries_cannot_hold():
    """a row at or above the tombstone mark, an id beyond the id space of the key map, an offset wider than 28 bits:
    refused on insert with KEY_OUT_OF_RANGE, a miss on lookup, absent on evict"""
    mem, tb, ne = _make_hash32(100)
    for bad in (0xFFFFFFFE, 0xFFFFFFFF, 1 << 32, (1 << 40) + 5):
        assert _insert(tb, np.array([bad], np.int64)) & hip.ST_KEY_OUT_OF_RANGE
        loc, off = _lookup(tb, np.array([bad], np.int64), fallback=7)
        assert loc[0] == 7 and off[0] == bad & 0xFFFFFFFF
        assert _evict(tb, np.array([bad], np.int64)) & hip.ST_EVICT_ABSENT
    assert _insert(tb, np.array([5], np.int64), np.array([1 << 28], np.uint32)) & hip.ST_KEY_OUT_OF_RANGE
    assert _census(tb) == [0, 0, ne]
    assert _insert(tb, np.array([0xFFFFFFFD, 5], np.int64), np.array([(1 << 28) - 1, 0], np.uint32), loc=3) == 0
    loc, off = _lookup(tb, np.array([0xFFFFFFFD, 5, 6], np.int64), fallback=7)
    assert loc.tolist() == [3, 3, 7] and off.tolist() == [(1 << 28) - 1, 0, 6]
    mul, inv, mask = _sparse_map(20)
    mem2, tb2, _ = _make_hash32(100, fb_mul=inv, fb_mask=mask)
    assert _insert(tb2, np.array([mask + 1], np.int64)) & hip.ST_KEY_OUT_OF_RANGE  # no row stands behind this id
    loc, off = _lookup(tb2, np.array([mask + 1], np.int64), fallback=7)
    assert loc[0] == 7


@pytest.mark.parametrize("load", [0.5, 0.7, 0.9])
def test_compact_hash_table_under_churn_follows_a_dict(load):
    """as test_hash_table_under_churn_follows_a_dict, on 8-byte entries: tombstones pile up between rounds, every
    present key returns its latest value, every evicted or never-inserted key misses"""
    rng = np.random.default_rng(int(load * 10) + 100)
    n = 40_000
    space = 0xFFFFFFFE
    mem, tb, ne = _make_hash32(n, load=load)
    model = {}
    keys = np.unique(rng.integers(0, space, size=2 * n))[:n].astype(np.int64)
    keys = rng.permutation(keys)
    offs = rng.integers(0, 1 << 28, size=n).astype(np.uint32)
    assert _insert(tb, keys, offs) == 0
    model.update(zip(keys.tolist(), offs.tolist()))
    gone = set()
    for rnd in range(12):
        present = np.fromiter(model.keys(), np.int64, len(model))
        ev = rng.choice(present, n // 10, replace=False)
        assert _evict(tb, ev) == 0
        for k in ev.tolist():
            del model[k]
            gone.add(k)
        fresh = np.setdiff1d(np.unique(rng.integers(0, space, size=n // 5)).astype(np.int64), present)[: n // 10]
        back = np.array(list(gone)[: n // 50], np.int64)
        ins = np.unique(np.concatenate([back, fresh]))
        ins = rng.permutation(ins)[: n // 10]
        ins_off = rng.integers(0, 1 << 28, size=len(ins)).astype(np.uint32)
        st = _insert(tb, ins, ins_off, loc=rnd % 16)
        assert st == 0, (rnd, st)
        for k, o in zip(ins.tolist(), ins_off.tolist()):
            model[k] = o | ((rnd % 16) << 28)
            gone.discard(k)
        present = np.fromiter(model.keys(), np.int64, len(model))
        absent = np.array(list(gone)[:5000] + rng.integers(1 << 33, 1 << 42, size=1000).tolist(), np.int64)
        loc, off = _lookup(tb, np.concatenate([present, absent]), fallback=99)
        want = np.array([model[k] for k in present.tolist()], np.uint32)
        assert (loc[len(present):] == 99).all(), rnd
        assert np.array_equal(loc[: len(present)], want >> 28) and np.array_equal(off[: len(present)], want & 0x0FFFFFFF), rnd
        occ, tomb, empty = _census(tb)
        assert occ == len(model) and occ + tomb + empty == ne, rnd


def test_compact_hash_table_dense_collisions_full_table_and_no_never_used_entry():
    n = 50_000
    keys = (np.arange(n, dtype=np.int64) * 7 + 3)
    mem, tb, ne = _make_hash32(n, load=0.9)
    half = n // 2
    assert _insert(tb, keys[:half], seq_base=100, loc=hip.LOC_LOCAL) == 0
    assert _insert(tb, keys[half:], seq_base=0, loc=hip.LOC_HOST) == 0
    loc, off = _lookup(tb, keys, fallback=9)
    assert (loc[:half] == 0).all() and (loc[half:] == 1).all()
    assert np.array_equal(off[:half], 100 + np.arange(half, dtype=np.uint32))
    assert np.array_equal(off[half:], np.arange(n - half, dtype=np.uint32))
    loc, off = _lookup(tb, keys + 1, fallback=9)
    assert (loc == 9).all()
    # every entry taken: one more key does not fit, and a lookup of an absent key ends after one lap
    mem2, tb2, ne2 = _make_hash32(10, load=0.9)
    assert _insert(tb2, np.arange(ne2, dtype=np.int64)) == 0
    assert _census(tb2) == [ne2, 0, 0]
    assert _insert(tb2, np.array([ne2 + 5], np.int64)) & hip.ST_TABLE_FULL
    loc, off = _lookup(tb2, np.array([10_000_000, 3], np.int64), fallback=1)
    assert loc.tolist() == [1, 0] and off[1] == 3
    # evicted entries are reused although no never-used entry is left
    assert _evict(tb2, np.array([3, 17], np.int64)) == 0
    assert _insert(tb2, np.array([1000, 1001], np.int64), np.array([7, 8], np.uint32)) == 0
    assert _census(tb2) == [ne2, 0, 0]
    loc, off = _lookup(tb2, np.array([1000, 1001, 3, 17, 4], np.int64), fallback=1)
    assert loc.tolist() == [0, 0, 1, 1, 0] and off[:2].tolist() == [7, 8]


# ------------------------------------------------------------------------------------------------------
# classify + partition + factored gather
# ------------------------------------------------------------------------------------------------------
def _classify(tb, keys_np, host_rows):
    n = len(keys_np)
    idx = dev_bytes(max(n, 1) * 8, fill=0xAB)
    counts = dev_zeros_u32(4)
    counts[2:] = 77  # the "next" pair must be cleared by the kernel
    st = dev_zeros_u32(1)
    fn = "ugk_classify_i64" if keys_np.dtype == np.int64 else "ugk_classify_u32"
    keys = to_dev(keys_np)
    hip.call(fn, tb, ptr(keys), n, host_rows, None, ptr(idx), ptr(counts), ptr(counts) + 8, ptr(st), None, None)
    sync()
    c = to_np(counts, np.uint32)
    return idx, counts, c, status_value(st), keys


@pytest.mark.parametrize("mode", ["flat", "hash", "hash32"])
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("n", [0, 1, 1023, 1024, 1025, 70_001])
def test_classify_partition_and_factored_gather(mode, kdtype, n):
    rng = np.random.default_rng(n + (7 if mode == "hash" else 0))
    nkeys, rb = 20_000, 512
    host = _rand_table(rng, nkeys, rb)
    cached = rng.choice(nkeys, 6_000, replace=False).astype(np.uint32)
    cap = 6_100
    cache = np.zeros((cap, rb), np.uint8)
    cache[: len(cached)] = host[cached]
    if mode == "flat":
        mem, tb = _make_flat(nkeys)
    else:
        mem, tb, _ = (_make_hash32 if mode == "hash32" else _make_hash)(len(cached))
    assert _insert(tb, cached.astype(kdtype)) == 0
    oflat = ORC.flat_table(nkeys)
    ORC.lib.orc_flat_insert(oflat, cached, np.arange(len(cached), dtype=np.uint32), len(cached))
    keys = (rng.zipf(1.1, size=n) % nkeys).astype(kdtype)

    idx, counts, c, st, keys_dev = _classify(tb, keys, nkeys)
    assert st == 0
    assert c[2] == 0 and c[3] == 0
    want_idx = ORC.sort_idx(ORC.lookup_src_dst(keys.astype(np.uint32), flat=oflat, fallback_loc=1))
    g = ORC.find_boundary(want_idx, 2) if n else np.zeros(3, np.uint32)
    assert c[0] == g[1] - g[0] and c[1] == g[2] - g[1] and c[0] + c[1] == n
    got = to_np(idx, IDX_DTYPE)[:n] if n else np.zeros(0, IDX_DTYPE)
    # same work items per group as the reference's sorted index, up to order inside a group
    def canon(a):
        return np.sort(a["dst_off"].astype(np.uint64) << 32 | a["src"].astype(np.uint64))
    want_hits = want_idx[: g[1]].copy()
    want_miss = want_idx[g[1]:].copy()
    want_miss["src"] &= 0x0FFFFFFF
    assert np.array_equal(canon(got[: c[0]]), canon(want_hits))
    assert np.array_equal(canon(got[n - c[1]:]), canon(want_miss))

    # factored extraction: host group and local group as two launches reading the device-side counts
    pin = pinned_from(host)
    mirror = pinned_from(np.array([0, 0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF], np.uint32))
    try:
        out = dev_bytes(n * rb, fill=0xCD)
        st2 = dev_zeros_u32(1)
        cache_dev = to_dev(cache)
        hip.call("ugk_gather_group", pin.ptr, nkeys, ptr(idx), ptr(counts), hip.LOC_HOST, n, ptr(out), n, rb, 4, ptr(st2),
                 mirror.ptr, None)
        hip.call("ugk_gather_group", ptr(cache_dev), cap, ptr(idx), ptr(counts), hip.LOC_LOCAL, n, ptr(out), n, rb, 0,
                 ptr(st2), mirror.ptr, None)
        assert status_value(st2) == 0
        if n:  # the gathers publish their group sizes in pinned host memory
            assert mirror.array.tolist() == [0, int(c[0]), int(c[1]), 0xFFFFFFFF]
        want_out, _ = ORC.extract_feat(keys.astype(np.uint32), cache, host, flat=oflat)
        assert to_np(out)[: n * rb].tobytes() == want_out.tobytes()
        assert want_out.tobytes() == host[keys.astype(np.int64)].tobytes()

        # fused single-kernel variant gives the same bytes
        out2 = dev_bytes(n * rb, fill=0x11)
        fn = "ugk_extract_mix_i64" if kdtype == np.int64 else "ugk_extract_mix_u32"
        for hint in (hip.HINT_UNKNOWN, 0, n):  # no guess; "all from the cache" (32 keys per wavefront); "none"
            out2.fill_(0x11)
            got_sizes = _extract_mix(fn, tb, keys_dev, n, cache_dev, cap, pin, nkeys, out2, rb, st2, mirror, hint)
            assert status_value(st2) == 0
            assert to_np(out2)[: n * rb].tobytes() == want_out.tobytes()
            assert got_sizes == [int(c[0]), int(c[1])]  # same group sizes as classify found
    finally:
        sync()
        pin.free()
        mirror.free()


def _extract_mix(fn, tb, keys_dev, n, cache_dev, cache_rows, pin, host_rows, out, rb, st, mirror,
                 hint=hip.HINT_UNKNOWN):
    """one fused launch; -> [rows from the cache, other rows], the sum of the words its workgroups leave in pinned
    host memory.  hint: the caller's guess of the second number, which may change the launch shape only."""
    words = PinnedArray((hip.lib().ugk_extract_mix_max_groups(),), np.uint64)
    try:
        words.array[...] = np.uint64(0xDEADBEEFDEADBEEF)
        groups = C.c_uint32(12345)
        hip.call(fn, tb, ptr(keys_dev), n, ptr(cache_dev), cache_rows, pin.ptr, host_rows, ptr(out), rb, ptr(st),
                 mirror.ptr if mirror is not None else None, words.ptr, C.byref(groups), hint, None)
        sync()
        g = groups.value
        assert (g == 0) if n == 0 else (1 <= g <= len(words.array))
        w = words.array[:g]
        assert (words.array[g:] == np.uint64(0xDEADBEEFDEADBEEF)).all()  # nothing written beyond the launched groups
        return [int((w & np.uint64(0xFFFFFFFF)).sum()), int((w >> np.uint64(32)).sum())]
    finally:
        words.free()


def test_outputs_beyond_4_GiB():
    """9M keys of 512-byte rows: the output (4.6 GB) passes 2^32 bytes, so every byte offset the kernels form must be a
    64-bit one.  table[r, c] is a closed form of (r, c); all three extraction paths are checked against it on the
    device, slice by slice."""
    rows, dim, n = 300_000, 128, 9_000_000
    rb = dim * 4
    assert n * rb > 1 << 32
    r = torch.arange(rows, device="cuda", dtype=torch.int32).unsqueeze(1)
    c = torch.arange(dim, device="cuda", dtype=torch.int32).unsqueeze(0)
    table = (r * 131 + c * 7919) ^ (r >> 3)
    g = torch.Generator(device="cuda").manual_seed(9)
    keys = torch.randint(0, rows, (n,), generator=g, device="cuda", dtype=torch.int32)
    keys[-1] = rows - 1
    keys[0] = 0

    def check(out):
        for lo in range(0, n, 1_000_000):
            k = keys[lo : lo + 1_000_000].unsqueeze(1)
            assert torch.equal(out[lo : lo + 1_000_000], (k * 131 + c * 7919) ^ (k >> 3)), lo

    st = dev_zeros_u32(1)
    out = torch.full((n, dim), 0x55555555, dtype=torch.int32, device="cuda")
    hip.call("ugk_gather_direct_u32", table.data_ptr(), rows, keys.data_ptr(), n, out.data_ptr(), rb, 0, ptr(st), None,
             None)
    assert status_value(st) == 0
    check(out)

    # every third row cached, in shuffled slots; the others are read from pinned host memory
    cached = np.arange(0, rows, 3, dtype=np.uint32)
    slots = np.random.default_rng(9).permutation(len(cached)).astype(np.uint32)
    mem, tb = _make_flat(rows)
    assert _insert(tb, cached, slots) == 0
    cache = torch.empty((len(cached), dim), dtype=torch.int32, device="cuda")
    cache[torch.from_numpy(slots.astype(np.int64)).cuda()] = table[torch.from_numpy(cached.astype(np.int64)).cuda()]
    pin = PinnedArray((rows, dim), np.int32)
    mirror = pinned_from(np.zeros(4, np.uint32))
    try:
        pin.array[...] = table.cpu().numpy()
        n_local = int((keys % 3 == 0).sum())
        out.fill_(0x55555555)
        sizes = _extract_mix("ugk_extract_mix_u32", tb, keys, n, cache, len(cached), pin, rows, out, rb, st, mirror)
        assert status_value(st) == 0 and sizes == [n_local, n - n_local]
        check(out)

        out.fill_(0x55555555)
        idx = dev_bytes(n * 8)
        counts = dev_zeros_u32(4)
        hip.call("ugk_classify_u32", tb, keys.data_ptr(), n, rows, None, ptr(idx), ptr(counts), ptr(counts) + 8, ptr(st),
                 None, None)
        hip.call("ugk_gather_group", pin.ptr, rows, ptr(idx), ptr(counts), hip.LOC_HOST, n, out.data_ptr(), n, rb, 0,
                 ptr(st), None, None)
        hip.call("ugk_gather_group", cache.data_ptr(), len(cached), ptr(idx), ptr(counts), hip.LOC_LOCAL, n,
                 out.data_ptr(), n, rb, 0, ptr(st), None, None)
        assert status_value(st) == 0
        assert to_np(counts, np.uint32)[:2].tolist() == [n_local, n - n_local]
        check(out)
    finally:
        sync()
        pin.free()
        mirror.free()


@pytest.mark.parametrize("kind", ["flat", "hash", "hash32"])
@pytest.mark.parametrize("rb", [32, 128, 512, 2048])
def test_extract_mix_at_every_launch_shape(kind, rb):
    """the fused kernel cuts a batch into wavefronts of 8, 16, 32 or 64 keys by the batch size, the table kind, the row
    size and the caller's hint; the bytes and the group sizes are the same at every shape"""
    rng = np.random.default_rng(rb)
    nkeys = 40_000
    host = _rand_table(rng, nkeys, rb)
    cached = rng.choice(nkeys, nkeys * 3 // 4, replace=False).astype(np.int64)
    slots = rng.permutation(len(cached)).astype(np.uint32)
    cache = np.zeros((len(cached), rb), np.uint8)
    cache[slots] = host[cached]
    if kind == "flat":
        mem, tb = _make_flat(nkeys)
    else:
        mem, tb, _ = (_make_hash32 if kind == "hash32" else _make_hash)(len(cached))
    assert _insert(tb, cached, slots) == 0
    is_cached = np.zeros(nkeys, bool)
    is_cached[cached] = True
    pin = pinned_from(host)
    mirror = pinned_from(np.zeros(4, np.uint32))
    try:
        st = dev_zeros_u32(1)
        d_cache = to_dev(cache)
        for n in (1, 63, 5_000, 70_000, 140_000, 270_000):
            keys = rng.integers(0, nkeys, size=n).astype(np.int64)
            d_keys = to_dev(keys)
            want = host[keys].tobytes()
            n_local = int(is_cached[keys].sum())
            for hint in (hip.HINT_UNKNOWN, 0):
                out = dev_bytes(n * rb, fill=0x3C)
                sizes = _extract_mix("ugk_extract_mix_i64", tb, d_keys, n, d_cache, len(cached), pin, nkeys, out, rb, st,
                                     mirror, hint)
                assert status_value(st) == 0
                assert sizes == [n_local, n - n_local], (n, hint)
                assert to_np(out)[: n * rb].tobytes() == want, (n, hint)
    finally:
        sync()
        pin.free()
        mirror.free()


def _pool_reference(table_f64, ids, seg_off, weights, combiner):
    """embedding_lookup_sparse in float64: weighted sum of every segment's rows, divided by the sum of the weights
    (mean) or the root of the sum of their squares (sqrtn); a zero denominator and an empty segment give a zero row"""
    n_rows = len(seg_off) - 1
    w = np.ones(len(ids), np.float64) if weights is None else weights.astype(np.float64)
    out = np.zeros((n_rows, table_f64.shape[1]), np.float64)
    seg = np.repeat(np.arange(n_rows), np.diff(seg_off))
    np.add.at(out, seg, table_f64[ids] * w[:, None])
    if combiner == 0:
        return out
    den = np.zeros(n_rows, np.float64)
    np.add.at(den, seg, w if combiner == 1 else w * w)
    if combiner == 2:
        den = np.sqrt(den)
    safe = np.where(den != 0, den, 1.0)
    return np.where(den[:, None] != 0, out / safe[:, None], 0.0)


def _bf16_bits(a32):
    """float32 values cut to bfloat16 bit patterns (uint16)"""
    return (np.ascontiguousarray(a32, np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def _bf16_values(bits):
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


_POOL_SHAPES = [(4, np.float32), (32, np.float32), (128, np.float32), (512, np.float32), (1024, np.float32),
                (8, np.float16), (64, np.float16), (256, np.float16), (2048, np.float16), (64, "bf16"), (256, "bf16")]
# every shape with the rows per lane group the launch picks, some of them with three and eight rows forced
_POOL_CASES = [(d, e, "") for d, e in _POOL_SHAPES] + [
    (d, e, r) for r in ("3", "8") for d, e in [(32, np.float32), (512, np.float32), (64, np.float16), (2048, np.float16),
                                               (64, "bf16")]]


@pytest.mark.parametrize("kind", ["none", "flat", "hash", "hash32"])
@pytest.mark.parametrize("dim,etype,rows_per_group", _POOL_CASES)
def test_pooled_extraction_matches_a_float64_segment_sum(kind, dim, etype, rows_per_group, monkeypatch):
    """ugk_extract_pool_*: rows looked up and combined per segment in one kernel (sum, mean, sqrtn; with and without
    weights, negative and zero ones among them; segments that are empty, single, longer than a lane group; three
    or eight output rows per lane group and pass, or as many as the launch picks by itself: one for these).  fp32
    rows within 1e-5 of the magnitude of the terms that were added (sum of |w x|, over the denominator), fp16 rows
    within 1e-3 of the result on top (the output is rounded to fp16); the counts are those of the ids by source, as for
    the plain fused extraction."""
    if rows_per_group:
        monkeypatch.setenv("UGK_POOL_ROWS", rows_per_group)
    rng = np.random.default_rng(dim + len(kind))
    nkeys = 20_000
    bf16 = isinstance(etype, str)
    esize = 2 if bf16 else np.dtype(etype).itemsize
    ecode = hip.ELEM_BF16 if bf16 else esize
    rb = dim * esize
    if bf16:  # numpy has no bfloat16: the table is its bit patterns, the values are those patterns widened
        host_bits = _bf16_bits(rng.standard_normal((nkeys, dim)))
        host = _bf16_values(host_bits)
        host_bytes = host_bits.view(np.uint8).reshape(nkeys, rb)
    else:
        host = rng.standard_normal((nkeys, dim)).astype(etype)
        host_bytes = host.view(np.uint8).reshape(nkeys, rb)
    if kind == "none":  # no table: the id is the row, the "host" table may be anywhere (here HBM)
        tb = hip.table(0, None, 0)
        cached = np.zeros(0, np.int64)
        mem = None
    else:
        cached = rng.choice(nkeys, nkeys * 3 // 4, replace=False).astype(np.int64)
        if kind == "flat":
            mem, tb = _make_flat(nkeys)
        else:
            mem, tb, _ = (_make_hash32 if kind == "hash32" else _make_hash)(len(cached))
    slots = rng.permutation(len(cached)).astype(np.uint32)
    cache = np.zeros((max(len(cached), 1), rb), np.uint8)
    if len(cached):
        cache[slots] = host_bytes[cached]
        assert _insert(tb, cached, slots) == 0
    is_cached = np.zeros(nkeys, bool)
    is_cached[cached] = True
    pin = pinned_from(host_bytes)
    mirror = pinned_from(np.zeros(4, np.uint32))
    words = PinnedArray((hip.lib().ugk_extract_mix_max_groups(),), np.uint64)
    try:
        st = dev_zeros_u32(1)
        d_cache = to_dev(cache)
        f64 = host.astype(np.float64)
        for n_rows in (1, 7, 3_000):
            lens = rng.choice([0, 1, 2, 5, 9, 40, 70], size=n_rows, p=[0.05, 0.3, 0.2, 0.2, 0.15, 0.07, 0.03])
            seg_off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
            nnz = int(seg_off[-1])
            ids = rng.integers(0, nkeys, size=max(nnz, 1)).astype(np.int64)[:nnz]
            wts = rng.standard_normal(nnz).astype(np.float32)
            wts[rng.random(nnz) < 0.1] = 0.0
            d_ids, d_off, d_w = to_dev(ids if nnz else np.zeros(1, np.int64)), to_dev(seg_off), to_dev(wts if nnz else np.zeros(1, np.float32))
            for combiner in (0, 1, 2):
                for weights in (None, wts):
                    out = dev_bytes(n_rows * rb, fill=0x7F)
                    groups = C.c_uint32(0)
                    hip.call("ugk_extract_pool_i64", tb, ptr(d_ids), ptr(d_off), None if weights is None else ptr(d_w),
                             n_rows, nnz, combiner, ecode, ptr(d_cache), len(cached), pin.ptr, nkeys,
                             ptr(out), rb, ptr(st), mirror.ptr, words.ptr, C.byref(groups), None)
                    sync()
                    assert status_value(st) == 0
                    w = words.array[:groups.value]
                    n_local = int(is_cached[ids].sum())
                    assert [int((w & np.uint64(0xFFFFFFFF)).sum()), int((w >> np.uint64(32)).sum())] == [n_local, nnz - n_local]
                    if bf16:
                        got = _bf16_values(to_np(out)[: n_rows * rb].view(np.uint16)).reshape(n_rows, dim).astype(np.float64)
                    else:
                        got = to_np(out)[: n_rows * rb].view(etype).reshape(n_rows, dim).astype(np.float64)
                    want = _pool_reference(f64, ids, seg_off, weights, combiner)
                    # fp32 adds of n terms are off by at most n 2^-24 of the terms' magnitudes; an fp16 output is
                    # rounded to 11 bits on top.  (A mean over signed weights that nearly cancel is large and still
                    # as accurate as its terms.)
                    absw = None if weights is None else np.abs(wts)
                    mag = _pool_reference(np.abs(f64), ids, seg_off, absw, 0)
                    if combiner:
                        den = _pool_reference(np.ones((nkeys, 1)), ids, seg_off,
                                              weights if combiner == 1 or weights is None else wts * wts, 0)
                        den = np.abs(den) if combiner == 1 else np.sqrt(den)
                        mag = np.where(den != 0, mag / np.where(den != 0, den, 1.0), 0.0)
                        if combiner == 1 and weights is not None:
                            # the sum of signed weights is itself a rounded sum: its relative error is that of its
                            # terms' magnitudes over what is left of them
                            sum_abs = _pool_reference(np.ones((nkeys, 1)), ids, seg_off, absw, 0)
                            mag = mag + np.abs(want) * np.where(den != 0, sum_abs / np.where(den != 0, den, 1.0), 0.0)
                    # (fp16 results below 2^-14 are subnormal: steps of 2^-24 whatever their size)
                    bound = 1e-5 * mag + (1e-3 * np.abs(want) + 2.0 ** -25 if etype == np.float16 else 0.0) + 1e-30
                    if bf16:  # a bfloat16 result is rounded to 8 bits
                        bound = bound + 2.0 ** -8 * np.abs(want)
                    if etype == np.float16:  # a mean over weights that nearly cancel may leave fp16's range
                        big = np.abs(want) > 6.0e4
                        assert np.isinf(got[big & (np.abs(want) > 6.6e4)]).all()
                        got, want = np.where(big, 0.0, got), np.where(big, 0.0, want)
                    worst = np.unravel_index(np.argmax(np.abs(got - want) - bound), got.shape)
                    assert (np.abs(got - want) <= bound).all(), "%s dim %d rows %d combiner %d weights %s: [%d, %d] got %r " \
                        "want %r bound %r ids %d" % (kind, dim, n_rows, combiner, weights is not None, worst[0], worst[1],
                                                    float(got[worst]), float(want[worst]), float(bound[worst]),
                                                    int(lens[worst[0]]))
    finally:
        sync()
        pin.free()
        mirror.free()
        words.free()


@pytest.mark.parametrize("rows_per_group", ["", "2", "8"])
def test_pooled_extraction_hand_worked(rows_per_group, monkeypatch):
    if rows_per_group:
        monkeypatch.setenv("UGK_POOL_ROWS", rows_per_group)
    # rows r = [r, 10 r]; segments {1, 2}, {3}, {}, {4, 4} with weights 1 2 | 3 | | 1 -1
    host = np.array([[r, 10 * r, 0, 0] for r in range(6)], np.float32)
    pin = pinned_from(host.view(np.uint8).reshape(6, 16))
    try:
        ids, off = to_dev(np.array([1, 2, 3, 4, 4], np.int64)), to_dev(np.array([0, 2, 3, 3, 5], np.int64))
        wts = to_dev(np.array([1, 2, 3, 1, -1], np.float32))
        st = dev_zeros_u32(1)
        cache = dev_bytes(16)

        def run(combiner, w):
            out = dev_bytes(4 * 16, fill=0x55)
            hip.call("ugk_extract_pool_i64", hip.table(0, None, 0), ptr(ids), ptr(off), w, 4, 5, combiner, 4, ptr(cache), 0,
                     pin.ptr, 6, ptr(out), 16, ptr(st), None, None, None, None)
            sync()
            assert status_value(st) == 0
            return to_np(out)[:64].view(np.float32).reshape(4, 4)[:, :2].tolist()

        assert run(0, None) == [[3, 30], [3, 30], [0, 0], [8, 80]]
        assert run(0, ptr(wts)) == [[5, 50], [9, 90], [0, 0], [0, 0]]
        assert run(1, None) == [[1.5, 15], [3, 30], [0, 0], [4, 40]]
        assert run(1, ptr(wts)) == [[5 / 3, 50 / 3], [3, 30], [0, 0], [0, 0]] or \
            np.allclose(run(1, ptr(wts)), [[5 / 3, 50 / 3], [3, 30], [0, 0], [0, 0]], rtol=1e-6)  # weights cancel: 0 / 0 -> 0
        got = run(2, ptr(wts))
        assert np.allclose(got, [[5 / 5 ** 0.5, 50 / 5 ** 0.5], [3, 30], [0, 0], [0, 0]], rtol=1e-6)
        # an id without a row flags the launch and adds nothing
        bad = to_dev(np.array([1, 77, 3, 4, 4], np.int64))
        out = dev_bytes(4 * 16)
        hip.call("ugk_extract_pool_i64", hip.table(0, None, 0), ptr(bad), ptr(off), None, 4, 5, 0, 4, ptr(cache), 0, pin.ptr,
                 6, ptr(out), 16, ptr(st), None, None, None, None)
        sync()
        assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE
        assert to_np(out)[:64].view(np.float32).reshape(4, 4)[0, :2].tolist() == [1, 10]
        # offsets that leave the ids (beyond nnz, negative, running backwards) flag the launch, read nothing and
        # give rows of zeros; the other rows are unharmed
        key = np.array([1, 2, 3, 4, 4])
        # offsets that stay inside the ids but do not begin at 0 or end at nnz flag the launch as well: the rows are what
        # the offsets say, the per-source counts of ids would not add up to nnz
        for broken in ([0, 2, 3, 3, 9], [0, 2, 3, 3, 1 << 40], [0, 2, -7, 3, 5], [0, 4, 3, 3, 5], [1, 2, 3, 3, 5],
                       [0, 2, 3, 3, 4]):
            st.zero_()
            boff = to_dev(np.array(broken, np.int64))
            out = dev_bytes(4 * 16, fill=0x55)
            hip.call("ugk_extract_pool_i64", hip.table(0, None, 0), ptr(ids), ptr(boff), None, 4, 5, 0, 4, ptr(cache), 0,
                     pin.ptr, 6, ptr(out), 16, ptr(st), None, None, None, None)
            sync()
            assert status_value(st) == hip.ST_BAD_SEGMENT, broken
            want = []
            for r in range(4):
                b, e = broken[r], broken[r + 1]
                s = float(key[b:e].sum()) if 0 <= b <= e <= 5 else 0.0
                want.append([s, 10 * s])
            assert to_np(out)[:64].view(np.float32).reshape(4, 4)[:, :2].tolist() == want, broken
    finally:
        sync()
        pin.free()


@pytest.mark.parametrize("kind", ["none", "flat", "hash", "hash32"])
@pytest.mark.parametrize("dim,etype", [(4, np.float32), (32, np.float32), (100, np.float32), (128, np.float32),
                                       (512, np.float32), (1024, np.float32), (64, np.float16), (2048, np.float16),
                                       (64, "bf16")])
def test_pooled_extraction_with_max_norm_matches_the_oracle(kind, dim, etype):
    """ugk_extract_pool_clip_*: every looked-up row is clipped to the l2 norm max_norm before it is weighted, in the
    same kernel; against the oracle's float64 statement (orc_pool_clip_f64) on rows whose norms lie on both sides of
    max_norm.  Tolerance as for the plain pooled extraction: 1e-5 of the magnitude of the terms (the norm is a fp32
    sum of up to 2048 squares, good to a few 1e-7 relative), fp16 / bf16 outputs rounded on top.  max_norm = 0 is
    the plain kernel, bit for bit."""
    rng = np.random.default_rng(dim + 3 * len(kind))
    nkeys = 8_000
    bf16 = isinstance(etype, str)
    esize = 2 if bf16 else np.dtype(etype).itemsize
    ecode = hip.ELEM_BF16 if bf16 else esize
    rb = dim * esize
    scale = rng.uniform(0.05, 3.0, size=(nkeys, 1)) / np.sqrt(dim)  # row norms between 0.05 and 3
    vals = rng.standard_normal((nkeys, dim)) * scale
    vals[:50] = 0.0  # rows of zeros have norm 0 and stay zeros
    if bf16:
        host_bits = _bf16_bits(vals)
        host = _bf16_values(host_bits)
        host_bytes = host_bits.view(np.uint8).reshape(nkeys, rb)
    else:
        host = vals.astype(etype)
        host_bytes = host.view(np.uint8).reshape(nkeys, rb)
    if kind == "none":
        tb, cached, mem = hip.table(0, None, 0), np.zeros(0, np.int64), None
    else:
        cached = rng.choice(nkeys, nkeys // 2, replace=False).astype(np.int64)
        mem, tb = _make_flat(nkeys) if kind == "flat" else (_make_hash32 if kind == "hash32" else _make_hash)(len(cached))[:2]
    slots = rng.permutation(len(cached)).astype(np.uint32)
    cache = np.zeros((max(len(cached), 1), rb), np.uint8)
    if len(cached):
        cache[slots] = host_bytes[cached]
        assert _insert(tb, cached, slots) == 0
    pin = pinned_from(host_bytes)
    try:
        st = dev_zeros_u32(1)
        d_cache = to_dev(cache)
        f64 = host.astype(np.float64)
        n_rows = 2_000
        lens = rng.choice([0, 1, 2, 5, 9, 40], size=n_rows, p=[0.05, 0.3, 0.25, 0.2, 0.15, 0.05])
        seg_off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        nnz = int(seg_off[-1])
        ids = rng.integers(0, nkeys, size=nnz).astype(np.int64)
        wts = rng.uniform(0.1, 2.0, size=nnz).astype(np.float32)
        d_ids, d_off, d_w = to_dev(ids), to_dev(seg_off), to_dev(wts)

        def run(entry, *norm):
            out = dev_bytes(n_rows * rb, fill=0x7F)
            hip.call(entry, tb, ptr(d_ids), ptr(d_off), ptr(d_w), n_rows, nnz, combiner, ecode, *norm, ptr(d_cache),
                     len(cached), pin.ptr, nkeys, ptr(out), rb, ptr(st), None, None, None, None)
            sync()
            assert status_value(st) == 0
            return to_np(out)[: n_rows * rb]

        for combiner in (0, 1, 2):
            assert run("ugk_extract_pool_clip_i64", 0.0).tobytes() == run("ugk_extract_pool_i64").tobytes()
            for max_norm in (0.4, 1.5, 100.0):
                raw = run("ugk_extract_pool_clip_i64", max_norm)
                got = (_bf16_values(raw.view(np.uint16)) if bf16 else raw.view(etype)).reshape(n_rows, dim).astype(np.float64)
                want = ORC.pool(f64, ids, seg_off, wts, combiner, max_norm=max_norm)
                mag = ORC.pool(np.abs(f64), ids, seg_off, wts, combiner, max_norm=max_norm)
                tol = 1e-5 * mag + 1e-30
                if esize == 2:
                    tol = tol + (2.0 ** -8 if bf16 else 1e-3) * np.abs(want) + 2.0 ** -24
                assert (np.abs(got - want) <= tol).all(), (combiner, max_norm, float(np.abs(got - want).max()))
                if max_norm == 100.0:  # beyond every row's norm: nothing is clipped
                    plain = ORC.pool(f64, ids, seg_off, wts, combiner)
                    assert (np.abs(got - plain) <= tol).all()
        with pytest.raises(hip.UgkError, match="max_norm"):
            hip.call("ugk_extract_pool_clip_i64", tb, ptr(d_ids), ptr(d_off), None, n_rows, nnz, 0, ecode, -1.0,
                     ptr(d_cache), len(cached), pin.ptr, nkeys, ptr(dev_bytes(n_rows * rb)), rb, ptr(st), None, None,
                     None, None)
    finally:
        sync()
        pin.free()


@pytest.mark.parametrize("n_rows,nnz", [(1, 0), (1, 1), (5, 0), (7, 3), (1000, 1000), (5000, 60_000), (300_000, 40_000),
                                        (3_000_000, 5), (1_000_000, 0), (200, 129)])
def test_segment_offsets_match_searchsorted(n_rows, nnz):
    """ugk_segment_offsets_i64: seg_off[r] = number of entries whose row is below r (rows without an entry among them)"""
    rng = np.random.default_rng(n_rows + nnz)
    rows = np.sort(rng.integers(0, n_rows, size=nnz)).astype(np.int64)
    st = dev_zeros_u32(1)
    d_rows = to_dev(rows if nnz else np.zeros(1, np.int64))
    out = to_dev(np.full(n_rows + 1, -7, np.int64))
    hip.call("ugk_segment_offsets_i64", ptr(d_rows), nnz, n_rows, ptr(out), ptr(st), None, None)
    sync()
    assert status_value(st) == 0
    assert np.array_equal(to_np(out), np.searchsorted(rows, np.arange(n_rows + 1), side="left"))


@pytest.mark.parametrize("bad", [[0, 2, 1, 3], [0, 1, 2, 9], [-1, 0, 1, 2], [3, 2, 1, 0], [0, 1, 2, 1 << 40]])
def test_segment_offsets_flag_rows_out_of_order_or_range(bad):
    st = dev_zeros_u32(1)
    out = to_dev(np.full(6, -7, np.int64))
    hip.call("ugk_segment_offsets_i64", ptr(to_dev(np.array(bad, np.int64))), 4, 5, ptr(out), ptr(st), None, None)
    sync()
    assert status_value(st) == hip.ST_BAD_SEGMENT
    got = to_np(out)
    assert ((got == -7) | ((got >= 0) & (got <= 4))).all()  # nothing written but offsets into the entries


def _fmix64(x):
    x = np.asarray(x, np.uint64).copy()
    x ^= x >> np.uint64(33)
    x *= np.uint64(0xFF51AFD7ED558CCD)
    x ^= x >> np.uint64(33)
    x *= np.uint64(0xC4CEB9FE1A85EC53)
    x ^= x >> np.uint64(33)
    return x


@pytest.mark.parametrize("kind", ["flat", "hash", "hash32"])
@pytest.mark.parametrize("rb", [64, 128, 512])
def test_rows_from_the_host_are_filed_in_the_stage_and_found_there(kind, rb):
    """ugk_extract_mix_staged_*: same output and group sizes as the plain extraction; afterwards every owner word with a
    tag names a host row whose bytes its entry holds, entries are where fmix64(row) & mask says, and rows of the cache
    are never filed.  ugk_gather_scatter_staged_u32: the bytes of ugk_gather_scatter_u32; the number of rows it reports
    as taken from the stage is the number of listed rows the owner words name."""
    rng = np.random.default_rng(rb + (kind == "hash"))
    nkeys, entries = 30_000, 4096
    host = _rand_table(rng, nkeys, rb)
    cached = rng.choice(nkeys, nkeys // 2, replace=False).astype(np.int64)
    slots = rng.permutation(len(cached)).astype(np.uint32)
    cache = np.zeros((len(cached), rb), np.uint8)
    cache[slots] = host[cached]
    if kind == "flat":
        mem, tb = _make_flat(nkeys)
    else:
        mem, tb, _ = (_make_hash32 if kind == "hash32" else _make_hash)(len(cached))
    assert _insert(tb, cached, slots) == 0
    is_cached = np.zeros(nkeys, bool)
    is_cached[cached] = True
    pin = pinned_from(host)
    mirror = pinned_from(np.zeros(4, np.uint32))
    try:
        st = dev_zeros_u32(1)
        d_cache = to_dev(cache)
        stage_rows = dev_bytes(entries * rb, fill=0xEE)
        owner = to_dev(np.zeros(entries, np.uint64))
        words = PinnedArray((hip.lib().ugk_extract_mix_max_groups(),), np.uint64)
        groups = C.c_uint32(0)
        seen_hosts = set()
        for epoch, n in enumerate((1, 700, 9_000, 70_000), start=1):
            keys = rng.integers(0, nkeys, size=n).astype(np.int64)
            d_keys = to_dev(keys)
            out = dev_bytes(n * rb, fill=0x3C)
            stage = hip.Stage(ptr(stage_rows), ptr(owner), entries - 1, epoch, 0)
            hip.call("ugk_extract_mix_staged_i64", tb, ptr(d_keys), n, ptr(d_cache), len(cached), pin.ptr, nkeys,
                     ptr(out), rb, ptr(st), mirror.ptr, words.ptr, C.byref(groups), hip.HINT_UNKNOWN, stage, None)
            sync()
            assert status_value(st) == 0
            w = words.array[: groups.value]
            n_local = int(is_cached[keys].sum())
            assert [int((w & np.uint64(0xFFFFFFFF)).sum()), int((w >> np.uint64(32)).sum())] == [n_local, n - n_local]
            assert to_np(out)[: n * rb].tobytes() == host[keys].tobytes()
            seen_hosts.update(keys[~is_cached[keys]].tolist())
            own = to_np(owner, np.uint64)[:entries]
            tags, rows = (own >> np.uint64(32)).astype(np.int64), (own & np.uint64(0xFFFFFFFF)).astype(np.int64)
            filled = np.flatnonzero(tags != 0)
            assert (len(filled) > 0) == bool(seen_hosts) and tags.max() <= epoch
            assert all(int(r) in seen_hosts for r in rows[filled])  # only rows that came from the host, never cached ones
            assert np.array_equal(_fmix64(rows[filled]) & np.uint64(entries - 1), filled.astype(np.uint64))
            got = to_np(stage_rows)[: entries * rb].reshape(entries, rb)
            assert np.array_equal(got[filled], host[rows[filled]])
            # every host row of this batch whose entry was free of this launch's tag before it is there now, or lost
            # its entry to another row of the same launch
            missed = np.unique(keys[~is_cached[keys]])
            h = (_fmix64(missed) & np.uint64(entries - 1)).astype(np.int64)
            assert (tags[h] != 0).all()
        # the staged gather: rows from everywhere, some filed, some not
        own = to_np(owner, np.uint64)[:entries]
        filed_rows = (own[(own >> np.uint64(32)) != 0] & np.uint64(0xFFFFFFFF)).astype(np.uint32)
        take = np.unique(np.concatenate([filed_rows[::2], rng.integers(0, nkeys, size=5000).astype(np.uint32)]))
        rng.shuffle(take)
        dst = rng.permutation(len(take) + 100)[: len(take)].astype(np.uint32)
        out_rows = len(take) + 100
        out = dev_bytes(out_rows * rb, fill=0x11)
        n_staged = dev_zeros_u32(1)
        d_take, d_dst = to_dev(take), to_dev(dst)
        stage = hip.Stage(ptr(stage_rows), ptr(owner), entries - 1, 0, 0)
        for cap in (0, 7):
            hip.call("ugk_gather_scatter_staged_u32", pin.ptr, nkeys, ptr(d_take), ptr(d_dst), len(take), ptr(out),
                     out_rows, rb, stage, cap, ptr(st), ptr(n_staged), None, None, None, None, None)
        sync()
        assert status_value(st) == 0
        want = np.full((out_rows, rb), 0x11, np.uint8)
        want[dst] = host[take]
        assert to_np(out)[: out_rows * rb].tobytes() == want.tobytes()
        in_stage = np.isin(take, filed_rows)
        assert int(to_np(n_staged, np.uint32)[0]) == 2 * int(in_stage.sum())
        # with a rest list: only what the stage holds is copied, the other rows are listed with their destinations
        out2 = dev_bytes(out_rows * rb, fill=0x11)
        rest_rows, rest_dst, rest_n = dev_zeros_u32(len(take)), dev_zeros_u32(len(take)), dev_zeros_u32(1)
        done_n = dev_zeros_u32(1)
        hip.call("ugk_gather_scatter_staged_u32", pin.ptr, nkeys, ptr(d_take), ptr(d_dst), len(take), ptr(out2),
                 out_rows, rb, stage, 3, ptr(st), None, ptr(rest_rows), ptr(rest_dst), ptr(rest_n), ptr(done_n), None)
        sync()
        assert status_value(st) == 0
        m = int(to_np(rest_n, np.uint32)[0])
        assert m == int((~in_stage).sum())
        got_rest = sorted(zip(to_np(rest_rows, np.uint32)[:m].tolist(), to_np(rest_dst, np.uint32)[:m].tolist()))
        assert got_rest == sorted(zip(take[~in_stage].tolist(), dst[~in_stage].tolist()))
        # ... and the rows that were copied, from the back of the same lists
        k = int(to_np(done_n, np.uint32)[0])
        assert k == int(in_stage.sum()) and k + m == len(take)
        got_done = sorted(zip(to_np(rest_rows, np.uint32)[m:len(take)].tolist(),
                              to_np(rest_dst, np.uint32)[m:len(take)].tolist()))
        assert got_done == sorted(zip(take[in_stage].tolist(), dst[in_stage].tolist()))
        want2 = np.full((out_rows, rb), 0x11, np.uint8)
        want2[dst[in_stage]] = host[take[in_stage]]
        assert to_np(out2)[: out_rows * rb].tobytes() == want2.tobytes()
        words.free()
    finally:
        sync()
        pin.free()
        mirror.free()


def test_classify_rejects_keys_beyond_the_host_table():
    mem, tb = _make_flat(100)
    keys = np.array([5, 100, 7, 1 << 33], np.int64)
    idx, counts, c, st, _ = _classify(tb, keys, 100)
    assert st & hip.ST_KEY_OUT_OF_RANGE
    assert c[0] == 0 and c[1] == 2
    got = to_np(idx, IDX_DTYPE)[:4]
    assert sorted(got[2:]["dst_off"].tolist()) == [0, 2] and sorted(got[2:]["src"].tolist()) == [5, 7]


def test_extract_mix_skips_keys_without_a_row_and_still_hands_over_its_counts():
    """a key beyond the host table flags the launch and leaves its output row alone; the skipped rows are counted with
    the host rows, the count words are left at zero, and the next (clean) launch reports exact group sizes"""
    rng = np.random.default_rng(11)
    nkeys, rb, n = 3000, 64, 2000
    host = _rand_table(rng, nkeys, rb)
    mem, tb = _make_flat(nkeys)
    cached = np.arange(0, nkeys, 3, dtype=np.uint32)
    assert _insert(tb, cached) == 0
    cache = host[cached].copy()
    keys = rng.integers(0, nkeys, size=n).astype(np.int64)
    bad = rng.choice(n, 37, replace=False)
    dirty = keys.copy()
    dirty[bad] = nkeys + rng.integers(0, 1 << 35, size=len(bad))
    pin = pinned_from(host)
    mirror = pinned_from(np.zeros(4, np.uint32))
    try:
        st = dev_zeros_u32(1)
        d_cache = to_dev(cache)
        for batch in (dirty, keys):
            out = dev_bytes(n * rb, fill=0x5A)
            d_keys = to_dev(batch)
            mirror.array[...] = 0
            st.zero_()
            sizes = _extract_mix("ugk_extract_mix_i64", tb, d_keys, n, d_cache, len(cached), pin, nkeys, out, rb, st,
                                 mirror)
            flagged = status_value(st)
            got = to_np(out)[: n * rb].reshape(n, rb)
            ok = batch < nkeys
            assert got[ok].tobytes() == host[batch[ok]].tobytes()
            assert (got[~ok] == 0x5A).all()
            local = int((batch[ok] % 3 == 0).sum())
            assert sizes == [local, n - local]
            if ok.all():
                assert flagged == 0 and mirror.array[0] == 0
            else:
                assert flagged & hip.ST_KEY_OUT_OF_RANGE and mirror.array[0] == hip.ST_KEY_OUT_OF_RANGE
    finally:
        sync()
        pin.free()
        mirror.free()


@pytest.mark.parametrize("row_bytes", [128, 64, 1024])
def test_extract_mix_other_row_sizes(row_bytes):
    rng = np.random.default_rng(row_bytes)
    nkeys = 5000
    host = _rand_table(rng, nkeys, row_bytes)
    cached = rng.choice(nkeys, 1500, replace=False).astype(np.uint32)
    cache = host[cached].copy()
    mem, tb, _ = _make_hash(len(cached))
    assert _insert(tb, cached) == 0
    keys = rng.integers(0, nkeys, size=10_001).astype(np.uint32)
    pin = pinned_from(host)
    try:
        out = dev_bytes(len(keys) * row_bytes)
        st = dev_zeros_u32(1)
        d_keys, d_cache = to_dev(keys), to_dev(cache)
        hip.call("ugk_extract_mix_u32", tb, ptr(d_keys), len(keys), ptr(d_cache), len(cached), pin.ptr,
                 nkeys, ptr(out), row_bytes, ptr(st), None, None, None, hip.HINT_UNKNOWN, None)
        assert status_value(st) == 0
        assert to_np(out)[: len(keys) * row_bytes].tobytes() == host[keys].tobytes()
    finally:
        sync()
        pin.free()


# ------------------------------------------------------------------------------------------------------
# dedup
# ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("n", [1, 255, 256, 257, 100_000])
def test_dedup_matches_numpy_unique(kdtype, n):
    rng = np.random.default_rng(n)
    space = (1 << 31) if kdtype == np.uint32 else (1 << 40)
    pool = rng.integers(0, space, size=max(n // 3, 1))
    ws_bytes = hip.lib().ugk_dedup_workspace_bytes(n)
    ws = dev_bytes(ws_bytes, fill=0)
    for epoch in (1, 2, 3):  # the workspace is reused without clearing
        keys = pool[rng.integers(0, len(pool), size=n)].astype(kdtype)
        uniq = dev_bytes(n * np.dtype(kdtype).itemsize)
        inv = dev_zeros_u32(n)
        nu = dev_zeros_u32(1)
        rep = dev_zeros_u32(n)
        fn = "ugk_dedup_i64" if kdtype == np.int64 else "ugk_dedup_u32"
        d_keys = to_dev(keys)
        hip.call(fn, ptr(d_keys), n, ptr(ws), ws_bytes, epoch, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
        sync()
        k = int(to_np(nu, np.uint32)[0])
        u = to_np(uniq, kdtype)[:k]
        i = to_np(inv, np.uint32)[:n]
        want_u, _ = ORC.dedup(keys.astype(np.int64))
        assert k == len(want_u) == len(np.unique(keys))
        assert np.array_equal(np.sort(u.astype(np.int64)), np.sort(want_u))
        assert i.max() < k and np.array_equal(u[i], keys)
        r = to_np(rep, np.uint32)[:k]
        assert np.array_equal(keys[r], u) and np.array_equal(i[r], np.arange(k))  # representatives


@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("n", [1000, 70_000, 300_000])
@pytest.mark.parametrize("shape", ["one_key", "two_keys", "geometric", "hot_and_cold"])
def test_dedup_of_skewed_keys(kdtype, n, shape):
    """batches whose duplicates meet inside a tile: the occurrences of a key elect one leader in LDS, and only leaders
    reach the device-wide set"""
    rng = np.random.default_rng(n + len(shape))
    space = (1 << 31) if kdtype == np.uint32 else (1 << 40)
    if shape == "one_key":
        keys = np.full(n, 12345 % space)
    elif shape == "two_keys":
        keys = np.where(rng.random(n) < 0.5, 7, space - 1)
    elif shape == "geometric":
        keys = (rng.geometric(0.01, size=n) * 2654435761) % space
    else:  # a tenth of the batch is one hot key, the rest are distinct
        keys = rng.choice(space, size=n, replace=False) if space > 10 * n else rng.integers(0, space, size=n)
        keys[rng.random(n) < 0.1] = 99
    keys = keys.astype(kdtype)
    ws_bytes = hip.lib().ugk_dedup_workspace_bytes(n)
    ws = dev_bytes(ws_bytes, fill=0)
    d_keys = to_dev(keys)
    for epoch in (1, 2):
        uniq = dev_bytes(n * np.dtype(kdtype).itemsize)
        inv, nu, rep = dev_zeros_u32(n), dev_zeros_u32(1), dev_zeros_u32(n)
        fn = "ugk_dedup_i64" if kdtype == np.int64 else "ugk_dedup_u32"
        hip.call(fn, ptr(d_keys), n, ptr(ws), ws_bytes, epoch, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
        sync()
        k = int(to_np(nu, np.uint32)[0])
        u = to_np(uniq, kdtype)[:k]
        i = to_np(inv, np.uint32)[:n]
        assert k == len(np.unique(keys))
        assert np.array_equal(np.sort(u), np.unique(keys))
        assert i.max() < k and np.array_equal(u[i], keys)
        r = to_np(rep, np.uint32)[:k]
        assert np.array_equal(keys[r], u) and np.array_equal(i[r], np.arange(k))


@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
def test_dedup_of_small_and_large_batches_sharing_one_workspace(kdtype):
    """One workspace, sized for the largest batch, serves batches of every smaller size in any order: the slot set and
    the per-occurrence ids sit where the workspace's own size puts them, so nothing a small batch writes can read as a
    claim of the current epoch to a larger one.  Few distinct keys and small epochs make stale words look plausible."""
    rng = np.random.default_rng(99)
    n_max = 40_000
    ws_bytes = hip.lib().ugk_dedup_workspace_bytes(n_max)
    ws = dev_bytes(ws_bytes, fill=0)
    fn = "ugk_dedup_i64" if kdtype == np.int64 else "ugk_dedup_u32"
    pool = rng.integers(0, 3000, size=600)
    epoch = 0
    for n in (700, 40_000, 1100, 33_000, 5, 40_000, 2050, 2049, 40_000, 1024, 39_999):
        epoch += 1
        keys = pool[rng.integers(0, len(pool), size=n)].astype(kdtype)
        uniq = dev_bytes(n * np.dtype(kdtype).itemsize)
        inv, nu, rep = dev_zeros_u32(n), dev_zeros_u32(1), dev_zeros_u32(n)
        hip.call(fn, ptr(to_dev(keys)), n, ptr(ws), ws_bytes, epoch, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
        sync()
        k = int(to_np(nu, np.uint32)[0])
        u = to_np(uniq, kdtype)[:k]
        i = to_np(inv, np.uint32)[:n]
        assert k == len(np.unique(keys)), (n, epoch)
        assert np.array_equal(np.sort(u), np.unique(keys))
        assert i.max() < k and np.array_equal(u[i], keys)
        r = to_np(rep, np.uint32)[:k]
        assert np.array_equal(keys[r], u) and np.array_equal(i[r], np.arange(k))
    # a batch the workspace was not sized for is refused, not squeezed in
    with pytest.raises(hip.UgkError):
        n = 4 * n_max
        hip.call(fn, ptr(to_dev(np.zeros(n, kdtype))), n, ptr(ws), ws_bytes, epoch + 1, ptr(dev_bytes(n * 8)),
                 ptr(dev_zeros_u32(n)), None, ptr(dev_zeros_u32(1)), None, None)


@pytest.mark.parametrize("mode", ["flat", "hash", "hash32"])
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("n", [1, 63, 64, 65, 4097, 200_000])
def test_nonlocal_flags_and_stable_selection(mode, kdtype, n):
    """the pre-filter in front of an extraction that skips the cache's rows: bit i = key i is not served by the cache
    (found with the host's location, or absent), the set bits compacted in ascending order, the keys picked by them —
    numpy's boolean mask, order kept"""
    rng = np.random.default_rng(n * 3 + (mode == "hash"))
    nkeys = 50_000
    local = rng.choice(nkeys, 15_000, replace=False).astype(kdtype)
    rest = np.setdiff1d(np.arange(nkeys), local)
    on_host = rng.choice(rest, 5_000, replace=False).astype(kdtype)  # present, with the host's location
    if mode == "flat":
        mem, tb = _make_flat(nkeys)
    else:
        mem, tb, _ = (_make_hash32 if mode == "hash32" else _make_hash)(20_000)
    assert _insert(tb, local) == 0
    assert _insert(tb, on_host, offs_np=on_host.astype(np.uint32), loc=1) == 0
    keys = rng.integers(0, nkeys, size=n).astype(kdtype)
    words = (n + 63) // 64
    flags = dev_bytes(words * 8 + 8, fill=0xAB)
    d_keys = to_dev(keys)
    sfx = "i64" if kdtype == np.int64 else "u32"
    hip.call("ugk_nonlocal_flags_" + sfx, tb, ptr(d_keys), n, ptr(flags), None)
    sync()
    want_mask = ~np.isin(keys, local)
    got_words = to_np(flags, np.uint64)[:words]
    got_mask = np.unpackbits(got_words.view(np.uint8), bitorder="little")[:n].astype(bool)
    assert np.array_equal(got_mask, want_mask)
    assert not np.unpackbits(got_words.view(np.uint8), bitorder="little")[n:].any()  # bits past the batch are clear
    assert to_np(flags, np.uint64)[words] == 0xABABABABABABABAB  # nothing written past the bitmap
    ws = dev_bytes(hip.lib().ugk_bitmap_workspace_bytes())
    total = PinnedArray((2,), np.uint32)
    hip.call("ugk_bitmap_count", ptr(flags), None, 0, n, ptr(ws), total.ptr, None)
    sync()
    m = int(total.array[0])
    assert m == int(want_mask.sum())
    if m:
        sel = dev_zeros_u32(m)
        out = dev_bytes(m * np.dtype(kdtype).itemsize)
        hip.call("ugk_bitmap_emit", ptr(flags), None, 0, n, ptr(ws), ptr(sel), m, None)
        hip.call("ugk_select_keys_" + sfx, ptr(d_keys), ptr(sel), m, ptr(out), None)
        sync()
        assert np.array_equal(to_np(sel, np.uint32)[:m], np.nonzero(want_mask)[0])
        assert np.array_equal(to_np(out, kdtype)[:m], keys[want_mask])
    total.free()


def test_classify_with_destination_map():
    """dst_map redirects the output row of key i; sources and group sizes are unchanged"""
    rng = np.random.default_rng(31)
    nkeys = 5000
    cached = rng.choice(nkeys, 1500, replace=False).astype(np.uint32)
    mem, tb = _make_flat(nkeys)
    assert _insert(tb, cached) == 0
    n = 3333
    keys = rng.integers(0, nkeys, size=n).astype(np.uint32)
    dmap = rng.permutation(10 * n)[:n].astype(np.uint32)
    idx0, _, c0, st0, _ = _classify(tb, keys, nkeys)
    idx = dev_bytes(n * 8, fill=0xAB)
    counts = dev_zeros_u32(4)
    st = dev_zeros_u32(1)
    d_keys, d_map = to_dev(keys), to_dev(dmap)
    hip.call("ugk_classify_u32", tb, ptr(d_keys), n, nkeys, ptr(d_map), ptr(idx), ptr(counts), ptr(counts) + 8,
             ptr(st), None, None)
    sync()
    c = to_np(counts, np.uint32)
    assert st0 == 0 and status_value(st) == 0 and c[0] == c0[0] and c[1] == c0[1]
    plain = to_np(idx0, IDX_DTYPE)[:n].copy()
    plain["dst_off"] = dmap[plain["dst_off"]]
    got = to_np(idx, IDX_DTYPE)[:n]

    def canon(a):
        return np.sort(a["dst_off"].astype(np.uint64) << 32 | a["src"].astype(np.uint64))
    assert np.array_equal(canon(got[: c[0]]), canon(plain[: c[0]]))
    assert np.array_equal(canon(got[c[0]:]), canon(plain[c[0]:]))


@pytest.mark.parametrize("row_bytes", [512, 64, 2048, 12, 100])
def test_replicate_rows_fills_duplicates_from_their_representative(row_bytes):
    rng = np.random.default_rng(row_bytes)
    n = 20_011
    keys = rng.integers(0, 3000, size=n)
    uniq, first, inv = np.unique(keys, return_index=True, return_inverse=True)
    table = _rand_table(rng, 3000, row_bytes)
    out = np.full((n, row_bytes), 0xEE, np.uint8)
    out[first] = table[uniq]  # what the gathers leave behind: representatives only
    d_out = to_dev(out)
    d_inv, d_rep = to_dev(inv.astype(np.uint32)), to_dev(first.astype(np.uint32))
    hip.call("ugk_replicate_rows", ptr(d_out), row_bytes, ptr(d_inv), ptr(d_rep), n, None)
    sync()
    assert to_np(d_out)[: n * row_bytes].tobytes() == table[keys].tobytes()
    assert hip.call("ugk_replicate_rows", ptr(d_out), row_bytes, None, None, 0, None) == 0


@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("sparse", [False, True])
@pytest.mark.parametrize("with_bitmap", [False, True])
def test_record_and_drain_match_bincount(kdtype, sparse, with_bitmap):
    """device-side hotness counters: record == numpy.bincount of the rows; drain hands out every non-zero counter
    exactly once as (count << 32 | row) and leaves the counters at zero; the optional bitmap of observed rows is
    "counter above zero" after every launch"""
    rng = np.random.default_rng(17 + sparse)
    num_rows = 100_003
    bits = 31 if kdtype == np.uint32 else 40
    mul = (0x9E3779B97F4A7C15 | 1) & ((1 << bits) - 1) if sparse else 0
    mask = (1 << bits) - 1 if sparse else 0
    inv = pow(mul, -1, 1 << bits) if sparse else 0
    counts = dev_zeros_u32(num_rows)
    observed = to_dev(np.zeros((num_rows + 63) // 64, np.uint64)) if with_bitmap else None

    def observed_rows():
        return np.flatnonzero(np.unpackbits(to_np(observed, np.uint8), bitorder="little"))

    st = dev_zeros_u32(1)
    want = np.zeros(num_rows, np.int64)
    for n in (1, 5000, 200_001):
        rows = (rng.zipf(1.2, size=n) % num_rows).astype(np.uint64)
        keys = ((rows * np.uint64(mul)) & np.uint64(mask)) if sparse else rows
        d_keys = to_dev(keys.astype(kdtype))
        fn = "ugk_record_i64" if kdtype == np.int64 else "ugk_record_u32"
        hip.call(fn, ptr(d_keys), n, inv, mask, ptr(counts), num_rows, ptr(observed), ptr(st), None, None)
        want += np.bincount(rows.astype(np.int64), minlength=num_rows)
        if with_bitmap:
            sync()
            assert np.array_equal(observed_rows(), np.flatnonzero(want))
    sync()
    assert status_value(st) == 0
    assert np.array_equal(to_np(counts, np.uint32)[:num_rows].astype(np.int64), want)

    # drain in two row ranges, the second with a list too short for it (left-over rows come with the next call)
    cap = 30_000
    entries = dev_bytes(cap * 8)
    n_entries = dev_zeros_u32(1)
    out = PinnedArray((2,), np.uint32)
    try:
        got = np.zeros(num_rows, np.int64)
        calls = 0
        for first, cnt in ((0, 50_001), (50_001, num_rows - 50_001)):
            while True:
                hip.call("ugk_record_drain", ptr(counts), first, cnt, ptr(observed), ptr(entries), cap, ptr(n_entries),
                         out.ptr, None)
                sync()
                calls += 1
                if with_bitmap:  # also half-way through: a bit is clear exactly where the counter was reset
                    assert np.array_equal(observed_rows(), np.flatnonzero(to_np(counts, np.uint32)[:num_rows]))
                k, more = int(out.array[0]), int(out.array[1])
                e = to_np(entries, np.uint64)[:k]
                r, c = (e & np.uint64(0xFFFFFFFF)).astype(np.int64), (e >> np.uint64(32)).astype(np.int64)
                assert len(np.unique(r)) == k and (c > 0).all() and ((r >= first) & (r < first + cnt)).all()
                assert (got[r] == 0).all()
                got[r] = c
                if not more:
                    break
                assert k == cap
                assert calls < 20
        assert np.array_equal(got, want)
        assert not to_np(counts, np.uint32)[:num_rows].any()
        assert int(to_np(n_entries, np.uint32)[0]) == 0
    finally:
        out.free()


def test_record_rejects_keys_without_a_row():
    counts = dev_zeros_u32(10)
    st = dev_zeros_u32(1)
    d_keys = to_dev(np.array([3, 10, -1, 3], np.int64))
    hip.call("ugk_record_i64", ptr(d_keys), 4, 0, 0, ptr(counts), 10, None, ptr(st), None, None)
    sync()
    assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE
    assert to_np(counts, np.uint32)[:10].tolist() == [0, 0, 0, 2, 0, 0, 0, 0, 0, 0]


@pytest.mark.parametrize("n_rows,n_entries", [(1, 1), (70, 500), (100_003, 250_000)])
def test_restore_adds_counts_back_and_marks_the_rows_observed(n_rows, n_entries):
    """ugk_record_restore is the way back of a drain: counts[row] += count for (count << 32 | row) words, rows may
    repeat, zero counts change nothing, the observed bit follows "counter above zero"; against numpy add.at"""
    rng = np.random.default_rng(n_rows)
    before = (rng.integers(0, 4, size=n_rows) * (rng.random(n_rows) < 0.3)).astype(np.uint32)
    rows = rng.integers(0, n_rows, size=n_entries).astype(np.uint64)
    cnts = (rng.integers(0, 1000, size=n_entries) * (rng.random(n_entries) < 0.8)).astype(np.uint64)
    words = (n_rows + 63) // 64
    pad = np.zeros(words * 64, bool)
    pad[:n_rows] = before > 0
    counts = to_dev(before)
    observed = to_dev(np.packbits(pad, bitorder="little").view(np.uint64))
    st = dev_zeros_u32(1)
    d_entries = to_dev((cnts << np.uint64(32)) | rows)
    hip.call("ugk_record_restore", ptr(d_entries), n_entries, ptr(counts), n_rows, ptr(observed), ptr(st), None)
    sync()
    assert status_value(st) == 0
    want = before.astype(np.uint64)
    np.add.at(want, rows.astype(np.int64), cnts)
    assert np.array_equal(to_np(counts, np.uint32)[:n_rows], want.astype(np.uint32))
    bits = np.unpackbits(to_np(observed, np.uint8)[: words * 8], bitorder="little")
    assert np.array_equal(bits[:n_rows].astype(bool), want > 0) and not bits[n_rows:].any()
    # what a drain hands over, handed back: the counters are what they were
    if n_rows > 1:
        entries = dev_bytes(n_rows * 8)
        n_out = dev_zeros_u32(1)
        out = PinnedArray((2,), np.uint32)
        try:
            hip.call("ugk_record_drain", ptr(counts), 0, n_rows, ptr(observed), ptr(entries), n_rows, ptr(n_out),
                     out.ptr, None)
            sync()
            k = int(out.array[0])
            assert k == int((want > 0).sum()) and not to_np(counts, np.uint32)[:n_rows].any()
            hip.call("ugk_record_restore", ptr(entries), k, ptr(counts), n_rows, ptr(observed), ptr(st), None)
            sync()
            assert np.array_equal(to_np(counts, np.uint32)[:n_rows], want.astype(np.uint32))
        finally:
            out.free()
    # a row outside the table is flagged and skipped
    bad = to_dev(np.array([(5 << 32) | n_rows], np.uint64))
    hip.call("ugk_record_restore", ptr(bad), 1, ptr(counts), n_rows, None, ptr(st), None)
    sync()
    assert status_value(st) & hip.ST_KEY_OUT_OF_RANGE
    assert np.array_equal(to_np(counts, np.uint32)[:n_rows], want.astype(np.uint32))


@pytest.mark.parametrize("first,cnt", [(0, 1), (1, 1), (3, 2), (1, 3), (2, 7), (5, 64), (7, 257), (0, 0)])
def test_drain_of_short_and_unaligned_row_ranges(first, cnt):
    total = 300
    host = np.arange(1, total + 1, dtype=np.uint32)  # every counter non-zero
    counts = to_dev(host)
    entries = dev_bytes(512 * 8)
    n_entries = dev_zeros_u32(1)
    out = PinnedArray((2,), np.uint32)
    try:
        hip.call("ugk_record_drain", ptr(counts), first, cnt, None, ptr(entries), 512, ptr(n_entries), out.ptr, None)
        sync()
        k = int(out.array[0])
        assert k == cnt and int(out.array[1]) == 0
        e = np.sort(to_np(entries, np.uint64)[:k])
        rows = np.arange(first, first + cnt, dtype=np.uint64)
        assert np.array_equal(e, np.sort(((rows + np.uint64(1)) << np.uint64(32)) | rows))
        left = to_np(counts, np.uint32)[:total]
        want = host.copy()
        want[first:first + cnt] = 0
        assert np.array_equal(left, want)  # nothing outside the range was touched
    finally:
        out.free()
