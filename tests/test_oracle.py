"""Pins every function of the CPU oracle against an independent definition (the reference holds no golden
vectors or unit tests for this path): published known answers, closed forms, numpy routines, brute force."""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import BUCKET_DTYPE, IDX_DTYPE, Oracle, _ptr, sz

ORC = Oracle()
L = ORC.lib
EMPTY = 0xFFFFFFFF


# ---------------------------------------------------------------------------------------------------
# MurmurHash3_x86_32: the published smhasher verification answers
# ---------------------------------------------------------------------------------------------------
MURMUR_KAT = [
    (b"", 0, 0x00000000),
    (b"", 1, 0x514E28B7),
    (b"", 0xFFFFFFFF, 0x81F16F39),
    (b"\xff\xff\xff\xff", 0, 0x76293B50),
    (b"\x21\x43\x65\x87", 0, 0xF55B516B),
    (b"\x21\x43\x65\x87", 0x5082EDEE, 0x2362F9DE),
    (b"\x21\x43\x65", 0, 0x7E4A8634),
    (b"\x21\x43", 0, 0xA0F7B07A),
    (b"\x21", 0, 0x72661CF4),
    (b"\x00\x00\x00\x00", 0, 0x2362F9DE),
    (b"\x00\x00\x00", 0, 0x85F0B427),
    (b"\x00\x00", 0, 0x30F4C306),
    (b"\x00", 0, 0x514E28B7),
    (b"test", 0, 0xBA6BD213),
    (b"test", 0x9747B28C, 0x704B81DC),
    (b"Hello, world!", 0, 0xC0363E43),
    (b"Hello, world!", 0x9747B28C, 0x24884CBA),
    (b"The quick brown fox jumps over the lazy dog", 0, 0x2E4FF723),
    (b"The quick brown fox jumps over the lazy dog", 0x9747B28C, 0x2FA826CD),
]


@pytest.mark.parametrize("data,seed,want", MURMUR_KAT)
def test_murmur3_known_answers(data, seed, want):
    assert L.orc_murmur3_32_bytes(data, len(data), seed) == want


def test_murmur3_u32_is_the_4_byte_little_endian_case():
    assert L.orc_murmur3_32_u32(0, 0) == 0x2362F9DE
    assert L.orc_murmur3_32_u32(0xFFFFFFFF, 0) == 0x76293B50
    assert L.orc_murmur3_32_u32(0x87654321, 0) == 0xF55B516B
    assert L.orc_murmur3_32_u32(0x87654321, 0x5082EDEE) == 0x2362F9DE


# ---------------------------------------------------------------------------------------------------
# TableSize, EmbCacheOff, capacity: closed forms on hand-worked cases
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("num,scale,want", [
    (2, 2, 8),          # log2(1)=0 -> 1<<1 = 2, << 2
    (3, 2, 8),
    (4, 2, 16),         # log2(2)=1 -> 1<<2 = 4
    (100, 2, 256),      # log2(50)=5.64 -> 1<<6 = 64
    (128, 2, 512),      # log2(64)=6 -> 1<<7 = 128
    (129, 2, 512),
    (1000, 2, 2048),    # log2(500)=8.97 -> 1<<9 = 512
    (1 << 20, 2, 1 << 22),
    (25_000_000, 2, 1 << 26),  # log2(12.5M)=23.58 -> 1<<24, <<2
    (100, 1, 128),
])
def test_table_size(num, scale, want):
    assert L.orc_table_size(num, scale) == want


def test_table_size_is_next_pow2_strictly_above_half():
    for n in range(2, 5000):
        p = L.orc_table_size(n, 0)
        assert p & (p - 1) == 0
        assert p > n // 2 and p <= 2 * (n // 2)


def test_pack_unpack():
    for loc, off in [(0, 0), (1, 5), (15, 0x0FFFFFFF), (8, 123456), (1, 0x0ABCDEF0)]:
        p = L.orc_pack(loc, off)
        assert p == ((loc << 28) + off) & 0xFFFFFFFF
        assert L.orc_loc(p) == loc and L.orc_off(p) == off


@pytest.mark.parametrize("n,pct,want", [
    (1000, 0.25, 251),                 # 1000 * 0.251
    (1_000_000, 0.10, 101_000),
    (100_000_000, 0.25, 25_100_000),
    (10, 0.5, 5),                      # 10 * 0.501 = 5.01
    (7, 0.3, 2),                       # 7 * 0.301 = 2.107
])
def test_cache_capacity(n, pct, want):
    assert L.orc_cache_capacity(n, pct) == want


# ---------------------------------------------------------------------------------------------------
# gather: numpy.take and a brute-force loop
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dim,dtype", [(128, np.float32), (64, np.float16), (1, np.float32), (25, np.float32),
                                       (3, np.uint8)])
@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
@pytest.mark.parametrize("omp", [False, True])
def test_gather_equals_numpy_take(dim, dtype, kdtype, omp):
    rng = np.random.default_rng(7)
    table = rng.integers(0, 255, size=(997, dim * np.dtype(dtype).itemsize), dtype=np.uint8).view(dtype)
    keys = rng.integers(0, 997, size=4099).astype(kdtype)
    got = ORC.gather(table, keys, omp=omp)
    want = np.take(table, keys.astype(np.int64), axis=0)
    assert got.tobytes() == want.tobytes()
    # brute force on a prefix
    for i in range(50):
        assert got[i].tobytes() == table[int(keys[i])].tobytes()


def test_gather_empty_and_edges():
    table = np.arange(40, dtype=np.float32).reshape(10, 4)
    assert ORC.gather(table, np.zeros(0, np.uint32)).shape == (0, 4)
    got = ORC.gather(table, np.array([9, 0, 9, 9], np.int64))
    assert np.array_equal(got, table[[9, 0, 9, 9]])
    with pytest.raises(IndexError):
        ORC.gather(table, np.array([10], np.uint32))
    with pytest.raises(IndexError):
        ORC.gather(table, np.array([-1], np.int64))


def test_gather_scatter():
    rng = np.random.default_rng(3)
    table = rng.standard_normal((100, 8)).astype(np.float32)
    keys = rng.permutation(100)[:30].astype(np.uint32)
    dst = rng.permutation(50)[:30].astype(np.uint32)
    out = np.zeros((50, 8), np.float32)
    L.orc_gather_scatter_u32(_ptr(table), keys, dst, 30, _ptr(out), 32)
    want = np.zeros((50, 8), np.float32)
    want[dst] = table[keys]
    assert out.tobytes() == want.tobytes()


# ---------------------------------------------------------------------------------------------------
# tables: dict-model invariants
# ---------------------------------------------------------------------------------------------------
def _rand_unique(rng, n, hi):
    return rng.choice(hi, size=n, replace=False).astype(np.uint32)


@pytest.mark.parametrize("n", [2, 17, 1000, 20000])
def test_simple_table_against_dict(n):
    rng = np.random.default_rng(n)
    keys = _rand_unique(rng, n, 1 << 30)
    vals = (rng.integers(0, 1 << 28, size=n).astype(np.uint32))
    t = ORC.simple_table(n)
    assert len(t) == L.orc_table_size(n, 2)
    assert ORC.simple_census(t) == (0, 0, len(t))
    assert ORC.simple_insert(t, keys, vals) == 0
    model = dict(zip(keys.tolist(), vals.tolist()))
    for k in keys[:500]:
        pos = ORC.simple_search(t, k)
        assert pos != EMPTY and t[pos]["val"] == model[int(k)] and t[pos]["state_key"] == k
    absent = _rand_unique(rng, 300, 1 << 30)
    for k in absent:
        if int(k) not in model:
            assert ORC.simple_search(t, k) == EMPTY
    assert ORC.simple_census(t) == (n, 0, len(t) - n)
    # duplicate insert is the reference's assert
    assert ORC.simple_insert(t, keys[:1], vals[:1]) == -1
    # evict half: tombstones keep the key, searches miss, census moves occupied -> invalid
    ev = keys[: n // 2]
    assert ORC.simple_evict(t, ev) == 0
    for k in ev[:200]:
        assert ORC.simple_search(t, k) == EMPTY
    for k in keys[n // 2:][:200]:
        assert ORC.simple_search(t, k) != EMPTY
    assert ORC.simple_census(t) == (n - n // 2, n // 2, len(t) - n)
    assert ORC.simple_evict(t, ev[:1]) == -1  # already gone
    # re-insert after evict succeeds and is found with the new value
    assert ORC.simple_insert(t, ev, np.full(len(ev), 42, np.uint32)) == 0
    for k in ev[:200]:
        pos = ORC.simple_search(t, k)
        assert pos != EMPTY and t[pos]["val"] == 42
    occ, inv, dflt = ORC.simple_census(t)
    assert occ == n and occ + inv + dflt == len(t)


def test_simple_probe_sequence_matches_definition():
    """first bucket = murmur(key) % size, then pos = murmur(pos + delta) % size with delta = 1, 2, ...
    (cache_hashtable.cuh:175-190), restated here in Python on top of the pinned hash."""
    n = 64
    rng = np.random.default_rng(1)
    keys = _rand_unique(rng, n, 1 << 20)
    t = ORC.simple_table(n)
    nb = len(t)
    py = {}  # pos -> key
    for k in keys.tolist():
        pos = L.orc_murmur3_32_u32(k, 0) % nb
        delta = 1
        while pos in py:
            pos = L.orc_murmur3_32_u32((pos + delta) & 0xFFFFFFFF, 0) % nb
            delta += 1
        py[pos] = k
    ORC.simple_insert(t, keys, np.arange(n, dtype=np.uint32))
    for pos, k in py.items():
        assert t[pos]["state_key"] == k
        assert ORC.simple_search(t, k) == pos


def test_flat_table_and_lookup_rule():
    rng = np.random.default_rng(5)
    nkeys = 5000
    cached = _rand_unique(rng, 1200, nkeys)
    vals = np.array([L.orc_pack(0, i) for i in range(len(cached))], np.uint32)
    flat = ORC.flat_table(nkeys)
    assert (flat == EMPTY).all()
    L.orc_flat_insert(flat, cached, vals, len(cached))
    simple = ORC.simple_table(len(cached))
    ORC.simple_insert(simple, cached, vals)
    q = rng.integers(0, nkeys, size=3000).astype(np.uint32)
    model = dict(zip(cached.tolist(), vals.tolist()))
    for tbl in ({"flat": flat}, {"simple": simple}):
        idx = ORC.lookup_src_dst(q, fallback_loc=1, **tbl)
        assert np.array_equal(idx["dst_off"], np.arange(len(q), dtype=np.uint32))
        want = np.array([model.get(int(k), (1 << 28) + int(k)) for k in q], np.uint32)
        assert np.array_equal(idx["src"], want)
    ev = cached[:100]
    L.orc_flat_evict(flat, ev, len(ev))
    assert (flat[ev] == EMPTY).all()


# ---------------------------------------------------------------------------------------------------
# sort + boundaries
# ---------------------------------------------------------------------------------------------------
def test_sort_is_ascending_u64_and_boundaries_are_bincount():
    rng = np.random.default_rng(11)
    for n, nloc in [(0, 2), (1, 2), (1000, 2), (5000, 4)]:
        idx = np.empty(n, IDX_DTYPE)
        idx["dst_off"] = np.arange(n, dtype=np.uint32)
        loc = rng.integers(0, nloc, size=n).astype(np.uint32)
        off = rng.integers(0, 1 << 28, size=n).astype(np.uint32)
        idx["src"] = (loc << 28) + off
        words = idx.view(np.uint64).copy()
        assert np.array_equal(words, (idx["src"].astype(np.uint64) << 32) | idx["dst_off"])
        ORC.sort_idx(idx)
        assert np.array_equal(idx.view(np.uint64), np.sort(words))
        g = ORC.find_boundary(idx, nloc)
        want = np.concatenate([[0], np.cumsum(np.bincount(loc, minlength=nloc))]).astype(np.uint32)
        if n > 0:
            # the reference leaves group_offset[1] at 0 when location 0 is empty and patches only i >= 1
            assert np.array_equal(g, want)
        assert g[nloc] == n


def test_boundary_empty_groups():
    # all entries from the host (loc 1): group 0 empty
    idx = np.empty(5, IDX_DTYPE)
    idx["dst_off"] = np.arange(5)
    idx["src"] = (1 << 28) + np.arange(5)
    assert ORC.find_boundary(idx, 2).tolist() == [0, 0, 5]
    idx["src"] = np.arange(5)  # all local
    assert ORC.find_boundary(idx, 2).tolist() == [0, 5, 5]
    # 3 locations, middle one empty -> fix-up loop copies the previous offset
    idx["src"] = np.array([0, 0, (2 << 28), (2 << 28) + 1, (2 << 28) + 2], np.uint32)
    assert ORC.find_boundary(idx, 3).tolist() == [0, 2, 2, 5]


# ---------------------------------------------------------------------------------------------------
# whole extraction = table[keys]
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode", ["flat", "simple"])
@pytest.mark.parametrize("row", [(128, np.float32), (64, np.float16)])
def test_extract_feat_equals_table_take(mode, row):
    dim, dt = row
    rng = np.random.default_rng(21)
    nkeys = 4000
    host = rng.integers(0, 255, size=(nkeys, dim * np.dtype(dt).itemsize), dtype=np.uint8).view(dt)
    cached = _rand_unique(rng, 900, nkeys)
    cache = np.zeros((1000, dim), dt)  # capacity > cached, slots [900,1000) unused
    cache[: len(cached)] = host[cached]
    vals = np.arange(len(cached), dtype=np.uint32)  # loc 0, slot i
    if mode == "flat":
        tbl = {"flat": ORC.flat_table(nkeys)}
        L.orc_flat_insert(tbl["flat"], cached, vals, len(cached))
    else:
        tbl = {"simple": ORC.simple_table(len(cached))}
        ORC.simple_insert(tbl["simple"], cached, vals)
    keys = rng.integers(0, nkeys, size=3001).astype(np.uint32)
    out, g = ORC.extract_feat(keys, cache, host, **tbl)
    assert out.tobytes() == host[keys].tobytes()
    nhit = int(np.isin(keys, cached).sum())
    assert g.tolist() == [0, nhit, len(keys)]
    # poisoned cache rows prove hits really come from the cache
    cache2 = cache.copy()
    cache2[: len(cached)] = 0
    out2, _ = ORC.extract_feat(keys, cache2, host, **tbl)
    hit = np.isin(keys, cached)
    assert (out2[hit] == 0).all() and out2[~hit].tobytes() == host[keys[~hit]].tobytes()


def test_extract_mix_equals_grouped():
    rng = np.random.default_rng(2)
    host = rng.standard_normal((300, 16)).astype(np.float32)
    cache = rng.standard_normal((50, 16)).astype(np.float32)
    n = 200
    idx = np.empty(n, IDX_DTYPE)
    idx["dst_off"] = rng.permutation(n)
    loc = rng.integers(0, 2, n).astype(np.uint32)
    off = np.where(loc == 0, rng.integers(0, 50, n), rng.integers(0, 300, n)).astype(np.uint32)
    idx["src"] = (loc << 28) + off
    out = np.zeros((n, 16), np.float32)
    srcs = (C.c_void_p * 2)(cache.ctypes.data, host.ctypes.data)
    L.orc_extract_mix(_ptr(idx), n, srcs, _ptr(out), 64)
    want = np.zeros_like(out)
    want[idx["dst_off"]] = np.where((loc == 0)[:, None], cache[np.minimum(off, 49)], host[off])
    assert out.tobytes() == want.tobytes()


# ---------------------------------------------------------------------------------------------------
# hotness ranking, placement, refresh, dedup
# ---------------------------------------------------------------------------------------------------
def test_freq_rank_is_count_desc_then_key_desc():
    rng = np.random.default_rng(9)
    stream = (rng.zipf(1.3, size=20000) % 500).astype(np.uint32)
    rk, rc = ORC.freq_rank(stream)
    keys, cnts = np.unique(stream, return_counts=True)
    order = np.lexsort((-keys.astype(np.int64), -cnts.astype(np.int64)))  # primary: count desc, then key desc
    assert np.array_equal(rk, keys[order]) and np.array_equal(rc, cnts[order])
    # hand-worked: counts {5:2, 7:2, 1:3, 9:1} -> 1, 7, 5, 9
    rk, rc = ORC.freq_rank(np.array([5, 7, 1, 1, 5, 7, 1, 9], np.uint32))
    assert rk.tolist() == [1, 7, 5, 9] and rc.tolist() == [3, 2, 2, 1]
    assert ORC.freq_rank(np.zeros(0, np.uint32))[0].size == 0


def test_rep_solve_takes_the_first_floor_n_pct_ranks():
    rank = np.array([4, 2, 9, 0, 1, 3, 5, 6, 7, 8], np.uint32)
    nid, nc = ORC.rep_solve(rank, 10, 30.0)
    assert nc == 3 and np.nonzero(nid == 0)[0].tolist() == [2, 4, 9]
    nid, nc = ORC.rep_solve(rank, 10, 25.0)  # floor(2.5)
    assert nc == 2 and np.nonzero(nid == 0)[0].tolist() == [2, 4]
    nid, nc = ORC.rep_solve(rank, 10, 0.0)
    assert nc == 0 and (nid == 1).all()
    nid, nc = ORC.rep_solve(rank, 10, 100.0)
    assert nc == 10 and (nid == 0).all()


def test_refresh_plan_set_algebra_and_free_list():
    rng = np.random.default_rng(13)
    n = 2000
    cap = 700
    old_local = set(rng.choice(n, 600, replace=False).tolist())
    new_local = set(rng.choice(n, 620, replace=False).tolist())
    old_block = np.array([0 if k in old_local else 1 for k in range(n)], np.uint32)
    new_block = np.array([0 if k in new_local else 1 for k in range(n)], np.uint32)
    slot_of = np.full(n, EMPTY, np.uint32)
    for s, k in enumerate(sorted(old_local)):
        slot_of[k] = s
    free = np.zeros(cap + n, np.uint32)
    free[: cap - 600] = np.arange(600, cap)
    n_free = sz(cap - 600)
    ev = np.zeros(n, np.uint32)
    ins = np.zeros(n, np.uint32)
    ins_slot = np.zeros(n, np.uint32)
    ne, ni = sz(0), sz(0)
    slot_before = slot_of.copy()
    rc = L.orc_refresh_plan(old_block, new_block, n, slot_of, free, C.byref(n_free), ev, C.byref(ne), ins,
                            ins_slot, C.byref(ni))
    assert rc == 0
    assert set(ev[: ne.value].tolist()) == old_local - new_local
    assert set(ins[: ni.value].tolist()) == new_local - old_local
    # conservation: free + cached == capacity, slots unique
    cached_slots = slot_of[slot_of != EMPTY]
    assert len(cached_slots) == len(new_local) == len(set(cached_slots.tolist()))
    assert n_free.value + len(cached_slots) == cap
    assert set(free[: n_free.value].tolist()).isdisjoint(cached_slots.tolist())
    # preserved keys keep their slot
    for k in old_local & new_local:
        assert slot_of[k] == slot_before[k]
    # inserted keys take the front of [old free list ++ evicted slots]
    want_front = list(range(600, cap)) + [int(slot_before[k]) for k in ev[: ne.value]]
    assert ins_slot[: ni.value].tolist() == want_front[: ni.value]


def test_refresh_plan_rejects_overflow():
    # 3 cached out of capacity 3, the new placement wants a 4th without evicting: the reference CHECKs
    old_block = np.array([0, 0, 0, 1, 1], np.uint32)
    new_block = np.array([0, 0, 0, 0, 1], np.uint32)
    slot_of = np.array([0, 1, 2, EMPTY, EMPTY], np.uint32)
    free = np.zeros(16, np.uint32)
    n_free, ne, ni = sz(0), sz(0), sz(0)
    tmp = [np.zeros(5, np.uint32) for _ in range(3)]
    assert L.orc_refresh_plan(old_block, new_block, 5, slot_of, free, C.byref(n_free), tmp[0], C.byref(ne), tmp[1],
                              tmp[2], C.byref(ni)) == -1


def test_dedup_matches_numpy_unique():
    rng = np.random.default_rng(17)
    for n in (0, 1, 1000, 50000):
        keys = (rng.zipf(1.2, size=n) % (1 << 40)).astype(np.int64) * 1_000_003
        uniq, inv = ORC.dedup(keys)
        assert np.array_equal(uniq[inv], keys)
        nu, first = np.unique(keys, return_index=True)
        assert np.array_equal(np.sort(uniq), nu)
        assert np.array_equal(uniq, keys[np.sort(first)])  # first-occurrence order


def test_pool_hand_worked_and_against_numpy():
    """orc_pool_f64 against the definition of embedding_lookup_sparse's combiners: hand-worked segments (an empty one,
    weights that cancel), then numpy.add.at over random ragged segments"""
    table = np.array([[r, 10.0 * r] for r in range(6)])
    ids, off = np.array([1, 2, 3, 4, 4]), np.array([0, 2, 3, 3, 5])
    w = np.array([1.0, 2.0, 3.0, 1.0, -1.0])
    assert ORC.pool(table, ids, off, None, "sum").tolist() == [[3, 30], [3, 30], [0, 0], [8, 80]]
    assert ORC.pool(table, ids, off, w, "sum").tolist() == [[5, 50], [9, 90], [0, 0], [0, 0]]
    assert ORC.pool(table, ids, off, None, "mean").tolist() == [[1.5, 15], [3, 30], [0, 0], [4, 40]]
    assert np.allclose(ORC.pool(table, ids, off, w, "mean"), [[5 / 3, 50 / 3], [3, 30], [0, 0], [0, 0]], rtol=1e-15)
    assert np.allclose(ORC.pool(table, ids, off, w, "sqrtn"),
                       [[5 / 5 ** 0.5, 50 / 5 ** 0.5], [3, 30], [0, 0], [0, 0]], rtol=1e-15)
    assert np.allclose(ORC.pool(table, ids, off, None, "sqrtn"),
                       [[3 / 2 ** 0.5, 30 / 2 ** 0.5], [3, 30], [0, 0], [8 / 2 ** 0.5, 80 / 2 ** 0.5]], rtol=1e-15)
    with pytest.raises(IndexError):
        ORC.pool(table, np.array([1, 6]), np.array([0, 2]), None, "sum")
    rng = np.random.default_rng(23)
    table = rng.standard_normal((500, 7))
    lens = rng.integers(0, 9, size=300)
    off = np.concatenate([[0], np.cumsum(lens)])
    ids = rng.integers(0, 500, size=off[-1])
    w = rng.random(off[-1]) + 0.1
    seg = np.repeat(np.arange(300), lens)
    for weights in (None, w):
        ww = np.ones(len(ids)) if weights is None else weights
        total = np.zeros((300, 7))
        np.add.at(total, seg, table[ids] * ww[:, None])
        den1, den2 = np.zeros(300), np.zeros(300)
        np.add.at(den1, seg, ww)
        np.add.at(den2, seg, ww * ww)
        assert np.allclose(ORC.pool(table, ids, off, weights, 0), total, rtol=1e-13, atol=1e-13)
        safe = lambda d: np.where(d != 0, d, 1.0)[:, None]
        assert np.allclose(ORC.pool(table, ids, off, weights, 1), np.where(den1[:, None] != 0, total / safe(den1), 0),
                           rtol=1e-13, atol=1e-13)
        assert np.allclose(ORC.pool(table, ids, off, weights, 2),
                           np.where(den2[:, None] != 0, total / safe(np.sqrt(den2)), 0), rtol=1e-13, atol=1e-13)


def test_oracle_reproduces_the_committed_golden_case():
    """tests/golden/extract_small.json was written by brute-force Python loops (tests/golden/make_fixtures.py), not
    by the oracle: ranking, placement, capacity and the gather must all land on it"""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "extract_small.json")) as f:
        g = json.load(f)
    n_item, pct = g["n_item"], g["cache_percentage"]
    stream = np.array(g["record_stream"], np.uint32)
    rk, rc = ORC.freq_rank(stream)
    assert rk.tolist() == g["rank_keys_observed"] and rc.tolist() == g["rank_counts_observed"]
    full_k, _ = ORC.full_rank(stream, n_item)
    nid, n_cached = ORC.rep_solve(full_k, n_item, pct * 100)
    assert np.nonzero(nid == 0)[0].tolist() == g["cached_keys"] and n_cached == len(g["cached_keys"])
    assert ORC.lib.orc_cache_capacity(n_item, pct) == g["capacity_rows"]
    table = np.array(g["table"], np.uint8)
    keys = np.array(g["lookup_keys"], np.int64)
    assert ORC.gather(table, keys).tolist() == g["expected_output"]
    assert [0, int((nid[keys] == 0).sum()), len(keys)] == g["expected_group_offset"]


def test_extract_flat_picks_the_source_per_row_like_numpy_where():
    """orc_extract_flat_i64_omp (the mixed-source step of bench.py's CPU leg): a row comes from the cache copy exactly
    when the flat table names a slot for it, from the host table otherwise.  The cache copy holds different bytes from
    the host rows here, so a wrong source, a wrong slot or a transposed argument shows; slots are a permutation, so
    slot != position in the list of cached rows.  Sparse ids: the row of an id by a brute-force search for the
    multiplier's inverse instead of a formula."""
    rng = np.random.default_rng(21)
    n_rows, rb, n_cached = 3000, 48, 700
    host = rng.integers(0, 256, size=(n_rows, rb), dtype=np.uint8)
    cached_rows = rng.choice(n_rows, n_cached, replace=False)
    slots = rng.permutation(n_cached + 50)[:n_cached]
    cache = rng.integers(0, 256, size=(n_cached + 50, rb), dtype=np.uint8)  # NOT the host rows
    flat = np.full(n_rows, 0xFFFFFFFF, np.uint32)
    flat[cached_rows] = slots  # location 0 in the top four bits
    keys = rng.integers(0, n_rows, size=5000)
    slot_of = np.full(n_rows, -1, np.int64)
    slot_of[cached_rows] = slots
    want = np.where((slot_of[keys] >= 0)[:, None], cache[np.maximum(slot_of[keys], 0)], host[keys])
    got, counts = ORC.extract_flat(flat, keys, cache, host)
    assert got.tobytes() == want.tobytes()
    assert counts == [int((slot_of[keys] >= 0).sum()), int((slot_of[keys] < 0).sum())]
    # a table entry of another location than 0 reads from the host table
    flat2 = flat.copy()
    flat2[cached_rows[:10]] = (1 << 28) + 5
    slot2 = slot_of.copy()
    slot2[cached_rows[:10]] = -1
    want2 = np.where((slot2[keys] >= 0)[:, None], cache[np.maximum(slot2[keys], 0)], host[keys])
    assert ORC.extract_flat(flat2, keys, cache, host)[0].tobytes() == want2.tobytes()
    # sparse ids: id = (row * mul) mod 2^bits; the inverse found by search on a small modulus
    bits, mul = 12, 0x9E3779B97F4A7C15 & 0xFFF | 1
    mask = (1 << bits) - 1
    inv = next(x for x in range(1, 1 << bits, 2) if (x * mul) & mask == 1)
    rows_b = rng.integers(0, n_rows, size=2000)
    ids = (rows_b * mul) & mask
    got3, _ = ORC.extract_flat(flat, ids, cache, host, key_inv=inv, key_mask=mask)
    want3 = np.where((slot_of[rows_b] >= 0)[:, None], cache[np.maximum(slot_of[rows_b], 0)], host[rows_b])
    assert got3.tobytes() == want3.tobytes()
    # keys without a row, and a slot outside the cache copy, are refused
    with pytest.raises(IndexError):
        ORC.extract_flat(flat, np.array([n_rows]), cache, host)
    with pytest.raises(IndexError):
        ORC.extract_flat(flat, np.array([-1]), cache, host)
    with pytest.raises(IndexError):
        ORC.extract_flat(flat, np.array([mask + 1]), cache, host, key_inv=inv, key_mask=mask)
    flat3 = flat.copy()
    flat3[cached_rows[0]] = len(cache)
    with pytest.raises(IndexError):
        ORC.extract_flat(flat3, np.array([cached_rows[0]]), cache, host)


def test_pool_with_max_norm_on_hand_worked_rows_and_against_numpy():
    """orc_pool_clip_f64: every looked-up row is clipped to the l2 norm max_norm before it is weighted.  Hand-worked:
    (3, 4) has norm 5, so max_norm 2.5 halves it and max_norm 10 leaves it alone; (0.6, 0.8) has norm 1 and is never
    touched; a zero row stays zero.  The denominator of mean / sqrtn is made of the weights alone."""
    table = np.array([[3.0, 4.0], [0.6, 0.8], [0.0, 0.0], [-6.0, 8.0]])
    ids = np.array([0, 1, 2, 3, 0])
    off = np.array([0, 2, 3, 5])
    w = np.array([1.0, 2.0, 5.0, 1.0, 3.0])
    got = ORC.pool(table, ids, off, None, "sum", max_norm=2.5)
    assert np.allclose(got, [[1.5 + 0.6, 2.0 + 0.8], [0, 0], [-1.5 + 1.5, 2.0 + 2.0]], rtol=0, atol=1e-15)
    got = ORC.pool(table, ids, off, w, "sum", max_norm=2.5)
    assert np.allclose(got, [[1.5 + 1.2, 2.0 + 1.6], [0, 0], [-1.5 + 4.5, 2.0 + 6.0]], rtol=0, atol=1e-15)
    got = ORC.pool(table, ids, off, w, "mean", max_norm=2.5)  # divided by 3, 5 and 4: the weights, not the clipped ones
    assert np.allclose(got, [[2.7 / 3, 3.6 / 3], [0, 0], [3.0 / 4, 8.0 / 4]], rtol=0, atol=1e-15)
    got = ORC.pool(table, ids, off, w, "sqrtn", max_norm=2.5)
    assert np.allclose(got, [[2.7 / 5 ** 0.5, 3.6 / 5 ** 0.5], [0, 0], [3.0 / 10 ** 0.5, 8.0 / 10 ** 0.5]], atol=1e-15)
    assert np.array_equal(ORC.pool(table, ids, off, w, "sum", max_norm=10.0), ORC.pool(table, ids, off, w, "sum"))
    assert np.array_equal(ORC.pool(table, ids, off, w, "sum", max_norm=None), ORC.pool(table, ids, off, w, "sum"))
    # against numpy on random segments
    rng = np.random.default_rng(12)
    table = rng.standard_normal((400, 9)) * rng.uniform(0.1, 4.0, size=(400, 1))
    lens = rng.integers(0, 7, size=200)
    off = np.concatenate([[0], np.cumsum(lens)])
    ids = rng.integers(0, 400, size=off[-1])
    w = rng.random(off[-1]) + 0.1
    seg = np.repeat(np.arange(200), lens)
    for max_norm in (0.5, 3.0):
        norms = np.linalg.norm(table, axis=1, keepdims=True)
        clipped = table * (max_norm / np.maximum(norms, max_norm))
        assert (np.linalg.norm(clipped, axis=1) <= max_norm * (1 + 1e-12)).all()
        total = np.zeros((200, 9))
        np.add.at(total, seg, clipped[ids] * w[:, None])
        den = np.zeros(200)
        np.add.at(den, seg, w)
        assert np.allclose(ORC.pool(table, ids, off, w, 0, max_norm=max_norm), total, rtol=1e-13, atol=1e-13)
        want = np.where(den[:, None] != 0, total / np.where(den != 0, den, 1.0)[:, None], 0)
        assert np.allclose(ORC.pool(table, ids, off, w, 1, max_norm=max_norm), want, rtol=1e-13, atol=1e-13)
