"""GPU parity tests through the drop-in boundary: the `collcache.torch` surface over libcoll_cache.so, used in the
reference's call order (config -> record_init -> record* -> create_emb_shm -> init_t -> lookup*, see
example/gnn/dgl_sample.py:238-259 of the reference) and checked bit-for-bit against the CPU oracle."""
import os
import sys
import threading
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))

from oracle_lib import Oracle  # noqa: E402

ORC = Oracle()

if torch.cuda.is_available():
    import collcache.torch as co
    from collcache.common import _basics, kLogL1FeatureBytes, kLogL1MissBytes, kLogL2CacheCopyTime


def zipf_ranks(rng, n, space, s):
    """bounded-Pareto inverse CDF used for the synthetic hotness (ranks in [0, space))"""
    u = rng.random(n)
    h = float(space)
    r = np.floor(((h ** (1 - s) - 1) * u + 1) ** (1 / (1 - s))).astype(np.int64)
    return np.clip(r - 1, 0, space - 1)


def make_config(num_total_item, pct, threads=8):
    return {"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
            "num_global_step_per_epoch": 100, "num_epoch": 1, "num_total_item": num_total_item,
            "omp_thread_num": threads}


@pytest.fixture(autouse=True)
def _fresh_cache(monkeypatch):
    for v in ("COLL_HASH_TABLE", "COLL_RECORD_INLINE_BYTES", "SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", "SAMGRAPH_COLL_CACHE_NO_GROUP",
              "COLL_DEDUP_KEYS", "COLL_DEDUP_MIN_KEYS", "COLL_GPU_RECORD", "COLL_GPU_RECORD_EVERY", "COLL_GPU_REFRESH",
              "COLL_GPU_REFRESH_KEEP", "COLL_GPU_REFRESH_STABLE", "COLL_REFRESH_RATE_GBPS",
              "COLL_GPU_RECORD_SEED", "COLL_DEVICE_KEY_LIST"):
        monkeypatch.delenv(v, raising=False)
    yield
    if torch.cuda.is_available():
        co.coll_torch_shutdown()


def fill_table(emb, rng):
    a = emb.numpy()
    a.view(np.uint8)[...] = rng.integers(0, 256, size=a.view(np.uint8).shape, dtype=np.uint8)
    if a.dtype == np.float32:
        # keep the bit patterns, but avoid NaN payload surprises in printing only; bytes are compared anyway
        pass
    return a


def expected_cached_set(stream_u32, n_item, pct):
    rank_k, _ = ORC.full_rank(stream_u32, n_item)
    nid, nc = ORC.rep_solve(rank_k, n_item, pct * 100)
    return np.nonzero(nid == 0)[0].astype(np.uint32), nid


def lookup_bytes(keys_t, n_item, pad=True):
    out = co.coll_torch_lookup_key_t_val_ret(0, keys_t, pad)
    return out


@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("pct", [1.0, 0.0])
def test_direct_mapping_full_and_no_cache(kdtype, pct):
    rng = np.random.default_rng(1)
    n_item, dim = 20_000, 128
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["table_kind"] == 0 and info["row_bytes"] == dim * 4
    for n in (1, 13, 4096, 30_001):
        keys = rng.integers(0, n_item, size=n)
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, True)
        assert out.shape == ((n + 7) // 8 * 8, dim) and out.dtype == torch.float32 and out.is_cuda
        got = out[:n].cpu().numpy()
        assert got.tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        g = _basics.last_group_offset(0)
        assert g == ([0, n, n] if pct == 1.0 else [0, 0, n])
        out2 = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out2.shape == (n, dim)
        assert out2.data_ptr() == out.data_ptr() or n > 4096  # one reused buffer unless it had to grow
    # profiler hooks of the lookup
    assert _basics.step_value(0, kLogL1FeatureBytes) == 1 * dim * 4
    assert _basics.step_value(0, kLogL2CacheCopyTime) > 0
    assert _basics.info(0)["lookups"] == 8


@pytest.mark.parametrize("pct", [1.0, 0.0, 0.3])
def test_build_of_every_replica_with_an_allocator_builder(pct):
    """CollCache::build(allocator_builder, ...) (facade.h:52-54, facade.cc:38-72) through its C hook: every replica
    (the one) is built with the allocator the builder makes for it, from the placement the object holds.  A partial
    cache is first built by coll_cache_init, then rebuilt the reference's way from the same placement."""
    import ctypes
    from collcache.torch import c_lib
    rng = np.random.default_rng(3)
    n_item, dim = 30_000, 64
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 60_000, n_item, 1.1)]
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    nid = None
    if 0.0 < pct < 1.0:
        co.coll_torch_record(0, torch.from_numpy(s0))
        co.coll_torch_init_t(0, 0, emb, pct)  # solves the placement
        _, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    else:
        c_lib._State.dev_id[0] = 0
        c_lib._setup_dims(dim, False)
    handed_out = []
    alloc, release = c_lib._make_allocator(0)

    def counting_alloc(nbytes, user):
        handed_out.append(nbytes)
        return alloc(nbytes, user)

    cb = c_lib.ALLOC_FN(counting_alloc)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _basics.C_LIB_CTYPES.coll_cache_build_all_c(cb, release, None, emb.data_ptr(), co.kF32, dim, pct, stream)
    info = _basics.info(0)
    assert info["cached_rows"] == (n_item if pct == 1.0 else 0 if pct == 0.0 else int((nid == 0).sum()))
    for n in (1, 5000, 40_000):
        keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
        want_local = n if pct == 1.0 else 0 if pct == 0.0 else int((nid[keys] == 0).sum())
        assert _basics.last_group_offset(0) == [0, want_local, n]
    if 0.0 < pct < 1.0:
        # the fused extraction needs no scratch; the set of a distinct-keys lookup comes from the builder's allocator
        assert not handed_out
        keys = perm[zipf_ranks(rng, 5000, n_item, 1.1)]
        rows, inverse = co.coll_torch_lookup_unique(0, torch.from_numpy(keys).cuda())
        assert rows[inverse.long()].cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
        assert handed_out


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH", "HASH16"])
@pytest.mark.parametrize("impl", ["", "SMMaskPhase", "DIRECT", "NONE"])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_partial_cache_matches_oracle(table_kind, impl, kdtype, monkeypatch):
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    rng = np.random.default_rng(7)
    n_item, dim, pct = 50_000, 128, 0.1
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    stream = []
    for _ in range(4):  # presample epochs
        keys = perm[zipf_ranks(rng, 40_000, n_item, 1.1)]
        stream.append(keys)
        co.coll_torch_record(0, torch.from_numpy(keys).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)

    want_cached, nid = expected_cached_set(np.concatenate(stream).astype(np.uint32), n_item, pct)
    info = _basics.info(0)
    assert info["table_kind"] == {"FLAT": 1, "HASH": 3, "HASH16": 2}[table_kind]  # HASH: 8-byte entries when they fit
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct)
    assert info["cached_rows"] == len(want_cached) == int(n_item * (pct * 100 / 100.0))
    assert info["free_slots"] == info["capacity_rows"] - info["cached_rows"]
    got_cached = np.zeros(len(want_cached), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got_cached.ctypes.data, len(got_cached)) == len(want_cached)
    assert np.array_equal(got_cached, want_cached)

    for n in (1, 1000, 65_536):
        keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        n_local = int((nid[keys] == 0).sum())
        assert _basics.last_group_offset(0) == [0, n_local, n]
    step = _basics.info(0)["lookups"] - 1
    assert _basics.step_value(step, kLogL1MissBytes) == (n - n_local) * dim * 4


@pytest.mark.parametrize("key_list", ["device", "host"])
@pytest.mark.parametrize("table_kind,sparse", [("FLAT", False), ("HASH", False), ("HASH", True), ("HASH16", True)])
@pytest.mark.parametrize("pct", [0.003, 0.1, 0.7])
def test_key_list_of_a_build_made_on_the_device_or_on_the_host(key_list, table_kind, sparse, pct, monkeypatch):
    """The ascending list of cached rows comes from a bitmap on the device (the default) or from the key -> block
    array on the host (COLL_DEVICE_KEY_LIST=0): the same cached set either way, the oracle's, with fewer rows observed
    than the cache holds (0.7: the lowest never-observed rows fill it up), with more (0.003, 0.1: the best-ranked
    ones), and a refresh through the host afterwards starts from the right list."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_DEVICE_KEY_LIST", "1" if key_list == "device" else "0")
    rng = np.random.default_rng(int(pct * 1000) + len(table_kind))
    n_item, dim = 70_003, 32
    MUL, BITS = 0x9E3779B97F4A7C15, 40

    def ids_of(rows):
        if not sparse:
            return torch.from_numpy(rows.astype(np.int64))
        return torch.from_numpy(((rows.astype(np.uint64) * np.uint64(MUL)) & np.uint64((1 << BITS) - 1)).astype(np.int64))

    co.config(make_config(n_item, pct))
    if sparse:
        _basics.set_key_map(MUL, BITS)
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 60_000, n_item, 1.05)]
    co.coll_torch_record(0, ids_of(s0))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)

    def check(stream_u32):
        want, nid = expected_cached_set(stream_u32, n_item, pct)
        got = np.zeros(len(want), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want)
        assert np.array_equal(got, want)
        rows = rng.integers(0, n_item, size=20_001)
        out = co.coll_torch_lookup_key_t_val_ret(0, ids_of(rows).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, rows).tobytes()
        assert _basics.last_group_offset(0)[1] == int((nid[rows] == 0).sum())

    observed = len(np.unique(s0))
    assert (observed > int(n_item * pct)) == (pct < 0.5)  # both sides of "more observed than cached" are covered
    check(s0.astype(np.uint32))
    s1 = perm[::-1][zipf_ranks(rng, 60_000, n_item, 1.05)]  # the other end of the table turns hot
    co.coll_torch_record(0, ids_of(s1))
    co.coll_torch_refresh(0, True)
    check(s1.astype(np.uint32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_compiled_c_lib_module_end_to_end(dtype, kdtype, tmp_path):
    """collcache.torch.c_lib_native, the pybind11 form of the reference's c_lib (adapter.cc:274-281), in the reference's
    call order: create_emb_shm (from a file) -> record -> init_t -> lookup; same bytes as the oracle's gather, the
    output a padded view of a reused buffer, coll_torch_test an uninitialised tensor of the output's shape"""
    import importlib
    native = importlib.import_module("collcache.torch.c_lib_native")
    rng = np.random.default_rng(77)
    n_item, dim, pct = 30_000, 64, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    np_dtype = np.float32 if dtype == torch.float32 else np.float16
    table = rng.standard_normal((n_item, dim)).astype(np_dtype)
    fname = str(tmp_path / "feat.bin")
    table.tofile(fname)
    try:
        emb = native.coll_torch_create_emb_shm(0, n_item, dim, dtype, fname)
        assert tuple(emb.shape) == (n_item, dim) and emb.dtype == dtype and emb.numpy().tobytes() == table.tobytes()
        perm = rng.permutation(n_item)
        s0 = perm[zipf_ranks(rng, 50_000, n_item, 1.1)]
        native.coll_torch_record(0, torch.from_numpy(s0).to(kdtype))
        native.coll_torch_init_t(0, 0, emb, pct)
        want_cached, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)
        assert _basics.info(0)["cached_rows"] == len(want_cached)
        for n in (1, 13, 4097):
            keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
            kt = torch.from_numpy(keys).to(kdtype).cuda()
            out = native.coll_torch_lookup_key_t_val_ret(0, kt, True)
            assert tuple(out.shape) == ((n + 7) // 8 * 8, dim) and out.dtype == dtype and out.is_cuda
            assert out[:n].cpu().numpy().tobytes() == table[keys].tobytes()
            assert _basics.last_group_offset(0) == [0, int((nid[keys] == 0).sum()), n]
            out2 = native.coll_torch_lookup_key_t_val_ret(0, kt, False)
            assert tuple(out2.shape) == (n, dim) and out2.data_ptr() == out.data_ptr()  # the reused buffer
            blank = native.coll_torch_test(0, kt)
            assert tuple(blank.shape) == (n, dim) and blank.dtype == torch.float32 and blank.is_cuda
    finally:
        native.coll_torch_shutdown()


@pytest.mark.parametrize("key_list", ["device", "host"])
@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
def test_build_from_an_explicit_rank_list(key_list, table_kind, monkeypatch):
    """coll_cache_init_ranked_c (the build_v2 overload with a rank list and a frequency list over all keys,
    facade.h:56-60): the first K keys of the list are the cached set, whatever order they come in"""
    from collcache.torch import c_lib  # the module `co` wraps: one _State
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_DEVICE_KEY_LIST", "1" if key_list == "device" else "0")
    rng = np.random.default_rng(31)
    n_item, dim, pct = 40_001, 16, 0.25
    co.config(make_config(n_item, pct))
    rank_keys = rng.permutation(n_item).astype(np.uint32)
    rank_freq = np.sort(rng.integers(0, 1000, size=n_item).astype(np.uint32))[::-1].copy()
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    torch.cuda.set_device(0)
    c_lib._State.dev_id[0] = 0
    alloc, release = c_lib._make_allocator(0)
    c_lib._setup_dims(dim, False)
    _basics.C_LIB_CTYPES.coll_cache_init_ranked_c(0, n_item, rank_keys.ctypes.data, rank_freq.ctypes.data, alloc, release,
                                                  None, emb.data_ptr(), c_lib.kF32, dim, float(pct),
                                                  c_lib._stream_handle(0))
    c_lib._State.host_tables.append(emb)
    k = int(n_item * (pct * 100 / 100.0))
    want = np.sort(rank_keys[:k])
    nid, nc = ORC.rep_solve(rank_keys, n_item, pct * 100)
    assert nc == k and np.array_equal(np.nonzero(nid == 0)[0].astype(np.uint32), want)
    got = np.zeros(k, np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, k) == k
    assert np.array_equal(got, want)
    keys = rng.integers(0, n_item, size=30_000)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
    assert _basics.last_group_offset(0) == [0, int((nid[keys] == 0).sum()), len(keys)]


@pytest.mark.parametrize("pct", [0.0, 0.1, 1.0])
@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_dedup_in_front_of_the_extraction(pct, table_kind, kdtype, monkeypatch):
    """COLL_DEDUP_KEYS=1: each distinct key is extracted once and the duplicates are copied inside the output; the
    output must stay identical to the plain gather, the group sizes count distinct keys."""
    if pct in (0.0, 1.0) and table_kind == "HASH":
        pytest.skip("direct mapping has no table")
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
    monkeypatch.setenv("COLL_DEDUP_MIN_KEYS", "64")
    rng = np.random.default_rng(21)
    n_item, dim = 30_000, 96
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    rec = perm[zipf_ranks(rng, 60_000, n_item, 1.2)]
    co.coll_torch_record(0, torch.from_numpy(rec).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(rec.astype(np.uint32), n_item, pct)
    # 50_000 after 1000 regrows the buffers; 8 is below the threshold (no dedup); the repeat reuses the set (epochs)
    for n in (8, 1000, 50_000, 50_000, 777):
        keys = perm[zipf_ranks(rng, n, n_item, 1.3)]
        if n == 777:
            keys[:] = keys[0]  # one distinct key
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes(), n
        uniq = np.unique(keys) if n >= 64 else keys
        if pct == 1.0:
            want = [0, len(uniq), len(uniq)]
        elif pct == 0.0:
            want = [0, 0, len(uniq)]
        else:
            want = [0, int((nid[uniq] == 0).sum()), len(uniq)]
        assert _basics.last_group_offset(0) == want


@pytest.mark.parametrize("impl", ["", "SMMaskPhase", "NONE"])
@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
def test_committed_golden_case_end_to_end(impl, table_kind, monkeypatch):
    """tests/golden/extract_small.json (written by brute-force Python, tests/golden/make_fixtures.py): record the
    stream, build, look the keys up — cached set, capacity, group sizes and every output byte as in the file"""
    import json
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    with open(os.path.join(ROOT, "tests", "golden", "extract_small.json")) as f:
        g = json.load(f)
    n_item, rb, pct = g["n_item"], g["row_bytes"], g["cache_percentage"]
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    co.coll_torch_record(0, torch.tensor(g["record_stream"], dtype=torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, rb // 4, torch.float32)
    emb.numpy().view(np.uint8)[...] = np.array(g["table"], np.uint8)
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["capacity_rows"] == g["capacity_rows"] and info["cached_rows"] == len(g["cached_keys"])
    got = np.zeros(len(g["cached_keys"]), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(got)
    assert got.tolist() == g["cached_keys"]
    for kdtype in (torch.int32, torch.int64):
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.tensor(g["lookup_keys"], dtype=kdtype).cuda(), False)
        assert out.cpu().numpy().view(np.uint8).tolist() == g["expected_output"]
        assert _basics.last_group_offset(0) == g["expected_group_offset"]


def test_fp16_table_and_small_rows():
    rng = np.random.default_rng(9)
    n_item, dim, pct = 30_000, 64, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    keys = rng.integers(0, n_item, size=100_000)
    co.coll_torch_record(0, torch.from_numpy(keys).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float16)
    table = fill_table(emb, rng)
    assert table.dtype == np.float16 and table.strides[0] == 128
    co.coll_torch_init_t(0, 0, emb, pct)
    q = rng.integers(0, n_item, size=10_001)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(q).to(torch.int32).cuda(), True)
    assert out.dtype == torch.float16 and out.shape == ((10_001 + 7) // 8 * 8, dim)
    assert out[:10_001].cpu().numpy().tobytes() == ORC.gather(table, q.astype(np.int64)).tobytes()


@pytest.mark.parametrize("pct", [1.0, 0.2, 0.0])
def test_bfloat16_table_is_looked_up_as_its_bytes(pct):
    """a bfloat16 table (an extension: the reference's adapter knows float32 and float16) moves through the library as
    two-byte elements; lookups return bfloat16 and the table's bytes.  The pooled lookup adds bfloat16 rows in fp32 and
    rounds the result to bfloat16 (8 bits: 2^-8 of the result on top of 1e-5 of the terms' magnitude)."""
    rng = np.random.default_rng(19)
    n_item, dim = 20_000, 48
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    co.coll_torch_record(0, torch.from_numpy(rng.integers(0, n_item, size=60_000)).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.bfloat16)
    raw = emb.view(torch.int16).numpy()
    raw[...] = rng.integers(-32768, 32768, size=raw.shape, dtype=np.int16)
    co.coll_torch_init_t(0, 0, emb, pct)
    q = rng.integers(0, n_item, size=9_999)
    keys = torch.from_numpy(q).cuda()
    out = co.coll_torch_lookup_key_t_val_ret(0, keys, False)
    assert out.dtype == torch.bfloat16 and out.shape == (len(q), dim)
    assert out.view(torch.int16).cpu().numpy().tobytes() == raw[q].tobytes()
    a = co.coll_torch_lookup_async(0, keys, False).clone()
    co.coll_torch_lookup_wait(0)
    assert a.view(torch.int16).cpu().numpy().tobytes() == raw[q].tobytes()
    assert co.c_lib.pooled_lookup_supported()
    vals = (raw.astype(np.int64) & 0xffff).astype(np.uint32) << np.uint32(16)
    with np.errstate(all="ignore"):
        vals = vals.view(np.float32).astype(np.float64)
    lens = rng.choice([0, 1, 3, 8], size=2_000)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    ids = rng.integers(0, n_item, size=int(off[-1]))
    w = rng.uniform(0.1, 2.0, size=len(ids)).astype(np.float32)
    got = co.coll_torch_lookup_pooled(0, torch.from_numpy(ids).cuda(), torch.from_numpy(off).cuda(),
                                      torch.from_numpy(w).cuda(), "mean")
    assert got.dtype == torch.bfloat16
    with np.errstate(all="ignore"):
        want = ORC.pool(vals, ids, off, w, "mean")
        mag_sum = ORC.pool(np.abs(vals), ids, off, w, "sum")
        mag = ORC.pool(np.abs(vals), ids, off, w, "mean")
    ok = np.isfinite(mag_sum) & (mag_sum < 1e36)  # random bit patterns: NaNs, infinities and sums that overflow aside
    bound = 1e-5 * np.where(ok, mag, 0.0) + 2.0 ** -8 * np.abs(np.where(ok, want, 0.0)) + 1e-37
    got64 = got.float().cpu().numpy().astype(np.float64)
    assert not (ok & ~(np.abs(got64 - np.where(ok, want, 0.0)) <= bound)).any()


@pytest.mark.parametrize("dim,dtype", [(3, torch.float32), (5, torch.float16), (1, torch.float32), (7, torch.float32)])
@pytest.mark.parametrize("pct", [0.2, 1.0, 0.0])
def test_rows_that_are_not_multiples_of_16_bytes(dim, dtype, pct):
    """12-, 10-, 4- and 28-byte rows: the 16-byte-lane kernels do not apply, narrower lanes take over"""
    rng = np.random.default_rng(dim)
    n_item = 9_000
    if dtype == torch.float16 and dim % 2:
        pytest.skip("fp16 rows travel as dim/2 fp32 words (operation.cc:132-136): the dimension must be even")
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    co.coll_torch_record(0, torch.from_numpy(rng.integers(0, n_item, size=40_000)).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, dtype)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    for n in (1, 4097):
        q = rng.integers(0, n_item, size=n)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(q).cuda(), False)
        assert out.shape == (n, dim)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, q.astype(np.int64)).tobytes()


def test_key_tensors_are_checked_and_strided_ones_accepted():
    rng = np.random.default_rng(3)
    n_item, dim = 5_000, 32
    co.config(make_config(n_item, 1.0))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, 1.0)
    q = rng.integers(0, n_item, size=(2000, 2))
    strided = torch.from_numpy(q).cuda()[:, 1]  # every second element: not contiguous
    assert not strided.is_contiguous()
    out = co.coll_torch_lookup_key_t_val_ret(0, strided, False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, q[:, 1].astype(np.int64)).tobytes()
    with pytest.raises(TypeError):
        co.coll_torch_lookup_key_t_val_ret(0, strided.to(torch.float32), False)
    with pytest.raises(ValueError):
        co.coll_torch_lookup_key_t_val_ret(0, strided.cpu(), False)


def test_create_emb_from_file(tmp_path):
    rng = np.random.default_rng(2)
    arr = rng.standard_normal((1000, 32)).astype(np.float32)
    f = tmp_path / "feat.bin"
    arr.tofile(f)
    co.config(make_config(1000, 1.0))
    emb = co.coll_torch_create_emb_shm(0, 1000, 32, torch.float32, str(f))
    assert emb.numpy().tobytes() == arr.tobytes()
    co.coll_torch_init_t(0, 0, emb, 1.0)
    q = torch.arange(999, -1, -1, dtype=torch.int32, device="cuda")
    assert co.coll_torch_lookup_key_t_val_ret(0, q, False).cpu().numpy().tobytes() == arr[::-1].tobytes()


def test_raw_model_directory_and_mock_table(tmp_path):
    """the serving stack's table formats (modelloader.cpp:52-107): a directory with `key` + `emb_vector`, or
    mock_<rows>_<dim>"""
    rng = np.random.default_rng(2)
    n_item, dim = 5_000, 24
    rows = rng.standard_normal((n_item, dim)).astype(np.float32)
    d = tmp_path / "model" / "sparse_embedding0"
    d.mkdir(parents=True)
    np.arange(n_item, dtype=np.int64).tofile(d / "key")
    rows.tofile(d / "emb_vector")
    co.config(make_config(n_item, 0.0))
    co.coll_cache_record_init(0)
    emb = co.coll_torch_load_raw_model(0, str(d))
    assert tuple(emb.shape) == (n_item, dim) and emb.dtype == torch.float32
    assert emb.numpy().tobytes() == rows.tobytes()
    co.coll_torch_init_t(0, 0, emb, 0.0)
    keys = rng.integers(0, n_item, size=777)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == rows[keys].tobytes()
    mock = co.coll_torch_load_raw_model(0, "mock_1000_16")
    assert tuple(mock.shape) == (1000, 16) and not mock.any()


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH", "HASH16"])
@pytest.mark.parametrize("foreground", [True, False])
@pytest.mark.parametrize("impl", ["", "SMMaskPhase"])
def test_refresh_evicts_and_inserts_like_the_oracle(table_kind, foreground, impl, monkeypatch):
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "100")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "512")
    rng = np.random.default_rng(11)
    n_item, dim, pct = 40_000, 128, 0.25
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm1 = rng.permutation(n_item)
    s1 = perm1[zipf_ranks(rng, 200_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s1).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    old_cached, old_nid = expected_cached_set(s1.astype(np.uint32), n_item, pct)
    cap = _basics.info(0)["capacity_rows"]

    def check_lookup(nid, seed):
        r = np.random.default_rng(seed)
        keys = r.integers(0, n_item, size=20_000)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        if nid is not None:
            assert _basics.last_group_offset(0)[1] == int((nid[keys] == 0).sum())

    check_lookup(old_nid, 1)
    # hotness moves: a new permutation for the next interval
    for rnd in range(2):
        perm2 = rng.permutation(n_item)
        s2 = perm2[zipf_ranks(rng, 200_000, n_item, 1.05)]
        co.coll_torch_record(0, torch.from_numpy(s2).to(torch.int32))
        new_cached, new_nid = expected_cached_set(s2.astype(np.uint32), n_item, pct)
        if foreground:
            co.coll_torch_refresh(0, True)
        else:
            # background refresh on its own thread while the caller keeps looking keys up
            t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
            t.start()
            i = 0
            while t.is_alive():
                check_lookup(None, 100 + i)
                i += 1
            t.join()
            assert i >= 1
        info = _basics.info(0)
        got = np.zeros(len(new_cached), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new_cached)
        assert np.array_equal(got, new_cached)
        assert info["cached_rows"] == len(new_cached) and info["free_slots"] + info["cached_rows"] == cap
        assert len(np.setdiff1d(old_cached, new_cached)) > 1000  # the refresh really moved rows
        check_lookup(new_nid, 2 + rnd)
        old_cached = new_cached


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH", "HASH16"])
@pytest.mark.parametrize("foreground", [True, False])
@pytest.mark.parametrize("keep", [False, True])
@pytest.mark.parametrize("stage", [0, 16384])
def test_refresh_on_the_device_places_like_the_oracle(table_kind, foreground, keep, stage, monkeypatch):
    """COLL_GPU_RECORD=1 + COLL_GPU_REFRESH=1: ranking, placement and the evict / insert lists of a refresh are computed
    on the device from the hotness the lookups counted there.  The cached set afterwards is the oracle's top set of the
    counted key stream (of the last interval, or of everything so far with COLL_GPU_REFRESH_KEEP=1), exactly as after
    a refresh on the host; the two kinds of refresh can alternate."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    if keep:
        monkeypatch.setenv("COLL_GPU_REFRESH_KEEP", "1")
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "100")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "512")
    if stage:  # lookups file the rows they fetch from the host table; foreground refreshes insert from there
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", str(stage))
    rng = np.random.default_rng(21)
    n_item, dim, pct = 50_001, 64, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 150_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    cached, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    cap = _basics.info(0)["capacity_rows"]
    counted = []  # what the device-side counters hold

    def lookup(keys, want_nid):
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(torch.int32).cuda(), False)
        counted.append(keys.astype(np.uint32))
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        if want_nid is not None:
            assert _basics.last_group_offset(0)[1] == int((want_nid[keys] == 0).sum())

    def refresh():
        if foreground:
            co.coll_torch_refresh(0, True)
            return
        t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
        t.start()
        while t.is_alive():  # a background refresh waits for one more lookup to pass; these are not counted
            out = co.coll_torch_lookup_key_t_val_ret(0, torch.zeros(0, dtype=torch.int32).cuda(), False)
            assert out.shape[0] == 0
            time.sleep(0.001)
        t.join()

    def check_cached(want):
        info = _basics.info(0)
        assert info["cached_rows"] == len(want) and info["free_slots"] + info["cached_rows"] == cap
        got = np.zeros(len(want), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want)
        assert np.array_equal(got, want)
        info = _basics.info(0)  # the same from the host-side lists, now up to date
        assert info["cached_rows"] == len(want) and info["free_slots"] + info["cached_rows"] == cap

    for rnd in range(3):
        swap = rng.choice(n_item, n_item // 10, replace=False)
        perm[swap] = perm[rng.permutation(swap)]
        for n in (30_000, 1, 40_000):
            lookup(perm[zipf_ranks(rng, n, n_item, 1.05)], nid)
        refresh()
        new_cached, nid = expected_cached_set(np.concatenate(counted), n_item, pct)
        assert len(np.setdiff1d(cached, new_cached)) > 200  # the refresh really moved rows
        if not keep:
            counted.clear()
        check_cached(new_cached)
        cached = new_cached
        lookup(rng.integers(0, n_item, size=20_000), nid)
    from_stage = _basics.C_LIB_CTYPES.coll_cache_rows_from_stage(0)
    # rows that come in were looked up (and missed) shortly before: the refresh finds most of them filed (a background
    # one in the stage it switched the lookups away from)
    assert (from_stage > 1000) if stage else (from_stage == 0)

    # a refresh on the host in between (hotness recorded on the host joins the device-side counts) ...
    extra = perm[zipf_ranks(rng, 60_000, n_item, 1.3)]
    co.coll_torch_record(0, torch.from_numpy(extra).to(torch.int32))
    co.coll_torch_refresh(0, True)
    cached, nid = expected_cached_set(np.concatenate(counted + [extra.astype(np.uint32)]), n_item, pct)
    counted.clear()  # the host refresh drained the counters
    check_cached(cached)
    lookup(rng.integers(0, n_item, size=20_000), nid)
    # ... and the device takes over again from the host-side lists
    lookup(perm[zipf_ranks(rng, 50_000, n_item, 0.9)], nid)
    refresh()
    cached, nid = expected_cached_set(np.concatenate(counted), n_item, pct)
    check_cached(cached)
    lookup(rng.integers(0, n_item, size=20_000), nid)


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("keep", [False, True])
def test_device_side_counters_seeded_with_the_hotness_the_cache_was_built_from(table_kind, keep, monkeypatch):
    """COLL_GPU_RECORD_SEED=1: the counters the lookups bump start from the ranking the build was given, so the first
    refresh on the device places by the presample and the counted lookups together; afterwards they go on as configured
    (kept: everything so far; otherwise the interval since the last refresh)"""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    monkeypatch.setenv("COLL_GPU_RECORD_SEED", "1")
    if keep:
        monkeypatch.setenv("COLL_GPU_REFRESH_KEEP", "1")
    rng = np.random.default_rng(91)
    n_item, dim, pct = 30_011, 16, 0.25
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 120_000, n_item, 1.1)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    counted = [s0.astype(np.uint32)]
    for rnd in range(3):
        swap = rng.choice(n_item, n_item // 10, replace=False)
        perm[swap] = perm[rng.permutation(swap)]
        keys = perm[zipf_ranks(rng, 20_000, n_item, 1.1)]
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        counted.append(keys.astype(np.uint32))
        co.coll_torch_refresh(0, True)
        want, nid = expected_cached_set(np.concatenate(counted), n_item, pct)
        if rnd == 0:  # without the seed the same refresh would have placed by the 20,000 counted keys alone
            unseeded, _ = expected_cached_set(keys.astype(np.uint32), n_item, pct)
            assert len(np.setdiff1d(want, unseeded)) > 1_000
        got = np.zeros(len(want), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want)
        assert np.array_equal(got, want), rnd
        if not keep:
            counted.clear()
        probe = rng.integers(0, n_item, size=5_000)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(probe).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, probe.astype(np.int64)).tobytes()
        assert _basics.last_group_offset(0)[1] == int((nid[probe] == 0).sum())
        counted.append(probe.astype(np.uint32))


def test_background_refresh_paced_by_a_rate_over_the_link(monkeypatch):
    """COLL_REFRESH_RATE_GBPS: the throttled copy of a background refresh pauses after each batch for as long as keeps
    it at that rate (instead of the fixed pause): same cached set, and the copy cannot have gone faster than asked"""
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "500")
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "1000000")  # would make this refresh take half a minute if it were used
    monkeypatch.setenv("COLL_REFRESH_RATE_GBPS", "0.004")
    rng = np.random.default_rng(78)
    n_item, dim, pct = 50_000, 32, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 150_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    old, _ = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    s1 = perm[::-1][zipf_ranks(rng, 150_000, n_item, 1.05)].copy()
    co.coll_torch_record(0, torch.from_numpy(s1).to(torch.int32))
    new, nid = expected_cached_set(s1.astype(np.uint32), n_item, pct)
    n_coming = len(np.setdiff1d(new, old))
    t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
    t0 = time.perf_counter()
    t.start()
    keys = rng.integers(0, n_item, size=3_000)
    want = ORC.gather(table, keys).tobytes()
    while t.is_alive():
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
        assert out.cpu().numpy().tobytes() == want
        time.sleep(0.002)
    t.join()
    took = time.perf_counter() - t0
    # all batches but the last are followed by their pause: (n - 500) rows of 128 bytes at 4 MB/s
    assert took >= 0.9 * (n_coming - 500) * dim * 4 / 0.004e9, (took, n_coming)
    assert took < 20
    got = np.zeros(len(new), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new)
    assert np.array_equal(got, new)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == want
    assert _basics.last_group_offset(0)[1] == int((nid[keys] == 0).sum())


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("kind", ["host", "device", "device_staged"])
@pytest.mark.parametrize("dim", [32, 16])
def test_rows_of_a_background_refresh_hit_as_they_arrive(table_kind, kind, dim, monkeypatch):
    """a background refresh copies its rows in throttled batches and publishes every batch behind its copy: lookups of
    the rows that come in, run beside the refresh, find more and more of them in the cache (never fewer), some of them
    long before the refresh ends, and always return table[keys].  Rows of 64 bytes share their 128-byte line with a
    neighbour: those are published only once the lookups in flight at the end of their copy have finished."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "4000")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "200")
    if kind != "host":
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
        monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    if kind == "device_staged":
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", "2048")
    rng = np.random.default_rng(77)
    n_item, pct = 50_000, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 150_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    old, _ = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    # the hot set moves to the other end of the permutation
    s1 = perm[::-1][zipf_ranks(rng, 150_000, n_item, 1.05)].copy()
    if kind == "host":
        co.coll_torch_record(0, torch.from_numpy(s1).to(torch.int32))
    else:
        for part in np.array_split(s1, 3):
            out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(part).to(torch.int32).cuda(), False)
            assert out.cpu().numpy().tobytes() == ORC.gather(table, part.astype(np.int64)).tobytes()
    new, _ = expected_cached_set(s1.astype(np.uint32), n_item, pct)
    coming = np.setdiff1d(new, old)
    assert len(coming) > 5_000
    probe = torch.from_numpy(coming.astype(np.int32)).cuda()
    want = ORC.gather(table, coming.astype(np.int64)).tobytes()
    t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
    t.start()
    hits = []
    while t.is_alive():
        out = co.coll_torch_lookup_key_t_val_ret(0, probe, False)
        assert out.cpu().numpy().tobytes() == want
        hits.append(_basics.last_group_offset(0)[1])
        time.sleep(0.002)
    t.join()
    out = co.coll_torch_lookup_key_t_val_ret(0, probe, False)
    assert out.cpu().numpy().tobytes() == want
    assert _basics.last_group_offset(0)[1] == len(coming)  # all of them cached in the end
    assert hits == sorted(hits), hits
    assert hits[0] < len(coming) // 2 and any(len(coming) // 2 < h < len(coming) for h in hits), hits[::5]
    got = np.zeros(len(new), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new)
    assert np.array_equal(got, new)


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("foreground", [True, False])
@pytest.mark.parametrize("keep", [False, True])
def test_stable_refresh_on_the_device_moves_only_rows_the_counters_tell_apart(table_kind, foreground, keep,
                                                                              monkeypatch):
    """COLL_GPU_REFRESH_STABLE=1: rows whose counts tie at the last count that gets in stay where they are.  The cache
    is filled from a ranking the device-side counters know nothing of and is wider than the set of rows the lookups
    touch, so a plain refresh would trade most never-counted cached rows for the lowest-numbered ones; the stable one
    brings in the counted rows only.  The cached set after every refresh is the top set by (count, cached before,
    row order), from a full sort."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH_STABLE", "1")
    if keep:
        monkeypatch.setenv("COLL_GPU_REFRESH_KEEP", "1")
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "100")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "512")
    rng = np.random.default_rng(33)
    n_item, dim, pct = 40_003, 32, 0.3
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 200_000, n_item, 0.8)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    cached, _ = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    k = len(cached)
    counts = np.zeros(n_item, np.int64)
    rows = np.arange(n_item, dtype=np.int64)

    def refresh():
        if foreground:
            co.coll_torch_refresh(0, True)
            return
        t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
        t.start()
        while t.is_alive():
            co.coll_torch_lookup_key_t_val_ret(0, torch.zeros(0, dtype=torch.int32).cuda(), False)
            time.sleep(0.001)
        t.join()

    moved = []
    for rnd in range(3):
        # a few thousand distinct rows per round, far fewer than the cache holds
        keys = perm[zipf_ranks(rng, 6_000, n_item, 1.2)] if rnd != 1 else rng.integers(0, n_item, size=2_500)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        np.add.at(counts, keys, 1)
        refresh()
        was = np.zeros(n_item, bool)
        was[cached] = True
        tie = np.where(counts > 0, rows, -rows)
        order = np.lexsort((tie, was, counts))[::-1]
        new_cached = np.sort(order[:k]).astype(np.uint32)
        plain, _ = expected_cached_set(np.repeat(rows, counts).astype(np.uint32), n_item, pct)
        moved.append((len(np.setdiff1d(cached, new_cached)), len(np.setdiff1d(cached, plain))))
        got = np.zeros(k, np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, k) == k
        assert np.array_equal(got, new_cached), rnd
        # every row that left was never counted, every row that came in was counted
        assert not counts[np.setdiff1d(cached, new_cached)].any() and counts[np.setdiff1d(new_cached, cached)].all()
        cached = new_cached
        if not keep:
            counts[:] = 0
        probe = rng.integers(0, n_item, size=1_500)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(probe).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, probe.astype(np.int64)).tobytes()
        np.add.at(counts, probe, 1)
    # (rows the stable refresh moved, rows a plain one would have moved)
    assert all(0 < stable < plain for stable, plain in moved) and moved[0][0] < moved[0][1] // 4, moved


@pytest.mark.parametrize("pct,impl,dedup", [(0.25, "", False), (0.25, "NONE", True), (0.25, "SMMaskPhase", False),
                                            (1.0, "", False), (0.0, "", True)])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_hotness_counted_on_the_device_ranks_like_the_host_recorder(pct, impl, dedup, kdtype, monkeypatch):
    """COLL_GPU_RECORD=1: the lookups count their keys in device-side counters; the ranking taken from them equals
    the oracle's ranking of the concatenated key stream (what coll_torch_record of the same keys gives), and a
    refresh driven by them caches the oracle's top set."""
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    if dedup:
        monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
        monkeypatch.setenv("COLL_DEDUP_MIN_KEYS", "64")
    rng = np.random.default_rng(33)
    n_item, dim = 30_000, 64
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm1 = rng.permutation(n_item)
    s1 = perm1[zipf_ranks(rng, 100_000, n_item, 1.1)]
    if 0.0 < pct < 1.0:  # the build consumes this ranking; without a partial cache nothing would
        co.coll_torch_record(0, torch.from_numpy(s1).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)

    perm2 = rng.permutation(n_item)
    stream = []
    for n in (1, 50_000, 3_000, 50_000):
        keys = perm2[zipf_ranks(rng, n, n_item, 1.1)]
        stream.append(keys)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(kdtype).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
    allk = np.concatenate(stream).astype(np.uint32)
    if 0.0 < pct < 1.0:
        # a host-side record joins the device-side counts
        extra = perm2[zipf_ranks(rng, 10_000, n_item, 1.1)]
        co.coll_torch_record(0, torch.from_numpy(extra).to(kdtype))
        allk = np.concatenate([allk, extra.astype(np.uint32)])
        new_cached, new_nid = expected_cached_set(allk, n_item, pct)
        co.coll_torch_refresh(0, True)
        got = np.zeros(len(new_cached), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new_cached)
        assert np.array_equal(got, new_cached)
        keys = rng.integers(0, n_item, size=20_000)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(kdtype).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        assert _basics.last_group_offset(0)[1] == (int((new_nid[keys] == 0).sum()) if not dedup else
                                                   int((new_nid[np.unique(keys)] == 0).sum()))
        allk = keys.astype(np.uint32)  # the refresh consumed the counts; only this last lookup is left
    want_k, want_c = ORC.freq_rank(allk)
    got_k = np.zeros(n_item, np.uint32)
    got_c = np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k)
    assert np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)
    assert _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, None, None, 0) == 0  # drained


@pytest.mark.parametrize("stream_ordered", [False, True])
@pytest.mark.parametrize("gpu_record", [False, True, "and_refresh"])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_serving_loop_records_a_prefix_and_refreshes_in_the_background(gpu_record, kdtype, stream_ordered, monkeypatch):
    """LookupManager::forward re-expressed (lookup_manager.cc:158-213): every step records the first share of its
    batch, looks the batch up, and at step refresh_iter starts a background refresh from what was recorded.
    stream_ordered: the steps are enqueued and left (coll_cache_forward_async*; a prefix counted on the host is counted
    later, by a later step, the wait or the ranking) and must record, look up and refresh exactly like the blocking
    ones."""
    if gpu_record:
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
    if gpu_record == "and_refresh":  # the background refresh is computed on the device as well
        monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    if stream_ordered:  # ... and the prefixes counted on the host are counted by the step itself, not by the thread
        monkeypatch.setenv("COLL_RECORD_INLINE_BYTES", str(1 << 20))
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "100")
    rng = np.random.default_rng(44)
    n_item, dim, pct, frac = 30_000, 32, 0.2, 0.5
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm1 = rng.permutation(n_item)
    co.coll_torch_record(0, torch.from_numpy(perm1[zipf_ranks(rng, 100_000, n_item, 1.1)]).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    co.coll_torch_forward_config(True, 3, frac, False)

    perm2 = rng.permutation(n_item)
    recorded = []
    for step in range(7):
        n = 40_000 + 1000 * step
        keys = perm2[zipf_ranks(rng, n, n_item, 1.1)]
        keys_dev = torch.from_numpy(keys).to(kdtype).cuda()
        out = co.coll_torch_forward(0, keys_dev, False, stream_ordered=stream_ordered)
        if stream_ordered:
            co.coll_torch_lookup_wait(0)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        recorded.append(keys[: int(n * frac)])
        if step < 3:
            assert co.coll_torch_forward_join() == 0
        if step == 3:
            # the refresh started at the end of this step; it waits for one more lookup to pass before it reuses
            # cache slots (an empty one will do, and records nothing)
            empty = torch.zeros(0, dtype=kdtype, device="cuda")
            while _basics.C_LIB_CTYPES.coll_cache_forward_refresh_ongoing():
                co.coll_torch_lookup_key_t_val_ret(0, empty, False)
                time.sleep(0.001)
            assert co.coll_torch_forward_join() == 1
            new_cached, new_nid = expected_cached_set(np.concatenate(recorded).astype(np.uint32), n_item, pct)
            got = np.zeros(len(new_cached), np.uint32)
            assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new_cached)
            assert np.array_equal(got, new_cached)
        if step > 3:
            assert _basics.last_group_offset(0)[1] == int((new_nid[keys] == 0).sum())
    assert co.coll_torch_forward_join() == 1  # not periodic: one refresh only
    # plain lookups count whole batches again
    co.coll_torch_forward_config(False, 0, frac, False)


@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_stream_ordered_serving_steps_count_their_prefixes_later(kdtype):
    """coll_cache_forward_async* with the hotness counted on the host: thirty steps enqueued back to back without a
    wait (more than the library has buffers for waiting prefixes); every step's prefix has been counted once
    coll_cache_lookup_wait returns, and the outputs are the table's rows."""
    rng = np.random.default_rng(61)
    n_item, dim, pct, frac = 20_000, 32, 0.3, 0.25
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    co.coll_torch_record(0, torch.from_numpy(rng.integers(0, n_item, size=60_000)).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    co.coll_torch_forward_config(True, 10 ** 9, frac, False)
    alive, recorded, outs = [], [], []
    for step in range(30):
        n = 4_000 + 16 * step
        keys = rng.integers(0, n_item, size=n)
        alive.append(torch.from_numpy(keys).to(kdtype).cuda())
        outs.append((keys, co.coll_torch_forward(0, alive[-1], False, stream_ordered=True).clone()))
        recorded.append(keys[: int(n * frac)])
    co.coll_torch_lookup_wait(0)
    for keys, out in outs:
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
    want_k, want_c = ORC.freq_rank(np.concatenate(recorded).astype(np.uint32))
    got_k, got_c = np.zeros(n_item, np.uint32), np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k) and np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)
    co.coll_torch_forward_config(False, 0, frac, False)


@pytest.mark.parametrize("pct,table_kind", [(1.0, "FLAT"), (0.0, "FLAT"), (0.25, "FLAT"), (0.25, "HASH")])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_stream_ordered_lookups(pct, table_kind, kdtype, monkeypatch):
    """coll_cache_lookup_async: batches are enqueued without waiting; what is enqueued behind them on the same stream
    (here: a clone of the reused output buffer) sees their rows; wait() collects status and group sizes; a refresh in
    between keeps everything exact."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "100")
    rng = np.random.default_rng(77)
    n_item, dim = 40_000, 128
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s1 = perm[zipf_ranks(rng, 100_000, n_item, 1.1)]
    partial = 0.0 < pct < 1.0
    if partial:
        co.coll_torch_record(0, torch.from_numpy(s1).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(s1.astype(np.uint32), n_item, pct) if partial else (None, None)

    def burst(nid):
        keep, clones, batches = [], [], []
        for n in (30_000, 1, 4096, 30_000, 12_345):
            keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
            kt = torch.from_numpy(keys).to(kdtype).cuda()
            keep.append(kt)  # the keys must outlive the enqueued work
            out = co.coll_torch_lookup_async(0, kt, False)
            clones.append(out.clone())  # enqueued behind the lookup on the same stream
            batches.append(keys)
        co.coll_torch_lookup_wait(0)
        for keys, c in zip(batches, clones):
            assert c.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        n = len(batches[-1])
        n_local = n if pct == 1.0 else 0 if pct == 0.0 else int((nid[batches[-1]] == 0).sum())
        assert _basics.last_group_offset(0) == [0, n_local, n]

    burst(nid)
    assert _basics.info(0)["lookups"] == 5
    if partial:
        perm2 = rng.permutation(n_item)
        s2 = perm2[zipf_ranks(rng, 100_000, n_item, 1.1)]
        co.coll_torch_record(0, torch.from_numpy(s2).to(kdtype))
        # enqueue a batch, then refresh in the background without waiting for it first
        keys = perm[zipf_ranks(rng, 20_000, n_item, 1.1)]
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        pre = co.coll_torch_lookup_async(0, kt, False).clone()
        t = threading.Thread(target=co.coll_torch_refresh, args=(0, False))
        t.start()
        t.join()
        assert pre.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        _, nid2 = expected_cached_set(s2.astype(np.uint32), n_item, pct)
        burst(nid2)
    # a blocking lookup settles what is in flight first
    keys = rng.integers(0, n_item, size=1000)
    kt = torch.from_numpy(keys).to(kdtype).cuda()
    a = co.coll_torch_lookup_async(0, kt, False).clone()
    b = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
    assert a.cpu().numpy().tobytes() == b.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()


@pytest.mark.parametrize("pct,stage", [(1.0, 0), (0.25, 0), (0.25, 4096)])
def test_stream_ordered_lookup_inside_a_captured_graph(pct, stage, monkeypatch):
    """a stream-ordered lookup is launches only (no synchronisation, no allocation, no memset node), so a caller can
    capture it; every replay, with eager work and synchronisations in between, must give the eager result.  With a
    stage of missed rows the captured launch carries one launch tag for all its replays (it files rows on the first
    one only); the refresh that follows reads the stage and the lookups after it are still exact."""
    if stage:
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", str(stage))
    rng = np.random.default_rng(5)
    n_item, dim, n = 20_000, 64, 8_192
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    if pct < 1.0:
        co.coll_torch_record(0, torch.from_numpy(rng.integers(0, n_item, size=60_000)).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    keys = torch.zeros(n, dtype=torch.int64, device="cuda")
    result = torch.zeros((n, dim), dtype=torch.float32, device="cuda")
    # warm-up outside the capture: the reused output buffer gets allocated here
    keys.copy_(torch.from_numpy(rng.integers(0, n_item, size=n)))
    co.coll_torch_lookup_async(0, keys, False)
    co.coll_torch_lookup_wait(0)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = co.coll_torch_lookup_async(0, keys, False)
        result.copy_(out)
    for it in range(4):
        q = rng.integers(0, n_item, size=n)
        keys.copy_(torch.from_numpy(q))
        g.replay()
        torch.cuda.synchronize()
        assert result.cpu().numpy().tobytes() == ORC.gather(table, q.astype(np.int64)).tobytes(), it
        # eager work between the replays
        eager = co.coll_torch_lookup_key_t_val_ret(0, keys, False)
        assert eager.cpu().numpy().tobytes() == result.cpu().numpy().tobytes()
    if stage:
        hot = rng.integers(0, n_item // 4, size=80_000)
        co.coll_torch_record(0, torch.from_numpy(hot).to(torch.int32))
        co.coll_torch_refresh(0, True)
        q = rng.integers(0, n_item, size=n)
        keys.copy_(torch.from_numpy(q))
        g.replay()
        torch.cuda.synchronize()
        assert result.cpu().numpy().tobytes() == ORC.gather(table, q.astype(np.int64)).tobytes()


def _random_case(seed):
    r = np.random.default_rng(1000 + seed)
    dims = [1, 2, 3, 4, 8, 12, 16, 31, 32, 64, 100, 128, 256, 300]
    return dict(seed=seed, n_item=int(r.integers(1, 60_000)), dim=int(r.choice(dims)),
                pct=float(r.choice([0.0, 0.01, 0.1, 0.37, 0.9, 0.999, 1.0])),
                table_kind=str(r.choice(["FLAT", "HASH", "HASH16"])), impl=str(r.choice(["", "SMMaskPhase", "NONE"])),
                i64=bool(r.integers(0, 2)), dedup=bool(r.integers(0, 4) == 0), gpu_record=bool(r.integers(0, 4) == 0),
                zipf=float(r.choice([0.6, 1.05, 1.4])), half=bool(r.integers(0, 3) == 0),
                stage=int(r.choice([0, 0, 1024])), host_list=bool(seed % 3 == 0))


# UGACHE_TEST_SEEDS widens the two seeded sweeps of this file for an occasional longer run
_SEEDS = int(os.environ.get("UGACHE_TEST_SEEDS", "0"))


@pytest.mark.parametrize("case", [_random_case(i) for i in range(max(96, _SEEDS))], ids=lambda c: "seed%d" % c["seed"])
def test_random_configurations_are_exact(case, monkeypatch):
    """seeded random sweep over table size, row width, cache share, table kind, extraction mode, key width and the
    optional stages: blocking and stream-ordered lookups of ragged batch sizes (0, 1, odd, larger than the table)
    must reproduce table[keys] byte for byte"""
    monkeypatch.setenv("COLL_HASH_TABLE", case["table_kind"])
    if case["impl"]:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", case["impl"])
    if case["dedup"]:
        monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
        monkeypatch.setenv("COLL_DEDUP_MIN_KEYS", "16")
    if case["gpu_record"]:
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
    if case["stage"]:
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", str(case["stage"]))
    if case["host_list"]:  # the key -> block array and its scans on the host, instead of the bitmap on the device
        monkeypatch.setenv("COLL_DEVICE_KEY_LIST", "0")
    rng = np.random.default_rng(case["seed"])
    n_item, dim, pct = case["n_item"], case["dim"], case["pct"]
    kdtype = torch.int64 if case["i64"] else torch.int32
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    co.coll_torch_record(0, torch.from_numpy(perm[zipf_ranks(rng, 5 * n_item + 10, n_item, case["zipf"])]).to(kdtype))
    fdtype = torch.float16 if case["half"] and dim % 2 == 0 else torch.float32
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, fdtype)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct) or pct in (0.0, 1.0)
    for n in (0, 1, 7, 63, 64, 65, 1023, int(rng.integers(2_000, 70_000))):
        keys = perm[zipf_ranks(rng, n, n_item, case["zipf"])] if n else np.zeros(0, np.int64)
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        want = ORC.gather(table, keys.astype(np.int64)).tobytes()
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out.shape == (n, dim) and out.cpu().numpy().tobytes() == want, ("blocking", n)
        g = _basics.last_group_offset(0)
        assert g[0] == 0 and g[1] <= g[2] <= n
        a = co.coll_torch_lookup_async(0, kt, False).clone()
        co.coll_torch_lookup_wait(0)
        assert a.cpu().numpy().tobytes() == want, ("stream-ordered", n)
    if 0.0 < pct < 1.0 and n_item > 100:
        co.coll_torch_record(0, torch.from_numpy(perm[::-1][zipf_ranks(rng, 3 * n_item, n_item, 1.1)].copy()).to(kdtype))
        co.coll_torch_refresh(0, True)
        info = _basics.info(0)
        assert info["free_slots"] + info["cached_rows"] == info["capacity_rows"]
        keys = rng.integers(0, n_item, size=5_000)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(kdtype).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
    if co.c_lib.pooled_lookup_supported():
        # the same cache through the pooled lookup, blocking and stream-ordered.  The table holds random bit patterns:
        # elements whose terms are not finite, or so large that an fp32 sum (or an fp16 result) may overflow, are left
        # out of the comparison; the others are within 1e-5 of the magnitude of their terms (fp16 rounding on top)
        with np.errstate(all="ignore"):
            vals = emb.float().numpy().astype(np.float64)
        n_rows = int(rng.integers(1, 4_000))
        lens = rng.choice([0, 1, 2, 5, 30], size=n_rows, p=[0.1, 0.5, 0.2, 0.15, 0.05])
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        ids = perm[zipf_ranks(rng, int(off[-1]), n_item, case["zipf"])] if off[-1] else np.zeros(0, np.int64)
        w = rng.uniform(0.1, 2.0, size=len(ids)).astype(np.float32)
        t_ids, t_off, t_w = torch.from_numpy(ids).to(kdtype).cuda(), torch.from_numpy(off).cuda(), torch.from_numpy(w).cuda()
        combiner = ("sum", "mean", "sqrtn")[case["seed"] % 3]
        with np.errstate(all="ignore"):
            want = ORC.pool(vals, ids, off, w, combiner)
            mag_sum = ORC.pool(np.abs(vals), ids, off, w, "sum")
            mag = ORC.pool(np.abs(vals), ids, off, w, combiner)
        ok = np.isfinite(mag_sum) & (mag_sum < 1e36) & (mag < (6.0e4 if fdtype == torch.float16 else 1e36))
        bound = 1e-5 * np.where(ok, mag, 0.0) + (1e-3 * np.abs(np.where(ok, want, 0.0)) + 2.0 ** -25
                                                 if fdtype == torch.float16 else 0.0) + 1e-30
        for stream_ordered in (False, True):
            got = co.coll_torch_lookup_pooled(0, t_ids, t_off, t_w, combiner, stream_ordered=stream_ordered)
            if stream_ordered:
                co.coll_torch_lookup_wait(0)
            assert _basics.last_group_offset(0)[2] == len(ids)
            got = got.float().cpu().numpy().astype(np.float64)
            assert got.shape == (n_rows, dim)
            bad = ok & ~(np.abs(got - np.where(ok, want, 0.0)) <= bound)
            assert not bad.any(), ("pooled", stream_ordered, combiner, int(bad.sum()))


@pytest.mark.parametrize("device", [False, True])
def test_refresh_of_a_table_too_small_for_spare_slots(device, monkeypatch):
    """400 rows, 10 % cached: the capacity (size_t)(400 * 0.101) = 40 equals the number of cached rows, so a refresh has
    exactly as many free slots (the evicted ones) as rows to insert.  The reference's strict check
    (cache_hashtable.cuh:648) would abort there; here the refresh goes through, on the host and on the device."""
    if device:
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
        monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    rng = np.random.default_rng(258)
    n_item, dim, pct = 400, 100, 0.1
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 2010, n_item, 1.4)]
    co.coll_torch_record(0, torch.from_numpy(s0))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["capacity_rows"] == 40 and info["cached_rows"] == 40 and info["free_slots"] == 0
    old, _ = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    s1 = perm[::-1][zipf_ranks(rng, 1200, n_item, 1.1)].copy()
    if device:
        co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(s1).cuda(), False)
    else:
        co.coll_torch_record(0, torch.from_numpy(s1))
    co.coll_torch_refresh(0, True)
    want, nid = expected_cached_set(s1.astype(np.uint32), n_item, pct)
    assert len(np.setdiff1d(old, want)) > 10
    got = np.zeros(len(want), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want)
    assert np.array_equal(got, want)
    info = _basics.info(0)
    assert info["cached_rows"] == 40 and info["free_slots"] == 0
    keys = rng.integers(0, n_item, size=5_000)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
    assert _basics.last_group_offset(0)[1] == int((nid[keys] == 0).sum())


def _random_refresh_case(seed):
    r = np.random.default_rng(5000 + seed)
    return dict(seed=seed, n_item=int(r.integers(130, 90_000)), dim=int(r.choice([4, 16, 32, 64, 100])),
                pct=float(r.choice([0.01, 0.1, 0.37, 0.9, 0.99])), table_kind=str(r.choice(["FLAT", "HASH", "HASH16"])),
                keep=bool(r.integers(0, 2)), sparse=bool(r.integers(0, 3) == 0), zipf=float(r.choice([0.6, 1.05, 1.4])),
                rounds=int(r.integers(2, 5)), stream_ordered=bool(r.integers(0, 3) == 0),
                stage=int(r.choice([0, 256, 65536])), stable=bool(r.integers(0, 3) == 0), host_list=bool(seed % 3 == 1))


@pytest.mark.parametrize("case", [_random_refresh_case(i) for i in range(max(24, _SEEDS // 2))],
                         ids=lambda c: "seed%d" % c["seed"])
def test_random_sequences_of_refreshes_on_the_device(case, monkeypatch):
    """seeded random sweep over table size, cache share (from nearly nothing cached to nearly everything), table kind,
    sparse ids, accumulating or per-interval hotness, ties to row order or to the cached rows first: after every refresh
    computed on the device the cached rows are the oracle's top set of the counted key stream (with
    COLL_GPU_REFRESH_STABLE the top set of a full sort by count, cached before, row order), slots are conserved and
    lookups reproduce table[keys]"""
    monkeypatch.setenv("COLL_HASH_TABLE", "HASH" if case["sparse"] else case["table_kind"])
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    monkeypatch.setenv("COLL_HASH_REBUILD_FRAC", "0.02")
    if case["stage"]:  # the refreshes of this test run in the foreground: they insert from the stage what they find there
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", str(case["stage"]))
    if case["keep"]:
        monkeypatch.setenv("COLL_GPU_REFRESH_KEEP", "1")
    if case["stable"]:
        monkeypatch.setenv("COLL_GPU_REFRESH_STABLE", "1")
    if case["host_list"]:
        monkeypatch.setenv("COLL_DEVICE_KEY_LIST", "0")
    rng = np.random.default_rng(case["seed"])
    n_item, dim, pct = case["n_item"], case["dim"], case["pct"]
    MUL, BITS = 0x9E3779B97F4A7C15, 40

    def ids_of(rows):
        if not case["sparse"]:
            return torch.from_numpy(rows.astype(np.int64))
        return torch.from_numpy(((rows.astype(np.uint64) * np.uint64(MUL)) & np.uint64((1 << BITS) - 1)).astype(np.int64))

    co.config(make_config(n_item, pct))
    if case["sparse"]:
        _basics.set_key_map(MUL, BITS)
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 3 * n_item, n_item, case["zipf"])]
    co.coll_torch_record(0, ids_of(s0))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    cap = _basics.info(0)["capacity_rows"]
    want, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    counted = []
    for rnd in range(case["rounds"]):
        swap = rng.choice(n_item, max(n_item // 8, 2), replace=False)
        perm[swap] = perm[rng.permutation(swap)]
        for n in (int(rng.integers(1, 2 * n_item + 2)), 1, int(rng.integers(1, 5_000))):
            rows = perm[zipf_ranks(rng, n, n_item, case["zipf"])]
            kt = ids_of(rows).cuda()
            if case["stream_ordered"]:
                out = co.coll_torch_lookup_async(0, kt, False).clone()
                co.coll_torch_lookup_wait(0)
            else:
                out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
            counted.append(rows.astype(np.uint32))
            assert out.cpu().numpy().tobytes() == ORC.gather(table, rows.astype(np.int64)).tobytes()
            assert _basics.last_group_offset(0)[1] == int((nid[rows] == 0).sum())
        co.coll_torch_refresh(0, True)
        if case["stable"]:
            counts = np.bincount(np.concatenate(counted), minlength=n_item)
            was = np.zeros(n_item, bool)
            was[want] = True
            all_rows = np.arange(n_item, dtype=np.int64)
            order = np.lexsort((np.where(counts > 0, all_rows, -all_rows), was, counts))[::-1]
            want = np.sort(order[:len(want)]).astype(np.uint32)
            nid = np.ones(n_item, nid.dtype)
            nid[want] = 0
        else:
            want, nid = expected_cached_set(np.concatenate(counted), n_item, pct)
        if not case["keep"]:
            counted.clear()
        info = _basics.info(0)
        assert info["cached_rows"] == len(want) and info["free_slots"] + info["cached_rows"] == cap
        if rnd % 2 == 1 or rnd == case["rounds"] - 1:  # the key list by way of the host-side lists, not every time
            got = np.zeros(len(want), np.uint32)
            assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want)
            assert np.array_equal(got, want)


def test_reference_cpu_runnable_config_full_size():
    """1M x 128 fp32 host table, 65536 int64 keys Zipf(1.1) over a seeded permutation, hottest 10 % cached."""
    rng = np.random.default_rng(1)
    n_item, dim, pct, n = 1_000_000, 128, 0.10, 65_536
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    emb.normal_(generator=torch.Generator().manual_seed(1))
    table = emb.numpy()
    perm = np.random.default_rng(2).permutation(n_item)
    r3 = np.random.default_rng(3)
    batches = [perm[zipf_ranks(r3, n, n_item, 1.1)] for _ in range(4)]
    for b in batches[:3]:
        co.coll_torch_record(0, torch.from_numpy(b))
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(np.concatenate(batches[:3]).astype(np.uint32), n_item, pct)
    assert _basics.info(0)["cached_rows"] == 100_000
    for b in batches:
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(b).cuda(), False)
        assert out.shape == (n, dim)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, b.astype(np.int64), omp=True).tobytes()
        assert _basics.last_group_offset(0) == [0, int((nid[b] == 0).sum()), n]


@pytest.mark.parametrize("impl,dedup", [("", False), ("SMMaskPhase", False), ("", True)])
def test_batch_whose_output_passes_4_GiB(impl, dedup, monkeypatch):
    """9M int64 keys of 512-byte rows through the library: 4.6 GB of output from a 30 % cache, checked on the device
    against a plain indexed read of the table (a byte copy either way)"""
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    if dedup:
        monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
    rng = np.random.default_rng(21)
    n_item, dim, pct, n = 300_000, 128, 0.3, 9_000_000
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    hot = perm[zipf_ranks(rng, 200_000, n_item, 1.1)]
    co.coll_torch_record(0, torch.from_numpy(hot))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(hot.astype(np.uint32), n_item, pct)
    keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
    kt = torch.from_numpy(keys).cuda()
    out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
    assert out.shape == (n, dim) and out.numel() * 4 > 1 << 32
    table_dev = emb.cuda().view(torch.int32)
    got = out.view(torch.int32)
    for lo in range(0, n, 1_000_000):
        assert torch.equal(got[lo : lo + 1_000_000], table_dev[kt[lo : lo + 1_000_000]]), lo
    if not dedup:
        assert _basics.last_group_offset(0) == [0, int((nid[keys] == 0).sum()), n]


def test_cache_of_more_than_2_pow_28_slots():
    """290M rows of 16 bytes, 95 % cached: 275M cache slots, more than the 28 bits of a flat entry hold, so the table is
    the open-addressing one with its 32-bit slot field.  Nothing is recorded, so rows [0, K) are the cached ones;
    table[r, c] = 4 r + c as int32 bits."""
    n_item, dim, pct, n = 290_000_000, 4, 0.95, 2_000_000
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    flat = emb.view(torch.int32).view(-1)
    for lo in range(0, flat.numel(), 1 << 28):
        hi = min(lo + (1 << 28), flat.numel())
        torch.arange(lo, hi, dtype=torch.int32, out=flat[lo:hi])
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    k = int(n_item * pct)
    assert info["table_kind"] == 2 and info["cached_rows"] == k
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct) > 1 << 28
    g = torch.Generator(device="cuda").manual_seed(12)
    keys = torch.randint(0, n_item, (n,), generator=g, device="cuda", dtype=torch.int64)
    keys[:4] = torch.tensor([0, k - 1, k, n_item - 1], device="cuda")
    out = co.coll_torch_lookup_key_t_val_ret(0, keys, False)
    want = (keys * 4).unsqueeze(1) + torch.arange(dim, device="cuda")
    assert torch.equal(out.view(torch.int32), want.to(torch.int32))
    assert _basics.last_group_offset(0) == [0, int((keys < k).sum()), n]


@pytest.mark.parametrize("gpu_record", [False, True, "and_refresh"])
def test_sparse_ids_hash_table_with_refresh_each_step(gpu_record, monkeypatch):
    """The hashtable-mode configuration, scaled down: ids are 64-bit values from a 2^40 space (id = row * odd mod 2^40),
    rows are 64 fp16 (128 B), the cached ids sit in the open-addressing table at 0.7 load, every step is followed by a
    refresh that evicts / inserts by the newly recorded hotness; tombstones trigger table rebuilds on the way."""
    monkeypatch.setenv("COLL_HASH_REBUILD_FRAC", "0.05")
    if gpu_record:  # the hotness of a refresh comes from the lookups themselves, counted per row on the device
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
    if gpu_record == "and_refresh":  # ... and is ranked, placed and turned into evict / insert lists there too
        monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    MUL, BITS = 0x9E3779B97F4A7C15, 40
    mask = np.uint64((1 << BITS) - 1)
    rng = np.random.default_rng(5)
    n_item, dim, pct, n = 400_000, 64, 0.10, 100_000

    def ids_of(rows):
        return ((rows.astype(np.uint64) * np.uint64(MUL)) & mask).astype(np.int64)

    co.config(make_config(n_item, pct))
    _basics.set_key_map(MUL, BITS)
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)

    def stream(k):
        return [perm[zipf_ranks(rng, n, n_item, 1.05)] for _ in range(k)]

    s0 = stream(4)
    for b in s0:
        co.coll_torch_record(0, torch.from_numpy(ids_of(b)))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float16)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["table_kind"] == 3 and info["row_bytes"] == 128  # sparse ids: the 8-byte entries, keyed by the row
    cached, nid = expected_cached_set(np.concatenate(s0).astype(np.uint32), n_item, pct)
    cap = info["capacity_rows"]
    assert info["cached_rows"] == len(cached)

    rebuilds = 0
    for step in range(6):
        rows_b = perm[zipf_ranks(rng, n, n_item, 1.05)]
        keys = torch.from_numpy(ids_of(rows_b)).cuda()
        assert int(keys.max()) > (1 << 32)  # genuinely wide ids
        out = co.coll_torch_lookup_key_t_val_ret(0, keys, False)
        assert out.dtype == torch.float16 and out.shape == (n, dim)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, rows_b.astype(np.int64)).tobytes()
        assert _basics.last_group_offset(0) == [0, int((nid[rows_b] == 0).sum()), n]
        # hotness drifts: part of the permutation is reshuffled, then re-ranked from what was recorded since
        swap = rng.choice(n_item, n_item // 50, replace=False)
        perm[swap] = perm[rng.permutation(swap)]
        s = stream(3)
        for b in s:
            if gpu_record:
                co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(ids_of(b)).cuda(), False)
            else:
                co.coll_torch_record(0, torch.from_numpy(ids_of(b)))
        co.coll_torch_refresh(0, True)
        seen = ([rows_b] + s) if gpu_record else s
        new_cached, nid = expected_cached_set(np.concatenate(seen).astype(np.uint32), n_item, pct)
        info = _basics.info(0)
        got = np.zeros(len(new_cached), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(new_cached)
        assert np.array_equal(got, new_cached)  # reported as row numbers
        assert info["free_slots"] + info["cached_rows"] == cap
        rebuilds = info["table_rebuilds"]
        cached = new_cached
    assert rebuilds >= 1


def test_serving_stack_from_a_ps_config_file(tmp_path):
    """The TF2 binding's serving stack for PyTorch (collcache.torch.serving): a ps_config JSON with the keys
    inference_utils.cpp:55-160 reads, a model directory of `key` + `emb_vector` files, Config -> record_hotness ->
    Init -> LookupLayer.  Every lookup reproduces table[keys]; the refresh armed by the configuration runs in the
    background at step coll_cache_refresh_iter and re-places by the recorded 5 % prefixes."""
    import json
    import collcache.torch.serving as hps
    rng = np.random.default_rng(77)
    n_item, dim = 20_000, 16
    rows = rng.standard_normal((n_item, dim)).astype(np.float32)
    model = tmp_path / "dlrm_sparse.model"
    model.mkdir()
    np.arange(n_item, dtype=np.int64).tofile(model / "key")
    rows.tofile(model / "emb_vector")
    cfg = {"iteration_per_epoch": 50, "epoch": 1, "coll_cache_enable_refresh": True, "coll_cache_refresh_iter": 4,
           "models": [{"model": "dlrm", "sparse_files": [str(model)], "gpucacheper": 0.3, "max_batch_size": 4096,
                       "deployed_device_list": [0], "maxnum_catfeature_query_per_table_per_sample": [26],
                       "embedding_vecsize_per_table": [dim], "max_vocabulary_size": [n_item]}]}
    path = tmp_path / "ps_config.json"
    path.write_text(json.dumps(cfg))
    try:
        assert hps.Config(ps_config_file=str(path)) == "OK"
        perm = rng.permutation(n_item)
        warm = [perm[zipf_ranks(rng, 30_000, n_item, 1.1)] for _ in range(3)]
        for b in warm:
            hps.record_hotness(torch.from_numpy(b).cuda())
        assert hps.Init(ps_config_file=str(path), global_batch_size=1024) == "OK"
        want_cached, nid = expected_cached_set(np.concatenate(warm).astype(np.uint32), n_item, 0.3)
        layer = hps.LookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim, emb_vec_dtype=torch.float32)
        perm2 = rng.permutation(n_item)
        recorded = []
        for step in range(8):
            keys = perm2[zipf_ranks(rng, 1024 * 26, n_item, 1.1)].reshape(1024, 26)
            emb = layer(torch.from_numpy(keys).cuda())
            assert tuple(emb.shape) == (1024, 26, dim) and emb.dtype == torch.float32
            assert emb.cpu().numpy().tobytes() == rows[keys].tobytes()
            assert _basics.last_group_offset(0)[1] == int((nid[keys.reshape(-1)] == 0).sum())
            recorded.append(keys.reshape(-1)[: int(keys.size * hps.RECORD_FRACTION)])
            if step == 4:  # the refresh started behind this step; let it finish (it waits for one more lookup)
                empty = torch.zeros(0, dtype=torch.int64, device="cuda")
                while _basics.C_LIB_CTYPES.coll_cache_forward_refresh_ongoing():
                    co.coll_torch_lookup_key_t_val_ret(0, empty, False)
                    time.sleep(0.001)
                assert co.coll_torch_forward_join() == 1
                _, nid = expected_cached_set(np.concatenate(recorded).astype(np.uint32), n_item, 0.3)
        # embedding_lookup_sparse over the cache: ragged rows of ids with weights, the three combiners, against float64
        sparse = hps.SparseLookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim, emb_vec_dtype=torch.float32)
        n_rows = 500
        lens = rng.integers(1, 9, size=n_rows)
        seg = np.repeat(np.arange(n_rows), lens)
        col = np.concatenate([np.arange(k) for k in lens])
        ids = perm2[zipf_ranks(rng, len(seg), n_item, 1.1)]
        w = rng.uniform(0.1, 2.0, size=len(seg)).astype(np.float32)
        ind = torch.from_numpy(np.stack([seg, col])).cuda()
        sp_ids = torch.sparse_coo_tensor(ind, torch.from_numpy(ids).cuda(), (n_rows, 8))
        sp_w = torch.sparse_coo_tensor(ind, torch.from_numpy(w).cuda(), (n_rows, 8))
        e64, w64 = rows[ids].astype(np.float64), w.astype(np.float64)
        for combiner in ("sum", "mean", "sqrtn", None):
            for weights in (sp_w, None):
                ww = w64 if weights is not None else np.ones_like(w64)
                want = np.zeros((n_rows, dim))
                np.add.at(want, seg, e64 * ww[:, None])
                if combiner in ("mean", None):
                    want /= np.bincount(seg, weights=ww, minlength=n_rows)[:, None]
                elif combiner == "sqrtn":
                    want /= np.sqrt(np.bincount(seg, weights=ww * ww, minlength=n_rows))[:, None]
                got = sparse(sp_ids, weights, combiner=combiner).cpu().numpy()
                assert got.shape == (n_rows, dim)
                # fp32 sums of at most 8 terms against float64: tolerance 1e-5 relative to the row's magnitude
                assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
                # the same with the unique done by the library's GPU hash set inside the lookup
                fused = hps.SparseLookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim,
                                              emb_vec_dtype=torch.float32, unique_in_library=True)
                got2 = fused(sp_ids, weights, combiner=combiner).cpu().numpy()
                assert np.allclose(got2, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
                # ... and with lookup and combination in one kernel of the library (one serving step each)
                pooled = hps.SparseLookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim,
                                               emb_vec_dtype=torch.float32, fused=True)
                before = _basics.info(0)["lookups"]
                got3 = pooled(sp_ids, weights, combiner=combiner).cpu().numpy()
                assert _basics.info(0)["lookups"] == before + 1
                assert np.allclose(got3, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
                assert np.allclose(got3, ORC.pool(rows, ids, np.concatenate([[0], np.cumsum(lens)]),
                                                  None if weights is None else w, combiner or "mean"),
                                   rtol=1e-5, atol=1e-5 * np.abs(want).max())
                # ... enqueued like any torch op instead of being a blocking serving step: the same kernel, same bytes
                ordered = hps.SparseLookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim,
                                                emb_vec_dtype=torch.float32, fused=True, stream_ordered=True)
                got4 = ordered(sp_ids, weights, combiner=combiner)
                co.coll_torch_lookup_wait(0)
                assert got4.cpu().numpy().tobytes() == got3.tobytes()
        # max_norm: every embedding clipped to that l2 norm before it is weighted -- the steps of the reference
        # (torch ops here), and lookup + clipping + combination in one kernel, both against the oracle
        norms = np.linalg.norm(rows.astype(np.float64), axis=1)
        for max_norm in (float(np.median(norms)), float(norms.max() * 2)):
            for combiner in ("sum", "mean", "sqrtn"):
                want = ORC.pool(rows, ids, np.concatenate([[0], np.cumsum(lens)]), w, combiner, max_norm=max_norm)
                tol = 1e-5 * np.abs(want).max()
                got = sparse(sp_ids, sp_w, combiner=combiner, max_norm=max_norm).cpu().numpy()
                assert np.allclose(got, want, rtol=1e-5, atol=tol)
                before = _basics.info(0)["lookups"]
                got5 = pooled(sp_ids, sp_w, combiner=combiner, max_norm=max_norm).cpu().numpy()
                assert _basics.info(0)["lookups"] == before + 1  # one fused serving step, not the unfused steps
                assert np.allclose(got5, want, rtol=1e-5, atol=tol)
                # the clipping does not stick to the lookups that follow
                plain = pooled(sp_ids, sp_w, combiner=combiner).cpu().numpy()
                assert np.allclose(plain, ORC.pool(rows, ids, np.concatenate([[0], np.cumsum(lens)]), w, combiner),
                                   rtol=1e-5, atol=tol)
        with pytest.raises(ValueError):
            sparse(sp_ids, None, combiner="max")
        with pytest.raises(ValueError):
            pooled(sp_ids, None, combiner="sum", max_norm=-1.0)
        hps.SetStepProfileValue(profile_type=kLogL1FeatureBytes, value=123.0)
        assert _basics.step_value(hps._last_step_key(), kLogL1FeatureBytes) == 123.0
        hps.Report()
    finally:
        hps.Shutdown()


@pytest.mark.parametrize("pct,table_kind", [(1.0, "FLAT"), (0.0, "FLAT"), (0.3, "FLAT"), (0.3, "HASH"), (0.3, "HASH16")])
@pytest.mark.parametrize("dtype,dim", [(torch.float32, 32), (torch.float16, 64), (torch.float32, 100)])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_pooled_lookup_through_the_library(pct, table_kind, dtype, dim, kdtype, monkeypatch):
    """coll_torch_lookup_pooled (coll_cache_lookup_pooled*): lookup and combination of ragged, weighted segments in one
    call, against the oracle's float64 combination of the same rows; the group sizes count the ids by source, and the
    ids are counted as hotness like those of any lookup.  Tolerance: 1e-5 of the magnitude of the terms (fp32 sums of
    at most 40 terms), plus fp16's rounding of the result where the table is fp16."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    rng = np.random.default_rng(int(pct * 10) + dim)
    n_item = 30_000
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 100_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, dtype)
    emb.copy_(torch.from_numpy(rng.standard_normal((n_item, dim)).astype(np.float32)).to(dtype))
    table = emb.float().numpy().astype(np.float64)
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct) if 0 < pct < 1 else (None, None)
    counted = []
    # (the last batch is one of mostly one id per sample, large enough for the launch to give a lane group four
    # output rows by itself)
    for n_rows in (1, 64, 5_000, 70_000):
        lens = rng.choice([0, 1, 3, 8, 40], size=n_rows, p=[0.05, 0.35, 0.3, 0.25, 0.05])
        if n_rows == 70_000:
            lens = rng.choice([0, 1, 2, 5], size=n_rows, p=[0.1, 0.8, 0.08, 0.02])
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        ids = perm[zipf_ranks(rng, int(off[-1]), n_item, 1.05)] if off[-1] else np.zeros(0, np.int64)
        w = rng.uniform(0.1, 2.0, size=len(ids)).astype(np.float32)
        t_ids, t_off, t_w = torch.from_numpy(ids).to(kdtype).cuda(), torch.from_numpy(off).cuda(), torch.from_numpy(w).cuda()
        for combiner in ("sum", "mean", "sqrtn"):
            for weights in (None, t_w):
                got = co.coll_torch_lookup_pooled(0, t_ids, t_off, weights, combiner)
                counted.append(ids.astype(np.uint32))
                assert tuple(got.shape) == (n_rows, dim) and got.dtype == dtype
                want = ORC.pool(table, ids, off, None if weights is None else w, combiner)
                mag = ORC.pool(np.abs(table), ids, off, None if weights is None else w, combiner)
                bound = 1e-5 * mag + (1e-3 * np.abs(want) + 2.0 ** -25 if dtype == torch.float16 else 0.0) + 1e-30
                assert (np.abs(got.float().cpu().numpy().astype(np.float64) - want) <= bound).all(), (n_rows, combiner)
                n_local = len(ids) if pct == 1.0 else 0 if pct == 0.0 else int((nid[ids] == 0).sum())
                assert _basics.last_group_offset(0) == [0, n_local, len(ids)]
    if not 0 < pct < 1:  # no ranking was needed to build: what was recorded up front is still waiting in the recorder
        counted.append(s0.astype(np.uint32))
    want_k, want_c = ORC.freq_rank(np.concatenate(counted))
    got_k, got_c = np.zeros(n_item, np.uint32), np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k) and np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)
    if dim == 100 and dtype == torch.float32:  # 400-byte rows: a multiple of 16 bytes, but not of whole lane groups
        assert co.c_lib.pooled_lookup_supported()


@pytest.mark.parametrize("pct,table_kind", [(1.0, "FLAT"), (0.0, "FLAT"), (0.3, "FLAT"), (0.3, "HASH"), (0.3, "HASH16")])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_stream_ordered_pooled_lookups(pct, table_kind, kdtype, monkeypatch):
    """coll_torch_lookup_pooled(stream_ordered=True) (coll_cache_lookup_pooled_async*): several batches enqueued back
    to back without a wait give, byte for byte, what the blocking call gives (the same kernel); the wait afterwards
    reports the group sizes of the last batch; the ids of every batch are counted as hotness."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    rng = np.random.default_rng(int(pct * 10) + 77)
    n_item, dim = 30_000, 32
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    s0 = rng.permutation(n_item)[zipf_ranks(rng, 100_000, n_item, 1.05)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    emb.copy_(torch.from_numpy(rng.standard_normal((n_item, dim)).astype(np.float32)))
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct) if 0 < pct < 1 else (None, None)
    batches = []
    for n_rows in (3_000, 1, 700):
        lens = rng.choice([0, 1, 3, 8, 40], size=n_rows, p=[0.05, 0.35, 0.3, 0.25, 0.05])
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        ids = rng.integers(0, n_item, size=int(off[-1]))
        w = rng.uniform(0.1, 2.0, size=len(ids)).astype(np.float32)
        batches.append((ids, torch.from_numpy(ids).to(kdtype).cuda(), torch.from_numpy(off).cuda(), torch.from_numpy(w).cuda()))
    want = [co.coll_torch_lookup_pooled(0, t_ids, t_off, t_w, "mean").cpu() for _, t_ids, t_off, t_w in batches]
    got = [co.coll_torch_lookup_pooled(0, t_ids, t_off, t_w, "mean", stream_ordered=True)
           for _, t_ids, t_off, t_w in batches]
    co.coll_torch_lookup_wait(0)
    for g, w_ in zip(got, want):
        assert g.cpu().numpy().tobytes() == w_.numpy().tobytes()
    last = batches[-1][0]
    n_local = len(last) if pct == 1.0 else 0 if pct == 0.0 else int((nid[last] == 0).sum())
    assert _basics.last_group_offset(0) == [0, n_local, len(last)]
    counted = [b[0].astype(np.uint32) for b in batches] * 2
    if not 0 < pct < 1:
        counted.append(s0.astype(np.uint32))
    want_k, want_c = ORC.freq_rank(np.concatenate(counted))
    got_k, got_c = np.zeros(n_item, np.uint32), np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k) and np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)


@pytest.mark.parametrize("pooled,pct", [(True, 1.0), (False, 1.0), (False, 0.25)])
def test_stream_ordered_lookup_recorded_into_a_graph_with_device_counters(pooled, pct, monkeypatch):
    """COLL_GPU_RECORD=1 and a stream-ordered lookup (pooled or plain) that the caller records into a graph: the
    counting is one more kernel of that graph on the caller's stream -- no stream and no event of the session takes part
    in the capture -- so every replay gives the eager result and counts the keys it read; the ranking drained afterwards
    equals the oracle's ranking of the eager batches plus one batch per replay.  The graph is destroyed before the
    shutdown in one case and outlives it in the others."""
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    rng = np.random.default_rng(78)
    n_item, dim, n = 30_000, 32, 4000
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    s0 = rng.integers(0, n_item, size=60_000)
    if pct < 1.0:
        co.coll_torch_record(0, torch.from_numpy(s0).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    emb.copy_(torch.from_numpy(rng.standard_normal((n_item, dim)).astype(np.float32)))
    co.coll_torch_init_t(0, 0, emb, pct)
    t_ids = torch.zeros(n, dtype=torch.int64, device="cuda")
    t_off = torch.from_numpy(np.arange(0, n + 1, 4, dtype=np.int64)).cuda()

    def lookup(stream_ordered):
        if pooled:
            return co.coll_torch_lookup_pooled(0, t_ids, t_off, None, "mean", stream_ordered=stream_ordered)
        return co.coll_torch_lookup_async(0, t_ids, False) if stream_ordered else \
            co.coll_torch_lookup_key_t_val_ret(0, t_ids, False)

    counted = []
    first = rng.integers(0, n_item, size=n)
    t_ids.copy_(torch.from_numpy(first))
    warm = lookup(True)  # outside the capture: reused buffers get allocated here
    co.coll_torch_lookup_wait(0)
    counted.append(first.astype(np.uint32))
    result = torch.zeros_like(warm)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        result.copy_(lookup(True))  # recorded, not run: nothing is counted here
    for it in range(3):
        q = rng.integers(0, n_item, size=n)
        t_ids.copy_(torch.from_numpy(q))
        result.zero_()
        g.replay()
        torch.cuda.synchronize()
        counted.append(q.astype(np.uint32))
        eager = lookup(False)  # eager work between the replays, counted on the session's own stream
        counted.append(q.astype(np.uint32))
        assert result.cpu().numpy().tobytes() == eager.cpu().numpy().tobytes(), it
    co.coll_torch_lookup_wait(0)
    if pct == 1.0 and pooled:
        del g  # the caller lets go of its graph before the shutdown; the other cases keep it beyond
    want_k, want_c = ORC.freq_rank(np.concatenate(counted))
    got_k, got_c = np.zeros(n_item, np.uint32), np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k) and np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)
    if pct < 1.0:  # a refresh on the device-side counts of replays and eager lookups, then one more replay
        q = rng.integers(0, n_item // 8, size=n)
        t_ids.copy_(torch.from_numpy(q))
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        co.coll_torch_refresh(0, True)
        g.replay()
        torch.cuda.synchronize()
        assert result.cpu().numpy().tobytes() == lookup(False).cpu().numpy().tobytes()
    co.coll_torch_shutdown()  # with the graph alive (unless deleted above); the fixture's second shutdown finds nothing


@pytest.mark.parametrize("impl", ["", "SMMaskPhase"])
def test_counting_every_third_lookup_on_the_device(impl, monkeypatch):
    """COLL_GPU_RECORD_EVERY=3: lookups 0, 3, 6, ... are counted, the others are not; the ranking drained from the
    device equals the oracle's ranking of exactly those batches"""
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_RECORD_EVERY", "3")
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    rng = np.random.default_rng(3)
    n_item, dim, pct = 10_000, 32, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    co.coll_torch_record(0, torch.from_numpy(rng.integers(0, n_item, size=50_000)).to(torch.int32))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    counted = []
    for i in range(8):
        keys = rng.integers(0, n_item, size=5_000 + i)
        out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(torch.int32).cuda(), False)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        if i % 3 == 0:
            counted.append(keys.astype(np.uint32))
    want_k, want_c = ORC.freq_rank(np.concatenate(counted))
    got_k = np.zeros(n_item, np.uint32)
    got_c = np.zeros(n_item, np.uint32)
    m = _basics.C_LIB_CTYPES.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k)
    assert np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH", "HASH16"])
@pytest.mark.parametrize("stage", [0, 8192])
@pytest.mark.parametrize("dim", [32, 12])
def test_lookups_stay_exact_while_the_device_refreshes_under_them(table_kind, stage, dim, monkeypatch):
    """a thread refreshes back to back on the device (background mode, hotness accumulating from the very lookups that
    run beside it) while the caller looks keys up: every output is table[keys], and when the dust settles the cache
    holds exactly its share of rows in exactly that many slots.  Rows of 128 bytes fill their lines; rows of 48 bytes
    share them with their neighbours, and are published only behind the lookups in flight."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_GPU_RECORD", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    monkeypatch.setenv("COLL_GPU_REFRESH_KEEP", "1")
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "50")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "256")
    monkeypatch.setenv("COLL_HASH_REBUILD_FRAC", "0.05")
    if stage:  # the refreshes read the stage of missed rows the lookups beside them have been switched away from
        monkeypatch.setenv("COLL_MISS_STAGE_ROWS", str(stage))
    rng = np.random.default_rng(91)
    n_item, pct = 60_000, 0.15
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    co.coll_torch_record(0, torch.from_numpy(perm[zipf_ranks(rng, 100_000, n_item, 1.05)]))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    cap = _basics.info(0)["capacity_rows"]
    stop, done = [False], [0]

    def refresher():
        while not stop[0]:
            co.coll_torch_refresh(0, False)
            done[0] += 1

    t = threading.Thread(target=refresher)
    t.start()
    try:
        for step in range(150):
            if step % 10 == 0:  # hotness keeps moving
                swap = rng.choice(n_item, n_item // 20, replace=False)
                perm[swap] = perm[rng.permutation(swap)]
            keys = perm[zipf_ranks(rng, int(rng.integers(1, 30_000)), n_item, 1.05)]
            out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
            assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes(), step
    finally:
        stop[0] = True
        while t.is_alive():  # a refresh in flight waits for one more lookup to pass
            co.coll_torch_lookup_key_t_val_ret(0, torch.zeros(0, dtype=torch.int64).cuda(), False)
            t.join(timeout=0.005)
    assert done[0] >= 3
    assert (_basics.C_LIB_CTYPES.coll_cache_rows_from_stage(0) > 0) == bool(stage)
    info = _basics.info(0)
    assert info["cached_rows"] == int(n_item * pct) and info["cached_rows"] + info["free_slots"] == cap
    got = np.zeros(info["cached_rows"], np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(got)
    assert len(np.unique(got)) == len(got)
    keys = rng.integers(0, n_item, size=40_000)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
    assert _basics.last_group_offset(0)[1] == int(np.isin(keys, got).sum())


@pytest.mark.parametrize("pct,table_kind", [(1.0, "FLAT"), (0.0, "FLAT"), (0.25, "FLAT"), (0.25, "HASH")])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_lookup_of_the_distinct_keys_with_inverse(pct, table_kind, kdtype, monkeypatch):
    """coll_cache_lookup_unique: every distinct key of the batch is extracted once; emb[inverse[i]] is the row of
    keys[i], the number of rows is numpy.unique's, and the group sizes are those of the distinct keys"""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    rng = np.random.default_rng(int(pct * 100) + (kdtype == torch.int64))
    n_item, dim = 30_000, 48
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 100_000, n_item, 1.2)]
    if 0.0 < pct < 1.0:
        co.coll_torch_record(0, torch.from_numpy(s0).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)[1] if 0.0 < pct < 1.0 else None
    for n in (1, 2, 63, 64, 65, 5_000, 120_000):
        keys = perm[zipf_ranks(rng, n, n_item, 1.2)]
        if n == 2:
            keys[1] = keys[0]
        rows, inverse = co.coll_torch_lookup_unique(0, torch.from_numpy(keys).to(kdtype).cuda())
        uniq = np.unique(keys)
        assert rows.shape == (len(uniq), dim) and inverse.shape == (n,) and inverse.dtype == torch.int32
        inv = inverse.cpu().numpy()
        assert inv.min() >= 0 and inv.max() == len(uniq) - 1
        got = rows.cpu().numpy()[inv]
        assert got.tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        g = _basics.last_group_offset(0)
        assert g[2] == len(uniq)
        if nid is not None:
            assert g[1] == int((nid[uniq] == 0).sum())
    rows, inverse = co.coll_torch_lookup_unique(0, torch.zeros(0, dtype=kdtype).cuda())
    assert rows.shape[0] == 0 and inverse.numel() == 0
    # an ordinary lookup afterwards is not deduplicated
    keys = rng.integers(0, n_item, size=10_000)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).to(kdtype).cuda(), False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
    assert _basics.last_group_offset(0)[2] == len(keys)


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("impl", ["", "SMMaskPhase", "NONE"])
@pytest.mark.parametrize("kdtype", [torch.int32, torch.int64])
def test_skip_local_extracts_only_what_the_cache_does_not_hold(table_kind, impl, kdtype, monkeypatch):
    """COLL_SKIP_LOCAL=1, the reference's aid for timing the other sources alone (cache_context.cu:728-741): the keys the
    cache serves are dropped in front of the extraction, the rest keep their order and their rows fill the first rows
    of the output (the reference numbers the destinations by position in the compacted key list); what lies behind
    them is not touched.  The variable is read by every lookup, so it can be switched on and off on a built cache."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    rng = np.random.default_rng(17)
    n_item, dim, pct = 60_000, 32, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    s0 = perm[zipf_ranks(rng, 100_000, n_item, 1.1)]
    co.coll_torch_record(0, torch.from_numpy(s0).to(kdtype))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    _, nid = expected_cached_set(s0.astype(np.uint32), n_item, pct)
    for n in (1, 64, 5000, 70_001):
        keys = perm[zipf_ranks(rng, n, n_item, 1.1)]
        kt = torch.from_numpy(keys).to(kdtype).cuda()
        full = co.coll_torch_lookup_key_t_val_ret(0, kt, False).clone()
        assert full.cpu().numpy().tobytes() == ORC.gather(table, keys.astype(np.int64)).tobytes()
        miss = keys[nid[keys] != 0]
        monkeypatch.setenv("COLL_SKIP_LOCAL", "1")
        # the reused output buffer still holds the rows of the full lookup: the untouched tail is recognisable
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        monkeypatch.delenv("COLL_SKIP_LOCAL")
        got = out.cpu().numpy()
        m = len(miss)
        assert _basics.last_group_offset(0) == [0, 0, m]
        assert got[:m].tobytes() == ORC.gather(table, miss.astype(np.int64)).tobytes()
        assert got[m:].tobytes() == full.cpu().numpy()[m:].tobytes()
        step = _basics.info(0)["lookups"] - 1
        assert _basics.step_value(step, kLogL1FeatureBytes) == _basics.step_value(step, kLogL1MissBytes) == m * dim * 4
    # every key cached: nothing is extracted
    hot = np.nonzero(nid == 0)[0][:1000]
    monkeypatch.setenv("COLL_SKIP_LOCAL", "1")
    co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(hot).to(kdtype).cuda(), False)
    assert _basics.last_group_offset(0) == [0, 0, 0]


# ---- the GNN-shaped and the DLR-shaped configuration ---------------------------------------------------------------
def zipf_ranks_dev(n, space, s, gen):
    """zipf_ranks on the device (same inverse CDF), for batches of a million keys and more"""
    u = torch.rand(n, generator=gen, device="cuda", dtype=torch.float64)
    h = float(space)
    r = torch.floor(((h ** (1.0 - s) - 1.0) * u + 1.0) ** (1.0 / (1.0 - s))).to(torch.int64) - 1
    return r.clamp_(0, space - 1)


_GNN_CASES = {}


def _gnn_case(n_item, n_keys, presample):
    """seeded GNN-shaped key stream: Zipf(0.9) ranks over a seeded permutation of the row ids; the presampled batches,
    the oracle's placement for them and a few lookup batches (the oracle's ranking of a 100M-row key space takes half a
    minute, so a case is computed once per size)"""
    key = (n_item, n_keys, presample)
    if key not in _GNN_CASES:
        _GNN_CASES.clear()  # one case at a time: the full-size one holds gigabytes
        gp = torch.Generator(device="cuda").manual_seed(2)
        perm = torch.randperm(n_item, generator=gp, device="cuda", dtype=torch.int64)
        gz = torch.Generator(device="cuda").manual_seed(3)
        pre = [perm[zipf_ranks_dev(n_keys, n_item, 0.9, gz)].cpu() for _ in range(presample)]
        sizes = (n_keys, n_keys, n_keys // 3 + 5, 65_536, n_keys)
        batches = [perm[zipf_ranks_dev(n, n_item, 0.9, gz)] for n in sizes]
        stream = torch.cat(pre).numpy().astype(np.uint32)
        _, nid = expected_cached_set(stream, n_item, 0.25)
        del stream, perm
        _GNN_CASES[key] = (pre, batches, nid)
    return _GNN_CASES[key]


@pytest.mark.parametrize("impl", ["", "SMMaskPhase"])
@pytest.mark.parametrize("dedup", [False, True])
def test_config3_gnn_quarter_cached_zipf_keys_with_dedup(impl, dedup, monkeypatch):
    """The GNN-feature-shaped configuration at 16M rows (the oracle covers that in seconds): 128 fp32 per row in pinned
    host memory, the top 25 % of the rows by the hotness of 50 presampled batches cached, batches of 2^20 int64 keys
    Zipf(0.9) of which nearly half are duplicates; fused and factored extraction, with and without COLL_DEDUP_KEYS.
    Output bytes, cached set and group sizes against the oracle, for batches of several sizes."""
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    if dedup:
        monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
    n_item, dim, pct, n_keys = 16_000_000, 128, 0.25, 1 << 20
    pre, batches, nid = _gnn_case(n_item, n_keys, 50)
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    for b in pre:
        co.coll_torch_record(0, b)
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    g = torch.Generator(device="cuda").manual_seed(1)
    for r0 in range(0, n_item, 2_000_000):
        emb[r0 : r0 + 2_000_000].copy_(torch.randn((2_000_000, dim), generator=g, device="cuda"))
    table = emb.numpy()
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["table_kind"] == 1 and info["cached_rows"] == n_item // 4 == int((nid == 0).sum())
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct)
    got_cached = np.zeros(info["cached_rows"], np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got_cached.ctypes.data, len(got_cached)) == len(got_cached)
    assert np.array_equal(got_cached, np.nonzero(nid == 0)[0])
    for kt in batches:
        keys = kt.cpu().numpy()
        n = len(keys)
        uniq = np.unique(keys)
        if n == n_keys:
            assert 0.35 < 1 - len(uniq) / n < 0.55  # the configuration's "about 40 % duplicates"
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out.shape == (n, dim)
        assert out.cpu().numpy().tobytes() == ORC.gather(table, keys, omp=True).tobytes()
        counted = uniq if dedup else keys
        assert _basics.last_group_offset(0) == [0, int((nid[counted] == 0).sum()), len(counted)]
    # the distinct keys and their inverse instead of the re-expanded rows
    rows, inverse = co.coll_torch_lookup_unique(0, batches[0])
    keys = batches[0].cpu().numpy()
    assert rows.shape[0] == len(np.unique(keys))
    assert torch.equal(rows[inverse.long()].view(torch.int32), emb.cuda()[batches[0]].view(torch.int32))


@pytest.mark.parametrize("impl,dedup", [("", False), ("SMMaskPhase", True)])
def test_config3_gnn_full_size_closed_form(impl, dedup, monkeypatch):
    """The same configuration at its full size: 100M rows x 128 fp32 = 51.2 GB pinned, 25M rows (12.8 GB) cached, 2^20
    int64 keys per batch.  table[r, c] = (128 r + c) mod 2^32 as int32 bits, so every output word is checked on the
    device without a second copy of the rows; cached set and group sizes against the oracle's placement."""
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    if dedup:
        monkeypatch.setenv("COLL_DEDUP_KEYS", "1")
    n_item, dim, pct, n_keys = 100_000_000, 128, 0.25, 1 << 20
    pre, batches, nid = _gnn_case(n_item, n_keys, 50)
    co.config(make_config(n_item, pct, threads=16))
    co.coll_cache_record_init(0)
    for b in pre:
        co.coll_torch_record(0, b)
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    words = emb.view(torch.int32)
    col = torch.arange(dim, device="cuda", dtype=torch.int64)
    for r0 in range(0, n_item, 4_000_000):
        r = torch.arange(r0, min(n_item, r0 + 4_000_000), device="cuda", dtype=torch.int64)
        words[r0 : r0 + len(r)].copy_(((r.unsqueeze(1) * dim + col) & 0xffffffff).to(torch.int32))
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["table_kind"] == 1 and info["cached_rows"] == 25_000_000 == int((nid == 0).sum())
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct)
    got_cached = np.zeros(info["cached_rows"], np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got_cached.ctypes.data, len(got_cached)) == len(got_cached)
    assert np.array_equal(got_cached, np.nonzero(nid == 0)[0])
    for kt in batches:
        n = len(kt)
        out = co.coll_torch_lookup_key_t_val_ret(0, kt, False)
        assert out.shape == (n, dim)
        want = ((kt.unsqueeze(1) * dim + col) & 0xffffffff).to(torch.int32)
        assert torch.equal(out.view(torch.int32), want)
        keys = kt.cpu().numpy()
        counted = np.unique(keys) if dedup else keys
        if n == n_keys:
            assert 0.3 < 1 - len(np.unique(keys)) / n < 0.45
        assert _basics.last_group_offset(0) == [0, int((nid[counted] == 0).sum()), len(counted)]


@pytest.mark.parametrize("impl", ["", "SMMaskPhase"])
def test_config4_dlr_26_fields_through_the_lookup_layer(impl, tmp_path, monkeypatch):
    """The DLR-shaped configuration with 262,144 rows per field (26 x 8M rows = 106 GB cannot be pinned on one box):
    26 tables of 128 fp32 concatenated into one id space, key = f * rows_per_field + perm_f[rank] with an independent
    seeded permutation and Zipf(1.2) ranks per field, the hottest 35.8 % of the id space cached (the configuration's 40 GB of
    106 GB), batches of 8192 samples x 26 fields as an int64 [8192, 26] tensor through the serving stack's LookupLayer,
    which returns [8192, 26, 128]."""
    import json
    import collcache.torch.serving as hps
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    fields, per_field, dim, samples = 26, 262_144, 128, 8192
    n_item = fields * per_field
    pct = (40e9 / 512) / (26 * 8_388_608)
    cfg = {"iteration_per_epoch": 200, "epoch": 1, "coll_cache_enable_refresh": False,
           "models": [{"model": "dlrm", "sparse_files": ["mock_%d_%d" % (n_item, dim)], "gpucacheper": pct,
                       "max_batch_size": samples, "deployed_device_list": [0],
                       "maxnum_catfeature_query_per_table_per_sample": [fields], "embedding_vecsize_per_table": [dim],
                       "max_vocabulary_size": [n_item]}]}
    path = tmp_path / "ps_config.json"
    path.write_text(json.dumps(cfg))
    gp = torch.Generator(device="cuda").manual_seed(2)
    perms = [torch.randperm(per_field, generator=gp, device="cuda", dtype=torch.int64) for _ in range(fields)]
    gz = torch.Generator(device="cuda").manual_seed(3)

    def make_batch(n_samples):
        cols = [perms[f][zipf_ranks_dev(n_samples, per_field, 1.2, gz)] + f * per_field for f in range(fields)]
        return torch.stack(cols, dim=1)  # [samples, fields]

    try:
        assert hps.Config(ps_config_file=str(path)) == "OK"
        pre = [make_batch(samples) for _ in range(100)]
        for b in pre:
            hps.record_hotness(b)
        emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
        g = torch.Generator(device="cuda").manual_seed(1)
        for r0 in range(0, n_item, per_field * 2):
            emb[r0 : r0 + per_field * 2].copy_(torch.randn((per_field * 2, dim), generator=g, device="cuda"))
        table = emb.numpy()
        assert hps.Init(ps_config_file=str(path), global_batch_size=samples, emb_table=emb) == "OK"
        stream = torch.cat([b.reshape(-1) for b in pre]).cpu().numpy().astype(np.uint32)
        want_cached, nid = expected_cached_set(stream, n_item, pct)
        info = _basics.info(0)
        assert info["cached_rows"] == len(want_cached) == int(n_item * (pct * 100 / 100.0))
        got_cached = np.zeros(len(want_cached), np.uint32)
        assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got_cached.ctypes.data, len(got_cached)) == len(want_cached)
        assert np.array_equal(got_cached, want_cached)
        layer = hps.LookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim, emb_vec_dtype=torch.float32)
        for n_samples in (samples, samples, 1000, 1, samples):
            keys = make_batch(n_samples)
            assert keys.shape == (n_samples, fields) and keys.dtype == torch.int64
            out = layer(keys)
            assert tuple(out.shape) == (n_samples, fields, dim) and out.dtype == torch.float32
            flat = keys.reshape(-1).cpu().numpy()
            # every field's keys stay inside that field's table
            assert np.array_equal(flat.reshape(n_samples, fields) // per_field, np.tile(np.arange(fields), (n_samples, 1)))
            assert out.cpu().numpy().tobytes() == ORC.gather(table, flat, omp=True).tobytes()
            assert _basics.last_group_offset(0) == [0, int((nid[flat] == 0).sum()), len(flat)]
    finally:
        hps.Shutdown()


@pytest.mark.parametrize("table_kind", ["FLAT", "HASH"])
@pytest.mark.parametrize("impl", ["", "SMMaskPhase"])
def test_refresh_on_one_stream_while_lookups_run_on_another(table_kind, impl, monkeypatch):
    """Stream-ordered lookups are enqueued on a stream of the caller's while a second thread refreshes the cache, in
    background mode, on the default stream: the refresh must wait for the lookups in flight on the OTHER stream (and,
    in the factored mode, for the gathers on the library's own streams) before it overwrites the slots of the rows it
    evicted.  Every output is table[keys]; at the end the cache holds what the oracle places for the last hotness."""
    monkeypatch.setenv("COLL_HASH_TABLE", table_kind)
    monkeypatch.setenv("COLL_REFRESH_SLEEP_US", "50")
    monkeypatch.setenv("COLL_REFRESH_BATCH_ROWS", "512")
    monkeypatch.setenv("COLL_HASH_REBUILD_FRAC", "0.02")
    if impl:
        monkeypatch.setenv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", impl)
    rng = np.random.default_rng(123)
    n_item, dim, pct = 80_000, 64, 0.2
    co.config(make_config(n_item, pct))
    co.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    co.coll_torch_record(0, torch.from_numpy(perm[zipf_ranks(rng, 150_000, n_item, 1.05)]))
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float32)
    table = fill_table(emb, rng)
    co.coll_torch_init_t(0, 0, emb, pct)
    stop, done, last_stream = [False], [0], [None]
    r2 = np.random.default_rng(5)

    def refresher():  # torch's current stream of this thread is the default stream
        while not stop[0] or done[0] < 3:
            p2 = r2.permutation(n_item)
            s = p2[zipf_ranks(r2, 150_000, n_item, 1.05)]
            co.coll_torch_record(0, torch.from_numpy(s))
            co.coll_torch_refresh(0, False)
            last_stream[0] = s
            done[0] += 1

    side = torch.cuda.Stream()
    t = threading.Thread(target=refresher)
    t.start()
    try:
        with torch.cuda.stream(side):
            for step in range(60):
                keep, clones, batches = [], [], []
                for _ in range(4):
                    keys = perm[zipf_ranks(rng, int(rng.integers(1, 40_000)), n_item, 1.05)]
                    kt = torch.from_numpy(keys).cuda()
                    keep.append(kt)
                    clones.append(co.coll_torch_lookup_async(0, kt, False).clone())
                    batches.append(keys)
                if step % 3 == 0:  # a blocking lookup in between settles the stream-ordered ones first
                    keys = perm[zipf_ranks(rng, 20_000, n_item, 1.05)]
                    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
                    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes(), step
                co.coll_torch_lookup_wait(0)
                for keys, c in zip(batches, clones):
                    assert c.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes(), step
    finally:
        stop[0] = True
        t.join()
    assert done[0] >= 3
    want_cached, nid = expected_cached_set(last_stream[0].astype(np.uint32), n_item, pct)
    got = np.zeros(len(want_cached), np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == len(want_cached)
    assert np.array_equal(got, want_cached)
    keys = rng.integers(0, n_item, size=30_000)
    out = co.coll_torch_lookup_key_t_val_ret(0, torch.from_numpy(keys).cuda(), False)
    assert out.cpu().numpy().tobytes() == ORC.gather(table, keys).tobytes()
    assert _basics.last_group_offset(0) == [0, int((nid[keys] == 0).sum()), len(keys)]
