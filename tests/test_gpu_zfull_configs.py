"""The two largest configurations at the size they are benchmarked at, through the drop-in boundary, with checks that
need no second copy of the table and no ranking of the whole key space on the host:

  * table words are a closed form of (row, column), so every output word is checked on the device;
  * the cached set is checked against the placement rule itself, evaluated on the device over the recorded key
    stream: rows in descending order of (count, row) -- FreqRecorder's order (freq_recorder.cc:274-281), which the
    oracle's orc_freq_rank restates and which a small sample at the top of each test compares with that oracle --
    followed by the never-recorded rows in ascending order (the tie rule of this build), the first num_cached of them;
  * group sizes follow from that set.

Smaller instances of the same configurations are compared with the oracle proper in test_gpu_collcache.py."""
import json
import os
import sys

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
    from collcache.common import _basics

ENV_VARS = ("COLL_HASH_TABLE", "COLL_GPU_RECORD", "COLL_GPU_REFRESH", "COLL_GPU_REFRESH_KEEP", "COLL_GPU_REFRESH_STABLE",
            "COLL_MISS_STAGE_ROWS", "SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL", "COLL_DEDUP_KEYS", "COLL_GPU_RECORD_SEED")


@pytest.fixture(autouse=True)
def _fresh_cache(monkeypatch):
    for v in ENV_VARS:
        monkeypatch.delenv(v, raising=False)
    yield
    if torch.cuda.is_available():
        co.coll_torch_shutdown()
        torch.cuda.empty_cache()


def zipf_ranks_dev(n, space, s, gen):
    """bounded-Pareto inverse CDF on the device (ranks in [0, space))"""
    u = torch.rand(n, generator=gen, device="cuda", dtype=torch.float64)
    h = float(space)
    r = torch.floor(((h ** (1.0 - s) - 1.0) * u + 1.0) ** (1.0 / (1.0 - s))).to(torch.int64) - 1
    return r.clamp_(0, space - 1)


def top_rows(rows_seen, n_item, num_cached):
    """bool[n_item] on the device: the num_cached best rows of the placement rule for the recorded rows `rows_seen`
    (a list of int64 device tensors of row numbers); also returns how many distinct rows were recorded"""
    counts = torch.zeros(n_item, dtype=torch.int32, device="cuda")
    one = None
    for r in rows_seen:
        if one is None or len(one) != len(r):
            one = torch.ones(len(r), dtype=torch.int32, device="cuda")
        counts.index_add_(0, r, one)
    observed = counts > 0
    n_obs = int(observed.sum())
    mask = torch.zeros(n_item, dtype=torch.bool, device="cuda")
    if n_obs <= num_cached:
        # every recorded row is in; the rest are the lowest never-recorded rows
        need = num_cached - n_obs
        pos = torch.cumsum((~observed).to(torch.int32), 0)  # never-recorded rows, counted in ascending order
        mask = observed | ((~observed) & (pos <= need))
    else:
        rows_obs = torch.nonzero(observed).squeeze(1)
        entry = (counts[rows_obs].to(torch.int64) << 32) | rows_obs  # FreqEntry as one word: (cnt << 32) | key
        best = torch.sort(entry, descending=True).values[:num_cached]
        mask[best & 0xffffffff] = True
    return mask, n_obs


def check_rule_against_the_oracle(seed):
    """the placement rule above on a sample the oracle ranks in no time: same first K rows as orc_freq_rank followed by
    the never-recorded rows ascending"""
    rng = np.random.default_rng(seed)
    n_item = 50_000
    stream = (rng.zipf(1.3, size=120_000) % n_item).astype(np.int64)
    rank_k, _ = ORC.full_rank(stream.astype(np.uint32), n_item)
    for k in (1, 700, len(np.unique(stream)), len(np.unique(stream)) + 9, n_item):
        mask, _ = top_rows([torch.from_numpy(stream).cuda()], n_item, k)
        want = np.zeros(n_item, bool)
        want[rank_k[:k]] = True
        assert np.array_equal(mask.cpu().numpy(), want), k


def cached_mask_from_library(n_item, n_cached):
    got = np.zeros(n_cached, np.uint32)
    assert _basics.C_LIB_CTYPES.coll_cache_get_cached_keys(0, got.ctypes.data, len(got)) == n_cached
    rows = torch.from_numpy(got.astype(np.int64)).cuda()
    assert bool((rows[1:] > rows[:-1]).all())  # reported ascending, no duplicates
    mask = torch.zeros(n_item, dtype=torch.bool, device="cuda")
    mask[rows] = True
    return mask


@pytest.mark.parametrize("refresh_on", ["host", "device"])
def test_config5_sparse_ids_hash_table_full_size(refresh_on, monkeypatch):
    """BASELINE configuration 5 at its stated size: 500M rows x 64 fp16 = 64 GB pinned, ids (row * odd) mod 2^40, 50M
    rows cached behind the open-addressing table (71.4M buckets at load 0.7), batches of up to 2^20 Zipf(1.05) ids.
    table word [r, w] = (32 r + w) mod 2^32.  Build, lookups of several sizes, then a refresh that replaces about 1 % of
    the cache -- ranked on the host from recorded batches, or counted, ranked and placed on the device -- and lookups
    again; with the device-side counters also a second refresh after 60M distinct rows have been looked up, which
    takes the two passes over all 500M counters and cuts a tie class of millions of rows."""
    check_rule_against_the_oracle(5)
    if refresh_on == "device":
        monkeypatch.setenv("COLL_GPU_RECORD", "1")
        monkeypatch.setenv("COLL_GPU_REFRESH", "1")
    MUL, BITS = 0x9E3779B97F4A7C15, 40
    n_item, dim, pct, n_keys = 500_000_000, 64, 0.1, 1 << 20
    words_per_row = dim // 2
    num_cached = int(n_item * (pct * 100 / 100.0))
    assert num_cached == 50_000_000

    def ids_of(rows_t):
        mul = torch.tensor(MUL - (1 << 64), dtype=torch.int64, device=rows_t.device)
        return (rows_t * mul) & ((1 << BITS) - 1)

    co.config({"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
               "num_global_step_per_epoch": 100, "num_epoch": 1, "num_total_item": n_item, "omp_thread_num": 16})
    _basics.set_key_map(MUL, BITS)
    co.coll_cache_record_init(0)
    gp = torch.Generator(device="cuda").manual_seed(2)
    perm = torch.randperm(n_item, generator=gp, device="cuda", dtype=torch.int64)
    gz = torch.Generator(device="cuda").manual_seed(3)

    def batch(n):
        return perm[zipf_ranks_dev(n, n_item, 1.05, gz)]

    pre = [batch(n_keys) for _ in range(50)]
    for b in pre:
        co.coll_torch_record(0, ids_of(b).cpu())
    emb = co.coll_torch_create_emb_shm(0, n_item, dim, torch.float16)
    words = emb.view(torch.int32)
    assert tuple(words.shape) == (n_item, words_per_row)
    col = torch.arange(words_per_row, device="cuda", dtype=torch.int64)
    for r0 in range(0, n_item, 8_000_000):
        r = torch.arange(r0, min(n_item, r0 + 8_000_000), device="cuda", dtype=torch.int64)
        words[r0 : r0 + len(r)].copy_(((r.unsqueeze(1) * words_per_row + col) & 0xffffffff).to(torch.int32))
    co.coll_torch_init_t(0, 0, emb, pct)
    info = _basics.info(0)
    assert info["table_kind"] == 3 and info["row_bytes"] == 128 and info["key_space"] == n_item
    assert info["cached_rows"] == num_cached
    assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct)
    cached, n_obs = top_rows(pre, n_item, num_cached)
    assert n_obs < num_cached  # the cache holds every presampled row and is filled up with never-recorded ones
    assert torch.equal(cached_mask_from_library(n_item, num_cached), cached)

    counted = []  # rows of every lookup since the device-side counters were last reset (by the build or a refresh)

    def lookup_and_check(rows_b, cached):
        keys = ids_of(rows_b).contiguous()
        out = co.coll_torch_lookup_key_t_val_ret(0, keys, False)
        assert out.dtype == torch.float16 and tuple(out.shape) == (len(rows_b), dim)
        want = ((rows_b.unsqueeze(1) * words_per_row + col) & 0xffffffff).to(torch.int32)
        assert torch.equal(out.view(torch.int32), want)
        assert _basics.last_group_offset(0) == [0, int(cached[rows_b].sum()), len(rows_b)]
        counted.append(rows_b)

    for n in (n_keys, n_keys, n_keys // 3 + 5, 65_536, 1):
        rows_b = batch(n)
        assert n < 1000 or int(ids_of(rows_b).max()) > (1 << 32)  # genuinely wide ids
        lookup_and_check(rows_b, cached)

    # a refresh that replaces about 1 % of the cache: 500k rows the cache does not hold become the hottest
    cold = torch.nonzero(~cached).squeeze(1)
    cold = cold[torch.randperm(len(cold), generator=gp, device="cuda")[:500_000]]
    if refresh_on == "host":
        recorded = [batch(n_keys) for _ in range(20)] + [cold] * 8
        for b in recorded:
            co.coll_torch_record(0, ids_of(b).cpu())
    else:
        for _ in range(2):
            lookup_and_check(cold, cached)
        recorded = list(counted)  # the device-side counters have seen every lookup since the build
    co.coll_torch_refresh(0, True)
    counted.clear()
    new_cached, n_obs = top_rows(recorded, n_item, num_cached)
    assert n_obs < num_cached
    info = _basics.info(0)
    assert info["cached_rows"] == num_cached and info["free_slots"] + info["cached_rows"] == info["capacity_rows"]
    assert torch.equal(cached_mask_from_library(n_item, num_cached), new_cached)
    assert int((new_cached & ~cached).sum()) >= 500_000  # the cold rows came in
    cached = new_cached
    for n in (n_keys, 70_001):
        lookup_and_check(batch(n), cached)
    lookup_and_check(cold, cached)
    assert _basics.last_group_offset(0) == [0, 500_000, 500_000]

    if refresh_on == "device":
        # More rows observed than the cache holds: 60M distinct rows looked up once each on top of the three lookups
        # above.  The placement now needs the histogram and split passes over all 500M counters and cuts the class of
        # rows counted once, larger row numbers first.
        for i in range(60):
            lookup_and_check(perm[i * 1_000_000 : (i + 1) * 1_000_000], cached)
        co.coll_torch_refresh(0, True)
        new_cached, n_obs = top_rows(counted, n_item, num_cached)
        counted.clear()
        assert n_obs > num_cached
        assert torch.equal(cached_mask_from_library(n_item, num_cached), new_cached)
        lookup_and_check(batch(n_keys), new_cached)
        lookup_and_check(cold, new_cached)


def test_config4_dlr_26_fields_half_size_through_the_lookup_layer(tmp_path):
    """BASELINE configuration 4 at the largest size one box pins (26 x 4M rows x 128 fp32 = 55.8 GB; the full 106 GB
    cannot be pinned): key = f * rows_per_field + perm_f[rank] with Zipf(1.2) ranks and an independent seeded
    permutation per field, 20 GB of rows cached, batches of 8192 samples x 26 fields as an int64 [8192, 26] tensor
    through the serving stack's LookupLayer, which returns [8192, 26, 128].  table word [r, c] = (128 r + c) mod 2^32."""
    import collcache.torch.serving as hps
    check_rule_against_the_oracle(4)
    fields, per_field, dim, samples = 26, 4_194_304, 128, 8192
    n_item = fields * per_field
    pct = (20e9 / 512) / n_item
    num_cached = int(n_item * (pct * 100 / 100.0))
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
        words = emb.view(torch.int32)
        col = torch.arange(dim, device="cuda", dtype=torch.int64)
        for r0 in range(0, n_item, 4_000_000):
            r = torch.arange(r0, min(n_item, r0 + 4_000_000), device="cuda", dtype=torch.int64)
            words[r0 : r0 + len(r)].copy_(((r.unsqueeze(1) * dim + col) & 0xffffffff).to(torch.int32))
        assert hps.Init(ps_config_file=str(path), global_batch_size=samples, emb_table=emb) == "OK"
        info = _basics.info(0)
        assert info["table_kind"] == 1 and info["row_bytes"] == 512 and info["key_space"] == n_item
        assert info["cached_rows"] == num_cached and info["cached_rows"] * 512 > 19.9e9
        assert info["capacity_rows"] == ORC.lib.orc_cache_capacity(n_item, pct)
        cached, n_obs = top_rows([b.reshape(-1) for b in pre], n_item, num_cached)
        assert n_obs < num_cached
        assert torch.equal(cached_mask_from_library(n_item, num_cached), cached)
        layer = hps.LookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim, emb_vec_dtype=torch.float32)
        field_of = torch.arange(fields, device="cuda", dtype=torch.int64)
        for n_samples in (samples, samples, 1000, 1, samples):
            keys = make_batch(n_samples)
            assert tuple(keys.shape) == (n_samples, fields) and keys.dtype == torch.int64
            assert bool((keys // per_field == field_of).all())  # every field's keys stay inside that field's table
            assert int(keys.max()) > (1 << 26)
            out = layer(keys)
            assert tuple(out.shape) == (n_samples, fields, dim) and out.dtype == torch.float32
            want = ((keys.reshape(-1, 1) * dim + col) & 0xffffffff).to(torch.int32)
            assert torch.equal(out.view(torch.int32).reshape(-1, dim), want)
            flat = keys.reshape(-1)
            assert _basics.last_group_offset(0) == [0, int(cached[flat].sum()), len(flat)]
    finally:
        hps.Shutdown()
