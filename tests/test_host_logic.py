"""CPU tests of the host logic behind the C-ABI (no GPU call): config marshalling, hotness recording and ranking,
frequency-ranked placement — each against the oracle / closed forms."""
import ctypes
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))

import collcache.common as cc  # noqa: E402
from oracle_lib import Oracle  # noqa: E402

ORC = Oracle()
C = cc._basics.C_LIB_CTYPES


def _config(num_total_item, pct=0.1, threads=4):
    cc._basics.shutdown()
    cc._basics.config({"cache_percentage": pct, "_cache_policy": cc.kCollCacheAsymmLink, "num_device": 1,
                       "num_global_step_per_epoch": 10, "num_epoch": 2, "num_total_item": num_total_item,
                       "omp_thread_num": threads})


@pytest.fixture(autouse=True)
def _teardown():
    yield
    cc._basics.shutdown()


def _zipf_keys(rng, n, space, s):
    u = rng.random(n)
    h = float(space)
    r = np.floor(((h ** (1 - s) - 1) * u + 1) ** (1 / (1 - s))).astype(np.int64)
    return np.clip(r - 1, 0, space - 1)


@pytest.mark.parametrize("kdtype", [np.uint32, np.int64])
def test_record_and_rank_match_oracle(kdtype):
    rng = np.random.default_rng(3)
    n_item = 50_000
    _config(n_item)
    cc._basics.coll_cache_record_init(0)
    perm = rng.permutation(n_item)
    stream = []
    for _ in range(5):
        keys = perm[_zipf_keys(rng, 70_000, n_item, 1.1)].astype(kdtype)
        stream.append(keys)
        if kdtype == np.int64:
            C.coll_cache_record_i64(0, keys.ctypes.data, len(keys))
        else:
            C.coll_cache_record(0, keys.ctypes.data, len(keys))
    assert C.coll_cache_max_num_keys() == 70_000
    allk = np.concatenate(stream).astype(np.uint32)
    want_k, want_c = ORC.freq_rank(allk)
    got_k = np.zeros(n_item, np.uint32)
    got_c = np.zeros(n_item, np.uint32)
    m = C.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
    assert m == len(want_k)
    assert np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c)
    # the counts were consumed: ranking again sees nothing new
    assert C.coll_cache_rank_hotness(0, None, None, 0) == 0


@pytest.mark.parametrize("batch", [900, 70_000])
def test_every_round_of_counts_starts_from_zero(batch):
    """Ranking drains the counters into a second array and recording goes on in a third: over several rounds
    (small batches take the one-thread loop, large ones the parallel one) each ranking holds that round's keys only"""
    rng = np.random.default_rng(11)
    n_item = 30_000
    _config(n_item)
    cc._basics.coll_cache_record_init(0)
    for rnd in range(4):
        keys = [(rng.zipf(1.3, size=batch) % n_item).astype(np.uint32) for _ in range(3)]
        for k in keys:
            C.coll_cache_record(0, k.ctypes.data, len(k))
        want_k, want_c = ORC.freq_rank(np.concatenate(keys))
        got_k = np.zeros(n_item, np.uint32)
        got_c = np.zeros(n_item, np.uint32)
        m = C.coll_cache_rank_hotness(0, got_k.ctypes.data, got_c.ctypes.data, n_item)
        assert m == len(want_k), rnd
        assert np.array_equal(got_k[:m], want_k) and np.array_equal(got_c[:m], want_c), rnd


@pytest.mark.parametrize("pct", [0.0, 0.1, 0.25, 0.333, 0.999])
def test_placement_matches_oracle_rep_solve(pct):
    rng = np.random.default_rng(5)
    n_item = 20_011
    stream = (rng.zipf(1.2, size=100_000) % n_item).astype(np.uint32)
    rank_k, rank_c = ORC.full_rank(stream, n_item)
    want, want_n = ORC.rep_solve(rank_k, n_item, pct * 100)
    got = np.zeros(n_item, np.uint32)
    n_cached = C.coll_cache_place_ranked(rank_k.ctypes.data, rank_c.ctypes.data, n_item, pct, got.ctypes.data)
    assert n_cached == want_n == int(n_item * (pct * 100 / 100.0))
    assert np.array_equal(got, want)
    # closed form: the cached set is the n_cached keys with the largest (count, key)
    cached = np.nonzero(got == 0)[0]
    assert set(cached.tolist()) == set(rank_k[:n_cached].tolist())


@pytest.mark.parametrize("pct,n_stream", [(0.05, 100_000), (0.4, 100_000), (0.9, 3_000), (0.0, 10), (0.999, 1)])
def test_placement_from_the_recorder_matches_the_full_rank_list(pct, n_stream):
    """the solver fed with the observed keys only (what init and refresh run) gives the placement of the full rank
    list, also when the cache is larger than the observed set and never-recorded keys fill it in ascending order"""
    rng = np.random.default_rng(n_stream)
    n_item = 70_000
    _config(n_item, pct)
    cc._basics.coll_cache_record_init(0)
    stream = (rng.zipf(1.2, size=n_stream) % n_item).astype(np.uint32)
    C.coll_cache_record(0, stream.ctypes.data, len(stream))
    rank_k, _ = ORC.full_rank(stream, n_item)
    want, want_n = ORC.rep_solve(rank_k, n_item, pct * 100)
    got = np.full(n_item, 7, np.uint32)
    n_cached = C.coll_cache_place_recorded(0, n_item, pct, got.ctypes.data)
    assert n_cached == want_n
    assert np.array_equal(got, want)
    if pct == 0.9:
        assert want_n > len(np.unique(stream))  # this case did reach into the never-recorded keys


def test_config_is_once_per_process_and_requires_keys():
    # violations abort() like the reference's CHECKs, so they are observed in a child process
    code = textwrap.dedent("""
        import sys
        sys.path.insert(0, %r)
        import collcache.common as cc
        cfg = {"cache_percentage": 0.1, "_cache_policy": 13, "num_device": 1, "num_global_step_per_epoch": 1,
               "num_epoch": 1, "num_total_item": 10, "omp_thread_num": 1}
        mode = sys.argv[1]
        if mode == "twice":
            cc._basics.config(cfg); cc._basics.config(cfg)
        elif mode == "missing":
            del cfg["num_total_item"]; cc._basics.config(cfg)
        elif mode == "two_gpus":
            cfg["num_device"] = 2; cc._basics.config(cfg)
        elif mode == "ok":
            cc._basics.config(cfg); cc._basics.coll_cache_record_init(0)
        print("survived")
    """ % os.path.join(ROOT, "ugache_amd"))
    for mode, ok in [("ok", True), ("twice", False), ("missing", False), ("two_gpus", False)]:
        p = subprocess.run([sys.executable, "-c", code, mode], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if ok:
            assert p.returncode == 0 and "survived" in p.stdout, p.stderr
        else:
            assert p.returncode == -6 and "survived" not in p.stdout  # SIGABRT
            assert "Check failed" in p.stderr


def test_wait_one_child_reports_failed_children():
    """coll_cache_wait_one_child (operation.cc:219-230): 1 for a child that exits non-zero or dies by signal."""
    code = textwrap.dedent("""
        import os, sys
        sys.path.insert(0, %r)
        import collcache.common as cc
        res = []
        for how in ("ok", "fail", "abort"):
            pid = os.fork()
            if pid == 0:
                if how == "ok": os._exit(0)
                if how == "fail": os._exit(3)
                os.abort()
            res.append(cc._basics.wait_one_child())
        print(res)
    """ % os.path.join(ROOT, "ugache_amd"))
    p = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert p.returncode == 0, p.stderr
    assert "[0, 1, 1]" in p.stdout


def test_profiler_hooks_store_and_report(capfd):
    _config(100)
    cc._basics.log_step_by_key(3, cc.kLogL1FeatureBytes, 4096.0)
    cc._basics.log_step_by_key(3, cc.kLogL2CacheCopyTime, 0.5)
    assert cc._basics.step_value(3, cc.kLogL1FeatureBytes) == 4096.0
    assert cc._basics.step_value(4, cc.kLogL1FeatureBytes) == 0.0
    cc._basics.report_step(3)
    out = capfd.readouterr().out
    assert "cache feat copy 0.500000" in out and "feature nbytes" in out


def _scrape_profiler_block(text):
    """what the reference's eval scripts do with a profiler block (eval/gnn/common/common_parser.py:311-336): the
    first word inside '[' of a header line prefixes the keys, every other line is 'L<n>' + cells split on '|', a cell
    is 'name value [unit]'"""
    import re
    unit = {"Bytes": 1, "KB": 1024, "MB": 1024 ** 2, "GB": 1024 ** 3}
    vals, prefix = {}, None
    for line in text.splitlines():
        if line.startswith("    ["):
            prefix = re.match(r"    \[([^ ]+) .*", line).group(1)
            continue
        if prefix is None or not line.startswith("        L"):
            continue
        line = line.strip()
        level, rest = line[:2], line[2:]
        for cell in rest.split("|"):
            item = prefix + " " + level + " " + cell.strip()
            m = re.match(r"([^\.]*) +([0-9\.]*)( (MB|Bytes|KB|GB))?", item)
            key, val = m.group(1).strip(), float(m.group(2))
            if m.group(3):
                val *= unit[m.group(4)]
            assert key not in vals, key
            vals[key] = val
    return vals


def test_step_report_has_the_layout_the_eval_scripts_scrape(capfd):
    _config(100)
    logged = {cc.kLogL1FeatureBytes: 3.0 * 1024 ** 2, cc.kLogL1MissBytes: 512.0 * 1024, cc.kLogL1RemoteBytes: 0.0,
              cc.kLogL2CacheCopyTime: 0.25, cc.kLogL3CacheGetIndexTime: 0.001, cc.kLogL3CacheCombineMissTime: 0.002,
              cc.kLogL3CacheCombineCacheTime: 0.003, cc.kLogL3CacheCombineRemoteTime: 0.0}
    for step, scale in ((0, 1.0), (1, 3.0)):
        for item, v in logged.items():
            cc._basics.log_step_by_key(step, item, v * scale)
    cc._basics.report_step_average(1)
    out = capfd.readouterr().out
    vals = _scrape_profiler_block(out)
    want = {"Step(average) L1 feature nbytes": 6.0 * 1024 ** 2, "Step(average) L1 miss nbytes": 1024.0 ** 2,
            "Step(average) L1 remote nbytes": 0.0, "Step(average) L2 cache feat copy": 0.5,
            "Step(average) L3 cache get_index": 0.002, "Step(average) L3 cache combine_miss": 0.004,
            "Step(average) L3 cache combine cache": 0.006, "Step(average) L3 cache combine remote": 0.0,
            "Step(average) L1 convert time": 0.0, "Step(average) L1 train": 0.0, "Step(average) L1 sample": 0.0}
    for k, v in want.items():
        assert k in vals, (k, sorted(vals))
        assert abs(vals[k] - v) <= 1e-6 * max(1.0, v), (k, vals[k], v)
    # the three header lines and every level's line count (7 + 3 + 8)
    assert out.count("Profiler Level") == 3 and out.count("\n        L1  ") == 7
    assert out.count("\n        L2  ") == 3 and out.count("\n        L3  ") == 8


def test_recorder_and_placement_reproduce_the_committed_golden_case():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "extract_small.json")) as f:
        g = json.load(f)
    n_item, pct = g["n_item"], g["cache_percentage"]
    _config(n_item, pct)
    cc._basics.coll_cache_record_init(0)
    stream = np.array(g["record_stream"], np.uint32)
    C.coll_cache_record(0, stream.ctypes.data, len(stream))
    got = np.full(n_item, 9, np.uint32)
    assert C.coll_cache_place_recorded(0, n_item, pct, got.ctypes.data) == len(g["cached_keys"])
    assert np.nonzero(got == 0)[0].tolist() == g["cached_keys"]
    C.coll_cache_record(0, stream.ctypes.data, len(stream))
    k = np.zeros(n_item, np.uint32)
    c = np.zeros(n_item, np.uint32)
    m = C.coll_cache_rank_hotness(0, k.ctypes.data, c.ctypes.data, n_item)
    assert k[:m].tolist() == g["rank_keys_observed"] and c[:m].tolist() == g["rank_counts_observed"]


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=120)
    assert p.returncode != 0 and p.stdout == ""
    assert "ONE GPU" in p.stderr and "--gpus 1" in p.stderr


def _ps_config(tmp_path, edit=None):
    import json
    cfg = {"iteration_per_epoch": 100, "epoch": 2, "coll_cache_refresh_iter": 7,
           "models": [{"model": "dlrm", "sparse_files": ["/models/dlrm_sparse.model"], "gpucacheper": 0.15,
                       "deployed_device_list": [0], "maxnum_catfeature_query_per_table_per_sample": [26],
                       "embedding_vecsize_per_table": [128], "max_vocabulary_size": [1000]}]}
    if edit:
        edit(cfg)
    p = tmp_path / "ps_config.json"
    p.write_text(json.dumps(cfg))
    return str(p)


def test_ps_config_is_read_like_the_serving_stack_reads_it(tmp_path):
    """keys, defaults and insisted-on keys of parameter_server_config (inference_utils.cpp:55-160)"""
    from collcache.torch.serving import PsConfig
    c = PsConfig(_ps_config(tmp_path))
    assert (c.iteration_per_epoch, c.epoch, c.coll_cache_refresh_iter) == (100, 2, 7)
    assert c.coll_cache_enable_refresh is False and c.use_multi_worker is False  # soft defaults
    assert c.coll_cache_policy == 13 and c.max_batch_size == 64 and c.i64_input_key is True
    assert c.model_name == "dlrm" and c.sparse_files == ["/models/dlrm_sparse.model"]
    assert abs(c.cache_size_percentage - 0.15) < 1e-12
    assert c.embedding_vecsize_per_table == [128] and c.max_vocabulary_size == [1000]
    assert c.maxnum_catfeature_query_per_table_per_sample == [26] and c.deployed_devices == [0]

    def no_gpucacheper(cfg):
        del cfg["models"][0]["gpucacheper"]
        del cfg["coll_cache_refresh_iter"]
        cfg["coll_cache_enable_refresh"] = True
        cfg["models"][0]["i64_input_key"] = False
    c = PsConfig(_ps_config(tmp_path, no_gpucacheper))
    assert abs(c.cache_size_percentage - 0.2) < 1e-12 and c.coll_cache_refresh_iter is None
    assert c.coll_cache_enable_refresh is True and c.i64_input_key is False


@pytest.mark.parametrize("broken", ["iteration_per_epoch", "epoch", "models", "sparse_files", "deployed_device_list",
                                    "embedding_vecsize_per_table", "two_models", "two_devices"])
def test_ps_config_without_a_required_key_aborts_with_a_message(tmp_path, broken):
    def edit(cfg):
        if broken in ("iteration_per_epoch", "epoch", "models"):
            del cfg[broken]
        elif broken == "two_models":
            cfg["models"].append(dict(cfg["models"][0]))
        elif broken == "two_devices":
            cfg["models"][0]["deployed_device_list"] = [0, 1]
        else:
            del cfg["models"][0][broken]
    path = _ps_config(tmp_path, edit)
    code = textwrap.dedent("""
        import sys
        sys.path.insert(0, %r)
        from collcache.torch.serving import PsConfig
        PsConfig(%r)
        print("not reached")
    """) % (os.path.join(ROOT, "ugache_amd"), path)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert r.returncode == -6 and "not reached" not in r.stdout  # abort(), like COLL_CHECK
    assert "ps_config:" in r.stderr
