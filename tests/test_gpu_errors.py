"""Error behaviour at the boundary on a GPU box: the reference's convention is CHECK -> message -> abort(), and a bad
key must never fault the GPU.  Each case runs in a child process (the parent never touches the GPU here)."""
import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

PRELUDE = textwrap.dedent("""
    import sys
    sys.path.insert(0, %r)
    import numpy as np, torch
    import collcache.torch as co
    cfg = lambda n, pct: {"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
                          "num_global_step_per_epoch": 10, "num_epoch": 1, "num_total_item": n, "omp_thread_num": 4}
""" % os.path.join(ROOT, "ugache_amd"))


def run(body, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([sys.executable, "-c", PRELUDE + textwrap.dedent(body)], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, env=e, timeout=170)


@pytest.mark.parametrize("pct", [1.0, 0.0, 0.3])
def test_key_out_of_range_aborts_with_a_message_instead_of_faulting(pct):
    p = run("""
        n = 5000
        co.config(cfg(n, %r)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, n, 3, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, n, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, %r)
        good = co.coll_torch_lookup_key_t_val_ret(0, torch.arange(100, dtype=torch.int32, device="cuda"), False)
        assert torch.equal(good.cpu(), emb[:100])
        print("good lookup ok", flush=True)
        bad = torch.tensor([1, 2, n, 3], dtype=torch.int32, device="cuda")
        co.coll_torch_lookup_key_t_val_ret(0, bad, False)
        print("survived")
    """ % (pct, pct))
    assert "good lookup ok" in p.stdout and "survived" not in p.stdout
    assert p.returncode == -6, p.stderr[-2000:]
    assert "extraction kernels reported status" in p.stderr and "outside the table" in p.stderr


@pytest.mark.parametrize("pct", [1.0, 0.3])
def test_stream_ordered_lookup_reports_a_bad_key_at_the_wait(pct):
    p = run("""
        n = 5000
        co.config(cfg(n, %r)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, n, 3, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, n, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, %r)
        bad = torch.tensor([1, 2, n + 7, 3], dtype=torch.int64, device="cuda")
        co.coll_torch_lookup_async(0, bad, False)
        torch.cuda.synchronize()
        print("enqueue returned", flush=True)
        co.coll_torch_lookup_wait(0)
        print("survived")
    """ % (pct, pct))
    assert "enqueue returned" in p.stdout and "survived" not in p.stdout
    assert p.returncode == -6, p.stderr[-2000:]
    assert "extraction kernels reported status" in p.stderr


def test_ordinary_host_memory_is_refused_for_a_partial_cache():
    p = run("""
        n = 1000
        co.config(cfg(n, 0.5)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, n, dtype=torch.int32))
        emb = torch.randn(n, 16)            # pageable host memory, not from coll_torch_create_emb_shm
        co.coll_torch_init_t(0, 0, emb, 0.5)
        print("survived")
    """)
    assert p.returncode == -6 and "survived" not in p.stdout
    assert "must be pinned" in p.stderr


def test_ordinary_host_memory_is_fine_for_a_full_cache():
    p = run("""
        n = 1000
        co.config(cfg(n, 1.0))
        emb = torch.randn(n, 16)
        co.coll_torch_init_t(0, 0, emb, 1.0)
        q = torch.randint(0, n, (333,), dtype=torch.int32)
        out = co.coll_torch_lookup_key_t_val_ret(0, q.cuda(), False)
        assert torch.equal(out.cpu(), emb[q.long()])
        print("survived")
    """)
    assert p.returncode == 0 and "survived" in p.stdout, p.stderr[-2000:]


def test_mock_table_env_is_rejected():
    p = run("""
        n = 1000
        co.config(cfg(n, 1.0))
        emb = torch.randn(n, 16)
        co.coll_torch_init_t(0, 0, emb, 1.0)
        print("survived")
    """, env={"SAMGRAPH_EMPTY_FEAT": "10"})
    assert p.returncode == -6 and "survived" not in p.stdout
    assert "SAMGRAPH_EMPTY_FEAT" in p.stderr


@pytest.mark.parametrize("gpu_record", ["0", "1"])
def test_a_process_that_never_calls_shutdown_still_exits_cleanly(gpu_record):
    """the serving loop owns a record thread and a refresh thread: a process that just ends (no coll_torch_shutdown,
    no join of the last refresh) must end with status 0, not in std::terminate or a failed call at unload"""
    p = run("""
        n = 60000
        co.config(cfg(n, 0.2)); co.coll_cache_record_init(0)
        rng = np.random.default_rng(0)
        co.coll_torch_record(0, torch.from_numpy(rng.zipf(1.2, 200000) % n).to(torch.int32))
        emb = co.coll_torch_create_emb_shm(0, n, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, 0.2)
        co.coll_torch_forward_config(True, 3, 0.5, True)
        for step in range(8):
            keys = torch.from_numpy((rng.zipf(1.1, 20000) + step * 1000) % n).to(torch.int64).cuda()
            out = co.coll_torch_forward(0, keys)
            assert torch.equal(out.cpu(), emb[keys.cpu()])
        # ... nor wait for the steps it enqueued last, whose prefixes nobody has counted yet
        kept = [torch.from_numpy(rng.integers(0, n, 4000)).cuda() for _ in range(3)]
        for keys in kept:
            co.coll_torch_forward(0, keys, stream_ordered=True)
        print("forwards ok", flush=True)
    """, env={"COLL_GPU_RECORD": gpu_record, "COLL_REFRESH_SLEEP_US": "20000"})
    assert "forwards ok" in p.stdout, p.stderr[-2000:]
    assert p.returncode == 0, p.stderr[-2000:]


@pytest.mark.parametrize("preload", ["1", "0"])
def test_a_process_that_configures_and_ends_at_once_exits_cleanly(preload):
    """coll_cache_config starts a helper thread that loads the kernels onto the device; a process that ends right
    behind the call (no build, no shutdown), one that shuts down right behind it, and one that configures again
    afterwards all end with status 0"""
    for body in ("""
        co.config(cfg(1000, 0.2))
        print("configured", flush=True)
    """, """
        co.config(cfg(1000, 0.2))
        co.coll_torch_shutdown()
        co.config(cfg(2000, 0.5)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, 2000, 3, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, 2000, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, 0.5)
        keys = torch.arange(0, 2000, 7, dtype=torch.int64, device="cuda")
        assert torch.equal(co.coll_torch_lookup_key_t_val_ret(0, keys, False).cpu(), emb[keys.cpu()])
        print("configured", flush=True)
    """):
        p = run(body, env={"COLL_PRELOAD_KERNELS": preload})
        assert "configured" in p.stdout, p.stderr[-2000:]
        assert p.returncode == 0, p.stderr[-2000:]


def test_pooled_lookup_with_offsets_beyond_the_ids_aborts_with_a_message():
    p = run("""
        n = 5000
        co.config(cfg(n, 0.3)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, n, 3, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, n, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, 0.3)
        ids = torch.arange(40, dtype=torch.int64, device="cuda")
        off = torch.arange(0, 41, 4, dtype=torch.int64, device="cuda")
        good = co.coll_torch_lookup_pooled(0, ids, off)
        assert torch.allclose(good.cpu(), emb[:40].reshape(10, 4, 32).sum(1), atol=1e-5)
        print("good lookup ok", flush=True)
        off[-1] = 4000
        co.coll_torch_lookup_pooled(0, ids, off)
        print("survived")
    """)
    assert "good lookup ok" in p.stdout and "survived" not in p.stdout, p.stderr[-2000:]
    assert p.returncode == -6, p.stderr[-2000:]
    assert "offsets of a pooled lookup" in p.stderr


def test_stream_ordered_pooled_lookup_reports_bad_offsets_at_the_wait():
    p = run("""
        n = 5000
        co.config(cfg(n, 0.3)); co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, n, 3, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, n, 32, torch.float32); emb.normal_()
        co.coll_torch_init_t(0, 0, emb, 0.3)
        ids = torch.arange(40, dtype=torch.int64, device="cuda")
        off = torch.arange(0, 41, 4, dtype=torch.int64, device="cuda")
        off[3] = -2
        out = co.coll_torch_lookup_pooled(0, ids, off, stream_ordered=True)
        torch.cuda.synchronize()
        print("enqueued", flush=True)
        co.coll_torch_lookup_wait(0)
        print("survived")
    """)
    assert "enqueued" in p.stdout and "survived" not in p.stdout, p.stderr[-2000:]
    assert p.returncode == -6, p.stderr[-2000:]
    assert "offsets of a pooled lookup" in p.stderr
