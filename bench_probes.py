"""Stand-alone measurements behind the launch rules of the extraction kernels, callable as `bench.py --probe NAME`.

Each probe drives the kernels through the C-ABI of include/ugache_hip.h on synthetic inputs and times them with two
HIP events around back-to-back launches on the launch stream.  They measure and print; they check only that no launch
flagged an error (the parity tests check results).

  kpw       keys per wavefront of the fused lookup + gather kernel (ugk_extract_mix_i64), every shape forced in turn
            with UGK_MIX_KPW, by table kind, row size, miss rate and batch size
  row_span  uniformly random rows of 128 and 512 bytes gathered out of one large pinned host allocation, the rows drawn
            from its first S GiB: what small rows reach over the host link, and how that depends on the span
  cu_mask   a host-link gather on a side stream next to an HBM gather on the main stream: side stream plain or
            confined to 8 / 16 / 32 compute units (ugk_stream_create_cu_masked), grid capped to 32 - 256 workgroups
  small_batch  serving-sized batches (1,024 - 131,072 keys that all hit) through the library: microseconds per blocking
            coll_cache_lookup_i64 and per stream-ordered coll_cache_lookup_async_i64, without a table (the whole table
            cached) and through the table of a half-cached key space (host clock around 2,000 calls)
  pooled    a multi-hot feature through the library: lookup + weighted combination per sample in one call
            (coll_torch_lookup_pooled) against the lookup of all ids followed by torch's index_add_ segment sum, and
            against unique -> lookup -> index_select -> index_add_ (the reference's sparse layer), by ids per sample
  link_latency  what bounds rows of 128 bytes read out of pinned host memory: (a) the latency of one dependent read, from a
            single lane that follows a chain of links scattered over the first S GiB of a 60 GiB allocation (and over
            HBM for comparison); (b) the rate of independent row reads by the number of bytes in flight (workgroups x
            loads in flight per lane), which shows where the link stops answering faster; (c) where the allocation's
            pages live (/proc/self/numa_maps).  Kernels: bench_probes_kernels.hip (libbench_probes.so)
  placement  the placement of a refresh on the device alone on the chip at config 5's size (500 M counters, some 57 M
            above zero, 50 M and 20 M rows wanted): counters kept (one pass when the last placement's threshold still
            holds, two when it does not) and counters reset (two passes)
  rw_ceiling  what the two sides of the all-hit gather reach alone on its own shapes: random 512-byte rows read and
            nothing written, a buffer written and nothing read, a plain copy, the gather itself; with an output that
            stays in the memory-side cache and with one that cannot
  sparse_layer  the serving stack's SparseLookupLayer end to end (a ps_config file and a model directory written to a
            temporary folder, Config -> record_hotness -> Init -> layer calls): the reference's steps (unique, lookup,
            gather, weighted segment sum), the same with the unique inside the library, and lookup + combination in
            one kernel as a blocking serving step and enqueued like a torch op
"""
import ctypes as C
import json
import os
import math
import sys
import time


def _event(hip):
    e = C.c_void_p()
    hip.call("ugk_event_create", C.byref(e))
    return e


def _elapsed_us(hip, a, b):
    ms = C.c_float()
    hip.call("ugk_event_elapsed_ms", a, b, C.byref(ms))
    return ms.value * 1e3


def _timed(hip, stream, fn, reps, warm=3):
    """average microseconds per call of fn(i), reps calls back to back between two events on `stream`"""
    for i in range(warm):
        fn(i)
    hip.call("ugk_stream_sync", stream)
    a, b = _event(hip), _event(hip)
    hip.call("ugk_event_record", a, stream)
    for i in range(reps):
        fn(i)
    hip.call("ugk_event_record", b, stream)
    hip.call("ugk_event_sync", b)
    us = _elapsed_us(hip, a, b) / reps
    hip.call("ugk_event_destroy", a)
    hip.call("ugk_event_destroy", b)
    return us


def _pinned(hip, nbytes):
    p = C.c_void_p()
    hip.call("ugk_host_malloc", C.byref(p), nbytes)
    return p


def _check_status(torch, st, what):
    if int(st[0].item()) != 0:
        sys.exit("probe %s: a launch flagged status %d" % (what, int(st[0].item())))


def probe_kpw(hip, torch, note, quick=False):
    rows = 2_000_000
    stream = C.c_void_p()
    hip.call("ugk_stream_create", C.byref(stream))
    words = _pinned(hip, hip.lib().ugk_extract_mix_max_groups() * 8)
    groups = C.c_uint32(0)
    st = torch.zeros(4, dtype=torch.int32, device="cuda")
    sizes = (8192, 65536, 262144) if quick else (8192, 32768, 65536, 131072, 212992, 262144, 524288, 1048576)
    cases = ((512, 1),) if quick else ((512, 1), (512, 10), (128, 1), (128, 10))
    out_rows = []
    saved = os.environ.get("UGK_MIX_KPW")
    # (BENCH_PROBE_TABLES: a comma-separated subset, to time one table without the others' allocations before it)
    for kind in os.environ.get("BENCH_PROBE_TABLES", "flat,hash,hash8").split(","):
        for rb, miss_pct in cases:
            ncache = int(rows * (1 - miss_pct / 100))
            if kind == "flat":
                mem = torch.empty(rows, dtype=torch.int32, device="cuda")
                hip.call("ugk_fill_u32", mem.data_ptr(), hip.EMPTY_U32, rows, stream)
                tb = hip.table(hip.TABLE_FLAT, mem.data_ptr(), rows)
            elif kind == "hash8":  # 8-byte entries keyed by the row, sixteen to a line
                ne = hip.lib().ugk_hash32_entries_for(ncache, float(os.environ.get("BENCH_PROBE_HASH_LOAD", "0.7")))
                mem = torch.empty(ne * 8 + 128, dtype=torch.uint8, device="cuda")
                base = (mem.data_ptr() + 127) // 128 * 128
                tb = hip.table(hip.TABLE_HASH32, base, ne)
                hip.call("ugk_table_init", tb, stream)
            else:
                # (BENCH_PROBE_HASH_LOAD: the same sweep over a sparser table, to see what the keys that need a second
                # line cost)
                nb = hip.lib().ugk_hash_buckets_for(ncache, float(os.environ.get("BENCH_PROBE_HASH_LOAD", "0.7")))
                mem = torch.empty(nb * 16 + 128, dtype=torch.uint8, device="cuda")
                base = (mem.data_ptr() + 127) // 128 * 128
                hip.call("ugk_hash_init", base, nb, stream)
                tb = hip.table(hip.TABLE_HASH, base, nb)
            cached = torch.arange(ncache, dtype=torch.int64, device="cuda")
            torch.cuda.synchronize()  # torch made the key list on its own stream; the insert reads it on this one
            hip.call("ugk_table_insert_i64", tb, cached.data_ptr(), None, 0, hip.LOC_LOCAL, ncache, st.data_ptr(), stream)
            cache = torch.randint(0, 2 ** 31 - 1, (ncache, rb // 4), dtype=torch.int32, device="cuda")
            host = _pinned(hip, rows * rb)
            C.memset(host, 7, rows * rb)
            pool = 8
            for n in sizes:
                keys = torch.randint(0, rows, (pool, n), device="cuda", dtype=torch.int64)
                out = torch.empty((n, rb // 4), dtype=torch.int32, device="cuda")
                torch.cuda.synchronize()
                row = {"table": kind, "row_bytes": rb, "miss_pct": miss_pct, "keys": n, "us_by_keys_per_wavefront": {}}
                for kpw in ("rule", 8, 16, 32, 64):
                    if kpw == "rule":
                        os.environ.pop("UGK_MIX_KPW", None)
                    else:
                        os.environ["UGK_MIX_KPW"] = str(kpw)

                    def go(i):
                        hip.call("ugk_extract_mix_i64", tb, keys[i % pool].data_ptr(), n, cache.data_ptr(), ncache,
                                 host, rows, out.data_ptr(), rb, st.data_ptr(), None, words, C.byref(groups),
                                 hip.HINT_UNKNOWN, stream)
                    row["us_by_keys_per_wavefront"][str(kpw)] = round(_timed(hip, stream, go, 50), 2)
                out_rows.append(row)
                note("kpw %s %d B %d %% misses, %d keys: %s" % (kind, rb, miss_pct, n, row["us_by_keys_per_wavefront"]))
                del keys, out
            _check_status(torch, st, "kpw")
            hip.call("ugk_host_free", host)
            del cache, mem, cached
            torch.cuda.empty_cache()
    if saved is None:
        os.environ.pop("UGK_MIX_KPW", None)
    else:
        os.environ["UGK_MIX_KPW"] = saved
    hip.call("ugk_host_free", words)
    return {"probe": "kpw", "table_rows": rows, "launches_timed": 50,
            "how": "ugk_extract_mix_i64 over a table of which 99 % / 90 % is cached (uniform keys); 'rule' = the "
                   "launcher's own choice, the others forced with UGK_MIX_KPW; 2 HIP events around 50 launches",
            "rows": out_rows}


def probe_row_span(hip, torch, note, quick=False):
    GiB = 1 << 30
    total = (8 if quick else 60) * GiB
    stream = C.c_void_p()
    hip.call("ugk_stream_create", C.byref(stream))
    t0 = time.perf_counter()
    host = _pinned(hip, total)
    note("pinned %d GiB in %.1f s" % (total // GiB, time.perf_counter() - t0))
    st = torch.zeros(4, dtype=torch.int32, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    res = []
    spans = (1, 4, 8) if quick else (1, 4, 16, 32, 60)
    for rb in (128, 512):
        for span in spans:
            rows = span * GiB // rb
            for n in (159_000, 262_144):
                keys = torch.randint(0, rows, (8, n), generator=g, device="cuda", dtype=torch.int64)
                out = torch.empty(n * rb, dtype=torch.uint8, device="cuda")
                torch.cuda.synchronize()
                by_cap = {}
                for cap in (128, 512, 0):
                    def go(i):
                        hip.call("ugk_gather_direct_i64", host, rows, keys[i % 8].data_ptr(), n, out.data_ptr(), rb,
                                 cap, st.data_ptr(), None, stream)
                    us = _timed(hip, stream, go, 8, warm=2)
                    by_cap[str(cap or "unlimited")] = round(n * rb / us / 1e3, 2)
                res.append({"row_bytes": rb, "span_GiB": span, "rows_per_launch": n, "GBps_by_workgroup_cap": by_cap})
                note("rows of %d B over the first %d GiB, n = %d: %s GB/s" % (rb, span, n, by_cap))
                del keys, out
    _check_status(torch, st, "row_span")
    hip.call("ugk_host_free", host)
    return {"probe": "row_span", "allocation_GiB": total // GiB,
            "how": "ugk_gather_direct_i64 of uniformly random rows of one pinned allocation (which the probe "
                   "does not fill), 2 HIP events around 8 launches", "rows": res}


def probe_cu_mask(hip, torch, note, quick=False):
    rows, rb = (4_194_304 if quick else 16_777_216), 512
    nbytes = rows * rb
    main, plain = C.c_void_p(), C.c_void_p()
    hip.call("ugk_stream_create", C.byref(main))
    hip.call("ugk_stream_create", C.byref(plain))
    host = _pinned(hip, nbytes)
    drows = 10_000_000
    dtable = torch.empty((drows, rb // 4), dtype=torch.float32, device="cuda").normal_()
    g = torch.Generator(device="cuda").manual_seed(4)
    n_miss, n_hit = 250_000, 800_000
    mk = torch.randint(0, rows, (n_miss,), generator=g, device="cuda", dtype=torch.int32)
    hk = torch.randint(0, drows, (n_hit,), generator=g, device="cuda", dtype=torch.int32)
    mout = torch.empty((n_miss, rb // 4), dtype=torch.float32, device="cuda")
    hout = torch.empty((n_hit, rb // 4), dtype=torch.float32, device="cuda")
    st = torch.zeros(4, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    ev = [_event(hip) for _ in range(4)]
    res = []

    def trial(side, blocks, label):
        last = None
        for _ in range(4):
            hip.call("ugk_event_record", ev[0], side)
            hip.call("ugk_gather_direct_u32", host, rows, mk.data_ptr(), n_miss, mout.data_ptr(), rb, blocks,
                     st.data_ptr(), None, side)
            hip.call("ugk_event_record", ev[1], side)
            hip.call("ugk_event_record", ev[2], main)
            hip.call("ugk_gather_direct_u32", dtable.data_ptr(), drows, hk.data_ptr(), n_hit, hout.data_ptr(), rb, 0,
                     st.data_ptr(), None, main)
            hip.call("ugk_event_record", ev[3], main)
            hip.call("ugk_stream_sync", side)
            hip.call("ugk_stream_sync", main)
            last = (_elapsed_us(hip, ev[0], ev[1]), _elapsed_us(hip, ev[2], ev[3]))
        res.append({"side_stream": label, "workgroup_cap": blocks, "host_gather_us": round(last[0], 1),
                    "host_gather_GBps": round(n_miss * rb / last[0] / 1e3, 2),
                    "concurrent_hbm_gather_us": round(last[1], 1)})
        note("%s, %d workgroups: host gather %.1f us (%.1f GB/s), HBM gather next to it %.1f us"
             % (label, blocks, last[0], n_miss * rb / last[0] / 1e3, last[1]))

    def alone():
        def go(i):
            hip.call("ugk_gather_direct_u32", dtable.data_ptr(), drows, hk.data_ptr(), n_hit, hout.data_ptr(), rb, 0,
                     st.data_ptr(), None, main)
        return _timed(hip, main, go, 8)

    hbm_alone = alone()
    note("HBM gather alone: %.1f us" % hbm_alone)
    for blocks in (32, 64, 128, 256):
        trial(plain, blocks, "plain")
    for ncu in (8, 16, 32):
        masked = C.c_void_p()
        hip.call("ugk_stream_create_cu_masked", C.byref(masked), ncu)
        for blocks in (32, 64, 128, 256):
            trial(masked, blocks, "confined to %d CUs" % ncu)
        hip.call("ugk_stream_destroy", masked)
    _check_status(torch, st, "cu_mask")
    hip.call("ugk_host_free", host)
    return {"probe": "cu_mask", "host_rows": rows, "row_bytes": rb, "host_gather_rows": n_miss, "hbm_gather_rows": n_hit,
            "hbm_gather_alone_us": round(hbm_alone, 1),
            "how": "ugk_gather_direct_u32 from pinned host memory on a side stream and from HBM on the main stream, "
                   "launched together, one event pair around each; the last of 4 rounds", "rows": res}


def probe_small_batch(hip, torch, note, quick=False):
    import collcache.torch as co
    from collcache.torch.c_lib import _basics

    Cl = _basics.C_LIB_CTYPES
    rows, dim, calls = 2_000_000, 128, (300 if quick else 2000)
    sizes = (1024, 65536) if quick else (1024, 8192, 26624, 65536, 131072)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out_rows = []
    for pct, label in ((1.0, "no table: the whole table cached"), (0.5, "flat table of a half-cached key space")):
        co.config({"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
                   "num_global_step_per_epoch": 10, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 8})
        co.coll_cache_record_init(0)
        # rows [0, rows / 2) are the hot ones: every key of the timed batches hits
        co.coll_torch_record(0, torch.arange(0, rows // 2, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, rows, dim, torch.float32)
        emb.normal_(generator=torch.Generator().manual_seed(1))
        co.coll_torch_init_t(0, 0, emb, pct)
        for n in sizes:
            keys = torch.randint(0, rows // 2, (8, n), device="cuda", dtype=torch.int64)
            ptrs = [keys[i].data_ptr() for i in range(8)]
            out = torch.empty((n, dim), dtype=torch.float32, device="cuda")
            torch.cuda.synchronize()
            for i in range(20):
                Cl.coll_cache_lookup_i64(0, ptrs[i % 8], n, out.data_ptr(), stream)
            t0 = time.perf_counter()
            for i in range(calls):
                Cl.coll_cache_lookup_i64(0, ptrs[i % 8], n, out.data_ptr(), stream)
            blocking = (time.perf_counter() - t0) / calls * 1e6
            assert torch.equal(out.cpu(), emb[keys[(calls - 1) % 8].cpu()])
            assert _basics.last_group_offset(0)[1] == n  # every key was served from HBM
            for i in range(20):
                Cl.coll_cache_lookup_async_i64(0, ptrs[i % 8], n, out.data_ptr(), stream)
            Cl.coll_cache_lookup_wait(0, stream)
            t0 = time.perf_counter()
            for i in range(calls):
                Cl.coll_cache_lookup_async_i64(0, ptrs[i % 8], n, out.data_ptr(), stream)
            Cl.coll_cache_lookup_wait(0, stream)
            ordered = (time.perf_counter() - t0) / calls * 1e6
            # the same stream-ordered calls recorded once into a HIP graph, 26 lookups (one per sparse field of a
            # recommendation model) per replay: what is left of the launch cost when the caller captures its step
            fields, replays = 26, max(calls // 26, 20)
            outs = torch.empty((fields, n, dim), dtype=torch.float32, device="cuda")
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cap = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                for f in range(fields):
                    Cl.coll_cache_lookup_async_i64(0, ptrs[f % 8], n, outs[f].data_ptr(), cap)
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(replays):
                graph.replay()
            torch.cuda.synchronize()
            replayed = (time.perf_counter() - t0) / (replays * fields) * 1e6
            Cl.coll_cache_lookup_wait(0, stream)
            assert torch.equal(outs[fields - 1].cpu(), emb[keys[(fields - 1) % 8].cpu()])
            out_rows.append({"path": label, "keys": n, "us_per_blocking_call": round(blocking, 2),
                             "us_per_stream_ordered_call": round(ordered, 2),
                             "us_per_call_in_a_replayed_graph_of_26": round(replayed, 2)})
            note("small_batch %s, %d keys: blocking %.1f us, stream-ordered %.1f us, in a replayed graph %.1f us"
                 % (label, n, blocking, ordered, replayed))
            del keys, out, outs, graph
        co.coll_torch_shutdown()
    # serving steps (a 5 % prefix recorded, a refresh configured but far away) at the same sizes: the prefix copied to
    # the host and counted there by the recorder's thread (the default; such a step blocks whatever is asked for), or
    # counted on the device, where a step can also be enqueued and left
    for gpu_record in (False, True):
        if gpu_record:
            os.environ["COLL_GPU_RECORD"] = "1"
        try:
            co.config({"cache_percentage": 0.5, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
                       "num_global_step_per_epoch": 10, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 8})
            co.coll_cache_record_init(0)
            co.coll_torch_record(0, torch.arange(0, rows // 2, dtype=torch.int32))
            emb = co.coll_torch_create_emb_shm(0, rows, dim, torch.float32)
            emb.normal_(generator=torch.Generator().manual_seed(1))
            co.coll_torch_init_t(0, 0, emb, 0.5)
            Cl.coll_cache_forward_config(1, 10 ** 12, 0.05, 0)
            for n in sizes:
                keys = torch.randint(0, rows // 2, (8, n), device="cuda", dtype=torch.int64)
                ptrs = [keys[i].data_ptr() for i in range(8)]
                out = torch.empty((n, dim), dtype=torch.float32, device="cuda")
                torch.cuda.synchronize()
                res = {}
                for name, fn in (("blocking", Cl.coll_cache_forward_i64), ("stream_ordered", Cl.coll_cache_forward_async_i64)):
                    for i in range(20):
                        fn(0, ptrs[i % 8], n, out.data_ptr(), stream)
                    Cl.coll_cache_lookup_wait(0, stream)
                    t0 = time.perf_counter()
                    for i in range(calls):
                        fn(0, ptrs[i % 8], n, out.data_ptr(), stream)
                    Cl.coll_cache_lookup_wait(0, stream)
                    res[name] = round((time.perf_counter() - t0) / calls * 1e6, 2)
                assert torch.equal(out.cpu(), emb[keys[(calls - 1) % 8].cpu()])
                label = "serving step, prefix counted on the %s" % ("device" if gpu_record else "host")
                out_rows.append({"path": label, "keys": n, "us_per_blocking_call": res["blocking"],
                                 "us_per_stream_ordered_call": res["stream_ordered"]})
                note("small_batch %s, %d keys: blocking %.1f us, stream-ordered %.1f us"
                     % (label, n, res["blocking"], res["stream_ordered"]))
                del keys, out
            Cl.coll_cache_forward_config(0, 0, 0.0, 0)
            co.coll_torch_shutdown()
        finally:
            os.environ.pop("COLL_GPU_RECORD", None)
    return {"probe": "small_batch", "table_rows": rows, "row_bytes": dim * 4, "calls_timed": calls,
            "how": "coll_cache_lookup_i64 / coll_cache_lookup_async_i64 (+ one coll_cache_lookup_wait) over 8 cycled "
                   "batches of uniformly random keys that all hit, host clock around the calls; the graph holds 26 "
                   "stream-ordered calls and is replayed back to back", "rows": out_rows}


def probe_pooled(hip, torch, note, quick=False):
    import collcache.torch as co

    rows, dim, calls = 10_000_000, 128, (20 if quick else 50)
    out_rows = []
    for pct, label in ((1.0, "whole table cached"), (0.5, "half of the rows cached, every id a hit")):
        co.config({"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
                   "num_global_step_per_epoch": 10, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 8})
        co.coll_cache_record_init(0)
        co.coll_torch_record(0, torch.arange(0, rows // 2, dtype=torch.int32))
        emb = co.coll_torch_create_emb_shm(0, rows, dim, torch.float32)
        emb.normal_(generator=torch.Generator().manual_seed(1))
        co.coll_torch_init_t(0, 0, emb, pct)
        for per_sample, zipf in ((1, 0.0), (2, 0.0), (4, 0.0), (16, 0.0), (16, 1.05)) if not quick else ((8, 0.0),):
            n_samples = 262_144 if per_sample <= 4 else 65_536
            nnz = n_samples * per_sample
            if zipf:  # duplicates among the ids, as a skewed multi-hot feature has them
                u = torch.rand(nnz, device="cuda", dtype=torch.float64)
                h = float(rows // 2)
                ids = (((h ** (1 - zipf) - 1) * u + 1) ** (1 / (1 - zipf))).long().clamp_(1, rows // 2) - 1
            else:
                ids = torch.randint(0, rows // 2, (nnz,), device="cuda", dtype=torch.int64)
            seg_off = torch.arange(0, nnz + 1, per_sample, device="cuda", dtype=torch.int64)
            seg = torch.arange(n_samples, device="cuda").repeat_interleave(per_sample)
            w = torch.rand(nnz, device="cuda", dtype=torch.float32) + 0.5

            def fused():
                return co.coll_torch_lookup_pooled(0, ids, seg_off, w, "sum")

            def fused_stream_ordered():
                return co.coll_torch_lookup_pooled(0, ids, seg_off, w, "sum", stream_ordered=True)

            def lookup_then_sum():
                e = co.coll_torch_lookup_key_t_val_ret(0, ids, False)
                out = torch.zeros((n_samples, dim), dtype=torch.float32, device="cuda")
                return out.index_add_(0, seg, e * w.unsqueeze(1))

            def unique_lookup_sum():
                uq, inv = torch.unique(ids, return_inverse=True)
                e = co.coll_torch_lookup_key_t_val_ret(0, uq, False).index_select(0, inv)
                out = torch.zeros((n_samples, dim), dtype=torch.float32, device="cuda")
                return out.index_add_(0, seg, e * w.unsqueeze(1))

            ref = lookup_then_sum()
            assert torch.allclose(fused(), ref, rtol=1e-4, atol=1e-4) and torch.allclose(unique_lookup_sum(), ref, rtol=1e-4, atol=1e-4)
            res = {}
            assert torch.equal(fused_stream_ordered(), fused())
            for name, fn in (("fused", fused), ("fused_stream_ordered", fused_stream_ordered),
                             ("lookup_then_sum", lookup_then_sum), ("unique_lookup_sum", unique_lookup_sum)):
                for _ in range(3):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(calls):
                    fn()
                torch.cuda.synchronize()
                res[name] = round((time.perf_counter() - t0) / calls * 1e6, 1)
                co.coll_torch_lookup_wait(0)
            moved = nnz * dim * 4 + n_samples * dim * 4 + nnz * 12
            out_rows.append({"cache": label, "samples": n_samples, "ids_per_sample": per_sample, "zipf": zipf,
                             "us_per_call": res, "fused_GBps_of_rows_read_and_written": round(moved / res["fused"] / 1e3, 1)})
            note("pooled %s, %d x %d ids (zipf %.2f): %s" % (label, n_samples, per_sample, zipf, res))
            del ids, seg, w, ref
        co.coll_torch_shutdown()
    return {"probe": "pooled", "table_rows": rows, "row_bytes": dim * 4, "calls_timed": calls,
            "how": "weighted sum per sample of fp32 rows; host clock around the calls, one synchronisation at the end; "
                   "the unfused forms use the library's plain lookup and torch ops", "rows": out_rows}


def probe_sparse_layer(hip, torch, note, quick=False):
    import shutil
    import tempfile

    import numpy as np

    import collcache.torch as co
    import collcache.torch.serving as hps

    rng = np.random.default_rng(1)
    n_item, dim, calls = (200_000 if quick else 2_000_000), 128, (5 if quick else 30)
    folder = tempfile.mkdtemp(prefix="ugache_probe_")
    out_rows = []
    try:
        model = os.path.join(folder, "m.model")
        os.mkdir(model)
        np.arange(n_item, dtype=np.int64).tofile(os.path.join(model, "key"))
        rng.standard_normal((n_item, dim), dtype=np.float32).tofile(os.path.join(model, "emb_vector"))
        cfg = {"iteration_per_epoch": 1000000, "epoch": 1, "coll_cache_enable_refresh": False,
               "models": [{"model": "dlrm", "sparse_files": [model], "gpucacheper": 0.5, "max_batch_size": 65536,
                           "deployed_device_list": [0], "maxnum_catfeature_query_per_table_per_sample": [16],
                           "embedding_vecsize_per_table": [dim], "max_vocabulary_size": [n_item]}]}
        path = os.path.join(folder, "ps_config.json")
        with open(path, "w") as f:
            json.dump(cfg, f)
        hps.Config(ps_config_file=path)
        hps.record_hotness(torch.arange(0, n_item // 2, device="cuda"))  # the rows every timed id hits
        hps.Init(ps_config_file=path, global_batch_size=65536)
        forms = (("reference_steps", {}), ("unique_in_library", {"unique_in_library": True}),
                 ("fused_serving_step", {"fused": True}), ("fused_stream_ordered", {"fused": True, "stream_ordered": True}))
        for n_rows, per in ((65536, 16), (262144, 1), (262144, 4)) if not quick else ((4096, 4),):
            nnz = n_rows * per
            seg = torch.arange(n_rows, device="cuda").repeat_interleave(per)
            col = torch.arange(per, device="cuda").repeat(n_rows)
            ids = torch.randint(0, n_item // 2, (nnz,), device="cuda")
            w = torch.rand(nnz, device="cuda") + 0.5
            ind = torch.stack([seg, col])
            sp_ids = torch.sparse_coo_tensor(ind, ids, (n_rows, per))
            sp_w = torch.sparse_coo_tensor(ind, w, (n_rows, per))
            res, ref = {}, None
            for name, kw in forms:
                layer = hps.SparseLookupLayer(model_name="dlrm", table_id=0, emb_vec_size=dim,
                                              emb_vec_dtype=torch.float32, **kw)
                got = layer(sp_ids, sp_w, combiner="sum")
                co.coll_torch_lookup_wait(0)
                ref = got if ref is None else ref
                assert torch.allclose(got, ref, rtol=1e-4, atol=1e-4)
                for _ in range(3):
                    layer(sp_ids, sp_w, combiner="sum")
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(calls):
                    layer(sp_ids, sp_w, combiner="sum")
                torch.cuda.synchronize()
                res[name] = round((time.perf_counter() - t0) / calls * 1e6, 1)
                co.coll_torch_lookup_wait(0)
            out_rows.append({"samples": n_rows, "ids_per_sample": per, "us_per_layer_call": res})
            note("sparse_layer %d x %d ids: %s" % (n_rows, per, res))
        hps.Shutdown()
    finally:
        shutil.rmtree(folder, ignore_errors=True)
    return {"probe": "sparse_layer", "table_rows": n_item, "row_bytes": dim * 4, "cache": "half of the rows, every id a hit",
            "calls_timed": calls, "how": "SparseLookupLayer(sp_ids, sp_weights, combiner='sum') on sparse COO inputs; "
            "host clock around the calls, one synchronisation at the end", "rows": out_rows}


def _probe_lib():
    """libbench_probes.so, built beside this file by __graft_entry__.build() from bench_probes_kernels.hip"""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libbench_probes.so")
    if not os.path.exists(path):
        sys.exit("probe link_latency needs libbench_probes.so: run `python __graft_entry__.py` first")
    lib = C.CDLL(path)
    lib.bp_last_error.restype = C.c_char_p
    lib.bp_chase.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_void_p, C.c_void_p]
    lib.bp_rows_inflight.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_size_t, C.c_int, C.c_uint, C.c_void_p,
                                     C.c_void_p]

    def call(name, *args):
        if getattr(lib, name)(*args) != 0:
            sys.exit("probe link_latency: %s" % lib.bp_last_error().decode())
    return call


def _numa_placement(addr):
    """the /proc/self/numa_maps line of the mapping that holds `addr`: policy, pages per node, page size"""
    try:
        best = None
        with open("/proc/self/numa_maps") as f:
            for line in f:
                start = int(line.split()[0], 16)
                if start <= addr and (best is None or start > best[0]):
                    best = (start, line.strip())
        online = open("/sys/devices/system/node/online").read().strip()
        fields = best[1].split() if best else []
        return {"mapping_start": hex(best[0]) if best else None, "policy": fields[1] if len(fields) > 1 else None,
                "pages_by_node": {f.split("=")[0]: int(f.split("=")[1]) for f in fields if f[0] == "N" and "=" in f},
                "kernelpagesize_kB": next((int(f.split("=")[1]) for f in fields if f.startswith("kernelpagesize_kB=")), None),
                "nodes_online": online}
    except Exception as e:  # the file is not there in every container
        return {"error": str(e)}


def probe_link_latency(hip, torch, note, quick=False):
    import numpy as np
    call = _probe_lib()
    GiB = 1 << 30
    total = (8 if quick else 60) * GiB
    stream = C.c_void_p()
    hip.call("ugk_stream_create", C.byref(stream))
    t0 = time.perf_counter()
    host = _pinned(hip, total)
    # contents: ascending words written by the device (all-zero lines could be moved faster than real rows)
    chunk = 1 << 30
    for off in range(0, total, chunk):
        hip.call("ugk_arange_u32", host.value + off, (off // 4) & 0xffffffff, chunk // 4, stream)
    hip.call("ugk_stream_sync", stream)
    note("pinned and filled %d GiB in %.1f s" % (total // GiB, time.perf_counter() - t0))
    placement = _numa_placement(host.value)
    note("placement of the allocation: %s" % placement)
    host_bytes = (C.c_uint8 * total).from_address(host.value)
    host_lines = np.frombuffer(host_bytes, dtype=np.uint64).reshape(-1, 16)  # 128-byte lines, link in word 0
    rng = np.random.default_rng(7)
    last = torch.zeros(2, dtype=torch.int64, device="cuda")
    spans = (1, 4, 8) if quick else (1, 4, 16, 32, 60)
    hops = 20_000
    scrub = np.empty(256 << 20, np.uint8)  # written after the chain, so that its lines leave the CPU's caches

    def chase(base_ptr, write_links, n_lines):
        nodes = rng.choice(n_lines, size=hops, replace=False).astype(np.uint64)
        write_links(nodes, np.roll(nodes, -1))
        scrub[:] = 1
        out = []
        for rep in range(3):
            a, b = _event(hip), _event(hip)
            hip.call("ugk_event_record", a, stream)
            call("bp_chase", base_ptr, 128, int(nodes[0]), hops, last.data_ptr(), stream)
            hip.call("ugk_event_record", b, stream)
            hip.call("ugk_event_sync", b)
            out.append(_elapsed_us(hip, a, b) / hops)
            hip.call("ugk_event_destroy", a)
            hip.call("ugk_event_destroy", b)
        assert int(last[0].item()) == int(nodes[0])  # the chain is a cycle of `hops` links
        return out

    def host_links(nodes, nxt):
        host_lines[nodes, 0] = nxt

    latency = []
    for span in spans:
        us = chase(host, host_links, span * GiB // 128)
        latency.append({"span_GiB": span, "us_per_dependent_read": [round(x, 3) for x in us]})
        note("pinned host memory, links over the first %d GiB: %s us per dependent read" % (span, latency[-1]["us_per_dependent_read"]))
    dev_lines = torch.zeros(((2 if quick else 8) * GiB // 128, 16), dtype=torch.int64, device="cuda")

    def dev_links(nodes, nxt):
        dev_lines[torch.from_numpy(nodes.astype(np.int64)).cuda(), 0] = torch.from_numpy(nxt.astype(np.int64)).cuda()
        torch.cuda.synchronize()

    hbm_us = chase(dev_lines.data_ptr(), dev_links, dev_lines.shape[0])
    note("HBM, links over %d GiB: %s us per dependent read" % (dev_lines.numel() * 8 // GiB, [round(x, 3) for x in hbm_us]))
    del dev_lines

    # (b) independent reads by bytes in flight
    n_rows = 1 << 20
    g = torch.Generator(device="cuda").manual_seed(1)
    grids = (8, 64, 512, 2048) if quick else (4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192)
    sink = torch.zeros(max(grids) * 256, dtype=torch.int32, device="cuda")
    sweep = []
    for rb in (128, 512):
        for span in (spans[-1],) if quick else (16, spans[-1]):
            rows = torch.randint(0, span * GiB // rb, (4, n_rows), generator=g, device="cuda", dtype=torch.int64).to(torch.int32)
            for unroll in (1, 2, 4, 8, 16):
                by_grid = {}
                for grid in grids:
                    def go(i):
                        call("bp_rows_inflight", host, rb, rows[i % 4].data_ptr(), n_rows, unroll, grid, sink.data_ptr(), stream)
                    us = _timed(hip, stream, go, 3, warm=1)
                    by_grid[str(grid)] = round(n_rows * rb / us / 1e3, 2)
                sweep.append({"row_bytes": rb, "span_GiB": span, "loads_in_flight_per_lane": unroll,
                              "KiB_in_flight_per_workgroup": unroll * 4, "GBps_by_workgroups": by_grid})
                note("rows of %d B over %d GiB, %2d loads per lane in flight: %s GB/s by workgroups" % (rb, span, unroll, by_grid))
            del rows
    hip.call("ugk_host_free", host)
    return {"probe": "link_latency", "allocation_GiB": total // GiB, "placement": placement,
            "dependent_reads": {"hops": hops, "line_bytes": 128, "pinned_host": latency,
                                "hbm_us_per_dependent_read": [round(x, 3) for x in hbm_us],
                                "how": "one lane follows a cycle of 20,000 links at random 128-byte lines of the first "
                                       "S GiB; 3 passes over the same cycle (the lines are not cached on the device: "
                                       "the passes agree); microseconds per link"},
            "independent_reads": {"rows_per_launch": n_rows, "rows": sweep,
                                  "how": "bp_rows_inflight: a grid of W workgroups of 256 lanes reads 2^20 listed rows, "
                                         "U 16-byte loads in flight per lane, nothing written; bytes in flight = "
                                         "min(W, resident workgroups) x 256 x U x 16; 2 HIP events around 3 launches"}}


def probe_rw_ceiling(hip, torch, note, quick=False):
    """What the two sides of the all-hit gather reach alone, on its own shapes: random 512-byte rows of a 5.12 GB table
    read and nothing written (bp_rows_inflight), a buffer written and nothing read (ugk_fill_u32), a plain copy
    (ugk_copy_rows), and the gather itself (ugk_gather_direct_u32) -- each with an output that stays in the 256 MB
    memory-side cache (134 MB, rewritten every launch) and with one that cannot (1 GiB).  Then the same for random
    128-byte rows of a 6.4 GB table (configuration 5's cache), 1 M rows per launch."""
    call = _probe_lib()
    stream = C.c_void_p()
    hip.call("ugk_stream_create", C.byref(stream))
    g = torch.Generator(device="cuda").manual_seed(3)
    st = torch.zeros(4, dtype=torch.int32, device="cuda")
    res = {}
    reps = 10 if quick else 30
    for rows, rb, sizes in ((10_000_000, 512, (262_144, 2_097_152)), (50_000_000, 128, (1_048_576,))):
        table = torch.empty(rows * rb // 4, dtype=torch.int32, device="cuda")
        hip.call("ugk_arange_u32", table.data_ptr(), 1, table.numel(), stream)
        for n in sizes:
            nbytes = n * rb
            keys = torch.randint(0, rows, (4, n), generator=g, device="cuda", dtype=torch.int32)
            out = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")
            src = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")
            sink = torch.zeros(8192 * 256, dtype=torch.int32, device="cuda")
            torch.cuda.synchronize()
            r = {}
            us = min(_timed(hip, stream, lambda i, u=u, w=w: call("bp_rows_inflight", table.data_ptr(), rb,
                                                                  keys[i % 4].data_ptr(), n, u, w, sink.data_ptr(), stream),
                            reps)
                     for u in (2, 4, 8) for w in (2048, 8192))
            r["random_rows_read_only"] = {"us": round(us, 2), "TBps": round(nbytes / us / 1e6, 3)}
            us = _timed(hip, stream, lambda i: hip.call("ugk_fill_u32", out.data_ptr(), i + 1, nbytes // 4, stream), reps)
            r["write_only"] = {"us": round(us, 2), "TBps": round(nbytes / us / 1e6, 3)}
            us = _timed(hip, stream, lambda i: hip.call("ugk_copy_rows", out.data_ptr(), src.data_ptr(), nbytes, stream), reps)
            r["plain_copy"] = {"us": round(us, 2), "TBps_read_plus_written": round(2 * nbytes / us / 1e6, 3)}
            us = _timed(hip, stream, lambda i: hip.call("ugk_gather_direct_u32", table.data_ptr(), rows, keys[i % 4].data_ptr(),
                                                        n, out.data_ptr(), rb, 0, st.data_ptr(), None, stream), reps)
            r["gather"] = {"us": round(us, 2), "TBps_read_plus_written": round((2 * nbytes + 4 * n) / us / 1e6, 3)}
            res["%d rows of %d B (%d MB out)" % (n, rb, nbytes >> 20)] = r
            note("%d rows of %d B: %s" % (n, rb, r))
            del keys, out, src, sink
            torch.cuda.empty_cache()
        del table
        torch.cuda.empty_cache()
    _check_status(torch, st, "rw_ceiling")
    return {"probe": "rw_ceiling", "tables": "10 M rows of 512 bytes, 50 M rows of 128 bytes, in HBM", "launches_timed": reps,
            "how": "2 HIP events around the launches; read-only: best of 2, 4, 8 loads per lane x 2048, 8192 workgroups",
            "sizes": res}


def probe_placement(hip, torch, note, quick=False):
    """The placement of a refresh on the device, alone on the chip, at config 5's size: 500 M counters of which some
    57 M are above zero (Zipf 1.05 over the rows, 200 M draws), K = 50 M and 20 M rows wanted.  ugk_rank_place with the
    counters kept (the first pass splits by the last placement's threshold on its way: timed with a workspace that has
    seen the same placement, and with one whose guess is wrong), with the counters reset after every placement (two
    passes), and ugk_rank_place_observed where it applies (K above the number of observed rows)."""
    stream = C.c_void_p()
    hip.call("ugk_stream_create", C.byref(stream))
    rows = 100_000_000 if quick else 500_000_000
    words = (rows + 63) // 64
    g = torch.Generator(device="cuda").manual_seed(5)
    counts = torch.zeros(rows, dtype=torch.int32, device="cuda")
    draws = 40_000_000 if quick else 200_000_000
    for _ in range(draws // 20_000_000):
        u = torch.rand(20_000_000, generator=g, device="cuda", dtype=torch.float64)
        r = (torch.exp(u * math.log(rows)) - 1).clamp_(0, rows - 1).to(torch.int64)  # log-uniform: ~ Zipf 1
        r = (r * 2654435761) % rows  # hot rows spread over the key space
        counts.index_add_(0, r, torch.ones_like(r, dtype=torch.int32))
        del u, r
    observed_n = int((counts > 0).sum().item())
    saved = counts.clone()
    # the observed-rows bitmap as the record kernel keeps it (bit r = counter r above zero), packed with torch
    pad = torch.zeros(words * 64, dtype=torch.bool, device="cuda")
    pad[:rows] = counts > 0
    weights = torch.ones(64, dtype=torch.int64, device="cuda") << torch.arange(64, device="cuda", dtype=torch.int64)
    obs_words = (pad.view(words, 64).to(torch.int64) * weights).sum(dim=1)  # bit 63 is the sign bit of the same word
    del pad
    ws = torch.zeros(hip.lib().ugk_rank_workspace_bytes() // 4 + 8, dtype=torch.int32, device="cuda")
    in_new = torch.empty(words, dtype=torch.int64, device="cuda")
    scratch = torch.empty(words, dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()
    reps = 5 if quick else 10
    res = {"rows": rows, "rows_observed": observed_n}
    for k in (rows // 10, rows // 25):
        r = {}

        def place(reset, observed):
            hip.call("ugk_rank_place", counts.data_ptr(), rows, k, ws.data_ptr(), in_new.data_ptr(), scratch.data_ptr(),
                     obs_words.data_ptr() if observed else None, reset, stream)

        us = _timed(hip, stream, lambda i: place(0, False), reps)
        r["counters_kept_guess_right"] = round(us, 1)
        other = rows // 3

        def place_after_another(i):
            hip.call("ugk_rank_place", counts.data_ptr(), rows, other if i % 2 == 0 else k, ws.data_ptr(),
                     in_new.data_ptr(), scratch.data_ptr(), None, 0, stream)

        us2 = _timed(hip, stream, place_after_another, 2 * reps, warm=2)
        r["counters_kept_alternating_with_another_k_per_pair"] = round(2 * us2, 1)

        def place_reset(i):
            hip.call("ugk_copy_rows", counts.data_ptr(), saved.data_ptr(), rows * 4, stream)
            place(1, False)

        us_copy = _timed(hip, stream, lambda i: hip.call("ugk_copy_rows", counts.data_ptr(), saved.data_ptr(), rows * 4,
                                                         stream), reps)
        us3 = _timed(hip, stream, place_reset, reps)
        r["counters_reset_two_passes"] = round(us3 - us_copy, 1)
        hip.call("ugk_copy_rows", counts.data_ptr(), saved.data_ptr(), rows * 4, stream)
        us4 = _timed(hip, stream, lambda i: place(0, True), reps)
        r["counters_kept_with_observed_bitmap"] = round(us4, 1)
        res["k=%d" % k] = r
        note("k=%d: %s" % (k, r))
    return {"probe": "placement", "launches_timed": reps, "unit": "us per placement, 2 HIP events around the launches",
            "sizes": res}


PROBES = {"placement": probe_placement, "rw_ceiling": probe_rw_ceiling, "link_latency": probe_link_latency, "sparse_layer": probe_sparse_layer, "pooled": probe_pooled, "kpw": probe_kpw, "row_span": probe_row_span, "cu_mask": probe_cu_mask, "small_batch": probe_small_batch}


def run(name, quick=False):
    import torch

    from ugache_amd import hip

    if not torch.cuda.is_available():
        sys.exit("probes need a GPU")
    t0 = time.perf_counter()

    def note(msg):
        print("[probe %6.1fs] %s" % (time.perf_counter() - t0, msg), file=sys.stderr, flush=True)

    res = PROBES[name](hip, torch, note, quick)
    info = hip.device_info(0)
    res["device"] = "%s %s" % (info["name"], info["arch"])
    print(json.dumps(res), flush=True)
    return res
