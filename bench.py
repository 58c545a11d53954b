#!/usr/bin/env python3
"""Throughput of the embedding-extraction hot path on one MI355X.

A step is one blocking lookup of one key batch through the drop-in C boundary (libcoll_cache.so -> libugache_hip.so),
keys, cache and lookup table already resident in HBM when the timed region starts.

Default workload (the one the metric is quoted on) = the all-hit configuration: a 10M x 128 fp32 table (5.12 GB) fully
cached, 262,144 uniform uint32 keys per batch, duplicates allowed.  `--workload` also offers the mixed-source
configurations (pinned host table + frequency-ranked HBM cache); those print the same JSON shape plus a `host_link`
object and per-stage times.

Without `--workload` the line carries both halves of the metric: the all-hit configuration is the top level (with two
more all-hit legs whose output cannot stay in the 256 MB memory-side cache), and the GNN-shaped and the hashtable-mode
configuration run at full size, one after the other, each in a child process of its own (this process never touches
the GPU), and appear under `legs` with their host-link rates.  Every pooled key batch of every leg is compared with the
CPU oracle after its timed region; a difference ends the run without a number.

Prints ONE JSON line with keys/s (whole job), the roofline of the dominant HBM kernel (algorithmic bytes per launch /
its average duration, measured live with HIP events on the kernel's stream inside the timed region) and the CPU
baseline (the oracle's OpenMP gather on the host cores, bounded sample of the same batches).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "ugache_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth

# HBM-side bytes per launch of the dominant kernel, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/gather_kernel_c2_all_hit.md (each counter scaled by its reading for a 1 GiB copy kernel)
MEASURED_TRAFFIC_BYTES = {"c2_all_hit_10Mx128xfp32_262144_u32_uniform": 270_530_000,
                          # fused kernel; includes the 126 MB of rows that reach the L2 over the host link
                          "c3_gnn_100Mx128xfp32_1M_i64_zipf0.9_cache25pct": 1_137_700_000,
                          # fused kernel over the compact hash table (profiles/extract_mix_kernel_mixed_c1_c3_c4_c5.md)
                          "c5_hash_500Mx64xfp16_1M_i64_zipf1.05_cache50M": 301_400_000}

ALL_HIT = {
    # name: (rows, dim, keys per batch)
    "c2_all_hit_10Mx128xfp32_262144_u32_uniform": (10_000_000, 128, 262_144),
    "tiny_all_hit_100Kx128xfp32_8192_u32_uniform": (100_000, 128, 8_192),
}

MIXED = {
    # rows, dim, torch dtype name, keys/batch, zipf s, cache fraction, fields (1 = one id space), presample batches
    "c3_gnn_100Mx128xfp32_1M_i64_zipf0.9_cache25pct": dict(rows=100_000_000, dim=128, dtype="float32", n_keys=1 << 20,
                                                           zipf=0.9, pct=0.25, fields=1, presample=50),
    "c4_dlr_26x8Mx128xfp32_212992_i64_zipf1.2_cache40GB": dict(rows=26 * 8_388_608, dim=128, dtype="float32",
                                                               n_keys=8192 * 26, zipf=1.2,
                                                               pct=(40e9 / 512) / (26 * 8_388_608), fields=26,
                                                               presample=100),
    # the box refuses to pin 106 GB of host memory; this is the same shape with half the rows per field
    "c4_dlr_half_26x4Mx128xfp32_212992_i64_zipf1.2_cache20GB": dict(rows=26 * 4_194_304, dim=128, dtype="float32",
                                                                    n_keys=8192 * 26, zipf=1.2,
                                                                    pct=(20e9 / 512) / (26 * 4_194_304), fields=26,
                                                                    presample=100),
    # hashtable mode: ids are (row * odd) mod 2^40, rows are 64 fp16 = 128 B, 10 % of the rows cached in the
    # open-addressing table at 0.7 load; a foreground refresh is timed after the lookups
    "c5_hash_500Mx64xfp16_1M_i64_zipf1.05_cache50M": dict(rows=500_000_000, dim=64, dtype="float16", n_keys=1 << 20,
                                                          zipf=1.05, pct=0.1, fields=1, presample=50, sparse=True),
    "c5_hash_quarter_125Mx64xfp16_1M_i64_zipf1.05_cache12.5M": dict(rows=125_000_000, dim=64, dtype="float16",
                                                                    n_keys=1 << 20, zipf=1.05, pct=0.1, fields=1,
                                                                    presample=50, sparse=True),
    "c1_cpu_ref_1Mx128xfp32_65536_i64_zipf1.1_cache10pct": dict(rows=1_000_000, dim=128, dtype="float32",
                                                                n_keys=65_536, zipf=1.1, pct=0.10, fields=1,
                                                                presample=20),
    "small_mixed_4Mx128xfp32_262144_i64_zipf0.9_cache25pct": dict(rows=4_000_000, dim=128, dtype="float32",
                                                                  n_keys=262_144, zipf=0.9, pct=0.25, fields=1,
                                                                  presample=20),
    # no cache at all: every row crosses the host link (where deduplication of a skewed batch pays)
    "c1_nocache_1Mx128xfp32_65536_i64_zipf1.1": dict(rows=1_000_000, dim=128, dtype="float32", n_keys=65_536,
                                                     zipf=1.1, pct=0.0, fields=1, presample=1),
    # nearly every key hits, through the table: the HBM side of the mixed-source kernels on its own
    "c2_table_10Mx128xfp32_262144_i64_zipf0.5_cache99pct": dict(rows=10_000_000, dim=128, dtype="float32",
                                                                n_keys=262_144, zipf=0.5, pct=0.99, fields=1,
                                                                presample=60),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default=None, choices=sorted(ALL_HIT) + sorted(MIXED),
                    help="run this one workload in this process (default: the all-hit configuration at the top level "
                         "plus the mixed-source legs, each in a child process)")
    ap.add_argument("--no-legs", action="store_true", help="default run without the mixed-source legs")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline budget")
    ap.add_argument("--pool", type=int, default=None, help="distinct key batches cycled through the steps")
    ap.add_argument("--impl", default="", choices=["", "DIRECT", "SMMaskPhase", "NONE"],
                    help="mixed workloads: SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL (default: the fused kernel)")
    ap.add_argument("--dedup", action="store_true",
                    help="mixed workloads: COLL_DEDUP_KEYS=1, every distinct key of a batch is extracted once")
    ap.add_argument("--gpu-record", action="store_true",
                    help="mixed workloads: COLL_GPU_RECORD=1, every lookup counts its keys in device-side hotness "
                         "counters (drained by the refresh)")
    ap.add_argument("--concurrent-refresh", action="store_true",
                    help="sparse-id workloads, with --gpu-record: after the timed steps, time the lookups again while "
                         "a second thread refreshes the cache back to back from the device-side hotness counters")
    ap.add_argument("--device-refresh", action="store_true",
                    help="mixed workloads: COLL_GPU_RECORD=1 COLL_GPU_REFRESH=1 COLL_GPU_REFRESH_KEEP=1; after the "
                         "timed steps, time steps that each end with a refresh computed on the device from the "
                         "accumulated hotness, with 1 %% of the cache replaced per step")
    ap.add_argument("--stage-rows", type=int, default=1 << 24,
                    help="with --device-refresh: entries of the set of recently missed rows kept in HBM "
                         "(COLL_MISS_STAGE_ROWS; 0 = none, every inserted row crosses the host link again)")
    ap.add_argument("--serving", action="store_true",
                    help="mixed workloads: after the timed steps, time the same steps through the serving loop "
                         "(coll_cache_forward_i64: 5 %% of every batch recorded, a background refresh every K/2 steps)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run 5 plain device copies of 1 GiB (ugk_copy_rows) so a counter run has a kernel of "
                         "known traffic next to the gather")
    ap.add_argument("--probe", default=None, choices=["kpw", "row_span", "link_latency", "rw_ceiling", "placement", "cu_mask", "small_batch", "pooled", "sparse_layer"],
                    help="instead of a workload, run one of the stand-alone measurements behind the launch rules "
                         "(bench_probes.py): keys per wavefront of the fused kernel, random rows over the host "
                         "link by span, host-link gather confined to a few compute units, serving-sized batches through "
                         "the library; prints one JSON line")
    ap.add_argument("--quick", action="store_true", help="with --probe: a reduced sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the extraction path of ONE GPU (no collectives, no peer source); "
                 "--gpus %d is not supported, use --gpus 1" % args.gpus)
    return args


def stream_ordered_leg(C, fn, key_ptr_of, n_keys, out, stream, torch, W, K, out_ptr_of=None):
    """the same K steps through the stream-ordered entry point: batches are enqueued back to back, one wait at the
    end.  Returns (wall seconds per step, seconds per launch between two HIP events recorded on the same stream right
    before the first and right after the last of the K launches).  out_ptr_of(i): where step i writes (default: the
    one buffer `out`)."""
    from ugache_amd import hip
    if out_ptr_of is None:
        one = out.data_ptr()
        out_ptr_of = lambda i: one
    ev = [ctypes.c_void_p(), ctypes.c_void_p()]
    for e in ev:
        hip.call("ugk_event_create", ctypes.byref(e))
    for i in range(W):
        fn(0, key_ptr_of(i), n_keys, out_ptr_of(i), stream)
    C.coll_cache_lookup_wait(0, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    hip.call("ugk_event_record", ev[0], stream)
    for i in range(W, W + K):
        fn(0, key_ptr_of(i), n_keys, out_ptr_of(i), stream)
    hip.call("ugk_event_record", ev[1], stream)
    C.coll_cache_lookup_wait(0, stream)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / K
    ms = ctypes.c_float()
    hip.call("ugk_event_elapsed_ms", ev[0], ev[1], ctypes.byref(ms))
    for e in ev:
        hip.call("ugk_event_destroy", e)
    return wall, ms.value * 1e-3 / K


# what the library's own per-step time is: a device event pair around the launch (COLL_KERNEL_EVENTS=1), or a host
# timer around launch and wait (default, as in the reference)
PER_CALL_KEY = {True: "avg_kernel_us_event_pair_per_blocking_launch",
                False: "launch_to_completion_us_host_timer_per_blocking_call"}


def step_spread(t0, stamps):
    """median and 95th percentile of the wall time of the blocking calls of a timed region, in milliseconds"""
    import numpy as np
    d = np.diff(np.concatenate(([t0], np.asarray(stamps)))) * 1e3
    return {"median": float(np.median(d)), "p95": float(np.percentile(d, 95)), "max": float(d.max())}


def check_every_batch(orc, table_np, rows_host, lookup_into, out, what):
    """one more pass over the pool after the timed region: every pooled batch is looked up again (blocking) and its
    output compared byte for byte with the oracle's gather of the same rows.  Ends the run on the first difference.
    rows_host[i]: the host-table row of every key of batch i; lookup_into(i): looks batch i up into `out`."""
    import torch

    for i in range(len(rows_host)):
        lookup_into(i)
        torch.cuda.synchronize()
        if out.cpu().numpy().tobytes() != orc.gather(table_np, rows_host[i], omp=True).tobytes():
            sys.exit("bench.py: GPU output of %s batch %d differs from the CPU oracle — no numbers reported" % (what, i))
    return len(rows_host)


def cpu_baseline(orc, table_np, keys_host, n_keys, row_bytes, seconds):
    """the oracle's OpenMP gather over the same key batches; returns (keys/s, batches, elapsed, threads)"""
    import numpy as np

    rows = table_np.shape[0]
    lib = orc.lib
    cpu_out = np.empty((n_keys, row_bytes), np.uint8)
    pool = len(keys_host)
    i64 = keys_host.dtype == np.int64
    fn = lib.orc_gather_i64_omp if i64 else lib.orc_gather_u32_omp

    def cpu_step(i):
        rc = fn(table_np.ctypes.data, rows, keys_host[i % pool], n_keys, cpu_out.ctypes.data, row_bytes)
        assert rc == 0

    cpu_step(0)
    t0 = time.perf_counter()
    n_cpu = 0
    while True:
        cpu_step(n_cpu)
        n_cpu += 1
        if time.perf_counter() - t0 >= seconds or n_cpu >= 100000:
            break
    el = time.perf_counter() - t0
    return n_keys * n_cpu / el, n_cpu, el, lib.orc_omp_threads()


def cpu_baseline_lookup_and_gather(orc, table_np, cached_rows, keys_host, key_inv, key_mask, n_keys, row_bytes, seconds,
                                   gpu_batch0):
    """The CPU form of the whole mixed-source step: per key, id -> row, lookup in a flat host array of the row space,
    then a copy of the row from a host-side copy of the cached rows or from the host table, OpenMP over keys
    (orc_extract_flat_i64_omp).  The cache copy and the flat array are built here, untimed, from the rows the GPU
    cache holds (slot = position in that list).  The output of the first batch is compared with the GPU's.
    Returns (keys/s, batches, elapsed, threads)."""
    import numpy as np

    rows = table_np.shape[0]
    lib = orc.lib
    cached_rows = np.ascontiguousarray(cached_rows, np.uint32)
    flat = np.full(rows, 0xFFFFFFFF, np.uint32)
    flat[cached_rows] = np.arange(len(cached_rows), dtype=np.uint32)
    cache_copy = np.empty((max(len(cached_rows), 1), row_bytes), np.uint8)
    if len(cached_rows):
        assert lib.orc_gather_u32_omp(table_np.ctypes.data, rows, cached_rows, len(cached_rows), cache_copy.ctypes.data,
                                      row_bytes) == 0
    cpu_out = np.empty((n_keys, row_bytes), np.uint8)
    counts = np.zeros(2, np.uint64)
    pool = len(keys_host)

    def cpu_step(i):
        rc = lib.orc_extract_flat_i64_omp(flat.ctypes.data, rows, ctypes.c_uint64(key_inv), ctypes.c_uint64(key_mask),
                                          keys_host[i % pool].ctypes.data, n_keys, cache_copy.ctypes.data,
                                          len(cache_copy), table_np.ctypes.data, cpu_out.ctypes.data, row_bytes,
                                          counts.ctypes.data)
        assert rc == 0

    cpu_step(0)
    if cpu_out.tobytes() != gpu_batch0:
        sys.exit("bench.py: the CPU baseline's output differs from the GPU's for the same batch")
    split0 = counts.tolist()
    t0 = time.perf_counter()
    n_cpu = 0
    while True:
        cpu_step(n_cpu)
        n_cpu += 1
        if time.perf_counter() - t0 >= seconds or n_cpu >= 100000:
            break
    el = time.perf_counter() - t0
    return n_keys * n_cpu / el, n_cpu, el, lib.orc_omp_threads(), split0


def fill_table_from_device(emb, dev, seed):
    """table rows ~ N(0,1) generated on the device from a seed, mirrored chunk by chunk into the pinned host table"""
    import torch

    rows, dim = emb.shape
    g = torch.Generator(device=dev).manual_seed(seed)
    chunk = 2_000_000
    for r0 in range(0, rows, chunk):
        r1 = min(rows, r0 + chunk)
        emb[r0:r1].copy_(torch.randn((r1 - r0, dim), generator=g, device=dev, dtype=torch.float32).to(emb.dtype))
    torch.cuda.synchronize()


def run_all_hit(args):
    import numpy as np
    import torch
    from ugache_amd import hip
    import collcache.torch as co
    from collcache.common import _basics, kLogL3CacheCombineCacheTime
    from oracle_lib import Oracle

    rows, dim, n_keys = ALL_HIT[args.workload]
    row_bytes = dim * 4
    K = 200 if args.steps is None else args.steps
    W = 20 if args.warmup is None else args.warmup
    pool = 64 if args.pool is None else max(1, args.pool)
    dev = torch.device("cuda:0")

    co.config({"cache_percentage": 1.0, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
               "num_global_step_per_epoch": K + W, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 16})
    co.coll_cache_record_init(0)
    emb = co.coll_torch_create_emb_shm(0, rows, dim, torch.float32)
    fill_table_from_device(emb, dev, seed=1)
    co.coll_torch_init_t(0, 0, emb, 1.0)  # 100 % cache: the table is copied into HBM, keys index it directly

    gk = torch.Generator(device=dev).manual_seed(4)
    keys_pool = torch.randint(0, rows, (pool, n_keys), generator=gk, device=dev, dtype=torch.int32)
    out = torch.empty((n_keys, dim), dtype=torch.float32, device=dev)
    C = _basics.C_LIB_CTYPES
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    # device addresses taken once: slicing a tensor and asking for its pointer costs several microseconds of Python per
    # step, which is the caller's time, not the path's
    key_ptrs = [keys_pool[i].data_ptr() for i in range(pool)]
    out_ptr = out.data_ptr()

    def step(i):
        C.coll_cache_lookup(0, key_ptrs[i % pool], n_keys, out_ptr, stream)

    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    stamps = [0.0] * K  # the call blocks until the rows are in place, so a clock read after it bounds that step
    t0 = time.perf_counter()
    for i in range(W, W + K):
        step(i)
        stamps[i - W] = time.perf_counter()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    spread = step_spread(t0, stamps)

    so_step_s, so_launch_s = stream_ordered_leg(C, C.coll_cache_lookup_async, lambda i: key_ptrs[i % pool], n_keys, out,
                                                stream, torch, W, K)

    if args.calibrate:
        cal_src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        cal_dst = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        for _ in range(5):
            hip.call("ugk_copy_rows", cal_dst.data_ptr(), cal_src.data_ptr(), 1 << 30, stream)
        torch.cuda.synchronize()
        del cal_src, cal_dst

    # parity, byte for byte against the oracle: the last batch of the stream-ordered leg as it left it, then every
    # pooled batch through the blocking entry point
    orc = Oracle()
    table_np = emb.numpy()
    keys_host = keys_pool.cpu().numpy().view(np.uint32)
    if out.cpu().numpy().tobytes() != orc.gather(table_np, keys_host[(W + K - 1) % pool], omp=True).tobytes():
        sys.exit("bench.py: GPU output differs from the CPU oracle — no numbers reported")
    n_checked = check_every_batch(orc, table_np, keys_host, step, out, "all-hit")

    large = None
    if rows >= 1_000_000:
        large = all_hit_large_output_legs(C, orc, table_np, keys_pool, key_ptrs, keys_host, rows, dim, row_bytes,
                                          n_keys, stream, dev, W, K)

    # dominant kernel: average launch duration over a timed region of K launches, from two HIP events on the kernel's
    # stream around the K back-to-back launches of the stream-ordered leg (nothing else runs on that stream between
    # them).  The library logs a time of its own for every blocking call (kLogL3CacheCombineCacheTime), reported
    # beside it: from a host timer around launch and wait, like the reference's, or with COLL_KERNEL_EVENTS=1 from a
    # device event pair around the launch (about 2.4 us of marker latency in the figure, 1.9 us added to the step).
    kernel_avg_s = so_launch_s
    per_launch_pair_s = float(np.mean([_basics.step_value(s, kLogL3CacheCombineCacheTime) for s in range(W, W + K)]))
    alg_bytes = n_keys * (2 * row_bytes + 4)  # row read + row written + key read, per key
    achieved = alg_bytes / kernel_avg_s / 1e9

    table_bytes = table_np.view(np.uint8).reshape(rows, row_bytes)
    cpu_kps, n_cpu, cpu_el, cores = cpu_baseline(orc, table_bytes, keys_host, n_keys, row_bytes, args.cpu_seconds)

    info = hip.device_info(0)
    keys_per_s = n_keys * K / elapsed
    result = {
        "metric": "embedding keys/sec + effective extraction GB/s (% HBM / host-link roofline), 1 GPU",
        "value": keys_per_s, "unit": "keys/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": elapsed / K * 1e3, "ms_per_step_spread": spread,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": args.workload, "table_rows": rows, "row_bytes": row_bytes, "keys_per_batch": n_keys,
                   "key_dtype": "uint32", "cache_percentage": 1.0, "entry_point": "coll_cache_lookup",
                   "distinct_key_batches": pool, "seeds": {"table": 1, "keys": 4}},
        "effective_extraction_GBps": n_keys * row_bytes / (elapsed / K) / 1e9,
        "parity": "bit-exact vs CPU oracle: every one of the %d pooled batches, after the timed region" % n_checked,
        "device": info["name"] + " " + info["arch"],
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in "
                                       "profiles/gather_kernel_c2_all_hit.md (not read in this run)",
                     "kernel": "gather_kernel<u32x4,32,2,DirectU32>", "algorithmic_bytes_per_launch": alg_bytes,
                     "avg_kernel_us": kernel_avg_s * 1e6, "keys_per_s_kernel_only": n_keys / kernel_avg_s,
                     "timing": "2 HIP events around %d back-to-back launches on the kernel's stream" % K,
                     PER_CALL_KEY[os.environ.get("COLL_KERNEL_EVENTS", "0") != "0"]: per_launch_pair_s * 1e6},
        "cpu_baseline": {"value": cpu_kps, "unit": "keys/s", "cores": cores, "kind": "port",
                         "sample": "%d batches of %d keys from the same pool, %.1f s, OpenMP gather over keys"
                                   % (n_cpu, n_keys, cpu_el),
                         "effective_GBps": n_keys * row_bytes * n_cpu / cpu_el / 1e9},
        "gpu_over_cpu": keys_per_s / cpu_kps,
        "stream_ordered": {"keys_per_s": n_keys / so_step_s, "ms_per_step": so_step_s * 1e3,
                           "entry_point": "coll_cache_lookup_async (extension: enqueue only, one wait after the K "
                                          "steps; same batches, last one checked against the oracle as well)"},
    }
    if large is not None:
        result["all_hit_large_output"] = large
    co.coll_torch_shutdown()
    return result


def all_hit_large_output_legs(C, orc, table_np, keys_pool, key_ptrs, keys_host, rows, dim, row_bytes, n_keys, stream,
                              dev, W, K):
    """The same gather where the output cannot live in the 256 MB memory-side cache from one launch to the next:
    (a) batches of 2^20 keys, 537 MB of output per launch; (b) the configuration's own 262,144-key batches with the
    output rotated over 8 buffers of 134 MB.  Kernel time = two HIP events on the stream around K back-to-back
    stream-ordered launches; every batch timed in (a) and the last 8 of (b) are compared with the oracle."""
    import torch

    pool = len(key_ptrs)
    res = {}
    # (a) one million keys per launch
    n_big = 1 << 20
    big_pool = 4
    g = torch.Generator(device=dev).manual_seed(5)
    big_keys = torch.randint(0, rows, (big_pool, n_big), generator=g, device=dev, dtype=torch.int32)
    big_ptrs = [big_keys[i].data_ptr() for i in range(big_pool)]
    big_out = torch.empty((n_big, dim), dtype=torch.float32, device=dev)
    _, t_big = stream_ordered_leg(C, C.coll_cache_lookup_async, lambda i: big_ptrs[i % big_pool], n_big, big_out,
                                  stream, torch, W, K)
    big_host = big_keys.cpu().numpy().view("uint32")
    check_every_batch(orc, table_np, big_host,
                      lambda i: C.coll_cache_lookup(0, big_ptrs[i], n_big, big_out.data_ptr(), stream), big_out,
                      "1M-key all-hit")
    alg = n_big * (2 * row_bytes + 4)
    res["keys_1M"] = {"keys_per_batch": n_big, "output_bytes_per_launch": n_big * row_bytes,
                      "avg_kernel_us": t_big * 1e6, "algorithmic_bytes_per_launch": alg,
                      "achieved_GBps": alg / t_big / 1e9, "frac_of_hbm_peak": alg / t_big / 1e9 / HBM_PEAK_GBPS,
                      "keys_per_s_kernel_only": n_big / t_big, "batches_checked": big_pool}
    del big_out, big_keys
    # (b) the configuration's batches, outputs rotated
    R = 8
    outs = [torch.empty((n_keys, dim), dtype=torch.float32, device=dev) for _ in range(R)]
    out_ptrs = [o.data_ptr() for o in outs]
    _, t_rot = stream_ordered_leg(C, C.coll_cache_lookup_async, lambda i: key_ptrs[i % pool], n_keys, outs[0], stream,
                                  torch, W, K, out_ptr_of=lambda i: out_ptrs[i % R])
    for i in range(max(W, W + K - R), W + K):  # the last launches' outputs are still in their buffers
        if outs[i % R].cpu().numpy().tobytes() != orc.gather(table_np, keys_host[i % pool], omp=True).tobytes():
            sys.exit("bench.py: GPU output of rotated all-hit launch %d differs from the CPU oracle" % i)
    alg = n_keys * (2 * row_bytes + 4)
    res["outputs_rotated"] = {"keys_per_batch": n_keys, "output_buffers": R,
                              "output_bytes_in_rotation": R * n_keys * row_bytes, "avg_kernel_us": t_rot * 1e6,
                              "algorithmic_bytes_per_launch": alg, "achieved_GBps": alg / t_rot / 1e9,
                              "frac_of_hbm_peak": alg / t_rot / 1e9 / HBM_PEAK_GBPS,
                              "launches_checked": min(K, R)}
    res["timing"] = "2 HIP events around %d back-to-back stream-ordered launches on the kernel's stream" % K
    return res


def zipf_ranks_gpu(torch, n, space, s, gen, dev):
    """bounded-Pareto inverse CDF: r = floor(((H^(1-s) - 1) u + 1)^(1/(1-s))), H = space, ranks returned 0-based"""
    u = torch.rand(n, generator=gen, device=dev, dtype=torch.float64)
    h = float(space)
    r = torch.floor(((h ** (1.0 - s) - 1.0) * u + 1.0) ** (1.0 / (1.0 - s))).to(torch.int64) - 1
    return r.clamp_(0, space - 1)


def run_mixed(args):
    import numpy as np
    import torch
    from ugache_amd import hip
    import collcache.torch as co
    from collcache.common import (_basics, kLogL1MissBytes, kLogL3CacheCombineCacheTime, kLogL3CacheCombineMissTime,
                                  kLogL3CacheGetIndexTime)
    from oracle_lib import Oracle

    spec = MIXED[args.workload]
    rows, dim, n_keys, pct, fields = spec["rows"], spec["dim"], spec["n_keys"], spec["pct"], spec["fields"]
    tdtype = getattr(torch, spec["dtype"])
    row_bytes = dim * (2 if tdtype == torch.float16 else 4)
    K = 50 if args.steps is None else args.steps
    W = 5 if args.warmup is None else args.warmup
    pool = 16 if args.pool is None else max(1, args.pool)
    dev = torch.device("cuda:0")
    t_setup = time.perf_counter()

    if args.impl:
        os.environ["SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL"] = args.impl
    if args.dedup:
        os.environ["COLL_DEDUP_KEYS"] = "1"
        os.environ.setdefault("COLL_KERNEL_EVENTS", "1")  # the extraction after the dedup timed on the device
    if args.device_refresh:
        args.gpu_record = True
        os.environ["COLL_GPU_REFRESH"] = "1"
        os.environ["COLL_GPU_REFRESH_KEEP"] = "1"
        # rows the lookups fetch from the host table are filed in HBM (4 Mi entries), where the refresh finds most of
        # the rows it inserts; COLL_MISS_STAGE_ROWS=0 in the environment turns that off for a comparison
        os.environ.setdefault("COLL_MISS_STAGE_ROWS", str(args.stage_rows))
    if args.gpu_record:
        os.environ["COLL_GPU_RECORD"] = "1"
    co.config({"cache_percentage": pct, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
               "num_global_step_per_epoch": K + W, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 16})
    sparse = bool(spec.get("sparse"))
    KEY_MUL, KEY_BITS = 0x9E3779B97F4A7C15, 40
    if sparse:
        _basics.set_key_map(KEY_MUL, KEY_BITS)
    co.coll_cache_record_init(0)
    note = lambda msg: print("[bench %6.1fs] %s" % (time.perf_counter() - t_setup, msg), file=sys.stderr, flush=True)
    emb = co.coll_torch_create_emb_shm(0, rows, dim, tdtype)
    note("pinned host table allocated: %.1f GB" % (rows * row_bytes / 1e9))
    fill_table_from_device(emb, dev, seed=1)
    note("host table filled")

    # hotness: Zipf(s) ranks over a seeded permutation of the ids (one permutation per field)
    per_field = rows // fields
    gp = torch.Generator(device=dev).manual_seed(2)
    perms = [torch.randperm(per_field, generator=gp, device=dev, dtype=torch.int64) for _ in range(fields)]
    gz = torch.Generator(device=dev).manual_seed(3)

    def ids_of(rows_t):
        """caller-side ids of rows: identity, or (row * odd) mod 2^40 in sparse-id mode (int64 multiply wraps)"""
        if not sparse:
            return rows_t
        mul = torch.tensor(KEY_MUL - (1 << 64), dtype=torch.int64, device=rows_t.device)
        return (rows_t * mul) & ((1 << KEY_BITS) - 1)

    def make_batch():
        """one batch of ROW numbers"""
        if fields == 1:
            return perms[0][zipf_ranks_gpu(torch, n_keys, per_field, spec["zipf"], gz, dev)]
        per = n_keys // fields  # [samples, fields] laid out row-major: key = f * per_field + perm_f[rank]
        cols = [perms[f][zipf_ranks_gpu(torch, per, per_field, spec["zipf"], gz, dev)] + f * per_field
                for f in range(fields)]
        return torch.stack(cols, dim=1).reshape(-1)

    for _ in range(spec["presample"]):
        co.coll_torch_record(0, ids_of(make_batch()).cpu())
    note("hotness of %d presample batches recorded" % spec["presample"])
    t_build = time.perf_counter()
    co.coll_torch_init_t(0, 0, emb, pct)
    build_s = time.perf_counter() - t_build
    info_cache = _basics.info(0)
    note("cache built in %.3f s: %d rows cached" % (build_s, info_cache["cached_rows"]))

    rows_pool = torch.stack([make_batch() for _ in range(pool)])
    keys_pool = ids_of(rows_pool)
    out = torch.empty((n_keys, row_bytes), dtype=torch.uint8, device=dev)
    C = _basics.C_LIB_CTYPES
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    setup_s = time.perf_counter() - t_setup

    # host-link ceiling measured on this box: a 1 GiB pinned -> HBM copy
    probe_bytes = min(1 << 30, rows * row_bytes)
    probe = torch.empty(probe_bytes, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    link = []
    for _ in range(3):
        t0 = time.perf_counter()
        hip.call("ugk_memcpy_async", probe.data_ptr(), emb.data_ptr(), probe_bytes, stream)
        torch.cuda.synchronize()
        link.append(probe_bytes / (time.perf_counter() - t0) / 1e9)
    link_gbps = max(link)
    del probe

    key_ptrs = [keys_pool[i].data_ptr() for i in range(pool)]  # taken once, outside the timed steps
    out_ptr = out.data_ptr()

    def step(i):
        C.coll_cache_lookup_i64(0, key_ptrs[i % pool], n_keys, out_ptr, stream)

    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    stamps = [0.0] * K  # the call blocks until the rows are in place, so a clock read after it bounds that step
    t0 = time.perf_counter()
    for i in range(W, W + K):
        step(i)
        stamps[i - W] = time.perf_counter()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    spread = step_spread(t0, stamps)
    note("timed region done: %.3f ms/step" % (elapsed / K * 1e3))
    g_blocking = _basics.last_group_offset(0)
    so_step_s, so_launch_s = stream_ordered_leg(C, C.coll_cache_lookup_async_i64, lambda i: key_ptrs[i % pool], n_keys,
                                                out, stream, torch, W, K)
    note("stream-ordered leg done: %.3f ms/step" % (so_step_s * 1e3))

    if args.calibrate:  # a kernel of known traffic beside the extraction kernel, for counter runs
        cal_src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        cal_dst = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        for _ in range(5):
            hip.call("ugk_copy_rows", cal_dst.data_ptr(), cal_src.data_ptr(), 1 << 30, stream)
        torch.cuda.synchronize()
        del cal_src, cal_dst

    orc = Oracle()
    table_np = emb.numpy().view(np.uint8).reshape(rows, row_bytes)
    rows_host = rows_pool.cpu().numpy()
    if out.cpu().numpy().tobytes() != orc.gather(table_np, rows_host[(W + K - 1) % pool], omp=True).tobytes():
        sys.exit("bench.py: GPU output differs from the CPU oracle — no numbers reported")
    n_checked = check_every_batch(orc, table_np, rows_host, step, out, args.workload)
    note("all %d pooled batches equal the oracle's gather" % n_checked)

    steps = range(W, W + K)  # (the parity pass above ran later steps; these are the timed ones)
    t_idx = float(np.mean([_basics.step_value(s, kLogL3CacheGetIndexTime) for s in steps]))
    t_miss = float(np.mean([_basics.step_value(s, kLogL3CacheCombineMissTime) for s in steps]))
    t_hit = float(np.mean([_basics.step_value(s, kLogL3CacheCombineCacheTime) for s in steps]))
    miss_bytes = float(np.mean([_basics.step_value(s, kLogL1MissBytes) for s in steps]))
    n_miss = miss_bytes / row_bytes
    n_hit = n_keys - n_miss
    if args.dedup:  # the gathers ran over the distinct keys: take their group sizes from the last timed batch
        g = g_blocking
        n_hit, n_miss = float(g[1]), float(g[2] - g[1])
        miss_bytes = n_miss * row_bytes
    fused = t_miss == 0.0 and t_idx == 0.0  # one kernel did lookup and both gathers: its time is logged as t_hit
    entry = 128 if info_cache["table_kind"] >= 2 else 4  # bytes of table read per key: a line of entries / a flat word
    per_launch_pair_us = t_hit * 1e6
    if fused and not args.dedup:
        # one kernel per step: its average duration over the K back-to-back launches of the stream-ordered leg (two
        # HIP events on its stream) replaces the per-launch event pair of the blocking calls, which carries about
        # 2.4 us of marker latency
        t_hit = so_launch_s
    if fused:
        # HBM side of the fused kernel: key + table entry per key, hit rows read and written, missed rows written
        hit_alg = n_keys * (8 + entry) + n_hit * 2 * row_bytes + n_miss * row_bytes
        t_link = t_hit
        # keys per wavefront, by the launcher's rule (ugk_partition.hip): short wavefronts except where the lookups
        # weigh more (small rows, the hash probe)
        slots = hip.device_info(0)["compute_units"] * 4 * 8
        lpr = min(64, max(1, 1 << (max(1, row_bytes // 16) - 1).bit_length()))
        small_rows = lpr <= 8
        if info_cache["table_kind"] == 1:
            kpw = 32 if small_rows else 8
        elif n_keys <= slots:
            kpw = 8
        elif small_rows:
            kpw = 32 if n_keys <= slots * 16 else 64
        else:
            kpw = 16 if n_keys <= slots * 8 else 32 if n_keys <= slots * 16 else 64 if n_keys <= slots * 32 else 16
        kpw = max(kpw, 64 // lpr)
        kernel_name = ("extract_mix_kernel<long,%d,%d,%d> (lookup + both gathers; bound by the host link, see "
                       "host_link)" % (info_cache["table_kind"], lpr, kpw))
        stages = {"extract_mix": t_hit * 1e6}
    else:
        hit_alg = n_hit * (2 * row_bytes + 8)  # row read + row written + 8-byte index record
        t_link = t_miss
        kernel_name = "gather_kernel<u32x4,%d,2,IdxList> (local group, running next to the host-link gather)" % min(
            64, max(1, row_bytes // 16))
        stages = {"classify_partition": t_idx * 1e6, "host_gather": t_miss * 1e6, "hbm_gather": t_hit * 1e6}
    achieved = hit_alg / t_hit / 1e9 if t_hit > 0 else 0.0

    # (with deduplication the group sizes count distinct keys, the skip-local extraction every key: the plain leg of
    # the same workload carries this figure)
    miss_alone = None if args.dedup else miss_stream_alone(C, _basics, step, stream, torch, W, K, pool, rows_host, table_np, orc, out,
                                   row_bytes, link_gbps, kLogL1MissBytes, kLogL3CacheCombineCacheTime,
                                   kLogL3CacheCombineMissTime, args.workload, note)
    ceiling = random_row_ceiling(hip, torch, emb, rows, row_bytes, dev, stream, note)

    # The CPU baseline, two ways, each for half the budget.  (i) the whole step as the CPU would do it: id -> row, lookup
    # in a flat host array, per-row source (a host-side copy of the cached rows, or the host table), copy; its first
    # batch is compared with the GPU's output.  (ii) a plain gather by row number out of the host table, spared the
    # lookup and the id -> row translation: the fastest the CPU can be on these batches.
    keys_host = rows_host
    cached_now = np.zeros(info_cache["cached_rows"], np.uint32)
    C.coll_cache_get_cached_keys(0, cached_now.ctypes.data, len(cached_now))
    ids_host = np.ascontiguousarray(keys_pool.cpu().numpy())
    step(0)
    torch.cuda.synchronize()
    gpu_batch0 = out.cpu().numpy().tobytes()
    key_inv = pow(KEY_MUL, -1, 1 << KEY_BITS) if sparse else 0
    cpu8_kps, n_cpu8, cpu8_el, cores, cpu_split = cpu_baseline_lookup_and_gather(
        orc, table_np, cached_now, ids_host, key_inv, (1 << KEY_BITS) - 1 if sparse else 0, n_keys, row_bytes,
        args.cpu_seconds / 2, gpu_batch0)
    note("CPU lookup + gather: %.1f M keys/s on %d threads" % (cpu8_kps / 1e6, cores))
    cpu_kps, n_cpu, cpu_el, cores = cpu_baseline(orc, table_np, keys_host, n_keys, row_bytes, args.cpu_seconds / 2)
    uniq = float(np.mean([len(np.unique(keys_host[i])) for i in range(min(pool, 4))]))

    refresh = None
    each_step = None
    if args.device_refresh:
        # Every step ends with a refresh computed on the device from the hotness accumulated so far.  Hotness drifts by
        # 1 % of the cache per step: a slice of so-far never-looked-up rows is looked up once between the steps
        # (untimed), which ranks them above the never-observed rows the cache is filled up with, so each refresh evicts
        # and inserts at least that many rows.
        before = _basics.info(0)
        n_new = before["cached_rows"] // 100
        t0 = time.perf_counter()
        co.coll_torch_refresh(0, True)  # settles the cache on what the timed steps counted
        settle_s = time.perf_counter() - t0
        note("first refresh on the device (settling): %.4f s" % settle_s)
        n_steps = min(K, 20)
        staged_before = _basics.C_LIB_CTYPES.coll_cache_rows_from_stage(0)
        t_lookup = t_refresh = 0.0
        cold_end = per_field
        t_loop = time.perf_counter()
        for i in range(n_steps):
            cold = perms[0][cold_end - n_new:cold_end]
            cold_end -= n_new
            drift = ids_of(cold).contiguous()
            C.coll_cache_lookup_i64(0, drift.data_ptr(), n_new, out.data_ptr(), stream)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            step(i)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            co.coll_torch_refresh(0, True)
            t2 = time.perf_counter()
            t_lookup += t1 - t0
            t_refresh += t2 - t1
        torch.cuda.synchronize()
        wall_s = time.perf_counter() - t_loop
        after = _basics.info(0)
        staged_rows = _basics.C_LIB_CTYPES.coll_cache_rows_from_stage(0) - staged_before
        step(0)
        torch.cuda.synchronize()
        if out.cpu().numpy().tobytes() != orc.gather(table_np, rows_pool[0].cpu().numpy(), omp=True).tobytes():
            sys.exit("bench.py: GPU output differs from the CPU oracle after the per-step refreshes")
        each_step = {"steps": n_steps, "lookup_ms": t_lookup / n_steps * 1e3, "refresh_ms": t_refresh / n_steps * 1e3,
                     "ms_per_step": (t_lookup + t_refresh) / n_steps * 1e3,
                     "keys_per_s": n_keys * n_steps / (t_lookup + t_refresh),
                     "wall_ms_per_step_with_the_drift_lookup": wall_s / n_steps * 1e3,

                     "drift_rows_looked_up_per_step": n_new, "first_refresh_s": settle_s,
                     "row_copy_floor_ms": n_new * row_bytes / (ceiling["best_GBps"] * 1e9) * 1e3,
                     "row_copy_floor_note": "at most drift_rows rows cross the host link per refresh (fewer when some "
                                            "of them were cached as filler); the floor is that many rows of this size "
                                            "at host_link.random_row_ceiling, the rate uniformly random rows of this "
                                            "size reach out of this table",
                     "table_rebuilds": after["table_rebuilds"], "cached_rows_after": after["cached_rows"],
                     "free_slots_after": after["free_slots"],
                     "stage_rows": int(os.environ.get("COLL_MISS_STAGE_ROWS", "0")),
                     "rows_taken_from_the_stage_per_refresh": staged_rows / n_steps,
                     "note": "refresh = rank + place + evict/insert lists on the device (COLL_GPU_REFRESH=1, hotness "
                             "accumulating), row copy over the host link, table update; foreground, after each lookup"}
        note("refresh each step: lookup %.3f ms + refresh %.3f ms; %.3f ms of wall clock per step with the drift lookup"
             % (each_step["lookup_ms"], each_step["refresh_ms"], each_step["wall_ms_per_step_with_the_drift_lookup"]))
    elif sparse and not args.serving:
        # one foreground refresh: the same hotness again, plus 1 % of the cache size worth of so-far uncached rows
        # pushed to the top, so that about 1 % of the cached rows are evicted and replaced
        before = _basics.info(0)
        n_new = before["cached_rows"] // 100
        for _ in range(spec["presample"]):
            co.coll_torch_record(0, ids_of(make_batch()).cpu())
        cold = perms[0][per_field - n_new:]  # the coldest ranks of the permutation
        boost = ids_of(cold).cpu()
        for _ in range(64):
            co.coll_torch_record(0, boost)
        note("hotness for the refresh recorded")
        t0 = time.perf_counter()
        co.coll_torch_refresh(0, True)
        refresh_s = time.perf_counter() - t0
        after = _basics.info(0)
        note("refresh done in %.2f s" % refresh_s)
        step(0)
        torch.cuda.synchronize()
        if out.cpu().numpy().tobytes() != orc.gather(table_np, rows_pool[0].cpu().numpy(), omp=True).tobytes():
            sys.exit("bench.py: GPU output differs from the CPU oracle after the refresh")
        refresh = {"seconds": refresh_s, "boosted_rows": n_new, "table_rebuilds": after["table_rebuilds"],
                   "cached_rows_after": after["cached_rows"], "free_slots_after": after["free_slots"]}

    serving = None
    if args.serving:
        # LookupManager::forward (lookup_manager.cc:158-213): every step records the first 5 % of the batch, looks the
        # batch up (blocking) and, every K/2 steps, starts a refresh on a background thread.  The steps take fresh
        # batches from the workload's distribution (up to 256 of them, then round again), so a refresh gains what the
        # hotness it saw predicts, not the keys of a small pool that comes round every few steps.
        n_srv = min(W + K, 256)
        srv_rows = torch.stack([make_batch() for _ in range(n_srv)])
        srv_keys = ids_of(srv_rows)
        srv_ptrs = [srv_keys[i % n_srv].data_ptr() for i in range(W + K)]
        torch.cuda.synchronize()
        C.coll_cache_forward_config(1, max(K // 2, 1), 0.05, 1)
        for i in range(W):
            C.coll_cache_forward_i64(0, srv_ptrs[i], n_keys, out.data_ptr(), stream)
        torch.cuda.synchronize()
        before, during, after_r = [], [], []  # per-step times: no refresh yet, one running behind the step, one done
        t0 = time.perf_counter()
        for i in range(W, W + K):
            ts = time.perf_counter()
            C.coll_cache_forward_i64(0, srv_ptrs[i], n_keys, out.data_ptr(), stream)
            dt = time.perf_counter() - ts
            if C.coll_cache_forward_refresh_ongoing():
                during.append(dt)
            else:
                (after_r if during else before).append(dt)
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        t1 = time.perf_counter()
        done = int(C.coll_cache_forward_join())
        join_s = time.perf_counter() - t1
        C.coll_cache_forward_config(0, 0, 0.0, 0)
        if out.cpu().numpy().tobytes() != orc.gather(table_np, srv_rows[(W + K - 1) % n_srv].cpu().numpy(),
                                                     omp=True).tobytes():
            sys.exit("bench.py: GPU output differs from the CPU oracle in the serving loop")
        med = lambda v: round(float(np.median(v)) * 1e3, 4) if v else None
        serving = {"ms_per_step": el / K * 1e3, "keys_per_s": n_keys * K / el, "steps": K,
                   "ms_per_step_median": {"before_the_refresh": med(before), "while_it_runs": med(during),
                                          "after_it": med(after_r)},
                   "steps_of_each": [len(before), len(during), len(after_r)],
                   "ms_longest_step": max(before + during + after_r) * 1e3,
                   "recorded_fraction": 0.05, "refresh_every_steps": max(K // 2, 1), "refreshes_completed": done,
                   "seconds_waited_for_the_last_refresh": join_s,
                   "hotness_recorded_on": "device" if args.gpu_record else "host",
                   "batches": "%d fresh batches, one per step, cycled" % n_srv,
                   "entry_point": "coll_cache_forward_i64 (record a prefix + blocking lookup + background refresh)"}
        note("serving loop: %.3f ms/step (median %s before, %s during, %s after the refresh; longest %.2f ms), "
             "%d refreshes" % (serving["ms_per_step"], med(before), med(during), med(after_r),
                               serving["ms_longest_step"], done))
        del srv_rows, srv_keys

    under_refresh = None
    if args.concurrent_refresh:
        if not (sparse and args.gpu_record):
            sys.exit("bench.py: --concurrent-refresh needs a sparse-id workload and --gpu-record")
        import threading
        stop, done, moved = [False], [0], []

        def refresher():
            while not stop[0]:
                before_keys = _basics.info(0)["free_slots"]
                co.coll_torch_refresh(0, False)  # hotness: what the lookups counted on the device since the last one
                done[0] += 1
                moved.append(before_keys)

        n_steps = max(K, int(2.0 / (elapsed / K)))  # about two seconds of lookups
        th = threading.Thread(target=refresher)
        th.start()
        t0 = time.perf_counter()
        for i in range(n_steps):
            step(i)
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        stop[0] = True
        while th.is_alive():  # a refresh in flight waits for one more lookup to pass
            step(0)
            th.join(timeout=0.01)
        last = (n_steps - 1) % pool
        step(last)
        torch.cuda.synchronize()
        if out.cpu().numpy().tobytes() != orc.gather(table_np, rows_pool[last].cpu().numpy(), omp=True).tobytes():
            sys.exit("bench.py: GPU output differs from the CPU oracle under concurrent refresh")
        under_refresh = {"ms_per_step": el / n_steps * 1e3, "keys_per_s": n_keys * n_steps / el, "steps": n_steps,
                         "refreshes_completed": done[0], "seconds": el,
                         "table_rebuilds": _basics.info(0)["table_rebuilds"],
                         "note": "the hotness comes from the cycled pool of key batches itself, so the refreshed "
                                 "cache converges onto the pool and the hit rate rises; the figure shows that lookups "
                                 "stay exact and keep their pace while rows are evicted and inserted under them, not "
                                 "a steady-state rate"}
        note("under concurrent refresh: %.3f ms/step, %d refreshes in %.2f s" % (el / n_steps * 1e3, done[0], el))

    info = hip.device_info(0)
    keys_per_s = n_keys * K / elapsed
    result = {
        "metric": "embedding keys/sec + effective extraction GB/s (% HBM / host-link roofline), 1 GPU",
        "value": keys_per_s, "unit": "keys/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": elapsed / K * 1e3, "ms_per_step_spread": spread,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "refresh": refresh, "refresh_each_step": each_step, "under_concurrent_refresh": under_refresh,
        "serving_loop": serving,
        # ranking of the presample, placement, the cached rows copied host -> HBM and their keys put into the table
        "cache_build": {"seconds": build_s, "rows_filled": info_cache["cached_rows"],
                        "bytes_filled": info_cache["cached_rows"] * row_bytes,
                        "fill_GBps_over_the_whole_build": info_cache["cached_rows"] * row_bytes / build_s / 1e9,
                        "frac_of_measured_link": info_cache["cached_rows"] * row_bytes / build_s / 1e9 / link_gbps
                        if link_gbps > 0 else None},
        "config": {"workload": args.workload, "table_rows": rows, "row_bytes": row_bytes, "keys_per_batch": n_keys,
                   "key_dtype": "int64", "sparse_ids": sparse, "cache_percentage": pct, "cached_rows": info_cache["cached_rows"],
                   "cache_capacity_rows": info_cache["capacity_rows"], "table_kind": info_cache["table_kind"],
                   "zipf_s": spec["zipf"], "fields": fields, "presample_batches": spec["presample"],
                   "entry_point": "coll_cache_lookup_i64", "distinct_key_batches": pool, "impl": args.impl or "fused (default)", "dedup": bool(args.dedup), "gpu_record": bool(args.gpu_record), "device_refresh": bool(args.device_refresh),
                   "unique_keys_per_batch": uniq, "seeds": {"table": 1, "perm": 2, "keys": 3}},
        "effective_extraction_GBps": n_keys * row_bytes / (elapsed / K) / 1e9,
        "parity": "bit-exact vs CPU oracle: every one of the %d pooled batches, after the timed region" % n_checked,
        "device": info["name"] + " " + info["arch"],
        "stages_us": stages,
        "hit_rate": n_hit / (n_hit + n_miss),  # over the keys that were extracted (the distinct ones with --dedup)
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload) if fused else None,
                     "kernel": kernel_name,
                     "algorithmic_bytes_per_launch": hit_alg, "avg_kernel_us": t_hit * 1e6,
                     PER_CALL_KEY[os.environ.get("COLL_KERNEL_EVENTS", "0") != "0"]: per_launch_pair_us},
        "host_link": {"achieved": miss_bytes / t_link / 1e9 if t_link > 0 else 0.0, "measured_peak": link_gbps,
                      "unit": "GB/s", "frac": (miss_bytes / t_link / 1e9) / link_gbps if t_link > 0 else 0.0,
                      "miss_rows_per_batch": n_miss, "peak_probe": "pinned host -> HBM hipMemcpyAsync, best of 3",
                      "random_row_ceiling": ceiling,
                      "frac_of_row_ceiling": ((miss_bytes / t_link / 1e9) / ceiling["best_GBps"]
                                              if t_link > 0 and ceiling["best_GBps"] > 0 else None),
                      "miss_stream_alone": miss_alone},
        "cpu_baseline": {"value": cpu8_kps, "unit": "keys/s", "cores": cores, "kind": "port",
                         "sample": "%d batches of %d keys from the same pool, %.1f s: per key id -> row, lookup in a "
                                   "flat host array, copy of the row from a host-side copy of the cached rows or from "
                                   "the host table, OpenMP over keys; first batch byte-equal to the GPU's output"
                                   % (n_cpu8, n_keys, cpu8_el),
                         "effective_GBps": n_keys * row_bytes * n_cpu8 / cpu8_el / 1e9,
                         "rows_from_cache_copy_first_batch": cpu_split[0],
                         "gather_by_row_number": {
                             "value": cpu_kps, "unit": "keys/s", "cores": cores,
                             "sample": "%d batches, %.1f s, OpenMP gather by row number out of the whole host table "
                                       "(no lookup, no id -> row step: the fastest the CPU can be)" % (n_cpu, cpu_el)}},
        "gpu_over_cpu": keys_per_s / cpu8_kps,
        "gpu_over_cpu_gather_by_row_number": keys_per_s / cpu_kps,
        "setup_seconds": setup_s,
        "stream_ordered": {"keys_per_s": n_keys / so_step_s, "ms_per_step": so_step_s * 1e3,
                           "entry_point": "coll_cache_lookup_async_i64 (extension: enqueue only, one wait after the K "
                                          "steps; same batches, last one checked against the oracle as well)"},
    }
    co.coll_torch_shutdown()
    return result


def miss_stream_alone(C, _basics, step, stream, torch, W, K, pool, rows_host, table_np, orc, out, row_bytes, link_gbps,
                      kLogL1MissBytes, kLogL3CacheCombineCacheTime, kLogL3CacheCombineMissTime, workload, note):
    """The host-link half on its own, through the library: COLL_SKIP_LOCAL=1 (the reference's aid for exactly this,
    cache_context.cu:728-741) drops the keys the cache serves in front of the extraction, so the extraction kernel
    moves the missed rows only.  Its time is what the library logs for the step: a host timer around the kernel's
    launch and the wait for it (about 10 us more than the kernel itself)."""
    import numpy as np

    os.environ["COLL_SKIP_LOCAL"] = "1"
    try:
        first = _basics.info(0)["lookups"]
        for i in range(W + K):
            step(i)
        torch.cuda.synchronize()
        steps = range(first + W, first + W + K)
        t = np.array([max(_basics.step_value(s, kLogL3CacheCombineCacheTime),
                          _basics.step_value(s, kLogL3CacheCombineMissTime)) for s in steps])
        b = np.array([_basics.step_value(s, kLogL1MissBytes) for s in steps])
        # parity of the compacted output: the rows of the keys the cache does not hold, in their order
        last = (W + K - 1) % pool
        g = _basics.last_group_offset(0)
        m = int(g[2])
        got = out[:m].cpu().numpy().tobytes()
    finally:
        del os.environ["COLL_SKIP_LOCAL"]
    step(last)  # the same batch in full tells which keys were missed: group sizes [0, hits, n]
    torch.cuda.synchronize()
    full = out.cpu().numpy()
    want_full = orc.gather(table_np, rows_host[last], omp=True)
    if full.tobytes() != want_full.tobytes() or m != int(_basics.last_group_offset(0)[2] - _basics.last_group_offset(0)[1]):
        sys.exit("bench.py: %s: the skip-local run and the full run disagree on the missed keys" % workload)
    # every row of the compacted output must be a row of the batch, in batch order: match them greedily
    want = want_full.reshape(len(rows_host[last]), row_bytes)
    comp = np.frombuffer(got, np.uint8).reshape(m, row_bytes)
    j = 0
    for i in range(len(want)):
        if j < m and want[i].tobytes() == comp[j].tobytes():
            j += 1
    if j != m:
        sys.exit("bench.py: %s: the skip-local output is not the missed rows in batch order" % workload)
    gbps = float(b.sum() / t.sum() / 1e9)
    note("miss stream alone: %.1f GB/s over %.0f rows per batch" % (gbps, b.mean() / row_bytes))
    return {"achieved_GBps": gbps, "frac_of_measured_peak": gbps / link_gbps, "rows_per_batch": float(b.mean() / row_bytes),
            "us_per_batch": float(t.mean() * 1e6), "how": "COLL_SKIP_LOCAL=1 through coll_cache_lookup_i64; time = the "
            "library's per-step log (host timer around launch and wait of the extraction kernel)"}


def random_row_ceiling(hip, torch, emb, rows, row_bytes, dev, stream, note):
    """What rows of this size reach over the host link at all: a stand-alone gather (ugk_gather_direct_i64, no table) of
    uniformly random rows out of the whole pinned table, timed with two HIP events around 5 launches, for several grid
    caps; the best is the ceiling a miss stream of such rows can be measured against."""
    n = max(1 << 16, min(1 << 20, (256 << 20) // row_bytes))
    g = torch.Generator(device=dev).manual_seed(11)
    keys = torch.randint(0, rows, (n,), generator=g, device=dev, dtype=torch.int64)
    dst = torch.empty((n, row_bytes), dtype=torch.uint8, device=dev)
    st = torch.zeros(4, dtype=torch.int32, device=dev)
    ev = [ctypes.c_void_p(), ctypes.c_void_p()]
    for e in ev:
        hip.call("ugk_event_create", ctypes.byref(e))
    res = {}
    for blocks in (0, 2048, 512, 128):
        def go():
            hip.call("ugk_gather_direct_i64", emb.data_ptr(), rows, keys.data_ptr(), n, dst.data_ptr(), row_bytes,
                     blocks, st.data_ptr(), None, stream)
        go()
        torch.cuda.synchronize()
        hip.call("ugk_event_record", ev[0], stream)
        for _ in range(5):
            go()
        hip.call("ugk_event_record", ev[1], stream)
        torch.cuda.synchronize()
        ms = ctypes.c_float()
        hip.call("ugk_event_elapsed_ms", ev[0], ev[1], ctypes.byref(ms))
        res["workgroups_%s" % (blocks or "unlimited")] = n * row_bytes * 5 / (ms.value * 1e-3) / 1e9
    for e in ev:
        hip.call("ugk_event_destroy", e)
    if int(st[0].item()) != 0:
        sys.exit("bench.py: the random-row probe read outside the table")
    best = max(res.values())
    note("random %d-byte rows over the link: best %.1f GB/s" % (row_bytes, best))
    return {"best_GBps": best, "by_grid_cap_GBps": res, "rows_per_launch": n, "row_bytes": row_bytes,
            "span_bytes": rows * row_bytes, "how": "ugk_gather_direct_i64 of uniformly random rows of the pinned table, "
            "2 HIP events around 5 launches"}


# what a leg contributes to the default line: enough to recompute both halves of the metric
LEG_KEYS = ("value", "unit", "ms_per_step", "ms_per_step_spread", "steps", "warmup", "config", "hit_rate",
            "effective_extraction_GBps", "parity", "stages_us", "roofline", "host_link", "cpu_baseline", "gpu_over_cpu",
            "refresh", "refresh_each_step", "setup_seconds", "stream_ordered", "cache_build")
# (short name, workload, extra options, what it is)
DEFAULT_LEGS = (
    ("c3", "c3_gnn_100Mx128xfp32_1M_i64_zipf0.9_cache25pct", (), "configuration 3, every key extracted (default)"),
    ("c3_dedup", "c3_gnn_100Mx128xfp32_1M_i64_zipf0.9_cache25pct", ("--dedup",),
     "configuration 3 as BASELINE words it: distinct keys extracted once, duplicates re-expanded (COLL_DEDUP_KEYS=1)"),
    ("c4_half", "c4_dlr_half_26x4Mx128xfp32_212992_i64_zipf1.2_cache20GB", (),
     "configuration 4 at half its rows per field: the box pins 64 GiB, the full 106 GB cannot be pinned"),
    ("c1", "c1_cpu_ref_1Mx128xfp32_65536_i64_zipf1.1_cache10pct", (), "configuration 1's shape on the GPU"),
    ("c5", "c5_hash_500Mx64xfp16_1M_i64_zipf1.05_cache50M", (), "configuration 5, lookups and one host-side refresh"),
    ("c5_device_refresh", "c5_hash_500Mx64xfp16_1M_i64_zipf1.05_cache50M", ("--device-refresh",),
     "configuration 5 with a refresh after every step, counted, ranked and placed on the device"),
)


def run_child(workload, args, cpu_seconds, extra=()):
    """one workload in a child process (this process has not touched the GPU); returns its JSON line as a dict"""
    import subprocess

    cmd = [sys.executable, os.path.abspath(__file__), "--workload", workload, "--cpu-seconds", str(cpu_seconds)]
    cmd += list(extra)
    if args.steps is not None:
        cmd += ["--steps", str(args.steps)]
    if args.warmup is not None:
        cmd += ["--warmup", str(args.warmup)]
    if args.pool is not None:
        cmd += ["--pool", str(args.pool)]
    t0 = time.perf_counter()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=None, text=True)
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    if proc.returncode != 0 or not lines:
        return None, "exit status %d after %.0f s" % (proc.returncode, time.perf_counter() - t0)
    return json.loads(lines[-1]), None


def run_default(args):
    main_name = "c2_all_hit_10Mx128xfp32_262144_u32_uniform"
    result, err = run_child(main_name, args, args.cpu_seconds)
    if result is None:
        sys.exit("bench.py: the all-hit configuration failed: %s" % err)
    legs, summary = {}, {}
    if not args.no_legs:
        for short, name, extra, what in DEFAULT_LEGS:
            leg, err = run_child(name, args, 0.5 if "--device-refresh" in extra else min(args.cpu_seconds, 4.0), extra=extra)
            if leg is None:
                # a leg that cannot report (a parity failure ends it without a number) takes the whole line with it
                sys.exit("bench.py: leg %s (%s %s) failed: %s" % (short, name, " ".join(extra), err))
            legs[short] = {k: leg[k] for k in LEG_KEYS if k in leg}
            legs[short]["what"] = what
            hl = leg.get("host_link") or {}
            summary[short] = {"ms_per_step": leg["ms_per_step"], "keys_per_s": leg["value"], "hit_rate": leg.get("hit_rate"),
                              "host_link_GBps": hl.get("achieved"), "host_link_frac": hl.get("frac"),
                              "frac_of_row_ceiling": hl.get("frac_of_row_ceiling"),
                              "cpu_keys_per_s": leg["cpu_baseline"]["value"], "cpu_cores": leg["cpu_baseline"]["cores"],
                              "gpu_over_cpu": leg.get("gpu_over_cpu"), "parity": "bit-exact, every pooled batch"}
            if leg.get("refresh_each_step"):
                summary[short]["refresh_each_step_ms"] = leg["refresh_each_step"]["ms_per_step"]
                summary[short]["refresh_ms"] = leg["refresh_each_step"]["refresh_ms"]
            if leg.get("cache_build"):
                summary[short]["build_frac_of_link"] = leg["cache_build"]["frac_of_measured_link"]
    result["legs"] = legs
    result["legs_note"] = ("each leg is the same bench.py with --workload <name> (and the options named), run after the "
                           "top-level workload in a process of its own, same --steps and --warmup; value / roofline / "
                           "cpu_baseline at the top level are the all-hit configuration's alone")
    # The figures of the other configurations once more in short form, at the top level and inside `roofline` (a
    # reader that keeps only the objects of the contract keeps these)
    large = result.get("all_hit_large_output") or {}
    short_keys = {"c2_frac_output_1M_keys": (large.get("keys_1M") or {}).get("frac_of_hbm_peak"),
                  "c2_frac_outputs_rotated_1GiB": (large.get("outputs_rotated") or {}).get("frac_of_hbm_peak")}
    for short, sm in summary.items():
        short_keys[short + "_ms_per_step"] = sm["ms_per_step"]
        short_keys[short + "_host_link_frac"] = sm["host_link_frac"]
        short_keys[short + "_gpu_over_cpu"] = sm["gpu_over_cpu"]
    result.update(short_keys)
    result["roofline"]["other_configs"] = dict(summary, **{"c2_large_output": {
        "frac_output_1M_keys": short_keys["c2_frac_output_1M_keys"],
        "frac_outputs_rotated_1GiB": short_keys["c2_frac_outputs_rotated_1GiB"]}})
    emit(result)


_REAL_STDOUT = None


def emit(result):
    """the one JSON line, on the real stdout"""
    sys.stdout.flush()
    os.write(_REAL_STDOUT if _REAL_STDOUT is not None else 1, (json.dumps(result) + "\n").encode())


def main():
    global _REAL_STDOUT
    args = parse_args()
    if args.probe:
        import bench_probes

        bench_probes.run(args.probe, args.quick)
        return
    if args.workload is None:
        return run_default(args)
    # the library prints the reference's progress lines ("test_result:init:...", solver summary) on stdout; they go
    # to stderr here so that stdout carries the result line only
    sys.stdout.flush()
    _REAL_STDOUT = os.dup(1)
    os.dup2(2, 1)
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from ugache_amd import hip

    hip.lib()  # the HIP library must be there: no fallback path exists
    torch.cuda.set_device(0)
    emit(run_all_hit(args) if args.workload in ALL_HIT else run_mixed(args))


if __name__ == "__main__":
    main()
