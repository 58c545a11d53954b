#!/usr/bin/env python3
"""Throughput of the embedding-extraction hot path on one MI355X.

A step is one blocking `coll_cache_lookup` of one key batch through the drop-in C boundary (libcoll_cache.so ->
libugache_hip.so), keys and table already resident in HBM.  Workload = the all-hit configuration: a 10M x 128 fp32
table (5.12 GB) fully cached, 262,144 uniform uint32 keys per batch, duplicates allowed.

Prints ONE JSON line with keys/s (whole job), the roofline of the dominant kernel (gather_kernel: algorithmic bytes
per launch / its average duration, measured live with HIP events on the kernel's stream inside the timed region)
and the CPU baseline (the oracle's OpenMP gather on the host cores, bounded sample of the same batches).
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
MEASURED_TRAFFIC_BYTES = {"c2_all_hit_10Mx128xfp32_262144_u32_uniform": 270_550_000}

WORKLOADS = {
    # name: (rows, dim, keys per batch, key dtype)
    "c2_all_hit_10Mx128xfp32_262144_u32_uniform": (10_000_000, 128, 262_144, "u32"),
    "tiny_all_hit_100Kx128xfp32_8192_u32_uniform": (100_000, 128, 8_192, "u32"),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2_all_hit_10Mx128xfp32_262144_u32_uniform", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline budget")
    ap.add_argument("--pool", type=int, default=64, help="distinct key batches cycled through the steps")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run 5 plain device copies of 1 GiB (ugk_copy_rows) so a counter run has a kernel of "
                         "known traffic next to the gather")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the extraction path of ONE GPU (no collectives, no peer source); "
                 "--gpus %d is not supported, use --gpus 1" % args.gpus)

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from ugache_amd import hip

    hip.lib()  # the HIP library must be there: no fallback path exists
    import collcache.torch as co
    from collcache.common import _basics, kLogL3CacheCombineCacheTime
    from oracle_lib import Oracle

    rows, dim, n_keys, _ = WORKLOADS[args.workload]
    row_bytes = dim * 4
    K, W = args.steps, args.warmup
    dev = torch.device("cuda:0")
    torch.cuda.set_device(0)

    # ---- synthetic table, filled on the device from a seed, mirrored into the pinned host table ---------------
    co.config({"cache_percentage": 1.0, "_cache_policy": co.kCollCacheAsymmLink, "num_device": 1,
               "num_global_step_per_epoch": K + W, "num_epoch": 1, "num_total_item": rows, "omp_thread_num": 16})
    co.coll_cache_record_init(0)
    emb = co.coll_torch_create_emb_shm(0, rows, dim, torch.float32)
    g = torch.Generator(device=dev).manual_seed(1)
    chunk = 1_000_000
    for r0 in range(0, rows, chunk):
        r1 = min(rows, r0 + chunk)
        emb[r0:r1].copy_(torch.randn((r1 - r0, dim), generator=g, device=dev, dtype=torch.float32))
    torch.cuda.synchronize()
    co.coll_torch_init_t(0, 0, emb, 1.0)  # 100 % cache: the table is copied into HBM, keys index it directly

    # ---- key batches (uniform with replacement, seed 4), resident in HBM ---------------------------------------
    gk = torch.Generator(device=dev).manual_seed(4)
    pool = max(1, args.pool)
    keys_pool = torch.randint(0, rows, (pool, n_keys), generator=gk, device=dev, dtype=torch.int32)
    out = torch.empty((n_keys, dim), dtype=torch.float32, device=dev)
    C = _basics.C_LIB_CTYPES
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        C.coll_cache_lookup(0, keys_pool[i % pool].data_ptr(), n_keys, out.data_ptr(), stream)

    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(W, W + K):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / K * 1e3
    keys_per_s = n_keys * K / elapsed

    if args.calibrate:
        cal_src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        cal_dst = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        for _ in range(5):
            hip.call("ugk_copy_rows", cal_dst.data_ptr(), cal_src.data_ptr(), 1 << 30, stream)
        torch.cuda.synchronize()
        del cal_src, cal_dst

    # ---- parity of the last timed batch, byte for byte against the oracle -------------------------------------
    orc = Oracle()
    table_np = emb.numpy()
    last_keys = keys_pool[(W + K - 1) % pool].cpu().numpy().view(np.uint32)
    want = orc.gather(table_np, last_keys, omp=True)
    if out.cpu().numpy().tobytes() != want.tobytes():
        sys.exit("bench.py: GPU output differs from the CPU oracle — no numbers reported")

    # ---- dominant kernel: per-launch duration from the HIP events the library records around the gather on its
    #      stream (logged per step as kLogL3CacheCombineCacheTime), averaged over the K timed steps --------------
    kernel_s = [_basics.step_value(s, kLogL3CacheCombineCacheTime) for s in range(W, W + K)]
    kernel_avg_s = float(np.mean(kernel_s))
    alg_bytes = n_keys * (2 * row_bytes + 4)  # row read + row written + key read, per key
    achieved = alg_bytes / kernel_avg_s / 1e9

    # ---- CPU baseline: the oracle's OpenMP gather over the same batches, bounded ------------------------------
    keys_host = keys_pool.cpu().numpy().view(np.uint32)
    cpu_out = np.empty((n_keys, dim), np.float32)
    lib = orc.lib
    cores = lib.orc_omp_threads()

    def cpu_step(i):
        rc = lib.orc_gather_u32_omp(table_np.ctypes.data, rows, keys_host[i % pool], n_keys, cpu_out.ctypes.data,
                                    row_bytes)
        assert rc == 0

    cpu_step(0)
    t0 = time.perf_counter()
    n_cpu = 0
    while True:
        cpu_step(n_cpu)
        n_cpu += 1
        if time.perf_counter() - t0 >= args.cpu_seconds or n_cpu >= 100000:
            break
    cpu_elapsed = time.perf_counter() - t0
    cpu_keys_per_s = n_keys * n_cpu / cpu_elapsed

    info = hip.device_info(0)
    result = {
        "metric": "embedding keys/sec + effective extraction GB/s (% HBM / host-link roofline), 1 GPU",
        "value": keys_per_s,
        "unit": "keys/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": args.workload, "table_rows": rows, "row_bytes": row_bytes, "keys_per_batch": n_keys,
                   "key_dtype": "uint32", "cache_percentage": 1.0, "entry_point": "coll_cache_lookup",
                   "distinct_key_batches": pool, "seeds": {"table": 1, "keys": 4}},
        "effective_extraction_GBps": n_keys * row_bytes / (elapsed / K) / 1e9,
        "parity": "bit-exact vs CPU oracle (last timed batch)",
        "device": info["name"] + " " + info["arch"],
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload), "kernel": "gather_kernel<u32x4,32,2,DirectU32>",
                     "algorithmic_bytes_per_launch": alg_bytes, "avg_kernel_us": kernel_avg_s * 1e6,
                     "keys_per_s_kernel_only": n_keys / kernel_avg_s},
        "cpu_baseline": {"value": cpu_keys_per_s, "unit": "keys/s", "cores": cores, "kind": "port",
                         "sample": "%d batches of %d keys from the same pool, %.1f s, OpenMP gather over keys"
                                   % (n_cpu, n_keys, cpu_elapsed),
                         "effective_GBps": n_keys * row_bytes * n_cpu / cpu_elapsed / 1e9},
        "gpu_over_cpu": keys_per_s / cpu_keys_per_s,
    }
    co.coll_torch_shutdown()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
