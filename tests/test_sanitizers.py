"""The host library under AddressSanitizer + UBSan and under ThreadSanitizer, on the CPU.

tests/sanitizer/ holds a plain CPU model of the kernel layer's C-ABI (test infrastructure, never part of the package)
and a driver that runs build -> lookups || background refreshes -> stream-ordered lookups || refresh -> serving loop ->
shutdown through the library's C boundary.  Both are compiled together with the library's own sources into one
executable per sanitizer; a sanitizer report, a wrong row or a refresh that never ran fails the test.
Stands in for the hand-rolled syncers of the reference (coll_cache_lib/cache_context.h:78-236), whose replacements
here (the in-flight counts, the remembered streams, the table swap of a rebuild) are what these runs exercise.
"""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sanitizer")
BUILD = os.path.join(HERE, "_build")


@pytest.fixture(scope="module")
def drivers():
    proc = subprocess.run(["make", "-j8", "-C", HERE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-4000:]
    return {"asan": os.path.join(BUILD, "driver_asan"), "tsan": os.path.join(BUILD, "driver_tsan")}


def _run(exe, table, refresh, steps):
    env = dict(os.environ)
    env["COLL_HASH_REBUILD_FRAC"] = "0.02"  # a few hundred evictions already rebuild the open-addressing table
    env["COLL_MISS_STAGE_ROWS"] = "4096"  # lookups file the rows they fetch from the host, foreground refreshes read them
    if table.startswith("HASH"):  # refreshes on the device keep cached rows that tie (the second placement path)
        env["COLL_GPU_REFRESH_STABLE"] = "1"
    else:  # the device-side counters start from the build's ranking, and the background copy is paced by a rate
        env["COLL_GPU_RECORD_SEED"] = "1"
        env["COLL_REFRESH_RATE_GBPS"] = "0.5"
        env["COLL_RECORD_INLINE_BYTES"] = "0"  # every recorded prefix goes through the recorder's thread
    if table == "HASH16" and refresh == "host":  # build and refresh through the host's key -> block array and key lists
        env["COLL_DEVICE_KEY_LIST"] = "0"
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    env["TSAN_OPTIONS"] = "halt_on_error=0:second_deadlock_stack=1"
    env.pop("LD_PRELOAD", None)  # the sanitizer runtimes insist on coming first
    proc = subprocess.run([exe, table, refresh, str(steps)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, env=env, timeout=600)
    return proc.returncode, proc.stdout


@pytest.mark.parametrize("refresh", ["host", "device"])
@pytest.mark.parametrize("table", ["FLAT", "HASH", "HASH16"])
def test_host_library_under_asan_and_ubsan(drivers, table, refresh):
    rc, out = _run(drivers["asan"], table, refresh, 150)
    assert "AddressSanitizer" not in out and "runtime error" not in out and "LeakSanitizer" not in out, out[-6000:]
    assert rc == 0 and out.rstrip().endswith("OK"), out[-3000:]
    if table.startswith("HASH"):  # the table swap of a rebuild ran beside the lookups
        rebuilds = [int(l.split(" table rebuilds")[0].split()[-1]) for l in out.splitlines() if " table rebuilds" in l]
        assert rebuilds and max(rebuilds) > 0, out[-3000:]


@pytest.mark.parametrize("refresh", ["host", "device"])
@pytest.mark.parametrize("table", ["FLAT", "HASH", "HASH16"])
def test_host_library_under_tsan(drivers, table, refresh):
    rc, out = _run(drivers["tsan"], table, refresh, 30)
    assert "ThreadSanitizer" not in out, out[-8000:]
    assert rc == 0 and out.rstrip().endswith("OK"), out[-3000:]
