"""Build recipe for the native libraries of this package (gfx950 only).

  libugache_hip.so  — hand-written HIP kernels behind the C-ABI of include/ugache_hip.h   (hipcc)
  libcoll_cache.so  — host C++ mirror of the reference's coll_cache_lib facade + extern "C" shim (g++),
                      linked against libugache_hip.so; it never includes a HIP header.

  collcache/torch/c_lib_native.*.so — the compiled form of collcache.torch.c_lib (pybind11, g++), linked against
                      libcoll_cache.so.

All are built in-tree.  `python -m ugache_amd.build` rebuilds everything.
"""
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "coll_cache_lib")
INCLUDE = os.path.join(ROOT, "include")

HIP_LIB = os.path.join(PKG, "libugache_hip.so")
HOST_LIB = os.path.join(PKG, "libcoll_cache.so")

HIP_SOURCES = ["ugk_runtime.hip", "ugk_gather.hip", "ugk_table.hip", "ugk_partition.hip", "ugk_pool.hip",
               "ugk_hotness.hip", "ugk_refresh.hip"]
OBJ_DIR = os.path.join(PKG, "_build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed FP32 instructions are kept out of every code object of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd, cwd=None):
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _compile_all(jobs):
    """jobs: (command, object file) pairs, run side by side (the long ones first); -> the object files"""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, max(len(jobs), 1))) as pool:
        outs = list(pool.map(lambda j: _run(j[0]), jobs))
    return [j[1] for j in jobs], "\n".join(o for o in outs if o.strip())


def build_hip(verbose=False):
    base = [hipcc_path()] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC]
    jobs = []
    for s in HIP_SOURCES:
        obj = os.path.join(OBJ_DIR, s + ".o")
        jobs.append((base + ["-c", os.path.join(CSRC, s), "-o", obj], obj))
    objs, out = _compile_all(jobs)
    out += _run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", HIP_LIB])
    if verbose and out.strip():
        print(out)
    return HIP_LIB


def host_sources():
    if not os.path.isdir(HOST):
        return []
    return sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cc"))


def build_host(verbose=False):
    srcs = host_sources()
    if not srcs:
        return None
    base = ["g++", "-O2", "-g", "-std=c++17", "-fPIC", "-fopenmp", "-pthread", "-Wall", "-Wextra",
            "-Wno-unused-parameter", "-I", INCLUDE, "-I", PKG]
    jobs = []
    for s in srcs:
        obj = os.path.join(OBJ_DIR, os.path.basename(s) + ".o")
        jobs.append((base + ["-c", s, "-o", obj], obj))
    objs, out = _compile_all(jobs)
    out += _run(["g++", "-shared", "-fopenmp", "-pthread"] + objs +
                ["-o", HOST_LIB, "-L", PKG, "-lugache_hip", "-Wl,-rpath,$ORIGIN", "-Wl,--no-undefined"])
    if verbose and out.strip():
        print(out)
    return HOST_LIB


def native_c_lib_path():
    import sysconfig
    return os.path.join(PKG, "collcache", "torch", "c_lib_native" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_native_c_lib(verbose=False):
    """the pybind11 extension module collcache.torch.c_lib_native over libcoll_cache.so"""
    import sysconfig

    import pybind11
    src = os.path.join(PKG, "collcache", "torch", "c_lib_native.cc")
    out = _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
                "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"], "-I", INCLUDE, src,
                "-o", native_c_lib_path(), "-L", PKG, "-lcoll_cache", "-Wl,-rpath,$ORIGIN/../.."])
    if verbose and out.strip():
        print(out)
    return native_c_lib_path()


def build_all(verbose=False):
    build_hip(verbose)
    build_host(verbose)
    build_native_c_lib(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built:", HIP_LIB, HOST_LIB if os.path.exists(HOST_LIB) else "(no host lib yet)", native_c_lib_path())
