"""CPU checks of the drop-in boundary: both shared libraries load, and export every symbol their headers declare
(no compute call is made here)."""
import ctypes
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(%s\w+)\s*\(" % prefix, text))
    # function-pointer typedefs are not symbols
    names -= set(re.findall(r"\(\s*\*\s*(%s\w+)\s*\)" % prefix, text))
    return names


def test_hip_library_exports_everything_ugache_hip_h_declares():
    from ugache_amd import hip
    lib = hip.lib()
    declared = _declared("ugache_hip.h", "ugk_")
    assert len(declared) > 40
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(hip.SIGNATURES), declared ^ set(hip.SIGNATURES)
    with open(os.path.join(ROOT, "include", "ugache_hip.h")) as f:
        version = int(re.search(r"#define UGK_ABI_VERSION (\d+)", f.read()).group(1))
    assert hip.call("ugk_abi_version") == version >= 3  # the built library is the header's
    assert lib.ugk_hash_buckets_for(50_000_000, 0.7) % 8 == 0
    assert lib.ugk_hash_buckets_for(50_000_000, 0.7) >= 50_000_000 / 0.7
    assert lib.ugk_dedup_workspace_bytes(1000) >= 2048 * 8 + 1024 * 4


def test_host_library_exports_everything_coll_cache_c_api_h_declares():
    import sys
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    import collcache.common as cc
    lib = cc._basics.C_LIB_CTYPES
    declared = _declared("coll_cache_c_api.h", "coll_cache_")
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(cc.C_API), declared ^ set(cc.C_API)
    # the reference's own extern "C" names (python/collcache/common/operation.h:31-61, operation.cc:205-209)
    for name in ["coll_cache_config", "coll_cache_log_step_by_key", "coll_cache_report_step_by_key",
                 "coll_cache_report_step_average_by_key", "coll_cache_train_barrier", "coll_cache_wait_one_child",
                 "coll_cache_print_memory_usage", "coll_cache_lookup", "coll_cache_record", "coll_cache_record_init"]:
        assert name in declared


def test_host_library_has_no_hip_symbols_of_its_own():
    """host C++ reaches the GPU only through the ugk_* C-ABI"""
    import subprocess
    out = subprocess.run(["nm", "-D", "--undefined-only", os.path.join(ROOT, "ugache_amd", "libcoll_cache.so")],
                         stdout=subprocess.PIPE, text=True).stdout
    undefined = [l.split()[-1] for l in out.splitlines() if l.strip()]
    assert any(u.startswith("ugk_") for u in undefined)
    assert not [u for u in undefined if u.startswith("hip") or u.startswith("__hip")]


def test_python_surface_matches_reference_names():
    import sys
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    import collcache.common as cc
    # policy ids and profiler item ids (python/collcache/common/__init__.py:47-171)
    assert cc.kCollCacheAsymmLink == 13 and cc.kRepCache == 12 and cc.kCollFineGrain == 18
    assert cc.cache_policies["coll_cache_asymm_link"] == 13
    assert cc.kLogL1FeatureBytes == 9 and cc.kLogL1MissBytes == 13 and cc.kLogL1RemoteBytes == 14
    assert cc.kLogL2CacheCopyTime == 27
    assert cc.kLogL3CacheGetIndexTime == 46 and cc.kLogL3CacheCombineMissTime == 50
    assert cc.kLogL3CacheCombineCacheTime == 51 and cc.kLogL3CacheCombineRemoteTime == 52
    assert cc.kLogL3LabelExtractTime == 53
    assert cc.kLogEpochFeatureBytes == 13 and cc.kLogEpochMissBytes == 14
    assert cc.gpu(1) == "cuda:1" and cc.cpu() == "cpu:0"


def test_torch_surface_has_the_reference_entry_points():
    """python/collcache/torch/adapter.py:29-54 and the module-level helpers of python/collcache/common/__init__.py
    (:47-171, 173-262), by name and by parameter list"""
    import inspect
    import sys
    torch = pytest.importorskip("torch")
    del torch
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    import collcache.torch as co
    want = {
        "config": ["run_config"],
        "coll_cache_record_init": ["replica_id"],
        "coll_torch_record": ["local_id", "keys"],
        "coll_torch_create_emb_shm": ["replica_id", "n_keys", "dim", "dtype", "fname"],
        "coll_torch_init_t": ["replica_id", "dev_id", "emb", "cache_percentage"],
        "coll_torch_lookup_key_t_val_ret": ["local_id", "keys", "pad_to_8"],
        "coll_torch_test": ["local_id", "keys"],
        "log_step_by_key": ["key", "item", "val"],
        "report_step": ["key"],
        "report_step_average": ["key"],
        "wait_one_child": [],
        "print_memory_usage": [],
    }
    for name, params in want.items():
        fn = getattr(co, name, None)
        assert callable(fn), name
        got = [p for p in inspect.signature(fn).parameters]
        assert got[: len(params)] == params, (name, got)
    assert inspect.signature(co.coll_torch_lookup_key_t_val_ret).parameters["pad_to_8"].default is True
    assert inspect.signature(co.coll_torch_create_emb_shm).parameters["fname"].default == ""
    assert co.kCollCacheAsymmLink == 13


def test_c_lib_module_of_the_torch_binding():
    """`from collcache.torch import c_lib` (python/collcache/torch/adapter.py:25) gives a module with the six entry
    points PYBIND11_MODULE(c_lib, m) defines (adapter.cc:274-281), with the C++ functions' parameter order"""
    import inspect
    pytest.importorskip("torch")
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    from collcache.torch import c_lib
    import collcache.torch as co
    want = {
        "coll_torch_init": ["replica_id", "key_space_size", "dev_id", "cpu_data", "dim", "cache_percentage",
                            "use_fp16"],                                       # adapter.cc:126-128
        "coll_torch_init_t": ["replica_id", "dev_id", "emb", "cache_percentage"],  # adapter.cc:151
        "coll_torch_test": ["local_id", "keys"],                                # adapter.cc:192
        "coll_torch_record": ["local_id", "keys"],                              # adapter.cc:270
        "coll_torch_lookup_key_t_val_ret": ["local_id", "keys", "pad_to_8"],    # adapter.cc:204
        "coll_torch_create_emb_shm": ["replica_id", "n_keys", "dim", "dtype", "fname"],  # adapter.cc:239
    }
    for name, params in want.items():
        fn = getattr(c_lib, name, None)
        assert callable(fn), name
        assert [p for p in inspect.signature(fn).parameters][: len(params)] == params, name
        # the adapter's function of the same name forwards to it
        assert callable(getattr(co, name)) and getattr(co, name) is not fn


def test_compiled_c_lib_module_is_built_and_has_the_six_entry_points():
    """collcache.torch.c_lib_native: the extension module of PYBIND11_MODULE(c_lib, m) (adapter.cc:274-281) built by
    python -m ugache_amd.build, linked against libcoll_cache.so; importing it needs no GPU"""
    pytest.importorskip("torch")
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    import importlib
    native = importlib.import_module("collcache.torch.c_lib_native")
    assert native.__file__.endswith(".so")
    for name in ("coll_torch_init", "coll_torch_init_t", "coll_torch_test", "coll_torch_record",
                 "coll_torch_lookup_key_t_val_ret", "coll_torch_create_emb_shm"):
        assert callable(getattr(native, name)), name
    # pybind11 puts the C++ signature into the docstring
    doc = native.coll_torch_lookup_key_t_val_ret.__doc__
    assert doc.startswith("coll_torch_lookup_key_t_val_ret(arg0:") and "arg1: object, arg2: bool) -> object" in doc
    assert "fname: str = ''" in native.coll_torch_create_emb_shm.__doc__


def test_serving_module_has_the_tf2_bindings_entry_points():
    """collcache.torch.serving carries the names the reference's inference scripts call on collcache_tf2
    (python_tf2/collcache_tf2/collcache_tf2/core/initialize.py:33-39, 79, 129, 292; core/lookup_layer.py:22;
    core/sparse_lookup_layer.py:27)"""
    torch = pytest.importorskip("torch")
    sys.path.insert(0, os.path.join(ROOT, "ugache_amd"))
    import inspect
    import collcache.torch.serving as hps
    want = ["Config", "Init", "Report", "NopDep", "wait_one_child", "SetStepProfileValue", "LookupLayer",
            "SparseLookupLayer"]
    for name in want:
        assert hasattr(hps, name), name
    assert list(inspect.signature(hps.LookupLayer.__init__).parameters)[1:5] == [
        "model_name", "table_id", "emb_vec_size", "emb_vec_dtype"]
    assert list(inspect.signature(hps.SparseLookupLayer.forward).parameters)[1:6] == [
        "sp_ids", "sp_weights", "name", "combiner", "max_norm"]
    assert issubclass(hps.LookupLayer, torch.nn.Module) and issubclass(hps.SparseLookupLayer, torch.nn.Module)
