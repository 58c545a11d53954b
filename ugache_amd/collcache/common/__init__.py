"""Counterpart of python/collcache/common/__init__.py of the reference: policy ids, profiler item ids and the
ctypes front (`_basics`) of the extern "C" shim.  The shared library is loaded at import time, as there; a missing
library is an ImportError, never a silent fallback."""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
LIB_PATH = os.path.join(_PKG_DIR, "libcoll_cache.so")

# python/collcache/common/__init__.py:47-65
kCacheByDegree = 0
kCacheByHeuristic = 1
kCacheByPreSample = 2
kCacheByDegreeHop = 3
kCacheByPreSampleStatic = 4
kCacheByFakeOptimal = 5
kDynamicCache = 6
kCacheByRandom = 7
kCollCache = 8
kCollCacheIntuitive = 9
kPartitionCache = 10
kPartRepCache = 11
kRepCache = 12
kCollCacheAsymmLink = 13
kCliquePart = 14
kCliquePartByDegree = 15
kSOK = 16
kHPS = 17
kCollFineGrain = 18


def cpu(device_id=0):
    return 'cpu:{:}'.format(device_id)


def gpu(device_id=0):
    return 'cuda:{:}'.format(device_id)


cache_policies = {
    'degree': kCacheByDegree,
    'heuristic': kCacheByHeuristic,
    'pre_sample': kCacheByPreSample,
    'degree_hop': kCacheByDegreeHop,
    'presample_static': kCacheByPreSampleStatic,
    'fake_optimal': kCacheByFakeOptimal,
    'dynamic_cache': kDynamicCache,
    'random': kCacheByRandom,
    'coll_cache': kCollCache,
    'coll_intuitive': kCollCacheIntuitive,
    'partition': kPartitionCache,
    'part_rep': kPartRepCache,
    'rep': kRepCache,
    'coll_cache_asymm_link': kCollCacheAsymmLink,
    'coll_fine_grain': kCollFineGrain,
    'clique_part': kCliquePart,
    'clique_part_by_degree': kCliquePartByDegree,
}

# step items, in the order of LogStepItem (coll_cache_lib/profiler.h)
_STEP_ITEMS = [
    "kLogL1NumSample", "kLogL1NumNode", "kLogL1SampleTotalTime", "kLogL1SampleTime", "kLogL1SendTime",
    "kLogL1RecvTime", "kLogL1CopyTime", "kLogL1ConvertTime", "kLogL1TrainTime", "kLogL1FeatureBytes",
    "kLogL1LabelBytes", "kLogL1IdBytes", "kLogL1GraphBytes", "kLogL1MissBytes", "kLogL1RemoteBytes",
    "kLogL1PrefetchAdvanced", "kLogL1GetNeighbourTime", "kLogL1SamplerId",
    "kLogL2ShuffleTime", "kLogL2LastLayerTime", "kLogL2LastLayerSize", "kLogL2CoreSampleTime", "kLogL2IdRemapTime",
    "kLogL2GraphCopyTime", "kLogL2IdCopyTime", "kLogL2ExtractTime", "kLogL2FeatCopyTime", "kLogL2CacheCopyTime",
    "kLogL3KHopSampleCooTime", "kLogL3KHopSampleKernelTime", "kLogL3KHopSampleSortCooTime",
    "kLogL3KHopSampleCountEdgeTime", "kLogL3KHopSampleCompactEdgesTime", "kLogL3RandomWalkSampleCooTime",
    "kLogL3RandomWalkTopKTime", "kLogL3RandomWalkTopKStep1Time", "kLogL3RandomWalkTopKStep2Time",
    "kLogL3RandomWalkTopKStep3Time", "kLogL3RandomWalkTopKStep4Time", "kLogL3RandomWalkTopKStep5Time",
    "kLogL3RandomWalkTopKStep6Time", "kLogL3RandomWalkTopKStep7Time", "kLogL3RemapFillUniqueTime",
    "kLogL3RemapPopulateTime", "kLogL3RemapMapNodeTime", "kLogL3RemapMapEdgeTime", "kLogL3CacheGetIndexTime",
    "KLogL3CacheCopyIndexTime", "kLogL3CacheExtractMissTime", "kLogL3CacheCopyMissTime", "kLogL3CacheCombineMissTime",
    "kLogL3CacheCombineCacheTime", "kLogL3CacheCombineRemoteTime", "kLogL3LabelExtractTime",
]
for _i, _name in enumerate(_STEP_ITEMS):
    globals()[_name] = _i

_EPOCH_ITEMS = [
    "kLogEpochSampleTime", "KLogEpochSampleGetCacheMissIndexTime", "kLogEpochSampleSendTime",
    "kLogEpochSampleTotalTime", "kLogEpochCoreSampleTime", "kLogEpochSampleCooTime", "kLogEpochIdRemapTime",
    "kLogEpochShuffleTime", "kLogEpochSampleKernelTime", "kLogEpochCopyTime", "kLogEpochConvertTime",
    "kLogEpochTrainTime", "kLogEpochTotalTime", "kLogEpochFeatureBytes", "kLogEpochMissBytes",
]
for _i, _name in enumerate(_EPOCH_ITEMS):
    globals()[_name] = _i

ALLOC_FN = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p)
RELEASE_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p)

# every symbol include/coll_cache_c_api.h declares: name -> (restype, argtypes)
C_API = {
    "coll_cache_config": (None, [ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_char_p), ctypes.c_size_t]),
    "coll_cache_log_step_by_key": (None, [ctypes.c_uint64, ctypes.c_int, ctypes.c_double]),
    "coll_cache_report_step_by_key": (None, [ctypes.c_uint64]),
    "coll_cache_report_step_average_by_key": (None, [ctypes.c_uint64]),
    "coll_cache_train_barrier": (None, []),
    "coll_cache_wait_one_child": (ctypes.c_int, []),
    "coll_cache_print_memory_usage": (None, []),
    "coll_cache_lookup": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_record": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]),
    "coll_cache_record_init": (None, [ctypes.c_int]),
    "coll_cache_init_c": (None, [ctypes.c_int, ctypes.c_size_t, ALLOC_FN, RELEASE_FN, ctypes.c_void_p,
                                 ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_double, ctypes.c_void_p]),
    "coll_cache_init_ranked_c": (None, [ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ALLOC_FN,
                                        RELEASE_FN, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t,
                                        ctypes.c_double, ctypes.c_void_p]),
    "coll_cache_build_all_c": (None, [ALLOC_FN, RELEASE_FN, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                      ctypes.c_size_t, ctypes.c_double, ctypes.c_void_p]),
    "coll_cache_lookup_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                     ctypes.c_void_p]),
    "coll_cache_record_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]),
    "coll_cache_set_key_map": (None, [ctypes.c_uint64, ctypes.c_int]),
    "coll_cache_refresh": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int]),
    "coll_cache_alloc_host_table": (ctypes.c_void_p, [ctypes.c_size_t]),
    "coll_cache_free_host_table": (None, [ctypes.c_void_p]),
    "coll_cache_max_num_keys": (ctypes.c_size_t, []),
    "coll_cache_set_max_num_keys": (None, [ctypes.c_size_t]),
    "coll_cache_last_group_offset": (None, [ctypes.c_int, ctypes.POINTER(ctypes.c_uint32 * 3)]),
    "coll_cache_get_info": (None, [ctypes.c_int, ctypes.POINTER(ctypes.c_uint64 * 8)]),
    "coll_cache_get_cached_keys": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]),
    "coll_cache_rows_from_stage": (ctypes.c_uint64, [ctypes.c_int]),
    "coll_cache_get_step_value": (ctypes.c_double, [ctypes.c_uint64, ctypes.c_int]),
    "coll_cache_rank_hotness": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "coll_cache_place_ranked": (ctypes.c_uint32, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_double,
                                                 ctypes.c_void_p]),
    "coll_cache_place_recorded": (ctypes.c_uint32, [ctypes.c_int, ctypes.c_uint32, ctypes.c_double, ctypes.c_void_p]),
    "coll_cache_lookup_unique": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                                   ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_lookup_unique_i64": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                                       ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_lookup_pooled": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                        ctypes.c_void_p]),
    "coll_cache_lookup_pooled_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_forward_pooled_async": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                              ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_forward_pooled_async_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                              ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_lookup_pooled_async": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                              ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_lookup_pooled_async_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                  ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                                  ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_set_pooled_max_norm": (None, [ctypes.c_int, ctypes.c_float]),
    "coll_cache_segment_offsets": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t,
                                          ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_forward_pooled": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.c_void_p]),
    "coll_cache_forward_pooled_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_forward_async": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                       ctypes.c_void_p]),
    "coll_cache_forward_async_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                       ctypes.c_void_p]),
    "coll_cache_lookup_async": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                       ctypes.c_void_p]),
    "coll_cache_lookup_async_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                           ctypes.c_void_p]),
    "coll_cache_lookup_wait": (None, [ctypes.c_int, ctypes.c_void_p]),
    "coll_cache_forward_config": (None, [ctypes.c_int, ctypes.c_uint64, ctypes.c_double, ctypes.c_int]),
    "coll_cache_forward": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]),
    "coll_cache_forward_i64": (None, [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                      ctypes.c_void_p]),
    "coll_cache_forward_refresh_ongoing": (ctypes.c_int, []),
    "coll_cache_forward_join": (ctypes.c_uint64, []),
    "coll_cache_shutdown": (None, []),
}

# DataType codes of coll_cache_lib/common.h
kF32, kF64, kF16, kU8, kI32, kI8, kI64, kF64_2, kF64_4 = range(9)


class CollCacheBasics(object):
    def __init__(self, lib_path=LIB_PATH):
        if not os.path.exists(lib_path):
            raise ImportError("%s is missing: build it with `python -m ugache_amd.build`" % lib_path)
        self.C_LIB_CTYPES = ctypes.CDLL(lib_path, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in C_API.items():
            fn = getattr(self.C_LIB_CTYPES, name)
            fn.restype = res
            fn.argtypes = args

    def config(self, run_config: dict):
        num_configs_items = len(run_config)
        config_keys = [str.encode(str(key)) for key in run_config.keys()]
        config_values = []
        for value in run_config.values():
            if isinstance(value, list):
                config_values.append(str.encode(' '.join([str(v) for v in value])))
            else:
                config_values.append(str.encode(str(value)))
        return self.C_LIB_CTYPES.coll_cache_config(
            (ctypes.c_char_p * num_configs_items)(*config_keys),
            (ctypes.c_char_p * num_configs_items)(*config_values),
            ctypes.c_size_t(num_configs_items))

    def log_step_by_key(self, key, item, val):
        return self.C_LIB_CTYPES.coll_cache_log_step_by_key(key, item, val)

    def report_step(self, key):
        return self.C_LIB_CTYPES.coll_cache_report_step_by_key(key)

    def report_step_average(self, key):
        return self.C_LIB_CTYPES.coll_cache_report_step_average_by_key(key)

    def train_barrier(self):
        return self.C_LIB_CTYPES.coll_cache_train_barrier()

    def wait_one_child(self):
        return self.C_LIB_CTYPES.coll_cache_wait_one_child()

    def print_memory_usage(self):
        return self.C_LIB_CTYPES.coll_cache_print_memory_usage()

    def coll_cache_record_init(self, replica_id):
        self.C_LIB_CTYPES.coll_cache_record_init(replica_id)

    # ---- beyond the reference's _basics: refresh, introspection, teardown ----
    def refresh(self, replica_id, stream=None, foreground=False):
        self.C_LIB_CTYPES.coll_cache_refresh(replica_id, stream, 1 if foreground else 0)

    def last_group_offset(self, replica_id=0):
        out = (ctypes.c_uint32 * 3)()
        self.C_LIB_CTYPES.coll_cache_last_group_offset(replica_id, ctypes.byref(out))
        return list(out)

    def info(self, replica_id=0):
        out = (ctypes.c_uint64 * 8)()
        self.C_LIB_CTYPES.coll_cache_get_info(replica_id, ctypes.byref(out))
        names = ["capacity_rows", "cached_rows", "table_kind", "row_bytes", "key_space", "lookups", "free_slots",
                 "table_rebuilds"]
        return dict(zip(names, list(out)))

    def step_value(self, key, item):
        return self.C_LIB_CTYPES.coll_cache_get_step_value(key, item)

    def set_key_map(self, mul, bits):
        self.C_LIB_CTYPES.coll_cache_set_key_map(mul, bits)

    def shutdown(self):
        self.C_LIB_CTYPES.coll_cache_shutdown()


_basics = CollCacheBasics()
