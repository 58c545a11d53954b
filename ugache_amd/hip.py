"""ctypes binding of include/ugache_hip.h (libugache_hip.so).

There is no fallback: if the library is missing or a call fails, an exception is raised.  Device buffers are
passed as integer addresses (e.g. ``tensor.data_ptr()``); torch is only used by callers for memory and streams.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libugache_hip.so")

ST_KEY_OUT_OF_RANGE = 0x1
ST_TABLE_FULL = 0x2
ST_DUP_KEY = 0x4
ST_EVICT_ABSENT = 0x8
ST_BAD_SEGMENT = 0x10
ST_PLACE_PROMISE = 0x20
ELEM_BF16 = 0x102

LOC_LOCAL = 0
LOC_HOST = 1
EMPTY_U32 = 0xFFFFFFFF
HINT_UNKNOWN = 0xFFFFFFFF

TABLE_NONE = 0
TABLE_FLAT = 1
TABLE_HASH = 2
TABLE_HASH32 = 3


class UgkError(RuntimeError):
    pass


class Table(C.Structure):
    """ugk_table_t"""
    _fields_ = [("kind", C.c_int32), ("reserved", C.c_int32), ("table", C.c_void_p), ("size", C.c_uint64),
                ("fb_mul", C.c_uint64), ("fb_mask", C.c_uint64)]


class Stage(C.Structure):
    """ugk_stage_t"""
    _fields_ = [("rows_dev", C.c_void_p), ("owner_dev", C.c_void_p), ("mask", C.c_uint64), ("epoch", C.c_uint32),
                ("reserved", C.c_uint32)]


class DeviceInfo(C.Structure):
    """ugk_device_info_t"""
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("wavefront_size", C.c_int32), ("total_mem", C.c_uint64), ("lds_per_block", C.c_uint64)]


_vp, _sz, _u32, _u64, _i = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int

# name -> argtypes (restype is int unless listed in _RESTYPES)
SIGNATURES = {
    "ugk_abi_version": [],
    "ugk_device_count": [C.POINTER(_i)],
    "ugk_set_device": [_i],
    "ugk_get_device_info": [_i, C.POINTER(DeviceInfo)],
    "ugk_mem_info": [C.POINTER(_sz), C.POINTER(_sz)],
    "ugk_malloc": [C.POINTER(_vp), _sz],
    "ugk_free": [_vp],
    "ugk_host_malloc": [C.POINTER(_vp), _sz],
    "ugk_host_free": [_vp],
    "ugk_pointer_kind": [_vp, C.POINTER(_i)],
    "ugk_stream_create": [C.POINTER(_vp)],
    "ugk_stream_create_cu_masked": [C.POINTER(_vp), _i],
    "ugk_stream_destroy": [_vp],
    "ugk_stream_sync": [_vp],
    "ugk_stream_is_capturing": [_vp, _vp],
    "ugk_stream_sync_ticket": [_vp, _vp, _u32, C.c_uint],
    "ugk_words_to_host_ticket": [_vp, C.c_uint, _vp, C.c_uint, _vp, _u32, C.c_uint, _vp],
    "ugk_preload_kernels": [],
    "ugk_device_sync": [],
    "ugk_event_create": [C.POINTER(_vp)],
    "ugk_event_destroy": [_vp],
    "ugk_event_record": [_vp, _vp],
    "ugk_event_sync": [_vp],
    "ugk_event_query": [_vp, _vp],
    "ugk_stream_wait_event": [_vp, _vp],
    "ugk_event_elapsed_ms": [_vp, _vp, C.POINTER(C.c_float)],
    "ugk_memcpy_async": [_vp, _vp, _sz, _vp],
    "ugk_fill_u32": [_vp, _u32, _sz, _vp],
    "ugk_arange_u32": [_vp, _u32, _sz, _vp],
    "ugk_copy_rows": [_vp, _vp, _sz, _vp],
    "ugk_set_output_hint": [C.c_int],
    "ugk_gather_direct_u32": [_vp, _u64, _vp, _sz, _vp, _sz, C.c_uint, _vp, _vp, _vp],
    "ugk_gather_direct_i64": [_vp, _u64, _vp, _sz, _vp, _sz, C.c_uint, _vp, _vp, _vp],
    "ugk_gather_scatter_u32": [_vp, _u64, _vp, _vp, _sz, _vp, _u64, _sz, C.c_uint, _vp, _vp, _vp],
    "ugk_gather_scatter_i64": [_vp, _u64, _vp, _vp, _sz, _vp, _u64, _sz, C.c_uint, _vp, _vp, _vp],
    "ugk_replicate_rows": [_vp, _sz, _vp, _vp, _sz, _vp],
    "ugk_gather_group": [_vp, _u64, _vp, _vp, _u32, _sz, _vp, _u64, _sz, C.c_uint, _vp, _vp, _vp],
    "ugk_gather_idx": [_vp, _u64, _vp, _sz, _vp, _sz, C.c_uint, _vp, _vp],
    "ugk_hash_buckets_for": [_sz, C.c_double],
    "ugk_hash_init": [_vp, _sz, _vp],
    "ugk_hash32_entries_for": [_sz, C.c_double],
    "ugk_table_init": [Table, _vp],
    "ugk_table_census": [Table, _vp, _vp],
    "ugk_table_insert_u32": [Table, _vp, _vp, _u32, _u32, _sz, _vp, _vp],
    "ugk_table_insert_i64": [Table, _vp, _vp, _u32, _u32, _sz, _vp, _vp],
    "ugk_table_evict_u32": [Table, _vp, _sz, _vp, _vp],
    "ugk_table_evict_i64": [Table, _vp, _sz, _vp, _vp],
    "ugk_table_evict_release_u32": [Table, _vp, _sz, _vp, _u64, _vp, _vp],
    "ugk_table_evict_release_i64": [Table, _vp, _sz, _vp, _u64, _vp, _vp],
    "ugk_table_lookup_u32": [Table, _vp, _sz, _u32, _vp, _vp, _vp],
    "ugk_table_lookup_i64": [Table, _vp, _sz, _u32, _vp, _vp, _vp],
    "ugk_hash_census": [_vp, _sz, _vp, _vp],
    "ugk_classify_u32": [Table, _vp, _sz, _u64, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_classify_i64": [Table, _vp, _sz, _u64, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_nonlocal_flags_u32": [Table, _vp, _sz, _vp, _vp],
    "ugk_nonlocal_flags_i64": [Table, _vp, _sz, _vp, _vp],
    "ugk_select_keys_u32": [_vp, _vp, _sz, _vp, _vp],
    "ugk_select_keys_i64": [_vp, _vp, _sz, _vp, _vp],
    "ugk_extract_mix_max_groups": [],
    "ugk_extract_mix_u32": [Table, _vp, _sz, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp, _vp, _vp, _u32, _vp],
    "ugk_extract_mix_i64": [Table, _vp, _sz, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp, _vp, _vp, _u32, _vp],
    "ugk_segment_offsets_i64": [_vp, _sz, _sz, _vp, _vp, _vp, _vp],
    "ugk_extract_pool_u32": [Table, _vp, _vp, _vp, _sz, _u64, C.c_int, C.c_int, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp,
                             _vp, _vp, _vp],
    "ugk_extract_pool_i64": [Table, _vp, _vp, _vp, _sz, _u64, C.c_int, C.c_int, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp,
                             _vp, _vp, _vp],
    "ugk_extract_pool_clip_u32": [Table, _vp, _vp, _vp, _sz, _u64, C.c_int, C.c_int, C.c_float, _vp, _u64, _vp, _u64,
                                  _vp, _sz, _vp, _vp, _vp, _vp, _vp],
    "ugk_extract_pool_clip_i64": [Table, _vp, _vp, _vp, _sz, _u64, C.c_int, C.c_int, C.c_float, _vp, _u64, _vp, _u64,
                                  _vp, _sz, _vp, _vp, _vp, _vp, _vp],
    "ugk_extract_mix_staged_u32": [Table, _vp, _sz, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp, _vp, _vp, _u32, Stage, _vp],
    "ugk_extract_mix_staged_i64": [Table, _vp, _sz, _vp, _u64, _vp, _u64, _vp, _sz, _vp, _vp, _vp, _vp, _u32, Stage, _vp],
    "ugk_gather_scatter_staged_u32": [_vp, _u64, _vp, _vp, _sz, _vp, _u64, _sz, Stage, C.c_uint, _vp, _vp, _vp, _vp,
                                      _vp, _vp, _vp],
    "ugk_dedup_workspace_bytes": [_sz],
    "ugk_dedup_u32": [_vp, _sz, _vp, _sz, _u32, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_dedup_i64": [_vp, _sz, _vp, _sz, _u32, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_dedup_static": [_vp, _u32, _sz, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_record_u32": [_vp, _sz, _u64, _u64, _vp, _u64, _vp, _vp, _vp, _vp],
    "ugk_record_i64": [_vp, _sz, _u64, _u64, _vp, _u64, _vp, _vp, _vp, _vp],
    "ugk_record_drain": [_vp, _u64, _u64, _vp, _vp, _u32, _vp, _vp, _vp],
    "ugk_rank_workspace_bytes": [],
    "ugk_record_restore": [_vp, _sz, _vp, _u64, _vp, _vp, _vp],
    "ugk_rank_place": [_vp, _u64, _u64, _vp, _vp, _vp, _vp, C.c_int, _vp],
    "ugk_rank_place_keep": [_vp, _u64, _u64, _vp, _vp, _vp, _vp, _vp, C.c_int, _vp],
    "ugk_rank_place_observed": [_vp, _u64, _u64, _vp, _vp, _vp, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp],
    "ugk_rank_threshold": [_vp, _vp, _vp],
    "ugk_bitmap_workspace_bytes": [],
    "ugk_bitmap_count": [_vp, _vp, C.c_int, _u64, _vp, _vp, _vp],
    "ugk_bitmap_emit": [_vp, _vp, C.c_int, _u64, _vp, _vp, _u64, _vp],
    "ugk_bitmap_count_diff": [_vp, _vp, _u64, _vp, _vp, _vp, _vp],
    "ugk_bitmap_emit_diff": [_vp, _vp, _u64, _vp, _vp, _vp, _u64, _vp, _u64, _vp],
    "ugk_bitmap_update": [_vp, _u64, _vp, _sz, C.c_int, _vp, _vp],
    "ugk_bitmap_set_through": [_vp, _u64, _vp, _vp, _vp],
    "ugk_rows_to_keys": [_vp, _sz, _u64, _u64, _vp, _vp],
    "ugk_last_error": [],
}
_RESTYPES = {"ugk_extract_mix_max_groups": C.c_uint, "ugk_hash_buckets_for": _sz, "ugk_hash32_entries_for": _sz, "ugk_dedup_workspace_bytes": _sz, "ugk_rank_workspace_bytes": _sz,
             "ugk_bitmap_workspace_bytes": _sz, "ugk_last_error": C.c_char_p}
_NO_CHECK = set(_RESTYPES) | {"ugk_abi_version"}

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built (``python -m ugache_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise UgkError("%s is missing: build it with `python -m ugache_amd.build`" % LIB_PATH)
        l = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, args in SIGNATURES.items():
            f = getattr(l, name)  # AttributeError if the symbol is not exported
            f.argtypes = args
            f.restype = _RESTYPES.get(name, C.c_int)
        _lib = l
    return _lib


def call(name, *args):
    """Call an entry point and raise UgkError with the library's message on a non-zero return."""
    f = getattr(lib(), name)
    rc = f(*args)
    if name in _NO_CHECK:
        return rc
    if rc != 0:
        raise UgkError("%s: %s" % (name, lib().ugk_last_error().decode()))
    return 0


def table(kind, ptr, size, fb_mul=0, fb_mask=0):
    return Table(kind, 0, ptr, size, fb_mul, fb_mask)


def device_info(dev=0):
    info = DeviceInfo()
    call("ugk_get_device_info", dev, C.byref(info))
    return {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
            "wavefront_size": info.wavefront_size, "total_mem": info.total_mem, "lds_per_block": info.lds_per_block}
