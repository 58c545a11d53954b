"""ctypes view of oracle/libugache_oracle.so for the tests (the oracle is the checker, never the product)."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_SO = os.path.join(ORACLE_DIR, "libugache_oracle.so")

u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
u64p = np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")
u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
vp = C.c_void_p
sz = C.c_size_t

IDX_DTYPE = np.dtype([("dst_off", np.uint32), ("src", np.uint32)])
BUCKET_DTYPE = np.dtype([("state_key", np.uint32), ("val", np.uint32)])


def _ptr(a):
    return None if a is None else a.ctypes.data_as(vp)


def load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR], stdout=subprocess.DEVNULL)
    lib = C.CDLL(_SO)
    lib.orc_murmur3_32_u32.restype = C.c_uint32
    lib.orc_murmur3_32_u32.argtypes = [C.c_uint32, C.c_uint32]
    lib.orc_murmur3_32_bytes.restype = C.c_uint32
    lib.orc_murmur3_32_bytes.argtypes = [C.c_char_p, C.c_int, C.c_uint32]
    lib.orc_table_size.restype = sz
    lib.orc_table_size.argtypes = [sz, sz]
    for f in ("orc_pack",):
        getattr(lib, f).restype = C.c_uint32
        getattr(lib, f).argtypes = [C.c_uint32, C.c_uint32]
    for f in ("orc_loc", "orc_off"):
        getattr(lib, f).restype = C.c_uint32
        getattr(lib, f).argtypes = [C.c_uint32]
    lib.orc_simple_init.argtypes = [vp, sz]
    lib.orc_simple_insert.restype = C.c_int
    lib.orc_simple_insert.argtypes = [vp, sz, u32p, u32p, sz]
    lib.orc_simple_search.restype = C.c_uint32
    lib.orc_simple_search.argtypes = [vp, sz, C.c_uint32]
    lib.orc_simple_evict.restype = C.c_int
    lib.orc_simple_evict.argtypes = [vp, sz, u32p, sz]
    lib.orc_simple_census.argtypes = [vp, sz, C.POINTER(sz * 3)]
    lib.orc_flat_init.argtypes = [u32p, sz]
    lib.orc_flat_insert.argtypes = [u32p, u32p, u32p, sz]
    lib.orc_flat_evict.argtypes = [u32p, u32p, sz]
    lib.orc_lookup_src_dst.argtypes = [vp, sz, vp, u32p, sz, C.c_uint32, vp]
    lib.orc_sort_idx.argtypes = [vp, sz]
    lib.orc_find_boundary.argtypes = [vp, sz, C.c_int, u32p]
    lib.orc_extract_group.argtypes = [vp, sz, vp, vp, sz]
    lib.orc_extract_mix.argtypes = [vp, sz, C.POINTER(vp), vp, sz]
    lib.orc_gather_u32.restype = C.c_int
    lib.orc_gather_u32.argtypes = [vp, sz, u32p, sz, vp, sz]
    lib.orc_gather_i64.restype = C.c_int
    lib.orc_gather_i64.argtypes = [vp, sz, i64p, sz, vp, sz]
    lib.orc_gather_scatter_u32.argtypes = [vp, u32p, u32p, sz, vp, sz]
    lib.orc_extract_feat.argtypes = [vp, sz, vp, u32p, sz, vp, vp, vp, sz, vp]
    lib.orc_freq_rank.restype = sz
    lib.orc_freq_rank.argtypes = [u32p, sz, u32p, u32p]
    lib.orc_rep_solve.restype = C.c_uint32
    lib.orc_rep_solve.argtypes = [u32p, C.c_uint32, C.c_double, u32p]
    lib.orc_cache_capacity.restype = sz
    lib.orc_cache_capacity.argtypes = [sz, C.c_double]
    lib.orc_refresh_plan.restype = C.c_int
    lib.orc_refresh_plan.argtypes = [u32p, u32p, C.c_uint32, u32p, u32p, C.POINTER(sz), u32p, C.POINTER(sz),
                                     u32p, u32p, C.POINTER(sz)]
    lib.orc_dedup_i64.restype = sz
    lib.orc_dedup_i64.argtypes = [i64p, sz, i64p, u32p]
    f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
    lib.orc_pool_f64.restype = C.c_int
    lib.orc_pool_f64.argtypes = [f64p, sz, sz, i64p, i64p, vp, sz, C.c_int, f64p]
    lib.orc_pool_clip_f64.restype = C.c_int
    lib.orc_pool_clip_f64.argtypes = [f64p, sz, sz, i64p, i64p, vp, sz, C.c_int, C.c_double, f64p]
    lib.orc_omp_threads.restype = C.c_int
    lib.orc_gather_u32_omp.restype = C.c_int
    lib.orc_gather_u32_omp.argtypes = [vp, sz, u32p, sz, vp, sz]
    lib.orc_gather_i64_omp.restype = C.c_int
    lib.orc_gather_i64_omp.argtypes = [vp, sz, i64p, sz, vp, sz]
    lib.orc_extract_flat_i64_omp.restype = C.c_int
    lib.orc_extract_flat_i64_omp.argtypes = [vp, sz, C.c_uint64, C.c_uint64, vp, sz, vp, sz, vp, vp, sz, vp]
    return lib


class Oracle:
    """numpy-friendly wrapper."""

    def __init__(self):
        self.lib = load()

    # --- gather -------------------------------------------------------------------------------
    def gather(self, table, keys, omp=False):
        table = np.ascontiguousarray(table)
        rb = table.strides[0]
        out = np.empty((len(keys),) + table.shape[1:], dtype=table.dtype)
        if keys.dtype == np.int64:
            f = self.lib.orc_gather_i64_omp if omp else self.lib.orc_gather_i64
        else:
            keys = keys.astype(np.uint32, copy=False)
            f = self.lib.orc_gather_u32_omp if omp else self.lib.orc_gather_u32
        rc = f(_ptr(table), table.shape[0], np.ascontiguousarray(keys), len(keys), _ptr(out), rb)
        if rc != 0:
            raise IndexError("key out of range")
        return out

    def extract_flat(self, flat, keys, cache, host_table, key_inv=0, key_mask=0):
        """the CPU baseline's mixed-source step; returns (rows, [n from the cache copy, n from the host table])"""
        host_table = np.ascontiguousarray(host_table)
        cache = np.ascontiguousarray(cache)
        rb = host_table.strides[0]
        out = np.empty((len(keys),) + host_table.shape[1:], dtype=host_table.dtype)
        counts = np.zeros(2, np.uint64)
        rc = self.lib.orc_extract_flat_i64_omp(_ptr(np.ascontiguousarray(flat, np.uint32)), host_table.shape[0],
                                               C.c_uint64(key_inv), C.c_uint64(key_mask),
                                               _ptr(np.ascontiguousarray(keys, np.int64)), len(keys), _ptr(cache),
                                               cache.shape[0], _ptr(host_table), _ptr(out), rb, _ptr(counts))
        if rc != 0:
            raise IndexError("key without a row, or slot outside the cache copy")
        return out, counts.tolist()

    # --- tables -------------------------------------------------------------------------------
    def simple_table(self, n_entries):
        nb = self.lib.orc_table_size(n_entries, 2)
        t = np.empty(nb, dtype=BUCKET_DTYPE)
        self.lib.orc_simple_init(_ptr(t), nb)
        return t

    def simple_insert(self, t, keys, vals):
        return self.lib.orc_simple_insert(_ptr(t), len(t), np.ascontiguousarray(keys, np.uint32),
                                          np.ascontiguousarray(vals, np.uint32), len(keys))

    def simple_search(self, t, key):
        return self.lib.orc_simple_search(_ptr(t), len(t), int(key))

    def simple_evict(self, t, keys):
        return self.lib.orc_simple_evict(_ptr(t), len(t), np.ascontiguousarray(keys, np.uint32), len(keys))

    def simple_census(self, t):
        out = (sz * 3)()
        self.lib.orc_simple_census(_ptr(t), len(t), C.byref(out))
        return tuple(out)

    def flat_table(self, nkeys):
        t = np.empty(nkeys, np.uint32)
        self.lib.orc_flat_init(t, nkeys)
        return t

    def lookup_src_dst(self, keys, simple=None, flat=None, fallback_loc=1):
        keys = np.ascontiguousarray(keys, np.uint32)
        idx = np.empty(len(keys), IDX_DTYPE)
        self.lib.orc_lookup_src_dst(_ptr(simple), 0 if simple is None else len(simple), _ptr(flat), keys, len(keys),
                                    fallback_loc, _ptr(idx))
        return idx

    def sort_idx(self, idx):
        self.lib.orc_sort_idx(_ptr(idx), len(idx))
        return idx

    def find_boundary(self, idx, num_location):
        g = np.zeros(num_location + 1, np.uint32)
        self.lib.orc_find_boundary(_ptr(idx), len(idx), num_location, g)
        return g

    def extract_feat(self, keys, cache, host_table, simple=None, flat=None):
        keys = np.ascontiguousarray(keys, np.uint32)
        host_table = np.ascontiguousarray(host_table)
        rb = host_table.strides[0]
        out = np.zeros((len(keys),) + host_table.shape[1:], host_table.dtype)
        g = np.zeros(3, np.uint32)
        self.lib.orc_extract_feat(_ptr(simple), 0 if simple is None else len(simple), _ptr(flat), keys, len(keys),
                                  _ptr(cache), _ptr(host_table), _ptr(out), rb, _ptr(g))
        return out, g

    # --- placement ----------------------------------------------------------------------------
    def freq_rank(self, stream):
        stream = np.ascontiguousarray(stream, np.uint32)
        rk = np.empty(len(stream), np.uint32)
        rc = np.empty(len(stream), np.uint32)
        m = self.lib.orc_freq_rank(stream, len(stream), rk, rc)
        return rk[:m].copy(), rc[:m].copy()

    def full_rank(self, stream, num_node):
        """observed keys in (count desc, key desc) order, then the never-seen keys in ascending order.
        The reference appends unseen keys in a thread-dependent order (freq_recorder.cc:305-333); ascending
        key is this build's documented tie rule."""
        rk, rc = self.freq_rank(stream)
        seen = np.zeros(num_node, bool)
        seen[rk] = True
        rest = np.nonzero(~seen)[0].astype(np.uint32)
        return np.concatenate([rk, rest]), np.concatenate([rc, np.zeros(len(rest), np.uint32)])

    def rep_solve(self, rank_keys, num_node, pct100):
        nid = np.empty(num_node, np.uint32)
        nc = self.lib.orc_rep_solve(np.ascontiguousarray(rank_keys, np.uint32), num_node, float(pct100), nid)
        return nid, nc

    def dedup(self, keys):
        keys = np.ascontiguousarray(keys, np.int64)
        uniq = np.empty(len(keys), np.int64)
        inv = np.empty(len(keys), np.uint32)
        nu = self.lib.orc_dedup_i64(keys, len(keys), uniq, inv)
        return uniq[:nu].copy(), inv

    # --- pooled lookup ------------------------------------------------------------------------
    def pool(self, table, ids, seg_off, weights, combiner, max_norm=None):
        """float64 combination of the rows of every segment; combiner: "sum" / "mean" / "sqrtn" or 0 / 1 / 2;
        max_norm: every row clipped to that l2 norm before it is weighted"""
        combiner = {"sum": 0, "mean": 1, "sqrtn": 2}.get(combiner, combiner)
        t = np.ascontiguousarray(table, dtype=np.float64)
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        seg_off = np.ascontiguousarray(seg_off, dtype=np.int64)
        w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float64)
        out = np.empty((len(seg_off) - 1, t.shape[1]), np.float64)
        if len(ids) == 0:
            ids = np.zeros(1, np.int64)
        rc = self.lib.orc_pool_clip_f64(t, t.shape[0], t.shape[1], ids, seg_off, None if w is None else w.ctypes.data,
                                        len(seg_off) - 1, combiner, float(max_norm or 0.0), out)
        if rc != 0:
            raise IndexError("id out of range")
        return out
