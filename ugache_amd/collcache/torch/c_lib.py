"""Counterpart of the reference's extension module `collcache.torch.c_lib` (python/collcache/torch/adapter.cc,
PYBIND11_MODULE(c_lib, m) at :274-281): coll_torch_init, coll_torch_init_t, coll_torch_test, coll_torch_record,
coll_torch_lookup_key_t_val_ret and coll_torch_create_emb_shm, importable as `from collcache.torch import c_lib`.

The reference binds these entry points with pybind11; here they are plain Python over the extern "C" shim, with
torch used only for what the C++ adapter used it for: device memory (the allocator handle and the reused output
buffer, adapter.cc:126-149, 204-237) and the stream.  Same names, argument meaning and return shapes.  The entry
points this build adds (stream-ordered and distinct-key lookups, the serving step, refresh, teardown) live here too;
`collcache.torch.adapter` re-exports everything under the reference's adapter.py names.
"""
import ctypes
import os
import sys

import torch

from ..common import *  # noqa: F401,F403
from ..common import ALLOC_FN, RELEASE_FN, _basics, kF16, kF32

_C = _basics.C_LIB_CTYPES


class _State:
    dev_id = {}            # replica -> device index
    external_dtype = torch.float32
    external_feat_dim = 0
    internal_feat_dim = 0
    batch_emb_reuse = None  # int8 tensor backing the reused output buffer
    out_views = {}          # padded batch length -> view of that buffer (slicing it anew costs microseconds per lookup)
    max_num_keys = 0        # what the library's max_num_keys was last set to from here
    last_keys = None        # key tensor of the most recent lookup
    held = {}              # device pointer -> tensor handed to the library by the allocator callback
    host_tables = []       # keeps pinned tables alive
    host_ptrs = []         # pinned allocations made by coll_torch_create_emb_shm
    alloc_cb = None
    release_cb = None


def _make_allocator(dev_id):
    """TorchMemHandle (adapter.h:37-46): library memory is an int8 torch tensor kept alive until released."""
    def _alloc(nbytes, _user):
        t = torch.empty((max(int(nbytes), 1),), dtype=torch.int8, device="cuda:%d" % dev_id)
        _State.held[t.data_ptr()] = t
        return t.data_ptr()

    def _release(ptr, _user):
        _State.held.pop(ptr, None)

    _State.alloc_cb = ALLOC_FN(_alloc)
    _State.release_cb = RELEASE_FN(_release)
    return _State.alloc_cb, _State.release_cb


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_handle(dev_id):
    # lookups run on torch's current stream, so they are ordered after whatever produced the keys
    if _raw_stream is not None:  # the handle without building a Stream object: a microsecond less per lookup
        return ctypes.c_void_p(_raw_stream(dev_id))
    return ctypes.c_void_p(torch.cuda.current_stream(dev_id).cuda_stream)


def _setup_dims(dim, use_fp16, dtype=None):
    """use_fp16: elements of two bytes (the reference's flag, adapter.cc:126-190); dtype says which two-byte type the
    lookups return (float16 unless the table is bfloat16, which the library moves as the same bytes)"""
    _State.external_feat_dim = dim
    if use_fp16:
        if dim % 2 != 0:
            sys.stderr.write("dimension must be even\n")
            os.abort()
        _State.external_dtype = dtype if dtype is not None else torch.float16
        _State.internal_feat_dim = dim // 2
    else:
        _State.external_dtype = torch.float32
        _State.internal_feat_dim = dim


def coll_torch_init_t(replica_id, dev_id, emb, cache_percentage):
    """adapter.cc:151-190: build the cache of `replica_id` on GPU `dev_id` from the host table `emb`."""
    torch.cuda.set_device(dev_id)
    _State.dev_id[replica_id] = dev_id
    alloc, release = _make_allocator(dev_id)
    use_fp16 = emb.dtype in (torch.float16, torch.bfloat16)  # two-byte elements: the same bytes to the library
    if not use_fp16 and emb.dtype != torch.float32:
        raise TypeError("embedding table must be float32, float16 or bfloat16, got %s" % emb.dtype)
    dim = emb.size(1)
    _setup_dims(dim, use_fp16, emb.dtype if use_fp16 else None)
    info_keys = emb.size(0)
    _C.coll_cache_init_c(replica_id, info_keys, alloc, release, None, emb.data_ptr(), kF16 if use_fp16 else kF32, dim,
                         float(cache_percentage), _stream_handle(dev_id))
    _State.host_tables.append(emb)


def coll_torch_init(replica_id, key_space_size, dev_id, cpu_data, dim, cache_percentage, use_fp16):
    """adapter.cc:126-149: same with a raw host pointer (integer address)."""
    torch.cuda.set_device(dev_id)
    _State.dev_id[replica_id] = dev_id
    alloc, release = _make_allocator(dev_id)
    _setup_dims(dim, use_fp16)
    _C.coll_cache_init_c(replica_id, key_space_size, alloc, release, None, cpu_data, kF16 if use_fp16 else kF32, dim,
                         float(cache_percentage), _stream_handle(dev_id))


def coll_torch_test(local_id, keys):
    """adapter.cc:192-203: an uninitialised tensor of the output's shape."""
    dev = _State.dev_id.get(local_id, 0)
    return torch.empty((keys.size(0), _State.external_feat_dim), dtype=torch.float32, device="cuda:%d" % dev)


def _lookup_into_reused_buffer(local_id, keys, pad_to_8, fn32, fn64):
    dev = _State.dev_id.get(local_id, 0)
    if keys.dtype not in (torch.int32, torch.int64, torch.uint32):
        raise TypeError("keys must be int32 / uint32 or int64, got %s" % keys.dtype)
    if not keys.is_cuda:
        raise ValueError("keys must live on the GPU (the reference reads key.data_ptr() from device code too)")
    if not keys.is_contiguous():
        keys = keys.contiguous()
    _State.last_keys = keys  # a stream-ordered lookup reads them after this call has returned
    n = keys.size(0)
    padded_len = (n + 7) // 8 * 8 if pad_to_8 else n
    tensor = _State.out_views.get(padded_len)
    if tensor is None:
        max_num_keys = _C.coll_cache_max_num_keys()
        if padded_len > max_num_keys:
            sys.stderr.write("Warning, found a larger batch, re allocating emb output now %d %d\n"
                             % (padded_len, max_num_keys))
            max_num_keys = max(max_num_keys, padded_len)
            _State.batch_emb_reuse = None
        if _State.batch_emb_reuse is None:
            max_num_keys = int(max_num_keys * 1.05)
            _C.coll_cache_set_max_num_keys(max_num_keys)
            _State.batch_emb_reuse = torch.empty((max(max_num_keys, 1) * _State.internal_feat_dim * 4,),
                                                 dtype=torch.int8, device="cuda:%d" % dev)
            _State.out_views.clear()  # they pointed into the old buffer
        elem = 4 if _State.external_dtype == torch.float32 else 2
        tensor = _State.batch_emb_reuse[: padded_len * _State.external_feat_dim * elem].view(
            _State.external_dtype).view(padded_len, _State.external_feat_dim)
        if len(_State.out_views) < 64:
            _State.out_views[padded_len] = tensor
    if keys.dtype == torch.int64:
        fn64(local_id, keys.data_ptr(), n, tensor.data_ptr(), _stream_handle(dev))
    else:
        fn32(local_id, keys.data_ptr(), n, tensor.data_ptr(), _stream_handle(dev))
    return tensor


def coll_torch_lookup_key_t_val_ret(local_id, keys, pad_to_8=True):
    """adapter.cc:204-237: look the keys (GPU int32/uint32 tensor, or int64) up; returns a [ceil8(N), dim] view of one
    reused output buffer — the next lookup overwrites it."""
    return _lookup_into_reused_buffer(local_id, keys, pad_to_8, _C.coll_cache_lookup, _C.coll_cache_lookup_i64)


def coll_torch_lookup_unique(local_id, keys):
    """the distinct keys of the batch looked up once (extension): returns (emb, inverse) with emb [num_distinct, dim] a
    view of the reused output buffer and inverse an int32 tensor [len(keys)] such that emb[inverse[i]] is the row of
    keys[i] — the `ids, idx = unique(ids); emb = lookup(ids)` of the TF2 sparse layer in one call, with the unique done
    by the library's GPU hash set (distinct keys come in order of first claim, not sorted)."""
    inverse = torch.empty((keys.numel(),), dtype=torch.int32, device=keys.device)
    found = [0]

    def fn32(replica, key_ptr, n, out_ptr, stream):
        found[0] = _C.coll_cache_lookup_unique(replica, key_ptr, n, out_ptr, inverse.data_ptr(), stream)

    def fn64(replica, key_ptr, n, out_ptr, stream):
        found[0] = _C.coll_cache_lookup_unique_i64(replica, key_ptr, n, out_ptr, inverse.data_ptr(), stream)

    out = _lookup_into_reused_buffer(local_id, keys.reshape(-1), False, fn32, fn64)
    return out[: found[0]], inverse


COMBINERS = {"sum": 0, "mean": 1, "sqrtn": 2}


def pooled_lookup_supported():
    """whether coll_torch_lookup_pooled can take the rows of the table that was built (a multiple of 16 bytes, at
    most 4096; fp32, fp16 or bfloat16 elements)"""
    elem = 4 if _State.external_dtype == torch.float32 else 2
    row_bytes = _State.external_feat_dim * elem
    return _State.external_dtype in _POOL_ELEM and row_bytes % 16 == 0 and 0 < row_bytes <= 4096


# element codes of the pooled lookup: the size for fp32 and fp16, UGK_ELEM_BF16 for bfloat16
_POOL_ELEM = {torch.float32: 4, torch.float16: 2, torch.bfloat16: 0x102}


def coll_torch_lookup_pooled(local_id, ids, seg_off, weights=None, combiner="sum", serving_step=False,
                             stream_ordered=False, max_norm=None):
    """lookup and per-sample combination of a multi-hot feature in one kernel (extension): segment r is
    ids[seg_off[r] : seg_off[r + 1]]; returns a new [len(seg_off) - 1, dim] tensor whose row r is the weighted sum of
    the segment's embeddings ("sum"), divided by the sum of the weights ("mean") or by the root of the sum of their
    squares ("sqrtn") — embedding_lookup_sparse without the [len(ids), dim] intermediate.  ids: GPU int32 / int64;
    seg_off: GPU int64, ascending, seg_off[0] == 0 and seg_off[-1] == len(ids); weights: GPU float32 or None.
    serving_step: the call is one step of the serving loop (as coll_torch_forward is for a plain lookup; with
    stream_ordered as well it blocks only if the step's prefix is counted on the host and exceeds 64 KB).
    stream_ordered: the call is enqueued on torch's current stream and returns without waiting, like any torch op
    (as coll_torch_lookup_async is for a plain lookup; `ids`, `seg_off` and `weights` must stay alive until the work has
    run; coll_torch_lookup_wait reports a bad id or offset and makes the group sizes available).
    max_norm: every looked-up embedding is clipped to this l2 norm before it is weighted (the layer's max_norm)."""
    dev = _State.dev_id.get(local_id, 0)
    if max_norm is not None and not float(max_norm) > 0:
        raise ValueError("max_norm must be a positive l2 norm or None, got %r" % (max_norm,))
    if not pooled_lookup_supported():
        raise ValueError("pooled lookups need rows of a multiple of 16 bytes, at most 4096, of fp32, fp16 or bfloat16 "
                         "elements")
    if ids.dtype not in (torch.int32, torch.int64, torch.uint32) or not ids.is_cuda:
        raise TypeError("ids must be a GPU tensor of int32 / uint32 or int64")
    if seg_off.dtype != torch.int64 or not seg_off.is_cuda or seg_off.dim() != 1 or seg_off.numel() < 1:
        raise TypeError("seg_off must be a one-dimensional GPU int64 tensor of num_rows + 1 offsets")
    if weights is not None and (weights.dtype != torch.float32 or not weights.is_cuda or weights.numel() != ids.numel()):
        raise TypeError("weights must be a GPU float32 tensor with one weight per id")
    ids, seg_off = ids.contiguous().reshape(-1), seg_off.contiguous()
    weights = None if weights is None else weights.contiguous().reshape(-1)
    n_rows = seg_off.numel() - 1
    out = torch.empty((n_rows, _State.external_feat_dim), dtype=_State.external_dtype, device="cuda:%d" % dev)
    if serving_step and stream_ordered:
        fn = (_C.coll_cache_forward_pooled_async_i64 if ids.dtype == torch.int64
              else _C.coll_cache_forward_pooled_async)
    elif serving_step:
        fn = _C.coll_cache_forward_pooled_i64 if ids.dtype == torch.int64 else _C.coll_cache_forward_pooled
    elif stream_ordered:
        fn = _C.coll_cache_lookup_pooled_async_i64 if ids.dtype == torch.int64 else _C.coll_cache_lookup_pooled_async
    else:
        fn = _C.coll_cache_lookup_pooled_i64 if ids.dtype == torch.int64 else _C.coll_cache_lookup_pooled
    if max_norm is not None:
        _C.coll_cache_set_pooled_max_norm(local_id, float(max_norm))
    try:
        fn(local_id, ids.data_ptr() if ids.numel() else None, seg_off.data_ptr(),
           None if weights is None else weights.data_ptr(), n_rows, ids.numel(), COMBINERS[combiner],
           _POOL_ELEM[_State.external_dtype], out.data_ptr(), _stream_handle(dev))
    finally:
        if max_norm is not None:  # the launch has taken it: the lookups that follow are not clipped
            _C.coll_cache_set_pooled_max_norm(local_id, 0.0)
    return out


def coll_torch_segment_offsets(local_id, rows, num_rows):
    """the seg_off coll_torch_lookup_pooled takes, from the row of every entry of a sparse feature in row-major order
    (extension): a new GPU int64 tensor of num_rows + 1 offsets, seg_off[r] = number of entries whose row is below r.
    One kernel on torch's current stream, no synchronisation (torch.bincount + cumsum make the same numbers and wait
    for the device on the way).  rows: GPU int64, ascending, inside [0, num_rows)."""
    if rows.dtype != torch.int64 or not rows.is_cuda:
        raise TypeError("rows must be a GPU int64 tensor")
    dev = _State.dev_id.get(local_id, 0)
    rows = rows.contiguous().reshape(-1)
    seg_off = torch.empty(int(num_rows) + 1, dtype=torch.int64, device=rows.device)
    _C.coll_cache_segment_offsets(local_id, rows.data_ptr() if rows.numel() else None, rows.numel(), int(num_rows),
                                  seg_off.data_ptr(), _stream_handle(dev))
    return seg_off


def coll_torch_lookup_async(local_id, keys, pad_to_8=True):
    """stream-ordered form of coll_torch_lookup_key_t_val_ret: the batch is enqueued on torch's current stream and
    the call returns without waiting, like any torch op; the returned view of the reused buffer is valid for work
    enqueued on that stream afterwards.  `keys` must stay alive until the work has run (keep a reference, or call
    coll_torch_lookup_wait)."""
    return _lookup_into_reused_buffer(local_id, keys, pad_to_8, _C.coll_cache_lookup_async,
                                      _C.coll_cache_lookup_async_i64)


def coll_torch_lookup_wait(local_id):
    """wait for the stream-ordered lookups enqueued so far; aborts if one of them met a key outside its table"""
    _C.coll_cache_lookup_wait(local_id, _stream_handle(_State.dev_id.get(local_id, 0)))


def coll_torch_forward_config(enable_refresh, refresh_iter, record_fraction=0.05, periodic=False):
    """the serving loop's settings (ps_config's coll_cache_enable_refresh / coll_cache_refresh_iter,
    python_tf2/collcache_tf2/collcache_tf2_cc/collcache_tf2_cc_infra/src/inference_utils.cpp:62-140)"""
    _C.coll_cache_forward_config(int(bool(enable_refresh)), int(refresh_iter), float(record_fraction),
                                 int(bool(periodic)))


def coll_torch_forward(local_id, keys, pad_to_8=True, stream_ordered=False):
    """one serving step (LookupManager::forward, lookup_manager.cc:158-213): the hotness of a prefix of the batch is
    recorded, the keys are looked up, and at the configured step a refresh starts on a background thread.  Returns
    the same reused buffer view as coll_torch_lookup_key_t_val_ret.  stream_ordered (extension): the lookup is
    enqueued on torch's current stream like coll_torch_lookup_async and the call returns without waiting (a prefix
    counted on the host is then counted by a later step or by coll_torch_lookup_wait; one beyond
    COLL_RECORD_INLINE_BYTES = 64 KB makes the step block all the same)."""
    if stream_ordered:
        return _lookup_into_reused_buffer(local_id, keys, pad_to_8, _C.coll_cache_forward_async,
                                          _C.coll_cache_forward_async_i64)
    return _lookup_into_reused_buffer(local_id, keys, pad_to_8, _C.coll_cache_forward, _C.coll_cache_forward_i64)


def coll_torch_forward_join():
    """wait for a background refresh started by coll_torch_forward; returns how many have completed"""
    return int(_C.coll_cache_forward_join())


def coll_torch_record(local_id, keys):
    """adapter.cc:270-272: count the hotness of a batch of keys (CPU tensor)."""
    if keys.is_cuda:
        keys = keys.cpu()
    keys = keys.contiguous()
    if keys.dtype == torch.int64:
        _C.coll_cache_record_i64(local_id, keys.data_ptr(), keys.numel())
    else:
        _C.coll_cache_record(local_id, keys.data_ptr(), keys.numel())


_ELEM = {torch.float32: 4, torch.float16: 2, torch.bfloat16: 2, torch.float64: 8, torch.int32: 4, torch.int64: 8, torch.uint8: 1,
         torch.int8: 1}


def coll_torch_create_emb_shm(replica_id, n_keys, dim, dtype, fname=""):
    """adapter.cc:239-268: the host embedding table as a CPU tensor [n_keys, dim].  The reference places it in POSIX
    shared memory and page-locks it later; here it is allocated pinned and GPU-mapped from the start.  If `fname` is
    given the file must hold exactly n_keys * dim elements and is read into the table."""
    nbytes = int(n_keys) * int(dim) * _ELEM[dtype]
    ptr = _C.coll_cache_alloc_host_table(max(nbytes, 64))
    _State.host_ptrs.append(ptr)
    buf = (ctypes.c_uint8 * max(nbytes, 64)).from_address(ptr)
    tensor = torch.frombuffer(buf, dtype=dtype, count=int(n_keys) * int(dim)).view(int(n_keys), int(dim))
    if fname != "":
        size = os.stat(fname).st_size
        if size != nbytes:
            sys.stderr.write("feat file on disk not equal with claimed shape %d != %dx%dx%d\n"
                             % (size, _ELEM[dtype], n_keys, dim))
            os.abort()
        with open(fname, "rb") as f:
            f.readinto(buf)
    return tensor


def coll_torch_load_raw_model(replica_id, path, dim=None, dtype=torch.float32):
    """the host table from the serving stack's model directory (RawModelLoader::master_load,
    python_tf2/collcache_tf2/collcache_tf2_cc/collcache_tf2_cc_infra/src/modelloader.cpp:52-107):
      `path`/key         int64 per row — only its length is used, the number of rows; row i belongs to key i
      `path`/emb_vector  the rows, `dtype` elements, read into the table as they are
    or `mock_<rows>_<dim>`: a table of that shape whose contents nobody defines (the reference leaves the mapped
    memory as it is; here it is zero-filled, so every key still has a row).  `dim` is only needed for a directory
    whose key file is empty.  Returns the pinned CPU tensor [rows, dim] for coll_torch_init_t."""
    name = os.path.basename(os.path.normpath(path))
    if name.startswith("mock_"):
        parts = name.split("_")
        n_keys, mdim = int(parts[1]), int(parts[-1])
        t = coll_torch_create_emb_shm(replica_id, n_keys, mdim, dtype)
        t.zero_()
        return t
    n_keys = os.stat(os.path.join(path, "key")).st_size // 8
    vec = os.path.join(path, "emb_vector")
    vec_bytes = os.stat(vec).st_size
    if dim is None:
        if n_keys == 0 or vec_bytes % (n_keys * _ELEM[dtype]) != 0:
            sys.stderr.write("emb_vector of %d bytes does not hold %d rows of whole %d-byte elements\n"
                             % (vec_bytes, n_keys, _ELEM[dtype]))
            os.abort()
        dim = vec_bytes // (n_keys * _ELEM[dtype])
    return coll_torch_create_emb_shm(replica_id, n_keys, dim, dtype, vec)


def coll_torch_refresh(replica_id, foreground=False):
    """re-place by the hotness recorded since the last build/refresh (the TF binding's LookupManager::refresh)."""
    dev = _State.dev_id.get(replica_id, 0)
    _basics.refresh(replica_id, _stream_handle(dev), foreground)


def coll_torch_shutdown():
    """drop the cache and every buffer it holds, including the tables made by coll_torch_create_emb_shm, which
    must not be used afterwards (the reference has no teardown)."""
    torch.cuda.synchronize()
    _State.last_keys = None
    _basics.shutdown()
    for p in _State.host_ptrs:
        _C.coll_cache_free_host_table(p)
    _State.host_ptrs.clear()
    _State.batch_emb_reuse = None
    _State.out_views.clear()
    _State.held.clear()
    _State.host_tables.clear()
    _State.dev_id.clear()
