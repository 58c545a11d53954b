"""Counterpart of python/collcache/torch/adapter.py of the reference: the names a PyTorch program imports from
`collcache.torch`, each a thin forwarder into the binding module `collcache.torch.c_lib` (adapter.py:25-60)."""
from ..common import *  # noqa: F401,F403
from ..common import _basics
from . import c_lib

config = _basics.config
log_step_by_key = _basics.log_step_by_key
report_step = _basics.report_step
report_step_average = _basics.report_step_average
wait_one_child = _basics.wait_one_child
print_memory_usage = _basics.print_memory_usage
coll_cache_record_init = _basics.coll_cache_record_init


def coll_torch_test(local_id, keys):
    return c_lib.coll_torch_test(local_id, keys)


def coll_torch_lookup_key_t_val_ret(local_id, keys, pad_to_8=True):
    return c_lib.coll_torch_lookup_key_t_val_ret(local_id, keys, pad_to_8)


def coll_torch_record(local_id, keys):
    c_lib.coll_torch_record(local_id, keys)


def coll_torch_init_t(replica_id, dev_id, emb, cache_percentage):
    c_lib.coll_torch_init_t(replica_id, dev_id, emb, cache_percentage)


def coll_torch_init(replica_id, key_space_size, dev_id, cpu_data, dim, cache_percentage, use_fp16):
    c_lib.coll_torch_init(replica_id, key_space_size, dev_id, cpu_data, dim, cache_percentage, use_fp16)


def coll_torch_create_emb_shm(replica_id, n_keys, dim, dtype, fname=""):
    return c_lib.coll_torch_create_emb_shm(replica_id, n_keys, dim, dtype, fname)


# what this build adds to the reference's surface
coll_torch_lookup_unique = c_lib.coll_torch_lookup_unique
coll_torch_lookup_pooled = c_lib.coll_torch_lookup_pooled
coll_torch_segment_offsets = c_lib.coll_torch_segment_offsets
coll_torch_lookup_async = c_lib.coll_torch_lookup_async
coll_torch_lookup_wait = c_lib.coll_torch_lookup_wait
coll_torch_forward_config = c_lib.coll_torch_forward_config
coll_torch_forward = c_lib.coll_torch_forward
coll_torch_forward_join = c_lib.coll_torch_forward_join
coll_torch_load_raw_model = c_lib.coll_torch_load_raw_model
coll_torch_refresh = c_lib.coll_torch_refresh
coll_torch_shutdown = c_lib.coll_torch_shutdown
