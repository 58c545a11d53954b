"""The serving stack of the reference's TF2 binding, for PyTorch: a ps_config JSON file configures the cache, a model
directory holds the table, a layer object looks keys up and the library records hotness and refreshes in the
background.

Mirrors, call for call,
  collcache_tf2.Config / Init / Report / wait_one_child / SetStepProfileValue
      (python_tf2/collcache_tf2/collcache_tf2/core/initialize.py:33-39, 79-127, 129-290, 292-295)
  collcache_tf2.LookupLayer (core/lookup_layer.py:22-110), collcache_tf2.SparseLookupLayer
      (core/sparse_lookup_layer.py:27-265)
over LookupManager::{config, record_hotness, init, forward} (python_tf2/collcache_tf2/collcache_tf2_cc/
collcache_tf2_cc_infra/src/lookup_manager.cc:49-212) and the ps_config parser
(collcache_tf2_cc_infra/src/inference_utils.cpp:55-160).  One process, one replica, one GPU.

Call order, as in the reference's inference scripts:
    Config(ps_config_file=...)            # parse, configure the library, open the hotness recorder
    record_hotness(keys) ...              # presampled batches
    Init(ps_config_file=..., global_batch_size=...)   # load the model, rank, place, fill the cache
    layer = LookupLayer(model_name, table_id, emb_vec_size, emb_vec_dtype)
    emb = layer(keys)                     # one LookupManager::forward step
"""
import json
import os
import sys

import torch

from . import adapter as _adapter
from . import c_lib as _c_lib
from ..common import _basics

# the share of every batch whose hotness the serving loop records (lookup_manager.cc:295-300: the first 5 %)
RECORD_FRACTION = 0.05


def _abort(msg):
    """the reference's COLL_CHECK: print and abort (collcache_tf2_cc_infra logging), no exception to catch"""
    sys.stderr.write("ps_config: %s\n" % msg)
    sys.stderr.flush()
    os.abort()


def _need(obj, key, where):
    if key not in obj:
        _abort('no "%s" in %s' % (key, where))
    return obj[key]


class PsConfig:
    """parameter_server_config (inference_utils.cpp:55-160): the keys it reads, their defaults and which of them it
    insists on"""

    def __init__(self, ps_config_file, global_replica_id=0):
        try:
            with open(ps_config_file) as f:
                cfg = json.load(f)
        except (OSError, ValueError) as e:
            _abort("cannot read %s: %s" % (ps_config_file, e))
        self.use_multi_worker = bool(cfg.get("use_multi_worker", False))
        self.coll_cache_refresh_iter = int(cfg["coll_cache_refresh_iter"]) if "coll_cache_refresh_iter" in cfg else None
        self.coll_cache_enable_refresh = bool(cfg.get("coll_cache_enable_refresh", False))
        self.iteration_per_epoch = int(_need(cfg, "iteration_per_epoch", "the configuration"))
        self.epoch = int(_need(cfg, "epoch", "the configuration"))
        self.coll_cache_policy = int(cfg.get("coll_cache_policy", 13))
        models = _need(cfg, "models", "the configuration")
        if not isinstance(models, list) or len(models) == 0:
            _abort("No model configurations in JSON. Is the file formatted correctly?")
        if len(models) != 1:
            _abort("only single inference parameter is supported")
        m = models[0]
        self.model_name = str(m.get("model", ""))
        self.max_batch_size = int(m.get("max_batch_size", 64))
        files = _need(m, "sparse_files", "the model")
        self.sparse_files = [str(x) for x in files] if isinstance(files, list) else []
        self.cache_size_percentage = float(m.get("gpucacheper", 0.2))
        self.i64_input_key = bool(m.get("i64_input_key", True))
        devs = _need(m, "deployed_device_list", "the model")
        self.deployed_devices = sorted(int(d) for d in devs) if isinstance(devs, list) else []
        q = _need(m, "maxnum_catfeature_query_per_table_per_sample", "the model")
        self.maxnum_catfeature_query_per_table_per_sample = [int(x) for x in q] if isinstance(q, list) else []
        v = _need(m, "embedding_vecsize_per_table", "the model")
        self.embedding_vecsize_per_table = [int(x) for x in v] if isinstance(v, list) else []
        self.max_vocabulary_size = [int(x) for x in m["max_vocabulary_size"]] if "max_vocabulary_size" in m else []
        self.global_replica_id = global_replica_id
        # hier_parameter_server.cpp:43-46 and lookup_manager.cc:52-66
        if len(self.sparse_files) != 1:
            _abort("Coll cache only support single sparse file for now")
        if len(self.embedding_vecsize_per_table) != len(self.sparse_files):
            _abort("The number of embedding tables doesn't match the size of 'sparse_files' in configuration.")
        if self.deployed_devices != [0]:
            _abort("deployed_device_list must be [0]: this build serves one replica on one GPU")
        if not self.max_vocabulary_size:
            _abort('no "max_vocabulary_size" in the model: it is the key space of the cache')


class _Manager:
    cfg = None
    initialized = False
    table = None
    device = 0


def Config(ps_config_file, **kwargs):
    """collcache_tf2.Config -> LookupManager::config: parse the file, configure the library
    (hier_parameter_server.cpp:55-69: cache share, policy, steps, epochs, key space) and open the hotness recorder"""
    cfg = PsConfig(ps_config_file)
    _adapter.config({
        "cache_percentage": cfg.cache_size_percentage, "_cache_policy": cfg.coll_cache_policy, "num_device": 1,
        "num_global_step_per_epoch": cfg.iteration_per_epoch, "num_epoch": cfg.epoch,
        "num_total_item": cfg.max_vocabulary_size[0], "omp_thread_num": int(kwargs.get("omp_thread_num", 8)),
    })
    _adapter.coll_cache_record_init(0)
    _Manager.cfg = cfg
    _Manager.initialized = False
    return "OK"


def record_hotness(keys, model_name=None, table_id=0):
    """LookupManager::record_hotness (lookup_manager.cc:143-157): the keys of a presampled batch, on any device; they
    are copied to the host and counted there"""
    if _Manager.cfg is None:
        _abort("Config() has not been called")
    want = torch.int64 if _Manager.cfg.i64_input_key else torch.int32
    _adapter.coll_torch_record(0, keys.detach().reshape(-1).to("cpu", want))


def Init(ps_config_file=None, global_batch_size=1, **kwargs):
    """collcache_tf2.Init -> LookupManager::init + init_per_replica (lookup_manager.cc:98-141, 214-312): load the model
    file, rank the recorded hotness, place and fill the cache, arm the background refresh"""
    if _Manager.cfg is None:
        if ps_config_file is None:
            _abort("Init() needs Config() first or a ps_config_file")
        Config(ps_config_file, **kwargs)
    cfg = _Manager.cfg
    if global_batch_size <= 0:
        _abort("global_batch_size must be > 0.")
    if global_batch_size > cfg.max_batch_size:
        _abort("global_batch_size / num_replicas_in_sync must be <= max_batchsize configured in ps_config.json.")
    dim = cfg.embedding_vecsize_per_table[0]
    # `emb_table` (an extension): a table that is in memory already, as coll_torch_create_emb_shm returns it, instead of
    # the model directory named by the configuration
    table = kwargs.get("emb_table")
    if table is None:
        table = _adapter.coll_torch_load_raw_model(0, cfg.sparse_files[0], dim=dim, dtype=torch.float32)
    if table.shape[0] != cfg.max_vocabulary_size[0] or table.shape[1] != dim:
        _abort("the model holds %d rows of %d values, the configuration says %d rows of %d"
               % (table.shape[0], table.shape[1], cfg.max_vocabulary_size[0], dim))
    _adapter.coll_torch_init_t(0, _Manager.device, table, cfg.cache_size_percentage)
    refresh_iter = cfg.coll_cache_refresh_iter if cfg.coll_cache_refresh_iter is not None else 0
    _adapter.coll_torch_forward_config(cfg.coll_cache_enable_refresh, refresh_iter, RECORD_FRACTION, False)
    _Manager.table = table
    _Manager.initialized = True
    return "OK"


class LookupLayer(torch.nn.Module):
    """collcache_tf2.LookupLayer (core/lookup_layer.py:22-110): keys of any shape in, their embedding vectors out,
    shape `inputs.shape + (emb_vec_size,)`.  The result is a view of the library's reused output buffer, valid until
    the next lookup (as everywhere in this binding; clone() to keep it)."""

    def __init__(self, model_name, table_id, emb_vec_size, emb_vec_dtype=torch.float32, **kwargs):
        super().__init__()
        self.model_name = model_name
        self.table_id = table_id
        self.emb_vec_size = emb_vec_size
        self.emb_vec_dtype = emb_vec_dtype
        # stream_ordered=True (extension): the step is enqueued on torch's current stream like any torch op (only a
        # recorded prefix beyond 64 KB that is counted on the host still makes it block)
        self.stream_ordered = bool(kwargs.get("stream_ordered", False))

    def check(self, inputs):
        """the configuration's say on a batch of keys (model, table, width, key type, size)"""
        cfg = _Manager.cfg
        if cfg is None or not _Manager.initialized:
            _abort("Init() has not been called")
        if self.model_name != cfg.model_name or self.table_id != 0:
            _abort("no table %d of model '%s' in the configuration" % (self.table_id, self.model_name))
        if self.emb_vec_size != cfg.embedding_vecsize_per_table[0]:
            _abort("emb_vec_size %d differs from the configured %d"
                   % (self.emb_vec_size, cfg.embedding_vecsize_per_table[0]))
        want = torch.int64 if cfg.i64_input_key else torch.int32
        if inputs.dtype != want:
            _abort("keys must be %s (i64_input_key = %s)" % (want, cfg.i64_input_key))
        if inputs.numel() > cfg.max_batch_size * cfg.maxnum_catfeature_query_per_table_per_sample[0]:
            _abort("%d keys exceed max_batch_size x maxnum_catfeature_query_per_table_per_sample" % inputs.numel())

    def forward(self, inputs):
        self.check(inputs)
        emb = _adapter.coll_torch_forward(0, inputs.reshape(-1), False, stream_ordered=self.stream_ordered)
        return emb.reshape(tuple(inputs.shape) + (self.emb_vec_size,))


class SparseLookupLayer(torch.nn.Module):
    """collcache_tf2.SparseLookupLayer (core/sparse_lookup_layer.py:27-265), i.e. embedding_lookup_sparse over the
    cache: `sp_ids` is an N x M sparse COO tensor of int64 ids in row-major order with at least one id per row,
    `sp_weights` a sparse tensor of the same indices or None; the distinct ids are looked up once
    (unique -> lookup -> gather, sparse_lookup_layer.py:196-209), multiplied by their weights and combined per row:
    "sum", "mean" (weighted sum / sum of weights) or "sqrtn" (weighted sum / sqrt of the sum of squared weights);
    `max_norm` clips every embedding's l2 norm before combining.  Returns [N, emb_vec_size]."""

    def __init__(self, model_name, table_id, emb_vec_size, emb_vec_dtype=torch.float32, **kwargs):
        super().__init__()
        self.lookup = LookupLayer(model_name, table_id, emb_vec_size, emb_vec_dtype)
        self.emb_vec_size = emb_vec_size
        self.unique_in_library = bool(kwargs.get("unique_in_library", False))
        # fused=True: lookup, clipping to max_norm and combination in one kernel of the library
        # (coll_torch_lookup_pooled) wherever that kernel can take the rows; the steps below otherwise
        self.fused = bool(kwargs.get("fused", False))
        # stream_ordered=True (with fused): the step is enqueued on torch's current stream like any torch op (only a
        # recorded prefix beyond 64 KB that is counted on the host still makes it block)
        self.stream_ordered = bool(kwargs.get("stream_ordered", False))

    def forward(self, sp_ids, sp_weights=None, name=None, combiner=None, max_norm=None):
        if combiner is None:
            combiner = "mean"
        if combiner not in ("mean", "sqrtn", "sum"):
            raise ValueError("combiner must be one of 'mean', 'sqrtn' or 'sum', got %s" % combiner)
        if not (isinstance(sp_ids, torch.Tensor) and sp_ids.is_sparse):
            raise TypeError("sp_ids must be a sparse COO tensor, got %s" % type(sp_ids))
        if sp_weights is not None and not (isinstance(sp_weights, torch.Tensor) and sp_weights.is_sparse):
            raise TypeError("sp_weights must be either None or a sparse COO tensor, got %s" % type(sp_weights))
        # entries as given (row-major order is the caller's contract); coalesce() would merge duplicate positions
        segment_ids = sp_ids._indices()[0]
        ids = sp_ids._values()
        if max_norm is not None and not float(max_norm) > 0:
            raise ValueError("max_norm must be a positive l2 norm or None, got %r" % (max_norm,))
        if self.fused and _c_lib.pooled_lookup_supported():
            self.lookup.check(ids)
            num_rows = int(sp_ids.shape[0])
            seg_off = _adapter.coll_torch_segment_offsets(0, segment_ids, num_rows)
            weights = None if sp_weights is None else sp_weights._values().float()
            return _adapter.coll_torch_lookup_pooled(0, ids, seg_off, weights, combiner, serving_step=True,
                                                     stream_ordered=self.stream_ordered, max_norm=max_norm)
        if self.unique_in_library:  # unique + lookup in one call, the unique by the library's GPU hash set
            self.lookup.check(ids)
            emb_unique, idx = _adapter.coll_torch_lookup_unique(0, ids)
            embeddings = emb_unique.index_select(0, idx.long())
        else:
            ids, idx = torch.unique(ids, return_inverse=True)
            embeddings = self.lookup(ids).index_select(0, idx)
        original_dtype = embeddings.dtype
        if embeddings.dtype in (torch.float16, torch.bfloat16):
            embeddings = embeddings.float()  # low-precision rows are combined in fp32
        if max_norm is not None:
            norms = embeddings.norm(dim=1, keepdim=True)
            embeddings = embeddings * torch.clamp(max_norm / norms.clamp_min(1e-30), max=1.0)
        num_rows = int(sp_ids.shape[0])
        if sp_weights is None:
            weights = torch.ones(embeddings.shape[0], dtype=embeddings.dtype, device=embeddings.device)
        else:
            weights = sp_weights._values().to(embeddings.dtype)
            embeddings = embeddings * weights.unsqueeze(1)

        def segment_sum(x):
            out = torch.zeros((num_rows,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
            return out.index_add_(0, segment_ids, x)

        combined = segment_sum(embeddings)
        if combiner == "mean":
            denom = segment_sum(weights).unsqueeze(1)
        elif combiner == "sqrtn":
            denom = segment_sum(weights * weights).sqrt().unsqueeze(1)
        else:
            denom = None
        if denom is not None:  # div_no_nan: a zero denominator gives zero
            combined = torch.where(denom != 0, combined / torch.where(denom != 0, denom, torch.ones_like(denom)),
                                   torch.zeros_like(combined))
        return combined.to(original_dtype)


def _last_step_key():
    """key of the last completed step of replica 0: steps * num_device + replica (hier_parameter_server.hpp:53-56)"""
    return max(int(_basics.info(0)["lookups"]) - 1, 0)


def Report():
    """collcache_tf2.Report -> LookupManager::report_avg: the step-average report the evaluation scripts scrape"""
    _adapter.report_step_average(_last_step_key())


def SetStepProfileValue(profile_type, value, **kwargs):
    """collcache_tf2.SetStepProfileValue(profile_type=, value=) -> LookupManager::set_step_profile_value
    (lookup_manager.h:57-63): logs one profiler item for the step that has just completed"""
    _adapter.log_step_by_key(_last_step_key(), int(profile_type), float(value))


def wait_one_child():
    return _adapter.wait_one_child()


def NopDep(dense, emb):
    """collcache_tf2.NopDep: `dense`, made to depend on `emb` having been computed.  A TensorFlow graph needs the
    dependency spelled out; here lookups are blocking or stream-ordered, so `dense` comes back as it is."""
    return dense


def Shutdown():
    """drop everything so that Config() may be called again (the reference has no teardown)"""
    _adapter.coll_torch_forward_join()
    _adapter.coll_torch_shutdown()
    _Manager.cfg = None
    _Manager.initialized = False
    _Manager.table = None
