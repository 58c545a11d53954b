#include "cache_context.h"

#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <iostream>

#include "facade.h"
#include "logging.h"
#include "timer.h"

namespace coll_cache_lib {

namespace {

// location ids with one GPU: the GPU is 0, the host is num_device == 1 (cache_context.cu:2421-2422)
constexpr int kLocalLoc = UGK_LOC_LOCAL;
constexpr int kCpuLoc = UGK_LOC_HOST;

int PointerKind(const void *p) {
  int kind = 0;
  UGK_CALL(ugk_pointer_kind(p, &kind));
  return kind;
}

void RequireDeviceAccessible(const void *cpu_data) {
  CHECK(PointerKind(cpu_data) != 0)
      << "the host embedding table must be pinned, GPU-mapped memory (ugk_host_malloc / coll_cache_alloc_host_table / "
         "a torch tensor created with pin_memory=True): this platform does not page-lock an existing allocation the "
         "way the reference does with cudaHostRegister";
}

}  // namespace

CacheContext::~CacheContext() { delete _new_hash_table; }

// cache_context.cu:1887-1904 — 0 % cache: every row is read from the host table
void CacheContext::build_no_cache(int location_id, std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_src_data,
                                  DataType dtype, size_t dim, Context gpu_ctx, StreamHandle stream) {
  RequireDeviceAccessible(cpu_src_data);
  _cpu_location_id = 0;
  _local_location_id = location_id;
  _num_location = 1;
  _cache_nbytes = 0;
  _device_cache_data.assign(1, cpu_src_data);
  _cache_nodes = 0;
  _cache_space_capacity = 0;
  LOG(INFO) << "Collaborative GPU cache (policy: no cache)";
  std::cout << "test_result:init:cache_nbytes=" << _cache_nbytes << "\n";
}

// cache_context.cu:1906-1938 — 100 % cache: the whole table is copied into HBM, keys index it directly
void CacheContext::build_full_cache(int location_id, std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_src_data,
                                    DataType dtype, size_t dim, Context gpu_ctx, size_t num_total_nodes,
                                    StreamHandle stream) {
  _cpu_location_id = -1;
  _local_location_id = location_id;
  _num_location = 1;
  Timer t;
  _cache_nbytes = num_total_nodes * _row_bytes;
  _cache_space_capacity = num_total_nodes;
  _cache_nodes = num_total_nodes;
  _device_cache_data_local_handle = _eager_gpu_mem_allocator(_cache_nbytes);
  void *local_cache = _device_cache_data_local_handle->ptr();
  UGK_CALL(ugk_memcpy_async(local_cache, cpu_src_data, _cache_nbytes, stream));
  UGK_CALL(ugk_stream_sync(stream));
  _device_cache_data.assign(1, local_cache);
  LOG(INFO) << "Collaborative GPU cache (policy: full cache) " << num_total_nodes << " nodes ( "
            << ToReadableSize(_cache_nbytes) << " | " << t.Passed() << " secs )";
  std::cout << "test_result:init:cache_nbytes=" << _cache_nbytes << "\n";
}

// the ascending list of the rows a placement caches, made on the device: bit r of a bitmap over the key space = row r
// is cached (the ranked rows that are cached, then the lowest `num_extra` rows that are not among them), compacted in
// order.  Waits for `stream`: the list is complete on return.
TensorPtr CacheContext::KeyListOnDevice(TensorPtr top_rows, size_t num_extra, size_t num_rows, StreamHandle stream,
                                        MemHandle *bits_out) {
  CHECK_NOTNULL(top_rows);
  const size_t num_top = top_rows->NumItem(), num_cached = num_top + num_extra;
  CHECK_LT(num_cached, num_rows);
  if (num_cached == 0) return Tensor::EmptyExternal(kI32, {0}, _eager_gpu_mem_allocator, _trainer_ctx, "");
  const size_t words = (num_rows + 63) / 64;
  MemHandle ranked = _eager_gpu_mem_allocator(words * 8), placed = num_extra ? _eager_gpu_mem_allocator(words * 8) : nullptr;
  MemHandle bm_ws = _eager_gpu_mem_allocator(ugk_bitmap_workspace_bytes());
  MemHandle rank_ws = num_extra ? _eager_gpu_mem_allocator(ugk_rank_workspace_bytes()) : nullptr;
  MemHandle st = _eager_gpu_mem_allocator(256);
  MemHandle total = PinnedHostAlloc(64);
  UGK_CALL(ugk_fill_u32(ranked->ptr<uint32_t>(), 0, words * 2, stream));
  UGK_CALL(ugk_fill_u32(st->ptr<uint32_t>(), 0, 1, stream));
  if (num_top > 0) {
    TensorPtr top_dev = Tensor::CopyToExternal(top_rows, _eager_gpu_mem_allocator, _trainer_ctx, stream);
    UGK_CALL(ugk_bitmap_update(ranked->ptr<uint64_t>(), num_rows, top_dev->CPtr<uint32_t>(), num_top, 1,
                               st->ptr<uint32_t>(), stream));
    UGK_CALL(ugk_stream_sync(stream));  // top_dev goes out of scope
  }
  const uint64_t *cached = ranked->ptr<uint64_t>();
  if (num_extra > 0) {
    // every ranked row is cached and the lowest rows that were not ranked fill the rest: the placement of a cache that
    // is larger than the set of observed rows
    UGK_CALL(ugk_rank_place_observed(nullptr, num_rows, num_cached, rank_ws->ptr(), placed->ptr<uint64_t>(),
                                     ranked->ptr<uint64_t>(), 0, nullptr, nullptr, nullptr, nullptr,
                                     st->ptr<uint32_t>(), stream));
    cached = placed->ptr<uint64_t>();
  }
  UGK_CALL(ugk_bitmap_count(cached, nullptr, 0, num_rows, bm_ws->ptr(), total->ptr<uint32_t>(), stream));
  uint32_t status = 0;
  UGK_CALL(ugk_memcpy_async(&status, st->ptr(), sizeof(status), stream));
  UGK_CALL(ugk_stream_sync(stream));
  CHECK_EQ(status, 0u) << "key list on the device: a ranked key is outside the key space (1) or the ranked keys are "
                          "not distinct (0x20)";
  CHECK_EQ((size_t)*total->ptr<uint32_t>(), num_cached) << "key list on the device: the ranked keys are not distinct";
  TensorPtr list = Tensor::EmptyExternal(kI32, {num_cached}, _eager_gpu_mem_allocator, _trainer_ctx, "");
  UGK_CALL(ugk_bitmap_emit(cached, nullptr, 0, num_rows, bm_ws->ptr(), list->Ptr<uint32_t>(), num_cached, stream));
  UGK_CALL(ugk_stream_sync(stream));  // the bitmaps go out of scope
  if (bits_out) *bits_out = num_extra > 0 ? placed : ranked;
  return list;
}

// cache_context.cu:2414-2599 — partial cache: frequency-ranked fill + lookup table
void CacheContext::build_with_advise_new_hash(int location_id, std::shared_ptr<CollCache> coll_cache_ptr,
                                              void *cpu_data, DataType dtype, size_t dim, Context gpu_ctx,
                                              double cache_percentage, StreamHandle stream) {
  RequireDeviceAccessible(cpu_data);
  CHECK_EQ(RunConfig::num_device, (size_t)1) << "this build serves one GPU and its host";
  _num_location = (int)RunConfig::num_device + 1;
  _cpu_location_id = (int)RunConfig::num_device;
  CHECK_EQ(_cpu_location_id, kCpuLoc);
  CHECK_EQ(location_id, kLocalLoc);
  _local_location_id = location_id;
  CHECK(coll_cache_ptr->HasPartialPlacement());
  CHECK_NOTNULL(coll_cache_ptr->_block_access_advise);
  CHECK_NOTNULL(coll_cache_ptr->_block_density);
  // The solver may have left the key -> block array unwritten and handed over what it placed from (the ranked keys
  // that are cached + how many never-observed keys fill the rest): then the ascending list of cached rows is made on
  // the device, from a bitmap of the key space, and no pass over per-key arrays of the whole key space runs on the
  // host.  Bitmap positions are 32-bit.
  if (coll_cache_ptr->_nid_to_block == nullptr && coll_cache_ptr->_placed_num_node >= 0xffffffffu)
    coll_cache_ptr->EnsureNidToBlock();
  const bool list_on_device = coll_cache_ptr->_nid_to_block == nullptr;
  const size_t num_total_nodes =
      list_on_device ? (size_t)coll_cache_ptr->_placed_num_node : coll_cache_ptr->_nid_to_block->Shape()[0];
  _num_total_nodes = num_total_nodes;
  Timer t;

  _device_cache_data.assign(_num_location, nullptr);
  _device_cache_data[_cpu_location_id] = cpu_data;

  // 1. keys this GPU caches (ascending key order), from the placement
  _new_hash_table = new CacheEntryManager;
  _new_hash_table->_device_id = gpu_ctx.device_id;
  TensorPtr *keys_for_each_source = _new_hash_table->_keys_for_each_src;
  const size_t num_block = coll_cache_ptr->_block_access_advise->Shape()[1];
  TensorPtr advise_line = Tensor::FromBlob(
      coll_cache_ptr->_block_access_advise->Ptr<uint8_t>() + (size_t)location_id * num_block, kU8, {num_block},
      CPU_CLIB(), "advise_line");
  TensorPtr cache_node_list;  // on the device, ascending
  if (list_on_device) {
    // the bitmap the list comes from is what the first refresh needs to know of this placement: the table keeps it
    MemHandle cached_bits;
    cache_node_list = KeyListOnDevice(coll_cache_ptr->_placed_top_rows, coll_cache_ptr->_placed_extra,
                                      num_total_nodes, stream, &cached_bits);
    _new_hash_table->AdoptBuildBits(cached_bits);
  } else {
    CacheEntryManager::DetectKeysForAllSource(coll_cache_ptr->_nid_to_block, advise_line, location_id,
                                              coll_cache_ptr->_block_density, num_total_nodes, keys_for_each_source,
                                              (int)RunConfig::num_device);
  }
  const size_t num_cached_nodes =
      list_on_device ? cache_node_list->NumItem() : keys_for_each_source[location_id]->NumItem();
  const double detect_s = t.Passed();
  _new_hash_table->_remote_keys = Tensor::Empty(kI32, {0}, CPU_CLIB(), "");
  const size_t num_cpu_nodes = num_total_nodes - num_cached_nodes;

  // 2. cache space: capacity leaves 0.1 % of the key space as slack for refresh (cache_context.cu:2473)
  _cache_space_capacity = (size_t)(num_total_nodes * (cache_percentage + 0.001));
  CHECK_LE(num_cached_nodes, _cache_space_capacity);
  _cache_nbytes = _cache_space_capacity * _row_bytes;
  _cache_nodes = num_cached_nodes;
  _device_cache_data_local_handle = _eager_gpu_mem_allocator(_cache_nbytes);
  _device_cache_data[_local_location_id] = _device_cache_data_local_handle->ptr();

  // 3. lookup table: flat (4 bytes per key of the key space) when that is small or when the reference would pick
  //    it (cache_context.cu:2489-2497), open addressing otherwise
  bool use_flat = TableSize(std::max<size_t>(num_cached_nodes, 2)) > num_total_nodes / 2 ||
                  num_total_nodes * sizeof(IdType) <= ((size_t)256 << 20);
  if (RunConfig::force_table_kind == 1) use_flat = true;
  if (RunConfig::force_table_kind >= 2) use_flat = false;
  if (RunConfig::key_map_mul != 0) {
    CHECK(RunConfig::force_table_kind != 1) << "sparse ids cannot index a flat table";
    use_flat = false;
  }
  // a flat entry packs (location << 28) + slot (cache_hashtable.h:20-28): beyond 2^28 slots only a bucket's 32-bit
  // slot field can name them all
  if (_cache_space_capacity > ((size_t)1 << 28)) {
    CHECK(RunConfig::force_table_kind != 1)
        << "a flat table addresses 2^28 cache slots, this cache has " << _cache_space_capacity;
    use_flat = false;
  }
  if (use_flat) {
    _new_hash_table->CreateFlat(_eager_gpu_mem_allocator, num_total_nodes, stream);
  } else {
    _new_hash_table->CreateHash(_eager_gpu_mem_allocator, std::max<size_t>(_cache_space_capacity, 1), num_total_nodes,
                                stream);
  }

  const double alloc_s = t.Passed() - detect_s;
  // 4. fill: rows of the cached keys host -> HBM in list order, slot = position in the list.  The copy is bound by
  //    the host link, which answers a grid of 128 workgroups a little faster than one that fills the chip (12.8 GB of
  //    512-byte rows: 0.235 against 0.243 s; 6.4 GB of 128-byte rows: 0.131 against 0.137 s; 64 and 1,024 workgroups
  //    are no better than the full grid).  (The table insert beside the copy, on a second stream, instead of behind
  //    it, was measured at 500M rows / 50M cached: the step went from 0.140 to 0.178 s, the link-bound copy kernel
  //    loses more than the insert takes.)
  double rows_s = 0;
  if (num_cached_nodes > 0) {
    if (!list_on_device)
      cache_node_list = Tensor::CopyToExternal(keys_for_each_source[location_id], _eager_gpu_mem_allocator,
                                               _trainer_ctx, stream);
    MemHandle st = _eager_gpu_mem_allocator(256);
    UGK_CALL(ugk_fill_u32(st->ptr<uint32_t>(), 0, 1, stream));
    UGK_CALL(ugk_gather_direct_u32(cpu_data, num_total_nodes, cache_node_list->CPtr<uint32_t>(), num_cached_nodes,
                                   _device_cache_data[_local_location_id], _row_bytes,
                                   PointerKind(cpu_data) == 1 ? RunConfig::fill_limit_block : 0u,  // 2: a table in HBM
                                   st->ptr<uint32_t>(), nullptr, stream));
    if (common::MinLogLevel() <= common::LogLevel::INFO) {  // the two parts of the step timed apart: one more wait
      UGK_CALL(ugk_stream_sync(stream));
      rows_s = t.Passed() - detect_s - alloc_s;
    }
    // (8-byte entries are keyed by the row: no id list)
    TensorPtr id_buffer;
    auto table_keys = RunConfig::key_map_mul == 0 || _new_hash_table->_table.kind == 3 ? cache_node_list
                      : list_on_device
                          ? _new_hash_table->RowsToTableKeys(cache_node_list, id_buffer, _eager_gpu_mem_allocator,
                                                             _trainer_ctx, stream)
                          : _new_hash_table->TableKeysToDevice(keys_for_each_source[location_id],
                                                               _eager_gpu_mem_allocator, _trainer_ctx, stream);
    _new_hash_table->InsertSeqOffWithLoc(table_keys, location_id, stream);
    uint32_t fill_status = 0;
    UGK_CALL(ugk_memcpy_async(&fill_status, st->ptr(), sizeof(fill_status), stream));
    UGK_CALL(ugk_stream_sync(stream));
    CHECK_EQ(fill_status, 0u) << "cache fill gathered a key outside the host table";
    _new_hash_table->CheckStatus(stream, "cache fill");
  }
  UGK_CALL(ugk_stream_sync(stream));
  const double fill_s = t.Passed() - detect_s - alloc_s;

  // 5. bookkeeping for refresh: cached key list and free slots [n_cached, capacity) (cache_context.cu:2577-2585)
  // (a list made on the device stays there until the host asks for it: CacheEntryManager::HostCachedKeys)
  if (list_on_device) _new_hash_table->_cached_keys_on_device = cache_node_list;
  else _new_hash_table->_cached_keys = keys_for_each_source[location_id];
  _new_hash_table->_cache_space_capacity = (IdType)_cache_space_capacity;
  _new_hash_table->cpu_location_id = _cpu_location_id;
  _new_hash_table->num_total_key = num_total_nodes;
  _new_hash_table->_free_offsets = Tensor::Empty(kI32, {_cache_space_capacity}, CPU_CLIB(), "free_offsets");
  _new_hash_table->_free_offsets->ForceScale(kI32, {_cache_space_capacity - num_cached_nodes}, CPU_CLIB(), "");
  for (size_t i = 0; i < _cache_space_capacity - num_cached_nodes; i++)
    _new_hash_table->_free_offsets->Ptr<IdType>()[i] = (IdType)(num_cached_nodes + i);
  // a refresh on the device works on bitmaps of the cached rows and of the taken slots: built now, the first such
  // refresh does not hold up, for the length of that build, the lookups that share its stream
  if (RunConfig::gpu_refresh && RunConfig::gpu_record)
    _new_hash_table->EnsureDeviceLists(_eager_gpu_mem_allocator, _trainer_ctx, stream);

  LOG(INFO) << "Asymm Coll cache (policy: " << (int)RunConfig::cache_policy << ") | local " << num_cached_nodes
            << " / " << num_total_nodes << " nodes ( " << ToPercentage(num_cached_nodes / (double)num_total_nodes)
            << "~" << ToPercentage(cache_percentage) << ") | cpu " << num_cpu_nodes << " / " << num_total_nodes
            << " | " << ToReadableSize(_cache_nbytes) << " | " << t.Passed() << " secs (key list " << detect_s
            << ", cache space + table " << alloc_s << ", rows + table insert " << fill_s << ", of which rows "
            << rows_s << ")";
  std::cout << "test_result:init:feat_nbytes=" << num_total_nodes * _row_bytes << "\n";
  std::cout << "test_result:init:cache_nbytes=" << _cache_nbytes << "\n";
}

// cache_context.cu:2601-2647
void CacheContext::build(std::function<MemHandle(size_t)> gpu_mem_allocator, int location_id,
                         std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_data, DataType dtype, size_t dim,
                         Context gpu_ctx, double cache_percentage, StreamHandle stream) {
  _coll_cache = coll_cache_ptr;
  _gpu_mem_allocator = gpu_mem_allocator;
  _trainer_ctx = gpu_ctx;
  _dtype = dtype;
  _dim = dim;
  _row_bytes = GetDataTypeBytes(dtype) * dim;
  _num_total_nodes = RunConfig::num_total_item;
  CHECK_NOTNULL(cpu_data);
  CHECK_GT(_row_bytes, (size_t)0);
  UGK_CALL(ugk_set_device(gpu_ctx.device_id));
  const int dev = gpu_ctx.device_id;
  _eager_gpu_mem_allocator = [dev](size_t nbytes) -> MemHandle { return EagerGPUAlloc(dev, nbytes); };

  CHECK(RunConfig::key_map_mul == 0 || (cache_percentage != 0 && cache_percentage != 1))
      << "sparse-id mode needs a partial cache (the direct-mapping paths index the table by key)";
  if (cache_percentage == 0) {
    return build_no_cache(location_id, coll_cache_ptr, cpu_data, dtype, dim, gpu_ctx, stream);
  } else if (cache_percentage == 1) {
    return build_full_cache(location_id, coll_cache_ptr, cpu_data, dtype, dim, gpu_ctx, RunConfig::num_total_item,
                            stream);
  } else if (_coll_cache->_block_access_advise) {
    build_with_advise_new_hash(location_id, coll_cache_ptr, cpu_data, dtype, dim, gpu_ctx, cache_percentage, stream);
  } else {
    LOG(FATAL) << "a partial cache needs a placement: call build_v2, which solves before it builds";
  }
}

// ---------------------------------------------------------------------------------------------------------
// ExtractSession
// ---------------------------------------------------------------------------------------------------------
ExtractSession::ExtractSession(std::shared_ptr<CacheContext> cache_ctx) : _cache_ctx(cache_ctx) {
  const int dev = _cache_ctx->_trainer_ctx.device_id;
  UGK_CALL(ugk_set_device(dev));
  UGK_CALL(ugk_stream_create(&_local_ext_stream));
  const auto &link_desc = RunConfig::coll_cache_link_desc;
  const int cpu_cus = link_desc.cpu_cu.empty() ? 0 : link_desc.cpu_cu[0];
  if (cpu_cus > 0) {
    UGK_CALL(ugk_stream_create_cu_masked(&_cpu_ext_stream, cpu_cus));
  } else {
    UGK_CALL(ugk_stream_create(&_cpu_ext_stream));
  }
  UGK_CALL(ugk_event_create(&_ev_classified));
  UGK_CALL(ugk_event_create(&_ev_local_done));
  UGK_CALL(ugk_event_create(&_ev_cpu_done));
  for (auto &e : _ev_t) UGK_CALL(ugk_event_create(&e));
  _state_handle = EagerGPUAlloc(dev, 256);
  uint32_t *state = _state_handle->ptr<uint32_t>();
  UGK_CALL(ugk_fill_u32(state, 0, 64, nullptr));
  UGK_CALL(ugk_stream_sync(nullptr));
  _state = state;
  _counts[0] = state + kStCounts0;
  _counts[1] = state + kStCounts1;
  _status = state + kStStatus;
  _mix_counts = PinnedHostAlloc((size_t)ugk_extract_mix_max_groups() * sizeof(uint64_t));
  _host_mirror_handle = PinnedHostAlloc(256);
  _host_mirror = _host_mirror_handle->ptr<uint32_t>();
  memset(_host_mirror, 0, 256);
  const auto &desc = RunConfig::coll_cache_link_desc;
  if (!desc.cpu_sm.empty()) _cpu_blocks = (unsigned)desc.cpu_sm[0];
  if (RunConfig::miss_stage_rows > 0 && !_cache_ctx->IsDirectMapping() && _cache_ctx->_row_bytes % 16 == 0 &&
      _cache_ctx->_num_total_nodes <= 0x100000000ull) {
    size_t entries = 1024;
    while (entries < RunConfig::miss_stage_rows) entries <<= 1;
    _stage_entries = entries;
    AllocStage(0, nullptr);
  }
  if (RunConfig::gpu_record) {
    const size_t rows = _cache_ctx->_num_total_nodes;
    _hot_counts = EagerGPUAlloc(dev, std::max<size_t>(rows, 1) * sizeof(uint32_t));
    UGK_CALL(ugk_fill_u32(_hot_counts->ptr<uint32_t>(), 0, rows, nullptr));
    if (RunConfig::gpu_refresh) {  // which rows have been counted at all: lets a placement skip the cold ones
      const size_t words = (std::max<size_t>(rows, 1) + 63) / 64;
      _hot_observed = EagerGPUAlloc(dev, words * 8);
      UGK_CALL(ugk_fill_u32(_hot_observed->ptr<uint32_t>(), 0, words * 2, nullptr));
    }
    const size_t cap = std::min<size_t>(std::max<size_t>(rows, 1), kHotDrainRows);
    _hot_entries = EagerGPUAlloc(dev, cap * sizeof(uint64_t));
    _hot_entries_host = PinnedHostAlloc(cap * sizeof(uint64_t));
    UGK_CALL(ugk_stream_create(&_record_stream));
    UGK_CALL(ugk_event_create(&_ev_rec_begin));
    UGK_CALL(ugk_event_create(&_ev_rec_done));
    UGK_CALL(ugk_event_create(&_ev_placed));
    UGK_CALL(ugk_stream_sync(nullptr));
  }
}

void ExtractSession::AllocStage(int which, StreamHandle stream) {
  const int dev = _cache_ctx->_trainer_ctx.device_id;
  _stage_rows[which] = EagerGPUAlloc(dev, _stage_entries * _cache_ctx->_row_bytes);
  _stage_owner[which] = EagerGPUAlloc(dev, _stage_entries * sizeof(uint64_t));
  UGK_CALL(ugk_fill_u32(_stage_owner[which]->ptr<uint32_t>(), 0, _stage_entries * 2, stream));
  UGK_CALL(ugk_stream_sync(stream));
  _stages[which].rows_dev = _stage_rows[which]->ptr();
  _stages[which].owner_dev = _stage_owner[which]->ptr<uint64_t>();
  _stages[which].mask = _stage_entries - 1;
}

const ugk_stage_t *ExtractSession::StageForRefresh(bool foreground, StreamHandle stream) {
  if (_stage_entries == 0) return nullptr;
  const int cur = _stage_active.load();
  if (foreground) return &_stages[cur];
  const int other = 1 - cur;
  if (_stages[other].rows_dev == nullptr) AllocStage(other, stream);
  _stage_active.store(other);  // lookups that start from here on file their rows in the other stage
  return &_stages[cur];        // readable once the lookups in flight at this point have finished
}

ExtractSession::~ExtractSession() {
  if (_record_stream) ugk_stream_destroy(_record_stream);
  if (_ev_rec_begin) ugk_event_destroy(_ev_rec_begin);
  if (_ev_rec_done) ugk_event_destroy(_ev_rec_done);
  if (_ev_placed) ugk_event_destroy(_ev_placed);
  ugk_stream_destroy(_local_ext_stream);
  ugk_stream_destroy(_cpu_ext_stream);
  ugk_event_destroy(_ev_classified);
  ugk_event_destroy(_ev_local_done);
  ugk_event_destroy(_ev_cpu_done);
  for (auto &e : _ev_t) ugk_event_destroy(e);
}

void ExtractSession::EnsureIdx(size_t num_nodes) {
  const size_t need = num_nodes * sizeof(ugk_idx_t);
  if (_idx_handle == nullptr || _idx_handle->nbytes() < need) {
    _idx_handle = nullptr;
    _idx_handle = _cache_ctx->_gpu_mem_allocator(need + need / 4 + 256);
    CHECK_NOTNULL(_idx_handle);
  }
}

void ExtractSession::CheckStatusWord(StreamHandle stream) const {
  if (_host_mirror[kMirError] == 0) return;  // common case: nothing to fetch from the device
  uint32_t st = 0;
  UGK_CALL(ugk_memcpy_async(&st, _status, sizeof(st), stream));
  UGK_CALL(ugk_stream_sync(stream));
  CHECK_EQ(st, 0u) << "extraction kernels reported status 0x" << std::hex << st << std::dec
                   << ((st & UGK_ST_KEY_OUT_OF_RANGE)
                           ? ": a key is outside the table it has to be read from (num_total_item=" +
                                 std::to_string(_cache_ctx->_num_total_nodes) + ")"
                           : "")
                   << ((st & UGK_ST_BAD_SEGMENT)
                           ? ": the offsets of a pooled lookup leave the list of ids, run backwards or do not span "
                             "it from 0 to the number of ids (or the rows they were made from are not in ascending "
                             "order inside [0, num_rows))"
                           : "");
}

static int GatherDirect(const void *src, uint64_t rows, const IdType *keys, size_t n, void *out, size_t rb,
                        unsigned max_blocks, uint32_t *status, uint32_t *mirror, StreamHandle s) {
  return ugk_gather_direct_u32(src, rows, keys, n, out, rb, max_blocks, status, mirror, s);
}
static int GatherDirect(const void *src, uint64_t rows, const Id64Type *keys, size_t n, void *out, size_t rb,
                        unsigned max_blocks, uint32_t *status, uint32_t *mirror, StreamHandle s) {
  return ugk_gather_direct_i64(src, rows, keys, n, out, rb, max_blocks, status, mirror, s);
}
static int GatherScatter(const void *src, uint64_t rows, const IdType *keys, const uint32_t *dst, size_t n, void *out,
                         uint64_t out_rows, size_t rb, unsigned max_blocks, uint32_t *status, uint32_t *mirror,
                         StreamHandle s) {
  return ugk_gather_scatter_u32(src, rows, keys, dst, n, out, out_rows, rb, max_blocks, status, mirror, s);
}
static int GatherScatter(const void *src, uint64_t rows, const Id64Type *keys, const uint32_t *dst, size_t n, void *out,
                         uint64_t out_rows, size_t rb, unsigned max_blocks, uint32_t *status, uint32_t *mirror,
                         StreamHandle s) {
  return ugk_gather_scatter_i64(src, rows, keys, dst, n, out, out_rows, rb, max_blocks, status, mirror, s);
}
static int Classify(ugk_table_t t, const IdType *keys, size_t n, uint64_t host_rows, const uint32_t *dst_map,
                    ugk_idx_t *idx, uint32_t *c, uint32_t *next, uint32_t *st, uint32_t *mirror, StreamHandle s) {
  return ugk_classify_u32(t, keys, n, host_rows, dst_map, idx, c, next, st, mirror, s);
}
static int Classify(ugk_table_t t, const Id64Type *keys, size_t n, uint64_t host_rows, const uint32_t *dst_map,
                    ugk_idx_t *idx, uint32_t *c, uint32_t *next, uint32_t *st, uint32_t *mirror, StreamHandle s) {
  return ugk_classify_i64(t, keys, n, host_rows, dst_map, idx, c, next, st, mirror, s);
}
static int Dedup(const IdType *keys, size_t n, void *ws, size_t ws_bytes, uint32_t epoch, IdType *uniq, uint32_t *inv,
                 uint32_t *rep, uint32_t *nu, uint32_t *nu_host, StreamHandle s) {
  return ugk_dedup_u32(keys, n, ws, ws_bytes, epoch, uniq, inv, rep, nu, nu_host, s);
}
static int Dedup(const Id64Type *keys, size_t n, void *ws, size_t ws_bytes, uint32_t epoch, Id64Type *uniq,
                 uint32_t *inv, uint32_t *rep, uint32_t *nu, uint32_t *nu_host, StreamHandle s) {
  return ugk_dedup_i64(keys, n, ws, ws_bytes, epoch, uniq, inv, rep, nu, nu_host, s);
}

static int Record(const IdType *keys, size_t n, uint64_t mul, uint64_t mask, uint32_t *counts, uint64_t rows,
                  uint64_t *observed, uint32_t *st, uint32_t *mirror, StreamHandle s) {
  return ugk_record_u32(keys, n, mul, mask, counts, rows, observed, st, mirror, s);
}
static int Record(const Id64Type *keys, size_t n, uint64_t mul, uint64_t mask, uint32_t *counts, uint64_t rows,
                  uint64_t *observed, uint32_t *st, uint32_t *mirror, StreamHandle s) {
  return ugk_record_i64(keys, n, mul, mask, counts, rows, observed, st, mirror, s);
}

// FreqRecorder::Record of this batch on the device (freq_recorder.cc:227-253).  It runs on a stream of its own behind
// an event on the caller's stream (the point where the keys are ready), so it overlaps the gathers; JoinRecord makes
// the caller's stream wait for it before the lookup returns (the keys belong to the caller again after that).
// RecordBegin marks that point and says whether this lookup is counted at all; the extraction kernels are launched
// next, and only then RecordLaunch enqueues the counting: its handful of API calls then run while the GPU already
// works on the batch instead of in front of it.  A lookup that the caller is recording into a HIP graph is counted
// by a record kernel on the caller's own stream instead (RecordPlan in the header says why).
ExtractSession::RecordPlan ExtractSession::RecordBegin(StreamHandle stream) {
  _record_pending = false;
  RecordPlan plan;
  if (!_hot_counts) return plan;
  int capturing = 0;
  UGK_CALL(ugk_stream_is_capturing(stream, &capturing));
  if (capturing == UGK_CAPTURE_QUERY_REFUSED) {
    // the runtime refuses the query where the stream may not be used at all (the legacy default stream while another
    // stream of the process records a graph): nothing is counted, and the launch that follows reports the misuse
    if (!_capture_query_refused_logged)
      LOG(WARNING) << "the capture state of the lookup's stream cannot be queried; this lookup is not counted";
    _capture_query_refused_logged = true;
    return plan;
  }
  if ((_num_lookups++ % RunConfig::gpu_record_every) != 0) return plan;
  if (capturing) {
    // A lookup that the caller records into a HIP graph: the record stream and the events of this session stay out of
    // that graph (see RecordPlan).  Every replay counts the keys the replayed lookup reads.
    plan.kind = RecordPlan::kCallersStream;
    plan.stream = stream;
    _counted_on_callers_stream.store(true);
    return plan;
  }
  UGK_CALL(ugk_event_record(_ev_rec_begin, stream));
  plan.kind = RecordPlan::kRecordStream;
  plan.after = _ev_rec_begin;
  return plan;
}

template <typename KeyT>
void ExtractSession::RecordLaunch(const KeyT *nodes, size_t num_nodes, const RecordPlan &plan) {
  if (plan.kind == RecordPlan::kNone) return;
  num_nodes = std::min(num_nodes, _record_limit);
  if (num_nodes == 0) return;
  if (plan.kind == RecordPlan::kCallersStream) {
    // in stream order behind the extraction, nothing to join
    UGK_CALL(Record(nodes, num_nodes, RunConfig::key_map_inv, RunConfig::key_map_mask, _hot_counts->ptr<uint32_t>(),
                    _cache_ctx->_num_total_nodes, ObservedBits(), _status, _host_mirror, plan.stream));
    return;
  }
  std::lock_guard<std::mutex> guard(_enqueue_mu);  // not in the middle of a placement's passes
  _keys_counted_since += num_nodes;
  UGK_CALL(ugk_stream_wait_event(_record_stream, plan.after));
  UGK_CALL(Record(nodes, num_nodes, RunConfig::key_map_inv, RunConfig::key_map_mask, _hot_counts->ptr<uint32_t>(),
                  _cache_ctx->_num_total_nodes, ObservedBits(), _status, _host_mirror, _record_stream));
  UGK_CALL(ugk_event_record(_ev_rec_done, _record_stream));
  _record_pending = true;
}

// the counting behind an event the caller has already recorded on its stream (the classify kernel's)
template <typename KeyT>
void ExtractSession::RecordKeys(const KeyT *nodes, size_t num_nodes, StreamHandle stream, void *after) {
  _record_pending = false;
  if (!_hot_counts || (_num_lookups++ % RunConfig::gpu_record_every) != 0) return;
  (void)stream;
  RecordPlan plan;
  plan.kind = RecordPlan::kRecordStream;
  plan.after = after;
  RecordLaunch(nodes, num_nodes, plan);
}

void ExtractSession::JoinRecord(StreamHandle stream) {
  if (!_record_pending) return;
  UGK_CALL(ugk_stream_wait_event(stream, _ev_rec_done));
  _record_pending = false;
}

// the same for a blocking lookup, after its own wait: the counting has normally finished by then, and waiting for
// its event on the host keeps a cross-stream dependency out of the caller's stream
void ExtractSession::JoinRecordOnHost() {
  if (!_record_pending) return;
  UGK_CALL(ugk_event_sync(_ev_rec_done));
  _record_pending = false;
}

bool ExtractSession::PlaceOnDevice(size_t num_cached, uint64_t *in_new_bits, uint64_t *scratch_bits,
                                   const uint64_t *keep_bits, void *rank_ws, bool reset_counts, const DiffCount *diff,
                                   StreamHandle stream) {
  CHECK_NOTNULL(_hot_counts) << "placement on the device needs the device-side hotness counters (COLL_GPU_RECORD=1)";
  const size_t rows = _cache_ctx->_num_total_nodes;
  std::lock_guard<std::mutex> no_drain(_drain_mu);
  std::lock_guard<std::mutex> guard(_enqueue_mu);
  const bool replays_count = _counted_on_callers_stream.load();
  if (replays_count) {
    // replays of a graph that counts run on the caller's stream, not on the record stream: the passes below start
    // behind whatever that stream holds at this point (a refresh that shares the stream of the replays, the usual
    // case, is thereby ordered against all of them; replays launched from elsewhere while the passes run are not)
    UGK_CALL(ugk_event_record(_ev_placed, stream));
    UGK_CALL(ugk_stream_wait_event(_record_stream, _ev_placed));
  }
  // every counting launch enqueued so far is in this sum, and on the record stream in front of the passes
  const uint64_t counted = _keys_counted_since.exchange(0);
  const uint64_t bound = _observed_known == UINT64_MAX ? UINT64_MAX : _observed_known + counted;
  if (_observed_known != UINT64_MAX) _observed_known = bound;  // stands until the placement's own count is read
  const bool few_observed = diff != nullptr && keep_bits == nullptr && !replays_count && ObservedBits() != nullptr &&
                            num_cached > 0 && num_cached < rows && bound < num_cached;
  if (few_observed) {
    UGK_CALL(ugk_rank_place_observed(_hot_counts->ptr<uint32_t>(), rows, num_cached, rank_ws, in_new_bits,
                                     ObservedBits(), reset_counts ? 1 : 0, diff->cached_bits, diff->evict_ws,
                                     diff->insert_ws, diff->totals_host, diff->status_dev, _record_stream));
  } else {
    UGK_CALL(ugk_rank_place_keep(_hot_counts->ptr<uint32_t>(), rows, num_cached, rank_ws, in_new_bits, scratch_bits,
                                 ObservedBits(), keep_bits, reset_counts ? 1 : 0, _record_stream));
    // how many rows are observed now: what lets the next placement skip the counters
    if (diff && !reset_counts && ObservedBits())
      UGK_CALL(ugk_bitmap_count(ObservedBits(), nullptr, 0, rows, diff->evict_ws, diff->totals_host + 2,
                                _record_stream));
  }
  _observed_word = diff && ObservedBits() ? diff->totals_host + 2 : nullptr;
  _placement_reset = reset_counts;
  UGK_CALL(ugk_event_record(_ev_placed, _record_stream));
  UGK_CALL(ugk_stream_wait_event(stream, _ev_placed));
  return few_observed;
}

void ExtractSession::PlacementWaitedFor() {
  std::lock_guard<std::mutex> guard(_enqueue_mu);
  if (_placement_reset) _observed_known = 0;  // keys counted while the passes ran are in _keys_counted_since
  else if (_observed_word) _observed_known = *_observed_word;
  else _observed_known = UINT64_MAX;
  _observed_word = nullptr;
}

void ExtractSession::SeedHotness(const FreqEntry *entries, size_t num_entries) {
  CHECK_NOTNULL(_hot_counts) << "seeding needs the device-side hotness counters (COLL_GPU_RECORD=1)";
  if (num_entries == 0) return;
  CHECK_NOTNULL(entries);
  UGK_CALL(ugk_set_device(_cache_ctx->_trainer_ctx.device_id));
  static_assert(sizeof(FreqEntry) == sizeof(uint64_t), "an entry is one (count << 32 | row) word");
  const size_t cap = _hot_entries->nbytes() / sizeof(uint64_t);
  std::lock_guard<std::mutex> guard(_drain_mu);
  _keys_counted_since += num_entries;
  uint64_t *dev_list = _hot_entries->ptr<uint64_t>();
  auto *host_list = _hot_entries_host->ptr<FreqEntry>();
  for (size_t first = 0; first < num_entries; first += cap) {
    const size_t cur = std::min(cap, num_entries - first);
    memcpy(host_list, entries + first, cur * sizeof(FreqEntry));  // pinned staging: the drain's own
    UGK_CALL(ugk_memcpy_async(dev_list, host_list, cur * sizeof(uint64_t), _record_stream));
    UGK_CALL(ugk_record_restore(dev_list, cur, _hot_counts->ptr<uint32_t>(), _cache_ctx->_num_total_nodes,
                                ObservedBits(), _status, _record_stream));
    UGK_CALL(ugk_stream_sync(_record_stream));
  }
  uint32_t st = 0;
  UGK_CALL(ugk_memcpy_async(&st, _status, sizeof(st), _record_stream));
  UGK_CALL(ugk_stream_sync(_record_stream));
  CHECK_EQ(st, 0u) << "seeding the hotness counters: a row is outside num_total_item=" << _cache_ctx->_num_total_nodes;
}

size_t ExtractSession::DrainHotness(FreqRecorder *recorder) {
  CHECK_NOTNULL(recorder);
  if (!_hot_counts) return 0;
  UGK_CALL(ugk_set_device(_cache_ctx->_trainer_ctx.device_id));
  const size_t rows = _cache_ctx->_num_total_nodes;
  const size_t cap = _hot_entries->nbytes() / sizeof(uint64_t);
  std::lock_guard<std::mutex> guard(_drain_mu);
  uint32_t *n_entries = _state + kStDrainEntries;       // device word, kept at zero between drains
  uint32_t *host_out = _host_mirror + kMirDrainCount;   // entries written, then "rows left over"
  uint64_t *dev_list = _hot_entries->ptr<uint64_t>();
  auto *host_list = _hot_entries_host->ptr<FreqEntry>();
  static_assert(sizeof(FreqEntry) == sizeof(uint64_t), "an entry is one (count << 32 | row) word");
  size_t moved = 0;
  recorder->BeginEntries();
  for (size_t first = 0; first < rows; first += cap) {
    const size_t cur = std::min(cap, rows - first);  // as many rows as the list has room for: nothing is left over
    UGK_CALL(ugk_record_drain(_hot_counts->ptr<uint32_t>(), first, cur, ObservedBits(), dev_list, (uint32_t)cap,
                              n_entries, host_out, _record_stream));
    UGK_CALL(ugk_stream_sync(_record_stream));
    const size_t got = host_out[0];
    CHECK_EQ(host_out[kMirDrainMore - kMirDrainCount], 0u);
    if (got == 0) continue;
    UGK_CALL(ugk_memcpy_async(host_list, dev_list, got * sizeof(uint64_t), _record_stream));
    UGK_CALL(ugk_stream_sync(_record_stream));
    recorder->AddEntries(host_list, got);
    moved += got;
  }
  {
    std::lock_guard<std::mutex> placed(_enqueue_mu);
    _observed_known = 0;  // every counter was handed over; what is counted from here on is in _keys_counted_since
  }
  return moved;
}

// Deduplication in front of the extraction: the distinct keys of the batch, the index of the first occurrence of
// each (where its row is gathered to) and, per input position, which distinct key it is.  One blocking wait: the
// host needs the number of distinct keys to size the launches that follow.
template <typename KeyT>
size_t ExtractSession::DedupKeys(const KeyT *nodes, size_t num_nodes, StreamHandle stream) {
  const size_t ws_bytes = ugk_dedup_workspace_bytes(num_nodes);
  auto alloc = _cache_ctx->_gpu_mem_allocator;
  if (_dedup_ws == nullptr || _dedup_ws_bytes < ws_bytes) {
    _dedup_ws = nullptr;
    const size_t grown = ugk_dedup_workspace_bytes(num_nodes + num_nodes / 4);
    _dedup_ws = alloc(grown);
    CHECK_NOTNULL(_dedup_ws);
    _dedup_ws_bytes = grown;  // the allocator may hand out more; the layout follows what was asked for and zero-filled
    UGK_CALL(ugk_fill_u32(_dedup_ws->ptr<uint32_t>(), 0, grown / 4, stream));
    _dedup_epoch = 0;
  }
  if (_dedup_out == nullptr || _dedup_cap < num_nodes) {
    _dedup_out = nullptr;
    _dedup_cap = (num_nodes + num_nodes / 4 + 63) / 64 * 64;
    _dedup_out = alloc(_dedup_cap * 16);
    CHECK_NOTNULL(_dedup_out);
  }
  if (++_dedup_epoch == 0) {  // the tag wrapped: stale entries of 2^32 batches ago must not read as current
    UGK_CALL(ugk_fill_u32(_dedup_ws->ptr<uint32_t>(), 0, _dedup_ws_bytes / 4, stream));
    _dedup_epoch = 1;
  }
  uint32_t *n_unique = _state + kStNumUnique;
  UGK_CALL(ugk_fill_u32(n_unique, 0, 1, stream));
  UGK_CALL(Dedup(nodes, num_nodes, _dedup_ws->ptr<void>(), _dedup_ws_bytes, _dedup_epoch, DedupUnique<KeyT>(),
                 DedupInverse(), DedupRep(), n_unique, _host_mirror + kMirNumUnique, stream));
  UGK_CALL(ugk_stream_sync(stream));
  const size_t nu = _host_mirror[kMirNumUnique];
  CHECK(nu >= 1 && nu <= num_nodes) << "deduplication produced " << nu << " keys from " << num_nodes;
  return nu;
}

static int ExtractMix(ugk_table_t t, const IdType *keys, size_t n, const void *cache, uint64_t cache_rows,
                      const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *st, uint32_t *mirror,
                      uint64_t *counts, uint32_t *groups, uint32_t hint, const ugk_stage_t *stage, StreamHandle s) {
  if (stage)
    return ugk_extract_mix_staged_u32(t, keys, n, cache, cache_rows, host, host_rows, out, rb, st, mirror, counts,
                                      groups, hint, *stage, s);
  return ugk_extract_mix_u32(t, keys, n, cache, cache_rows, host, host_rows, out, rb, st, mirror, counts, groups, hint,
                             s);
}
static int ExtractMix(ugk_table_t t, const Id64Type *keys, size_t n, const void *cache, uint64_t cache_rows,
                      const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *st, uint32_t *mirror,
                      uint64_t *counts, uint32_t *groups, uint32_t hint, const ugk_stage_t *stage, StreamHandle s) {
  if (stage)
    return ugk_extract_mix_staged_i64(t, keys, n, cache, cache_rows, host, host_rows, out, rb, st, mirror, counts,
                                      groups, hint, *stage, s);
  return ugk_extract_mix_i64(t, keys, n, cache, cache_rows, host, host_rows, out, rb, st, mirror, counts, groups, hint,
                             s);
}

static int ExtractPool(ugk_table_t t, const IdType *ids, const int64_t *seg_off, const float *w, size_t n_rows,
                       uint64_t nnz, int combiner, int elem_bytes, float max_norm, const void *cache,
                       uint64_t cache_rows, const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *st,
                       uint32_t *mirror, uint64_t *counts, uint32_t *groups, StreamHandle s) {
  return ugk_extract_pool_clip_u32(t, ids, seg_off, w, n_rows, nnz, combiner, elem_bytes, max_norm, cache, cache_rows,
                                   host, host_rows, out, rb, st, mirror, counts, groups, s);
}
static int ExtractPool(ugk_table_t t, const Id64Type *ids, const int64_t *seg_off, const float *w, size_t n_rows,
                       uint64_t nnz, int combiner, int elem_bytes, float max_norm, const void *cache,
                       uint64_t cache_rows, const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *st,
                       uint32_t *mirror, uint64_t *counts, uint32_t *groups, StreamHandle s) {
  return ugk_extract_pool_clip_i64(t, ids, seg_off, w, n_rows, nnz, combiner, elem_bytes, max_norm, cache, cache_rows,
                                   host, host_rows, out, rb, st, mirror, counts, groups, s);
}

static int NonLocalFlags(ugk_table_t t, const IdType *keys, size_t n, uint64_t *flags, StreamHandle s) {
  return ugk_nonlocal_flags_u32(t, keys, n, flags, s);
}
static int NonLocalFlags(ugk_table_t t, const Id64Type *keys, size_t n, uint64_t *flags, StreamHandle s) {
  return ugk_nonlocal_flags_i64(t, keys, n, flags, s);
}
static int SelectKeys(const IdType *keys, const uint32_t *sel, size_t m, IdType *out, StreamHandle s) {
  return ugk_select_keys_u32(keys, sel, m, out, s);
}
static int SelectKeys(const Id64Type *keys, const uint32_t *sel, size_t m, Id64Type *out, StreamHandle s) {
  return ugk_select_keys_i64(keys, sel, m, out, s);
}

// COLL_SKIP_LOCAL=1 (cache_context.cu:728-741), a measurement aid of the reference: the keys the local cache serves
// are dropped in front of the extraction, the others keep their order and are extracted into the first rows of the
// output, so that the traffic of the other sources can be timed on its own.  Returns how many keys are left; they are
// in SkipKeys().  One blocking wait, for that count (the reference waits there as well).
template <typename KeyT>
size_t ExtractSession::SelectNonLocal(const ugk_table_t &table, const KeyT *nodes, size_t num_nodes,
                                      StreamHandle stream) {
  const size_t words = (num_nodes + 63) / 64;
  const size_t need = words * 8 + num_nodes * 4 + num_nodes * sizeof(KeyT) + ugk_bitmap_workspace_bytes() + 64;
  if (_skip_handle == nullptr || _skip_handle->nbytes() < need) {
    _skip_handle = nullptr;
    _skip_handle = _cache_ctx->_gpu_mem_allocator(need + need / 4);
    CHECK_NOTNULL(_skip_handle);
  }
  // [bitmap | bitmap workspace | compacted keys | selected positions], each 8-byte aligned
  char *base = _skip_handle->ptr<char>();
  uint64_t *flags = reinterpret_cast<uint64_t *>(base);
  void *bm_ws = base + words * 8;
  _skip_keys = base + words * 8 + (ugk_bitmap_workspace_bytes() + 7) / 8 * 8;
  uint32_t *sel = reinterpret_cast<uint32_t *>(static_cast<char *>(_skip_keys) + num_nodes * sizeof(KeyT));
  UGK_CALL(NonLocalFlags(table, nodes, num_nodes, flags, stream));
  UGK_CALL(ugk_bitmap_count(flags, nullptr, 0, num_nodes, bm_ws, _host_mirror + kMirSkipCount, stream));
  UGK_CALL(ugk_stream_sync(stream));
  const size_t m = _host_mirror[kMirSkipCount];
  CHECK_LE(m, num_nodes);
  if (m == 0) return 0;
  UGK_CALL(ugk_bitmap_emit(flags, nullptr, 0, num_nodes, bm_ws, sel, m, stream));
  UGK_CALL(SelectKeys(nodes, sel, m, static_cast<KeyT *>(_skip_keys), stream));
  return m;
}

void ExtractSession::NoteOutput(const void *output, size_t nbytes) {
  int hint = _out_hint;
  if (_out_ptr[(_out_next + kOutRing - 1) % kOutRing] != output || _out_bytes[(_out_next + kOutRing - 1) % kOutRing] != nbytes) {
    _out_ptr[_out_next] = output;
    _out_bytes[_out_next] = nbytes;
    _out_next = (_out_next + 1) % kOutRing;
    // bytes of the distinct buffers among the last few outputs (the ring only grows on a change of buffer, so one
    // reused buffer occupies one entry)
    size_t distinct = 0;
    for (int i = 0; i < kOutRing; i++) {
      bool seen = _out_ptr[i] == nullptr;
      for (int j = 0; j < i && !seen; j++) seen = _out_ptr[j] == _out_ptr[i];
      if (!seen) distinct += _out_bytes[i];
    }
    hint = distinct > ((size_t)192 << 20) ? UGK_OUTPUT_STREAMS : UGK_OUTPUT_AUTO;
  }
  // the hint is a thread's own in the kernel library: set it on every call that may come from another thread than
  // the last one did, which costs a store
  UGK_CALL(ugk_set_output_hint(hint));
  _out_hint = hint;
}

// group sizes of the last fused launch: the sum of the words its workgroups left in pinned host memory
void ExtractSession::SumMixCounts() {
  const uint64_t *w = _mix_counts->ptr<uint64_t>();
  uint64_t local = 0, others = 0;
  for (uint32_t g = 0; g < _mix_groups; g++) {
    local += (uint32_t)w[g];
    others += w[g] >> 32;
  }
  _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL] = (uint32_t)local;
  _host_mirror[kMirGroupSizes + UGK_LOC_HOST] = (uint32_t)others;
}

// The wait of a blocking lookup.  By default a ticket written by a one-lane kernel behind the batch's kernels is polled
// in the pinned mirror: it turns up a few microseconds before a wait for the stream returns (COLL_SPIN_WAIT=0: wait for
// the stream, as the reference does).
void ExtractSession::WaitForBatch(StreamHandle stream) {
  if (RunConfig::spin_wait_us == 0) {
    UGK_CALL(ugk_stream_sync(stream));
    return;
  }
  if (++_ticket == 0) _ticket = 1;
  UGK_CALL(ugk_stream_sync_ticket(stream, _host_mirror + kMirTicket, _ticket, RunConfig::spin_wait_us));
}

// A lookup the refresh thread must wait for: counted from before it reads the table handle until its output is complete
// (blocking lookups) or until its kernels are enqueued on their stream (stream-ordered ones, which the refresh then
// finds by waiting for that stream).
struct ExtractSession::InFlight {
  ExtractSession *s;
  explicit InFlight(ExtractSession *session) : s(session) { s->_blocking_started.fetch_add(1); }
  ~InFlight() { s->_blocking_finished.fetch_add(1); }
};

// cache_context.cu:1199-1794
template <typename KeyT>
void ExtractSession::ExtractFeatImpl(const KeyT *nodes, size_t num_nodes, void *output, StreamHandle stream,
                                     uint64_t task_key) {
  CacheContext *ctx = _cache_ctx.get();
  auto profiler = ctx->_coll_cache ? ctx->_coll_cache->_profiler : nullptr;
  const size_t rb = ctx->_row_bytes;
  const size_t nbytes = num_nodes * rb;
  InFlight in_flight(this);  // from before the first kernel reads the table until the output is complete
  Wait(stream);  // stream-ordered lookups still in flight share the mirror words this call reads
  _group_offset[0] = 0;
  if (num_nodes == 0) {
    _group_offset[1] = _group_offset[2] = 0;
    ctx->progress.fetch_add(1);
    return;
  }
  CHECK_NOTNULL(nodes);
  CHECK_NOTNULL(output);
  NoteOutput(output, nbytes);

  // with deduplication the extraction proper runs over the distinct keys and writes each row where the key first
  // occurs; the duplicates are filled in from there at the end
  const size_t num_input = num_nodes;
  const KeyT *input_nodes = nodes;
  const uint32_t *dst_map = nullptr, *inverse = nullptr;
  float ms_dedup = 0;
  const bool skip_local = !ctx->IsDirectMapping() && GetEnv("COLL_SKIP_LOCAL") == "1";
  if (RunConfig::dedup_keys && num_nodes >= RunConfig::dedup_min_keys && !_skip_dedup && !skip_local) {
    UGK_CALL(ugk_event_record(_ev_t[2], stream));
    const size_t nu = DedupKeys(nodes, num_nodes, stream);
    UGK_CALL(ugk_event_record(_ev_t[3], stream));
    nodes = DedupUnique<KeyT>();
    dst_map = DedupRep();
    inverse = DedupInverse();
    num_nodes = nu;
  }

  if (ctx->IsDirectMapping()) {
    // fast path: no table, one gather.  Full cache reads HBM with the whole chip; no cache reads the host table
    // with the host-link budget.
    CHECK_EQ(ctx->_num_location, 1);
    const bool from_host = ctx->_cpu_location_id != -1;
    // the logged combine time: a host timer around launch and wait, as in the reference (Timer around Combine + StreamSync,
    // cache_context.cu:1206-1216, 1312-1315), or with COLL_KERNEL_EVENTS=1 the kernel's duration from an event pair on its
    // stream, which costs 1.9 us per step
    const RecordPlan keys_ready = RecordBegin(stream);
    const bool events = RunConfig::kernel_events;
    Timer t_host;
    if (events) UGK_CALL(ugk_event_record(_ev_t[0], stream));
    if (dst_map == nullptr) {
      UGK_CALL(GatherDirect(ctx->_device_cache_data[0], ctx->_num_total_nodes, nodes, num_nodes, output, rb,
                            from_host ? _cpu_blocks : 0, _status, _host_mirror, stream));
    } else {
      UGK_CALL(GatherScatter(ctx->_device_cache_data[0], ctx->_num_total_nodes, nodes, dst_map, num_nodes, output,
                             num_input, rb, from_host ? _cpu_blocks : 0, _status, _host_mirror, stream));
    }
    if (events) UGK_CALL(ugk_event_record(_ev_t[1], stream));
    RecordLaunch(input_nodes, num_input, keys_ready);
    if (dst_map) UGK_CALL(ugk_replicate_rows(output, rb, inverse, dst_map, num_input, stream));
    WaitForBatch(stream);
    const double host_time = t_host.Passed();
    JoinRecordOnHost();
    CheckStatusWord(stream);
    float combine_ms = 0;
    if (events) {
      // the ticket behind the batch can turn up before the runtime has seen the event in front of it complete
      UGK_CALL(ugk_event_sync(_ev_t[1]));
      UGK_CALL(ugk_event_elapsed_ms(_ev_t[0], _ev_t[1], &combine_ms));
    }
    const double combine_time = events ? combine_ms * 1e-3 : host_time;
    _group_offset[1] = from_host ? 0 : (uint32_t)num_nodes;
    _group_offset[2] = (uint32_t)num_nodes;
    if (profiler && task_key != 0xffffffffffffffffull) {
      profiler->LogStep(task_key, kLogL1FeatureBytes, nbytes);
      if (!from_host) {
        profiler->LogStep(task_key, kLogL3CacheCombineCacheTime, combine_time);
      } else {
        profiler->LogStep(task_key, kLogL1MissBytes, nbytes);
        profiler->LogStep(task_key, kLogL3CacheCombineMissTime, combine_time);
        profiler->LogEpochAdd(task_key, kLogEpochMissBytes, nbytes);
      }
      profiler->LogEpochAdd(task_key, kLogEpochFeatureBytes, nbytes);
    }
    ctx->progress.fetch_add(1);
    return;
  }

  const ugk_table_t table = ctx->_new_hash_table->Table();
  const void *cache = ctx->_device_cache_data[ctx->_local_location_id];
  const void *host = ctx->_device_cache_data[ctx->_cpu_location_id];
  const uint64_t cache_rows = ctx->_cache_space_capacity;
  const uint64_t host_rows = ctx->_num_total_nodes;

  if (skip_local) {
    num_nodes = SelectNonLocal(table, nodes, num_nodes, stream);
    nodes = static_cast<const KeyT *>(_skip_keys);
    if (num_nodes == 0) {
      _group_offset[1] = _group_offset[2] = 0;
      ctx->progress.fetch_add(1);
      return;
    }
  }
  const size_t nbytes_extracted = skip_local ? num_nodes * rb : nbytes;

  // the fused kernel moves 16-byte vectors; rows or buffers that are not multiples of 16 bytes take the factored
  // path, whose gathers fall back to narrower lanes
  const bool vec16 = (((uintptr_t)cache | (uintptr_t)host | (uintptr_t)output | (uintptr_t)rb) & 15u) == 0;
  if (RunConfig::concurrent_link_impl == kDirectNoGroup && dst_map == nullptr && vec16) {
    // one fused lookup + gather kernel, source chosen per row (cache_context.cu:1295-1329).  The default here: the
    // host link is busy from the first wavefront on, with no classify pass and no cross-stream hand-off in front of
    // it, and since the link bounds a mixed batch it does not matter that host loads spread over the chip slow the
    // HBM loads next to them.
    const RecordPlan keys_ready = RecordBegin(stream);
    const bool events = RunConfig::kernel_events;
    Timer t_host;
    if (events) UGK_CALL(ugk_event_record(_ev_t[0], stream));
    // The hint caps the launch to a few workgroups, which is right for a batch of host rows only and three times too
    // slow for one that mostly hits: it is given where the share is known (the keys COLL_SKIP_LOCAL selected all come
    // from outside the cache), not guessed from the previous batch.
    const uint32_t hint = skip_local ? (uint32_t)num_nodes : UGK_HINT_UNKNOWN;
    UGK_CALL(ExtractMix(table, nodes, num_nodes, cache, cache_rows, host, host_rows, output, rb, _status,
                        _host_mirror, _mix_counts->ptr<uint64_t>(), &_mix_groups, hint, NextStage(stream, false), stream));
    if (events) UGK_CALL(ugk_event_record(_ev_t[1], stream));
    RecordLaunch(input_nodes, num_input, keys_ready);
    WaitForBatch(stream);
    const double host_time = t_host.Passed();
    JoinRecordOnHost();
    CheckStatusWord(stream);
    SumMixCounts();
    const uint32_t n_local = _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL],
                   n_miss = _host_mirror[kMirGroupSizes + UGK_LOC_HOST];
    CHECK_EQ((size_t)n_local + n_miss, num_nodes);
    float mix_ms = (float)(host_time * 1e3);
    if (events) {
      UGK_CALL(ugk_event_sync(_ev_t[1]));  // see the direct-mapping branch
      UGK_CALL(ugk_event_elapsed_ms(_ev_t[0], _ev_t[1], &mix_ms));
    }
    _group_offset[1] = n_local;
    _group_offset[2] = (uint32_t)num_nodes;
    if (profiler && task_key != 0xffffffffffffffffull) {
      profiler->LogStep(task_key, kLogL1FeatureBytes, nbytes_extracted);
      profiler->LogStep(task_key, kLogL1MissBytes, (double)n_miss * rb);
      profiler->LogStep(task_key, kLogL3CacheCombineCacheTime, mix_ms * 1e-3);
      profiler->LogEpochAdd(task_key, kLogEpochFeatureBytes, nbytes_extracted);
      profiler->LogEpochAdd(task_key, kLogEpochMissBytes, (double)n_miss * rb);
    }
    ctx->progress.fetch_add(1);
    return;
  }

  // classify + partition on the caller's stream, then one gather per source
  EnsureIdx(num_nodes);
  ugk_idx_t *idx = _idx_handle->ptr<ugk_idx_t>();
  uint32_t *cur = _counts[_cur], *next = _counts[_cur ^ 1];
  bool joined_on_host = false;
  UGK_CALL(ugk_event_record(_ev_t[0], stream));
  UGK_CALL(Classify(table, nodes, num_nodes, host_rows, dst_map, idx, cur, next, _status, _host_mirror, stream));
  UGK_CALL(ugk_event_record(_ev_classified, stream));
  // the classify kernel is short and latency-bound: the counting starts behind it, beside the gathers
  RecordKeys(input_nodes, num_input, stream, _ev_classified);
  if (RunConfig::concurrent_link_impl != kNoConcurrentLink) {
    // factored extraction: two concurrent kernels that read their group bounds from the device-side counters.
    // A long host-link gather runs on the stream confined to a few CUs, so its slow loads do not clog the memory
    // pipelines the HBM gather needs; the HBM gather then stays on the caller's stream.  A short host-link gather
    // (decided from the previous batch) stays on the caller's stream right behind the classify kernel instead, which
    // saves the cross-stream hand-off on the critical path.
    // The HBM gather always runs on a library stream created non-blocking: the confined stream cannot be created
    // that way, so a caller passing the legacy null stream would otherwise see its HBM gather serialised behind
    // the host-link gather by the null stream's implicit synchronisation.
    if (_host_on_main) {
      UGK_CALL(ugk_gather_group(host, host_rows, idx, cur, UGK_LOC_HOST, num_nodes, output, num_input, rb,
                                _cpu_blocks_inline, _status, _host_mirror, stream));
      UGK_CALL(ugk_event_record(_ev_cpu_done, stream));
    } else {
      UGK_CALL(ugk_stream_wait_event(_cpu_ext_stream, _ev_classified));
      UGK_CALL(ugk_gather_group(host, host_rows, idx, cur, UGK_LOC_HOST, num_nodes, output, num_input, rb, _cpu_blocks,
                                _status, _host_mirror, _cpu_ext_stream));
      UGK_CALL(ugk_event_record(_ev_cpu_done, _cpu_ext_stream));
    }
    UGK_CALL(ugk_stream_wait_event(_local_ext_stream, _ev_classified));
    UGK_CALL(ugk_gather_group(cache, cache_rows, idx, cur, UGK_LOC_LOCAL, num_nodes, output, num_input, rb, 0,
                              _status, _host_mirror, _local_ext_stream));
    UGK_CALL(ugk_event_record(_ev_local_done, _local_ext_stream));
    // with nothing left to enqueue behind the gathers the host waits for their two events itself (below); only the
    // re-expansion of a deduplicated batch needs both groups complete inside the caller's stream
    joined_on_host = dst_map == nullptr;
    if (!joined_on_host) {
      if (!_host_on_main) UGK_CALL(ugk_stream_wait_event(stream, _ev_cpu_done));
      UGK_CALL(ugk_stream_wait_event(stream, _ev_local_done));
    }
  } else {
    // sequential: host group, then local group (cache_context.cu:1719-1792)
    UGK_CALL(ugk_gather_group(host, host_rows, idx, cur, UGK_LOC_HOST, num_nodes, output, num_input, rb, 0,
                              _status, _host_mirror, stream));
    UGK_CALL(ugk_event_record(_ev_cpu_done, stream));
    UGK_CALL(ugk_gather_group(cache, cache_rows, idx, cur, UGK_LOC_LOCAL, num_nodes, output, num_input, rb, 0,
                              _status, _host_mirror, stream));
    UGK_CALL(ugk_event_record(_ev_local_done, stream));
  }
  if (dst_map) UGK_CALL(ugk_replicate_rows(output, rb, inverse, dst_map, num_input, stream));
  // the blocking wait of the call; the gathers have written their group sizes (and the kernels any error flag) into
  // the pinned mirror, so no device-to-host copy is needed.  Waiting for the events of the two gather streams on the
  // host keeps two cross-stream dependencies out of the caller's stream, which cost more than the wait itself.
  if (joined_on_host) {
    UGK_CALL(ugk_event_sync(_ev_cpu_done));
    UGK_CALL(ugk_event_sync(_ev_local_done));
  } else {
    UGK_CALL(ugk_stream_sync(stream));
  }
  JoinRecordOnHost();
  const uint32_t n_local = _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL],
                 n_miss = _host_mirror[kMirGroupSizes + UGK_LOC_HOST];
  _cur ^= 1;
  CheckStatusWord(stream);
  CHECK_EQ((size_t)n_local + n_miss, num_nodes);
  _group_offset[1] = n_local;
  _group_offset[2] = (uint32_t)num_nodes;

  float ms_idx = 0, ms_miss = 0, ms_local = 0;
  UGK_CALL(ugk_event_elapsed_ms(_ev_t[0], _ev_classified, &ms_idx));
  UGK_CALL(ugk_event_elapsed_ms(_ev_classified, _ev_cpu_done, &ms_miss));
  if (RunConfig::concurrent_link_impl != kNoConcurrentLink) {
    UGK_CALL(ugk_event_elapsed_ms(_ev_classified, _ev_local_done, &ms_local));
    _host_on_main = ms_miss < 0.25f;  // placement of the next batch's host-link gather
  } else {
    UGK_CALL(ugk_event_elapsed_ms(_ev_cpu_done, _ev_local_done, &ms_local));
  }
  if (dst_map) UGK_CALL(ugk_event_elapsed_ms(_ev_t[2], _ev_t[3], &ms_dedup));
  ms_idx += ms_dedup;
  if (profiler && task_key != 0xffffffffffffffffull) {
    profiler->LogStep(task_key, kLogL1FeatureBytes, nbytes_extracted);
    profiler->LogStep(task_key, kLogL1MissBytes, (double)n_miss * rb);
    profiler->LogStep(task_key, kLogL1RemoteBytes, 0);
    profiler->LogStep(task_key, kLogL3CacheGetIndexTime, ms_idx * 1e-3);
    profiler->LogStep(task_key, kLogL3CacheCombineMissTime, ms_miss * 1e-3);
    profiler->LogStep(task_key, kLogL3CacheCombineRemoteTime, 0);
    profiler->LogStep(task_key, kLogL3CacheCombineCacheTime, ms_local * 1e-3);
  }
  ctx->progress.fetch_add(1);
}

template <typename KeyT>
void ExtractSession::ExtractFeatAsyncImpl(const KeyT *nodes, size_t num_nodes, void *output, StreamHandle stream) {
  CacheContext *ctx = _cache_ctx.get();
  const size_t rb = ctx->_row_bytes;
  if (num_nodes == 0) return;
  CHECK_NOTNULL(nodes);
  CHECK_NOTNULL(output);
  const bool dedup = RunConfig::dedup_keys && num_nodes >= RunConfig::dedup_min_keys;
  NoteOutput(output, num_nodes * rb);
  NoteAsyncStream(stream);  // before the first kernel is enqueued: a refresh that does not see the stream yet has
                            // finished its evictions before that kernel can start
  // Between reading the table handle and enqueueing the kernel that uses it this call is "in flight" on the host: a
  // refresh that swaps the table for a rebuilt one waits for the count before it waits for the stream and frees the old
  // buckets, so the kernel below never reads freed memory.
  InFlight enqueueing(this);
  if (ctx->IsDirectMapping() && !dedup) {
    const bool from_host = ctx->_cpu_location_id != -1;
    const RecordPlan keys_ready = RecordBegin(stream);
    UGK_CALL(GatherDirect(ctx->_device_cache_data[0], ctx->_num_total_nodes, nodes, num_nodes, output, rb,
                          from_host ? _cpu_blocks : 0, _status, _host_mirror, stream));
    RecordLaunch(nodes, num_nodes, keys_ready);
    JoinRecord(stream);
    _async_last_fused = false;
    _async_swap_counts = false;
    // what a blocking lookup would have read from the mirror
    _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL] = from_host ? 0 : (uint32_t)num_nodes;
    _host_mirror[kMirGroupSizes + UGK_LOC_HOST] = from_host ? (uint32_t)num_nodes : 0;
  } else if (!ctx->IsDirectMapping() && !dedup && RunConfig::concurrent_link_impl == kDirectNoGroup &&
             (((uintptr_t)ctx->_device_cache_data[ctx->_local_location_id] |
               (uintptr_t)ctx->_device_cache_data[ctx->_cpu_location_id] | (uintptr_t)output | (uintptr_t)rb) &
              15u) == 0) {
    const RecordPlan keys_ready = RecordBegin(stream);
    UGK_CALL(ExtractMix(ctx->_new_hash_table->Table(), nodes, num_nodes,
                        ctx->_device_cache_data[ctx->_local_location_id], ctx->_cache_space_capacity,
                        ctx->_device_cache_data[ctx->_cpu_location_id], ctx->_num_total_nodes, output, rb, _status,
                        _host_mirror, _mix_counts->ptr<uint64_t>(), &_mix_groups, UGK_HINT_UNKNOWN,
                        NextStage(stream, true), stream));
    RecordLaunch(nodes, num_nodes, keys_ready);
    JoinRecord(stream);
    _async_last_fused = true;
    _async_swap_counts = false;
  } else {
    Wait(stream);
    ExtractFeatImpl<KeyT>(nodes, num_nodes, output, stream, 0xffffffffffffffffull);
    return;
  }
  _async_pending++;
  _async_last_nodes = num_nodes;
}

template <typename KeyT>
size_t ExtractSession::ExtractUniqueImpl(const KeyT *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                                         StreamHandle stream, uint64_t task_key) {
  Wait(stream);
  if (num_nodes == 0) {
    ExtractFeatImpl<KeyT>(nodes, 0, output, stream, task_key);
    return 0;
  }
  CHECK_NOTNULL(nodes);
  CHECK_NOTNULL(output);
  CHECK_NOTNULL(inverse_out);
  const size_t nu = DedupKeys(nodes, num_nodes, stream);
  UGK_CALL(ugk_memcpy_async(inverse_out, DedupInverse(), num_nodes * sizeof(uint32_t), stream));
  _skip_dedup = true;
  ExtractFeatImpl<KeyT>(DedupUnique<KeyT>(), nu, output, stream, task_key);  // blocks: the copy above is done too
  _skip_dedup = false;
  return nu;
}

size_t ExtractSession::ExtractUnique(const IdType *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                                     StreamHandle stream, uint64_t task_key) {
  CHECK(RunConfig::key_map_mul == 0 || RunConfig::key_map_mask <= 0xffffffffull)
      << "sparse ids wider than 32 bits need the 64-bit lookup";
  return ExtractUniqueImpl<IdType>(nodes, num_nodes, output, inverse_out, stream, task_key);
}

size_t ExtractSession::ExtractUnique64(const Id64Type *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                                       StreamHandle stream, uint64_t task_key) {
  return ExtractUniqueImpl<Id64Type>(nodes, num_nodes, output, inverse_out, stream, task_key);
}

void ExtractSession::ExtractFeatAsync(const IdType *nodes, const size_t num_nodes, void *output,
                                      StreamHandle stream) {
  CHECK(RunConfig::key_map_mul == 0 || RunConfig::key_map_mask <= 0xffffffffull)
      << "sparse ids wider than 32 bits need the 64-bit lookup";
  ExtractFeatAsyncImpl<IdType>(nodes, num_nodes, output, stream);
}

void ExtractSession::ExtractFeatAsync64(const Id64Type *nodes, const size_t num_nodes, void *output,
                                        StreamHandle stream) {
  ExtractFeatAsyncImpl<Id64Type>(nodes, num_nodes, output, stream);
}

void ExtractSession::NoteAsyncStream(StreamHandle stream) {
  if (_async_any && stream == _async_stream_last) return;  // the common case costs a compare
  std::lock_guard<std::mutex> guard(_async_mu);
  if (std::find(_async_streams.begin(), _async_streams.end(), stream) == _async_streams.end())
    _async_streams.push_back(stream);
  _async_stream_last = stream;
  _async_any = true;
}

void ExtractSession::WaitForLookupsInFlight(bool foreground, double timeout_s, const StreamHandle *ordered_on) {
  if (!foreground) {
    // A lookup counts itself before it reads the table: one that is not counted yet starts after the evictions (or the
    // table swap) have completed.  Blocking lookups stay counted until their output is complete, stream-ordered ones
    // until their kernels are enqueued, which is why the streams are waited for after the count, not before.
    const size_t started = _blocking_started.load();
    Timer t0;
    while (_blocking_finished.load() < started) {
      if (t0.PassedSec() >= timeout_s) {
        LOG(ERROR) << "refresh: a lookup that started before the eviction has not returned after " << timeout_s
                   << " s; going on";
        break;
      }
      usleep(20);
    }
  }
  std::vector<StreamHandle> streams;
  {
    std::lock_guard<std::mutex> guard(_async_mu);
    streams = _async_streams;
  }
  for (StreamHandle s : streams)
    if (ordered_on == nullptr || s != *ordered_on) UGK_CALL(ugk_stream_sync(s));
}

void ExtractSession::Wait(StreamHandle stream) {
  if (_async_pending == 0) return;
  UGK_CALL(ugk_stream_sync(stream));
  if (stream == _stage_writer) _stage_writer_busy = false;
  CheckStatusWord(stream);
  if (_async_last_fused) SumMixCounts();
  uint32_t n_local = _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL], n_miss = _host_mirror[kMirGroupSizes + UGK_LOC_HOST];
  CHECK_EQ((size_t)n_local + n_miss, _async_last_nodes);
  if (_async_swap_counts) std::swap(n_local, n_miss);  // a pooled lookup of a table that is all in HBM
  _group_offset[0] = 0;
  _group_offset[1] = n_local;
  _group_offset[2] = (uint32_t)_async_last_nodes;
  _cache_ctx->progress.fetch_add(_async_pending);
  _async_pending = 0;
}

// the checks and the launch the blocking and the stream-ordered pooled lookup share; true if the one source of a
// direct mapping is the HBM copy (the kernel then counts its ids as "from the host table")
template <typename KeyT>
bool ExtractSession::LaunchPooled(const KeyT *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                                  size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream) {
  CacheContext *ctx = _cache_ctx.get();
  const size_t rb = ctx->_row_bytes;
  CHECK_NOTNULL(seg_off);
  CHECK_NOTNULL(output);
  CHECK(num_nodes == 0 || nodes != nullptr);
  CHECK(combiner >= 0 && combiner <= 2) << "combiner is 0 (sum), 1 (mean) or 2 (sqrtn)";
  CHECK(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == UGK_ELEM_BF16)
      << "rows are combined as fp32 (4), fp16 (2) or bfloat16 (UGK_ELEM_BF16) elements";
  CHECK(rb % 16 == 0 && rb <= 4096 && rb % (elem_bytes & 0xf) == 0)
      << "pooled lookups take rows of a multiple of 16 bytes up to 4096, not " << rb;
  NoteOutput(output, num_rows * rb);
  // without a table the id is the row and everything comes from the one source there is (HBM for a full cache, the
  // host table for none); otherwise the table decides per id, as in the fused extraction
  ugk_table_t table{};
  const void *cache = nullptr, *host = nullptr;
  uint64_t cache_rows = 0;
  const bool direct = ctx->IsDirectMapping();
  if (direct) {
    table.kind = 0;
    host = ctx->_device_cache_data[0];
  } else {
    table = ctx->_new_hash_table->Table();
    cache = ctx->_device_cache_data[ctx->_local_location_id];
    host = ctx->_device_cache_data[ctx->_cpu_location_id];
    cache_rows = ctx->_cache_space_capacity;
  }
  CHECK((((uintptr_t)cache | (uintptr_t)host | (uintptr_t)output) & 15u) == 0) << "pooled lookup: misaligned buffer";
  const RecordPlan keys_ready = RecordBegin(stream);
  UGK_CALL(ExtractPool(table, nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, _pool_max_norm, cache,
                       cache_rows, host, ctx->_num_total_nodes, output, rb, _status, _host_mirror,
                       _mix_counts->ptr<uint64_t>(), &_mix_groups, stream));
  if (num_nodes) RecordLaunch(nodes, num_nodes, keys_ready);
  return direct && ctx->_cpu_location_id == -1;
}

template <typename KeyT>
void ExtractSession::ExtractPooledImpl(const KeyT *nodes, const int64_t *seg_off, const float *weights,
                                       size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                                       StreamHandle stream, uint64_t task_key) {
  CacheContext *ctx = _cache_ctx.get();
  auto profiler = ctx->_coll_cache ? ctx->_coll_cache->_profiler : nullptr;
  const size_t rb = ctx->_row_bytes;
  InFlight in_flight(this);  // from before the kernel reads the table until the output is complete
  Wait(stream);
  _group_offset[0] = 0;
  if (num_rows == 0) {
    _group_offset[1] = _group_offset[2] = 0;
    ctx->progress.fetch_add(1);
    return;
  }
  Timer t_host;
  const bool all_from_hbm =
      LaunchPooled(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream);
  WaitForBatch(stream);
  const double host_time = t_host.Passed();
  JoinRecordOnHost();
  CheckStatusWord(stream);
  SumMixCounts();
  uint32_t n_local = _host_mirror[kMirGroupSizes + UGK_LOC_LOCAL], n_miss = _host_mirror[kMirGroupSizes + UGK_LOC_HOST];
  CHECK_EQ((size_t)n_local + n_miss, num_nodes);
  if (all_from_hbm) std::swap(n_local, n_miss);
  _group_offset[1] = n_local;
  _group_offset[2] = (uint32_t)num_nodes;
  if (profiler && task_key != 0xffffffffffffffffull) {
    profiler->LogStep(task_key, kLogL1FeatureBytes, (double)num_nodes * rb);
    profiler->LogStep(task_key, kLogL1MissBytes, (double)n_miss * rb);
    profiler->LogStep(task_key, kLogL3CacheCombineCacheTime, host_time);
    profiler->LogEpochAdd(task_key, kLogEpochFeatureBytes, (double)num_nodes * rb);
    profiler->LogEpochAdd(task_key, kLogEpochMissBytes, (double)n_miss * rb);
  }
  ctx->progress.fetch_add(1);
}

void ExtractSession::SegmentOffsets(const int64_t *sorted_rows, size_t num_entries, size_t num_rows, int64_t *seg_off,
                                    StreamHandle stream) {
  CHECK_NOTNULL(seg_off);
  CHECK(num_entries == 0 || sorted_rows != nullptr);
  UGK_CALL(ugk_segment_offsets_i64(sorted_rows, num_entries, num_rows, seg_off, _status, _host_mirror, stream));
}

// the stream-ordered form: kernel launches only, completed by Wait() like a stream-ordered plain lookup
template <typename KeyT>
void ExtractSession::ExtractPooledAsyncImpl(const KeyT *nodes, const int64_t *seg_off, const float *weights,
                                            size_t num_rows, size_t num_nodes, int combiner, int elem_bytes,
                                            void *output, StreamHandle stream) {
  if (num_rows == 0) return;
  NoteAsyncStream(stream);
  InFlight enqueueing(this);  // see ExtractFeatAsyncImpl
  _async_swap_counts =
      LaunchPooled(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream);
  JoinRecord(stream);
  _async_last_fused = true;
  _async_pending++;
  _async_last_nodes = num_nodes;
}

void ExtractSession::ExtractPooledAsync(const IdType *nodes, const int64_t *seg_off, const float *weights,
                                        size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                                        StreamHandle stream) {
  ExtractPooledAsyncImpl<IdType>(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream);
}

void ExtractSession::ExtractPooledAsync64(const Id64Type *nodes, const int64_t *seg_off, const float *weights,
                                          size_t num_rows, size_t num_nodes, int combiner, int elem_bytes,
                                          void *output, StreamHandle stream) {
  ExtractPooledAsyncImpl<Id64Type>(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream);
}

void ExtractSession::ExtractPooled(const IdType *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                                   size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream,
                                   uint64_t task_key) {
  ExtractPooledImpl<IdType>(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream, task_key);
}

void ExtractSession::ExtractPooled64(const Id64Type *nodes, const int64_t *seg_off, const float *weights,
                                     size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                                     StreamHandle stream, uint64_t task_key) {
  ExtractPooledImpl<Id64Type>(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output, stream,
                              task_key);
}

void ExtractSession::ExtractFeat(const IdType *nodes, const size_t num_nodes, void *output, StreamHandle stream,
                                 uint64_t task_key) {
  CHECK(RunConfig::key_map_mul == 0 || RunConfig::key_map_mask <= 0xffffffffull)
      << "sparse ids wider than 32 bits need the 64-bit lookup";
  ExtractFeatImpl<IdType>(nodes, num_nodes, output, stream, task_key);
}

void ExtractSession::ExtractFeat64(const Id64Type *nodes, const size_t num_nodes, void *output, StreamHandle stream,
                                   uint64_t task_key) {
  ExtractFeatImpl<Id64Type>(nodes, num_nodes, output, stream, task_key);
}

// ---------------------------------------------------------------------------------------------------------
// RefreshSession
// ---------------------------------------------------------------------------------------------------------
RefreshSession::~RefreshSession() {
  if (low_pri_stream) ugk_stream_destroy(low_pri_stream);
}

TensorPtr RefreshSession::Empty1DReuse(TensorPtr &preserved_buffer, DataType dtype, std::vector<size_t> shape,
                                       Context ctx) {
  CHECK_EQ(shape.size(), (size_t)1);
  if (preserved_buffer && preserved_buffer->CanForceScale(dtype, shape)) {
    preserved_buffer->ForceScale(dtype, shape, ctx, "");
    return preserved_buffer;
  }
  preserved_buffer = Tensor::EmptyExternal(dtype, shape, _cache_ctx->_eager_gpu_mem_allocator, ctx, "");
  return preserved_buffer;
}

TensorPtr RefreshSession::CopyTo1DReuse(TensorPtr &preserved_buffer, TensorPtr src, Context ctx,
                                        StreamHandle stream) {
  auto ret = Empty1DReuse(preserved_buffer, src->Type(), src->Shape(), ctx);
  UGK_CALL(ugk_memcpy_async(ret->MutableData(), src->Data(), src->NumBytes(), stream));
  UGK_CALL(ugk_stream_sync(stream));  // src is pageable host memory owned by the caller
  return ret;
}

// cache_context.cu:4045-4052.  The reference waits until `progress` has moved by one (or 20 s have passed); here the
// session knows which lookups are in flight, on whichever stream, so the wait is for exactly those and an idle cache
// is not waited for at all.
void RefreshSession::WaitForOneLookup(ExtractSession *session, bool foreground, const StreamHandle *ordered_on) {
  AnonymousBarrier::_refresh_instance->Wait();
  if (session) session->WaitForLookupsInFlight(foreground, 20.0, ordered_on);
}

void RefreshSession::CopyRowsIntoSlots(const uint32_t *rows_dev, const uint32_t *slots_dev, size_t num_rows,
                                       bool foreground, StreamHandle copy_stream, const ugk_stage_t *stage) {
  CacheContext *ctx = _cache_ctx.get();
  auto table = ctx->_new_hash_table;
  const Context gpu_ctx = ctx->_trainer_ctx;
  const int local = ctx->_local_location_id;
  const void *host = ctx->_device_cache_data[ctx->_cpu_location_id];
  void *cache = ctx->_device_cache_data[ctx->_local_location_id];
  // [0] error bits, [8] rows taken from the stage so far, [9] rows left for the link, [10] rows taken this time
  uint32_t *status = _status_handle->ptr<uint32_t>();
  // Rows that do not fill whole 128-byte lines share a line with the slot next door.  A lookup kernel that runs while
  // the copy does may hold such a line in the L2 of its XCD from reading the neighbour — the L2s of different XCDs only
  // agree at kernel boundaries — and would read the stale half once the table names the new row.  Those rows are
  // published only after every lookup that was in flight when their copy completed has finished.
  const bool rows_share_lines = ctx->_row_bytes % 128 != 0 || reinterpret_cast<uintptr_t>(cache) % 128 != 0;
  auto session = ctx->_coll_cache ? ctx->_coll_cache->session(local) : nullptr;
  // the rows of a list, or of a part of one, become visible to lookups: behind their copy on the same stream
  auto publish = [&](const uint32_t *rows, const uint32_t *slots, size_t n) {
    if (n == 0) return;
    if (!foreground && rows_share_lines && session) {
      UGK_CALL(ugk_stream_sync(copy_stream));
      session->WaitForLookupsInFlight(false, 20.0);
    }
    table->PublishRows(rows, slots, n, local, __publish_ids, ctx->_eager_gpu_mem_allocator, gpu_ctx, copy_stream);
  };
  if (foreground) {
    // Nothing runs beside a foreground refresh: one launch copies every row.  Without a stage all of them cross the host
    // link, on a capped grid: rows of 512 bytes and more cross it faster from 128 workgroups than from as many as the
    // rows would fill (56.9 against 52.7 GB/s).  With a stage most rows are read from HBM (they were missed by the last
    // few lookups, which filed them there), which wants the whole chip, so that launch is not capped and the few rows
    // the stage does not hold cross the link at the lower of the two rates.  One more launch publishes them.
    if (stage)
      UGK_CALL(ugk_gather_scatter_staged_u32(host, ctx->_num_total_nodes, rows_dev, slots_dev, num_rows, cache,
                                             ctx->_cache_space_capacity, ctx->_row_bytes, *stage, 0, status, status + 8,
                                             nullptr, nullptr, nullptr, nullptr, copy_stream));
    else
      UGK_CALL(ugk_gather_scatter_u32(host, ctx->_num_total_nodes, rows_dev, slots_dev, num_rows, cache,
                                      ctx->_cache_space_capacity, ctx->_row_bytes, 128, status, nullptr, copy_stream));
    // (Publishing beside the copy instead of behind it was measured at config 5 twice.  On the second stream: the step
    // "row copy + insert" went from 0.245 to 0.318 ms.  As one launch whose workgroups took the two jobs in turn: 121 us
    // against 55 us for the copy and 61 us for the insert one after the other.  Neither waits with the chip idle:
    // 462,000 rows at random places of the stage and as many lines at random places of the table share what
    // scattered accesses to HBM can get.)
    publish(rows_dev, slots_dev, num_rows);
  } else {
    if (stage) {
      // A background refresh takes what the stage holds in one launch (HBM to HBM, nothing for the lookups to share the
      // link with), publishes those rows at once and is left with a short list for the throttled copy below.
      TensorPtr rest_rows = Empty1DReuse(__rest_rows, kI32, {num_rows}, gpu_ctx);
      TensorPtr rest_slots = Empty1DReuse(__rest_slots, kI32, {num_rows}, gpu_ctx);
      UGK_CALL(ugk_fill_u32(status + 9, 0, 2, copy_stream));
      UGK_CALL(ugk_gather_scatter_staged_u32(host, ctx->_num_total_nodes, rows_dev, slots_dev, num_rows, cache,
                                             ctx->_cache_space_capacity, ctx->_row_bytes, *stage,
                                             RunConfig::refresh_limit_block, status, status + 8,
                                             rest_rows->Ptr<uint32_t>(), rest_slots->Ptr<uint32_t>(), status + 9,
                                             status + 10, copy_stream));
      uint32_t left_done[2] = {0, 0};
      UGK_CALL(ugk_memcpy_async(left_done, status + 9, sizeof(left_done), copy_stream));
      UGK_CALL(ugk_stream_sync(copy_stream));
      CHECK_LE((size_t)left_done[0] + left_done[1], num_rows);
      rows_dev = rest_rows->CPtr<uint32_t>();
      slots_dev = rest_slots->CPtr<uint32_t>();
      publish(rows_dev + (num_rows - left_done[1]), slots_dev + (num_rows - left_done[1]), left_done[1]);
      num_rows = left_done[0];
    }
    // the rest crosses the link in small throttled batches so that the lookups keep it (cache_context.cu:4054-4090);
    // every batch is published behind its copy, so its rows hit from then on
    const size_t batch = std::max<size_t>(RunConfig::refresh_batch_rows, 1);
    for (size_t begin = 0; begin < num_rows; begin += batch) {
      const size_t cur = std::min(batch, num_rows - begin);
      Timer t_batch;
      UGK_CALL(ugk_gather_scatter_u32(host, ctx->_num_total_nodes, rows_dev + begin, slots_dev + begin, cur, cache,
                                      ctx->_cache_space_capacity, ctx->_row_bytes, RunConfig::refresh_limit_block,
                                      status, nullptr, copy_stream));
      publish(rows_dev + begin, slots_dev + begin, cur);
      if (begin + batch < num_rows) {
        UGK_CALL(ugk_stream_sync(copy_stream));
        if (RunConfig::refresh_rate_gbps > 0) {
          // a share of the link instead of a fixed pause: the batch should have taken bytes / rate
          const double due_s = (double)cur * ctx->_row_bytes / (RunConfig::refresh_rate_gbps * 1e9) - t_batch.Passed();
          if (due_s > 0) usleep((useconds_t)(due_s * 1e6));
        } else {
          usleep(RunConfig::refresh_sleep_us);
        }
      }
    }
  }
  if (copy_stream == stream) return;  // the caller looks at the status word when it waits for its stream
  uint32_t st = 0;
  UGK_CALL(ugk_memcpy_async(&st, status, sizeof(st), copy_stream));
  UGK_CALL(ugk_stream_sync(copy_stream));
  CHECK_EQ(st, 0u) << "refresh row copy touched a row outside its table";
}

uint64_t RefreshSession::RowsFromStage() {
  if (!_status_handle) return 0;
  uint32_t n = 0;
  UGK_CALL(ugk_memcpy_async(&n, _status_handle->ptr<uint32_t>() + 8, sizeof(n), stream));
  UGK_CALL(ugk_stream_sync(stream));
  return n;
}

// cache_context.cu:3944-4107, the one-GPU part: steps 1-3, 5 and 6
void RefreshSession::refresh_after_solve_new(bool foreground) {
  CacheContext *ctx = _cache_ctx.get();
  auto table = ctx->_new_hash_table;
  CHECK_NOTNULL(table) << "refresh needs a partial cache (0 < cache_percentage < 1)";
  const Context gpu_ctx = ctx->_trainer_ctx;
  const int local = ctx->_local_location_id;
  auto coll_cache = ctx->_coll_cache;
  UGK_CALL(ugk_set_device(gpu_ctx.device_id));
  if (low_pri_stream == nullptr) UGK_CALL(ugk_stream_create(&low_pri_stream));
  if (!_status_handle) {
    _status_handle = EagerGPUAlloc(gpu_ctx.device_id, 256);
    UGK_CALL(ugk_fill_u32(_status_handle->ptr<uint32_t>(), 0, 64, stream));
  }

  // which stage of recently missed rows the row copy may read (a background refresh switches the lookups to the other
  // one here, long before the wait for the lookups in flight that precedes the copy)
  const ugk_stage_t *stage = nullptr;
  if (auto s0 = coll_cache->session(ctx->_local_location_id)) stage = s0->StageForRefresh(foreground, stream);
  table->EnsureHostLists(ctx->_eager_gpu_mem_allocator, gpu_ctx, stream);  // after a refresh on the device
  table->DropBuildBits();  // this refresh goes through the host's lists
  // Step 1: key list of the new placement
  Timer t_phase;
  double detect_s = 0, evict_s = 0, wait_s = 0, insert_s = 0;
  TensorPtr key_list_of_each_src[9] = {nullptr};
  const size_t num_block = coll_cache->_block_access_advise->Shape()[1];
  TensorPtr advise_line = Tensor::FromBlob(coll_cache->_block_access_advise->Ptr<uint8_t>() + (size_t)local * num_block,
                                           kU8, {num_block}, CPU_CLIB(), "advise_line");
  CacheEntryManager::DetectKeysForAllSource(coll_cache->_nid_to_block, advise_line, local, coll_cache->_block_density,
                                            RunConfig::num_total_item, key_list_of_each_src,
                                            (int)RunConfig::num_device);
  const size_t num_new_local_key = key_list_of_each_src[local]->NumItem();
  CHECK(num_new_local_key <= ctx->_cache_space_capacity) << "cache space can not hold refreshed new cache";

  // Steps 2 and 3: keys to insert = new local and not old local; keys to evict = old local and not new local
  // (DetectKeysWithCond over the other placement's nid_to_block in the reference, cache_context.cu:3975-4003).
  // Both lists are ascending (DetectKeysForAllSource), so the two differences are merges.
  const IdType *new_keys = key_list_of_each_src[local]->CPtr<IdType>();
  table->HostCachedKeys(stream);
  const IdType *old_keys = table->_cached_keys->CPtr<IdType>();
  const size_t num_old_local_key = table->_cached_keys->NumItem();
  TensorPtr new_insert_keys = CacheEntryManager::SortedDifference(new_keys, num_new_local_key, old_keys, num_old_local_key);
  const size_t num_preserved_key = num_new_local_key - new_insert_keys->NumItem();
  TensorPtr new_evict_keys = CacheEntryManager::SortedDifference(old_keys, num_old_local_key, new_keys, num_new_local_key);
  const size_t num_evicted = new_evict_keys->NumItem();
  CHECK_EQ(num_evicted + num_preserved_key, table->_cached_keys->NumItem());
  detect_s = t_phase.Passed();
  t_phase.Reset();
  if (num_evicted > 0) {
    auto evict_keys_gpu = RunConfig::key_map_mul == 0
                              ? CopyTo1DReuse(__keys_buffer, new_evict_keys, gpu_ctx, stream)
                              : table->TableKeysToDevice(new_evict_keys, ctx->_eager_gpu_mem_allocator, gpu_ctx, stream);
    auto evict_offs_gpu = Empty1DReuse(__offs_buffer, kI32, {num_evicted}, gpu_ctx);
    table->LookupOffset(evict_keys_gpu, evict_offs_gpu, stream);
    TensorPtr evict_offs_cpu = Tensor::Empty(kI32, {num_evicted}, CPU_CLIB(), "");
    UGK_CALL(ugk_memcpy_async(evict_offs_cpu->MutableData(), evict_offs_gpu->Data(), evict_offs_gpu->NumBytes(),
                              stream));
    UGK_CALL(ugk_stream_sync(stream));
    table->ReturnOffset(evict_offs_cpu);
    CHECK(num_evicted <= table->_free_offsets->NumItem());
    table->Evict(evict_keys_gpu, stream);
    table->CheckStatus(stream, "refresh evict");
  }
  LOG(INFO) << "refresh: preserved " << num_preserved_key << ", evict " << num_evicted << ", insert "
            << new_insert_keys->NumItem() << ", free slots " << table->_free_offsets->NumItem();

  evict_s = t_phase.Passed();
  t_phase.Reset();
  // Step 5: let one more lookup finish, so that no gather in flight still reads a slot about to be reused.  With
  // stream-ordered lookups "finished" is a matter of the stream: everything enqueued before this point still saw
  // the old table, everything after it sees the evicted keys as misses.
  auto session = coll_cache->session(ctx->_local_location_id);
  WaitForOneLookup(session.get(), foreground);

  wait_s = t_phase.Passed();
  t_phase.Reset();
  // Step 6: copy the new rows host -> HBM into slots taken from the front of the free list, then publish them
  const size_t num_insert = new_insert_keys->NumItem();
  if (num_insert > 0) {
    auto insert_keys_gpu = CopyTo1DReuse(__keys_buffer, new_insert_keys, gpu_ctx, low_pri_stream);
    auto reserved_offset =
        CopyTo1DReuse(__offs_buffer, table->ReserveOffsetFront((IdType)num_insert), gpu_ctx, low_pri_stream);
    CopyRowsIntoSlots(insert_keys_gpu->CPtr<uint32_t>(), reserved_offset->CPtr<uint32_t>(), num_insert, foreground,
                      low_pri_stream, stage);  // waits for the copy stream: rows copied and published
    table->CheckStatus(stream, "refresh insert");
  }
  AnonymousBarrier::_refresh_instance->Wait();

  insert_s = t_phase.Passed();
  t_phase.Reset();
  table->_cached_keys = key_list_of_each_src[local];
  table->_cached_keys_on_device = nullptr;
  table->_dev_lists_valid = false;  // the host lists hold the truth now
  ctx->_cache_nodes = num_new_local_key;
  const bool rebuilt = table->MaybeRebuild(ctx->_eager_gpu_mem_allocator, gpu_ctx, local, stream, [&]() {
    if (session) session->WaitForLookupsInFlight(foreground, 20.0);
  });
  LOG(INFO) << "refresh: key lists " << detect_s << " s, evict " << evict_s << " s, wait for a lookup " << wait_s
            << " s, row copy + insert " << insert_s << " s, table rebuild " << (rebuilt ? t_phase.Passed() : 0.0)
            << " s";
  CHECK_EQ(table->_free_offsets->NumItem() + num_new_local_key, ctx->_cache_space_capacity);
}

void RefreshSession::refresh_after_solve_main(bool foreground) { refresh_after_solve_new(foreground); }

void RefreshSession::refresh_on_device(ExtractSession *session, size_t num_cached, bool foreground) {
  CacheContext *ctx = _cache_ctx.get();
  auto table = ctx->_new_hash_table;
  CHECK_NOTNULL(table) << "refresh needs a partial cache (0 < cache_percentage < 1)";
  CHECK_NOTNULL(session);
  CHECK(session->CountsOnDevice()) << "refresh on the device needs the device-side hotness counters";
  CHECK_LE(num_cached, (size_t)ctx->_cache_space_capacity) << "cache space can not hold refreshed new cache";
  const Context gpu_ctx = ctx->_trainer_ctx;
  const int local = ctx->_local_location_id;
  const auto &alloc = ctx->_eager_gpu_mem_allocator;
  const size_t num_rows = ctx->_num_total_nodes, capacity = ctx->_cache_space_capacity;
  UGK_CALL(ugk_set_device(gpu_ctx.device_id));
  if (low_pri_stream == nullptr) UGK_CALL(ugk_stream_create(&low_pri_stream));
  if (!_status_handle) {
    _status_handle = EagerGPUAlloc(gpu_ctx.device_id, 256);
    UGK_CALL(ugk_fill_u32(_status_handle->ptr<uint32_t>(), 0, 64, stream));
  }
  const ugk_stage_t *stage = session->StageForRefresh(foreground, stream);  // see refresh_after_solve_new
  Timer t_phase;
  table->EnsureDeviceLists(alloc, gpu_ctx, stream);
  const double sync_s = t_phase.Passed();
  t_phase.Reset();

  // Steps 1-3: the new placement as a bitmap, then evict = cached & ~new and insert = new & ~cached, ascending.  Both
  // sets are counted before the one wait that tells the host their sizes.
  // COLL_GPU_REFRESH_STABLE: rows that tie at the last count that gets in stay where they are (cached or not)
  // (a placement that knows that fewer rows were observed than the cache holds counts both sets on its way)
  const ExtractSession::DiffCount diff = {table->InCacheBits(), table->_dev_bm_ws->ptr(), table->_dev_bm_ws2->ptr(),
                                          table->DevWords() + 8, _status_handle->ptr<uint32_t>()};
  const bool counted = session->PlaceOnDevice(
      num_cached, table->InNewBits(), table->_dev_scratch_bits->ptr<uint64_t>(),
      RunConfig::gpu_refresh_stable ? table->InCacheBits() : nullptr, table->_dev_rank_ws->ptr(),
      !RunConfig::gpu_refresh_keep, &diff, stream);
  if (!counted) table->CountDiff(table->InCacheBits(), table->InNewBits(), num_rows, stream);  // the same pinned words
  ApplyPlacedBits(session, num_cached, foreground, stage, true,
                  counted ? "placement (from the observed rows alone)" : "placement", sync_s, t_phase);
}

// A refresh whose placement the host has ranked (FreqRecorder + solver: the default) applied like one computed on the
// device.  The placement arrives as what it was computed from: the ranked rows that are cached and how many of the
// lowest other rows fill the rest.  Their bits make the bitmap of rows cached after the refresh; what leaves and what
// comes in are its differences with the bitmap of rows cached now.  No array over the key space is written or
// scanned on the host (config 5: 2 GB written by the solver and read by the key-list scan, 0.45 s of a 0.48 s
// refresh).
void RefreshSession::refresh_from_ranked_rows(ExtractSession *session, TensorPtr top_rows, size_t num_extra,
                                              bool foreground) {
  CacheContext *ctx = _cache_ctx.get();
  auto table = ctx->_new_hash_table;
  CHECK_NOTNULL(table) << "refresh needs a partial cache (0 < cache_percentage < 1)";
  CHECK_NOTNULL(top_rows);
  const Context gpu_ctx = ctx->_trainer_ctx;
  const auto &alloc = ctx->_eager_gpu_mem_allocator;
  const size_t num_rows = ctx->_num_total_nodes;
  const size_t num_top = top_rows->NumItem(), num_cached = num_top + num_extra;
  CHECK_LE(num_cached, (size_t)ctx->_cache_space_capacity) << "cache space can not hold refreshed new cache";
  CHECK_LT(num_cached, num_rows);
  UGK_CALL(ugk_set_device(gpu_ctx.device_id));
  if (low_pri_stream == nullptr) UGK_CALL(ugk_stream_create(&low_pri_stream));
  if (!_status_handle) {
    _status_handle = EagerGPUAlloc(gpu_ctx.device_id, 256);
    UGK_CALL(ugk_fill_u32(_status_handle->ptr<uint32_t>(), 0, 64, stream));
  }
  const ugk_stage_t *stage = session ? session->StageForRefresh(foreground, stream) : nullptr;
  Timer t_phase;
  table->EnsureDeviceLists(alloc, gpu_ctx, stream);
  const double sync_s = t_phase.Passed();
  t_phase.Reset();
  const size_t words = (num_rows + 63) / 64;
  // the ranked rows' bits: straight into the new bitmap when they are all of it, else into the scratch bitmap, from
  // which the placement adds the lowest rows that are not among them
  uint64_t *ranked_bits = num_extra ? table->_dev_scratch_bits->ptr<uint64_t>() : table->InNewBits();
  UGK_CALL(ugk_fill_u32(reinterpret_cast<uint32_t *>(ranked_bits), 0, words * 2, stream));
  if (num_top > 0) {
    TensorPtr top_dev = CopyTo1DReuse(__ranked_rows, top_rows, gpu_ctx, stream);
    UGK_CALL(ugk_bitmap_update(ranked_bits, num_rows, top_dev->CPtr<uint32_t>(), num_top, 1,
                               _status_handle->ptr<uint32_t>(), stream));
  }
  if (num_extra > 0) {
    UGK_CALL(ugk_rank_place_observed(nullptr, num_rows, num_cached, table->_dev_rank_ws->ptr(), table->InNewBits(),
                                     ranked_bits, 0, table->InCacheBits(), table->_dev_bm_ws->ptr(),
                                     table->_dev_bm_ws2->ptr(), table->DevWords() + 8,
                                     _status_handle->ptr<uint32_t>(), stream));
  } else {
    table->CountDiff(table->InCacheBits(), table->InNewBits(), num_rows, stream);
  }
  ApplyPlacedBits(session, num_cached, foreground, stage, false, "placement ranked on the host", sync_s, t_phase);
}

// The second half of a refresh whose new placement stands in the table's bitmap of rows cached after it, with the two
// counts (rows that leave, rows that come in) on their way into the pinned words 8 and 9: waits for the counts, lists
// evict = cached & ~new and insert = new & ~cached, then steps 4 - 6 of refresh_after_solve_new on device lists.
void RefreshSession::ApplyPlacedBits(ExtractSession *session, size_t num_cached, bool foreground,
                                     const ugk_stage_t *stage, bool placed_from_counters, const char *how,
                                     double sync_s, Timer &t_phase) {
  CacheContext *ctx = _cache_ctx.get();
  auto table = ctx->_new_hash_table;
  const Context gpu_ctx = ctx->_trainer_ctx;
  const auto &alloc = ctx->_eager_gpu_mem_allocator;
  const size_t num_rows = ctx->_num_total_nodes, capacity = ctx->_cache_space_capacity;
  volatile uint32_t *n_evict_word = table->DevWords() + 8, *n_insert_word = table->DevWords() + 9;
  table->WaitByTicket(stream);
  if (placed_from_counters) session->PlacementWaitedFor();
  const size_t num_evicted = *n_evict_word, num_insert = *n_insert_word;
  TensorPtr evict_rows, insert_rows;  // both lists in one pass over the two bitmaps
  table->EmitDiff(table->InCacheBits(), table->InNewBits(), num_rows, num_evicted, num_insert, __evict_rows,
                  __insert_rows, &evict_rows, &insert_rows, alloc, gpu_ctx, stream);
  const size_t num_old = table->_num_cached;
  CHECK_LE(num_evicted, num_old);
  const size_t num_preserved_key = num_old - num_evicted;
  CHECK_EQ(num_preserved_key + num_insert, std::min(num_cached, num_rows));
  const double place_s = t_phase.Passed();
  t_phase.Reset();

  // Step 4: the evicted keys leave the table, their slots become free.  A foreground refresh looks at the status words
  // of its kernels once, at the end; a background one, which lookups run beside, after every step.
  if (num_evicted > 0) {
    TensorPtr evict_keys = table->RowsToTableKeys(evict_rows, __evict_ids, alloc, gpu_ctx, stream);
    table->EvictRelease(evict_keys, stream);  // one launch: the key leaves the table, its slot the slot bitmap
    if (!foreground) table->CheckStatus(stream, "refresh evict");
  }
  LOG(INFO) << "refresh on the device: preserved " << num_preserved_key << ", evict " << num_evicted << ", insert "
            << num_insert << ", free slots " << table->_num_free + num_evicted;
  const double evict_s = t_phase.Passed();
  t_phase.Reset();

  // Step 5: let one more lookup finish, so that no gather in flight still reads a slot about to be reused
  // (a foreground refresh copies on its own stream: lookups enqueued there are in front of the copy as it is)
  WaitForOneLookup(session, foreground, foreground ? &stream : nullptr);
  const double wait_s = t_phase.Passed();
  t_phase.Reset();

  // Step 6: the first free slots, ascending, take the new rows, ascending; then the keys are published.  (A foreground
  // refresh that returned here and left copy, publication and the slot bitmap's update running on the copy stream
  // beside the caller's next lookup was measured: the call got 0.15 ms shorter, a whole step no shorter, because that
  // lookup holds every wavefront slot of the chip while it waits for the host link.)
  const size_t num_free_expected = table->_num_free + num_evicted;
  volatile uint32_t *n_free_word = nullptr;
  if (num_insert > 0) {
    CHECK_LE(num_insert, num_free_expected) << "free cache slots exhausted";
    // how many slots are free is known without looking (what was free plus what was evicted); the count the compaction
    // makes on its way is compared with that once the refresh has been waited for
    n_free_word = table->CountBits(table->SlotUsedBits(), nullptr, true, capacity, 0, stream);
    TensorPtr slots =
        table->EmitBits(table->SlotUsedBits(), nullptr, true, capacity, 0, num_insert, __free_slots, alloc, gpu_ctx, stream);
    if (foreground) {
      // nothing runs beside a foreground refresh: the copy goes on the refresh's own stream, behind the lists it reads
      CopyRowsIntoSlots(insert_rows->CPtr<uint32_t>(), slots->CPtr<uint32_t>(), num_insert, true, stream, stage);
    } else {
      UGK_CALL(ugk_stream_sync(stream));  // the lists are read on the copy stream next
      CopyRowsIntoSlots(insert_rows->CPtr<uint32_t>(), slots->CPtr<uint32_t>(), num_insert, false, low_pri_stream,
                        stage);
    }
    // the slots taken are the lowest free ones: every bit up to the last of them is set now
    UGK_CALL(ugk_bitmap_set_through(table->SlotUsedBits(), capacity, slots->CPtr<uint32_t>() + (num_insert - 1),
                                    _status_handle->ptr<uint32_t>(), stream));
  }
  uint32_t stw[9] = {0};  // [0] status bits, [8] rows taken from the stage so far
  // one launch brings the table's status word and these nine to the host, one wait by ticket ends the refresh
  const uint32_t table_status = table->StatusAndWords(_status_handle->ptr<uint32_t>(), 9, stw, stream);
  CHECK_EQ(table_status, 0u) << "refresh on the device: table maintenance kernel reported status 0x" << std::hex
                             << table_status
                             << " (1 key out of range, 2 table full, 4 duplicate key, 8 evict of absent key)";
  CHECK_EQ(stw[0], 0u) << "refresh on the device: a listed row or slot is outside its table or bitmap (1), or the "
                          "placement found more observed rows than the host's bound allows (0x20)";
  const uint32_t from_stage = stw[8] - _rows_from_stage;
  _rows_from_stage = stw[8];
  if (n_free_word) CHECK_EQ((size_t)*n_free_word, num_free_expected);
  AnonymousBarrier::_refresh_instance->Wait();
  const double insert_s = t_phase.Passed();
  t_phase.Reset();

  std::swap(table->_dev_in_cache, table->_dev_in_new);
  table->_num_cached = num_preserved_key + num_insert;
  table->_num_free = capacity - table->_num_cached;
  table->_host_lists_valid = false;  // the bitmaps hold the truth now
  table->_cached_keys_on_device = nullptr;
  ctx->_cache_nodes = table->_num_cached;
  const bool rebuilt = table->MaybeRebuild(alloc, gpu_ctx, ctx->_local_location_id, stream, [&]() {
    if (session) session->WaitForLookupsInFlight(foreground, 20.0);
  });
  LOG(INFO) << "refresh on the device: bitmaps " << sync_s << " s, " << how << " + key lists " << place_s << " s, evict "
            << evict_s << " s, wait for a lookup " << wait_s << " s, row copy + insert " << insert_s
            << " s (" << from_stage << " of " << num_insert << " rows from the stage), table rebuild "
            << (rebuilt ? t_phase.Passed() : 0.0) << " s";
}


}  // namespace coll_cache_lib
