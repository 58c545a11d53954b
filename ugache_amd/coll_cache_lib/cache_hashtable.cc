#include "cache_hashtable.h"

#include <algorithm>

namespace coll_cache_lib {
namespace common {

namespace {
uint32_t *StatusPtr(CacheEntryManager *m, StreamHandle stream) {
  if (!m->_status_handle) {
    m->_status_handle = EagerGPUAlloc(m->_device_id, 256);
    UGK_CALL(ugk_fill_u32(m->_status_handle->ptr<uint32_t>(), 0, 64, stream));
  }
  return m->_status_handle->ptr<uint32_t>();
}

void *Align128(void *p) { return reinterpret_cast<void *>((reinterpret_cast<uintptr_t>(p) + 127) / 128 * 128); }
}  // namespace

void CacheEntryManager::CreateFlat(const std::function<MemHandle(size_t)> &allocator, size_t num_keys,
                                   StreamHandle stream) {
  LOG(INFO) << "flat lookup table over " << num_keys << " keys, " << ToReadableSize(num_keys * sizeof(IdType));
  _table_handle = allocator(num_keys * sizeof(IdType));
  CHECK_NOTNULL(_table_handle);
  _table = {1, 0, _table_handle->ptr(), num_keys, 0, 0};
  UGK_CALL(ugk_fill_u32(_table_handle->ptr<uint32_t>(), kEmptyPos, num_keys, stream));
  RunConfig::use_flat_hashtable = true;
}

namespace {
size_t HashEntryBytes(int kind) { return kind == 3 ? sizeof(uint64_t) : sizeof(ugk_bucket_t); }
size_t HashEntriesFor(int kind, size_t num_entries) {
  return kind == 3 ? ugk_hash32_entries_for(num_entries, RunConfig::hash_load_factor)
                   : ugk_hash_buckets_for(num_entries, RunConfig::hash_load_factor);
}
}  // namespace

bool CacheEntryManager::CompactHashFits(size_t num_slots, size_t num_host_rows) {
  // an 8-byte entry names its key by the host row (below 0xfffffffe: the two values above mark never-used and evicted
  // entries) and packs the slot into 28 bits beside the 4-bit location
  return num_host_rows <= 0xfffffffeull && num_slots <= ((size_t)1 << 28);
}

void CacheEntryManager::CreateHash(const std::function<MemHandle(size_t)> &allocator, size_t num_entries,
                                   size_t num_host_rows, StreamHandle stream) {
  int kind = CompactHashFits(num_entries, num_host_rows) ? 3 : 2;
  if (RunConfig::force_table_kind == 16) kind = 2;
  if (RunConfig::force_table_kind == 8) {
    CHECK(kind == 3) << "COLL_HASH_TABLE=HASH8: 8-byte entries hold rows below 0xfffffffe and 2^28 slots; this cache has "
                     << num_host_rows << " rows and " << num_entries << " slots";
  }
  const size_t ne = HashEntriesFor(kind, num_entries);
  LOG(INFO) << "open-addressing lookup table for " << num_entries << " entries: " << ne << " entries of "
            << HashEntryBytes(kind) << " bytes, " << ToReadableSize(ne * HashEntryBytes(kind));
  _table_handle = allocator(ne * HashEntryBytes(kind) + 128);
  CHECK_NOTNULL(_table_handle);
  void *base = Align128(_table_handle->ptr());
  _table = {kind, 0, base, ne, RunConfig::key_map_inv, RunConfig::key_map_mask};
  UGK_CALL(ugk_table_init(_table, stream));
  RunConfig::use_flat_hashtable = false;
}

TensorPtr CacheEntryManager::HostCachedKeys(StreamHandle stream) {
  if (_cached_keys_on_device) {
    const size_t n = _cached_keys_on_device->NumItem();
    _cached_keys = Tensor::Empty(kI32, {n}, CPU_CLIB(), "cached_keys");
    if (n) {
      UGK_CALL(ugk_set_device(_device_id));
      UGK_CALL(ugk_memcpy_async(_cached_keys->MutableData(), _cached_keys_on_device->Data(), n * sizeof(IdType), stream));
      UGK_CALL(ugk_stream_sync(stream));
    }
    _cached_keys_on_device = nullptr;
  }
  return _cached_keys;
}

TensorPtr CacheEntryManager::TableKeysToDevice(TensorPtr host_rows, const std::function<MemHandle(size_t)> &allocator,
                                               Context ctx, StreamHandle stream) {
  // (8-byte entries are keyed by the row: the list is the key list)
  if (RunConfig::key_map_mul == 0 || _table.kind == 3) return Tensor::CopyToExternal(host_rows, allocator, ctx, stream);
  const size_t n = host_rows->NumItem();
  TensorPtr ids = Tensor::Empty(kI64, {n}, CPU_CLIB(), "");
  const IdType *rows = host_rows->CPtr<IdType>();
  int64_t *out = ids->Ptr<int64_t>();
#pragma omp parallel for num_threads(std::max(1, RunConfig::solver_omp_thread_num_per_gpu)) if (n > 65536)
  for (size_t i = 0; i < n; i++) out[i] = (int64_t)RunConfig::KeyOfRow(rows[i]);
  return Tensor::CopyToExternal(ids, allocator, ctx, stream);
}

void CacheEntryManager::LookupOffset(TensorPtr keys, TensorPtr off, StreamHandle stream) {
  CHECK_EQ(keys->NumItem(), off->NumItem());
  if (keys->Type() == kI64)
    UGK_CALL(ugk_table_lookup_i64(_table, keys->CPtr<int64_t>(), keys->NumItem(), (uint32_t)cpu_location_id, nullptr,
                                  off->Ptr<uint32_t>(), stream));
  else
    UGK_CALL(ugk_table_lookup_u32(RowView(), keys->CPtr<uint32_t>(), keys->NumItem(), (uint32_t)cpu_location_id, nullptr,
                                  off->Ptr<uint32_t>(), stream));
}

void CacheEntryManager::InsertWithLoc(TensorPtr keys, TensorPtr off, int loc, StreamHandle stream) {
  CHECK_EQ(keys->NumItem(), off->NumItem());
  if (keys->Type() == kI64)
    UGK_CALL(ugk_table_insert_i64(_table, keys->CPtr<int64_t>(), off->CPtr<uint32_t>(), 0, (uint32_t)loc,
                                  keys->NumItem(), StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_insert_u32(RowView(), keys->CPtr<uint32_t>(), off->CPtr<uint32_t>(), 0, (uint32_t)loc,
                                  keys->NumItem(), StatusPtr(this, stream), stream));
}

void CacheEntryManager::InsertSeqOffWithLoc(TensorPtr keys, int loc, StreamHandle stream) {
  if (keys->Type() == kI64)
    UGK_CALL(ugk_table_insert_i64(_table, keys->CPtr<int64_t>(), nullptr, 0, (uint32_t)loc, keys->NumItem(),
                                  StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_insert_u32(RowView(), keys->CPtr<uint32_t>(), nullptr, 0, (uint32_t)loc, keys->NumItem(),
                                  StatusPtr(this, stream), stream));
}

void CacheEntryManager::Evict(TensorPtr keys_to_evict, StreamHandle stream) {
  if (keys_to_evict->Type() == kI64)
    UGK_CALL(ugk_table_evict_i64(_table, keys_to_evict->CPtr<int64_t>(), keys_to_evict->NumItem(),
                                 StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_evict_u32(RowView(), keys_to_evict->CPtr<uint32_t>(), keys_to_evict->NumItem(),
                                 StatusPtr(this, stream), stream));
  if (_table.kind >= 2) _num_tombstones += keys_to_evict->NumItem();
}

void CacheEntryManager::EvictRelease(TensorPtr keys_to_evict, StreamHandle stream) {
  if (keys_to_evict->Type() == kI64)
    UGK_CALL(ugk_table_evict_release_i64(_table, keys_to_evict->CPtr<int64_t>(), keys_to_evict->NumItem(),
                                         SlotUsedBits(), _cache_space_capacity, StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_evict_release_u32(RowView(), keys_to_evict->CPtr<uint32_t>(), keys_to_evict->NumItem(),
                                         SlotUsedBits(), _cache_space_capacity, StatusPtr(this, stream), stream));
  if (_table.kind >= 2) _num_tombstones += keys_to_evict->NumItem();
}

bool CacheEntryManager::MaybeRebuild(const std::function<MemHandle(size_t)> &allocator, Context ctx, int loc,
                                     StreamHandle stream, const std::function<void()> &wait_for_lookups) {
  if (_table.kind < 2) return false;
  const double limit = RunConfig::hash_rebuild_tombstone_frac * (double)_table.size;
  if ((double)_num_tombstones <= limit) return false;
  // _num_tombstones counts evictions; inserts reuse tombstones they pass, so look before rebuilding
  uint64_t *census_dev = reinterpret_cast<uint64_t *>(StatusPtr(this, stream) + 16);
  uint64_t census[3] = {0, 0, 0};
  UGK_CALL(ugk_table_census(_table, census_dev, stream));
  UGK_CALL(ugk_memcpy_async(census, census_dev, sizeof(census), stream));
  UGK_CALL(ugk_stream_sync(stream));
  _num_tombstones = census[1];
  if ((double)_num_tombstones <= limit) return false;
  TensorPtr keys, offs, key_buffer;
  size_t n = 0;
  if (_dev_lists_valid) {  // the cached rows are known on the device: the key list never leaves it
    TensorPtr rows = CompactBits(InCacheBits(), nullptr, false, num_total_key, SIZE_MAX, _dev_list_buffer, allocator,
                                 ctx, stream, &n);
    keys = RowsToTableKeys(rows, key_buffer, allocator, ctx, stream);
  } else {
    if (_cached_keys_on_device) {  // the list of the build is still on the device
      n = _cached_keys_on_device->NumItem();
      keys = RowsToTableKeys(_cached_keys_on_device, key_buffer, allocator, ctx, stream);
    } else {
      n = _cached_keys->NumItem();
      keys = TableKeysToDevice(_cached_keys, allocator, ctx, stream);
    }
  }
  LOG(INFO) << "rebuilding the lookup table: " << _num_tombstones << " tombstones in " << _table.size << " entries, "
            << n << " live keys";
  offs = Tensor::EmptyExternal(kI32, {n}, allocator, ctx, "");
  if (n > 0) LookupOffset(keys, offs, stream);
  // the keys go into a second table; the one in use keeps serving lookups until the swap
  MemHandle fresh_handle = allocator(_table.size * HashEntryBytes(_table.kind) + 128);
  CHECK_NOTNULL(fresh_handle);
  ugk_table_t fresh = _table;
  fresh.table = Align128(fresh_handle->ptr());
  UGK_CALL(ugk_table_init(fresh, stream));
  ugk_table_t fresh_rows = fresh;  // as 32-bit row numbers address it (RowView)
  if (fresh_rows.kind == 3) fresh_rows.fb_mul = fresh_rows.fb_mask = 0;
  if (n > 0) {
    if (keys->Type() == kI64)
      UGK_CALL(ugk_table_insert_i64(fresh, keys->CPtr<int64_t>(), offs->CPtr<uint32_t>(), 0, (uint32_t)loc, n,
                                    StatusPtr(this, stream), stream));
    else
      UGK_CALL(ugk_table_insert_u32(fresh_rows, keys->CPtr<uint32_t>(), offs->CPtr<uint32_t>(), 0, (uint32_t)loc, n,
                                    StatusPtr(this, stream), stream));
  }
  CheckStatus(stream, "table rebuild");  // waits for the stream: the new table is complete
  {
    std::lock_guard<std::mutex> guard(_table_mu);
    _table = fresh;
    std::swap(_table_handle, fresh_handle);
  }
  if (wait_for_lookups) wait_for_lookups();
  fresh_handle = nullptr;  // the old buckets
  _num_tombstones = 0;
  _num_rebuilds++;
  return true;
}

namespace {
TensorPtr ReuseList(TensorPtr &buffer, DataType dtype, size_t n, const std::function<MemHandle(size_t)> &allocator,
                    Context ctx) {
  const std::vector<size_t> shape = {n};
  if (buffer && buffer->CanForceScale(dtype, shape)) {
    buffer->ForceScale(dtype, shape, ctx, "");
    return buffer;
  }
  // room to grow: these lists change size from refresh to refresh
  const size_t elem = dtype == kI64 ? 8 : 4;
  buffer = Tensor::EmptyExternal(kU8, {std::max<size_t>(n + n / 4, 1024) * elem}, allocator, ctx, "");
  buffer->ForceScale(dtype, shape, ctx, "");
  return buffer;
}
}  // namespace

TensorPtr CacheEntryManager::CompactBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits,
                                         size_t limit, TensorPtr &buffer,
                                         const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                         StreamHandle stream, size_t *total_out) {
  uint32_t *total = DevWords();
  UGK_CALL(ugk_bitmap_count(a, b, invert_a ? 1 : 0, nbits, _dev_bm_ws->ptr(), total, stream));
  UGK_CALL(ugk_stream_sync(stream));
  const size_t found = *total;
  if (total_out) *total_out = found;
  const size_t n = std::min(found, limit);
  TensorPtr list = ReuseList(buffer, kI32, n, allocator, ctx);
  if (n) UGK_CALL(ugk_bitmap_emit(a, b, invert_a ? 1 : 0, nbits, _dev_bm_ws->ptr(), list->Ptr<uint32_t>(), n, stream));
  return list;
}

volatile uint32_t *CacheEntryManager::CountBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits,
                                                int which, StreamHandle stream) {
  CHECK(which == 0 || which == 1);
  uint32_t *total = DevWords() + 8 + which;
  void *ws = which == 0 ? _dev_bm_ws->ptr() : _dev_bm_ws2->ptr();
  UGK_CALL(ugk_bitmap_count(a, b, invert_a ? 1 : 0, nbits, ws, total, stream));
  return total;
}

TensorPtr CacheEntryManager::EmitBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits, int which,
                                      size_t n, TensorPtr &buffer, const std::function<MemHandle(size_t)> &allocator,
                                      Context ctx, StreamHandle stream) {
  TensorPtr list = ReuseList(buffer, kI32, n, allocator, ctx);
  const void *ws = which == 0 ? _dev_bm_ws->ptr() : _dev_bm_ws2->ptr();
  if (n) UGK_CALL(ugk_bitmap_emit(a, b, invert_a ? 1 : 0, nbits, ws, list->Ptr<uint32_t>(), n, stream));
  return list;
}

void CacheEntryManager::CountDiff(const uint64_t *a, const uint64_t *b, uint64_t nbits, StreamHandle stream) {
  UGK_CALL(ugk_bitmap_count_diff(a, b, nbits, _dev_bm_ws->ptr(), _dev_bm_ws2->ptr(), DevWords() + 8, stream));
}

void CacheEntryManager::EmitDiff(const uint64_t *a, const uint64_t *b, uint64_t nbits, size_t n_ab, size_t n_ba,
                                 TensorPtr &buffer_ab, TensorPtr &buffer_ba, TensorPtr *list_ab, TensorPtr *list_ba,
                                 const std::function<MemHandle(size_t)> &allocator, Context ctx, StreamHandle stream) {
  *list_ab = ReuseList(buffer_ab, kI32, n_ab, allocator, ctx);
  *list_ba = ReuseList(buffer_ba, kI32, n_ba, allocator, ctx);
  UGK_CALL(ugk_bitmap_emit_diff(a, b, nbits, _dev_bm_ws->ptr(), _dev_bm_ws2->ptr(),
                                n_ab ? (*list_ab)->Ptr<uint32_t>() : nullptr, n_ab,
                                n_ba ? (*list_ba)->Ptr<uint32_t>() : nullptr, n_ba, stream));
}

// pinned words of the table (64): [0] CompactBits' total, [8..10] the counts of a refresh, [16] the ticket of
// WaitByTicket, [32] the ticket of StatusAndWords and [33 ...] its words
void CacheEntryManager::WaitByTicket(StreamHandle stream) {
  CHECK(_dev_words) << "the table's pinned words come with its device lists";
  if (RunConfig::spin_wait_us == 0) {
    UGK_CALL(ugk_stream_sync(stream));
    return;
  }
  if (++_ticket == 0) _ticket = 1;
  UGK_CALL(ugk_stream_sync_ticket(stream, DevWords() + 16, _ticket, RunConfig::spin_wait_us));
}

uint32_t CacheEntryManager::StatusAndWords(const uint32_t *extra_dev, unsigned n_extra, uint32_t *extra_out,
                                           StreamHandle stream) {
  CHECK_LE(n_extra, 30u);
  CHECK(_dev_words) << "the table's pinned words come with its device lists";
  if (++_ticket == 0) _ticket = 1;
  uint32_t *dst = DevWords() + 32;
  UGK_CALL(ugk_words_to_host_ticket(StatusPtr(this, stream), 1, extra_dev, n_extra, dst, _ticket,
                                    RunConfig::spin_wait_us, stream));
  for (unsigned i = 0; i < n_extra; ++i) extra_out[i] = dst[2 + i];
  return dst[1];
}

TensorPtr CacheEntryManager::RowsToTableKeys(TensorPtr rows_dev, TensorPtr &buffer,
                                             const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                             StreamHandle stream) {
  if (RunConfig::key_map_mul == 0 || _table.kind == 3) return rows_dev;  // 8-byte entries are keyed by the row
  const size_t n = rows_dev->NumItem();
  TensorPtr ids = ReuseList(buffer, kI64, n, allocator, ctx);
  UGK_CALL(ugk_rows_to_keys(rows_dev->CPtr<uint32_t>(), n, RunConfig::key_map_mul, RunConfig::key_map_mask,
                            ids->Ptr<int64_t>(), stream));
  return ids;
}

void CacheEntryManager::PublishRows(const uint32_t *rows_dev, const uint32_t *slots_dev, size_t n, int loc,
                                    TensorPtr &id_buffer, const std::function<MemHandle(size_t)> &allocator,
                                    Context ctx, StreamHandle stream) {
  if (n == 0) return;
  if (RunConfig::key_map_mul == 0 || _table.kind == 3) {
    UGK_CALL(ugk_table_insert_u32(RowView(), rows_dev, slots_dev, 0, (uint32_t)loc, n, StatusPtr(this, stream), stream));
    return;
  }
  TensorPtr ids = ReuseList(id_buffer, kI64, n, allocator, ctx);
  UGK_CALL(ugk_rows_to_keys(rows_dev, n, RunConfig::key_map_mul, RunConfig::key_map_mask, ids->Ptr<int64_t>(), stream));
  UGK_CALL(ugk_table_insert_i64(_table, ids->CPtr<int64_t>(), slots_dev, 0, (uint32_t)loc, n, StatusPtr(this, stream),
                                stream));
}

void CacheEntryManager::EnsureDeviceLists(const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                          StreamHandle stream) {
  const size_t row_words = (num_total_key + 63) / 64, slot_words = ((size_t)_cache_space_capacity + 63) / 64;
  if (!_dev_words) {
    if (!_dev_in_cache) _dev_in_cache = EagerGPUAlloc(_device_id, row_words * 8);  // else: the build's bitmap
    _dev_in_new = EagerGPUAlloc(_device_id, row_words * 8);
    _dev_scratch_bits = EagerGPUAlloc(_device_id, row_words * 8);
    _dev_slot_used = EagerGPUAlloc(_device_id, std::max<size_t>(slot_words, 1) * 8);
    _dev_rank_ws = EagerGPUAlloc(_device_id, ugk_rank_workspace_bytes());
    _dev_bm_ws = EagerGPUAlloc(_device_id, ugk_bitmap_workspace_bytes());
    _dev_bm_ws2 = EagerGPUAlloc(_device_id, ugk_bitmap_workspace_bytes());
    _dev_words = PinnedHostAlloc(256);
    memset(_dev_words->ptr(), 0, 256);
  }
  if (_dev_lists_valid) return;
  CHECK(_host_lists_valid);
  const size_t n = NumCached();
  UGK_CALL(ugk_fill_u32(_dev_slot_used->ptr<uint32_t>(), 0, std::max<size_t>(slot_words, 1) * 2, stream));
  if (_build_bits_fresh) {
    // nothing has changed the cache since the build: its bitmap stands, its rows sit in slots 0 .. n - 1
    _build_bits_fresh = false;
    CHECK_EQ(_free_offsets->NumItem() + n, (size_t)_cache_space_capacity);
    if (n > 0) {
      uint32_t *status = StatusPtr(this, stream);
      uint32_t *last = status + 32;  // a device word for the position of the last slot taken
      UGK_CALL(ugk_fill_u32(last, (uint32_t)(n - 1), 1, stream));
      UGK_CALL(ugk_bitmap_set_through(SlotUsedBits(), _cache_space_capacity, last, status, stream));
      CheckStatus(stream, "placement bitmaps");
    }
    _num_cached = n;
    _num_free = _free_offsets->NumItem();
    _dev_lists_valid = true;
    return;
  }
  UGK_CALL(ugk_fill_u32(_dev_in_cache->ptr<uint32_t>(), 0, row_words * 2, stream));
  if (n > 0) {
    TensorPtr rows = _cached_keys_on_device;  // the list of the build, if it is still on the device
    if (!rows) {
      rows = ReuseList(_dev_list_buffer, kI32, n, allocator, ctx);
      UGK_CALL(ugk_memcpy_async(rows->MutableData(), _cached_keys->Data(), n * sizeof(IdType), stream));
      UGK_CALL(ugk_stream_sync(stream));  // the source is pageable host memory
    }
    uint32_t *status = StatusPtr(this, stream);
    UGK_CALL(ugk_bitmap_update(InCacheBits(), num_total_key, rows->CPtr<uint32_t>(), n, 1, status, stream));
    TensorPtr key_buffer;
    TensorPtr keys = RowsToTableKeys(rows, key_buffer, allocator, ctx, stream);
    TensorPtr slots = Tensor::EmptyExternal(kI32, {n}, allocator, ctx, "");
    LookupOffset(keys, slots, stream);
    UGK_CALL(ugk_bitmap_update(SlotUsedBits(), _cache_space_capacity, slots->CPtr<uint32_t>(), n, 1, status, stream));
    CheckStatus(stream, "placement bitmaps");
  }
  _num_cached = n;
  _num_free = _free_offsets->NumItem();
  CHECK_EQ(_num_cached + _num_free, (size_t)_cache_space_capacity);
  _dev_lists_valid = true;
}

void CacheEntryManager::EnsureHostLists(const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                        StreamHandle stream) {
  if (_host_lists_valid) {
    HostCachedKeys(stream);
    return;
  }
  _cached_keys_on_device = nullptr;  // superseded by what the bitmaps say
  CHECK(_dev_lists_valid);
  UGK_CALL(ugk_set_device(_device_id));
  size_t n_cached = 0, n_free = 0;
  TensorPtr rows =
      CompactBits(InCacheBits(), nullptr, false, num_total_key, SIZE_MAX, _dev_list_buffer, allocator, ctx, stream,
                  &n_cached);
  _cached_keys = Tensor::Empty(kI32, {n_cached}, CPU_CLIB(), "cached_keys");
  if (n_cached) UGK_CALL(ugk_memcpy_async(_cached_keys->MutableData(), rows->Data(), n_cached * sizeof(IdType), stream));
  UGK_CALL(ugk_stream_sync(stream));
  TensorPtr slots = CompactBits(SlotUsedBits(), nullptr, true, _cache_space_capacity, SIZE_MAX, _dev_list_buffer,
                                allocator, ctx, stream, &n_free);
  _free_offsets = Tensor::Empty(kI32, {(size_t)_cache_space_capacity}, CPU_CLIB(), "free_offsets");
  _free_offsets->ForceScale(kI32, {n_free}, CPU_CLIB(), "");
  if (n_free) UGK_CALL(ugk_memcpy_async(_free_offsets->MutableData(), slots->Data(), n_free * sizeof(IdType), stream));
  UGK_CALL(ugk_stream_sync(stream));
  CHECK_EQ(n_cached, _num_cached);
  CHECK_EQ(n_free, _num_free);
  CHECK_EQ(n_cached + n_free, (size_t)_cache_space_capacity);
  _host_lists_valid = true;
}

void CacheEntryManager::CheckStatus(StreamHandle stream, const char *what) {
  uint32_t st = 0;
  UGK_CALL(ugk_memcpy_async(&st, StatusPtr(this, stream), sizeof(st), stream));
  UGK_CALL(ugk_stream_sync(stream));
  CHECK_EQ(st, 0u) << what << ": table maintenance kernel reported status 0x" << std::hex << st
                   << " (1 key out of range, 2 table full, 4 duplicate key, 8 evict of absent key)";
}

void CacheEntryManager::ReturnOffset(TensorPtr new_offsets) {
  CHECK(new_offsets->Ctx().device_type == kCPU);
  const size_t old_num = _free_offsets->NumItem();
  _free_offsets->ForceScale(kI32, {old_num + new_offsets->NumItem()}, CPU_CLIB(), "");
  memcpy(_free_offsets->Ptr<IdType>() + old_num, new_offsets->Data(), new_offsets->NumItem() * sizeof(IdType));
}

TensorPtr CacheEntryManager::ReserveOffsetFront(IdType n) {
  // the reference insists on one slot more than it takes (cache_hashtable.cuh:648), which a table so small that the
  // 0.1 % of spare capacity rounds to no slot at all (capacity == cached rows) can never offer; taking every free
  // slot is fine
  CHECK(_free_offsets->Shape()[0] >= n) << "free cache slots exhausted: " << _free_offsets->Shape()[0] << " < " << n;
  TensorPtr ret = Tensor::CopyBlob(_free_offsets->CPtr<IdType>(), kI32, {(size_t)n}, CPU_CLIB(), CPU_CLIB(), "");
  const size_t rest = _free_offsets->NumItem() - n;
  memmove(_free_offsets->Ptr<IdType>(), _free_offsets->Ptr<IdType>() + n, rest * sizeof(IdType));
  _free_offsets->ForceScale(kI32, {rest}, CPU_CLIB(), "");
  return ret;
}

TensorPtr CacheEntryManager::SortedDifference(const IdType *a, size_t na, const IdType *b, size_t nb) {
  const int nthr = std::max(1, RunConfig::solver_omp_thread_num_per_gpu);
  const size_t chunk = (na + nthr - 1) / nthr;
  std::vector<size_t> counts(nthr + 1, 0);
  // thread t owns a[lo, hi) and walks b from the first element not below a[lo]
  auto walk = [&](int t, IdType *dst) -> size_t {
    const size_t lo = std::min(na, chunk * t), hi = std::min(na, chunk * (t + 1));
    if (lo >= hi) return 0;
    size_t j = std::lower_bound(b, b + nb, a[lo]) - b;
    size_t out = 0;
    for (size_t i = lo; i < hi; i++) {
      while (j < nb && b[j] < a[i]) j++;
      if (j < nb && b[j] == a[i]) continue;
      if (dst) dst[out] = a[i];
      out++;
    }
    return out;
  };
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) counts[t + 1] = walk(t, nullptr);
  for (int t = 0; t < nthr; t++) counts[t + 1] += counts[t];
  TensorPtr out = Tensor::Empty(kI32, {counts[nthr]}, CPU_CLIB(), "");
  IdType *dst = out->Ptr<IdType>();
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) walk(t, dst + counts[t]);
  return out;
}

void CacheEntryManager::DetectKeysForAllSource(TensorPtr nid_to_block, TensorPtr block_access_advise,
                                               int local_location_id, TensorPtr block_density, size_t num_total_item,
                                               TensorPtr *node_list_of_src, int num_gpu) {
  CHECK_EQ(block_access_advise->Shape().size(), (size_t)1);
  CHECK_LE(num_gpu, 8);
  const IdType *n2b = nid_to_block->CPtr<IdType>();
  const uint8_t *advise = block_access_advise->CPtr<uint8_t>();
  const size_t num_block = block_access_advise->Shape()[0];
  const int nthr = std::max(1, RunConfig::solver_omp_thread_num_per_gpu);
  const size_t chunk = (num_total_item + nthr - 1) / nthr;
  // One GPU is one list: with the usual two blocks "key k is read from the GPU" is the comparison n2b[k] == b for the
  // one block b the GPU serves, which the compiler turns into a vector compare over the whole key space; other
  // shapes go through the block -> source table.
  int only_block = -1;
  if (num_gpu == 1) {
    int served = 0;
    for (size_t blk = 0; blk < num_block; blk++)
      if (advise[blk] == 0) {
        served++;
        only_block = (int)blk;
      }
    if (served != 1) only_block = -1;
  }
  // two passes (count, then fill) so every list comes out in ascending key order
  std::vector<std::vector<size_t>> counts(num_gpu, std::vector<size_t>(nthr + 1, 0));
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(num_total_item, chunk * t), hi = std::min(num_total_item, chunk * (t + 1));
    if (only_block >= 0) {
      const IdType want = (IdType)only_block;
      size_t c = 0;
      for (size_t k = lo; k < hi; k++) c += n2b[k] == want;
      counts[0][t + 1] = c;
    } else {
      size_t c[8] = {0};
      for (size_t k = lo; k < hi; k++) {
        const int src = advise[n2b[k]];
        if (src < num_gpu) c[src]++;
      }
      for (int d = 0; d < num_gpu; d++) counts[d][t + 1] = c[d];
    }
  }
  for (int d = 0; d < num_gpu; d++) {
    for (int t = 0; t < nthr; t++) counts[d][t + 1] += counts[d][t];
    node_list_of_src[d] = Tensor::Empty(kI32, {counts[d][nthr]}, CPU_CLIB(), "");
  }
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(num_total_item, chunk * t), hi = std::min(num_total_item, chunk * (t + 1));
    if (only_block >= 0) {
      const IdType want = (IdType)only_block;
      IdType *dst = node_list_of_src[0]->Ptr<IdType>() + counts[0][t];
      for (size_t k = lo; k < hi; k++)
        if (n2b[k] == want) *dst++ = (IdType)k;
    } else {
      size_t pos[8];
      for (int d = 0; d < num_gpu; d++) pos[d] = counts[d][t];
      for (size_t k = lo; k < hi; k++) {
        const int src = advise[n2b[k]];
        if (src < num_gpu) node_list_of_src[src]->Ptr<IdType>()[pos[src]++] = (IdType)k;
      }
    }
  }
  (void)local_location_id;
  (void)block_density;
}

}  // namespace common
}  // namespace coll_cache_lib
