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

void CacheEntryManager::CreateHash(const std::function<MemHandle(size_t)> &allocator, size_t num_entries,
                                   StreamHandle stream) {
  const size_t nb = ugk_hash_buckets_for(num_entries, RunConfig::hash_load_factor);
  LOG(INFO) << "open-addressing lookup table for " << num_entries << " entries: " << nb << " buckets, "
            << ToReadableSize(nb * sizeof(ugk_bucket_t));
  _table_handle = allocator(nb * sizeof(ugk_bucket_t) + 128);
  CHECK_NOTNULL(_table_handle);
  void *base = Align128(_table_handle->ptr());
  _table = {2, 0, base, nb, RunConfig::key_map_inv, RunConfig::key_map_mask};
  UGK_CALL(ugk_hash_init(static_cast<ugk_bucket_t *>(base), nb, stream));
  RunConfig::use_flat_hashtable = false;
}

TensorPtr CacheEntryManager::TableKeysToDevice(TensorPtr host_rows, const std::function<MemHandle(size_t)> &allocator,
                                               Context ctx, StreamHandle stream) {
  if (RunConfig::key_map_mul == 0) return Tensor::CopyToExternal(host_rows, allocator, ctx, stream);
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
    UGK_CALL(ugk_table_lookup_u32(_table, keys->CPtr<uint32_t>(), keys->NumItem(), (uint32_t)cpu_location_id, nullptr,
                                  off->Ptr<uint32_t>(), stream));
}

void CacheEntryManager::InsertWithLoc(TensorPtr keys, TensorPtr off, int loc, StreamHandle stream) {
  CHECK_EQ(keys->NumItem(), off->NumItem());
  if (keys->Type() == kI64)
    UGK_CALL(ugk_table_insert_i64(_table, keys->CPtr<int64_t>(), off->CPtr<uint32_t>(), 0, (uint32_t)loc,
                                  keys->NumItem(), StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_insert_u32(_table, keys->CPtr<uint32_t>(), off->CPtr<uint32_t>(), 0, (uint32_t)loc,
                                  keys->NumItem(), StatusPtr(this, stream), stream));
}

void CacheEntryManager::InsertSeqOffWithLoc(TensorPtr keys, int loc, StreamHandle stream) {
  if (keys->Type() == kI64)
    UGK_CALL(ugk_table_insert_i64(_table, keys->CPtr<int64_t>(), nullptr, 0, (uint32_t)loc, keys->NumItem(),
                                  StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_insert_u32(_table, keys->CPtr<uint32_t>(), nullptr, 0, (uint32_t)loc, keys->NumItem(),
                                  StatusPtr(this, stream), stream));
}

void CacheEntryManager::Evict(TensorPtr keys_to_evict, StreamHandle stream) {
  if (keys_to_evict->Type() == kI64)
    UGK_CALL(ugk_table_evict_i64(_table, keys_to_evict->CPtr<int64_t>(), keys_to_evict->NumItem(),
                                 StatusPtr(this, stream), stream));
  else
    UGK_CALL(ugk_table_evict_u32(_table, keys_to_evict->CPtr<uint32_t>(), keys_to_evict->NumItem(),
                                 StatusPtr(this, stream), stream));
  if (_table.kind == 2) _num_tombstones += keys_to_evict->NumItem();
}

bool CacheEntryManager::MaybeRebuild(const std::function<MemHandle(size_t)> &allocator, Context ctx, int loc,
                                     StreamHandle stream) {
  if (_table.kind != 2) return false;
  if ((double)_num_tombstones <= RunConfig::hash_rebuild_tombstone_frac * (double)_table.size) return false;
  const size_t n = _cached_keys->NumItem();
  LOG(INFO) << "rebuilding the lookup table: " << _num_tombstones << " tombstones in " << _table.size << " buckets, "
            << n << " live keys";
  TensorPtr keys = TableKeysToDevice(_cached_keys, allocator, ctx, stream);
  TensorPtr offs = Tensor::EmptyExternal(kI32, {n}, allocator, ctx, "");
  if (n > 0) LookupOffset(keys, offs, stream);
  UGK_CALL(ugk_hash_init(static_cast<ugk_bucket_t *>(_table.table), _table.size, stream));
  if (n > 0) InsertWithLoc(keys, offs, loc, stream);
  CheckStatus(stream, "table rebuild");
  _num_tombstones = 0;
  _num_rebuilds++;
  return true;
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
  CHECK(_free_offsets->Shape()[0] > n) << "free cache slots exhausted: " << _free_offsets->Shape()[0] << " <= " << n;
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
