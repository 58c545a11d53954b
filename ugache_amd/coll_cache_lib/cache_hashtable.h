// Host-side owner of the GPU lookup table and of the cache-slot bookkeeping.  Same role and method names as
// CacheEntryManager in the reference (coll_cache_lib/cuda/cache_hashtable.cuh:529-849); the table itself
// lives behind the C-ABI of ugache_hip.h (flat table for dense ids, open addressing otherwise).
#pragma once

#include <cmath>
#include <cstring>
#include <functional>
#include <mutex>
#include <vector>

#include "common.h"
#include "logging.h"
#include "run_config.h"
#include "ugache_hip.h"

namespace coll_cache_lib {
namespace common {

constexpr IdType kEmptyPos = 0xffffffff;  // cache_hashtable.h:17

// packed (location, offset) value of the flat table, identical to cache_hashtable.h:20-28
struct EmbCacheOff {
  IdType data;
  EmbCacheOff(IdType loc, IdType off) { data = (loc << 28) + off; }
  IdType loc() const { return (data >> 28) & 0x0f; }
  IdType off() const { return data & 0x0fffffff; }
};

// cache_hashtable.cu:222-225; kept for the flat-vs-open-addressing decision rule
inline size_t TableSize(const size_t num, const size_t scale = 2) {
  const size_t next_pow2 = (size_t)1 << static_cast<size_t>(1 + std::log2((double)(num >> 1)));
  return next_pow2 << scale;
}

class CacheEntryManager {
 public:
  TensorPtr _cached_keys;   // host, u32: keys currently cached on this GPU
  // A build that made its key list on the device leaves the list there; the host's copy is fetched when something asks
  // for it (a refresh through the host, a table rebuild from the host's list, coll_cache_get_cached_keys).  While it
  // waits here _cached_keys is null and _host_lists_valid stays true: the list is the host's, just not copied yet.
  TensorPtr _cached_keys_on_device;
  TensorPtr HostCachedKeys(StreamHandle stream);
  TensorPtr _remote_keys;   // always empty with one GPU
  TensorPtr _free_offsets;  // host, u32: free cache slots, allocation sized for the whole capacity
  ugk_table_t _table = {0, 0, nullptr, 0, 0, 0};
  MemHandle _table_handle;
  // A rebuild publishes a new table while lookups run on another thread: they take their copy of the handle through
  // Table(), the rebuild swaps it under the same lock and frees the old buckets only once the lookups that may still
  // hold them have finished.
  mutable std::mutex _table_mu;
  ugk_table_t Table() const {
    std::lock_guard<std::mutex> guard(_table_mu);
    return _table;
  }
  MemHandle _status_handle;  // device status word for maintenance kernels
  IdType _cache_space_capacity = 0;
  size_t num_total_key = 0;
  int cpu_location_id = 1;
  int _device_id = 0;
  TensorPtr _keys_for_each_src[9];

  // allocate and clear the table (FlatHashTable / SimpleHashTable ctors, cache_hashtable.cu:432-457, 588-607)
  void CreateFlat(const std::function<MemHandle(size_t)> &allocator, size_t num_keys, StreamHandle stream);
  // 8-byte entries keyed by the host row when `num_entries` slots and `num_host_rows` rows fit them, else 16-byte
  // buckets keyed by the id (COLL_HASH_TABLE=HASH16 / HASH8 force one)
  void CreateHash(const std::function<MemHandle(size_t)> &allocator, size_t num_entries, size_t num_host_rows,
                  StreamHandle stream);
  static bool CompactHashFits(size_t num_slots, size_t num_host_rows);

  // Device copy of a host list of row numbers in the form the table is keyed by: the uint32 row numbers
  // themselves, or — in sparse-id mode — the int64 caller-side ids of those rows.
  TensorPtr TableKeysToDevice(TensorPtr host_rows, const std::function<MemHandle(size_t)> &allocator, Context ctx,
                              StreamHandle stream);
  // The methods below take device tensors of table keys (kI32 row numbers or kI64 ids, see above).
  // cuh:574-582 — off[i] = slot of keys[i] (the key's host row when absent)
  void LookupOffset(TensorPtr keys, TensorPtr off, StreamHandle stream);
  // cuh:601-608
  void InsertWithLoc(TensorPtr keys, TensorPtr off, int loc, StreamHandle stream);
  void InsertSeqOffWithLoc(TensorPtr keys, int loc, StreamHandle stream);
  // cuh:622-625
  void Evict(TensorPtr keys_to_evict, StreamHandle stream);
  // the same, and the evicted keys' slots leave the slot bitmap (SlotUsedBits) in the same launch: what LookupOffset +
  // ReturnOffset + Evict do together when the bookkeeping lives on the device
  void EvictRelease(TensorPtr keys_to_evict, StreamHandle stream);
  // cuh:635-655 — free-list: returned offsets go to the back, reservations come from the front
  void ReturnOffset(TensorPtr new_offsets);
  TensorPtr ReserveOffsetFront(IdType num_new_insert_keys);
  // aborts if a maintenance kernel flagged an error (duplicate insert, absent evict, full table ...)
  void CheckStatus(StreamHandle stream, const char *what);
  // Evictions leave tombstones in the open-addressing table.  Once they exceed
  // RunConfig::hash_rebuild_tombstone_frac of the buckets the cached keys are inserted, with their current slots, into
  // a second table of the same size, which then takes the place of the first.  Lookups racing with the rebuild keep
  // hitting in the old table until the swap; `wait_for_lookups` (may be empty) is called after the swap and must return
  // only when no lookup that took the old handle is still running, after which the old buckets are released.
  bool MaybeRebuild(const std::function<MemHandle(size_t)> &allocator, Context ctx, int loc, StreamHandle stream,
                    const std::function<void()> &wait_for_lookups);
  size_t _num_tombstones = 0;
  size_t _num_rebuilds = 0;

  // ---- the same bookkeeping on the device, for refreshes that never leave it -----------------------------------
  // Membership of the cache as one bit per row of the host table, occupancy of the cache as one bit per slot.  A
  // refresh on the device reads and updates these; a refresh on the host reads and updates _cached_keys and
  // _free_offsets.  Whichever ran last holds the truth, the other side is brought up to date when it is next needed.
  MemHandle _dev_in_cache, _dev_in_new;  // ceil(num_total_key / 64) words each
  MemHandle _dev_scratch_bits;           // as large, scratch of the placement
  MemHandle _dev_slot_used;              // ceil(capacity / 64) words
  MemHandle _dev_rank_ws, _dev_bm_ws;    // workspaces of ugk_rank_* / ugk_bitmap_*
  MemHandle _dev_bm_ws2;                 // a second one, so that two compactions can be counted before one wait
  MemHandle _dev_words;                  // pinned host words the kernels report counts in
  bool _build_bits_fresh = false;        // _dev_in_cache came from the build and nothing has changed the cache since
  uint32_t _ticket = 0;                  // last value written behind a stream for WaitByTicket / StatusAndWords
  TensorPtr _dev_list_buffer;            // scratch list for bringing either side up to date
  bool _dev_lists_valid = false;
  bool _host_lists_valid = true;
  size_t _num_cached = 0, _num_free = 0;  // valid when the host lists are not
  size_t NumCached() const {
    if (!_host_lists_valid) return _num_cached;
    if (_cached_keys_on_device) return _cached_keys_on_device->NumItem();
    return _cached_keys ? _cached_keys->NumItem() : 0;
  }
  size_t NumFree() const { return _host_lists_valid ? (_free_offsets ? _free_offsets->NumItem() : 0) : _num_free; }
  uint64_t *InCacheBits() const { return _dev_in_cache->ptr<uint64_t>(); }
  uint64_t *InNewBits() const { return _dev_in_new->ptr<uint64_t>(); }
  uint64_t *SlotUsedBits() const { return _dev_slot_used->ptr<uint64_t>(); }
  uint32_t *DevWords() const { return _dev_words->ptr<uint32_t>(); }
  // the table as 32-bit row numbers address it: a compact table stores its keys by the row, so with sparse ids the
  // lists of rows a refresh works on need no translation into ids
  ugk_table_t RowView() const {
    ugk_table_t t = _table;
    if (t.kind == 3) t.fb_mul = t.fb_mask = 0;
    return t;
  }
  // bitmaps from the host lists (allocates them on first use)
  void EnsureDeviceLists(const std::function<MemHandle(size_t)> &allocator, Context ctx, StreamHandle stream);
  // host lists from the bitmaps: cached rows ascending, free slots ascending
  void EnsureHostLists(const std::function<MemHandle(size_t)> &allocator, Context ctx, StreamHandle stream);
  // |S| and the first `limit` elements of S = set bits of (invert_a ? ~a : a) & ~b below nbits, ascending, in a device
  // list taken from `buffer` (grown when too small); blocks once, for the count
  TensorPtr CompactBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits, size_t limit,
                        TensorPtr &buffer, const std::function<MemHandle(size_t)> &allocator, Context ctx,
                        StreamHandle stream, size_t *total_out);
  // The two halves of CompactBits for callers that count several sets before they wait once: CountBits enqueues the
  // count of set `which` (0 or 1, each with a workspace of its own) and returns the pinned word it will land in;
  // EmitBits, after the bitmaps' count is known (waited for, or known by other means), enqueues the list of the first n
  // elements.
  volatile uint32_t *CountBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits, int which,
                               StreamHandle stream);
  TensorPtr EmitBits(const uint64_t *a, const uint64_t *b, bool invert_a, uint64_t nbits, int which, size_t n,
                     TensorPtr &buffer, const std::function<MemHandle(size_t)> &allocator, Context ctx,
                     StreamHandle stream);
  // A build that made its key list from a bitmap on the device hands the bitmap over: until a refresh changes the
  // cache it is the bitmap of cached rows, and the slots taken are 0 .. cached - 1 (the build fills them in list
  // order), so the first refresh finds both bitmaps without a pass over the key list and a lookup of every key.
  void AdoptBuildBits(MemHandle bits) {
    if (!_dev_in_cache) {
      _dev_in_cache = bits;
      _build_bits_fresh = bits != nullptr;
    }
  }
  void DropBuildBits() { _build_bits_fresh = false; }
  // the counts of both differences of two bitmaps (sets 0 = a & ~b and 1 = b & ~a) from one pass, into the pinned
  // words CountBits would write
  void CountDiff(const uint64_t *a, const uint64_t *b, uint64_t nbits, StreamHandle stream);
  // both differences of two bitmaps in one launch, counted as sets 0 (a & ~b) and 1 (b & ~a): the first n_ab and n_ba
  // elements into lists taken from the two buffers
  void EmitDiff(const uint64_t *a, const uint64_t *b, uint64_t nbits, size_t n_ab, size_t n_ba, TensorPtr &buffer_ab,
                TensorPtr &buffer_ba, TensorPtr *list_ab, TensorPtr *list_ba,
                const std::function<MemHandle(size_t)> &allocator, Context ctx, StreamHandle stream);
  // waits for `stream` by a ticket in the table's pinned words (spin_us == 0: by the runtime)
  void WaitByTicket(StreamHandle stream);
  // status words of the table's kernels and n_extra more device words (<= 30), brought to the host by one launch and
  // one wait by ticket; returns the table's status word, the extra words land in extra_out
  uint32_t StatusAndWords(const uint32_t *extra_dev, unsigned n_extra, uint32_t *extra_out, StreamHandle stream);
  // device list of host rows -> device list of table keys (the rows themselves, or their ids in sparse-id mode)
  TensorPtr RowsToTableKeys(TensorPtr rows_dev, TensorPtr &buffer, const std::function<MemHandle(size_t)> &allocator,
                            Context ctx, StreamHandle stream);
  // InsertWithLoc for device lists of host rows and their slots (raw pointers: parts of longer lists)
  void PublishRows(const uint32_t *rows_dev, const uint32_t *slots_dev, size_t n, int loc, TensorPtr &id_buffer,
                   const std::function<MemHandle(size_t)> &allocator, Context ctx, StreamHandle stream);

  // cuh:693-740 — keys of `inputs` satisfying cond, in input order (deterministic, unlike the reference's
  // thread-interleaved order)
  template <typename InputIterator, typename CondT>
  TensorPtr DetectKeysWithCond(InputIterator inputs, size_t num_input, CondT cond, size_t max_result_storage = 0) {
    const int nthr = std::max(1, RunConfig::solver_omp_thread_num_per_gpu);
    std::vector<size_t> counts(nthr + 1, 0);
    const size_t chunk = (num_input + nthr - 1) / nthr;
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
    for (int t = 0; t < nthr; t++) {
      size_t c = 0;
      const size_t lo = std::min(num_input, chunk * t), hi = std::min(num_input, chunk * (t + 1));
      for (size_t i = lo; i < hi; i++) c += cond(inputs[i]) ? 1 : 0;
      counts[t + 1] = c;
    }
    for (int t = 0; t < nthr; t++) counts[t + 1] += counts[t];
    const size_t total = counts[nthr];
    if (max_result_storage != 0) CHECK_LE(total, max_result_storage);
    TensorPtr out = Tensor::Empty(kI32, {total}, CPU_CLIB(), "");
    IdType *dst = out->Ptr<IdType>();
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
    for (int t = 0; t < nthr; t++) {
      size_t pos = counts[t];
      const size_t lo = std::min(num_input, chunk * t), hi = std::min(num_input, chunk * (t + 1));
      for (size_t i = lo; i < hi; i++)
        if (cond(inputs[i])) dst[pos++] = inputs[i];
    }
    return out;
  }

  // a \ b for two ascending key lists, ascending again: what DetectKeysWithCond computes when the condition is "not in
  // the other placement", as a parallel merge over the two lists instead of one random read per key into a per-key
  // array of the whole key space
  static TensorPtr SortedDifference(const IdType *a, size_t na, const IdType *b, size_t nb);

  // cuh:741-835 — per-source key lists from nid_to_block + this GPU's line of the access advise.
  // node_list_of_src[dev] is filled for dev in [0, num_gpu); keys whose source is the host are not listed.
  static void DetectKeysForAllSource(TensorPtr nid_to_block, TensorPtr block_access_advise, int local_location_id,
                                     TensorPtr block_density, size_t num_total_item, TensorPtr *node_list_of_src,
                                     int num_gpu = 1);
};

}  // namespace common
}  // namespace coll_cache_lib
