// Per-GPU cache state and the sessions that work on it.  Class names, public members and method signatures
// follow coll_cache_lib/cache_context.h of the reference (CacheContext :256-339, ExtractSession :420-512,
// RefreshSession :514-532) so that the facade and its callers are source compatible; the bodies are a
// single-GPU, HIP-stream design:
//   * no per-source worker threads and job syncers: the calling thread enqueues the classify kernel on the
//     caller's stream and the two per-source gathers on two library-owned streams, ordered by events;
//   * no host round trip between lookup and gather: group sizes stay in device memory, the gathers read them;
//   * one blocking synchronisation per lookup (the API stays synchronous: output is complete on return).
#pragma once

#include <atomic>
#include <cstdint>
#include <functional>
#include <memory>
#include <mutex>
#include <vector>

#include "cache_hashtable.h"
#include "common.h"
#include "freq_recorder.h"
#include "profiler.h"
#include "run_config.h"
#include "timer.h"
#include "ugache_hip.h"

namespace coll_cache_lib {

using namespace common;

class CollCache;
class ExtractSession;
class RefreshSession;

class CacheContext {
 public:
  std::atomic<size_t> progress{0};  // completed lookups; refresh waits on it (cache_context.h:258)

 private:
  BarHandle _barrier;
  Context _trainer_ctx;
  DataType _dtype = kF32;
  size_t _dim = 0;
  size_t _row_bytes = 0;
  int _num_location = -1;
  int _cpu_location_id = -1;
  int _local_location_id = -1;
  size_t _cache_nbytes = 0;
  size_t _cache_nodes = 0;
  size_t _cache_space_capacity = 0;  // rows
  size_t _num_total_nodes = 0;
  std::shared_ptr<CollCache> _coll_cache;
  CacheEntryManager *_new_hash_table = nullptr;
  // per location: [local] = cache in HBM, [cpu] = host table (cache_context.h:285)
  std::vector<void *> _device_cache_data;
  MemHandle _device_cache_data_local_handle;
  std::function<MemHandle(size_t)> _gpu_mem_allocator;
  std::function<MemHandle(size_t)> _eager_gpu_mem_allocator;

  friend class ExtractSession;
  friend class RefreshSession;
  friend class CollCache;

  inline bool IsDirectMapping() { return _new_hash_table == nullptr; }

  void build_no_cache(int location_id, std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_data, DataType dtype,
                      size_t dim, Context gpu_ctx, StreamHandle stream = nullptr);
  void build_full_cache(int location_id, std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_data, DataType dtype,
                        size_t dim, Context gpu_ctx, size_t num_total_nodes, StreamHandle stream = nullptr);
  // bits_out (optional): receives the bitmap the list was compacted from (bit r = row r is cached)
  TensorPtr KeyListOnDevice(TensorPtr top_rows, size_t num_extra, size_t num_rows, StreamHandle stream,
                            MemHandle *bits_out = nullptr);
  void build_with_advise_new_hash(int location_id, std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_data,
                                  DataType dtype, size_t dim, Context gpu_ctx, double cache_percentage,
                                  StreamHandle stream = nullptr);

 public:
  CacheContext(BarHandle barrier) : _barrier(barrier) {}
  ~CacheContext();
  void build(std::function<MemHandle(size_t)> gpu_mem_allocator, int location_id,
             std::shared_ptr<CollCache> coll_cache_ptr, void *cpu_data, DataType dtype, size_t dim, Context gpu_ctx,
             double cache_percentage, StreamHandle stream = nullptr);
  // introspection used by tests and reports
  size_t CacheCapacityRows() const { return _cache_space_capacity; }
  size_t CachedRows() const { return _cache_nodes; }
  size_t RowBytes() const { return _row_bytes; }
  int TableKind() const { return _new_hash_table ? _new_hash_table->_table.kind : 0; }
  const CacheEntryManager *EntryManager() const { return _new_hash_table; }
  // brings the host-side key and slot lists up to date after a refresh on the device (not while a refresh runs)
  void SyncHostLists() {
    if (_new_hash_table) _new_hash_table->EnsureHostLists(_eager_gpu_mem_allocator, _trainer_ctx, nullptr);
  }
};

class ExtractSession {
  // words of the device-side state block (64 zero-filled uint32)
  enum StateWord { kStCounts0 = 0, kStCounts1 = 2, kStStatus = 4, kStNumUnique = 5, kStDrainEntries = 6 };
  // words of the pinned host mirror the kernels write; [1] and [2] are indexed 1 + location
  enum MirrorWord { kMirError = 0, kMirGroupSizes = 1, kMirNumUnique = 3, kMirDrainCount = 4, kMirDrainMore = 5,
                    kMirSkipCount = 6, kMirTicket = 7 };
  std::shared_ptr<CacheContext> _cache_ctx;
  MemHandle _idx_handle;          // ugk_idx_t[n], from the caller's allocator, regrown on demand
  MemHandle _state_handle;        // device: two counter pairs + status word
  MemHandle _host_mirror_handle;  // pinned host, written by the kernels: [0] error flag, [1] #local, [2] #host
  uint32_t *_counts[2] = {nullptr, nullptr};
  uint32_t *_status = nullptr;
  uint32_t *_host_mirror = nullptr;
  int _cur = 0;
  StreamHandle _local_ext_stream = nullptr;
  StreamHandle _cpu_ext_stream = nullptr;
  void *_ev_classified = nullptr, *_ev_local_done = nullptr, *_ev_cpu_done = nullptr;
  void *_ev_t[4] = {nullptr, nullptr, nullptr, nullptr};
  unsigned _cpu_blocks = 32;        // workgroups of the host-link gather on its own (CU-confined) stream
  unsigned _cpu_blocks_inline = 32; // ... when it runs on the caller's stream instead
  bool _host_on_main = false;  // host-link gather on the caller's stream (short miss groups) or on the confined stream
  uint32_t _group_offset[3] = {0, 0, 0};
  // deduplication in front of the extraction (RunConfig::dedup_keys)
  MemHandle _dedup_ws;   // epoch-tagged set, zero-filled when allocated
  MemHandle _dedup_out;  // [n] distinct keys | [n] inverse | [n] first occurrence
  size_t _dedup_ws_bytes = 0;  // size the set was laid out and zero-filled for
  uint32_t _dedup_epoch = 0;
  size_t _dedup_cap = 0;  // keys the three arrays are sized for (distinct keys take 8 bytes each whatever the type)
  template <typename KeyT>
  KeyT *DedupUnique() const { return _dedup_out->ptr<KeyT>(); }
  uint32_t *DedupInverse() const { return reinterpret_cast<uint32_t *>(_dedup_out->ptr<char>() + _dedup_cap * 8); }
  uint32_t *DedupRep() const { return DedupInverse() + _dedup_cap; }
  template <typename KeyT>
  size_t DedupKeys(const KeyT *nodes, size_t num_nodes, StreamHandle stream);

  // hotness counters on the device (RunConfig::gpu_record)
  MemHandle _hot_counts;         // uint32 per row of the host table
  MemHandle _hot_observed;       // one bit per row: its counter is above zero (kept when refreshes run on the device)
  uint64_t *ObservedBits() const { return _hot_observed ? _hot_observed->ptr<uint64_t>() : nullptr; }
  MemHandle _hot_entries;        // compact (count << 32 | row) list of one drain step
  MemHandle _hot_entries_host;   // pinned copy of it
  StreamHandle _record_stream = nullptr;  // record kernels and drains run here, beside the extraction
  void *_ev_rec_begin = nullptr, *_ev_rec_done = nullptr, *_ev_placed = nullptr;
  bool _record_pending = false;
  size_t _record_limit = SIZE_MAX;
  std::mutex _drain_mu;  // one drain at a time: they share the entry list and its pinned copy
  // held while a record kernel, or the passes of a placement, are enqueued on the record stream, so that no record
  // kernel lands between two passes and all of them see one state of the counters (a placement holds both)
  std::mutex _enqueue_mu;
  uint32_t *_state = nullptr;
  void JoinRecord(StreamHandle stream);
  void JoinRecordOnHost();
  size_t _num_lookups = 0;
  static constexpr size_t kHotDrainRows = 32u << 20;  // rows per drain step = capacity of the entry list
  template <typename KeyT>
  void RecordKeys(const KeyT *nodes, size_t num_nodes, StreamHandle stream, void *after);
  // How the keys of the lookup that is being enqueued get counted on the device: not at all, by a record kernel on
  // the session's record stream behind the event `after` (which the caller's stream has recorded), or by a record
  // kernel on the caller's own stream.  The last is for a lookup that the caller is recording into a HIP graph: no
  // stream and no event of the session may become part of a graph that the caller owns, replays and destroys when it
  // likes, so there the counting is one more kernel node of that graph, behind the extraction.
  struct RecordPlan {
    enum Kind { kNone, kRecordStream, kCallersStream } kind = kNone;
    void *after = nullptr;
    StreamHandle stream = nullptr;
  };
  RecordPlan RecordBegin(StreamHandle stream);
  template <typename KeyT>
  void RecordLaunch(const KeyT *nodes, size_t num_nodes, const RecordPlan &plan);
  bool _capture_query_refused_logged = false;
  std::atomic<bool> _counted_on_callers_stream{false};  // some lookup was recorded into a graph together with its counting
  // bound on the rows observed (counter above zero): what the last placement saw plus every key counted since
  std::atomic<uint64_t> _keys_counted_since{0};
  uint64_t _observed_known = UINT64_MAX;        // UINT64_MAX: no placement has looked yet
  const uint32_t *_observed_word = nullptr;     // pinned word the placement in flight writes the count to
  bool _placement_reset = false;

  MemHandle _mix_counts;           // pinned: one word per workgroup of the fused kernel, its two row counts
  uint32_t _mix_groups = 0;        // workgroups of the last fused launch
  bool _async_last_fused = false;  // the last stream-ordered lookup was a fused launch (its counts wait to be summed)
  void SumMixCounts();
  uint32_t _ticket = 0;  // last ticket a blocking lookup waited for (kMirTicket)
  void WaitForBatch(StreamHandle stream);
  // Rows that crossed the host link, kept for the next refresh (COLL_MISS_STAGE_ROWS): written by the fused extraction,
  // read by the refresh's row copy.  A foreground refresh runs while no lookup does and reads the stage the lookups
  // write.  A background refresh runs beside lookups, so there are two stages then: it switches the lookups over to
  // the other one, waits (as it does anyway before it reuses slots) for the lookups that may still write the one it
  // keeps, and reads that.  The second stage is allocated by the first background refresh.
  MemHandle _stage_rows[2], _stage_owner[2];
  ugk_stage_t _stages[2] = {{nullptr, nullptr, 0, 0, 0}, {nullptr, nullptr, 0, 0, 0}};
  ugk_stage_t _stage_launch = {nullptr, nullptr, 0, 0, 0};  // what a launch is handed: the active stage with a fresh tag
  std::atomic<int> _stage_active{0};
  size_t _stage_entries = 0;  // 0: no stage
  uint32_t _stage_epoch = 0;
  void AllocStage(int which, StreamHandle stream);
  // Called after the lookup has counted itself in flight (InFlight): a refresh that switched the stages before it
  // sampled that count then either sees this lookup in the count or this lookup sees the switch.
  // Rows are filed by the launches of one stream at a time: launches on one stream run one after the other, launches
  // on two streams may overlap, and two overlapping launches could both claim an entry and mix the bytes of two rows
  // in it.  A lookup on another stream than the last one that filed rows gets no stage while that one may still run
  // (a stream-ordered lookup that has not been waited for); a blocking lookup has finished when it returns.
  StreamHandle _stage_writer = nullptr;
  bool _stage_writer_busy = false;
  const ugk_stage_t *NextStage(StreamHandle stream, bool stream_ordered) {
    if (_stage_entries == 0) return nullptr;
    if (_stage_writer_busy && stream != _stage_writer) return nullptr;
    _stage_writer = stream;
    _stage_writer_busy = stream_ordered;
    _stage_launch = _stages[_stage_active.load()];
    if (++_stage_epoch == 0) _stage_epoch = 1;
    _stage_launch.epoch = _stage_epoch;
    return &_stage_launch;
  }
  size_t _async_pending = 0;       // stream-ordered lookups enqueued since the last Wait()
  size_t _async_last_nodes = 0;    // size of the last of them
  bool _async_swap_counts = false;  // the last of them counted ids read from HBM as "from the host table"
  // What a refresh has to see finished before it reuses the slots of evicted rows: blocking lookups are counted when
  // they start and when they end, the streams stream-ordered lookups were enqueued on are remembered (normally one).
  struct InFlight;
  std::atomic<size_t> _blocking_started{0}, _blocking_finished{0};
  std::mutex _async_mu;
  std::vector<StreamHandle> _async_streams;  // guarded by _async_mu
  bool _async_any = false;                   // the lookup thread's own: _async_stream_last is valid
  StreamHandle _async_stream_last = nullptr;
  void NoteAsyncStream(StreamHandle stream);
  template <typename KeyT>
  void ExtractFeatAsyncImpl(const KeyT *nodes, size_t num_nodes, void *output, StreamHandle stream);

  template <typename KeyT>
  void ExtractFeatImpl(const KeyT *nodes, size_t num_nodes, void *output, StreamHandle stream, uint64_t task_key);
  template <typename KeyT>
  size_t ExtractUniqueImpl(const KeyT *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                           StreamHandle stream, uint64_t task_key);
  template <typename KeyT>
  void ExtractPooledImpl(const KeyT *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                         size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream,
                         uint64_t task_key);
  template <typename KeyT>
  bool LaunchPooled(const KeyT *nodes, const int64_t *seg_off, const float *weights, size_t num_rows, size_t num_nodes,
                    int combiner, int elem_bytes, void *output, StreamHandle stream);
  template <typename KeyT>
  void ExtractPooledAsyncImpl(const KeyT *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                              size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream);
  // Where the outputs of the last lookups went.  A caller that hands the same buffer over every time (the reference's
  // adapter does, adapter.cc:204-237) finds its rows in the memory-side cache; one that rotates over more buffers than
  // that cache holds is better served by streaming stores, and the kernels are told so (ugk_set_output_hint).
  static constexpr int kOutRing = 8;
  const void *_out_ptr[kOutRing] = {nullptr};
  size_t _out_bytes[kOutRing] = {0};
  int _out_next = 0;
  int _out_hint = UGK_OUTPUT_AUTO;
  void NoteOutput(const void *output, size_t nbytes);
  bool _skip_dedup = false;  // the keys handed to ExtractFeatImpl are distinct already
  // COLL_SKIP_LOCAL=1: the keys the cache does not serve, compacted in their order, and the scratch around them
  MemHandle _skip_handle;
  void *_skip_keys = nullptr;
  template <typename KeyT>
  size_t SelectNonLocal(const ugk_table_t &table, const KeyT *nodes, size_t num_nodes, StreamHandle stream);
  void EnsureIdx(size_t num_nodes);
  void CheckStatusWord(StreamHandle stream) const;

 public:
  ExtractSession(std::shared_ptr<CacheContext> cache_ctx);
  ~ExtractSession();
  // cache_context.h:510.  nodes: device pointer to num_nodes keys; output: device [num_nodes, dim]; blocking.
  void ExtractFeat(const IdType *nodes, const size_t num_nodes, void *output, StreamHandle stream,
                   uint64_t task_key);
  // same for 64-bit keys (dense ids below num_total_item); an extension over the reference
  void ExtractFeat64(const Id64Type *nodes, const size_t num_nodes, void *output, StreamHandle stream,
                     uint64_t task_key);
  // Lookup and per-sample combination of a multi-hot feature in one kernel (an extension; embedding_lookup_sparse
  // behind the TF2 sparse layer, sparse_lookup_layer.py:196-265): output[r, :] = the rows of the ids
  // nodes[seg_off[r] .. seg_off[r + 1]) times their weights (null: 1), summed (combiner 0), divided by the sum of the
  // weights (1) or by the root of the sum of their squares (2); elements are fp32 (elem_bytes 4) or fp16 (2), added in
  // fp32.  nodes, seg_off (num_rows + 1 int64 offsets), weights: device pointers; output: device [num_rows, dim];
  // blocking.  Rows must be multiples of 16 bytes of at most 4096.  The group sizes afterwards count ids.
  void ExtractPooled(const IdType *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                     size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream,
                     uint64_t task_key);
  void ExtractPooled64(const Id64Type *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                       size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream,
                       uint64_t task_key);
  // The offsets a pooled lookup takes, from the row of every entry of a sparse feature in row-major order:
  // seg_off[r] = entries whose row is below r, r = 0 .. num_rows.  One launch on `stream`, no wait; entries out of
  // order or outside [0, num_rows) are reported by the next lookup's status check.
  void SegmentOffsets(const int64_t *sorted_rows, size_t num_entries, size_t num_rows, int64_t *seg_off,
                      StreamHandle stream);
  // the same enqueued on `stream` without waiting (kernel launches only); Wait() completes it like a stream-ordered
  // plain lookup: status checked, group sizes of the last batch made available
  void ExtractPooledAsync(const IdType *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                          size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream);
  void ExtractPooledAsync64(const Id64Type *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                            size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream);
  // The distinct keys of the batch looked up once (an extension; the "unique -> lookup -> gather(idx)" of the TF2
  // layer, sparse_lookup_layer.py:196-209, with the unique inside): output[u, :] = row of the u-th distinct key
  // (in order of first claim, not sorted), inverse_out[i] = which distinct key position i holds, so that
  // output[inverse_out[i], :] is the row of nodes[i].  output needs room for num_nodes rows, inverse_out (device) for
  // num_nodes words.  Blocking.  Returns the number of distinct keys.
  size_t ExtractUnique(const IdType *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                       StreamHandle stream, uint64_t task_key);
  size_t ExtractUnique64(const Id64Type *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                         StreamHandle stream, uint64_t task_key);
  // Stream-ordered variants (an extension; the reference's lookup always blocks): the kernels of the batch are
  // enqueued on `stream` and the call returns without waiting; `output` is complete for whatever is enqueued on the
  // same stream afterwards.  All stream-ordered lookups of a session must use one stream.  Error flags, group sizes
  // and profiler values are collected by Wait().  Batches the fused / direct kernels cannot take (deduplication on,
  // rows not multiples of 16 bytes, a factored mode selected) run through the blocking path instead.
  void ExtractFeatAsync(const IdType *nodes, const size_t num_nodes, void *output, StreamHandle stream);
  void ExtractFeatAsync64(const Id64Type *nodes, const size_t num_nodes, void *output, StreamHandle stream);
  // blocks until every stream-ordered lookup enqueued so far has finished, aborts if one of them met a key outside
  // its table, and makes LastGroupOffset() describe the last of them
  void Wait(StreamHandle stream);
  // For a refresh, between evicting rows and overwriting their slots: returns once every lookup that may have
  // resolved a key to one of those slots has finished reading — the stream-ordered ones enqueued so far (a wait for
  // each stream they went to; the streams must still exist, so call Wait() before destroying one) and, unless
  // `foreground` says that no lookup runs beside the refresh, the blocking ones that had started (bounded by
  // `timeout_s`).  Lookups that start later see the evicted keys as misses and read the host table.
  // ordered_on (may be null): a stream the caller enqueues everything that follows on; lookups enqueued there are
  // ordered in front of it already and are not waited for on the host
  void WaitForLookupsInFlight(bool foreground, double timeout_s, const StreamHandle *ordered_on = nullptr);
  // {0, #local, n} of the last lookup — the reference's group_offset (cache_context.cu:825-847)
  const uint32_t *LastGroupOffset() const { return _group_offset; }
  // moves what the lookups have counted on the device since the last call into `recorder` (FreqRecorder::Record's
  // result for the same keys); safe to call from another thread while lookups run.  Returns the rows moved.
  size_t DrainHotness(FreqRecorder *recorder);
  // Ranks the rows by what the lookups have counted on the device (same order as FreqRecorder::Sort, never-counted
  // rows behind the counted ones in ascending order) and sets bit r of in_new_bits for the num_cached best rows.
  // Runs on the record stream, ordered against the counting of every lookup; `stream` waits for the result.
  // reset_counts: the next interval starts from zero, as after DrainHotness.  keep_bits (may be null): rows that
  // win ties at the last count that gets in (ugk_rank_place_keep).
  bool CountsOnDevice() const { return _hot_counts != nullptr; }
  // adds counts known on the host (entries with distinct or repeated rows) to the device-side counters
  void SeedHotness(const FreqEntry *entries, size_t num_entries);
  int DeviceId() const { return _cache_ctx->_trainer_ctx.device_id; }
  // what a foreground refresh may read rows from besides the host table (null: nothing)
  const ugk_stage_t *StageForRefresh(bool foreground, StreamHandle stream);
  // What changes, counted on the way when the placement can tell (DiffCount non-null and the return value true): the
  // two workspaces are left ready for ugk_bitmap_emit and totals_host[0..1] (pinned) receive the rows that leave and
  // that come in once `stream` has been waited for.  That is the case when fewer rows can have been observed than the
  // cache holds (the rows observed at the last placement plus the keys counted since stay below num_cached, no tie
  // rule, no counting inside a caller's graph): then no pass over the counters is made either.
  struct DiffCount {
    const uint64_t *cached_bits;
    void *evict_ws, *insert_ws;
    uint32_t *totals_host;  // three pinned words; [2] receives the rows observed
    uint32_t *status_dev;
  };
  bool PlaceOnDevice(size_t num_cached, uint64_t *in_new_bits, uint64_t *scratch_bits, const uint64_t *keep_bits,
                     void *rank_ws, bool reset_counts, const DiffCount *diff, StreamHandle stream);
  // after `stream` has been waited for: the host learns how many rows the placement saw observed
  void PlacementWaitedFor();
  // the device-side counting of the following lookups covers only the first `num_keys` keys of a batch
  // (the recorded prefix of LookupManager's record thread); SIZE_MAX, the default: the whole batch
  void SetRecordLimit(size_t num_keys) { _record_limit = num_keys; }
  // the pooled lookups that follow clip every looked-up row to this l2 norm before it is weighted (the max_norm of
  // the sparse layer, sparse_lookup_layer.py:95-140); 0, the default: no clipping
  void SetPooledMaxNorm(float max_norm) { _pool_max_norm = max_norm; }

 private:
  float _pool_max_norm = 0.f;

 public:
};

class RefreshSession {
 public:
  StreamHandle stream = nullptr;
  StreamHandle low_pri_stream = nullptr;  // a second default-priority stream: row copies of the refresh
  std::shared_ptr<CacheContext> _cache_ctx;
  void refresh_after_solve_main(bool foreground);
  // The whole refresh on the device (RunConfig::gpu_refresh): placement from the device-side hotness counters of
  // `session`, evict = cached & ~new and insert = new & ~cached as bitmap compactions, free slots from the slot bitmap;
  // then the same evict / wait / copy / insert steps as refresh_after_solve_new (cache_context.cu:3944-4107).
  void refresh_on_device(ExtractSession *session, size_t num_cached, bool foreground);
  // A placement ranked on the host, given as the ranked rows that are cached (distinct) plus `num_extra` of the lowest
  // other rows, applied through the same bitmaps and device lists (session may be null: no lookups to wait for).
  void refresh_from_ranked_rows(ExtractSession *session, TensorPtr top_rows, size_t num_extra, bool foreground);
  ~RefreshSession();

 private:
  void refresh_after_solve_new(bool foreground);
  void ApplyPlacedBits(ExtractSession *session, size_t num_cached, bool foreground, const ugk_stage_t *stage,
                       bool placed_from_counters, const char *how, double sync_s, common::Timer &t_phase);
  TensorPtr Empty1DReuse(TensorPtr &preserved_buffer, DataType dtype, std::vector<size_t> shape, Context ctx);
  TensorPtr CopyTo1DReuse(TensorPtr &preserved_buffer, TensorPtr src, Context ctx, StreamHandle stream);
  // step 5: lets one more lookup finish, so that no gather in flight still reads a slot about to be reused
  void WaitForOneLookup(ExtractSession *session, bool foreground, const StreamHandle *ordered_on = nullptr);
  uint32_t _rows_from_stage = 0;  // what status word 8 read after the last refresh on the device
  TensorPtr __rest_rows, __rest_slots;  // rows a background refresh did not find in the stage
 public:
  // rows the refreshes of this session have taken from the stage instead of the host table so far (blocks)
  uint64_t RowsFromStage();
 private:
  // copies the listed host rows into the listed cache slots and publishes them in the table (step 6): in one launch
  // each when in the foreground; behind running lookups in small throttled batches, every batch published as soon as
  // it has arrived, so the hit rate climbs while the refresh runs instead of at its end
  void CopyRowsIntoSlots(const uint32_t *rows_dev, const uint32_t *slots_dev, size_t num_rows, bool foreground,
                         StreamHandle copy_stream, const ugk_stage_t *stage);
  TensorPtr __publish_ids;  // table keys of the rows being published (sparse ids)
  TensorPtr __keys_buffer;
  TensorPtr __offs_buffer;
  TensorPtr __evict_rows, __insert_rows, __free_slots, __evict_ids, __evict_slots;
  TensorPtr __ranked_rows;  // device copy of the rows a host-ranked placement caches
  MemHandle _status_handle;
};

}  // namespace coll_cache_lib
