// Hotness counting on the host: the input of the frequency-ranked cache fill and of refresh.
// Same role and call sequence as coll_cache_lib/freq_recorder.{h,cc} of the reference
// (Record -> LocalCombineToShared -> GlobalCombine -> Sort, freq_recorder.cc:227-293) and the same rank order:
// entries {key, cnt} compared as the 64-bit word (cnt << 32 | key), descending, i.e. higher count first and,
// among equal counts, the larger key first.  Keys are dense ids below num_nodes, so counts live in one flat
// array updated with atomic adds instead of per-thread hash maps.
#pragma once

#include <cstdint>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"

namespace coll_cache_lib {
namespace common {

using CntT = IdType;
using OffT = uint32_t;

struct FreqEntry {
  IdType key;
  CntT cnt;
};
static_assert(sizeof(FreqEntry) == 8, "FreqEntry is sorted as one 64-bit word");

// a vector whose resize() leaves new elements as they are: lists of tens of millions of entries are sized first and
// filled by many threads afterwards, and zeroing them in between on one thread would cost as much as the fill
template <typename T>
struct DefaultInitAllocator : std::allocator<T> {
  template <typename U>
  struct rebind {
    using other = DefaultInitAllocator<U>;
  };
  using std::allocator<T>::allocator;
  template <typename U>
  void construct(U *p) noexcept {
    ::new (static_cast<void *>(p)) U;
  }
  template <typename U, typename... Args>
  void construct(U *p, Args &&...args) {
    ::new (static_cast<void *>(p)) U(std::forward<Args>(args)...);
  }
};
using FreqEntryList = std::vector<FreqEntry, DefaultInitAllocator<FreqEntry>>;

struct LegacyFreqBuf {
  std::vector<uint32_t> rank_vec, freq_vec;
};

// Distinct observed keys with their counts; after FreqRecorder::Sort() in rank order.
struct ContFreqBuf {
  FreqEntryList entries;
  FreqEntry *buf = nullptr;  // == entries.data()
  size_t size() const { return entries.size(); }
  void add(const IdType &key, const CntT &cnt);  // linear probe over `entries`; for small hand-built buffers
  CntT get(const IdType &key) const;
  // all num_node keys in rank order: observed keys first, then the never-seen ones in ascending key order
  // (the reference appends them in a thread-dependent order, freq_recorder.cc:305-333)
  void GetLegacyFreqRank(LegacyFreqBuf *output, size_t total_num_node) const;
  void sort_desc();
  // the k best-ranked entries in front (in no particular order), the rest behind them: what a placement of k keys
  // needs of the order, in linear time; k >= size() leaves the list as it is
  void select_top(size_t k);
};

class FreqRecorder {
 public:
  FreqRecorder(size_t num_nodes, int local_id);
  ~FreqRecorder();
  template <typename KeyT>
  void Record(const KeyT *inputs, size_t num_input);
  // Counts gathered elsewhere (the device-side counters).  BeginEntries opens one hand-over; the AddEntries calls that
  // follow bring entries whose keys are distinct within the hand-over.  As long as nothing was recorded on the host
  // the entries are kept as a list and become the ranking input directly, so a refresh driven by the device-side
  // counters never scans the per-key arrays of the whole key space.
  void BeginEntries();
  void AddEntries(const FreqEntry *entries, size_t num_entries);
  void LocalCombineToShared();
  void GlobalCombine();
  void Sort();
  void SelectTop(size_t k);
  inline size_t NumNodes() const { return _num_nodes; }
  // true when counts wait here for the next ranking (recorded on the host, or handed over from the device)
  bool HasCounts() {
    std::lock_guard<std::mutex> combine(_combine_mu);
    std::lock_guard<std::mutex> g(_mu);
    return _live_dirty || _shared_dirty || !_handed_over.empty() || !_direct.empty();
  }
  ContFreqBuf *global_cont_freq_buf;

 private:
  size_t _num_nodes;
  int _local_id;
  // one counter per key of the key space, in anonymous mappings so that pages nobody counted in are never touched
  CntT *_live = nullptr;    // counts being recorded
  CntT *_spare = nullptr;   // all zero: takes the place of _live when LocalCombineToShared drains it
  CntT *_shared = nullptr;  // counts handed over by LocalCombineToShared
  bool _live_dirty = false, _shared_dirty = false;  // the array holds a non-zero counter
  FreqEntryList _handed_over;                      // entries of the open hand-over, not in the arrays
  FreqEntryList _direct;                           // what LocalCombineToShared listed straight from the counters
  size_t _last_listed = 0;                         // how many keys the last such listing found (sizes the next one's lists)
                                                    // (ascending, distinct keys), not in the shared array
  void ScatterHandedOver(FreqEntryList &list, CntT *into);
  // _mu guards what recording touches (_live, _live_dirty, _handed_over) and is held for one batch at most;
  // _combine_mu guards the rest (_spare, _shared, _shared_dirty, the ranked list) for the length of a scan of the
  // key space.  Where both are held, _combine_mu is taken first.
  std::mutex _mu, _combine_mu;
};

}  // namespace common
}  // namespace coll_cache_lib
