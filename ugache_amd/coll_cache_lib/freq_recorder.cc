#include "freq_recorder.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <sys/mman.h>
#ifdef _OPENMP
#include <parallel/algorithm>
#endif

#include "logging.h"
#include "run_config.h"

namespace coll_cache_lib {
namespace common {

void ContFreqBuf::add(const IdType &key, const CntT &cnt) {
  for (auto &e : entries) {
    if (e.key == key) {
      e.cnt += cnt;
      return;
    }
  }
  entries.push_back({key, cnt});
  buf = entries.data();
}

CntT ContFreqBuf::get(const IdType &key) const {
  for (auto &e : entries)
    if (e.key == key) return e.cnt;
  return 0;
}

void ContFreqBuf::sort_desc() {
  uint64_t *w = reinterpret_cast<uint64_t *>(entries.data());
#ifdef _OPENMP
  __gnu_parallel::sort(w, w + entries.size(), std::greater<uint64_t>());
#else  // a build without OpenMP (the thread-sanitizer one): same order, one thread
  std::sort(w, w + entries.size(), std::greater<uint64_t>());
#endif
  buf = entries.data();
}

void ContFreqBuf::select_top(size_t k) {
  // every rank word is distinct (the key sits in its low half), so the k best entries are one set
  uint64_t *w = reinterpret_cast<uint64_t *>(entries.data());
  if (k == 0 || k >= entries.size()) return;
#ifdef _OPENMP
  __gnu_parallel::nth_element(w, w + k, w + entries.size(), std::greater<uint64_t>());
#else
  std::nth_element(w, w + k, w + entries.size(), std::greater<uint64_t>());
#endif
  buf = entries.data();
}

void ContFreqBuf::GetLegacyFreqRank(LegacyFreqBuf *output, size_t total_num_node) const {
  output->rank_vec.resize(total_num_node);
  output->freq_vec.assign(total_num_node, 0);
  std::vector<uint8_t> seen(total_num_node, 0);
  const size_t m = entries.size();
  CHECK_LE(m, total_num_node);
  for (size_t r = 0; r < m; r++) {
    CHECK_LT(entries[r].key, total_num_node);
    output->rank_vec[r] = entries[r].key;
    output->freq_vec[r] = entries[r].cnt;
    seen[entries[r].key] = 1;
  }
  size_t pos = m;
  for (size_t k = 0; k < total_num_node; k++)
    if (!seen[k]) output->rank_vec[pos++] = (uint32_t)k;
  CHECK_EQ(pos, total_num_node);
}

namespace {
int ScanThreads() { return std::max(1, RunConfig::solver_omp_thread_num_per_gpu); }
}  // namespace

namespace {
constexpr size_t kHugePage = size_t(2) << 20;
size_t CounterBytes(size_t num_nodes) {
  return (std::max<size_t>(num_nodes, 1) * sizeof(CntT) + kHugePage - 1) / kHugePage * kHugePage;
}
/** Zeroed counters in an anonymous mapping: pages nobody counts in are never touched, and the mapping asks for huge
 *  pages, so a batch of keys spread over a table of gigabytes faults in and walks a thousand pages, not a million. */
CntT *MapCounters(size_t num_nodes) {
  const size_t bytes = CounterBytes(num_nodes);
  void *raw = mmap(nullptr, bytes + kHugePage, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  CHECK(raw != MAP_FAILED) << "no memory for the counters of " << num_nodes << " keys";
  // keep the 2 MiB-aligned part: give the rest back
  char *lo = static_cast<char *>(raw);
  char *p = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(lo) + kHugePage - 1) & ~uintptr_t(kHugePage - 1));
  if (p > lo) munmap(lo, p - lo);
  if (p + bytes < lo + bytes + kHugePage) munmap(p + bytes, lo + bytes + kHugePage - (p + bytes));
  madvise(p, bytes, MADV_HUGEPAGE);  // advice only: small pages serve as well, slower
  return reinterpret_cast<CntT *>(p);
}
void UnmapCounters(CntT *p, size_t num_nodes) {
  if (p) munmap(p, CounterBytes(num_nodes));
}
}  // namespace

FreqRecorder::FreqRecorder(size_t num_nodes, int local_id) : _num_nodes(num_nodes), _local_id(local_id) {
  CHECK(num_nodes < std::numeric_limits<IdType>::max() / 2);
  _live = MapCounters(num_nodes);
  _spare = MapCounters(num_nodes);
  _shared = MapCounters(num_nodes);
  global_cont_freq_buf = new ContFreqBuf;
}

FreqRecorder::~FreqRecorder() {
  delete global_cont_freq_buf;
  UnmapCounters(_live, _num_nodes);
  UnmapCounters(_spare, _num_nodes);
  UnmapCounters(_shared, _num_nodes);
}

template <typename KeyT>
void FreqRecorder::Record(const KeyT *input, size_t num_inputs) {
  std::lock_guard<std::mutex> g(_mu);
  CntT *cnt = _live;
  const size_t n_nodes = _num_nodes;
  bool bad = false;
  const auto row_of = [n_nodes](uint64_t key, bool *bad_key) -> uint64_t {
    const uint64_t k = RunConfig::RowOfKey(key);
    *bad_key = k >= n_nodes || (RunConfig::key_map_mul && key > RunConfig::key_map_mask);
    return k;
  };
  if (num_inputs > 65536) {
#pragma omp parallel for num_threads(RunConfig::solver_omp_thread_num_per_gpu) reduction(|| : bad)
    for (size_t i = 0; i < num_inputs; i++) {
      bool b;
      const uint64_t k = row_of((uint64_t)input[i], &b);
      if (b)
        bad = true;
      else
        __atomic_fetch_add(&cnt[k], 1u, __ATOMIC_RELAXED);
    }
  } else {
    // one thread under the recorder's lock: plain increments, which (unlike locked ones) leave the loads of later
    // keys free to run ahead; the counters of a large table are far apart in memory, so the one needed 16 keys from
    // now is asked for early
    for (size_t i = 0; i < num_inputs; i++) {
      bool b;
      if (i + 16 < num_inputs) {
        const uint64_t ahead = row_of((uint64_t)input[i + 16], &b);
        if (!b) __builtin_prefetch(&cnt[ahead], 1);
      }
      const uint64_t k = row_of((uint64_t)input[i], &b);
      if (b)
        bad = true;
      else
        cnt[k]++;
    }
  }
  if (num_inputs) _live_dirty = true;
  CHECK(!bad) << "FreqRecorder::Record: a key has no row among num_total_item=" << n_nodes;
}
template void FreqRecorder::Record<Id64Type>(const Id64Type *input, size_t num_inputs);
template void FreqRecorder::Record<IdType>(const IdType *input, size_t num_inputs);

void FreqRecorder::ScatterHandedOver(FreqEntryList &list, CntT *into) {
  const size_t n = list.size(), n_nodes = _num_nodes;
  const FreqEntry *e = list.data();
  bool bad = false;
#pragma omp parallel for num_threads(ScanThreads()) reduction(|| : bad) if (n > 65536)
  for (size_t i = 0; i < n; i++) {
    if (e[i].key >= n_nodes)
      bad = true;
    else
      __atomic_fetch_add(&into[e[i].key], e[i].cnt, __ATOMIC_RELAXED);
  }
  CHECK(!bad) << "FreqRecorder: a handed-over row is outside num_total_item=" << n_nodes;
  list.clear();
}

void FreqRecorder::BeginEntries() {
  std::lock_guard<std::mutex> g(_mu);
  if (_handed_over.empty()) return;
  // an earlier hand-over is still pending: its keys may come again, so it goes into the array now
  ScatterHandedOver(_handed_over, _live);
  _live_dirty = true;
}

void FreqRecorder::AddEntries(const FreqEntry *entries, size_t num_entries) {
  std::lock_guard<std::mutex> g(_mu);
  _handed_over.insert(_handed_over.end(), entries, entries + num_entries);
}

void FreqRecorder::LocalCombineToShared() {
  std::lock_guard<std::mutex> combine(_combine_mu);
  CntT *drained;
  {
    // the recording side goes on in the other array at once: the scan below runs beside it
    std::lock_guard<std::mutex> g(_mu);
    if (!_live_dirty) return;  // nothing was counted on the host: no scan
    drained = _live;
    _live = _spare;
    _spare = drained;
    _live_dirty = false;
  }
  CntT *shared = _shared;
  const size_t n = _num_nodes;
  if (!_shared_dirty && _direct.empty()) {
    // Nothing waits in the shared array: the counted keys leave the drained array as entries at once (count, size the
    // list, fill), instead of being added into the shared array, which was then counted and listed in two more passes
    // over the whole key space.  Ascending key order whatever the thread count, as GlobalCombine lists them.  Most
    // counters are zero: sixteen of them (one 64-byte line) are looked at as eight words first.
    static_assert(sizeof(CntT) == 4, "sixteen counters to a 64-byte line");
    typedef uint64_t __attribute__((may_alias)) Word;
    const int nthr = ScanThreads();
    const size_t chunk = ((n + nthr - 1) / nthr + 15) / 16 * 16;  // whole lines per thread
    auto for_each_counted = [&](size_t lo, size_t hi, auto &&fn) {
      size_t k = lo;
      for (; k + 16 <= hi; k += 16) {
        const Word *w = reinterpret_cast<const Word *>(drained + k);
        if ((w[0] | w[1] | w[2] | w[3] | w[4] | w[5] | w[6] | w[7]) == 0) continue;
        for (size_t j = k; j < k + 16; j++)
          if (drained[j]) fn(j);
      }
      for (; k < hi; k++)
        if (drained[k]) fn(k);
    };
    // One pass over the counters: every thread lists the counted keys of its part in a list of its own (sized by what
    // the last round found, not zeroed, grown if that was too little) and clears them; the lists are then copied end
    // to end.  (Counting first to size one list and filling it in a second pass read the 2 GB of counters of 500 M keys
    // twice: 0.042 s with 18 M keys counted, where this takes 0.037 s; what is left is one read of the counters and the
    // clearing of the counted ones at what the host's memory gives sixteen threads.)
    std::vector<FreqEntryList> part(nthr);
    const size_t guess = std::max<size_t>(1024, (_last_listed / nthr) * 3 / 2);
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
    for (int t = 0; t < nthr; t++) {
      FreqEntryList &mine = part[t];
      mine.resize(guess);
      size_t pos = 0;
      for_each_counted(std::min(n, chunk * t), std::min(n, chunk * (t + 1)), [&](size_t k) {
        if (pos == mine.size()) mine.resize(mine.size() * 2);
        mine[pos++] = {(IdType)k, drained[k]};
        drained[k] = 0;
      });
      mine.resize(pos);
    }
    std::vector<size_t> first(nthr + 1, 0);
    for (int t = 0; t < nthr; t++) first[t + 1] = first[t] + part[t].size();
    _direct.resize(first[nthr]);  // not zeroed (FreqEntryList)
    FreqEntry *out = _direct.data();
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
    for (int t = 0; t < nthr; t++) {
      if (!part[t].empty()) memcpy(out + first[t], part[t].data(), part[t].size() * sizeof(FreqEntry));
      FreqEntryList().swap(part[t]);
    }
    _last_listed = first[nthr];
    return;
  }
  if (!_direct.empty()) ScatterHandedOver(_direct, shared);  // an earlier round still waits as a list: both add up
  _shared_dirty = true;
#pragma omp parallel for num_threads(ScanThreads())
  for (size_t i = 0; i < n; i++) {
    if (drained[i]) {  // the recorded keys are a small part of the key space: write only where something was counted
      shared[i] += drained[i];
      drained[i] = 0;
    }
  }
}

void FreqRecorder::GlobalCombine() {
  std::lock_guard<std::mutex> combine(_combine_mu);
  FreqEntryList handed_over;
  {
    std::lock_guard<std::mutex> g(_mu);
    handed_over.swap(_handed_over);
  }
  auto &e = global_cont_freq_buf->entries;
  e.clear();
  if (!_direct.empty()) {
    if (!_shared_dirty && handed_over.empty()) {  // what LocalCombineToShared listed is the list
      e.swap(_direct);
      _direct.clear();
      global_cont_freq_buf->buf = e.data();
      LOG(INFO) << "freq recorder global combine: " << e.size() << " distinct keys";
      return;
    }
    ScatterHandedOver(_direct, _shared);  // keys may repeat across the lists: they add up in the array
    _shared_dirty = true;
  }
  if (!_shared_dirty) {
    // only handed-over entries (distinct keys): they are the list, whatever their order — Sort() follows
    const size_t n_nodes = _num_nodes;
    for (const auto &x : handed_over) CHECK_LT((size_t)x.key, n_nodes);
    e.swap(handed_over);
    global_cont_freq_buf->buf = e.data();
    LOG(INFO) << "freq recorder global combine: " << e.size() << " distinct keys (handed over)";
    return;
  }
  if (!handed_over.empty()) ScatterHandedOver(handed_over, _shared);
  _shared_dirty = false;
  // count, scan, fill: the entries come out in ascending key order whatever the thread count
  const int nthr = ScanThreads();
  const size_t n = _num_nodes, chunk = (n + nthr - 1) / nthr;
  CntT *shared = _shared;
  std::vector<size_t> first(nthr + 1, 0);
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(n, chunk * t), hi = std::min(n, chunk * (t + 1));
    size_t c = 0;
    for (size_t k = lo; k < hi; k++) c += shared[k] != 0;
    first[t + 1] = c;
  }
  for (int t = 0; t < nthr; t++) first[t + 1] += first[t];
  e.resize(first[nthr]);
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(n, chunk * t), hi = std::min(n, chunk * (t + 1));
    size_t pos = first[t];
    for (size_t k = lo; k < hi; k++)
      if (shared[k]) {
        e[pos++] = {(IdType)k, shared[k]};
        shared[k] = 0;  // the next round of counts starts from zero
      }
  }
  global_cont_freq_buf->buf = e.data();
  LOG(INFO) << "freq recorder global combine: " << e.size() << " distinct keys";
}

void FreqRecorder::SelectTop(size_t k) { global_cont_freq_buf->select_top(k); }

void FreqRecorder::Sort() {
  global_cont_freq_buf->sort_desc();
  auto &e = global_cont_freq_buf->entries;
  if (e.size() >= 5)
    LOG(INFO) << "top 5 freq is " << e[0].cnt << "," << e[1].cnt << "," << e[2].cnt << "," << e[3].cnt << ","
              << e[4].cnt;
}

}  // namespace common
}  // namespace coll_cache_lib
