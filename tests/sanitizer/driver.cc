// TEST INFRASTRUCTURE ONLY: drives the host library through its C boundary (include/coll_cache_c_api.h) on the CPU,
// linked against the CPU model of the kernel layer next to this file, so that the library's threads can run under
// AddressSanitizer / UBSan and ThreadSanitizer:
//   build -> blocking lookups on one thread  ||  hotness records + background refreshes on another
//         -> stream-ordered lookups on one stream  ||  a refresh on another stream
//         -> the serving loop (coll_cache_forward) with its own background refresh thread
//         -> stream-ordered lookups that a caller records into a graph on a stream of its own, a refresh on that stream,
//            the shutdown while the graph still lives (the model lists every call that breaks a rule of such a capture
//            or ties an object of the library to the caller's graph)
//         -> shutdown,
// once per table kind and per refresh kind (host lists / device bitmaps).  Every looked-up row is compared with the
// host table, so a refresh that reused a slot too early is also seen as a wrong row.
//
// usage: driver <FLAT|HASH> <host|device> [lookup steps per phase, default 150]
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#include "coll_cache_c_api.h"
#include "ugache_hip.h"
#include "ugk_cpu_model.h"

namespace {

constexpr size_t kRows = 20000, kDim = 32;  // 128-byte rows
float cell(size_t row, size_t col) { return (float)(row * 131 + col * 7) * 0.5f; }

std::vector<uint32_t> skewed_keys(std::mt19937_64 &g, size_t n, uint64_t shift) {
  // a hot set that moves with `shift`, so that every refresh has rows to evict and to insert
  std::vector<uint32_t> k(n);
  for (auto &x : k) {
    const uint64_t r = g();
    x = (r & 3) ? (uint32_t)((shift + (r >> 8) % (kRows / 5)) % kRows) : (uint32_t)((r >> 8) % kRows);
  }
  return k;
}

long check_rows(const float *table, const float *out, const uint32_t *keys, size_t n) {
  long bad = 0;
  for (size_t i = 0; i < n; ++i)
    if (memcmp(out + i * kDim, table + (size_t)keys[i] * kDim, kDim * sizeof(float)) != 0) ++bad;
  return bad;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc != 3 && argc != 4) {
    fprintf(stderr, "usage: %s <FLAT|HASH> <host|device> [steps]\n", argv[0]);
    return 2;
  }
  const int steps = argc == 4 ? atoi(argv[3]) : 150;
  const bool on_device = strcmp(argv[2], "device") == 0;
  setenv("COLL_HASH_TABLE", argv[1], 1);
  setenv("COLL_GPU_RECORD", on_device ? "1" : "0", 1);
  setenv("COLL_GPU_REFRESH", on_device ? "1" : "0", 1);
  setenv("SAMGRAPH_LOG_LEVEL", "warn", 0);

  const char *keys[] = {"cache_percentage", "_cache_policy", "num_device", "num_global_step_per_epoch", "num_epoch",
                        "num_total_item",   "omp_thread_num"};
  const char *vals[] = {"0.25", "13", "1", "10", "1", "20000", "4"};
  long bad_rows = 0;
  for (int round = 0; round < 2; ++round) {
    coll_cache_config(keys, vals, 7);
    float *table = static_cast<float *>(coll_cache_alloc_host_table(kRows * kDim * sizeof(float)));
    for (size_t r = 0; r < kRows; ++r)
      for (size_t c = 0; c < kDim; ++c) table[r * kDim + c] = cell(r, c);
    std::mt19937_64 g(17 + round);
    coll_cache_record_init(0);
    for (int b = 0; b < 20; ++b) {
      auto k = skewed_keys(g, 4096, 0);
      coll_cache_record(0, k.data(), k.size());
    }
    coll_cache_init_c(0, kRows, nullptr, nullptr, nullptr, table, /*kF32*/ 0, kDim, 0.25, nullptr);

    // 1. blocking lookups and records on this thread, background refreshes on another
    std::atomic<bool> stop{false};
    std::atomic<int> refreshes{0};
    std::thread refresher([&] {
      while (!stop.load()) {
        coll_cache_refresh(0, nullptr, /*foreground=*/0);
        refreshes.fetch_add(1);
        std::this_thread::sleep_for(std::chrono::milliseconds(2));
      }
    });
    std::vector<float> out(4096 * kDim);
    for (int step = 0; step < steps || refreshes.load() < 3; ++step) {
      auto k = skewed_keys(g, 1 + g() % 4096, (uint64_t)step * 97);
      if (!on_device) coll_cache_record(0, k.data(), k.size());
      coll_cache_lookup(0, k.data(), k.size(), out.data(), nullptr);
      bad_rows += check_rows(table, out.data(), k.data(), k.size());
      if (step > 100 * steps) break;
    }
    stop.store(true);
    refresher.join();

    // 2. stream-ordered lookups on the null stream while a refresh runs on a stream of its own
    {
      std::thread one_refresh([&] { coll_cache_refresh(0, nullptr, /*foreground=*/0); });
      std::vector<std::vector<uint32_t>> batches;
      std::vector<std::vector<float>> outs;
      for (int b = 0; b < 8; ++b) {
        batches.push_back(skewed_keys(g, 2048, 5000 + b));
        outs.emplace_back(2048 * kDim);
      }
      for (int b = 0; b < 8; ++b)
        coll_cache_lookup_async(0, batches[b].data(), batches[b].size(), outs[b].data(), nullptr);
      coll_cache_lookup_wait(0, nullptr);
      one_refresh.join();
      for (int b = 0; b < 8; ++b) bad_rows += check_rows(table, outs[b].data(), batches[b].data(), batches[b].size());
    }

    // 3. wide keys, the distinct-keys lookup, a foreground refresh
    {
      std::vector<int64_t> k64(3000);
      std::vector<uint32_t> k32(3000), inverse(3000);
      for (size_t i = 0; i < k64.size(); ++i) k32[i] = (uint32_t)(k64[i] = (int64_t)(g() % (kRows / 50)));
      if (!on_device) coll_cache_record_i64(0, k64.data(), k64.size());
      coll_cache_lookup_i64(0, k64.data(), k64.size(), out.data(), nullptr);
      bad_rows += check_rows(table, out.data(), k32.data(), k32.size());
      coll_cache_refresh(0, nullptr, /*foreground=*/1);
      const size_t nu = coll_cache_lookup_unique(0, k32.data(), k32.size(), out.data(), inverse.data(), nullptr);
      for (size_t i = 0; i < k32.size(); ++i)
        if (inverse[i] >= nu ||
            memcmp(out.data() + (size_t)inverse[i] * kDim, table + (size_t)k32[i] * kDim, kDim * sizeof(float)) != 0)
          ++bad_rows;
    }

    // 4. the serving loop with its own background refresh thread
    coll_cache_forward_config(1, 7, 0.25, 1);
    for (int step = 0; step < std::max(steps / 2, 24); ++step) {
      auto k = skewed_keys(g, 3000, 9000 + (uint64_t)step * 53);
      if (step % 3 == 2) {  // a step that is enqueued and left (it blocks where the prefix is counted on the host)
        coll_cache_forward_async(0, k.data(), k.size(), out.data(), nullptr);
        coll_cache_lookup_wait(0, nullptr);
      } else {
        coll_cache_forward(0, k.data(), k.size(), out.data(), nullptr);
      }
      bad_rows += check_rows(table, out.data(), k.data(), k.size());
    }
    // 5. pooled lookups (segments of ids combined per sample): plain, as steps of the serving loop, stream-ordered
    for (int step = 0; step < 8; ++step) {
      auto k = skewed_keys(g, 2000, 20000 + (uint64_t)step * 31);
      std::vector<int64_t> off(1, 0);
      while ((size_t)off.back() < k.size()) off.push_back(std::min<int64_t>((int64_t)k.size(), off.back() + (int64_t)(g() % 6)));
      std::vector<float> w(k.size());
      for (auto &x : w) x = 0.5f + (float)(g() % 100) / 100.f;
      const size_t n_rows = off.size() - 1;
      const int combiner = step % 3;
      if (step < 3)
        coll_cache_lookup_pooled(0, k.data(), off.data(), step == 1 ? nullptr : w.data(), n_rows, k.size(), combiner, 4,
                                 out.data(), nullptr);
      else if (step < 6)
        coll_cache_forward_pooled(0, k.data(), off.data(), w.data(), n_rows, k.size(), combiner, 4, out.data(), nullptr);
      else {
        // the offsets made by the library from the row of every id
        std::vector<int64_t> row_of(k.size()), made(off.size(), -1);
        for (size_t r = 0; r < n_rows; ++r)
          for (int64_t j = off[r]; j < off[r + 1]; ++j) row_of[j] = (int64_t)r;
        coll_cache_segment_offsets(0, row_of.data(), row_of.size(), n_rows, made.data(), nullptr);
        if (made != off) ++bad_rows;
        coll_cache_lookup_pooled_async(0, k.data(), made.data(), w.data(), n_rows, k.size(), combiner, 4, out.data(),
                                       nullptr);
        coll_cache_lookup_wait(0, nullptr);
      }
      for (size_t r = 0; r < n_rows; ++r)
        for (size_t c = 0; c < kDim; ++c) {
          double sum = 0, den = 0;
          for (int64_t j = off[r]; j < off[r + 1]; ++j) {
            const double wj = step == 1 ? 1.0 : w[j];
            sum += wj * table[(size_t)k[j] * kDim + c];
            den += combiner == 2 ? wj * wj : wj;
          }
          if (combiner == 2) den = std::sqrt(den);
          const double want = combiner == 0 ? sum : den != 0 ? sum / den : 0.0;
          if (std::fabs(out[r * kDim + c] - want) > 1e-4 * (1.0 + std::fabs(want))) ++bad_rows;
        }
    }
    // 6. a caller records stream-ordered lookups, plain and pooled, and a serving step into a graph on its own stream.
    //    With the hotness counted on the device the lookups count inside that graph; nothing of the library but kernels
    //    on the caller's stream may take part in the capture.
    void *caller_stream = nullptr;
    std::vector<void *> extra_streams;
    int graph = 0;
    {
      if (ugk_stream_create(&caller_stream) != 0) return 1;
      const uint32_t marked = 4242;  // a key every captured batch holds 64 times
      auto k = skewed_keys(g, 2048, 31000);
      for (size_t i = 0; i < 64; ++i) k[i * 7] = marked;
      std::vector<int64_t> off(1, 0);
      while ((size_t)off.back() < k.size()) off.push_back(std::min<int64_t>((int64_t)k.size(), off.back() + 4));
      std::vector<float> pooled((off.size() - 1) * kDim), plain(k.size() * kDim), step_out(k.size() * kDim);
      coll_cache_lookup_wait(0, nullptr);
      coll_cache_forward_join();  // the foreground refresh below must not meet one of the serving loop's
      if (ugk_model_capture_begin(caller_stream) != 0) return 1;
      coll_cache_lookup_async(0, k.data(), k.size(), plain.data(), caller_stream);
      coll_cache_lookup_pooled_async(0, k.data(), off.data(), nullptr, off.size() - 1, k.size(), 0, 4, pooled.data(),
                                     caller_stream);
      coll_cache_forward_async(0, k.data(), k.size(), step_out.data(), caller_stream);
      if (ugk_model_capture_end(caller_stream, &graph) != 0) return 1;
      coll_cache_lookup_wait(0, caller_stream);
      bad_rows += check_rows(table, plain.data(), k.data(), k.size());
      bad_rows += check_rows(table, step_out.data(), k.data(), k.size());
      for (size_t r = 0; r + 1 < off.size(); ++r)
        for (size_t c = 0; c < kDim; ++c) {
          double sum = 0;
          for (int64_t j = off[r]; j < off[r + 1]; ++j) sum += table[(size_t)k[j] * kDim + c];
          if (std::fabs(pooled[r * kDim + c] - sum) > 1e-4 * (1.0 + std::fabs(sum))) ++bad_rows;
        }
      // an eager lookup and a foreground refresh on the stream the graph was recorded on
      coll_cache_lookup_async(0, k.data(), k.size(), plain.data(), caller_stream);
      coll_cache_lookup_wait(0, caller_stream);
      coll_cache_refresh(0, caller_stream, /*foreground=*/1);
      coll_cache_lookup(0, k.data(), k.size(), plain.data(), caller_stream);
      bad_rows += check_rows(table, plain.data(), k.data(), k.size());
      if (on_device) {
        // the two plain lookups and the pooled one counted every key, the serving step its recorded quarter: the marked
        // key was counted at least 3 x 64 times by launches inside the capture
        coll_cache_lookup_async(0, k.data(), k.size(), plain.data(), caller_stream);  // counted eagerly: 64 more
        coll_cache_lookup_wait(0, caller_stream);
        std::vector<uint32_t> rk(kRows), rc(kRows);
        const size_t n = coll_cache_rank_hotness(0, rk.data(), rc.data(), kRows);
        uint32_t seen = 0;
        for (size_t i = 0; i < n; ++i)
          if (rk[i] == marked) seen = rc[i];
        if (seen < 64) {
          fprintf(stderr, "the marked key was counted %u times after the refresh, 64 expected from the last lookup\n", seen);
          return 1;
        }
      }
      // stream-ordered lookups on two streams with no wait between them: the second must not file rows in the stage the
      // first may still be writing (the model reports two unordered writers of one stage)
      void *second_stream = nullptr;
      if (ugk_stream_create(&second_stream) != 0) return 1;
      coll_cache_lookup_async(0, k.data(), k.size(), plain.data(), caller_stream);
      coll_cache_lookup_async(0, k.data(), k.size(), step_out.data(), second_stream);
      coll_cache_lookup_wait(0, second_stream);
      coll_cache_lookup_wait(0, caller_stream);
      bad_rows += check_rows(table, plain.data(), k.data(), k.size());
      bad_rows += check_rows(table, step_out.data(), k.data(), k.size());
      coll_cache_refresh(0, caller_stream, /*foreground=*/1);  // also waits for, and forgets nothing of, both streams
      extra_streams.push_back(second_stream);
      if (round == 1) ugk_model_graph_destroy(graph);  // round 0 shuts down while the caller still holds its graph
    }
    const uint64_t done = coll_cache_forward_join();
    uint64_t info[8];
    coll_cache_get_info(0, info);
    printf("round %d: %d background refreshes, %llu from the serving loop, %llu table rebuilds, %llu rows cached of "
           "%llu slots, %ld bad rows\n",
           round, refreshes.load(), (unsigned long long)done, (unsigned long long)info[7],
           (unsigned long long)info[1], (unsigned long long)info[0], bad_rows);
    if (done == 0 || refreshes.load() < 3) {
      fprintf(stderr, "the refreshes this run is about did not happen\n");
      return 1;
    }
    coll_cache_shutdown();
    coll_cache_free_host_table(table);
    ugk_model_graph_destroy(graph);
    ugk_stream_destroy(caller_stream);
    for (void *st : extra_streams) ugk_stream_destroy(st);
    char text[4096];
    if (const size_t broken = ugk_model_violations(text, sizeof(text))) {
      fprintf(stderr, "%zu calls broke a rule that the model of the kernel layer checks:\n%s", broken, text);
      return 1;
    }
    ugk_model_reset();
  }
  if (bad_rows) {
    fprintf(stderr, "%ld looked-up rows differ from the host table\n", bad_rows);
    return 1;
  }
  printf("OK\n");
  return 0;
}
