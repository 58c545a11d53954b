// Process-wide configuration, mirroring coll_cache_lib/run_config.{h,cc} of the reference for the fields the
// extraction path reads (run_config.h:30-111; LoadConfigFromEnv run_config.cc:84-172).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "common.h"

namespace coll_cache_lib {
namespace common {

// How ExtractFeat combines the two sources (run_config.h ConcurrentLinkImpl; only the variants that make
// sense with one GPU and its host are kept).
enum ConcurrentLinkImpl {
  kNoConcurrentLink = 0,  // host group, then local group, on the caller's stream
  kSMMaskPhase,           // the two groups as concurrent kernels on their own streams (SMMaskPhase / MPSPhase)
  kDirectNoGroup,         // default: one fused lookup+gather kernel, no partition (also SAMGRAPH_COLL_CACHE_NO_GROUP=DIRECT)
};

namespace coll_cache {
// Single-GPU slice of AsymmLinkDesc (coll_cache/asymm_link_desc.{h,cc}): no peer links, a compute budget for
// the host-miss gather and one for the local gather, and the bandwidth figures the placement model assumes.
struct AsymmLinkDesc {
  std::vector<std::vector<std::vector<int>>> link_src;  // [dst gpu][link][src gpus]; empty lists with one GPU
  std::vector<int> cpu_sm;     // workgroups given to the host-miss gather (the reference counts SMs)
  std::vector<int> cpu_cu;     // compute units the host-miss gather is confined to (0 = no confinement)
  std::vector<int> local_sm;   // 0 = fill the chip
  double local_bw_GBps = 0;    // HBM
  double cpu_bw_GBps = 0;      // host link
  std::string gpu_model;
  static AsymmLinkDesc AutoBuild(Context ctx);
};
}  // namespace coll_cache

struct RunConfig {
  static bool is_configured;
  static CachePolicy cache_policy;
  static double cache_percentage;
  static size_t num_device;
  static std::vector<int> device_id_list;
  static bool cross_process;
  static int worker_id;
  static uint64_t num_global_step_per_epoch;
  static uint64_t num_epoch;
  static uint64_t num_total_item;
  static int omp_thread_num;
  static int solver_omp_thread_num;
  static int solver_omp_thread_num_per_gpu;
  static int refresher_omp_thread_num;
  static int refresher_omp_thread_num_per_gpu;
  static size_t option_empty_feat;  // SAMGRAPH_EMPTY_FEAT mock tables are not supported: must stay 0
  static ConcurrentLinkImpl concurrent_link_impl;
  static size_t coll_cache_scale_nb;
  static bool use_flat_hashtable;
  static double coll_cache_hyperparam_T_local;
  static double coll_cache_hyperparam_T_cpu;
  static coll_cache::AsymmLinkDesc coll_cache_link_desc;
  // knobs of this implementation
  static bool device_key_list;         // COLL_DEVICE_KEY_LIST, default 1: a build gets its ascending list of cached
                                       // rows from a bitmap on the device instead of from a key -> block array
                                       // over the whole key space on the host
  static unsigned fill_limit_block;    // COLL_FILL_LIMIT_BLOCK, default 128: workgroups of a build's row copy over the
                                       // host link (0: as many as the rows fill)
  static double hash_load_factor;      // COLL_HASH_LOAD_FACTOR, default 0.7
  static int force_table_kind;         // COLL_HASH_TABLE=FLAT|HASH|HASH16|HASH8 -> 1|2|16|8, 0 = decide by size;
                                       // HASH picks the entry width itself, HASH16 / HASH8 name it (bytes)
  static size_t refresh_batch_rows;    // COLL_REFRESH_BATCH_ROWS, default 4092 (cache_context.cu:4057)
  static unsigned refresh_sleep_us;    // COLL_REFRESH_SLEEP_US, default 3000 (cache_context.cu:4069)
  static unsigned refresh_limit_block; // COLL_REFRESH_LIMIT_BLOCK, default 20 (cache_context.cu:4068)
  // COLL_REFRESH_RATE_GBPS, default 0 = off: instead of the fixed sleep, a background refresh sleeps after each batch
  // for as long as keeps its copy over the host link at this many GB/s on average
  static double refresh_rate_gbps;
  // COLL_RECORD_INLINE_BYTES: a serving step counts a recorded prefix of up to this many bytes itself (a copy kernel in
  // front of the lookup, counted after it) instead of handing it to the recorder's thread; 0 = always the thread
  static size_t record_inline_bytes;
  static bool gpu_record;          // COLL_GPU_RECORD=1: every lookup counts its keys in device-side hotness counters
  static size_t gpu_record_every;  // COLL_GPU_RECORD_EVERY, default 1: ... only every n-th lookup
  // COLL_GPU_REFRESH=1 (with COLL_GPU_RECORD=1): a refresh whose hotness was all counted on the device ranks, places
  // and diffs on the device too; the host sees two short key lists instead of per-key arrays of the key space
  static bool gpu_refresh;
  // COLL_GPU_REFRESH_KEEP=1: such a refresh leaves the counters as they are (hotness accumulates over refreshes)
  // instead of starting the next interval from zero
  static bool gpu_refresh_keep;
  // COLL_GPU_REFRESH_STABLE=1: among rows whose counts tie at the last count that gets in, such a refresh prefers the
  // rows cached now, so it moves no row that the counters do not tell apart from the one it would replace
  static bool gpu_refresh_stable;
  // COLL_GPU_RECORD_SEED=1: the device-side counters start from the hotness the cache was built from (the ranking
  // handed to the build) instead of from zero, so the first refreshes on the device weigh what the lookups counted
  // against what the build knew
  static bool gpu_record_seed;
  // COLL_MISS_STAGE_ROWS=n (0 = off): the fused extraction also files the rows it takes from the host table in a
  // direct-mapped set of n (rounded up to a power of two) rows in HBM, and a foreground refresh takes the rows it inserts
  // from there when it finds them instead of over the host link again
  static size_t miss_stage_rows;
  // COLL_SPIN_WAIT=us (default 5000; 0 = off): a blocking lookup polls a ticket its last kernel is followed by, for up
  // to this long, before it falls back to waiting for the stream
  static unsigned spin_wait_us;
  static bool kernel_events;  // COLL_KERNEL_EVENTS: per-step kernel times from device events (1) or a host timer (0)
  static bool dedup_keys;        // COLL_DEDUP_KEYS=1: extract each distinct key of a batch once, then copy the duplicates
  static size_t dedup_min_keys;  // COLL_DEDUP_MIN_KEYS, default 4096: shorter batches skip the deduplication
  static double hash_rebuild_tombstone_frac;  // COLL_HASH_REBUILD_FRAC, default 0.15: rebuild the table after refresh
                                              // once this share of its buckets are tombstones
  // Sparse-id mode (an extension; the reference's keys are dense uint32 row numbers): the caller's key of host row
  // r is (r * key_map_mul) mod 2^bits with key_map_mul odd, a bijection on the id space, so the library can turn
  // a key back into its row with key_map_inv.  key_map_mul == 0: keys are row numbers.
  static uint64_t key_map_mul;
  static uint64_t key_map_inv;
  static uint64_t key_map_mask;
  static void SetKeyMap(uint64_t mul, int bits);
  static inline uint64_t KeyOfRow(uint64_t row) { return key_map_mul ? ((row * key_map_mul) & key_map_mask) : row; }
  static inline uint64_t RowOfKey(uint64_t key) { return key_map_mul ? ((key * key_map_inv) & key_map_mask) : key; }

  static void LoadConfigFromEnv();
  static inline uint64_t GetBatchKey(uint64_t epoch, uint64_t step) { return epoch * num_global_step_per_epoch + step; }
  static inline uint64_t GetEpochFromKey(uint64_t key) { return num_global_step_per_epoch ? key / num_global_step_per_epoch : 0; }
  static inline uint64_t GetStepFromKey(uint64_t key) { return num_global_step_per_epoch ? key % num_global_step_per_epoch : key; }
  static inline bool UseGPUCache() { return cache_percentage > 0; }
};

}  // namespace common
}  // namespace coll_cache_lib
