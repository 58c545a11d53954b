#include "run_config.h"

#include <algorithm>
#include <cstdlib>

#include "logging.h"
#include "ugache_hip.h"

namespace coll_cache_lib {
namespace common {

bool RunConfig::is_configured = false;
CachePolicy RunConfig::cache_policy = kCollCacheAsymmLink;
double RunConfig::cache_percentage = 0;
size_t RunConfig::num_device = 1;
std::vector<int> RunConfig::device_id_list = {0};
bool RunConfig::cross_process = false;
int RunConfig::worker_id = 0;
uint64_t RunConfig::num_global_step_per_epoch = 0;
uint64_t RunConfig::num_epoch = 0;
uint64_t RunConfig::num_total_item = 0;
int RunConfig::omp_thread_num = 40;
int RunConfig::solver_omp_thread_num = 40;
int RunConfig::solver_omp_thread_num_per_gpu = 5;
int RunConfig::refresher_omp_thread_num = 8;
int RunConfig::refresher_omp_thread_num_per_gpu = 1;
size_t RunConfig::option_empty_feat = 0;
ConcurrentLinkImpl RunConfig::concurrent_link_impl = kDirectNoGroup;
size_t RunConfig::coll_cache_scale_nb = 16;
bool RunConfig::use_flat_hashtable = true;
double RunConfig::coll_cache_hyperparam_T_local = 1;
double RunConfig::coll_cache_hyperparam_T_cpu = 8000.0 / 50.0;
coll_cache::AsymmLinkDesc RunConfig::coll_cache_link_desc;
double RunConfig::hash_load_factor = 0.7;
int RunConfig::force_table_kind = 0;
bool RunConfig::device_key_list = true;
unsigned RunConfig::fill_limit_block = 128;
size_t RunConfig::refresh_batch_rows = 4092;
unsigned RunConfig::refresh_sleep_us = 3000;
unsigned RunConfig::refresh_limit_block = 20;
double RunConfig::refresh_rate_gbps = 0;
size_t RunConfig::record_inline_bytes = 64 << 10;
double RunConfig::hash_rebuild_tombstone_frac = 0.15;
bool RunConfig::gpu_record = false;
size_t RunConfig::gpu_record_every = 1;
bool RunConfig::gpu_refresh = false;
bool RunConfig::gpu_refresh_keep = false;
bool RunConfig::gpu_refresh_stable = false;
bool RunConfig::gpu_record_seed = false;
size_t RunConfig::miss_stage_rows = 0;
unsigned RunConfig::spin_wait_us = 5000;
bool RunConfig::kernel_events = false;
bool RunConfig::dedup_keys = false;
size_t RunConfig::dedup_min_keys = 4096;
uint64_t RunConfig::key_map_mul = 0;
uint64_t RunConfig::key_map_inv = 0;
uint64_t RunConfig::key_map_mask = 0;

void RunConfig::SetKeyMap(uint64_t mul, int bits) {
  if (mul == 0) {
    key_map_mul = key_map_inv = key_map_mask = 0;
    return;
  }
  CHECK(mul & 1) << "the key-map multiplier must be odd to be invertible modulo a power of two";
  CHECK(bits >= 1 && bits <= 62) << "key space of 2^" << bits << " ids is not supported";
  // inverse of an odd number modulo 2^64 by Newton's iteration (each step doubles the number of correct bits)
  uint64_t inv = mul;
  for (int i = 0; i < 6; i++) inv *= 2 - mul * inv;
  CHECK_EQ(mul * inv, (uint64_t)1);
  key_map_mul = mul;
  key_map_inv = inv;
  key_map_mask = (bits == 64) ? ~0ull : ((1ull << bits) - 1);
}

void RunConfig::LoadConfigFromEnv() {
  // every knob goes back to its default first, so a process that builds a second cache sees only its current
  // environment
  concurrent_link_impl = kDirectNoGroup;
  coll_cache_scale_nb = 16;
  hash_load_factor = 0.7;
  force_table_kind = 0;
  device_key_list = true;
  fill_limit_block = 128;
  refresh_batch_rows = 4092;
  refresh_sleep_us = 3000;
  refresh_limit_block = 20;
  refresh_rate_gbps = 0;
  record_inline_bytes = 64 << 10;
  refresher_omp_thread_num = 8;
  hash_rebuild_tombstone_frac = 0.15;
  dedup_keys = false;
  dedup_min_keys = 4096;
  gpu_record = false;
  gpu_record_every = 1;
  gpu_refresh = false;
  gpu_refresh_keep = false;
  gpu_refresh_stable = false;
  gpu_record_seed = false;
  miss_stage_rows = 0;
  spin_wait_us = 5000;
  kernel_events = false;
  if (GetEnv("SAMGRAPH_EMPTY_FEAT") != "" && GetEnv("SAMGRAPH_EMPTY_FEAT") != "0") {
    LOG(FATAL) << "SAMGRAPH_EMPTY_FEAT (mock host table) is not supported by this build: every key must have a "
                  "real row in the host table";
  }
  const std::string no_group = GetEnv("SAMGRAPH_COLL_CACHE_NO_GROUP");
  const std::string impl = GetEnv("SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL");
  // The reference defaults to its factored extraction (MPSPhase on its platforms).  With one GPU and its host as the
  // only two sources the fused kernel is the faster one on this hardware, so it is what an unset variable selects;
  // the reference's names still select the reference's structure.
  if (no_group == "DIRECT" || impl == "DIRECT" || impl == "") {
    concurrent_link_impl = kDirectNoGroup;
  } else if (impl == "SMMaskPhase" || impl == "MPSPhase") {
    concurrent_link_impl = kSMMaskPhase;
  } else if (impl == "NONE" || impl == "NoConcurrent") {
    concurrent_link_impl = kNoConcurrentLink;
  } else {
    LOG(FATAL) << "concurrent link impl '" << impl << "' has no counterpart on one GPU (use SMMaskPhase, DIRECT or NONE)";
  }
  if (GetEnv("COLL_CACHE_SCALE") != "") coll_cache_scale_nb = std::stoul(GetEnv("COLL_CACHE_SCALE"));
  if (GetEnv("COLL_HASH_LOAD_FACTOR") != "") hash_load_factor = std::stod(GetEnv("COLL_HASH_LOAD_FACTOR"));
  if (GetEnv("COLL_DEVICE_KEY_LIST") != "") device_key_list = GetEnv("COLL_DEVICE_KEY_LIST") != "0";
  if (GetEnv("COLL_FILL_LIMIT_BLOCK") != "") fill_limit_block = (unsigned)std::stoul(GetEnv("COLL_FILL_LIMIT_BLOCK"));
  const std::string tbl = GetEnv("COLL_HASH_TABLE");
  if (tbl == "FLAT") force_table_kind = 1;
  else if (tbl == "HASH") force_table_kind = 2;
  else if (tbl == "HASH16") force_table_kind = 16;
  else if (tbl == "HASH8") force_table_kind = 8;
  else if (tbl != "") LOG(FATAL) << "COLL_HASH_TABLE must be FLAT, HASH, HASH16 or HASH8, got " << tbl;
  if (GetEnv("COLL_REFRESH_THREADS") != "") refresher_omp_thread_num = std::max(1, std::stoi(GetEnv("COLL_REFRESH_THREADS")));
  if (GetEnv("COLL_REFRESH_BATCH_ROWS") != "") refresh_batch_rows = std::stoul(GetEnv("COLL_REFRESH_BATCH_ROWS"));
  if (GetEnv("COLL_REFRESH_SLEEP_US") != "") refresh_sleep_us = std::stoul(GetEnv("COLL_REFRESH_SLEEP_US"));
  if (GetEnv("COLL_REFRESH_LIMIT_BLOCK") != "") refresh_limit_block = std::stoul(GetEnv("COLL_REFRESH_LIMIT_BLOCK"));
  if (GetEnv("COLL_REFRESH_RATE_GBPS") != "") refresh_rate_gbps = std::stod(GetEnv("COLL_REFRESH_RATE_GBPS"));
  if (GetEnv("COLL_RECORD_INLINE_BYTES") != "")
    record_inline_bytes = std::min<size_t>(std::stoul(GetEnv("COLL_RECORD_INLINE_BYTES")), (size_t)16 << 20);
  if (GetEnv("COLL_GPU_RECORD") != "") gpu_record = GetEnv("COLL_GPU_RECORD") != "0";
  if (GetEnv("COLL_GPU_REFRESH") != "") gpu_refresh = GetEnv("COLL_GPU_REFRESH") != "0";
  if (GetEnv("COLL_GPU_REFRESH_KEEP") != "") gpu_refresh_keep = GetEnv("COLL_GPU_REFRESH_KEEP") != "0";
  if (GetEnv("COLL_GPU_REFRESH_STABLE") != "") gpu_refresh_stable = GetEnv("COLL_GPU_REFRESH_STABLE") != "0";
  if (GetEnv("COLL_GPU_RECORD_SEED") != "") gpu_record_seed = GetEnv("COLL_GPU_RECORD_SEED") != "0";
  if (GetEnv("COLL_SPIN_WAIT") != "") spin_wait_us = (unsigned)std::stoul(GetEnv("COLL_SPIN_WAIT"));
  if (GetEnv("COLL_MISS_STAGE_ROWS") != "") miss_stage_rows = (size_t)std::stoull(GetEnv("COLL_MISS_STAGE_ROWS"));
  if (GetEnv("COLL_KERNEL_EVENTS") != "") kernel_events = GetEnv("COLL_KERNEL_EVENTS") != "0";
  if (GetEnv("COLL_GPU_RECORD_EVERY") != "")
    gpu_record_every = std::max<size_t>(1, std::stoull(GetEnv("COLL_GPU_RECORD_EVERY")));
  if (GetEnv("COLL_DEDUP_KEYS") != "") dedup_keys = GetEnv("COLL_DEDUP_KEYS") != "0";
  if (GetEnv("COLL_DEDUP_MIN_KEYS") != "") dedup_min_keys = std::stoull(GetEnv("COLL_DEDUP_MIN_KEYS"));
  if (GetEnv("COLL_HASH_REBUILD_FRAC") != "") hash_rebuild_tombstone_frac = std::stod(GetEnv("COLL_HASH_REBUILD_FRAC"));
  LOG(INFO) << "using concurrent impl " << concurrent_link_impl;
}

namespace coll_cache {

AsymmLinkDesc AsymmLinkDesc::AutoBuild(Context ctx) {
  // The reference aborts on anything that is not an A100/V100 (asymm_link_desc.cc:247-292).  Here any device
  // the HIP layer can open is accepted; the numbers are MI355X's (HBM3E ~8 TB/s, PCIe Gen5 x16 host link).
  AsymmLinkDesc desc;
  ugk_device_info_t info;
  UGK_CALL(ugk_get_device_info(ctx.device_id, &info));
  desc.gpu_model = info.name;
  desc.link_src.assign(RunConfig::num_device, {});
  // The host-link gather runs on a stream confined to a few CUs (COLL_CPU_CU_NUM, default 8, 0 = unconfined) and
  // is launched with COLL_CPU_SM_NUM_OVERRIDE workgroups (default 128 when confined, 32 otherwise).  Measured on
  // MI355X: 64-256 workgroups packed on 8 CUs read the host table at 95 % of the link while the HBM gather next to
  // it keeps its speed; the same workgroups spread over the chip slow the HBM gather down 5-10x.
  int cpu_cus = 8;
  if (GetEnv("COLL_CPU_CU_NUM") != "") cpu_cus = std::stoi(GetEnv("COLL_CPU_CU_NUM"));
  CHECK_GE(cpu_cus, 0);
  CHECK_LE(cpu_cus, info.compute_units);
  int cpu_blocks = cpu_cus > 0 ? 128 : 32;
  if (GetEnv("COLL_CPU_SM_NUM_OVERRIDE") != "") cpu_blocks = std::stoi(GetEnv("COLL_CPU_SM_NUM_OVERRIDE"));
  CHECK_GT(cpu_blocks, 0);
  desc.cpu_sm.assign(RunConfig::num_device, cpu_blocks);
  desc.cpu_cu.assign(RunConfig::num_device, cpu_cus);
  desc.local_sm.assign(RunConfig::num_device, 0);
  desc.local_bw_GBps = 8000;
  desc.cpu_bw_GBps = 50;
  if (GetEnv("COLL_CPU_TIME_OVERRIDE") != "") RunConfig::coll_cache_hyperparam_T_cpu = std::stod(GetEnv("COLL_CPU_TIME_OVERRIDE"));
  return desc;
}

}  // namespace coll_cache
}  // namespace common
}  // namespace coll_cache_lib
