// C++ side of the shim: python/collcache/common/operation.h:28-29 of the reference.
#pragma once

#include <cstddef>
#include <functional>

#include "coll_cache_c_api.h"
#include "common.h"

namespace coll_cache_lib {
namespace common {

void coll_cache_init(int replica_id, size_t key_space_size, std::function<MemHandle(size_t)> allocator,
                     void *cpu_data, DataType dtype, size_t dim, double cache_percentage, StreamHandle stream);
extern size_t max_num_keys;

}  // namespace common
}  // namespace coll_cache_lib
