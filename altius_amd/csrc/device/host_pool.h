// Process-wide pool of pinned (page-locked) host memory for the tensors that cross PCIe.
#pragma once

#include <cstddef>

#include "../core/tensor.h"

namespace altius {

struct HostPoolStats {
    size_t live_bytes = 0;    // handed out and not yet returned
    size_t cached_bytes = 0;  // returned, kept for reuse
    size_t pinned_allocations = 0;  // hipHostMalloc calls so far
    size_t reuses = 0;              // requests served from the cache
};

// Allocator to hand to Tensor::from_raw / uninit_of_type: blocks of at least 64 KiB come from
// the pinned pool whenever a device is present; for smaller ones, and on a machine without a
// device, it returns nullptr and the tensor falls back to malloc.
std::shared_ptr<HostBlock> pinned_host_block(size_t bytes);

HostPoolStats host_pool_stats();

// Frees every cached block; live blocks are unaffected.  Returns the number of bytes freed.
size_t host_pool_trim();

}  // namespace altius
