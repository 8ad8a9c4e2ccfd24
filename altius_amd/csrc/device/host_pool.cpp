// Pinned host memory pool.
//
// The reference moves host tensors into and out of `run` (crates/session_interpreter/src/session.rs:66-134);
// here every such tensor crosses PCIe once in each direction.  From pageable memory the runtime
// stages the copy through its own bounce buffers at a few GB/s; from page-locked memory the copy
// is one DMA transfer at link speed.  Page-locking is expensive (the pages are faulted in and
// registered with the device), so blocks are recycled: a freed tensor's block goes to a size-bucketed
// free list and serves the next tensor of that bucket.
#include "host_pool.h"

#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <new>
#include <vector>


namespace altius {

namespace {

constexpr size_t MIN_PINNED_BYTES = 64 * 1024;       // smaller tensors are not worth a registration
constexpr size_t SMALL_GRANULE = 64 * 1024;          // bucket size below 1 MiB
constexpr size_t LARGE_GRANULE = 1024 * 1024;        // bucket size from 1 MiB up
constexpr size_t MAX_CACHED_BYTES = size_t(8) << 30;  // beyond this, returned blocks are freed at once

struct Pool {
    std::mutex mu;
    std::map<size_t, std::vector<uint8_t *>> free_lists;  // bucket bytes -> blocks
    HostPoolStats stats;
    int device_state = 0;  // 0 unknown, 1 a device is present, -1 none
};

// Never destroyed: blocks may outlive static destruction order, and the runtime may already be
// gone when static destructors run.
Pool &pool() {
    static Pool *p = new Pool();
    return *p;
}

size_t bucket_of(size_t bytes) {
    const size_t g = bytes < LARGE_GRANULE ? SMALL_GRANULE : LARGE_GRANULE;
    return (bytes + g - 1) / g * g;
}

void release_block(uint8_t *ptr, size_t size, void *) {
    Pool &p = pool();
    const size_t bucket = bucket_of(size);
    {
        std::lock_guard<std::mutex> lock(p.mu);
        p.stats.live_bytes -= bucket;
        if (p.stats.cached_bytes + bucket <= MAX_CACHED_BYTES) {
            p.free_lists[bucket].push_back(ptr);
            p.stats.cached_bytes += bucket;
            return;
        }
    }
    (void)hipHostFree(ptr);
}

}  // namespace

std::shared_ptr<HostBlock> pinned_host_block(size_t bytes) {
    if (bytes < MIN_PINNED_BYTES) return nullptr;  // caller falls back to malloc
    Pool &p = pool();
    const size_t bucket = bucket_of(bytes);
    uint8_t *ptr = nullptr;
    {
        std::lock_guard<std::mutex> lock(p.mu);
        if (p.device_state == 0) {
            int n = 0;
            p.device_state = (hipGetDeviceCount(&n) == hipSuccess && n > 0) ? 1 : -1;
            if (p.device_state < 0) (void)hipGetLastError();
        }
        if (p.device_state < 0) return nullptr;
        auto it = p.free_lists.find(bucket);
        if (it != p.free_lists.end() && !it->second.empty()) {
            ptr = it->second.back();
            it->second.pop_back();
            p.stats.cached_bytes -= bucket;
            p.stats.reuses++;
        }
    }
    if (!ptr) {
        void *raw = nullptr;
        // Portable: usable from every device of the process, whichever is current now.
        if (hipHostMalloc(&raw, bucket, hipHostMallocPortable) != hipSuccess) {
            (void)hipGetLastError();
            host_pool_trim();  // cached blocks of other sizes may be what exhausts the limit
            if (hipHostMalloc(&raw, bucket, hipHostMallocPortable) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
        }
        ptr = static_cast<uint8_t *>(raw);
        std::lock_guard<std::mutex> lock(p.mu);
        p.stats.pinned_allocations++;
    }
    std::shared_ptr<HostBlock> b(new (std::nothrow) HostBlock());
    if (!b) {
        (void)hipHostFree(ptr);
        return nullptr;
    }
    b->ptr = ptr;
    b->size = bytes;
    b->release = release_block;
    std::lock_guard<std::mutex> lock(p.mu);
    p.stats.live_bytes += bucket;
    return b;
}

HostPoolStats host_pool_stats() {
    Pool &p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    return p.stats;
}

size_t host_pool_trim() {
    Pool &p = pool();
    std::vector<uint8_t *> blocks;
    size_t freed = 0;
    {
        std::lock_guard<std::mutex> lock(p.mu);
        for (auto &kv : p.free_lists) {
            for (uint8_t *b : kv.second) blocks.push_back(b);
            freed += kv.first * kv.second.size();
            kv.second.clear();
        }
        p.stats.cached_bytes = 0;
    }
    for (uint8_t *b : blocks) (void)hipHostFree(b);
    return freed;
}

}  // namespace altius
