// Host storage allocation for tensors.
#include "tensor.h"

#include <new>

namespace altius {

namespace {

void free_block(uint8_t *ptr, size_t, void *) { std::free(ptr); }

}  // namespace

std::shared_ptr<HostBlock> malloc_host_block(size_t bytes) {
    std::shared_ptr<HostBlock> b(new (std::nothrow) HostBlock());
    if (!b) return nullptr;
    if (bytes) {
        // 64-byte alignment: whole cache lines for the CPU copy into the block.
        const size_t rounded = (bytes + 63) & ~size_t(63);
        b->ptr = static_cast<uint8_t *>(std::aligned_alloc(64, rounded));
        if (!b->ptr) return nullptr;
        b->release = free_block;
    }
    b->size = bytes;
    return b;
}

std::shared_ptr<HostBlock> allocate_host_block(size_t bytes, HostAllocator preferred) {
    if (preferred) {
        if (auto b = preferred(bytes)) return b;
    }
    return malloc_host_block(bytes);
}

}  // namespace altius
