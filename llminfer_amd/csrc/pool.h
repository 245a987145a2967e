// Two-class best-fit block pool over an injected backing allocator.
// Policy of base::CUDADeviceAllocator (code/source/base/alloc_cu.cpp:7-119),
// re-backed by hipMalloc in production and by any callback pair in tests.
#ifndef LLMI_POOL_H
#define LLMI_POOL_H

#include <cstddef>
#include <map>
#include <set>
#include <utility>

#include "llmi_hip.h"

struct llmi_pool {
    // Ordered by (bytes, address): lower_bound({bytes, nullptr}) is the
    // smallest free block that fits (alloc.h:42-45).
    using Block = std::pair<size_t, void*>;
    struct Busy {
        size_t bytes;
        bool big;
    };

    static constexpr size_t kClassSplit = 1024 * 1024;  // "> 1 MiB" is the big class (alloc_cu.cpp:21)

    llmi_pool(llmi_backing_alloc_fn a, llmi_backing_free_fn f, void* u) : alloc_fn(a), free_fn(f), user(u) {}
    ~llmi_pool();
    llmi_pool(const llmi_pool&) = delete;
    llmi_pool& operator=(const llmi_pool&) = delete;

    void* allocate(size_t bytes);
    int release(void* ptr);
    size_t trim();
    void stats(llmi_pool_stats* out) const;

    llmi_backing_alloc_fn alloc_fn;
    llmi_backing_free_fn free_fn;
    void* user;
    std::set<Block> big_free, small_free;
    std::map<void*, Busy> busy;
    size_t backing_allocs = 0, reuses = 0;
    size_t big_busy_bytes = 0, big_free_bytes = 0, small_busy_bytes = 0, small_free_bytes = 0;
    size_t big_busy_blocks = 0, small_busy_blocks = 0;
};

#endif
