#include "pool.h"

llmi_pool::~llmi_pool() {
    trim();
    // Blocks still busy are the caller's leak, but their memory goes back too.
    for (auto& kv : busy) free_fn(kv.first, user);
    busy.clear();
}

void* llmi_pool::allocate(size_t bytes) {
    if (bytes == 0) return nullptr;  // alloc_cu.cpp:8-10
    const bool big = bytes > kClassSplit;
    std::set<Block>& free_set = big ? big_free : small_free;

    auto it = free_set.lower_bound(Block(bytes, nullptr));
    // Big blocks are reused only with less than 1 MiB of slack (alloc_cu.cpp:23-24);
    // small blocks with any slack (alloc_cu.cpp:52-53).
    if (it != free_set.end() && (!big || it->first - bytes < kClassSplit)) {
        const Block blk = *it;
        free_set.erase(it);
        busy[blk.second] = Busy{blk.first, big};
        (big ? big_free_bytes : small_free_bytes) -= blk.first;
        (big ? big_busy_bytes : small_busy_bytes) += blk.first;
        (big ? big_busy_blocks : small_busy_blocks) += 1;
        ++reuses;
        return blk.second;
    }

    void* ptr = nullptr;
    if (alloc_fn(&ptr, bytes, user) != 0 || ptr == nullptr) return nullptr;  // alloc_cu.cpp:35-42,65-72
    ++backing_allocs;
    busy[ptr] = Busy{bytes, big};
    (big ? big_busy_bytes : small_busy_bytes) += bytes;
    (big ? big_busy_blocks : small_busy_blocks) += 1;
    return ptr;
}

int llmi_pool::release(void* ptr) {
    if (ptr == nullptr) return LLMI_OK;  // alloc_cu.cpp:82-84
    auto it = busy.find(ptr);
    if (it == busy.end()) return LLMI_ERR_UNKNOWN_POINTER;  // the reference CHECK-fails (alloc_cu.cpp:86-87)
    const Busy b = it->second;
    busy.erase(it);
    (b.big ? big_free : small_free).insert(Block(b.bytes, ptr));  // alloc_cu.cpp:90-98: never handed back
    (b.big ? big_busy_bytes : small_busy_bytes) -= b.bytes;
    (b.big ? big_free_bytes : small_free_bytes) += b.bytes;
    (b.big ? big_busy_blocks : small_busy_blocks) -= 1;
    return LLMI_OK;
}

size_t llmi_pool::trim() {
    size_t released = 0;
    for (std::set<Block>* s : {&big_free, &small_free}) {
        for (const Block& blk : *s) {
            free_fn(blk.second, user);
            released += blk.first;
        }
        s->clear();
    }
    big_free_bytes = small_free_bytes = 0;
    return released;
}

void llmi_pool::stats(llmi_pool_stats* out) const {
    out->backing_allocs = backing_allocs;
    out->reuses = reuses;
    out->big_busy_blocks = big_busy_blocks;
    out->big_free_blocks = big_free.size();
    out->small_busy_blocks = small_busy_blocks;
    out->small_free_blocks = small_free.size();
    out->big_busy_bytes = big_busy_bytes;
    out->big_free_bytes = big_free_bytes;
    out->small_busy_bytes = small_busy_bytes;
    out->small_free_bytes = small_free_bytes;
}
