// Device memory of the objects handed to callers (index and candidate arrays).
//
// hipMalloc and hipFree cost tens of microseconds each and a fit or query makes several,
// which is a visible share of a 1-2 ms call.  Freed blocks are therefore kept per device
// and handed out again to requests of the same size class (sizes are rounded up by at
// most 12.5%).  The cache is bounded (CULSH_POOL_MAX_MB, default 8192, 0 = no caching) and
// culsh_memory_trim() returns it to the driver.
#include <map>
#include <mutex>
#include <unordered_map>

#include "common.hpp"

namespace culsh_amd {
namespace {

struct Pool {
    std::mutex mu;
    struct Live { size_t size; int device; };
    std::unordered_map<void*, Live> live;                       // blocks handed out
    std::map<int, std::multimap<size_t, void*>> cached;         // device -> size -> block
    size_t cached_bytes = 0;
    size_t limit = 0;
    bool limit_read = false;
};

Pool& pool() {
    static Pool* p = new Pool();  // never destroyed: the HIP runtime may already be gone at exit
    return *p;
}

size_t size_class(size_t bytes) {
    if (bytes <= 4096) return 4096;
    int top = 63 - __builtin_clzll(static_cast<unsigned long long>(bytes));
    const size_t step = size_t(1) << (top - 3);  // eight classes per power of two
    return (bytes + step - 1) & ~(step - 1);
}

// drops cached blocks (largest first) until at most `keep` bytes stay; caller holds the lock
void evict(Pool& p, size_t keep) {
    while (p.cached_bytes > keep) {
        std::multimap<size_t, void*>* biggest = nullptr;
        for (auto& kv : p.cached)
            if (!kv.second.empty() && (!biggest || kv.second.rbegin()->first > biggest->rbegin()->first))
                biggest = &kv.second;
        if (!biggest) break;
        auto it = std::prev(biggest->end());
        count_allocation_call();
        (void)hipFree(it->second);
        p.cached_bytes -= it->first;
        biggest->erase(it);
    }
}

}  // namespace

hipError_t dev_malloc(void** out, size_t bytes) {
    *out = nullptr;
    Pool& p = pool();
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    const size_t sz = size_class(bytes);
    std::lock_guard<std::mutex> lock(p.mu);
    if (!p.limit_read) {
        const char* v = std::getenv("CULSH_POOL_MAX_MB");
        p.limit = ((v && *v) ? static_cast<size_t>(std::strtoull(v, nullptr, 10)) : size_t(8192)) << 20;
        p.limit_read = true;
    }
    auto& fl = p.cached[device];
    auto it = fl.find(sz);
    if (it != fl.end()) {
        *out = it->second;
        p.cached_bytes -= sz;
        fl.erase(it);
    } else {
        count_allocation_call();
        e = hipMalloc(out, sz);
        if (e != hipSuccess) {  // give the cache back and try once more
            (void)hipGetLastError();
            evict(p, 0);
            count_allocation_call();
            e = hipMalloc(out, sz);
            if (e != hipSuccess) return e;
        }
    }
    p.live[*out] = {sz, device};
    return hipSuccess;
}

void dev_free(void* ptr) {
    if (!ptr) return;
    Pool& p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    auto it = p.live.find(ptr);
    if (it == p.live.end()) {  // not from dev_malloc
        count_allocation_call();
        (void)hipFree(ptr);
        return;
    }
    const Pool::Live meta = it->second;
    p.live.erase(it);
    if (meta.size > p.limit) {
        count_allocation_call();
        (void)hipFree(ptr);
        return;
    }
    // hipFree waits for the device; a block that may be handed out again needs the same guarantee
    (void)hipDeviceSynchronize();
    p.cached[meta.device].emplace(meta.size, ptr);
    p.cached_bytes += meta.size;
    evict(p, p.limit);
}

void dev_trim() {
    Pool& p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    evict(p, 0);
}

}  // namespace culsh_amd
