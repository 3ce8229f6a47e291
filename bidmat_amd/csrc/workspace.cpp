#include "workspace.hpp"
#include <array>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

namespace bm {

int opt_plan_pool_mb();

namespace {
struct Slot { void* ptr = nullptr; size_t bytes = 0; };
using SlotSet = std::array<Slot, WS_NSLOTS>;
std::map<std::pair<int, hipStream_t>, SlotSet> g_sets;      // (device, stream) -> slots
std::mutex g_mu;
std::map<int, std::recursive_mutex> g_device_mu;            // nodes of a std::map never move

bool debug_mem() {
    static int v = -1;
    if (v < 0) { const char* e = getenv("BIDMAT_DEBUG_MEM"); v = (e && e[0] == '1') ? 1 : 0; }
    return v == 1;
}

hipError_t free_set(SlotSet& set) {
    hipError_t e = hipSuccess;
    for (Slot& s : set) {
        if (s.ptr) {
            hipError_t f = hipFree(s.ptr);
            if (f != hipSuccess) e = f;
            s.ptr = nullptr; s.bytes = 0;
        }
    }
    return e;
}
}  // namespace

void* ws_get(WsSlot slot, size_t bytes, hipError_t* err, hipStream_t stream) {
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_mu);
    Slot& s = g_sets[{dev, stream}][slot];
    if (bytes == 0) bytes = 256;
    if (s.bytes >= bytes) return s.ptr;
    if (s.ptr) {
        // hipFree waits for the device, so work that still reads the old buffer finishes first.
        *err = hipFree(s.ptr);
        s.ptr = nullptr; s.bytes = 0;
        if (*err != hipSuccess) return nullptr;
    }
    // same growth factor as the reference's recycled buffers (Mat.recycleGrow = 1.2)
    size_t want = bytes + bytes / 5;
    want = (want + 255) & ~size_t(255);
    *err = hipMalloc(&s.ptr, want);
    if (*err != hipSuccess) {
        (void)hipGetLastError();            // handled here: do not leave it for the next launch check
        *err = hipMalloc(&s.ptr, bytes);
        want = bytes;
        if (*err != hipSuccess) { (void)hipGetLastError(); s.ptr = nullptr; return nullptr; }
    }
    s.bytes = want;
    if (debug_mem())
        fprintf(stderr, "[bidmathip] workspace slot %d -> %zu bytes on device %d, stream %p\n", (int)slot, want, dev, (void*)stream);
    return s.ptr;
}

hipError_t ws_drop(WsSlot slot, hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_sets.find({dev, stream});
    if (it == g_sets.end()) return hipSuccess;
    Slot& s = it->second[slot];
    if (s.ptr) {
        e = hipFree(s.ptr);
        s.ptr = nullptr; s.bytes = 0;
    }
    return e;
}

hipError_t ws_drop_stream(hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_sets.find({dev, stream});
    if (it == g_sets.end()) return hipSuccess;
    e = free_set(it->second);
    g_sets.erase(it);
    return e;
}

hipError_t ws_release() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_sets.begin(); it != g_sets.end();) {
        if (it->first.first == dev) {
            hipError_t f = free_set(it->second);
            if (f != hipSuccess) e = f;
            it = g_sets.erase(it);
        } else {
            ++it;
        }
    }
    return e;
}

// ---- pool of plan blocks
namespace {
struct PoolBlock { void* p; size_t bytes; };
struct Pool {
    std::vector<PoolBlock> kept;                 // idle blocks
    std::map<void*, size_t> live;                // blocks handed out
    size_t kept_bytes = 0;
};
std::map<int, Pool> g_pools;
std::mutex g_pool_mu;
}  // namespace

void* pool_alloc(size_t bytes, hipError_t* err) {
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (bytes == 0) bytes = 256;
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& pool = g_pools[dev];
    // best fit among the kept blocks that do not waste more than a quarter
    int best = -1;
    for (int i = 0; i < (int)pool.kept.size(); ++i) {
        const size_t b = pool.kept[i].bytes;
        if (b >= bytes && b <= bytes + bytes / 4 + (1u << 20) && (best < 0 || b < pool.kept[best].bytes)) best = i;
    }
    if (best >= 0) {
        PoolBlock blk = pool.kept[best];
        pool.kept.erase(pool.kept.begin() + best);
        pool.kept_bytes -= blk.bytes;
        pool.live[blk.p] = blk.bytes;
        return blk.p;
    }
    void* p = nullptr;
    *err = hipMalloc(&p, bytes);
    if (*err != hipSuccess) {
        // out of memory with idle blocks in the pool: give them back to the device and try once more
        (void)hipGetLastError();
        for (PoolBlock& b : pool.kept) (void)hipFree(b.p);
        pool.kept.clear();
        pool.kept_bytes = 0;
        *err = hipMalloc(&p, bytes);
        if (*err != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    }
    pool.live[p] = bytes;
    return p;
}

hipError_t pool_free(void* p) {
    if (!p) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& pool = g_pools[dev];
    auto it = pool.live.find(p);
    if (it == pool.live.end()) return hipFree(p);          // not from this device's pool
    const size_t bytes = it->second;
    pool.live.erase(it);
    const size_t limit = (size_t)opt_plan_pool_mb() << 20;
    if (bytes > limit) return hipFree(p);
    // make room: the oldest kept blocks go first
    while (!pool.kept.empty() && pool.kept_bytes + bytes > limit) {
        e = hipFree(pool.kept.front().p);
        pool.kept_bytes -= pool.kept.front().bytes;
        pool.kept.erase(pool.kept.begin());
        if (e != hipSuccess) return e;
    }
    pool.kept.push_back(PoolBlock{p, bytes});
    pool.kept_bytes += bytes;
    return hipSuccess;
}

hipError_t pool_release() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& pool = g_pools[dev];
    for (PoolBlock& b : pool.kept) {
        hipError_t f = hipFree(b.p);
        if (f != hipSuccess) e = f;
    }
    pool.kept.clear();
    pool.kept_bytes = 0;
    return e;
}

std::unique_lock<std::recursive_mutex> device_lock() {
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::recursive_mutex* m;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        m = &g_device_mu[dev];
    }
    return std::unique_lock<std::recursive_mutex>(*m);
}

size_t ws_bytes() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_mu);
    size_t t = 0;
    for (auto& kv : g_sets)
        if (kv.first.first == dev)
            for (const Slot& s : kv.second) t += s.bytes;
    return t;
}

}  // namespace bm
