#include "workspace.hpp"
#include <mutex>
#include <cstdio>
#include <cstdlib>

namespace bm {

namespace {
constexpr int kMaxDevices = 64;
struct Slot { void* ptr = nullptr; size_t bytes = 0; };
Slot g_slots[kMaxDevices][WS_NSLOTS];
std::mutex g_mu;

bool debug_mem() {
    static int v = -1;
    if (v < 0) { const char* e = getenv("BIDMAT_DEBUG_MEM"); v = (e && e[0] == '1') ? 1 : 0; }
    return v == 1;
}
}  // namespace

void* ws_get(WsSlot slot, size_t bytes, hipError_t* err) {
    *err = hipSuccess;
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) { *err = hipErrorInvalidDevice; return nullptr; }
    std::lock_guard<std::mutex> lock(g_mu);
    Slot& s = g_slots[dev][slot];
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
        *err = hipMalloc(&s.ptr, bytes);
        want = bytes;
        if (*err != hipSuccess) { s.ptr = nullptr; return nullptr; }
    }
    s.bytes = want;
    if (debug_mem()) fprintf(stderr, "[bidmathip] workspace slot %d -> %zu bytes on device %d\n", (int)slot, want, dev);
    return s.ptr;
}

hipError_t ws_drop(WsSlot slot) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mu);
    Slot& s = g_slots[dev][slot];
    if (s.ptr) {
        e = hipFree(s.ptr);
        s.ptr = nullptr; s.bytes = 0;
    }
    return e;
}

hipError_t ws_release() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mu);
    for (int i = 0; i < WS_NSLOTS; ++i) {
        Slot& s = g_slots[dev][i];
        if (s.ptr) {
            hipError_t f = hipFree(s.ptr);
            if (f != hipSuccess) e = f;
            s.ptr = nullptr; s.bytes = 0;
        }
    }
    return e;
}

size_t ws_bytes() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    std::lock_guard<std::mutex> lock(g_mu);
    size_t t = 0;
    for (int i = 0; i < WS_NSLOTS; ++i) t += g_slots[dev][i].bytes;
    return t;
}

}  // namespace bm
