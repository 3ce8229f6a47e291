// Per-device scratch buffers owned by the library (column-pointer copies, overflow-segment
// tables, partial sums). Buffers grow on demand and are reused by later calls; calls that
// share a device are expected to be stream-ordered with respect to each other.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace bm {

enum WsSlot {
    WS_JC = 0,        // int[ncols+1]  column pointer derived from ic (reference-shaped entries)
    WS_OVF,           // int[ncols+1]  exclusive scan of extra segments per column
    WS_PARTIAL,       // float[novf*k] partial sums of overflow segments
    WS_SCAN,          // int[...]      block sums of the scan
    WS_MISC,          // small scalars (max row, fingerprints)
    WS_REDUCE,        // float[...]    partials of the dense reductions
    WS_TRANS_IN,      // float[...]    transposed dense operand of S*A / S^T*A
    WS_TRANS_OUT,     // float[...]    transposed result of S*A / S^T*A
    WS_PLAN,          // bytes         temporaries of a plan build (dropped again when large)
    WS_NSLOTS
};

// Returns a device buffer of at least `bytes` for `slot` on the current device (nullptr and
// *err set on failure). Growing a slot frees the old buffer after a device synchronise.
void* ws_get(WsSlot slot, size_t bytes, hipError_t* err);
// Frees one slot of the current device.
hipError_t ws_drop(WsSlot slot);
// Frees every slot of the current device.
hipError_t ws_release();
// Total bytes currently held on the current device.
size_t ws_bytes();

}  // namespace bm
