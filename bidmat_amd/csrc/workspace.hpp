// Scratch buffers owned by the library (column-pointer copies, overflow-segment tables, partial
// sums), one set per (device, stream): calls enqueued on different streams never share scratch,
// calls on one stream are ordered by the stream. Buffers grow on demand and are reused.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <mutex>

namespace bm {

enum WsSlot {
    WS_JC = 0,        // int[ncols+1]  column pointer derived from ic (reference-shaped entries)
    WS_OVF,           // int[ncols+1]  exclusive scan of extra segments per column
    WS_PARTIAL,       // float[novf*k] partial sums of overflow segments
    WS_ROWPARTIAL,    // float[nseg*k] partial sums of a plan's row segments (A*^S, row sums)
    WS_SCAN,          // int[...]      block sums of the scan
    WS_MISC,          // small scalars (max row, fingerprints)
    WS_REDUCE,        // float[...]    partials of the dense reductions
    WS_TRANS_IN,      // float[...]    transposed dense operand of S*A / S^T*A
    WS_TRANS_OUT,     // float[...]    transposed result of S*A / S^T*A
    WS_PLAN,          // bytes         temporaries of a plan build sized by the rows
    WS_PLAN_ROWS_A,   // bytes         temporaries of the row side of a plan build (dropped again when large)
    WS_PLAN_ROWS_B,   // bytes         likewise, the part sized by the nonzeros of light rows
    WS_TRANSPOSE,     // bytes         sort buffers of the sparse transpose
    WS_ROWSUM,        // bytes         exact row sums: block maxima, 64-bit accumulators, flags
    WS_ROWSUM_TABLES, // u64[...]      exact row sums: the accumulator tables of the workgroups
    WS_NSLOTS
};

// Returns a device buffer of at least `bytes` for `slot` of `stream` on the current device
// (nullptr and *err set on failure). Growing a slot frees the old buffer, which waits for the
// device first.
void* ws_get(WsSlot slot, size_t bytes, hipError_t* err, hipStream_t stream = nullptr);
// Frees one slot of `stream` on the current device.
hipError_t ws_drop(WsSlot slot, hipStream_t stream = nullptr);
// Frees every slot of `stream` on the current device (called when a stream is destroyed).
hipError_t ws_drop_stream(hipStream_t stream);
// Frees every slot of every stream of the current device.
hipError_t ws_release();
// Total bytes currently held on the current device.
size_t ws_bytes();

// Device memory of plans comes from a small pool per device: a block given back is kept (up to
// opt_plan_pool_mb() MiB in all) and handed out again to a request it fits without wasting more than a
// quarter, so that callers who build a plan per minibatch do not pay hipMalloc + hipFree (each a device-wide
// synchronisation) for the same sizes over and over. Blocks must be idle when they are given back.
void* pool_alloc(size_t bytes, hipError_t* err);
hipError_t pool_free(void* p);
// Frees every kept block of the current device.
hipError_t pool_release();

// Host threads that share a device also share its scratch buffers and cached plans. Every entry
// point that takes scratch or a cached plan holds this lock of the current device from its first
// ws_get to its last launch (the blocking entries: until their synchronisation), so that another
// thread can neither refill a buffer between "table built" and "kernel that reads it enqueued" nor
// grow (free) a buffer whose address was just handed out. Recursive: entries may nest.
std::unique_lock<std::recursive_mutex> device_lock();

}  // namespace bm
