// A static device array of the library that the streams of a GPU share (partial sums of a split GEMM, partial
// results of split attention).  The library allocates nothing, so such an array is a `static __device__` symbol;
// launches that use it from different streams are ordered by an event, and a stream under graph capture is not given
// the array at all (the caller then runs its unsplit kernel).
#pragma once
#include <mutex>

#include "common.h"

namespace mi {

struct SharedScratch {
    std::mutex mu;
    void* ptr = nullptr;
    hipEvent_t done = nullptr;
    hipStream_t last = nullptr;
    bool used = false, broken = false;
};

// The array for a launch on stream `s` of the current device, or nullptr if it can not be had (capturing stream,
// more than 16 devices, a failing runtime call).  `per_device` has 16 entries; `symbol` is HIP_SYMBOL(array).  The
// lock is held until `lock` goes out of scope: the caller enqueues its kernels under it, so the order in which streams
// take the array is the order of their launches.  The previous user, if it ran on another stream, has to finish
// first: an event recorded on that stream now (it covers everything the stream has been given so far) is awaited by
// this one.
template <typename Symbol>
void* acquire_shared_scratch(SharedScratch* per_device, const Symbol& symbol, hipStream_t s, std::unique_lock<std::mutex>& lock) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return nullptr;
    SharedScratch& st = per_device[dev];
    lock = std::unique_lock<std::mutex>(st.mu);
    if (st.broken) return nullptr;
    if (!st.ptr) {
        if (hipGetSymbolAddress(&st.ptr, symbol) != hipSuccess ||
            hipEventCreateWithFlags(&st.done, hipEventDisableTiming) != hipSuccess) {
            st.broken = true;
            st.ptr = nullptr;
            (void)hipGetLastError();
            return nullptr;
        }
    }
    if (st.used && st.last != s) {
        bool ordered;
        if (hipEventRecord(st.done, st.last) == hipSuccess) {
            ordered = hipStreamWaitEvent(s, st.done, 0) == hipSuccess;
        } else {   // that stream no longer exists: what it was given is done once the device is idle
            (void)hipGetLastError();
            ordered = hipDeviceSynchronize() == hipSuccess;
        }
        if (!ordered) {
            (void)hipGetLastError();
            return nullptr;
        }
    }
    st.last = s;
    st.used = true;
    return st.ptr;
}

}  // namespace mi
