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
    hipEvent_t done = nullptr;   // recorded by every user behind its last launch, on its own stream
    bool used = false, broken = false;
};

// The array as held by one call: `ptr` is null if it can not be had (capturing stream, more than 16 devices, a failing
// runtime call).  The holder enqueues its kernels while the lease lives, so the order in which streams take the array
// is the order of their launches.  When the lease ends it records the array's event on the holder's own stream, still
// under the lock; the next holder makes its stream wait for that event before anything else.  Only the stream of the
// call at hand is ever touched: a stream that has been destroyed or has gone into capture since it used the array
// plays no part.
class ScratchLease {
public:
    ScratchLease() = default;
    ScratchLease(const ScratchLease&) = delete;
    ScratchLease& operator=(const ScratchLease&) = delete;
    ~ScratchLease() {
        if (!ptr_) return;
        if (hipEventRecord(st_->done, s_) == hipSuccess) {
            st_->used = true;
        } else {   // nothing orders the next holder behind this one: the array is not handed out again
            (void)hipGetLastError();
            st_->broken = true;
        }
    }
    void* get() const { return ptr_; }

    // `per_device` has 16 entries; `symbol` is HIP_SYMBOL(array).
    template <typename Symbol>
    void* acquire(SharedScratch* per_device, const Symbol& symbol, hipStream_t s) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return nullptr;
        }
        SharedScratch& st = per_device[dev];
        lock_ = std::unique_lock<std::mutex>(st.mu);
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
        // (a wait for an event recorded on the same stream costs nothing; the handles are not compared, since a
        // destroyed stream's handle can come back as a new stream's)
        if (st.used && hipStreamWaitEvent(s, st.done, 0) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        st_ = &st;
        s_ = s;
        ptr_ = st.ptr;
        return ptr_;
    }

private:
    std::unique_lock<std::mutex> lock_;   // declared first: released after the destructor body has recorded the event
    SharedScratch* st_ = nullptr;
    hipStream_t s_ = nullptr;
    void* ptr_ = nullptr;
};

}  // namespace mi
