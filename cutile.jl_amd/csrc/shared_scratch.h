// A static device array of the library that the streams of a GPU share (partial sums of a split GEMM, partial
// results of split attention).  The library allocates nothing, so such an array is a `static __device__` symbol;
// launches that use it from different streams are ordered by an event, and a stream under graph capture is not given
// the array at all (the caller then runs its unsplit kernel) unless the caller has promised, through
// mi_scratch_under_capture, to keep the replays of its graphs apart from one another and from other users of the arrays.
#pragma once
#include <mutex>

#include "common.h"

namespace mi {

struct SharedScratch {
    std::mutex mu;
    void* ptr = nullptr;
    hipEvent_t done = nullptr;   // once several streams use the array: recorded by every holder behind its last launch
    hipStream_t last = nullptr;  // the previous holder's stream (compared, not used, except once: see acquire)
    bool used = false, broken = false;
    bool multi = false;          // holders on more than one stream have been seen
};

// The array as held by one call: `ptr` is null if it can not be had (capturing stream, more than 16 devices, a failing
// runtime call).  The holder enqueues its kernels while the lease lives, so the order in which streams take the array
// is the order of their launches.  As long as every holder has come on the same stream, the stream's own order is all
// there is to it and no event is touched (an event recorded behind every launch costs 2.5 to 3 us per call: a marker
// between two kernels of a 25 us loop).  The first holder that comes on another stream switches the array to events
// for good: from then on a lease that ends records the event on the holder's own stream, still under the lock, and
// the next holder makes its stream wait for it.  Only that one switch records on the previous holder's stream (whose
// launches no event covers yet); should that stream be gone or under capture by then, the call at hand is refused
// the array and runs its unsplit kernel.
class ScratchLease {
public:
    ScratchLease() = default;
    ScratchLease(const ScratchLease&) = delete;
    ScratchLease& operator=(const ScratchLease&) = delete;
    ~ScratchLease() {
        if (!ptr_) return;
        st_->used = true;
        st_->last = s_;
        if (st_->multi && hipEventRecord(st_->done, s_) != hipSuccess) {
            // nothing orders the next holder behind this one: the array is not handed out again
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
        if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        SharedScratch& st = per_device[dev];
        if (cap != hipStreamCaptureStatusNone) {
            // A launch that is being recorded runs later, as often as the graph is replayed and on whatever stream:
            // no event of this call can order it.  The array is handed out only if the caller has taken that
            // ordering upon itself, and only once an eager call has made its address known (the lookup is not
            // a thing to do inside a capture).  Nothing of the lease's own bookkeeping is touched.
            if (!scratch_under_capture()) return nullptr;
            std::unique_lock<std::mutex> lk(st.mu);
            return st.broken ? nullptr : st.ptr;
        }
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
        if (st.used && st.multi) {
            if (hipStreamWaitEvent(s, st.done, 0) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
        } else if (st.used && st.last != s) {
            st.multi = true;
            hipStreamCaptureStatus prev = hipStreamCaptureStatusNone;
            const bool ordered = hipStreamIsCapturing(st.last, &prev) == hipSuccess && prev == hipStreamCaptureStatusNone &&
                                 hipEventRecord(st.done, st.last) == hipSuccess && hipStreamWaitEvent(s, st.done, 0) == hipSuccess;
            if (!ordered) {
                (void)hipGetLastError();
                st.used = false;   // (whatever that stream was given has long been enqueued; the next holders order themselves by the event)
                return nullptr;
            }
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
