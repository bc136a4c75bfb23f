// A second stream for launches of one call that do not depend on each other (the backward's dQ and dK/dV kernels: both
// read what the row-dots kernel wrote, neither reads what the other writes).  On shapes that do not fill the device the two
// kernels share it instead of waiting for each other; the callers hold the rule for when that pays.
//
//   SideStreamLease side(main);           // takes a (stream, two events) set of the current device out of a pool
//   if (side.fork() == hipSuccess) ...    // side.stream() now starts behind everything enqueued on main so far
//   launch A on side.stream(), B on main
//   side.join();                          // main continues behind A
//
// The sets are created on demand (default priority, non-blocking with respect to the null stream), handed out under a
// mutex for the duration of one call's enqueueing and never destroyed: as many exist as calls were ever enqueueing at the
// same moment on a device.  Calls that take the same set one after the other queue their side launches behind each other,
// which is an ordering nobody needs but harmless.
// No side stream is used (active() is false; the caller launches everything on main) when the main stream is being
// captured into a graph - a side stream would stay part of that capture until it ends, and the next call to take it from
// the pool would be recorded into somebody else's graph - when INCIN_ROCM_BWD_STREAMS=1 is set in the environment (one
// stream: per-kernel times in a trace are then times of kernels that had the device to themselves), or when creating the
// set fails.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

namespace incin_rocm {

struct SideStreamSet {
    int device = -1;
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
};

inline std::mutex& side_stream_mutex()
{
    static std::mutex m;
    return m;
}
inline std::vector<SideStreamSet>& side_stream_pool()
{
    static std::vector<SideStreamSet>* pool = new std::vector<SideStreamSet>();      // (never freed: streams outlive static destructors)
    return *pool;
}

class SideStreamLease {
public:
    // wanted = false: no set is taken (active() is false), for callers whose rule says that this call gains nothing
    explicit SideStreamLease(hipStream_t main, bool wanted = true) : main_(main)
    {
        if (!wanted) return;
        const char* one = getenv("INCIN_ROCM_BWD_STREAMS");
        if (one && strcmp(one, "1") == 0) return;
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(main, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return;
        }
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return;
        {
            std::lock_guard<std::mutex> lock(side_stream_mutex());
            std::vector<SideStreamSet>& pool = side_stream_pool();
            for (size_t i = 0; i < pool.size(); ++i)
                if (pool[i].device == dev) {
                    set_ = pool[i];
                    pool[i] = pool.back();
                    pool.pop_back();
                    return;
                }
        }
        SideStreamSet s;
        s.device = dev;
        if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); return; }
        if (hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            if (s.fork) (void)hipEventDestroy(s.fork);
            (void)hipStreamDestroy(s.stream);
            return;
        }
        set_ = s;
    }
    ~SideStreamLease()
    {
        if (set_.stream == nullptr) return;
        std::lock_guard<std::mutex> lock(side_stream_mutex());
        side_stream_pool().push_back(set_);
    }
    SideStreamLease(const SideStreamLease&) = delete;
    SideStreamLease& operator=(const SideStreamLease&) = delete;

    bool active() const { return set_.stream != nullptr; }
    hipStream_t stream() const { return set_.stream; }
    // the side stream waits for everything enqueued on the main stream so far
    hipError_t fork()
    {
        hipError_t e = hipEventRecord(set_.fork, main_);
        return e != hipSuccess ? e : hipStreamWaitEvent(set_.stream, set_.fork, 0);
    }
    // the main stream waits for everything enqueued on the side stream so far
    hipError_t join()
    {
        hipError_t e = hipEventRecord(set_.join, set_.stream);
        return e != hipSuccess ? e : hipStreamWaitEvent(main_, set_.join, 0);
    }

private:
    hipStream_t main_;
    SideStreamSet set_;
};

}  // namespace incin_rocm
