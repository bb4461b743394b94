// Do two HIP streams run side by side?  The runtime maps the streams of a process onto a few hardware queues
// (GPU_MAX_HW_QUEUES, 4 by default) when they are first used; two streams that share a queue take turns, whatever the
// program asks for.  A pipeline that keeps two 25 MB buckets in flight to overlap the latency-bound launches of one
// with the codec launches of the other gains nothing from such a pair (measured: 31 µs per bucket instead of 18.5),
// so it asks before it settles on its streams.
//
// The probe: a single-wave kernel that spins for a fixed number of dependent multiply-adds (about 0.1 ms), timed once
// alone on `a` and once on `a` and `b` at the same time, between two events on `a`.  Side by side the pair takes as long
// as one (measured: 113 us alone, 138 us as a pair with its two event hand-overs); on one queue, twice as long (242 us).
// One wave on one CU leaves the rest of the chip free, so the answer does not depend on what else the kernels would
// compete for.  A queue works through its packets in order whichever stream they came from, so the same answer tells a
// caller whether an event recorded on `a` can complete before work enqueued earlier on `b` has finished.
#include "dq_launch.h"

#include <hip/hip_runtime.h>

#include <mutex>

namespace dq {

namespace {

// volatile: nothing ever reads the result, and a store that nobody can observe would take the loop with it
__device__ volatile float spin_sink[2][64];

__global__ __launch_bounds__(64) void spin_kernel(int slot, int iterations)
{
    float v = (float)threadIdx.x * 1e-3f;
    for (int i = 0; i < iterations; i++) v = __builtin_fmaf(v, 1.000001f, 1e-7f); // bounded: every wave leaves the loop
    spin_sink[slot][threadIdx.x] = v;
}

struct Events {
    hipEvent_t first = nullptr, last = nullptr, side = nullptr;
    ~Events()
    {
        if (first) (void)hipEventDestroy(first);
        if (last) (void)hipEventDestroy(last);
        if (side) (void)hipEventDestroy(side);
    }
};

#define DQ_TRY(call)                      \
    do {                                  \
        const hipError_t e_ = (call);     \
        if (e_ != hipSuccess) return e_;  \
    } while (0)

hipError_t timed(hipStream_t a, hipStream_t b, bool pair, const Events &ev, int iterations, float *ms)
{
    DQ_TRY(hipEventRecord(ev.first, a));
    if (pair) DQ_TRY(hipStreamWaitEvent(b, ev.first, 0));
    hipLaunchKernelGGL(spin_kernel, dim3(1), dim3(64), 0, a, 0, iterations);
    if (pair) {
        hipLaunchKernelGGL(spin_kernel, dim3(1), dim3(64), 0, b, 1, iterations);
        DQ_TRY(hipEventRecord(ev.side, b));
        DQ_TRY(hipStreamWaitEvent(a, ev.side, 0));
    }
    DQ_TRY(hipGetLastError());
    DQ_TRY(hipEventRecord(ev.last, a));
    DQ_TRY(hipEventSynchronize(ev.last));
    return hipEventElapsedTime(ms, ev.first, ev.last);
}

} // namespace

hipError_t probe_streams_overlap(hipStream_t a, hipStream_t b, int *overlap)
{
    constexpr int kIterations = 8192, kTakes = 3;
    if (a == b) {
        *overlap = 0;
        return hipSuccess;
    }
    Events ev;
    DQ_TRY(hipEventCreate(&ev.first));
    DQ_TRY(hipEventCreate(&ev.last));
    DQ_TRY(hipEventCreate(&ev.side));
    float ms = 0.0f;
    DQ_TRY(timed(a, b, true, ev, 64, &ms)); // first use of either stream: queue set-up and code upload stay out of the figures
    float alone = 1e30f, both = 1e30f;
    for (int k = 0; k < kTakes; k++) {
        DQ_TRY(timed(a, b, false, ev, kIterations, &ms));
        alone = ms < alone ? ms : alone;
        DQ_TRY(timed(a, b, true, ev, kIterations, &ms));
        both = ms < both ? ms : both;
    }
    *overlap = both < 1.5f * alone;
    return hipSuccess;
}

// `stream` waits for everything enqueued on `after` so far: an event recorded on `after`, waited for by `stream`.  The events
// come from a small ring per device, created on first use (timing disabled) and reused: a wait refers to the record that
// was current when the wait was enqueued, so recording the event again later does not disturb it.  Meant for callers that
// hand every bucket to a worker stream from a hot loop -- creating an event per hand-over, which is what a framework's
// wait_stream does, costs the host as much as enqueueing the bucket's four kernels.
hipError_t stream_order_after(hipStream_t stream, hipStream_t after, int device)
{
    if (stream == after) return hipSuccess;
    constexpr int kRing = 64, kDevices = 64;
    static std::mutex lock;
    static hipEvent_t ring[kDevices][kRing];
    static unsigned next[kDevices];
    if (device < 0 || device >= kDevices) return hipErrorInvalidDevice;
    hipEvent_t ev;
    {
        std::lock_guard<std::mutex> hold(lock);
        const unsigned slot = next[device]++ % kRing;
        if (!ring[device][slot]) DQ_TRY(hipEventCreateWithFlags(&ring[device][slot], hipEventDisableTiming));
        ev = ring[device][slot];
    }
    DQ_TRY(hipEventRecord(ev, after));
    return hipStreamWaitEvent(stream, ev, 0);
}

#undef DQ_TRY

} // namespace dq
