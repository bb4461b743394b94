// The search for the offset u of the dynamic bit-width rule
// (testbed_evaluation/new_comm_hooks/comm_hooks.py:73-139) without a pass over the norms per probe.
//
// The reference evaluates the average width at every probe of u with ten torch ops and a reduction over the
// norm tensors of all buckets, and reads the sum back to the host each time (up to 33 probes per search).
// The width of a superchunk depends on its norm only through the bf16 pattern, and as a function of the
// pattern it is a step function with two steps.  So:
//   norm_histogram_kernel   counts the norm patterns of a bucket's statistics into a histogram (one pass per
//                           bucket, accumulated over the buckets of a training step);
//   bitrate_search_kernel   one workgroup: turns the histogram into suffix counts, then runs the reference's
//                           whole bisection (or its incremental correction) in double, each probe being two
//                           threshold searches over the patterns and two look-ups.
// The result (u, average width, target - average) equals what the torch ops of the reference give for the same
// norms: the counts are exact integers and the arithmetic of the search is the same IEEE double arithmetic.
#include "dq_bitwidth.cuh"
#include "dq_launch.h"

namespace dq {

namespace {

constexpr int kSearchThreads = 1024;
constexpr int kBinsPerThread = 32;             // 1024 x 32 = 32768 >= kNanBin + 1

__global__ __launch_bounds__(kHistThreads) void norm_histogram_kernel(const uint16_t *__restrict__ stats, int64_t nsc,
                                                                     uint32_t *__restrict__ hist)
{
    __shared__ uint32_t local[kHistWords];
    count_norm_patterns(stats, nsc, (int64_t)blockIdx.x * kHistBatch, (int64_t)gridDim.x * kHistBatch, hist, local);
}

struct Probe {
    double avg, delta;
};

// out[0..2] = u, average width, target - average; out[3] = number of probes.  hist: pattern counts in, zeros out.
// prev_u_dev != nullptr: the starting point of the correction is *prev_u_dev (it may be out[0] of the previous search)
__global__ __launch_bounds__(kSearchThreads) void bitrate_search_kernel(uint32_t *__restrict__ hist, int mode, double prev_u,
                                                                       const double *prev_u_dev, double target,
                                                                       double *out)
{
    __shared__ uint32_t part[kSearchThreads];
    __shared__ int thr[2];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    if (prev_u_dev) prev_u = *prev_u_dev; // read by every thread long before thread 0 writes out[]

    // suffix counts in place: hist[p] = number of norms whose pattern is >= p, p = 0 .. kMaxPattern
    uint32_t v[kBinsPerThread];
    uint32_t own = 0;
#pragma unroll
    for (int k = 0; k < kBinsPerThread; k++) {
        const int p = kBinsPerThread * t + k;
        v[k] = p <= kMaxPattern ? hist[p] : 0u;
        own += v[k];
    }
    part[t] = own;
    __syncthreads();
    for (int off = 1; off < kSearchThreads; off <<= 1) {
        const uint32_t x = t + off < kSearchThreads ? part[t + off] : 0u;
        __syncthreads();
        part[t] += x;
        __syncthreads();
    }
    uint32_t run = part[t] - own; // the bins of the threads above
#pragma unroll
    for (int k = kBinsPerThread - 1; k >= 0; k--) {
        const int p = kBinsPerThread * t + k;
        run += v[k];
        if (p <= kMaxPattern) hist[p] = run;
    }
    __syncthreads();
    const uint64_t total = (uint64_t)hist[0] + hist[kNanBin];

    int probes = 0;
    // every thread evaluates the same doubles, so the control flow below is uniform without a broadcast
    const auto probe = [&](double u) {
        width_thresholds((float)u, thr, wave, lane);
        __syncthreads();
        const int t4 = thr[0], t8 = thr[1];
        const uint64_t n4 = t4 <= kMaxPattern ? hist[t4] : 0u, n8 = t8 <= kMaxPattern ? hist[t8] : 0u;
        __syncthreads();
        probes++;
        Probe r;
        r.avg = total ? (double)(2 * total + 2 * n4 + 4 * n8) / (double)total : 0.0;
        r.delta = target - r.avg;
        return r;
    };
    const double u_min = -10.0, u_max = 60.0, tol = 0.1;
    double res_u, res_avg, res_delta;
    if (mode == 0) {
        // comm_hooks.py:94-114
        double low = u_min, high = u_max;
        Probe r = probe(high);
        double best_u = high, best_avg = r.avg, best_delta = r.delta;
        bool done = false;
        for (int it = 0; it < 32 && !done; it++) {
            const double mid = (low + high) * 0.5;
            r = probe(mid);
            if (__builtin_fabs(r.delta) < __builtin_fabs(best_delta)) {
                best_u = mid; best_avg = r.avg; best_delta = r.delta;
            }
            if (__builtin_fabs(r.delta) <= tol) {
                best_u = mid; best_avg = r.avg; best_delta = r.delta;
                done = true;
            } else if (r.delta > 0) {
                low = mid;
            } else {
                high = mid;
            }
        }
        res_u = best_u; res_avg = best_avg; res_delta = best_delta;
    } else {
        // comm_hooks.py:117-139
        const double start = __builtin_fmax(u_min, __builtin_fmin(u_max, prev_u));
        Probe r = probe(start);
        res_u = start; res_avg = r.avg; res_delta = r.delta;
        if (!(__builtin_fabs(r.delta) <= tol)) {
            const double old_delta = r.delta;
            double step = old_delta;
            bool done = false;
            for (int it = 0; it < 32 && !done; it++) {
                const double cand = __builtin_fmax(u_min, __builtin_fmin(u_max, start + step));
                r = probe(cand);
                if (__builtin_fabs(r.delta) < __builtin_fabs(res_delta)) {
                    res_u = cand; res_avg = r.avg; res_delta = r.delta;
                }
                if (__builtin_fabs(r.delta) <= tol || old_delta * r.delta >= 0) {
                    res_u = cand; res_avg = r.avg; res_delta = r.delta;
                    done = true;
                }
                step *= 0.5;
            }
        }
    }
    if (t == 0) {
        out[0] = res_u; out[1] = res_avg; out[2] = res_delta; out[3] = (double)probes;
    }
    // ready for the next accumulation
#pragma unroll
    for (int k = 0; k < kBinsPerThread; k++) hist[kBinsPerThread * t + k] = 0u;
}

} // namespace

int64_t bitrate_hist_ints() { return (int64_t)kSearchThreads * kBinsPerThread; }

hipError_t launch_norm_histogram(const void *stats, int64_t nsc, uint32_t *hist, hipStream_t stream)
{
    const unsigned grid = (unsigned)std::min<int64_t>((nsc + kHistBatch - 1) / kHistBatch, 1024);
    hipLaunchKernelGGL(norm_histogram_kernel, dim3(grid), dim3(kHistThreads), 0, stream, static_cast<const uint16_t *>(stats), nsc,
                       hist);
    return hipGetLastError();
}

hipError_t launch_bitrate_search(uint32_t *hist, int mode, double prev_u, const double *prev_u_dev, double target, double *out,
                                 hipStream_t stream)
{
    hipLaunchKernelGGL(bitrate_search_kernel, dim3(1), dim3(kSearchThreads), 0, stream, hist, mode, prev_u, prev_u_dev, target,
                       out);
    return hipGetLastError();
}

} // namespace dq
