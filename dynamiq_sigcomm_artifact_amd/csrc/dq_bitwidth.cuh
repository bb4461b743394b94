// The dynamic bit-width rule on the device (testbed_evaluation/new_comm_hooks/comm_hooks.py:64-70) and the two
// norm patterns at which the width changes, shared by the group plan and the search for the offset u.
#pragma once

#include "dq_device.cuh"

namespace dq {

__device__ __forceinline__ float round_bf16(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }

// testbed_evaluation/new_comm_hooks/comm_hooks.py:64-70 on a bf16 norm: every torch op computes in
// binary32 and rounds its result to bf16
__device__ __forceinline__ int64_t qbits_of_norm(uint32_t norm_bits, float u)
{
    const float eps = 1e-20f;
    float x = bf16_bits_to_f32(norm_bits);
    x = (x != x) ? x : round_bf16(x > eps ? x : eps);
    x = round_bf16(log2_det(x));
    x = round_bf16(x * (float)(4.0 / (512.0 / 17.0)));
    x = round_bf16(x + u);
    x = (x != x) ? x : round_bf16(x > eps ? x : eps);
    x = round_bf16(log2_det(x));
    x = __builtin_floorf(x);
    int z = (x != x) ? 1 : (x < 1.0f ? 1 : (x > 3.0f ? 3 : (int)x));
    return (int64_t)1 << z;
}

constexpr int kMaxPattern = 0x7f80; // +infinity: the patterns 0 .. 0x7f80 are the non-negative norms in ascending order

// The width is a monotone step function of the bf16 norm pattern (every operation of the rule is monotone, and
// neighbouring bf16 values are 2^-8 apart, far more than the error of the log2 polynomial), so two patterns
// describe it for a given u.
// index of the first of 64 probes lo + step * (l + 1) (clamped to kMaxPattern) whose width is >= target; 64 if none
__device__ __forceinline__ int first_width_probe(float u, int lo, int step, int lane, int64_t target)
{
    const int p = min(lo + step * (lane + 1), kMaxPattern);
    const uint64_t hit = __builtin_amdgcn_ballot_w64(qbits_of_norm((uint32_t)p, u) >= target);
    return hit ? __builtin_ctzll(hit) : 64;
}

// wave 0 finds thr[0] = the smallest pattern of width >= 4, wave 1 thr[1] = that of width 8
// (kMaxPattern + 1 when no pattern reaches it); other waves do nothing.  No barrier inside.
__device__ __forceinline__ void width_thresholds(float u, int *thr, int wave, int lane)
{
    if (wave > 1) return;
    const int64_t target = wave == 0 ? 4 : 8;
    int t = kMaxPattern + 1;
    const int a = first_width_probe(u, -1, 512, lane, target);
    if (a < 64) {
        const int lo = -1 + 512 * a;
        const int b = first_width_probe(u, lo, 8, lane, target);
        const int lo2 = lo + 8 * b;
        t = lo2 + 1 + first_width_probe(u, lo2, 1, lane, target);
    }
    if (lane == 0) thr[wave] = t;
}

// ---- histogram of the norm patterns (what the search for u works on) ----------------------------------

constexpr int kNanBin = kMaxPattern + 1; // NaN norms: 2 bits whatever u is

// negative norms (and -0) are clamped to the same epsilon as +0: bin 0
__device__ __forceinline__ int bin_of(uint32_t pattern)
{
    if (pattern <= (uint32_t)kMaxPattern) return (int)pattern;
    return (pattern & 0x7fffu) > (uint32_t)kMaxPattern ? kNanBin : 0;
}

// A workgroup of kHistThreads threads counts batches of up to 8192 norms in LDS -- 16-bit counters, two per word,
// so the whole range of patterns fits into 64 KB -- and adds the non-zero counters to the histogram in memory
// after each batch: a few hundred atomics per batch instead of one per norm, most of which would hit the same
// few hundred words.  The workgroup takes the batches first, first + stride, ...; local: kHistWords words of LDS.
constexpr int kHistThreads = 1024;
constexpr int kHistBatch = 8192; // norms per batch (a 16-bit counter holds up to 65535)
constexpr int kHistWords = 16384; // 32768 counters

__device__ __forceinline__ void count_norm_patterns(const uint16_t *__restrict__ stats, int64_t nsc, int64_t first,
                                                    int64_t stride, uint32_t *__restrict__ hist, uint32_t *local)
{
    const int t = threadIdx.x;
    for (int64_t batch0 = first; batch0 < nsc; batch0 += stride) {
        for (int w = t; w < kHistWords; w += kHistThreads) local[w] = 0u;
        __syncthreads();
        const int64_t end = min(batch0 + kHistBatch, nsc);
        for (int64_t i = batch0 + t; i < end; i += kHistThreads) {
            const int bin = bin_of(stats[2 * i + 1]);
            atomicAdd(&local[bin >> 1], 1u << (16 * (bin & 1)));
        }
        __syncthreads();
        for (int w = t; w < kHistWords; w += kHistThreads) {
            const uint32_t pair = local[w];
            if (pair & 0xffffu) atomicAdd(&hist[2 * w], pair & 0xffffu);
            if (pair >> 16) atomicAdd(&hist[2 * w + 1], pair >> 16);
        }
        __syncthreads();
    }
}

} // namespace dq
