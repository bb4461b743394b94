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

} // namespace dq
