// Stable partition of the superchunks of a bucket by their bit width: what three
// torch.nonzero(qbits == w) calls produce in the reference
// (testbed_evaluation/new_comm_hooks/comm_hooks.py:964-966), as two launches and no
// host synchronisation.
//
//   order[0 .. n8)            indices i with qbits[i] == 8, ascending
//   order[n8 .. n8+n4)        indices with qbits[i] == 4, ascending
//   order[n8+n4 .. n8+n4+n2)  indices with qbits[i] == 2, ascending
//   work[0..2] = n8, n4, n2;  work[3] = superchunks of any other width (in no group)
//   work[4 + 4*b + w]         per-tile counts (tile b = superchunks [1024 b, 1024 b + 1024))
#include "dq_launch.h"

namespace dq {

namespace {

constexpr int kTile = 1024; // superchunks per workgroup
constexpr int kThreads = 256;
constexpr int kPer = kTile / kThreads;

__device__ __forceinline__ int width_class(int64_t q) { return q == 8 ? 0 : q == 4 ? 1 : q == 2 ? 2 : 3; }

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

// where the widths come from: an int64 array, or the norm column of the interleaved bf16 stats
struct WidthsFromArray {
    const int64_t *qbits;
    __device__ __forceinline__ int64_t operator()(int64_t i) const { return qbits[i]; }
};
struct WidthsFromStats {
    const uint16_t *stats;
    float u;
    __device__ __forceinline__ int64_t operator()(int64_t i) const { return qbits_of_norm(stats[2 * i + 1], u); }
};

// three 21-bit counters in one word
__device__ __forceinline__ uint64_t one_of(int cls) { return cls < 3 ? (uint64_t)1 << (21 * cls) : 0; }
__device__ __forceinline__ int field(uint64_t p, int cls) { return (int)((p >> (21 * cls)) & 0x1fffff); }

template <class W>
__global__ __launch_bounds__(kThreads) void plan_count_kernel(W widths, int64_t nsc, int32_t *__restrict__ work)
{
    __shared__ int cnt[4];
    if (threadIdx.x < 4) cnt[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x * kPer;
    int c[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        if (base + k < nsc) c[width_class(widths(base + k))]++;
    }
#pragma unroll
    for (int w = 0; w < 4; w++) {
        if (c[w]) atomicAdd(&cnt[w], c[w]);
    }
    __syncthreads();
    if (threadIdx.x < 4) work[4 + 4 * blockIdx.x + threadIdx.x] = cnt[threadIdx.x];
}

template <class W>
__global__ __launch_bounds__(kThreads) void plan_place_kernel(W widths, int64_t *__restrict__ qbits_out, int64_t nsc,
                                                              int ntiles, int32_t *__restrict__ order,
                                                              int32_t *__restrict__ work)
{
    __shared__ int before[4], total[4];
    __shared__ uint64_t wave_sum[kThreads / 64];
    if (threadIdx.x < 4) {
        before[threadIdx.x] = 0;
        total[threadIdx.x] = 0;
    }
    __syncthreads();
    {
        int t[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
        for (int tile = threadIdx.x; tile < ntiles; tile += kThreads) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const int c = work[4 + 4 * tile + w];
                t[w] += c;
                if (tile < (int)blockIdx.x) b[w] += c;
            }
        }
#pragma unroll
        for (int w = 0; w < 4; w++) {
            if (t[w]) atomicAdd(&total[w], t[w]);
            if (b[w]) atomicAdd(&before[w], b[w]);
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x < 4) work[threadIdx.x] = total[threadIdx.x];

    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x * kPer;
    int cls[kPer];
    uint64_t mine = 0;
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        cls[k] = 3;
        if (base + k < nsc) {
            const int64_t q = widths(base + k);
            if (qbits_out) qbits_out[base + k] = q;
            cls[k] = width_class(q);
        }
        mine += one_of(cls[k]);
    }
    // inclusive scan over the wave, then over the waves of the workgroup
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint64_t incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint64_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint64_t excl = incl - mine;
    for (int w = 0; w < wave; w++) excl += wave_sum[w];

    const int group_base[3] = {0, total[0], total[0] + total[1]};
    int pos[3];
#pragma unroll
    for (int w = 0; w < 3; w++) pos[w] = group_base[w] + before[w] + field(excl, w);
#pragma unroll
    for (int k = 0; k < kPer; k++) {
#pragma unroll
        for (int w = 0; w < 3; w++) {
            if (cls[k] == w) order[pos[w]++] = (int32_t)(base + k);
        }
    }
}

} // namespace

int64_t group_plan_work_ints(int64_t nsc) { return 4 + 4 * ((nsc + kTile - 1) / kTile); }

template <class W>
static hipError_t run_plan(W widths, int64_t *qbits_out, int64_t nsc, int32_t *order, int32_t *work, hipStream_t stream)
{
    const int ntiles = (int)((nsc + kTile - 1) / kTile);
    hipLaunchKernelGGL(plan_count_kernel<W>, dim3(ntiles), dim3(kThreads), 0, stream, widths, nsc, work);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(plan_place_kernel<W>, dim3(ntiles), dim3(kThreads), 0, stream, widths, qbits_out, nsc, ntiles, order, work);
    return hipGetLastError();
}

hipError_t launch_group_plan(const int64_t *qbits, int64_t nsc, int32_t *order, int32_t *work, hipStream_t stream)
{
    return run_plan(WidthsFromArray{qbits}, nullptr, nsc, order, work, stream);
}

hipError_t launch_group_plan_stats(const void *stats, float u, int64_t nsc, int64_t *qbits_out, int32_t *order,
                                   int32_t *work, hipStream_t stream)
{
    return run_plan(WidthsFromStats{static_cast<const uint16_t *>(stats), u}, qbits_out, nsc, order, work, stream);
}

} // namespace dq
