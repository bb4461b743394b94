// The fixed-proportion allocation (testbed_evaluation/new_comm_hooks/comm_hooks.py:710-721) for buckets too long for the
// one-launch counting sort of dq_grouping.hip: the reference's training scripts give DDP a bucket cap of 4000 MB for the
// DynamiQ hooks (testbed_evaluation/train_llm_causal.py:416), i.e. one bucket of millions of superchunks.
//
//   keys     key_i = the 16-bit descending-order key of the norm pattern of superchunk i (NaN first, then +inf ... +0 = -0
//            ... -inf: the order of dq_group_plan_sorted), value_i = i
//   sort     stable least-significant-digit radix sort of the (key, value) pairs over the 16 key bits (rocPRIM through
//            hipCUB, double-buffered: its scratch is a few histograms), so equal norms keep ascending index
//   split    the first `top` values to the 8-bit list, the last `bottom` to the 2-bit list, the rest to the 4-bit list;
//            work[0..3] = the counts
// Everything lives in the caller's `work` buffer; no allocation, no host synchronisation.
#include <algorithm>

#include <hipcub/hipcub.hpp>

#include "dq_bitwidth.cuh"
#include "dq_launch.h"

namespace dq {

namespace {

constexpr int kSortBlock = 256;

__host__ __device__ inline size_t align256(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

// Scratch of the radix sort with double buffers: what the library itself asks for on this device for this many pairs (a
// host-side query that launches nothing), padded by an eighth, and never less than nsc / 8 + 64 KiB (the sizes seen so far
// are 0.034-0.10 bytes per item plus a constant).  Without a device to ask (a host that only sizes buffers) the floor alone.
inline size_t sort_scratch_bound(int64_t nsc)
{
    size_t bound = align256((size_t)nsc / 8 + 65536);
    hipcub::DoubleBuffer<uint16_t> keys(nullptr, nullptr);
    hipcub::DoubleBuffer<int32_t> vals(nullptr, nullptr);
    size_t asked = 0;
    if (nsc <= (int64_t)0x7fffffff &&
        hipcub::DeviceRadixSort::SortPairs(nullptr, asked, keys, vals, (int)nsc, 0, 16, nullptr) == hipSuccess)
        bound = std::max(bound, align256(asked + asked / 8));
    else
        (void)hipGetLastError();
    return bound;
}

struct LargePlanLayout {
    size_t keys[2], vals[2], scratch, total; // byte offsets into the workspace behind the 8-int header
};

inline LargePlanLayout layout_for(int64_t nsc)
{
    LargePlanLayout l;
    size_t at = 0;
    for (int k = 0; k < 2; k++) { l.keys[k] = at; at += align256((size_t)nsc * sizeof(uint16_t)); }
    for (int k = 0; k < 2; k++) { l.vals[k] = at; at += align256((size_t)nsc * sizeof(int32_t)); }
    l.scratch = at;
    l.total = at + sort_scratch_bound(nsc);
    return l;
}

__device__ __forceinline__ uint32_t descending_key16(uint32_t pattern)
{
    const uint32_t mag = pattern & 0x7fffu;
    if (mag > (uint32_t)kMaxPattern) return 0u;  // NaN of either sign
    if (pattern & 0x8000u) return 0x7fffu + mag; // -0 -> 0x7fff (the key of +0), -inf -> 0xff7f
    return 0x7fffu - mag;                        // +inf -> 0x7f, +0 -> 0x7fff
}

__global__ __launch_bounds__(kSortBlock) void sort_keys_kernel(const uint32_t *__restrict__ pairs, int64_t nsc,
                                                               uint16_t *__restrict__ keys, int32_t *__restrict__ vals)
{
    const int64_t i = (int64_t)blockIdx.x * kSortBlock + threadIdx.x;
    if (i >= nsc) return;
    keys[i] = (uint16_t)descending_key16(pairs[i] >> 16); // a (mean, norm) pair: the norm is the high half
    vals[i] = (int32_t)i;
}

__global__ __launch_bounds__(kSortBlock) void sort_split_kernel(const int32_t *__restrict__ sorted, int64_t nsc, int64_t top,
                                                                int64_t bottom, int64_t *__restrict__ qbits_out,
                                                                int32_t *__restrict__ order, int32_t *__restrict__ work)
{
    const int64_t p = (int64_t)blockIdx.x * kSortBlock + threadIdx.x;
    if (p == 0) {
        work[0] = (int32_t)top;
        work[1] = (int32_t)(nsc - top - bottom);
        work[2] = (int32_t)bottom;
        work[3] = 0;
    }
    if (p >= nsc) return;
    const int32_t i = sorted[p];
    const int64_t mid_end = nsc - bottom;
    int region;
    int64_t at;
    if (p < top) region = 0, at = p;
    else if (p < mid_end) region = 1, at = p - top;
    else region = 2, at = p - mid_end;
    order[(int64_t)region * nsc + at] = i;
    if (qbits_out) qbits_out[i] = region == 0 ? 8 : (region == 1 ? 4 : 2);
}

} // namespace

// int32 entries of `work` for dq_group_plan_sorted on nsc > 65535 superchunks
int64_t group_plan_sorted_large_work_ints(int64_t nsc) { return 8 + (int64_t)((layout_for(nsc).total + 3) / 4) + 64; }

hipError_t launch_group_plan_sorted_large(const void *stats, int64_t nsc, int64_t top, int64_t bottom, int64_t *qbits_out,
                                          int32_t *order, int32_t *work, int64_t work_ints, hipStream_t stream)
{
    if (nsc > (int64_t)0x7fffffff || work_ints < group_plan_sorted_large_work_ints(nsc)) return hipErrorInvalidValue;
    // the arrays start at the first 256-byte boundary behind the header
    char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(work + 8) + 255) & ~(uintptr_t)255);
    const LargePlanLayout l = layout_for(nsc);
    const size_t scratch_room = l.total - l.scratch;
    hipcub::DoubleBuffer<uint16_t> keys(reinterpret_cast<uint16_t *>(base + l.keys[0]), reinterpret_cast<uint16_t *>(base + l.keys[1]));
    hipcub::DoubleBuffer<int32_t> vals(reinterpret_cast<int32_t *>(base + l.vals[0]), reinterpret_cast<int32_t *>(base + l.vals[1]));
    size_t scratch_bytes = 0;
    hipError_t e = hipcub::DeviceRadixSort::SortPairs(nullptr, scratch_bytes, keys, vals, (int)nsc, 0, 16, stream);
    if (e != hipSuccess) return e;
    if (scratch_bytes > scratch_room) return hipErrorOutOfMemory;
    const unsigned blocks = (unsigned)((nsc + kSortBlock - 1) / kSortBlock);
    hipLaunchKernelGGL(sort_keys_kernel, dim3(blocks), dim3(kSortBlock), 0, stream, static_cast<const uint32_t *>(stats), nsc,
                       keys.Current(), vals.Current());
    e = hipcub::DeviceRadixSort::SortPairs(base + l.scratch, scratch_bytes, keys, vals, (int)nsc, 0, 16, stream);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sort_split_kernel, dim3(blocks), dim3(kSortBlock), 0, stream, vals.Current(), nsc, top, bottom, qbits_out,
                       order, work);
    return hipGetLastError();
}

} // namespace dq
