// Superchunk (256-element) mean-centring and its inverse.
//
// superchunk_mean_center: one wave owns one superchunk.  Lane L holds elements
// L, L+64, L+128, L+192, which makes the reference's fixed reduction tree
// (shared-memory halving, stride 128 -> 1, csrc/cuda_hadamard.cu:1286-1292)
// two in-lane adds followed by six "lane L += lane L+stride" steps; the sum is
// therefore associated exactly as in the reference and the statistics are
// bit-identical.  Numerics: csrc/cuda_hadamard.cu:1257-1349.
//
// superchunk_add_mean_copy: pure streaming, csrc/cuda_hadamard.cu:1351-1369.
#include "dq_device.cuh"
#include "dq_launch.h"

namespace dq {

template <int CTRL> __device__ __forceinline__ float dpp_shift(float v)
{
    // lanes without a source inside the row receive 0 (bound_ctrl); they only
    // feed partial sums that the reduction never reads again
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

template <int DT>
__global__ __launch_bounds__(256) void mean_center_kernel(const void *__restrict__ src, void *__restrict__ residual,
                                                          uint16_t *__restrict__ stats, int64_t n, int64_t nsc,
                                                          float world)
{
    typedef ElemIO<DT> IO;
    const int lane = threadIdx.x & 63;
    const int64_t sc = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sc >= nsc) return;
    const int64_t start = sc * 256;
    int64_t valid64 = n - start;
    const int valid = (int)(valid64 > 256 ? 256 : (valid64 < 0 ? 0 : valid64));

    float v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int l = lane + 64 * k;
        v[k] = (l < valid) ? IO::load(src, start + l) / world : 0.0f;
    }
    // stride 128 then 64 (in lane)
    float sum = (v[0] + v[2]) + (v[1] + v[3]);
    float sq = (v[0] * v[0] + v[2] * v[2]) + (v[1] * v[1] + v[3] * v[3]);
    // stride 32, 16 (across rows), then 8, 4, 2, 1 (inside the row)
    sum += __shfl_down(sum, 32, 64);
    sq += __shfl_down(sq, 32, 64);
    sum += __shfl_down(sum, 16, 64);
    sq += __shfl_down(sq, 16, 64);
    sum += dpp_shift<0x108>(sum); // row_shl:8 -> lane i reads lane i+8
    sq += dpp_shift<0x108>(sq);
    sum += dpp_shift<0x104>(sum);
    sq += dpp_shift<0x104>(sq);
    sum += dpp_shift<0x102>(sum);
    sq += dpp_shift<0x102>(sq);
    sum += dpp_shift<0x101>(sum);
    sq += dpp_shift<0x101>(sq);
    const float total = __shfl(sum, 0, 64);
    const float mean = valid > 0 ? total / (float)valid : 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int l = lane + 64 * k;
        IO::store(residual, start + l, (l < valid) ? v[k] - mean : 0.0f);
    }
    if (lane == 0) {
        stats[2 * sc] = (uint16_t)f32_to_bf16_bits(mean);
        stats[2 * sc + 1] = (uint16_t)f32_to_bf16_bits(sq);
    }
}

template <int DT>
__global__ __launch_bounds__(256) void add_mean_copy_kernel(const void *__restrict__ residual, void *__restrict__ dst,
                                                            const uint16_t *__restrict__ stats, int64_t begin, int64_t n)
{
    typedef ElemIO<DT> IO;
    // 8 consecutive elements per thread, begin % 8 == 0: a group never straddles a superchunk
    const int64_t i0 = begin + ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i0 >= n) return;
    const float mean = bf16_bits_to_f32(stats[2 * (i0 >> 8)]);
    const int cnt = (int)min((int64_t)8, n - i0);
    for (int k = 0; k < cnt; k++) IO::store(dst, i0 + k, IO::load(residual, i0 + k) + mean);
}

// 16-byte vector variant for 2-byte element types with aligned pointers
template <int DT>
__global__ __launch_bounds__(256) void add_mean_copy_vec_kernel(const uint4 *__restrict__ residual, uint4 *__restrict__ dst,
                                                                const uint16_t *__restrict__ stats, int64_t nvec)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvec) return;
    const float mean = bf16_bits_to_f32(stats[2 * (i >> 5)]);
    uint4 r = residual[i];
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float lo, hi;
        if (DT == DQ_BF16) {
            lo = __uint_as_float(w[k] << 16) + mean;
            hi = __uint_as_float(w[k] & 0xffff0000u) + mean;
            w[k] = f32x2_to_bf16x2(lo, hi);
        } else {
            lo = f16_bits_to_f32(w[k] & 0xffffu) + mean;
            hi = f16_bits_to_f32(w[k] >> 16) + mean;
            w[k] = f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
        }
    }
    dst[i] = make_uint4(w[0], w[1], w[2], w[3]);
}

hipError_t launch_mean_center(const void *src, void *residual, void *stats, int64_t n, int world_size, int dtype,
                              hipStream_t stream)
{
    const int64_t nsc = (n + 255) / 256;
    dim3 grid((unsigned)((nsc + 3) / 4)), block(256);
    uint16_t *st = static_cast<uint16_t *>(stats);
    const float world = (float)world_size;
    switch (dtype) {
    case DQ_F16: hipLaunchKernelGGL(mean_center_kernel<DQ_F16>, grid, block, 0, stream, src, residual, st, n, nsc, world); break;
    case DQ_BF16: hipLaunchKernelGGL(mean_center_kernel<DQ_BF16>, grid, block, 0, stream, src, residual, st, n, nsc, world); break;
    default: hipLaunchKernelGGL(mean_center_kernel<DQ_F32>, grid, block, 0, stream, src, residual, st, n, nsc, world); break;
    }
    return hipGetLastError();
}

hipError_t launch_add_mean_copy(const void *residual, void *dst, const void *stats, int64_t n, int dtype,
                                hipStream_t stream)
{
    const uint16_t *st = static_cast<const uint16_t *>(stats);
    const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
    int64_t done = 0;
    if (aligned && dtype != DQ_F32 && n >= 8) {
        const int64_t nvec = n / 8;
        dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
        if (dtype == DQ_BF16)
            hipLaunchKernelGGL(add_mean_copy_vec_kernel<DQ_BF16>, grid, block, 0, stream, static_cast<const uint4 *>(residual),
                               static_cast<uint4 *>(dst), st, nvec);
        else
            hipLaunchKernelGGL(add_mean_copy_vec_kernel<DQ_F16>, grid, block, 0, stream, static_cast<const uint4 *>(residual),
                               static_cast<uint4 *>(dst), st, nvec);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        done = nvec * 8;
        if (done == n) return hipSuccess;
    }
    const int64_t rest = n - done;
    dim3 grid((unsigned)((rest + 2047) / 2048)), block(256);
    switch (dtype) {
    case DQ_F16: hipLaunchKernelGGL(add_mean_copy_kernel<DQ_F16>, grid, block, 0, stream, residual, dst, st, done, n); break;
    case DQ_BF16: hipLaunchKernelGGL(add_mean_copy_kernel<DQ_BF16>, grid, block, 0, stream, residual, dst, st, done, n); break;
    default: hipLaunchKernelGGL(add_mean_copy_kernel<DQ_F32>, grid, block, 0, stream, residual, dst, st, done, n); break;
    }
    return hipGetLastError();
}

} // namespace dq
