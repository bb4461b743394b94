// EDEN bit-plane packing (csrc/cuda_packing.cu:11-29,76-95) and the THC-style
// in-place stochastic rounding (csrc/cuda_hadamard.cu:607-627).
//
// Packing on wave64: one lane per bin, one 64-bit ballot per bit plane, whose
// halves are the two consecutive 32-bin words of that plane.
#include "dq_device.cuh"
#include "dq_launch.h"

namespace dq {

__global__ __launch_bounds__(256) void bins_to_bits_kernel(const int32_t *__restrict__ bins, int64_t nbins,
                                                           uint32_t *__restrict__ arr, int nbits)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t words = nbins >> 5;
    const int lane = threadIdx.x & 63;
    const uint32_t b = (i < nbins) ? (uint32_t)bins[i] : 0u;
    const int64_t w = i >> 5;
    for (int p = 0; p < nbits; p++) {
        const uint64_t m = __ballot((b >> p) & 1u);
        if ((lane & 31) == 0 && w < words) arr[(int64_t)p * words + w] = (uint32_t)(m >> (lane & 32));
    }
}

// four consecutive bins per thread: they share the word of every bit plane
__global__ __launch_bounds__(256) void bits_to_bins_kernel(int32_t *__restrict__ bins, int64_t nbins,
                                                           const uint32_t *__restrict__ arr, int nbits)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= nbins) return;
    const int64_t words = nbins >> 5;
    const int64_t w = i >> 5;
    const int t = (int)(i & 31);
    int32_t v[4] = {0, 0, 0, 0};
    for (int p = 0; p < nbits; p++) {
        const uint32_t word = arr[(int64_t)p * words + w] >> t;
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] += (int32_t)((word >> k) & 1u) << p;
    }
    *reinterpret_cast<int4 *>(bins + i) = make_int4(v[0], v[1], v[2], v[3]);
}

hipError_t launch_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int nbits, hipStream_t stream)
{
    hipLaunchKernelGGL(bins_to_bits_kernel, dim3((unsigned)((nbins + 255) / 256)), dim3(256), 0, stream, bins, nbins, arr, nbits);
    return hipGetLastError();
}

hipError_t launch_bits_to_bins(int32_t *bins, int64_t nbins, const uint32_t *arr, int nbits, hipStream_t stream)
{
    // nbins is a multiple of 32 and bins a whole tensor: groups of four are 16-byte aligned
    hipLaunchKernelGGL(bits_to_bins_kernel, dim3((unsigned)((nbins / 4 + 255) / 256)), dim3(256), 0, stream, bins, nbins, arr, nbits);
    return hipGetLastError();
}

// four consecutive elements per thread share one Philox block keyed by
// (seed, element index / 4); u = top 24 bits * 2^-24 in [0, 1)
__global__ __launch_bounds__(256) void quantization_kernel(float *__restrict__ vec, int64_t n, float div_factor,
                                                           float tensor_max, uint32_t k0, uint32_t k1)
{
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t i0 = g * 4;
    if (i0 >= n) return;
    uint32_t c[4] = {(uint32_t)g, (uint32_t)((uint64_t)g >> 32), 0u, 0u};
    philox4x32_10(c, k0, k1);
    const int cnt = (int)min((int64_t)4, n - i0);
    for (int k = 0; k < cnt; k++) {
        float t = vec[i0 + k] / div_factor;
        t = t < tensor_max ? t : tensor_max;
        t = t > -tensor_max ? t : -tensor_max;
        const float fl = __builtin_floorf(t);
        const float prob = t - fl;
        const float u = (float)(c[k] >> 8) * 5.9604644775390625e-08f;
        vec[i0 + k] = fl + ((u < prob) ? 1.0f : 0.0f);
    }
}

hipError_t launch_quantization(float *vec, int64_t n, float div_factor, float tensor_max, uint64_t seed, hipStream_t stream)
{
    const int64_t groups = (n + 3) / 4;
    hipLaunchKernelGGL(quantization_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, stream, vec, n, div_factor,
                       tensor_max, (uint32_t)seed, (uint32_t)(seed >> 32));
    return hipGetLastError();
}

} // namespace dq
