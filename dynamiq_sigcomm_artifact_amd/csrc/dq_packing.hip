// EDEN bit-plane packing (csrc/cuda_packing.cu:11-29,76-95) and the THC-style
// in-place stochastic rounding (csrc/cuda_hadamard.cu:607-627).
//
#include "dq_device.cuh"
#include "dq_launch.h"

namespace dq {

// sixteen consecutive bins per thread, i.e. half a word of every bit plane: the bins' bytes go through two
// 8 x 8 bit transposes (one per eight bins), after which byte j of a result is plane 8 s + j of those bins
template <bool VEC>
__global__ __launch_bounds__(256) void bins_to_bits_kernel(const int32_t *__restrict__ bins, int64_t nbins,
                                                           uint32_t *__restrict__ arr, int nbits)
{
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t first = g * 16;
    if (first >= nbins) return; // nbins is a multiple of 32
    const int64_t words = nbins >> 5;
    uint32_t b[16];
    if (VEC) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int4 v = *reinterpret_cast<const int4 *>(bins + first + 4 * q);
            b[4 * q] = (uint32_t)v.x; b[4 * q + 1] = (uint32_t)v.y; b[4 * q + 2] = (uint32_t)v.z; b[4 * q + 3] = (uint32_t)v.w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) b[k] = (uint32_t)bins[first + k];
    }
    uint16_t *half = reinterpret_cast<uint16_t *>(arr) + g;
    for (int s = 0; 8 * s < nbits; s++) {
        uint64_t lo = 0, hi = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            lo |= (uint64_t)((b[k] >> (8 * s)) & 0xffu) << (8 * k);
            hi |= (uint64_t)((b[8 + k] >> (8 * s)) & 0xffu) << (8 * k);
        }
        lo = transpose8x8(lo);
        hi = transpose8x8(hi);
        const int planes = min(8, nbits - 8 * s);
        for (int j = 0; j < planes; j++)
            half[(int64_t)(8 * s + j) * words * 2] = (uint16_t)(((lo >> (8 * j)) & 0xffu) | (((hi >> (8 * j)) & 0xffu) << 8));
    }
}

// the inverse: sixteen consecutive bins per thread from its half word of every plane (the transpose is its own
// inverse); the bins leave through a per-wave LDS tile so that the lanes store contiguous 16-byte pieces
__global__ __launch_bounds__(256) void bits_to_bins_kernel(int32_t *__restrict__ bins, int64_t nbins,
                                                           const uint32_t *__restrict__ arr, int nbits)
{
    __shared__ __attribute__((aligned(16))) uint4 tiles[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t first = g * 16, wave_first = (g - lane) * 16;
    const int64_t words = nbins >> 5;
    const bool in = first < nbins; // nbins is a multiple of 32
    uint32_t b[16];
#pragma unroll
    for (int k = 0; k < 16; k++) b[k] = 0;
    if (in) {
        const uint16_t *half = reinterpret_cast<const uint16_t *>(arr) + g;
        for (int s = 0; 8 * s < nbits; s++) {
            uint64_t lo = 0, hi = 0;
            const int planes = min(8, nbits - 8 * s);
            for (int j = 0; j < planes; j++) {
                const uint32_t h = half[(int64_t)(8 * s + j) * words * 2];
                lo |= (uint64_t)(h & 0xffu) << (8 * j);
                hi |= (uint64_t)(h >> 8) << (8 * j);
            }
            lo = transpose8x8(lo);
            hi = transpose8x8(hi);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                b[k] |= (uint32_t)((lo >> (8 * k)) & 0xffu) << (8 * s);
                b[8 + k] |= (uint32_t)((hi >> (8 * k)) & 0xffu) << (8 * s);
            }
        }
    }
    if (wave_first >= nbins) return; // the whole wave
    store_wave_words16(tiles[wave], b, reinterpret_cast<uint4 *>(bins + wave_first), lane,
                       (int)min((int64_t)256, (nbins - wave_first) >> 2));
}

hipError_t launch_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int nbits, hipStream_t stream)
{
    const dim3 grid((unsigned)((nbins / 16 + 255) / 256)), block(256);
    if ((reinterpret_cast<uintptr_t>(bins) & 15) == 0)
        hipLaunchKernelGGL(bins_to_bits_kernel<true>, grid, block, 0, stream, bins, nbins, arr, nbits);
    else
        hipLaunchKernelGGL(bins_to_bits_kernel<false>, grid, block, 0, stream, bins, nbins, arr, nbits);
    return hipGetLastError();
}

hipError_t launch_bits_to_bins(int32_t *bins, int64_t nbins, const uint32_t *arr, int nbits, hipStream_t stream)
{
    // nbins is a multiple of 32 and bins 16-byte aligned: so is every group of sixteen
    hipLaunchKernelGGL(bits_to_bins_kernel, dim3((unsigned)((nbins / 16 + 255) / 256)), dim3(256), 0, stream, bins, nbins, arr, nbits);
    return hipGetLastError();
}

// four consecutive elements per thread share one Philox block keyed by
// (seed, element index / 4); u = top 24 bits * 2^-24 in [0, 1)
__global__ __launch_bounds__(256) void quantization_kernel(float *__restrict__ vec, int64_t n, float div_factor,
                                                           float tensor_max, uint32_t k0, uint32_t k1, bool vec16)
{
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t i0 = g * 4;
    if (i0 >= n) return;
    uint32_t c[4] = {(uint32_t)g, (uint32_t)((uint64_t)g >> 32), 0u, 0u};
    philox4x32_10(c, k0, k1);
    const int cnt = (int)min((int64_t)4, n - i0);
    auto round_one = [&](float x, uint32_t word) {
        float t = x / div_factor;
        t = t < tensor_max ? t : tensor_max;
        t = t > -tensor_max ? t : -tensor_max;
        const float fl = __builtin_floorf(t);
        const float prob = t - fl;
        const float u = (float)(word >> 8) * 5.9604644775390625e-08f;
        return fl + ((u < prob) ? 1.0f : 0.0f);
    };
    if (cnt == 4 && vec16) {
        // the thread's four elements in one 16-byte access each way
        float4 *p = reinterpret_cast<float4 *>(vec + i0);
        float4 x = *p;
        x.x = round_one(x.x, c[0]);
        x.y = round_one(x.y, c[1]);
        x.z = round_one(x.z, c[2]);
        x.w = round_one(x.w, c[3]);
        *p = x;
        return;
    }
    for (int k = 0; k < cnt; k++) vec[i0 + k] = round_one(vec[i0 + k], c[k]);
}

hipError_t launch_quantization(float *vec, int64_t n, float div_factor, float tensor_max, uint64_t seed, hipStream_t stream)
{
    const int64_t groups = (n + 3) / 4;
    hipLaunchKernelGGL(quantization_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, stream, vec, n, div_factor,
                       tensor_max, (uint32_t)seed, (uint32_t)(seed >> 32), (reinterpret_cast<uintptr_t>(vec) & 15) == 0);
    return hipGetLastError();
}

} // namespace dq
