// Superchunk (256-element) mean-centring and its inverse.
//
// superchunk_mean_center reproduces the reference's fixed reduction tree
// (shared-memory halving, stride 128 -> 1, csrc/cuda_hadamard.cu:1286-1292), so the
// sums are associated exactly as in the reference and the statistics are
// bit-identical.  Numerics: csrc/cuda_hadamard.cu:1257-1349.
//
//  * mean_center_tile_kernel (16-byte aligned buffers, whole superchunks): one wave owns
//    four superchunks; the tile comes in with 16-byte loads, is staged in LDS, and the
//    lane (row r, column j) picks up elements j + 16 k of superchunk r.  Strides 128..16
//    of the tree are then fifteen in-lane adds and strides 8..1 four row-shift steps.
//    The residual takes the same way back and leaves with 16-byte stores.
//  * mean_center_kernel (anything else, and the ragged last superchunk): one wave per
//    superchunk, lane L holds elements L + 64 k.
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
__global__ __launch_bounds__(64) void mean_center_tile_kernel(const void *__restrict__ src, void *__restrict__ residual,
                                                             uint32_t *__restrict__ stats, float *__restrict__ mean_out,
                                                             int64_t nsc, WorldDiv wd)
{
    constexpr int ESZ = DT == DQ_F32 ? 4 : 2;
    constexpr int SPR = 16 * ESZ;            // 16-byte slots per superchunk
    constexpr int RS = 256 * ESZ + 16 * ESZ; // padded LDS row stride: the four rows of a tile use disjoint banks
    __shared__ __attribute__((aligned(16))) uint8_t tile[4 * RS];

    const int lane = threadIdx.x;
    const int row = lane >> 4, j = lane & 15;
    const int64_t sc0 = (int64_t)blockIdx.x * 4;
    if (sc0 >= nsc) return;
    const int rows_here = (int)min((int64_t)4, nsc - sc0);
    const int nslots = rows_here * SPR;
    const u32x4 *gin = reinterpret_cast<const u32x4 *>(static_cast<const char *>(src) + sc0 * 256 * ESZ);
    u32x4 *gout = reinterpret_cast<u32x4 *>(static_cast<char *>(residual) + sc0 * 256 * ESZ);

    // every lane loads (the slot index is clamped into the tile), so all loads are in flight together
    const u32x4 raw0 = gin[min(lane, nslots - 1)];
    const u32x4 raw1 = gin[min(lane + 64, nslots - 1)];
    u32x4 raw2 = raw0, raw3 = raw0;
    if (ESZ == 4) {
        raw2 = gin[min(lane + 128, nslots - 1)];
        raw3 = gin[min(lane + 192, nslots - 1)];
    }
#define DQ_SLOT_PTR(s) reinterpret_cast<u32x4 *>(tile + ((s) / SPR) * RS + ((s) % SPR) * 16)
    if (lane < nslots) *DQ_SLOT_PTR(lane) = raw0;
    if (lane + 64 < nslots) *DQ_SLOT_PTR(lane + 64) = raw1;
    if (ESZ == 4) {
        if (lane + 128 < nslots) *DQ_SLOT_PTR(lane + 128) = raw2;
        if (lane + 192 < nslots) *DQ_SLOT_PTR(lane + 192) = raw3;
    }
    wave_lds_sync();

    uint8_t *mine = tile + row * RS + j * ESZ;
    float v[16];
    if (row < rows_here) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            if (DT == DQ_F32)
                v[k] = *reinterpret_cast<const float *>(mine + 16 * k * ESZ);
            else if (DT == DQ_BF16)
                v[k] = bf16_bits_to_f32(*reinterpret_cast<const uint16_t *>(mine + 16 * k * ESZ));
            else
                v[k] = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(mine + 16 * k * ESZ));
        }
        // one branch for the wave on the kind of world size, not one select per element between the two quotients
        if (wd.pow2) {
#pragma unroll
            for (int k = 0; k < 16; k++) v[k] = v[k] * wd.inv;
        } else {
            wd.divide16(v);
        }
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) v[k] = 0.0f;
    }
    // strides 128, 64, 32, 16: element j + 16 k pairs with k + 8, k + 4, k + 2, k + 1
    float a[8], b[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        a[k] = v[k] + v[k + 8];
        b[k] = v[k] * v[k] + v[k + 8] * v[k + 8];
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        a[k] += a[k + 4];
        b[k] += b[k + 4];
    }
    float sum = (a[0] + a[2]) + (a[1] + a[3]);
    float sq = (b[0] + b[2]) + (b[1] + b[3]);
    // strides 8, 4, 2, 1 inside the row of 16 lanes
    sum += dpp_shift<0x108>(sum);
    sq += dpp_shift<0x108>(sq);
    sum += dpp_shift<0x104>(sum);
    sq += dpp_shift<0x104>(sq);
    sum += dpp_shift<0x102>(sum);
    sq += dpp_shift<0x102>(sq);
    sum += dpp_shift<0x101>(sum);
    sq += dpp_shift<0x101>(sq);
    const float mean = __shfl(sum, lane & 48, 64) * 0.00390625f; // / 256, exact
    if (row < rows_here && j == 0) {
        stats[sc0 + row] = f32_to_bf16_bits(mean) | (f32_to_bf16_bits(sq) << 16);
        if (mean_out) mean_out[sc0 + row] = mean;
    }
    if (!residual) return; // statistics only
    if (row < rows_here) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const float r = v[k] - mean;
            if (DT == DQ_F32)
                *reinterpret_cast<float *>(mine + 16 * k * ESZ) = r;
            else if (DT == DQ_BF16)
                *reinterpret_cast<uint16_t *>(mine + 16 * k * ESZ) = (uint16_t)f32_to_bf16_bits(r);
            else
                *reinterpret_cast<uint16_t *>(mine + 16 * k * ESZ) = (uint16_t)f32_to_f16_bits(r);
        }
    }
    wave_lds_sync();
    // (with the streaming hint: the residual is not read again here, and the kernel that reads it next finds it no later --
    // 25 MB bf16 bucket over HBM 8.3 -> 6.0 us, mean-centre followed by compress 15.8 -> 14.5 us)
    if (lane < nslots) __builtin_nontemporal_store(*DQ_SLOT_PTR(lane), gout + lane);
    if (lane + 64 < nslots) __builtin_nontemporal_store(*DQ_SLOT_PTR(lane + 64), gout + lane + 64);
    if (ESZ == 4) {
        if (lane + 128 < nslots) __builtin_nontemporal_store(*DQ_SLOT_PTR(lane + 128), gout + lane + 128);
        if (lane + 192 < nslots) __builtin_nontemporal_store(*DQ_SLOT_PTR(lane + 192), gout + lane + 192);
    }
#undef DQ_SLOT_PTR
}

template <int DT>
__global__ __launch_bounds__(256) void mean_center_kernel(const void *__restrict__ src, void *__restrict__ residual,
                                                          uint16_t *__restrict__ stats, float *__restrict__ mean_out,
                                                          int64_t n, int64_t sc_begin, int64_t nsc, float world)
{
    typedef ElemIO<DT> IO;
    const int lane = threadIdx.x & 63;
    const int64_t sc = sc_begin + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
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
    if (residual) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int l = lane + 64 * k;
            IO::store(residual, start + l, (l < valid) ? v[k] - mean : 0.0f);
        }
    }
    if (lane == 0) {
        stats[2 * sc] = (uint16_t)f32_to_bf16_bits(mean);
        stats[2 * sc + 1] = (uint16_t)f32_to_bf16_bits(sq);
        if (mean_out) mean_out[sc] = mean;
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

// 16-byte vector variant for aligned pointers: eight 2-byte elements or four binary32 elements per thread
template <int DT>
__global__ __launch_bounds__(256) void add_mean_copy_vec_kernel(const uint4 *__restrict__ residual, uint4 *__restrict__ dst,
                                                                const uint16_t *__restrict__ stats, int64_t nvec)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvec) return;
    const float mean = bf16_bits_to_f32(stats[2 * (i >> (DT == DQ_F32 ? 6 : 5))]);
    uint4 r = residual[i];
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float lo, hi;
        if (DT == DQ_F32) {
            w[k] = __float_as_uint(__uint_as_float(w[k]) + mean);
        } else if (DT == DQ_BF16) {
            lo = __uint_as_float(w[k] << 16) + mean;
            hi = __uint_as_float(w[k] & 0xffff0000u) + mean;
            w[k] = f32x2_to_bf16x2(lo, hi);
        } else {
            lo = f16_bits_to_f32(w[k] & 0xffffu) + mean;
            hi = f16_bits_to_f32(w[k] >> 16) + mean;
            w[k] = f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
        }
    }
    stream_store(dst + i, make_uint4(w[0], w[1], w[2], w[3]));
}

template <int DT>
static hipError_t run_mean_center(const void *src, void *residual, void *stats, float *mean_out, int64_t n,
                                  int world_size, hipStream_t stream)
{
    const int64_t nsc = (n + 255) / 256;
    int64_t done = 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(residual)) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(stats) & 3) == 0;
    if (aligned && n >= 256) {
        done = n / 256;
        const WorldDiv wd = make_world_div(world_size, DT == DQ_F32 ? 4 : 2);
        hipLaunchKernelGGL(mean_center_tile_kernel<DT>, dim3((unsigned)((done + 3) / 4)), dim3(64), 0, stream, src, residual,
                           static_cast<uint32_t *>(stats), mean_out, done, wd);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess || done == nsc) return e;
    }
    hipLaunchKernelGGL(mean_center_kernel<DT>, dim3((unsigned)((nsc - done + 3) / 4)), dim3(256), 0, stream, src, residual,
                       static_cast<uint16_t *>(stats), mean_out, n, done, nsc, (float)world_size);
    return hipGetLastError();
}

// residual == nullptr: statistics only; mean_out (nullable) receives the binary32 means
hipError_t launch_mean_center(const void *src, void *residual, void *stats, float *mean_out, int64_t n, int world_size,
                              int dtype, hipStream_t stream)
{
    switch (dtype) {
    case DQ_F16: return run_mean_center<DQ_F16>(src, residual, stats, mean_out, n, world_size, stream);
    case DQ_BF16: return run_mean_center<DQ_BF16>(src, residual, stats, mean_out, n, world_size, stream);
    default: return run_mean_center<DQ_F32>(src, residual, stats, mean_out, n, world_size, stream);
    }
}

hipError_t launch_add_mean_copy(const void *residual, void *dst, const void *stats, int64_t n, int dtype,
                                hipStream_t stream)
{
    const uint16_t *st = static_cast<const uint16_t *>(stats);
    const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
    int64_t done = 0;
    const int per = dtype == DQ_F32 ? 4 : 8; // elements per 16 bytes
    if (aligned && n >= 8) {
        const int64_t nvec = n / 8 * (8 / per); // whole groups of eight elements: the kernel for the rest starts at one
        dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
        if (dtype == DQ_F32)
            hipLaunchKernelGGL(add_mean_copy_vec_kernel<DQ_F32>, grid, block, 0, stream, static_cast<const uint4 *>(residual),
                               static_cast<uint4 *>(dst), st, nvec);
        else if (dtype == DQ_BF16)
            hipLaunchKernelGGL(add_mean_copy_vec_kernel<DQ_BF16>, grid, block, 0, stream, static_cast<const uint4 *>(residual),
                               static_cast<uint4 *>(dst), st, nvec);
        else
            hipLaunchKernelGGL(add_mean_copy_vec_kernel<DQ_F16>, grid, block, 0, stream, static_cast<const uint4 *>(residual),
                               static_cast<uint4 *>(dst), st, nvec);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        done = nvec * per;
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
