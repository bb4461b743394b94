// Generic scaling-quantisation kernels: any element type (fp16 / bf16 / fp32),
// any strategy (0 AEE, 1 MEE, 2/3 hierarchical), any power-of-two chunk size
// up to 32 and any code width 2..8.  One thread owns one chunk and walks it
// serially; the 16 chunks of a hierarchical superchunk sit in one 16-lane DPP
// row, so the superchunk maximum is a row reduction without LDS or barriers.
//
// These kernels are the catch-all behind the C ABI: they also serve buffers
// whose alignment rules out the vectorised chunk-16 kernels.  Numerics follow
// csrc/cuda_hadamard.cu:768-861,941-1234 (flat) and
// csrc/cuda_hierarchical_mee.cu:698-1294 (hierarchical) of the reference.
#include "dq_device.cuh"
#include "dq_launch.h"

namespace dq {

constexpr int kGenericBlock = 256;

// ---- per-chunk bit packing ---------------------------------------------------

struct BytePacker {
    uint8_t *out;
    uint32_t acc;
    int nacc;
    __device__ __forceinline__ BytePacker(uint8_t *p) : out(p), acc(0), nacc(0) {}
    __device__ __forceinline__ void put(int code, int nbits)
    {
        acc |= (uint32_t)code << nacc;
        nacc += nbits;
        while (nacc >= 8) {
            *out++ = (uint8_t)acc;
            acc >>= 8;
            nacc -= 8;
        }
    }
};

__device__ __forceinline__ int chunk_code(const uint8_t *cb, int i, int nbits)
{
    int bit = i * nbits;
    uint32_t v = cb[bit >> 3];
    if ((bit & 7) + nbits > 8) v |= (uint32_t)cb[(bit >> 3) + 1] << 8;
    return (int)((v >> (bit & 7)) & ((1u << nbits) - 1u));
}

// maximum over a 16-lane row with the half-precision max rule
__device__ __forceinline__ float row16_hmax(float v)
{
    v = h_max(v, dpp_f32<0xB1>(v));
    v = h_max(v, dpp_f32<0x4E>(v));
    v = h_max(v, dpp_f32<0x141>(v));
    v = h_max(v, dpp_f32<0x140>(v));
    return v;
}

// ---- compress ----------------------------------------------------------------

template <int DT, int RDT, bool HIER, bool MEE>
__global__ __launch_bounds__(kGenericBlock) void generic_compress_kernel(
    const void *__restrict__ src, uint8_t *__restrict__ dst, const void *__restrict__ rnd,
    int64_t nchunks, int nbits, int C, MeeParams mp)
{
    typedef ElemIO<DT> IO;
    const int64_t chunk = (int64_t)blockIdx.x * kGenericBlock + threadIdx.x;
    const bool active = chunk < nchunks; // hierarchical: whole 16-lane rows are active or not
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int64_t base = chunk * C;

    // pass 1: chunk absmax
    float a = 0.0f;
    if (active) {
        a = __builtin_fabsf(IO::load(src, base));
        for (int i = 1; i < C; i++) {
            float v = __builtin_fabsf(IO::load(src, base + i));
            a = (DT == DQ_F16) ? h_max(a, v) : __builtin_fmaxf(a, v);
        }
    }

    float d;             // scale the codes are computed against
    uint8_t *cb;         // first code byte of this chunk
    if (DT == DQ_F16) {
        const float eps_h = rh(1e-7f);
        float s = h_add(h_div(a, MEE ? mp.cmm : (float)R), eps_h);
        if (HIER) {
            float g = row16_hmax(s);
            float unit = h_div(g, 255.0f);
            int q = sat_u16(__builtin_ceilf(h_mul(h_div(s, g), 255.0f)));
            q = min(q, 255);
            d = h_mul((float)q, unit);
            const int CB = PB + 1;
            const int64_t rec = (chunk >> 4) * (16 * CB + 2);
            cb = dst + rec + (chunk & 15) * CB;
            if (active) {
                cb[PB] = (uint8_t)q;
                if ((chunk & 15) == 0) {
                    uint32_t ub = f32_to_f16_bits(unit);
                    dst[rec + 16 * CB] = (uint8_t)ub;
                    dst[rec + 16 * CB + 1] = (uint8_t)(ub >> 8);
                }
            }
        } else {
            d = s;
            cb = dst + chunk * (PB + 2);
            if (active) {
                uint32_t sb = f32_to_f16_bits(s);
                cb[PB] = (uint8_t)sb;
                cb[PB + 1] = (uint8_t)(sb >> 8);
            }
        }
    } else {
        if (HIER) {
            float s = pos_scale(MEE ? a / pos_scale(mp.cmm) + 1e-7f : a / (float)R + 1e-7f);
            float g = pos_scale(row16_max(s));
            uint32_t ustore = f32_to_bf16_bits(pos_scale(g / 255.0f));
            float unit = pos_scale(bf16_bits_to_f32(ustore));
            float ratio = pos_scale(s) / pos_scale(g) * 255.0f;
            if (!__builtin_isfinite(ratio)) ratio = ratio > 0.0f ? 255.0f : 1.0f;
            int q = sat_u16(__builtin_ceilf(ratio));
            q = min(max(q, 1), 255);
            d = pos_scale(pos_scale((float)q * unit));
            const int CB = PB + 1;
            const int64_t rec = (chunk >> 4) * (16 * CB + 2);
            cb = dst + rec + (chunk & 15) * CB;
            if (active) {
                cb[PB] = (uint8_t)q;
                if ((chunk & 15) == 0) {
                    dst[rec + 16 * CB] = (uint8_t)ustore;
                    dst[rec + 16 * CB + 1] = (uint8_t)(ustore >> 8);
                }
            }
        } else {
            uint32_t sb = f32_to_bf16_bits(MEE ? a / mp.cmm + 1e-7f : a / (float)R + 1e-7f);
            d = bf16_bits_to_f32(sb);
            cb = dst + chunk * (PB + 2);
            if (active) {
                cb[PB] = (uint8_t)sb;
                cb[PB + 1] = (uint8_t)(sb >> 8);
            }
        }
    }
    if (!active) return;

    // pass 2: codes
    BytePacker pk(cb);
    for (int i = 0; i < C; i++) {
        float v = IO::load(src, base + i);
        float r = ElemIO<RDT>::load(rnd, base + i);
        int sv;
        if (DT == DQ_F16) {
            float x = h_div(v, d);
            if (MEE) x = mee_inverse_half(x, mp.c, mp.l2b);
            sv = sr_half(x, r);
        } else if (HIER) {
            float x = v / d;
            if (MEE) x = mee_inverse_guarded(x, mp.c, mp.l2b);
            sv = sr_guarded(x, r);
        } else {
            float x = v / d;
            if (MEE) x = mee_inverse_plain(x, mp.c, mp.l2b);
            sv = sr_plain(x, r);
        }
        pk.put(clamp_code(sv, R), nbits);
    }
}

// ---- decompress ----------------------------------------------------------------

template <int DT, bool HIER, bool MEE, bool ADD>
__global__ __launch_bounds__(kGenericBlock) void generic_decompress_kernel(
    const uint8_t *__restrict__ src, void *__restrict__ dst, int64_t nchunks, int nbits, int C,
    MeeParams mp)
{
    typedef ElemIO<DT> IO;
    const int64_t chunk = (int64_t)blockIdx.x * kGenericBlock + threadIdx.x;
    if (chunk >= nchunks) return;
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int64_t base = chunk * C;

    const uint8_t *cb;
    float sc;
    if (HIER) {
        const int CB = PB + 1;
        const int64_t rec = (chunk >> 4) * (16 * CB + 2);
        cb = src + rec + (chunk & 15) * CB;
        uint32_t ub = (uint32_t)src[rec + 16 * CB] | ((uint32_t)src[rec + 16 * CB + 1] << 8);
        if (DT == DQ_F16)
            sc = h_mul((float)cb[PB], f16_bits_to_f32(ub));
        else
            sc = nonneg_scale((float)cb[PB] * nonneg_scale(bf16_bits_to_f32(ub)));
    } else {
        cb = src + chunk * (PB + 2);
        uint32_t sb = (uint32_t)cb[PB] | ((uint32_t)cb[PB + 1] << 8);
        sc = (DT == DQ_F16) ? f16_bits_to_f32(sb) : bf16_bits_to_f32(sb);
    }

    for (int i = 0; i < C; i++) {
        int code = chunk_code(cb, i, nbits);
        float lev = MEE ? f16_bits_to_f32(mp.table[code]) : (float)(code - R);
        float v;
        if (DT == DQ_F16) {
            v = h_mul(lev, sc);
            if (ADD) v = h_add(IO::load(dst, base + i), v);
        } else {
            v = ADD ? __builtin_fmaf(lev, sc, IO::load(dst, base + i)) : lev * sc;
        }
        IO::store(dst, base + i, v);
    }
}

// ---- launchers -----------------------------------------------------------------

template <int DT, bool HIER, bool MEE>
static hipError_t launch_compress_t(const void *src, uint8_t *dst, const void *rnd, int64_t n,
                                    int nbits, int C, const MeeParams &mp, bool rand_bf16, hipStream_t stream)
{
    int64_t nchunks = n / C;
    unsigned grid = (unsigned)((nchunks + kGenericBlock - 1) / kGenericBlock);
    if (DT == DQ_F32 && rand_bf16)
        hipLaunchKernelGGL((generic_compress_kernel<DT, DQ_BF16, HIER, MEE>), dim3(grid), dim3(kGenericBlock), 0,
                           stream, src, dst, rnd, nchunks, nbits, C, mp);
    else
        hipLaunchKernelGGL((generic_compress_kernel<DT, DT, HIER, MEE>), dim3(grid), dim3(kGenericBlock), 0,
                           stream, src, dst, rnd, nchunks, nbits, C, mp);
    return hipGetLastError();
}

template <int DT, bool HIER, bool MEE>
static hipError_t launch_decompress_t(const uint8_t *src, void *dst, int64_t n, int nbits, int C,
                                      const MeeParams &mp, int add, hipStream_t stream)
{
    int64_t nchunks = n / C;
    unsigned grid = (unsigned)((nchunks + kGenericBlock - 1) / kGenericBlock);
    if (add)
        hipLaunchKernelGGL((generic_decompress_kernel<DT, HIER, MEE, true>), dim3(grid),
                           dim3(kGenericBlock), 0, stream, src, dst, nchunks, nbits, C, mp);
    else
        hipLaunchKernelGGL((generic_decompress_kernel<DT, HIER, MEE, false>), dim3(grid),
                           dim3(kGenericBlock), 0, stream, src, dst, nchunks, nbits, C, mp);
    return hipGetLastError();
}

#define DQ_DISPATCH_DT(DT_, ...)                                        \
    switch (DT_) {                                                      \
    case DQ_F16: { constexpr int kDT = DQ_F16; __VA_ARGS__; } break;    \
    case DQ_BF16: { constexpr int kDT = DQ_BF16; __VA_ARGS__; } break;  \
    default: { constexpr int kDT = DQ_F32; __VA_ARGS__; } break;        \
    }

hipError_t launch_generic_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n,
                                   int nbits, int C, int dtype, int strategy, const MeeParams &mp,
                                   hipStream_t stream)
{
    hipError_t e = hipSuccess;
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
    DQ_DISPATCH_DT(dtype, {
        switch (strategy) {
        case 0: e = launch_compress_t<kDT, false, false>(src, dst, rnd, n, nbits, C, mp, rb16, stream); break;
        case 1: e = launch_compress_t<kDT, false, true>(src, dst, rnd, n, nbits, C, mp, rb16, stream); break;
        case 2: e = launch_compress_t<kDT, true, false>(src, dst, rnd, n, nbits, C, mp, rb16, stream); break;
        default: e = launch_compress_t<kDT, true, true>(src, dst, rnd, n, nbits, C, mp, rb16, stream); break;
        }
    });
    return e;
}

hipError_t launch_generic_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int C,
                                     int dtype, int strategy, const MeeParams &mp, int add,
                                     hipStream_t stream)
{
    hipError_t e = hipSuccess;
    DQ_DISPATCH_DT(dtype, {
        switch (strategy) {
        case 0: e = launch_decompress_t<kDT, false, false>(src, dst, n, nbits, C, mp, add, stream); break;
        case 1: e = launch_decompress_t<kDT, false, true>(src, dst, n, nbits, C, mp, add, stream); break;
        case 2: e = launch_decompress_t<kDT, true, false>(src, dst, n, nbits, C, mp, add, stream); break;
        default: e = launch_decompress_t<kDT, true, true>(src, dst, n, nbits, C, mp, add, stream); break;
        }
    });
    return e;
}

} // namespace dq
