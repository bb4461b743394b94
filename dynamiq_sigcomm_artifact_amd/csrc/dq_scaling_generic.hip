// Generic scaling-quantisation kernels: any element type (fp16 / bf16 / fp32),
// any strategy (0 AEE, 1 MEE, 2/3 hierarchical), any power-of-two chunk size
// up to 32 and any code width 2..8.  One thread owns one chunk and walks it
// serially; the 16 chunks of a hierarchical superchunk sit in one 16-lane DPP
// row, so the superchunk maximum is a row reduction without LDS or barriers.
//
// These kernels are the catch-all behind the C ABI: they also serve buffers
// whose alignment rules out the vectorised chunk-16 kernels.  For chunks of 8
// and 32 elements in 16-byte aligned buffers the chunk size is a template
// argument (CT): the thread's chunk then comes in through 16-byte loads and
// stays in registers for both passes, and decoded chunks leave through a
// swizzled per-wave LDS tile as lane-contiguous 16-byte stores.  Numerics follow
// csrc/cuda_hadamard.cu:768-861,941-1234 (flat) and
// csrc/cuda_hierarchical_mee.cu:698-1294 (hierarchical) of the reference.
#include <type_traits>

#include "dq_launch.h"
#include "dq_tile16.cuh"

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

// ---- a chunk of a compile-time size in registers ---------------------------------

template <int DT> __device__ __forceinline__ float elem_from_bits(uint32_t b)
{
    return DT == DQ_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}
template <int DT> __device__ __forceinline__ uint32_t elem_to_bits(float v)
{
    return DT == DQ_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
}

// 16-byte pieces of a chunk of CT elements
template <int DT, int CT> struct ChunkShape {
    static constexpr int kBytes = CT * (int)sizeof(typename ElemIO<DT>::storage);
    static constexpr int kSlots = kBytes / 16;
};

// the chunk starts on a 16-byte boundary
template <int DT, int CT>
__device__ __forceinline__ void load_chunk(const void *p, int64_t base, float (&v)[CT])
{
    constexpr int S = ChunkShape<DT, CT>::kSlots;
    const uint4 *q = reinterpret_cast<const uint4 *>(static_cast<const char *>(p) + base * (ChunkShape<DT, CT>::kBytes / CT));
#pragma unroll
    for (int j = 0; j < S; j++) {
        const uint4 w = q[j];
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (DT == DQ_F32) {
                v[4 * j + k] = __uint_as_float(ww[k]);
            } else {
                v[8 * j + 2 * k] = elem_from_bits<DT>(ww[k] & 0xffffu);
                v[8 * j + 2 * k + 1] = elem_from_bits<DT>(ww[k] >> 16);
            }
        }
    }
}

// The same chunk kept as loaded (two 16-bit elements per register) and widened at each use: half the registers of
// the float array for fp16 / bf16, which decides how many waves fit on a SIMD when a lane holds 32 elements and
// their 32 random values
template <int DT, int CT> struct PackedChunk {
    static constexpr int kWords = ChunkShape<DT, CT>::kBytes / 4;
    uint32_t w[kWords];
    __device__ __forceinline__ void load(const void *p, int64_t base)
    {
        const uint4 *q = reinterpret_cast<const uint4 *>(static_cast<const char *>(p) + base * (ChunkShape<DT, CT>::kBytes / CT));
#pragma unroll
        for (int j = 0; j < kWords / 4; j++) {
            const uint4 v = q[j];
            w[4 * j] = v.x; w[4 * j + 1] = v.y; w[4 * j + 2] = v.z; w[4 * j + 3] = v.w;
        }
    }
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int j = 0; j < kWords; j++) w[j] = 0u;
    }
    __device__ __forceinline__ float get(int i) const
    {
        if (DT == DQ_F32) return __uint_as_float(w[i]);
        return elem_from_bits<DT>((w[i >> 1] >> (16 * (i & 1))) & 0xffffu);
    }
    // bfloat16 / binary32 only.  The binary32 bit pattern of max |element| in integer order (a NaN sorts above infinity)
    __device__ __forceinline__ uint32_t absmax_bits() const
    {
        if (DT == DQ_F32) {
            uint32_t m = w[0] & 0x7fffffffu;
#pragma unroll
            for (int k = 1; k < kWords; k++) m = max(m, w[k] & 0x7fffffffu);
            return m;
        }
        uint32_t m = w[0] & 0x7fff7fffu;
#pragma unroll
        for (int k = 1; k < kWords; k++) m = pk_max_u16(m, w[k] & 0x7fff7fffu);
        return max(m << 16, m & 0xffff0000u);
    }
    // every element in [+0, 1]
    __device__ __forceinline__ bool unit_interval() const
    {
        uint32_t m = w[0];
#pragma unroll
        for (int k = 1; k < kWords; k++) m = DT == DQ_F32 ? max(m, w[k]) : pk_max_u16(m, w[k]);
        return DT == DQ_F32 ? m <= 0x3f800000u : max(m & 0xffffu, m >> 16) <= 0x3f80u;
    }
};

// elements [OFF, OFF + 16) of a chunk as the 16-element operand of estimate_codes(); positions at and beyond the
// chunk's end read as `pad`
template <class CHUNK, int OFF, int CT> struct Sixteen {
    const CHUNK &c;
    float pad;
    __device__ __forceinline__ float get(int i) const { return OFF + i < CT ? c.get(OFF + i < CT ? OFF + i : 0) : pad; }
};

struct MeeReciprocals {
    double inv_c, inv_l2b;
};

// A wave's chunks, S 16-byte pieces per lane, leave as lane-contiguous pieces (see swz()).  tile: 64 S slots of
// LDS owned by the wave; dst: where the wave's first piece goes; valid: pieces inside the destination.
template <int S>
__device__ __forceinline__ void store_wave_slots(uint4 *tile, const uint4 (&slot)[S], uint4 *dst, int lane, int valid)
{
#pragma unroll
    for (int j = 0; j < S; j++) tile[swz(S * lane + j)] = slot[j];
    wave_lds_sync();
#pragma unroll
    for (int k = 0; k < S; k++) {
        const int s = 64 * k + lane;
        if (s < valid) stream_store(dst + s, tile[swz(s)]);
    }
}

// LDS bytes for the packed run of a wave's 64 chunks of CT elements at up to 8 bits (flat: 64 (CT + 2),
// hierarchical: 4 (16 (CT + 1) + 2)), its 16-byte phase and the rounding up to whole 16-byte pieces
template <int CT> struct WindowBytes { static constexpr int value = CT ? 64 * CT + 160 : 16; };

// ---- compress ----------------------------------------------------------------

// CT: the chunk size when it is 8 or 32 and src and rnd are 16-byte aligned, else 0.  NB: the code width when it is
// 2, 4 or 8 and CT is not 0 (the packing loop then unrolls into constant shifts), else 0
template <int DT, int RDT, bool HIER, bool MEE, int CT, int NB>
__global__ __launch_bounds__(kGenericBlock) void generic_compress_kernel(
    const void *__restrict__ src, uint8_t *__restrict__ dst, const void *__restrict__ rnd,
    int64_t nchunks, int nbits_rt, int Crt, MeeParams mp)
{
    const int nbits = NB ? NB : nbits_rt;
    typedef ElemIO<DT> IO;
    constexpr int kUnroll = CT ? CT : 1;
    const int C = CT ? CT : Crt;
    const int64_t chunk = (int64_t)blockIdx.x * kGenericBlock + threadIdx.x;
    const bool active = chunk < nchunks; // hierarchical: whole 16-lane rows are active or not
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int64_t base = chunk * C;

    PackedChunk<DT, (CT ? CT : 8)> ev;
    PackedChunk<RDT, (CT ? CT : 8)> rv;
    if (CT) {
        if (active) {
            ev.load(src, base);
            rv.load(rnd, base);
        } else {
            ev.zero();
            rv.zero();
        }
    }

    // pass 1: chunk absmax
    float a = 0.0f;
    if (active) {
        a = __builtin_fabsf(CT ? ev.get(0) : IO::load(src, base));
#pragma unroll kUnroll
        for (int i = 1; i < C; i++) {
            float v = __builtin_fabsf(CT ? ev.get(CT ? i : 0) : IO::load(src, base + i));
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

    // pass 2: codes.  v / d is the correctly rounded quotient either way: with the chunk in registers and d an
    // ordinary number it is the product with 1/d in double (see div_exact), otherwise the IEEE division
    BytePacker pk(cb);
    const auto codes = [&](auto fast) {
        const double yd = decltype(fast)::value ? recip_f64(d) : 0.0;
#pragma unroll kUnroll
        for (int i = 0; i < C; i++) {
            float v = CT ? ev.get(CT ? i : 0) : IO::load(src, base + i);
            float r = CT ? rv.get(CT ? i : 0) : ElemIO<RDT>::load(rnd, base + i);
            float x = decltype(fast)::value ? (DT == DQ_F16 ? div_by(v, yd) : div_exact(v, d, yd)) : v / d;
            int sv;
            if (DT == DQ_F16) {
                x = rh(x);
                if (MEE) x = mee_inverse_half(x, mp.c, mp.l2b);
                sv = sr_half(x, r);
            } else if (HIER) {
                if (MEE) x = mee_inverse_guarded(x, mp.c, mp.l2b);
                sv = sr_guarded(x, r);
            } else {
                if (MEE) x = mee_inverse_plain(x, mp.c, mp.l2b);
                sv = sr_plain(x, r);
            }
            pk.put(clamp_code(sv, R), nbits);
        }
    };
    const uint32_t db = __float_as_uint(d);
    const bool ordinary = db >= 0x0d800000u && db <= 0x71800000u; // a normal number in [2^-100, 2^100]
    if constexpr (CT != 0 && NB != 0 && DT != DQ_F16) {
        // binary32 arithmetic: when every lane of the wave has an ordinary scale, finite elements (so |v| <= (R + 1) d)
        // and random values in [0, 1], the codes come from the estimate with its exact redo near the rounding
        // boundaries, sixteen elements at a time (dq_tile16.cuh)
        const bool lane_ok = ordinary && ev.absmax_bits() <= 0x71800000u && rv.unit_interval();
        if (__builtin_amdgcn_ballot_w64(!lane_ok) == 0) {
            MeeReciprocals rc;
            rc.inv_c = MEE ? recip_f64(mp.c) : 0.0;
            rc.inv_l2b = MEE ? recip_f64(mp.l2b) : 0.0;
            constexpr int kGroup = CT < 16 ? CT : 16; // elements per call
            constexpr int kGroupBytes = kGroup * NB / 8;
            auto group = [&](auto off) {
                constexpr int OFF = decltype(off)::value;
                uint32_t w[Rec<NB>::WORDS];
#pragma unroll
                for (int k = 0; k < Rec<NB>::WORDS; k++) w[k] = 0;
                // padding: v = 0 with r = 1/2 is never in doubt
                const Sixteen<decltype(ev), OFF, CT> v16{ev, 0.0f};
                const Sixteen<decltype(rv), OFF, CT> r16{rv, 0.5f};
                estimate_codes<NB, MEE>(v16, r16, d, rc, w);
#pragma unroll
                for (int k = 0; k < kGroupBytes; k++) cb[OFF * NB / 8 + k] = (uint8_t)(w[k >> 2] >> (8 * (k & 3)));
            };
            group(std::integral_constant<int, 0>{});
            if constexpr (CT > 16) group(std::integral_constant<int, 16>{});
            return;
        }
    }
    if (CT && ordinary)
        codes(std::true_type{});
    else
        codes(std::false_type{});
}

// ---- decompress ----------------------------------------------------------------

// CT: the chunk size when it is 8 or 32 and dst is 16-byte aligned, else 0; NB as in generic_compress_kernel
template <int DT, bool HIER, bool MEE, bool ADD, int CT, int NB>
__global__ __launch_bounds__(kGenericBlock) void generic_decompress_kernel(
    const uint8_t *__restrict__ src, void *__restrict__ dst, int64_t nchunks, int nbits_rt, int Crt,
    MeeParams mp)
{
    const int nbits = NB ? NB : nbits_rt;
    typedef ElemIO<DT> IO;
    constexpr int CR = CT ? CT : 1;
    constexpr int S = ChunkShape<DT, CR>::kSlots;
    __shared__ __attribute__((aligned(16))) uint4 tiles[(CT && S > 1) ? kGenericBlock / 64 : 1][(CT && S > 1) ? 64 * S : 1];
    const int C = CT ? CT : Crt;
    const int64_t chunk = (int64_t)blockIdx.x * kGenericBlock + threadIdx.x;
    const bool active = chunk < nchunks;
    if (!CT && !active) return;
    const int lane = threadIdx.x & 63;
    const int64_t wave_first = chunk - lane;
    if (CT && wave_first >= nchunks) return; // the whole wave
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int64_t base = chunk * C;

    // CT: the wave's packed run comes in as 16-byte pieces into an LDS window (byte k of the run at win[mis + k])
    __shared__ __attribute__((aligned(16))) uint8_t wins[CT ? kGenericBlock / 64 : 1][WindowBytes<CT>::value];
    const int64_t run_start = !CT ? 0 : HIER ? (wave_first >> 4) * (16 * (PB + 1) + 2) : wave_first * (PB + 2);
    const uint8_t *ibase;
    if constexpr (CT != 0) {
        const uint8_t *g = src + run_start;
        const int mis = (int)(reinterpret_cast<uintptr_t>(g) & 15);
        const int nact = (int)min((int64_t)64, nchunks - wave_first);
        const int total = HIER ? (nact >> 4) * (16 * (PB + 1) + 2) : nact * (PB + 2);
        const int nvec = (mis + total + 15) >> 4;
        const u32x4 *ga = reinterpret_cast<const u32x4 *>(g - mis);
        u32x4 *wv = reinterpret_cast<u32x4 *>(wins[threadIdx.x >> 6]);
        for (int v = lane; v < nvec; v += 64) wv[v] = ga[v];
        wave_lds_sync();
        ibase = wins[threadIdx.x >> 6] + mis;
    } else {
        ibase = src;
    }

    float out[CR];
#pragma unroll
    for (int i = 0; i < CR; i++) out[i] = 0.0f;
    if (active) {
        const uint8_t *cb;
        float sc;
        if (HIER) {
            const int CB = PB + 1;
            const int64_t rec = (chunk >> 4) * (16 * CB + 2) - run_start;
            cb = ibase + rec + (chunk & 15) * CB;
            uint32_t ub = (uint32_t)ibase[rec + 16 * CB] | ((uint32_t)ibase[rec + 16 * CB + 1] << 8);
            if (DT == DQ_F16)
                sc = h_mul((float)cb[PB], f16_bits_to_f32(ub));
            else
                sc = nonneg_scale((float)cb[PB] * nonneg_scale(bf16_bits_to_f32(ub)));
        } else {
            cb = ibase + (chunk * (PB + 2) - run_start);
            uint32_t sb = (uint32_t)cb[PB] | ((uint32_t)cb[PB + 1] << 8);
            sc = (DT == DQ_F16) ? f16_bits_to_f32(sb) : bf16_bits_to_f32(sb);
        }
        float old[CR];
        if (CT && ADD) load_chunk<DT, CR>(dst, base, old);

#pragma unroll CR
        for (int i = 0; i < C; i++) {
            int code = chunk_code(cb, i, nbits);
            float lev = MEE ? f16_bits_to_f32(mp.table[code]) : (float)(code - R);
            float v;
            if (DT == DQ_F16) {
                v = h_mul(lev, sc);
                if (ADD) v = h_add(CT ? old[CT ? i : 0] : IO::load(dst, base + i), v);
            } else {
                v = ADD ? __builtin_fmaf(lev, sc, CT ? old[CT ? i : 0] : IO::load(dst, base + i)) : lev * sc;
            }
            if (CT)
                out[CT ? i : 0] = v;
            else
                IO::store(dst, base + i, v);
        }
    }
    if constexpr (CT != 0) {
        uint4 slot[S];
#pragma unroll
        for (int j = 0; j < S; j++) {
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if (DT == DQ_F32)
                    w[k] = __float_as_uint(out[4 * j + k]);
                else
                    w[k] = elem_to_bits<DT>(out[8 * j + 2 * k]) | (elem_to_bits<DT>(out[8 * j + 2 * k + 1]) << 16);
            }
            slot[j] = make_uint4(w[0], w[1], w[2], w[3]);
        }
        uint4 *wave_dst = reinterpret_cast<uint4 *>(static_cast<char *>(dst) + wave_first * ChunkShape<DT, CR>::kBytes);
        if constexpr (S == 1) {
            if (active) stream_store(wave_dst + lane, slot[0]);
        } else {
            const int valid = (int)min((int64_t)64, nchunks - wave_first) * S;
            store_wave_slots<S>(tiles[threadIdx.x >> 6], slot, wave_dst, lane, valid);
        }
    }
}

// ---- launchers -----------------------------------------------------------------

template <int DT, bool HIER, bool MEE>
static hipError_t launch_compress_t(const void *src, uint8_t *dst, const void *rnd, int64_t n,
                                    int nbits, int C, const MeeParams &mp, bool rand_bf16, hipStream_t stream)
{
    int64_t nchunks = n / C;
    unsigned grid = (unsigned)((nchunks + kGenericBlock - 1) / kGenericBlock);
    const int ct = (aligned16(src) && aligned16(rnd) && (C == 8 || C == 32)) ? C : 0;
#define DQ_GENERIC_COMPRESS_NB(RDT, CT, NB)                                                                                 \
    hipLaunchKernelGGL((generic_compress_kernel<DT, RDT, HIER, MEE, CT, NB>), dim3(grid), dim3(kGenericBlock), 0, stream, src, \
                       dst, rnd, nchunks, nbits, C, mp)
#define DQ_GENERIC_COMPRESS(RDT, CT)                                  \
    do {                                                              \
        if (CT != 0 && nbits == 2) DQ_GENERIC_COMPRESS_NB(RDT, CT, (CT ? 2 : 0));      \
        else if (CT != 0 && nbits == 4) DQ_GENERIC_COMPRESS_NB(RDT, CT, (CT ? 4 : 0)); \
        else if (CT != 0 && nbits == 8) DQ_GENERIC_COMPRESS_NB(RDT, CT, (CT ? 8 : 0)); \
        else DQ_GENERIC_COMPRESS_NB(RDT, CT, 0);                      \
    } while (0)
    if (DT == DQ_F32 && rand_bf16) {
        if (ct == 32) DQ_GENERIC_COMPRESS(DQ_BF16, 32);
        else if (ct == 8) DQ_GENERIC_COMPRESS(DQ_BF16, 8);
        else DQ_GENERIC_COMPRESS(DQ_BF16, 0);
    } else {
        if (ct == 32) DQ_GENERIC_COMPRESS(DT, 32);
        else if (ct == 8) DQ_GENERIC_COMPRESS(DT, 8);
        else DQ_GENERIC_COMPRESS(DT, 0);
    }
#undef DQ_GENERIC_COMPRESS
#undef DQ_GENERIC_COMPRESS_NB
    return hipGetLastError();
}

template <int DT, bool HIER, bool MEE>
static hipError_t launch_decompress_t(const uint8_t *src, void *dst, int64_t n, int nbits, int C,
                                      const MeeParams &mp, int add, hipStream_t stream)
{
    int64_t nchunks = n / C;
    unsigned grid = (unsigned)((nchunks + kGenericBlock - 1) / kGenericBlock);
    const int ct = (aligned16(dst) && (C == 8 || C == 32)) ? C : 0;
#define DQ_GENERIC_DECOMPRESS_NB(ADD, CT, NB)                                                                                 \
    hipLaunchKernelGGL((generic_decompress_kernel<DT, HIER, MEE, ADD, CT, NB>), dim3(grid), dim3(kGenericBlock), 0, stream, src, \
                       dst, nchunks, nbits, C, mp)
#define DQ_GENERIC_DECOMPRESS(ADD, CT)                                \
    do {                                                              \
        if (CT != 0 && nbits == 2) DQ_GENERIC_DECOMPRESS_NB(ADD, CT, (CT ? 2 : 0));      \
        else if (CT != 0 && nbits == 4) DQ_GENERIC_DECOMPRESS_NB(ADD, CT, (CT ? 4 : 0)); \
        else if (CT != 0 && nbits == 8) DQ_GENERIC_DECOMPRESS_NB(ADD, CT, (CT ? 8 : 0)); \
        else DQ_GENERIC_DECOMPRESS_NB(ADD, CT, 0);                    \
    } while (0)
    if (add) {
        if (ct == 32) DQ_GENERIC_DECOMPRESS(true, 32);
        else if (ct == 8) DQ_GENERIC_DECOMPRESS(true, 8);
        else DQ_GENERIC_DECOMPRESS(true, 0);
    } else {
        if (ct == 32) DQ_GENERIC_DECOMPRESS(false, 32);
        else if (ct == 8) DQ_GENERIC_DECOMPRESS(false, 8);
        else DQ_GENERIC_DECOMPRESS(false, 0);
    }
#undef DQ_GENERIC_DECOMPRESS
#undef DQ_GENERIC_DECOMPRESS_NB
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
