// Vectorised chunk-16 kernels for the shapes outside the production kernel of
// dq_scaling_hier16.hip: binary16 elements (every strategy; all arithmetic is the
// reference's op-by-op half arithmetic, i.e. an fp32 operation followed by one rounding to
// binary16) and the flat strategies 0 / 1 for bf16 and fp32 elements (PB code bytes + a
// 2-byte scale per chunk, no superchunk level).
//
// Same decomposition as the production kernel: one lane = one chunk (128-bit loads), one
// single-wave workgroup = 64 chunks = one contiguous run of the packed stream, assembled in
// (or pulled through) an LDS window whose offset equals the global address modulo 16;
// decoded elements are transposed through a swizzled LDS tile so that every store
// instruction covers 1 KiB.  Divisions by the chunk's scale use the exact double-reciprocal
// product when every scale of the wave is an ordinary number, IEEE division otherwise.
//
// Numerics: csrc/cuda_hadamard.cu:768-861,941-1234 (flat), csrc/cuda_hierarchical_mee.cu:698-930
// (binary16 hierarchical) of the reference.
#include "dq_launch.h"
#include "dq_tile16.cuh"

namespace dq {

namespace {

constexpr int kChunksPerWave = 64;

template <int NBITS, bool HIER> struct Geo {
    static constexpr int PB = 2 * NBITS;
    static constexpr int CB = HIER ? PB + 1 : PB + 2; // bytes of one chunk in the stream
    static constexpr int REC = 16 * CB + 2;           // hierarchical record
    static constexpr int FULL = HIER ? 4 * REC : kChunksPerWave * CB;
    static constexpr int WIN = ((FULL + 15 + 15) / 16) * 16;
    __device__ static __forceinline__ int bytes(int chunks) { return HIER ? (chunks >> 4) * REC : chunks * CB; }
    __device__ static __forceinline__ int offset(int chunk) { return HIER ? (chunk >> 4) * REC + (chunk & 15) * CB : chunk * CB; }
    __host__ __device__ static __forceinline__ int64_t stream_offset(int64_t chunk) { return HIER ? (chunk >> 4) * REC : chunk * CB; }
};

// maximum over a 16-lane row with the half-precision max rule (a NaN operand is dropped)
__device__ __forceinline__ float row16_hmax(float v)
{
    v = h_max(v, dpp_f32<0xB1>(v));
    v = h_max(v, dpp_f32<0x4E>(v));
    v = h_max(v, dpp_f32<0x141>(v));
    v = h_max(v, dpp_f32<0x140>(v));
    return v;
}

// a scale the double-reciprocal division is proven for: normal, 2^-100 <= d <= 2^100
__device__ __forceinline__ bool ordinary_scale(float d)
{
    const uint32_t b = __float_as_uint(d);
    return b >= 0x0d800000u && b <= 0x71800000u;
}

// a / b correctly rounded to binary32 for binary16-valued a and b (b an ordinary scale or a lattice constant), given
// y = RN32(1 / b): q0 = RN(a y) is within an ulp of the quotient, the remainder a - q0 b then fits binary32 and the fused
// operation computes it exactly, and RN(q0 + rem y) is the correctly rounded quotient (Markstein's theorem; its one
// exception, a divisor whose significand is all ones, needs 24 significant bits).  y is the double reciprocal rounded
// to binary32: 1 / b with an 11-bit b stays 2^-36 (relative) clear of every binary32 rounding boundary unless it is
// representable, so rounding the double (within 2^-51) rounds the reciprocal itself.  Quotients and remainders stay
// normal numbers for these operands; the sign of a zero quotient is not kept (no code depends on it).
__device__ __forceinline__ float div_half_operands(float a, float b, float y)
{
    const float q0 = a * y;
    const float rem = __builtin_fmaf(-q0, b, a);
    return __builtin_fmaf(rem, y, q0);
}

// The codes of a binary16 chunk with the half-precision operations done by the machine's own binary16 instructions
// (IEEE, round to nearest even: the same value as the binary32 operation followed by one rounding that the op-by-op
// chain below spells out, without the two conversions around every operation).  For a wave whose scales are all
// ordinary, whose elements hold no NaN and whose random values lie in [0, 1]: every quotient is then finite and below
// 2 R in magnitude, so none of the saturating conversions of the reference's chain can fire, floor, the two
// differences, ceil and their sum are small integers or exact, and the clamp can be taken on the binary16 sum.
// A zero quotient needs no case of its own under MEE: the lattice coordinate of 0 is log2(0 / c + 1) / l2b = +0.
template <int NBITS, bool MEE, class RR, class ARG>
__device__ __forceinline__ void half_codes_native(const Raw16<DQ_F16> &v, const RR &r, float d, double yd, const ARG &mp,
                                                  uint32_t (&w)[Rec<NBITS>::WORDS])
{
    constexpr int R = Rec<NBITS>::R;
    const float y = (float)yd;
    const float yc = MEE ? (float)mp.inv_c : 0.0f, yl = MEE ? (float)mp.inv_l2b : 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        _Float16 x = (_Float16)div_half_operands(v.get(i), d, y);
        if (MEE) {
            const _Float16 arg = (_Float16)div_half_operands((float)__builtin_fabsf16(x), mp.c, yc) + (_Float16)1.0f;
            const _Float16 lg = (_Float16)log2_det_ge1((float)arg);
            const _Float16 lat = (_Float16)div_half_operands((float)lg, mp.l2b, yl);
            x = x < (_Float16)0.0f ? -lat : lat;
        }
        const _Float16 fl = __builtin_floorf16(x);
        const _Float16 t = (x - fl) - (_Float16)r.get(i);
        _Float16 c = fl + __builtin_ceilf16(t);
        c = c < (_Float16)(-R) ? (_Float16)(-R) : c;
        c = c > (_Float16)R ? (_Float16)R : c;
        words_put<NBITS>(w, i, (uint32_t)(int)(c + (_Float16)R));
    }
}

template <int DT, int RDT, int NBITS, bool HIER, bool MEE>
__global__ __launch_bounds__(64) void tile16_compress_kernel(const void *__restrict__ src, uint8_t *__restrict__ dst,
                                                            const void *__restrict__ rnd, int64_t nchunks, int vec,
                                                            RandKey key, MeeArg<NBITS, MEE> mp)
{
    typedef Geo<NBITS, HIER> G;
    constexpr int R = Rec<NBITS>::R;
    __shared__ __attribute__((aligned(16))) uint8_t win_out[G::WIN];

    const int lane = threadIdx.x;
    const int64_t c0 = (int64_t)blockIdx.x * kChunksPerWave;
    if (c0 >= nchunks) return;
    const int chunks_here = (int)min((int64_t)kChunksPerWave, nchunks - c0);
    const bool active = lane < chunks_here;
    const int total = G::bytes(chunks_here);

    Raw16<DT> v;
    Raw16<RDT> r;
    if (active) {
        v.load(src, (c0 + lane) * 16, vec & 1);
        if constexpr (RDT == DQ_PHILOX)
            r.generate(key, c0 + lane);
        else
            r.load(rnd, (c0 + lane) * 16, vec & 2);
    } else {
        v.zero();
        r.zero();
    }

    float a;
    bool half_nan = false; // binary16 elements: the wave holds a NaN
    if constexpr (DT == DQ_F16) {
        // the largest magnitude as an integer maximum of the bit patterns; a NaN sorts above infinity, and only then does
        // the reference's maximum (which passes over a NaN operand) need its own comparisons
        const uint32_t amax = v.absmax_half_bits();
        half_nan = __builtin_amdgcn_ballot_w64(amax > 0x7c00u) != 0;
        a = f16_bits_to_f32(amax);
        if (half_nan) {
            a = __builtin_fabsf(v.get(0));
#pragma unroll
            for (int i = 1; i < 16; i++) a = h_max(a, __builtin_fabsf(v.get(i)));
        }
    } else {
        a = __builtin_fabsf(v.get(0));
#pragma unroll
        for (int i = 1; i < 16; i++) a = __builtin_fmaxf(a, __builtin_fabsf(v.get(i)));
    }

    float d;             // the scale the codes are computed against
    uint32_t tail_bits;  // what follows the code bytes of this chunk: q (hier) or the 2-byte scale (flat)
    uint32_t unit_bits = 0;
    if (DT == DQ_F16) {
        const float eps_h = rh(1e-7f);
        const float s = h_add(h_div(a, MEE ? mp.cmm : (float)R), eps_h);
        if (HIER) {
            const float g = row16_hmax(s);
            const float unit = h_div(g, 255.0f);
            int q = sat_u16(__builtin_ceilf(h_mul(h_div(s, g), 255.0f)));
            q = min(q, 255);
            d = h_mul((float)q, unit);
            tail_bits = (uint32_t)q;
            unit_bits = f32_to_f16_bits(unit);
        } else {
            d = s;
            tail_bits = f32_to_f16_bits(s);
        }
    } else {
        // flat, fp32 arithmetic: the codes are computed against the bf16-rounded scale
        tail_bits = f32_to_bf16_bits(MEE ? a / mp.cmm + 1e-7f : a / (float)R + 1e-7f);
        d = bf16_bits_to_f32(tail_bits);
    }

    const bool fast = __builtin_amdgcn_ballot_w64(!ordinary_scale(d)) == 0;
    uint32_t w[Rec<NBITS>::WORDS];
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = 0;
    // binary32 arithmetic, ordinary scales (so every element is finite and at most (R + 1) d) and random values in
    // [0, 1]: the codes come from the estimate with its exact redo near the rounding boundaries
    bool estimated = false;
    if constexpr (DT != DQ_F16) {
        // the largest-magnitude search above passes over NaN elements (as the reference's does), so the scale says
        // nothing about them: v * 0 summed over the chunk is NaN exactly when one of them is not finite
        float finite = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) finite = __builtin_fmaf(v.get(i), 0.0f, finite);
        estimated = fast && __builtin_amdgcn_ballot_w64(!r.unit_interval() || finite != finite) == 0;
        if (estimated) estimate_codes<NBITS, MEE>(v, r, d, mp, w);
    }
    const double yd = fast && !estimated ? recip_f64(d) : 0.0;
    if constexpr (DT == DQ_F16) {
        // (estimated doubles as "the codes are done")
        estimated = fast && !half_nan && __builtin_amdgcn_ballot_w64(!r.unit_interval()) == 0;
        if (estimated) half_codes_native<NBITS, MEE>(v, r, d, yd, mp, w);
    }
    // the element-wise chain, compiled once per kind of division: with the choice made per element the compiler
    // computes both quotients and selects
    auto chain = [&](auto by_reciprocal) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float e = v.get(i);
        // (a binary16 element divided by a binary16 scale is never subnormal in binary32)
        float x = decltype(by_reciprocal)::value ? (DT == DQ_F16 ? div_by(e, yd) : div_exact(e, d, yd)) : e / d;
        int sv;
        if (DT == DQ_F16) {
            x = rh(x);
            if (MEE) {
                // mee_inverse_half with the divisions by the table constants done exactly
                const float ax = __builtin_fabsf(x);
                if (!(ax > 0.0f)) {
                    x = 0.0f;
                } else {
                    const float arg = h_add(rh(div_by(ax, mp.inv_c)), 1.0f);
                    const float lat = rh(div_by(rh(log2_det(arg)), mp.inv_l2b));
                    x = x < 0.0f ? -lat : lat;
                }
            }
            sv = sr_half(x, r.get(i));
        } else {
            if (MEE) {
                const float ax = __builtin_fabsf(x);
                if (!(ax > 0.0f)) {
                    x = 0.0f;
                } else {
                    const float lat = div_by(log2_det(div_by(ax, mp.inv_c) + 1.0f), mp.inv_l2b);
                    x = x < 0.0f ? -lat : lat;
                }
            }
            sv = sr_plain(x, r.get(i));
        }
        words_put<NBITS>(w, i, (uint32_t)clamp_code(sv, R));
    }
    };
    if (!estimated) {
        if (fast)
            chain(std::true_type{});
        else
            chain(std::false_type{});
    }

    uint8_t *gout = dst + G::stream_offset(c0);
    const int mis = (int)(reinterpret_cast<uintptr_t>(gout) & 15);
    if (active) {
        uint8_t *p = win_out + mis + G::offset(lane);
        chunk_write<NBITS>(p, w, tail_bits); // PB code bytes + the low byte of tail_bits
        if (!HIER) p[G::PB + 1] = (uint8_t)(tail_bits >> 8);
        if (HIER && (lane & 15) == 0) {
            p[16 * G::CB] = (uint8_t)unit_bits;
            p[16 * G::CB + 1] = (uint8_t)(unit_bits >> 8);
        }
    }
    wave_lds_sync();
    window_flush(win_out, gout, mis, total, lane);
}

template <int DT, int NBITS, bool HIER, bool MEE, bool ADD>
__global__ __launch_bounds__(64) void tile16_decompress_kernel(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                              int64_t nchunks, int vec, MeeArg<NBITS, MEE> mp)
{
    typedef Geo<NBITS, HIER> G;
    constexpr int R = Rec<NBITS>::R;
    constexpr int S = Raw16<DT>::kSlots;
    __shared__ __attribute__((aligned(16))) uint8_t win_in[G::WIN];
    __shared__ __attribute__((aligned(16))) uint4 tile_out[64 * S];
    __shared__ float table[MEE ? (1 << NBITS) : 1];

    const int lane = threadIdx.x;
    const int64_t c0 = (int64_t)blockIdx.x * kChunksPerWave;
    if (c0 >= nchunks) return;
    const int chunks_here = (int)min((int64_t)kChunksPerWave, nchunks - c0);
    const bool active = lane < chunks_here;
    const int total = G::bytes(chunks_here);
    const int64_t e0 = c0 * 16;
    const uint8_t *gin = src + G::stream_offset(c0);

    const WinRegs wr = window_fetch(gin, total, lane);
    Raw16<DT> acc;
    if (ADD && active) acc.load(dst, e0 + lane * 16, vec);
    TableRegs<NBITS> tr;
    if (MEE) tr = table_fetch<NBITS>(mp, lane);
    const int mis_in = window_commit(win_in, wr, gin, total, lane);
    if (MEE) table_commit<NBITS>(table, tr, lane);
    wave_lds_sync();

    Raw16<DT> out;
    if (active) {
        const uint8_t *p = win_in + mis_in + G::offset(lane);
        uint32_t cw[Rec<NBITS>::WORDS], tail;
        chunk_read<NBITS>(p, cw, tail);
        float sc;
        if (HIER) {
            const uint8_t *rec_end = win_in + mis_in + (lane >> 4) * G::REC + 16 * G::CB;
            const uint32_t ub = (uint32_t)rec_end[0] | ((uint32_t)rec_end[1] << 8);
            sc = h_mul((float)tail, f16_bits_to_f32(ub)); // HIER is instantiated for binary16 only
        } else {
            const uint32_t sb = tail | ((uint32_t)p[G::PB + 1] << 8);
            sc = (DT == DQ_F16) ? f16_bits_to_f32(sb) : bf16_bits_to_f32(sb);
        }
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t code = words_get<NBITS>(cw, i);
            const float lev = MEE ? table[code] : (float)((int)code - R);
            if (DT == DQ_F16) {
                const float val = h_mul(lev, sc);
                t[i] = ADD ? h_add(acc.get(i), val) : val;
            } else {
                t[i] = ADD ? __builtin_fmaf(lev, sc, acc.get(i)) : lev * sc;
            }
        }
        out.set(t);
    } else {
        out.zero();
    }
    if (vec) {
        if (active) {
#pragma unroll
            for (int k = 0; k < S; k++) tile_out[swz(S * lane + k)] = out.slot(k);
        }
        wave_lds_sync();
        const int nslots = chunks_here * S;
        uint4 *g = reinterpret_cast<uint4 *>(static_cast<char *>(dst) + e0 * (DT == DQ_F32 ? 4 : 2));
#pragma unroll
        for (int k = 0; k < S; k++) {
            const int s = 64 * k + lane;
            if (s < nslots) {
                if (ADD)
                    g[s] = tile_out[swz(s)];
                else
                    stream_store(g + s, tile_out[swz(s)]);
            }
        }
    } else if (active) {
        out.store(dst, e0 + lane * 16, false);
    }
}

inline unsigned grid_for(int64_t nchunks) { return (unsigned)((nchunks + kChunksPerWave - 1) / kChunksPerWave); }

template <int DT, int RDT, int NBITS, bool MEE>
hipError_t run_compress(const void *src, uint8_t *dst, const void *rnd, int64_t nchunks, bool hier, const MeeParams &mp,
                        RandKey key, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    const int vec = (aligned16(src) ? 1 : 0) | (aligned16(rnd) ? 2 : 0);
    dim3 grid(grid_for(nchunks)), block(64);
    if (DT == DQ_F16 && hier)
        hipLaunchKernelGGL((tile16_compress_kernel<DQ_F16, RDT, NBITS, true, MEE>), grid, block, 0, stream, src, dst, rnd, nchunks, vec, key, arg);
    else
        hipLaunchKernelGGL((tile16_compress_kernel<DT, RDT, NBITS, false, MEE>), grid, block, 0, stream, src, dst, rnd, nchunks, vec, key, arg);
    return hipGetLastError();
}

template <int DT, int NBITS, bool MEE>
hipError_t run_decompress(const uint8_t *src, void *dst, int64_t nchunks, bool hier, int add, const MeeParams &mp,
                          hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    const int vec = aligned16(dst) ? 1 : 0;
    dim3 grid(grid_for(nchunks)), block(64);
    if (DT == DQ_F16 && hier) {
        if (add)
            hipLaunchKernelGGL((tile16_decompress_kernel<DQ_F16, NBITS, true, MEE, true>), grid, block, 0, stream, src, dst, nchunks, vec, arg);
        else
            hipLaunchKernelGGL((tile16_decompress_kernel<DQ_F16, NBITS, true, MEE, false>), grid, block, 0, stream, src, dst, nchunks, vec, arg);
    } else {
        if (add)
            hipLaunchKernelGGL((tile16_decompress_kernel<DT, NBITS, false, MEE, true>), grid, block, 0, stream, src, dst, nchunks, vec, arg);
        else
            hipLaunchKernelGGL((tile16_decompress_kernel<DT, NBITS, false, MEE, false>), grid, block, 0, stream, src, dst, nchunks, vec, arg);
    }
    return hipGetLastError();
}

// the uniform values of the in-kernel stream written out as a tensor: element e = chunk e / 16, byte e % 16
template <int DT>
__global__ __launch_bounds__(256) void philox_uniform_kernel(void *__restrict__ out, int64_t n, RandKey key)
{
    const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk * 16 >= n) return;
    Raw16<DQ_PHILOX> r;
    r.generate(key, chunk);
    const int cnt = (int)min((int64_t)16, n - chunk * 16);
    for (int i = 0; i < cnt; i++) ElemIO<DT>::store(out, chunk * 16 + i, r.get(i));
}

#define DQ_T16_NBITS_MEE(FN, PRE, ...)                                                                    \
    switch (nbits) {                                                                                      \
    case 2: return mee ? FN<PRE, 2, true>(__VA_ARGS__) : FN<PRE, 2, false>(__VA_ARGS__);                  \
    case 3: return mee ? FN<PRE, 3, true>(__VA_ARGS__) : FN<PRE, 3, false>(__VA_ARGS__);                  \
    case 4: return mee ? FN<PRE, 4, true>(__VA_ARGS__) : FN<PRE, 4, false>(__VA_ARGS__);                  \
    case 5: return mee ? FN<PRE, 5, true>(__VA_ARGS__) : FN<PRE, 5, false>(__VA_ARGS__);                  \
    case 6: return mee ? FN<PRE, 6, true>(__VA_ARGS__) : FN<PRE, 6, false>(__VA_ARGS__);                  \
    case 7: return mee ? FN<PRE, 7, true>(__VA_ARGS__) : FN<PRE, 7, false>(__VA_ARGS__);                  \
    default: return mee ? FN<PRE, 8, true>(__VA_ARGS__) : FN<PRE, 8, false>(__VA_ARGS__);                 \
    }
#define DQ_T16_COMMA ,

} // namespace

// dtype F16 with any strategy, or BF16 / F32 with strategy 0 / 1; chunk size 16
hipError_t launch_tile16_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n, int nbits, int dtype,
                                  int strategy, const MeeParams &mp, hipStream_t stream, const RandKey *philox)
{
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
    const bool mee = (strategy & 1) != 0, hier = strategy >= 2;
    const int64_t nchunks = n / 16;
    const RandKey key = philox ? *philox : RandKey{0, 0};
    if (philox) {
        if (dtype == DQ_F16) {
            DQ_T16_NBITS_MEE(run_compress, DQ_F16 DQ_T16_COMMA DQ_PHILOX, src, dst, rnd, nchunks, hier, mp, key, stream)
        } else if (dtype == DQ_BF16) {
            DQ_T16_NBITS_MEE(run_compress, DQ_BF16 DQ_T16_COMMA DQ_PHILOX, src, dst, rnd, nchunks, false, mp, key, stream)
        } else {
            DQ_T16_NBITS_MEE(run_compress, DQ_F32 DQ_T16_COMMA DQ_PHILOX, src, dst, rnd, nchunks, false, mp, key, stream)
        }
    }
    if (dtype == DQ_F16) {
        DQ_T16_NBITS_MEE(run_compress, DQ_F16 DQ_T16_COMMA DQ_F16, src, dst, rnd, nchunks, hier, mp, key, stream)
    } else if (dtype == DQ_BF16) {
        DQ_T16_NBITS_MEE(run_compress, DQ_BF16 DQ_T16_COMMA DQ_BF16, src, dst, rnd, nchunks, false, mp, key, stream)
    } else if (rb16) {
        DQ_T16_NBITS_MEE(run_compress, DQ_F32 DQ_T16_COMMA DQ_BF16, src, dst, rnd, nchunks, false, mp, key, stream)
    } else {
        DQ_T16_NBITS_MEE(run_compress, DQ_F32 DQ_T16_COMMA DQ_F32, src, dst, rnd, nchunks, false, mp, key, stream)
    }
}

hipError_t launch_philox_uniform(void *out, int64_t n, int dtype, uint64_t seed, uint64_t step, hipStream_t stream)
{
    const RandKey key{seed, step};
    dim3 grid((unsigned)(((n + 15) / 16 + 255) / 256)), block(256);
    switch (dtype) {
    case DQ_F16: hipLaunchKernelGGL(philox_uniform_kernel<DQ_F16>, grid, block, 0, stream, out, n, key); break;
    case DQ_BF16: hipLaunchKernelGGL(philox_uniform_kernel<DQ_BF16>, grid, block, 0, stream, out, n, key); break;
    default: hipLaunchKernelGGL(philox_uniform_kernel<DQ_F32>, grid, block, 0, stream, out, n, key); break;
    }
    return hipGetLastError();
}

hipError_t launch_tile16_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int dtype, int strategy,
                                    const MeeParams &mp, int add, hipStream_t stream)
{
    dtype &= 0xf;
    const bool mee = (strategy & 1) != 0, hier = strategy >= 2;
    const int64_t nchunks = n / 16;
    if (dtype == DQ_F16) {
        DQ_T16_NBITS_MEE(run_decompress, DQ_F16, src, dst, nchunks, hier, add, mp, stream)
    } else if (dtype == DQ_BF16) {
        DQ_T16_NBITS_MEE(run_decompress, DQ_BF16, src, dst, nchunks, false, add, mp, stream)
    } else {
        DQ_T16_NBITS_MEE(run_decompress, DQ_F32, src, dst, nchunks, false, add, mp, stream)
    }
}

} // namespace dq
