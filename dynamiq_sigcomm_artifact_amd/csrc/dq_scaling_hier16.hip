// Vectorised hierarchical scaling-quantisation kernels for the production
// shape: chunk 16, superchunk 16 chunks (256 elements), bf16 or fp32 elements,
// strategies 2 (AEE) and 3 (MEE), code widths 2..8.
//
// Work decomposition (wave64, one wave per workgroup, no barriers):
//   * one lane owns one chunk: 16 consecutive elements = 32 B (bf16) / 64 B
//     (fp32) of 128-bit loads, so the chunk maximum needs no cross-lane traffic
//     and every per-chunk scalar is computed once per 16 elements;
//   * one 16-lane DPP row owns one superchunk: the superchunk maximum is four
//     DPP max steps, no LDS;
//   * one wave owns a tile of 4 consecutive superchunks = one contiguous run of
//     4 records (328..1096 bytes) of the packed stream.  Records are 82/146/274
//     bytes and never 16-byte aligned, so a run is assembled in an LDS window
//     whose offset equals the global address modulo 16 and streamed out with
//     aligned 128-bit stores (ragged head / tail bytes singly); packed input is
//     pulled through the same kind of window with aligned 128-bit loads;
//   * one single-wave workgroup per tile, ~50 VGPRs, 8 waves per SIMD: many
//     small workgroups let the dispatcher balance the chip better than a
//     persistent loop with software prefetch did (4.7 -> 5.4 TB/s at 1 GiB), and
//     a 25 MB bucket (6400 tiles) fits the machine in one resident round.
//
// VALU budget.  The quantiser is VALU-bound if written naively (IEEE division,
// NaN/Inf/out-of-range guards per element).  Two measures keep it HBM-bound:
//   * exact division by a chunk-constant: x/d == (float)((double)x * (1/d in
//     double)).  The product carries a relative error < 2^-51 while a binary32
//     quotient of binary32 operands is never closer than 2^-49 (relative) to a
//     rounding boundary without being exactly representable, so the result is
//     the correctly rounded quotient for every finite x -- three full-rate
//     instructions per element instead of the ~10-instruction division
//     expansion;
//   * a wave-uniform fast path: if every element of the wave is finite and
//     below 2^100 and every random value lies in [0, 1] (one packed integer
//     maximum per element finds out), the guards of the general formula cannot
//     fire and are skipped; otherwise the whole wave takes the guarded path.
//     Both paths produce the same bytes on the inputs the fast path accepts.
//
// Numerics: csrc/cuda_hierarchical_mee.cu:203-343 (compress), 345-505
// (decompress) and 526-696 (fused decompress-accumulate-recompress).
#include "dq_launch.h"
#include "dq_tile16.cuh"

namespace dq {



// ---- the math of one chunk ---------------------------------------------------------------------

// decode 16 levels of one chunk: t = lev*sc (+ t when ADD)
template <int NBITS, bool MEE, bool ADD>
__device__ __forceinline__ void chunk_decode(const uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t q, uint32_t unit_bits,
                                             const float *table, float (&t)[16])
{
    const float us = nonneg_scale(bf16_bits_to_f32(unit_bits));
    const float sc = nonneg_scale((float)q * us);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint32_t code = words_get<NBITS>(w, i);
        const float lev = MEE ? table[code] : (float)((int)code - Rec<NBITS>::R);
        t[i] = ADD ? __builtin_fmaf(lev, sc, t[i]) : lev * sc;
    }
}

// general (guarded) quantiser of one chunk against its superchunk row
template <int NBITS, bool MEE, class RV, class RR, class ARG>
__device__ __forceinline__ void chunk_encode_guarded(const RV &v, const RR &r, const ARG &mp,
                                                     uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t &q, uint32_t &unit_bits)
{
    constexpr int R = Rec<NBITS>::R;
    float a = __builtin_fabsf(v.get(0));
#pragma unroll
    for (int i = 1; i < 16; i++) a = __builtin_fmaxf(a, __builtin_fabsf(v.get(i)));
    const float s = pos_scale(MEE ? a / pos_scale(mp.cmm) + 1e-7f : a / (float)R + 1e-7f);
    const float g = pos_scale(row16_max(s));
    unit_bits = f32_to_bf16_bits(pos_scale(g / 255.0f));
    const float unit = pos_scale(bf16_bits_to_f32(unit_bits));
    float ratio = pos_scale(s) / pos_scale(g) * 255.0f;
    if (!__builtin_isfinite(ratio)) ratio = ratio > 0.0f ? 255.0f : 1.0f;
    int qi = sat_u16(__builtin_ceilf(ratio));
    qi = min(max(qi, 1), 255);
    q = (uint32_t)qi;
    const float d = pos_scale(pos_scale((float)qi * unit));
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float x = v.get(i) / d;
        if (MEE) x = mee_inverse_guarded(x, mp.c, mp.l2b);
        words_put<NBITS>(w, i, (uint32_t)clamp_code(sr_guarded(x, r.get(i)), R));
    }
}

// the same quantiser for a wave whose elements are all finite and <= 2^100 in
// magnitude (amax_bits is the integer-order maximum of |v|) and whose random
// values all lie in [0, 1]: none of the guards can fire
template <int NBITS, bool MEE, class RV, class RR, class ARG>
__device__ __forceinline__ void chunk_encode_fast(const RV &v, const RR &r, uint32_t amax_bits, const ARG &mp,
                                                  uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t &q, uint32_t &unit_bits)
{
    constexpr int R = Rec<NBITS>::R;
    const float a = __uint_as_float(amax_bits);
    float s;
    if (MEE)
        s = div_by(a, mp.inv_cmm) + 1e-7f;
    else
        s = (R == 1 ? a : div_by(a, 1.0 / (double)R)) + 1e-7f; // >= 1e-7, finite
    const float g = row16_max(s);
    unit_bits = f32_to_bf16_bits(div_by(g, 1.0 / 255.0));
    const float unit = bf16_bits_to_f32(unit_bits);
    const float ratio = div_by(s, recip_f64(g)) * 255.0f;
    int qi = (int)__builtin_ceilf(ratio);
    qi = min(max(qi, 1), 255);
    q = (uint32_t)qi;
    const float d = (float)qi * unit; // exact: 8 x 8 significant bits
    const double yd = recip_f64(d);
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float x = div_by(v.get(i), yd);
        if (MEE) {
            const float arg = div_by(__builtin_fabsf(x), mp.inv_c) + 1.0f;
            const float lat = div_by(log2_det_ge1(arg), mp.inv_l2b);
            x = __builtin_copysignf(lat, x);
        }
        const float fl = __builtin_floorf(x);
        const float c = __builtin_ceilf((x - fl) - r.get(i));
        const int sv = (int)(fl + c); // |fl| <= R + 1 and c in {-1, 0, 1}: exact
        words_put<NBITS>(w, i, (uint32_t)(min(max(sv, -R), R) + R));
    }
}

constexpr uint32_t kFastMaxBits = 0x71800000u; // 2^100

// ---- kernels ------------------------------------------------------------------------------------

// compress (FUSED = false) or decode-accumulate-recompress (FUSED = true); workgroup = one wave = one tile.
// Record k of the packed streams (and row k of rnd) belongs to superchunk rows[k] of src
// (to superchunk k when rows is null).
template <int DT, int RDT, int NBITS, bool MEE, bool FUSED>
__global__ __launch_bounds__(64) void hier16_compress_kernel(const void *__restrict__ src, const uint8_t *__restrict__ recv,
                                                            uint8_t *__restrict__ dst, const void *__restrict__ rnd,
                                                            const int32_t *__restrict__ rows, int64_t nsc, int vec,
                                                            RandKey key, MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    __shared__ __attribute__((aligned(16))) uint8_t win_out[RC::WIN];
    __shared__ __attribute__((aligned(16))) uint8_t win_in[FUSED ? RC::WIN : 16];
    __shared__ float table[(MEE && FUSED) ? (1 << NBITS) : 1];

    const int lane = threadIdx.x;
    const int row = lane >> 4, j = lane & 15;
    const int64_t sc0 = (int64_t)blockIdx.x * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows_here = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const bool active = row < rows_here;
    const int total = rows_here * RC::REC;

    // all global loads of the tile are issued before anything waits on them
    Raw16<DT> v;
    Raw16<RDT> r;
    if (active) {
        if constexpr (RDT == DQ_PHILOX)
            r.generate(key, sc0 * 16 + lane);
        else
            r.load(rnd, (sc0 * 16 + lane) * 16, vec & 2);
        const int64_t sc_src = rows ? (int64_t)rows[sc0 + row] : sc0 + row;
        v.load(src, (sc_src * 16 + j) * 16, vec & 1);
    } else {
        v.zero();
        r.zero();
    }
    WinRegs wr;
    if (FUSED) wr = window_fetch(recv + sc0 * RC::REC, total, lane);
    if (MEE && FUSED) {
        for (int k = lane; k < (1 << NBITS); k += 64) table[k] = f16_bits_to_f32(mp.table[k]);
    }

    if (FUSED) {
        const int mis_in = window_commit(win_in, wr, recv + sc0 * RC::REC, total, lane);
        wave_lds_sync();
        if (active) {
            const uint8_t *rec = win_in + mis_in + row * RC::REC;
            uint32_t cw[RC::WORDS], cq;
            chunk_read<NBITS>(rec + j * RC::CB, cw, cq);
            const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
            float t[16];
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = v.get(i);
            chunk_decode<NBITS, MEE, true>(cw, cq, ub, table, t);
            v.set(t); // rounds the sum to the element type
        }
    }

    uint32_t w[RC::WORDS], q, ub;
    const uint32_t amax = v.absmax_bits();
    const bool lane_fast = amax <= kFastMaxBits && r.unit_interval();
    if (__builtin_amdgcn_ballot_w64(!lane_fast) == 0)
        chunk_encode_fast<NBITS, MEE>(v, r, amax, mp, w, q, ub);
    else
        chunk_encode_guarded<NBITS, MEE>(v, r, mp, w, q, ub);

    uint8_t *gout = dst + sc0 * RC::REC;
    const int mis = (int)(reinterpret_cast<uintptr_t>(gout) & 15);
    if (active) {
        uint8_t *rec = win_out + mis + row * RC::REC;
        chunk_write<NBITS>(rec + j * RC::CB, w, q);
        if (j == 0) {
            rec[16 * RC::CB] = (uint8_t)ub;
            rec[16 * RC::CB + 1] = (uint8_t)(ub >> 8);
        }
    }
    wave_lds_sync();
    window_flush(win_out, gout, mis, total, lane);
}


// Record k decodes into superchunk rows[k] of dst (superchunk k when rows is null). With stats
// (interleaved bf16 pairs, the mean first) the stored value is T(float(T(decoded)) + mean of the
// destination superchunk); elements at or beyond `limit` are not written.
template <int DT, int NBITS, bool MEE, bool ADD>
__global__ __launch_bounds__(64) void hier16_decompress_kernel(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                              const int32_t *__restrict__ rows,
                                                              const uint16_t *__restrict__ stats, int64_t limit,
                                                              int64_t nsc, int vec, MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    constexpr int S = Raw16<DT>::kSlots;
    constexpr int ESZ = DT == DQ_F32 ? 4 : 2;
    constexpr int EP = 16 / ESZ; // elements per 16-byte slot
    __shared__ __attribute__((aligned(16))) uint8_t win_in[RC::WIN];
    __shared__ __attribute__((aligned(16))) uint4 tile_out[64 * S];
    __shared__ float table[MEE ? (1 << NBITS) : 1];

    const int lane = threadIdx.x;
    const int row = lane >> 4, j = lane & 15;
    const int64_t sc0 = (int64_t)blockIdx.x * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows_here = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const bool active = row < rows_here;
    const int total = rows_here * RC::REC;

    const WinRegs wr = window_fetch(src + sc0 * RC::REC, total, lane);
    // destination superchunk of this lane's chunk, and of the slots this lane stores after the transpose
    int64_t d_own = sc0 + row;
    int64_t d_slot[S];
#pragma unroll
    for (int k = 0; k < S; k++) d_slot[k] = sc0 + (64 * k + lane) / (16 * S);
    if (rows) {
        if (active) d_own = rows[sc0 + row];
#pragma unroll
        for (int k = 0; k < S; k++) {
            const int rr = (64 * k + lane) / (16 * S);
            if (rr < rows_here) d_slot[k] = rows[sc0 + rr];
        }
    }
    Raw16<DT> acc;
    if (ADD && active) acc.load(dst, d_own * 256 + j * 16, vec);
    float mean = 0.0f;
    if (stats && active) mean = bf16_bits_to_f32(stats[2 * d_own]);
    if (MEE) {
        for (int k = lane; k < (1 << NBITS); k += 64) table[k] = f16_bits_to_f32(mp.table[k]);
    }

    const int mis_in = window_commit(win_in, wr, src + sc0 * RC::REC, total, lane);
    wave_lds_sync();
    Raw16<DT> out;
    if (active) {
        const uint8_t *rec = win_in + mis_in + row * RC::REC;
        uint32_t cw[RC::WORDS], cq;
        chunk_read<NBITS>(rec + j * RC::CB, cw, cq);
        const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
        float t[16];
        if (ADD) {
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = acc.get(i);
        }
        chunk_decode<NBITS, MEE, ADD>(cw, cq, ub, table, t);
        out.set(t);
        if (stats) {
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = out.get(i) + mean;
            out.set(t);
        }
    } else {
        out.zero();
    }
    char *dbytes = static_cast<char *>(dst);
    if (vec) {
        // transpose through LDS so that every store instruction writes whole superchunks contiguously
        if (active) {
#pragma unroll
            for (int k = 0; k < S; k++) tile_out[swz(S * lane + k)] = out.slot(k);
        }
        wave_lds_sync();
        const int nslots = rows_here * 16 * S;
#pragma unroll
        for (int k = 0; k < S; k++) {
            const int s = 64 * k + lane;
            if (s < nslots) {
                const int64_t e = d_slot[k] * 256 + (s % (16 * S)) * EP;
                const uint4 val = tile_out[swz(s)];
                if (e + EP <= limit) {
                    *reinterpret_cast<uint4 *>(dbytes + e * ESZ) = val;
                } else {
                    const uint32_t part[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                    for (int i = 0; i < EP; i++) {
                        if (e + i < limit) {
                            if (DT == DQ_F32)
                                reinterpret_cast<uint32_t *>(dbytes)[e + i] = part[i];
                            else
                                reinterpret_cast<uint16_t *>(dbytes)[e + i] = (uint16_t)(part[i >> 1] >> (16 * (i & 1)));
                        }
                    }
                }
            }
        }
    } else if (active) {
        const int64_t e = d_own * 256 + j * 16;
        if (e + 16 <= limit) {
            out.store(dst, e, false);
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if (e + i < limit) {
                    if (DT == DQ_F32)
                        reinterpret_cast<uint32_t *>(dbytes)[e + i] = out.w[i];
                    else
                        reinterpret_cast<uint16_t *>(dbytes)[e + i] = (uint16_t)(out.w[i >> 1] >> (16 * (i & 1)));
                }
            }
        }
    }
}

// ---- launchers ------------------------------------------------------------------------------------


// one single-wave workgroup per tile of 4 superchunks
static inline unsigned grid_for(int64_t nsc) { return (unsigned)((nsc + kRowsPerWave - 1) / kRowsPerWave); }

template <int DT, int RDT, int NBITS, bool MEE>
static hipError_t run_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd, const int32_t *rows,
                               int64_t nsc, bool fused, const MeeParams &mp, RandKey key, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    dim3 grid(grid_for(nsc)), block(64);
    const int vec = (aligned16(src) ? 1 : 0) | (aligned16(rnd) ? 2 : 0);
    if (fused)
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, true>), grid, block, 0, stream, src, recv, dst, rnd, rows, nsc, vec, key, arg);
    else
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, false>), grid, block, 0, stream, src, recv, dst, rnd, rows, nsc, vec, key, arg);
    return hipGetLastError();
}

template <int DT, int NBITS, bool MEE>
static hipError_t run_decompress(const uint8_t *src, void *dst, const int32_t *rows, const uint16_t *stats, int64_t limit,
                                 int64_t nsc, int add, const MeeParams &mp, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    dim3 grid(grid_for(nsc)), block(64);
    const int vec = aligned16(dst) ? 1 : 0;
    if (add)
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, true>), grid, block, 0, stream, src, dst, rows, stats, limit, nsc, vec, arg);
    else
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, false>), grid, block, 0, stream, src, dst, rows, stats, limit, nsc, vec, arg);
    return hipGetLastError();
}

// FN<dtype..., NBITS, MEE>(args) for the runtime (nbits, mee)
#define DQ_NBITS_MEE(FN, PRE, ...)                                                                        \
    switch (nbits) {                                                                                      \
    case 2: return mee ? FN<PRE, 2, true>(__VA_ARGS__) : FN<PRE, 2, false>(__VA_ARGS__);                  \
    case 3: return mee ? FN<PRE, 3, true>(__VA_ARGS__) : FN<PRE, 3, false>(__VA_ARGS__);                  \
    case 4: return mee ? FN<PRE, 4, true>(__VA_ARGS__) : FN<PRE, 4, false>(__VA_ARGS__);                  \
    case 5: return mee ? FN<PRE, 5, true>(__VA_ARGS__) : FN<PRE, 5, false>(__VA_ARGS__);                  \
    case 6: return mee ? FN<PRE, 6, true>(__VA_ARGS__) : FN<PRE, 6, false>(__VA_ARGS__);                  \
    case 7: return mee ? FN<PRE, 7, true>(__VA_ARGS__) : FN<PRE, 7, false>(__VA_ARGS__);                  \
    default: return mee ? FN<PRE, 8, true>(__VA_ARGS__) : FN<PRE, 8, false>(__VA_ARGS__);                 \
    }

#define DQ_COMMA ,

static hipError_t dispatch_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd,
                                    const int32_t *rows, int64_t nsc, bool fused, int nbits, int dtype, bool mee,
                                    const MeeParams &mp, hipStream_t stream, const RandKey *philox = nullptr)
{
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
    const RandKey key = philox ? *philox : RandKey{0, 0};
    if (philox) {
        if (dtype == DQ_BF16) {
            DQ_NBITS_MEE(run_compress, DQ_BF16 DQ_COMMA DQ_PHILOX, src, recv, dst, rnd, rows, nsc, fused, mp, key, stream)
        } else {
            DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_PHILOX, src, recv, dst, rnd, rows, nsc, fused, mp, key, stream)
        }
    }
    if (dtype == DQ_BF16) {
        DQ_NBITS_MEE(run_compress, DQ_BF16 DQ_COMMA DQ_BF16, src, recv, dst, rnd, rows, nsc, fused, mp, key, stream)
    } else if (rb16) {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_BF16, src, recv, dst, rnd, rows, nsc, fused, mp, key, stream)
    } else {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_F32, src, recv, dst, rnd, rows, nsc, fused, mp, key, stream)
    }
}

hipError_t launch_hier16_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n, int nbits, int dtype,
                                  bool mee, const MeeParams &mp, hipStream_t stream)
{
    return dispatch_compress(src, nullptr, dst, rnd, nullptr, n / 256, false, nbits, dtype, mee, mp, stream);
}

hipError_t launch_hier16_dec_comp(const uint8_t *recv, const void *inp, uint8_t *send, const void *rnd, int64_t n,
                                  int nbits, int dtype, bool mee, const MeeParams &mp, hipStream_t stream)
{
    return dispatch_compress(inp, recv, send, rnd, nullptr, n / 256, true, nbits, dtype, mee, mp, stream);
}

hipError_t launch_hier16_compress_philox(const void *src, const uint8_t *recv, uint8_t *dst, int64_t n, int nbits, int dtype,
                                         bool mee, const MeeParams &mp, uint64_t seed, uint64_t step, hipStream_t stream)
{
    const RandKey key{seed, step};
    return dispatch_compress(src, recv, dst, nullptr, nullptr, n / 256, recv != nullptr, nbits, dtype, mee, mp, stream, &key);
}

hipError_t launch_hier16_compress_rows(const void *src, const uint8_t *recv, const int32_t *rows, uint8_t *dst,
                                       const void *rnd, int64_t nrows, int nbits, int dtype, bool mee,
                                       const MeeParams &mp, hipStream_t stream)
{
    return dispatch_compress(src, recv, dst, rnd, rows, nrows, recv != nullptr, nbits, dtype, mee, mp, stream);
}

static hipError_t dispatch_decompress(const uint8_t *src, void *dst, const int32_t *rows, const uint16_t *stats,
                                      int64_t limit, int64_t nsc, int nbits, int dtype, bool mee, const MeeParams &mp,
                                      int add, hipStream_t stream)
{
    if ((dtype & 0xf) == DQ_BF16) {
        DQ_NBITS_MEE(run_decompress, DQ_BF16, src, dst, rows, stats, limit, nsc, add, mp, stream)
    } else {
        DQ_NBITS_MEE(run_decompress, DQ_F32, src, dst, rows, stats, limit, nsc, add, mp, stream)
    }
}

hipError_t launch_hier16_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int dtype, bool mee,
                                    const MeeParams &mp, int add, hipStream_t stream)
{
    return dispatch_decompress(src, dst, nullptr, nullptr, n, n / 256, nbits, dtype, mee, mp, add, stream);
}

hipError_t launch_hier16_decompress_rows(const uint8_t *src, void *dst, const int32_t *rows, const void *stats,
                                         int64_t limit, int64_t nrows, int nbits, int dtype, bool mee,
                                         const MeeParams &mp, int add, hipStream_t stream)
{
    return dispatch_decompress(src, dst, rows, static_cast<const uint16_t *>(stats), limit, nrows, nbits, dtype, mee, mp,
                               add, stream);
}

} // namespace dq
