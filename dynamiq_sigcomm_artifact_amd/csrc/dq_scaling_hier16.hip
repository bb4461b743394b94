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
#include "dq_hier16_tiles.cuh"
#include "dq_launch.h"

namespace dq {



// ---- kernels ------------------------------------------------------------------------------------

// workgroup = one wave = one tile; the bodies live in dq_hier16_tiles.cuh
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
    const Center none{nullptr, 0, {0.0f, 0.0, 0, 0, 0, 0.0f}};
    const int64_t tile = blockIdx.x;
    compress_tile<DT, RDT, NBITS, MEE, FUSED>(src, recv, dst, rnd, row_ids_plain(rows), nsc, tile, vec, key, none, mp, win_out,
                                              win_in, table, threadIdx.x);
}

// LONG: the wave takes kTilesPerWaveLong consecutive tiles of a row list and fetches their entries with one load (RowIds).
// A variant of its own: the loop costs registers (about 50 instead of 20), which the one-tile kernel need not pay.  The
// encoder has no such variant: its time on long buckets goes into arithmetic, not into the wait for the row list, and
// looped it holds every literal of its tile body in a register of its own (over 100 registers).
constexpr int kTilesPerWaveLong = 4;

template <int DT, int NBITS, bool MEE, bool ADD, bool LONG>
__global__ __launch_bounds__(64) void hier16_decompress_kernel(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                              const int32_t *__restrict__ rows,
                                                              const uint16_t *__restrict__ stats, int64_t limit,
                                                              int64_t nsc, int vec, MeeArg<NBITS, MEE> mp)
{
    __shared__ __attribute__((aligned(16))) uint8_t win_in[Rec<NBITS>::WIN];
    __shared__ __attribute__((aligned(16))) uint4 tile_out[64 * Raw16<DT>::kSlots];
    __shared__ float table[MEE ? (1 << NBITS) : 1];
    if constexpr (LONG) {
        const int64_t tile0 = (int64_t)blockIdx.x * kTilesPerWaveLong;
        const RowIds ids = row_ids_prefetch(rows, tile0 * kRowsPerWave, kTilesPerWaveLong * kRowsPerWave, nsc, threadIdx.x);
#pragma unroll 1
        for (int t = 0; t < kTilesPerWaveLong; t++) {
            decompress_tile<DT, NBITS, MEE, ADD>(src, dst, ids, stats, limit, nsc, tile0 + t, vec, mp, win_in, tile_out, table);
            wave_lds_sync(); // window, table and output tile are reused by the next tile
        }
    } else {
        const int64_t tile = blockIdx.x;
        decompress_tile<DT, NBITS, MEE, ADD>(src, dst, row_ids_plain(rows), stats, limit, nsc, tile, vec, mp, win_in, tile_out,
                                             table);
    }
}

// ---- launchers ------------------------------------------------------------------------------------


// one single-wave workgroup per tile of 4 superchunks (per kTilesPerWaveLong tiles in the LONG decoder)
static inline unsigned grid_for(int64_t nsc, int tiles = 1)
{
    const int64_t per = (int64_t)kRowsPerWave * tiles;
    return (unsigned)((nsc + per - 1) / per);
}

constexpr int64_t kLongRun = 262144; // superchunks of a row list: 16384 waves of four tiles, two rounds of a full chip

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
    dim3 block(64);
    const int vec = aligned16(dst) ? 1 : 0;
    if (rows && nsc >= kLongRun && !add) {
        // a long row list (the decoder of the grouped pipelines on the reference's whole-model buckets)
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, false, true>), dim3(grid_for(nsc, kTilesPerWaveLong)), block, 0,
                           stream, src, dst, rows, stats, limit, nsc, vec, arg);
        return hipGetLastError();
    }
    dim3 grid(grid_for(nsc));
    if (add)
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, true, false>), grid, block, 0, stream, src, dst, rows, stats, limit, nsc, vec, arg);
    else
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, false, false>), grid, block, 0, stream, src, dst, rows, stats, limit, nsc, vec, arg);
    return hipGetLastError();
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
