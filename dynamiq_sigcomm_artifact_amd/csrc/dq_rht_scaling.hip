// Blocked randomized Hadamard transform fused with the hierarchical chunk-16 quantiser.
//
// rht_blocked followed by scaling_compress moves every element through HBM three times (read, write the
// rotated vector, read it again); the inverse pair likewise.  Here the rotated tile never leaves the
// workgroup: a workgroup owns a tile of 2^kt consecutive floats (whole transform blocks of up to 2^15) in
// LDS.  One lane owns one chunk of 16 consecutive floats at both ends: it loads the chunk (64 bytes), flips
// the signs and does the stages of strides 1..8 on its registers, the remaining stages run as LDS passes of
// up to five stages each, and the lane then reads its chunk back and quantises it.  With the LDS index padded
// by one float per 16 a chunk is 16 consecutive words and neighbouring lanes are 17 words apart, so these
// accesses are free of bank conflicts.  The inverse kernel decodes records into registers, does the first
// stages there, finishes in LDS and stores fp32 with coalesced 16-byte stores.
//
// Results are bit for bit those of the two-call sequences: the butterflies run in the same order
// (dq_fwht.cuh), the scale is applied by the same single multiplication, and the quantiser is the tile body
// of the hier16 kernels (dq_hier16_tiles.cuh).  Numerics of the quantiser: csrc/cuda_hierarchical_mee.cu:203-505;
// of the transform: csrc/cuda_hadamard.cu:66-157,534-605 with the sign flip and 1/sqrt(block) of
// testbed_evaluation/new_comm_hooks/thc_hooks.py:95-107 folded in.
#include "dq_fwht.cuh"
#include "dq_hier16_tiles.cuh"
#include "dq_launch.h"

namespace dq {

namespace {

struct RhtTileArgs {
    const void *sign;  // may be null: fp32 +-1 values, or (sign_bits) one bit per element, set = negative
    int sign_bits;
    int64_t n;         // elements, a multiple of 256 and of the transform block
    int kt;            // log2 tile elements
    int kb;            // log2 transform block, <= kt
    float scale;
    int vec;           // 16-byte accesses to the fp32 vector and the sign vector allowed
};

// the sign flip of elements g .. g + 3 (g a multiple of 4) / of element g.  A packed sign flips the sign bit,
// which is what the multiplication by -1.0f does to every number
__device__ __forceinline__ void flip4(float4 &v, const RhtTileArgs &a, int64_t g)
{
    if (!a.sign) return;
    if (a.sign_bits) {
        const uint32_t w = static_cast<const uint32_t *>(a.sign)[g >> 5] >> (g & 31);
        v.x = __uint_as_float(__float_as_uint(v.x) ^ ((w & 1u) << 31));
        v.y = __uint_as_float(__float_as_uint(v.y) ^ ((w & 2u) << 30));
        v.z = __uint_as_float(__float_as_uint(v.z) ^ ((w & 4u) << 29));
        v.w = __uint_as_float(__float_as_uint(v.w) ^ ((w & 8u) << 28));
    } else {
        const float4 s = *reinterpret_cast<const float4 *>(static_cast<const float *>(a.sign) + g);
        v.x *= s.x; v.y *= s.y; v.z *= s.z; v.w *= s.w;
    }
}

__device__ __forceinline__ float flip1(float v, const RhtTileArgs &a, int64_t g)
{
    if (!a.sign) return v;
    if (a.sign_bits) {
        const uint32_t w = static_cast<const uint32_t *>(a.sign)[g >> 5] >> (g & 31);
        return __uint_as_float(__float_as_uint(v) ^ (w << 31));
    }
    return v * static_cast<const float *>(a.sign)[g];
}

// 16 consecutive elements starting at g (a multiple of 16), sign-flipped; zeros at and beyond n
__device__ __forceinline__ void load_chunk(float (&v)[16], const float *__restrict__ x, const RhtTileArgs &a, int64_t g)
{
    if (g + 16 <= a.n && a.vec) {
        const float4 *p = reinterpret_cast<const float4 *>(x + g);
        float4 q[4] = {p[0], p[1], p[2], p[3]};
        if (a.sign && a.sign_bits) {
            const uint32_t w = static_cast<const uint32_t *>(a.sign)[g >> 5] >> (g & 31);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                q[k].x = __uint_as_float(__float_as_uint(q[k].x) ^ (((w >> (4 * k)) & 1u) << 31));
                q[k].y = __uint_as_float(__float_as_uint(q[k].y) ^ (((w >> (4 * k + 1)) & 1u) << 31));
                q[k].z = __uint_as_float(__float_as_uint(q[k].z) ^ (((w >> (4 * k + 2)) & 1u) << 31));
                q[k].w = __uint_as_float(__float_as_uint(q[k].w) ^ (((w >> (4 * k + 3)) & 1u) << 31));
            }
        } else if (a.sign) {
            const float4 *sp = reinterpret_cast<const float4 *>(static_cast<const float *>(a.sign) + g);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float4 sg = sp[k];
                q[k].x *= sg.x; q[k].y *= sg.y; q[k].z *= sg.z; q[k].w *= sg.w;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[4 * k] = q[k].x; v[4 * k + 1] = q[k].y; v[4 * k + 2] = q[k].z; v[4 * k + 3] = q[k].w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = g + i < a.n ? flip1(x[g + i], a, g + i) : 0.0f;
    }
}

// floats of LDS holding the padded tile, rounded up so that what follows is 16-byte aligned
__host__ __device__ inline int padded_tile_floats(int kt)
{
    const int tile = 1 << kt;
    return (tile + tile / 16 + 1 + 3) & ~3;
}

template <int RDT, int NBITS, bool MEE>
__global__ void rht_compress_kernel(const float *__restrict__ x, uint8_t *__restrict__ dst, const void *__restrict__ rnd,
                                    RhtTileArgs a, int rvec, RandKey key, MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int tile = 1 << a.kt;
    const int64_t origin = (int64_t)blockIdx.x << a.kt;

    // every lane loads chunks of 16 consecutive floats (64 bytes, as the quantiser's own kernels do), flips the
    // signs and does the stages of strides 1..8 on its registers; elements beyond n (a ragged last tile) are zero
    const int nchunks = tile >> 4;
    for (int c = tid; c < nchunks; c += nthreads) {
        float v[16];
        load_chunk(v, x, a, origin + c * 16);
        chunk_stages(v, a.kb);
        float *mine = lds + c * 17; // pad_idx(16 c + i) = 17 c + i
#pragma unroll
        for (int i = 0; i < 16; i++) mine[i] = v[i];
    }
    fwht_lds_stages_after4(lds, a.kt, a.kb, tid, nthreads);

    // quantise: a wave takes runs of 64 chunks (4 superchunks, one contiguous run of records)
    const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
    uint8_t *win_out = reinterpret_cast<uint8_t *>(lds + padded_tile_floats(a.kt)) + wave * RC::WIN;
    const int64_t nsc_total = a.n >> 8, sc_origin = origin >> 8;
    const int tile_sc = max(1, tile >> 8);
    for (int run = wave; run * kRowsPerWave < tile_sc; run += nwaves) {
        const int64_t sc0 = sc_origin + run * kRowsPerWave;
        if (sc0 >= nsc_total) break;
        const int rows_here = (int)min((int64_t)min(kRowsPerWave, tile_sc - run * kRowsPerWave), nsc_total - sc0);
        Raw16<DQ_F32> v;
        Raw16<RDT> r;
        if ((lane >> 4) < rows_here) {
            if constexpr (RDT == DQ_PHILOX)
                r.generate(key, sc0 * 16 + lane);
            else
                r.load(rnd, (sc0 * 16 + lane) * 16, rvec);
            const float *mine = lds + (run * 64 + lane) * 17; // pad_idx(16 c + i) = 17 c + i
#pragma unroll
            for (int i = 0; i < 16; i++) v.w[i] = __float_as_uint(mine[i] * a.scale);
        } else {
            v.zero();
            r.zero();
        }
        encode_store_run<NBITS, MEE>(v, r, mp, dst + sc0 * RC::REC, rows_here, win_out);
        wave_lds_sync(); // the window is reused by this wave's next run
    }
}

template <int NBITS, bool MEE>
__global__ void irht_decompress_kernel(const uint8_t *__restrict__ src, float *__restrict__ x, RhtTileArgs a,
                                       MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int tile = 1 << a.kt;
    const int64_t origin = (int64_t)blockIdx.x << a.kt;
    const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
    uint8_t *windows = reinterpret_cast<uint8_t *>(lds + padded_tile_floats(a.kt));
    uint8_t *win_in = windows + wave * RC::WIN;
    float *table = reinterpret_cast<float *>(windows + nwaves * RC::WIN);
    if (MEE) {
        for (int k = tid; k < (1 << NBITS); k += nthreads) table[k] = f16_bits_to_f32(mp.table[k]);
        __syncthreads();
    }

    // decode the tile's records into LDS, one lane per chunk; chunks beyond n become zeros
    const int64_t nsc_total = a.n >> 8, sc_origin = origin >> 8;
    const int tile_sc = max(1, tile >> 8);
    for (int run = wave; run * kRowsPerWave < tile_sc; run += nwaves) {
        const int64_t sc0 = sc_origin + run * kRowsPerWave;
        const int rows_here = sc0 < nsc_total
                                  ? (int)min((int64_t)min(kRowsPerWave, tile_sc - run * kRowsPerWave), nsc_total - sc0)
                                  : 0;
        const int row = lane >> 4, j = lane & 15;
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; i++) t[i] = 0.0f;
        if (rows_here > 0) {
            const int total = rows_here * RC::REC;
            const uint8_t *g = src + sc0 * RC::REC;
            const WinRegs wr = window_fetch(g, total, lane);
            const int mis = window_commit(win_in, wr, g, total, lane);
            wave_lds_sync();
            if (row < rows_here) {
                const uint8_t *rec = win_in + mis + row * RC::REC;
                uint32_t cw[RC::WORDS], cq;
                chunk_read<NBITS>(rec + j * RC::CB, cw, cq);
                const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
                chunk_decode<NBITS, MEE, false>(cw, cq, ub, table, t);
            }
            wave_lds_sync(); // the window is reused by this wave's next run
        }
        const int c = run * 64 + lane;
        if (c * 16 < tile) {
            chunk_stages(t, a.kb);
            float *mine = lds + c * 17;
#pragma unroll
            for (int i = 0; i < 16; i++) mine[i] = t[i];
        }
    }
    fwht_lds_stages_after4(lds, a.kt, a.kb, tid, nthreads);

    // store (coalesced): scale, then sign flip
    if (a.vec) {
        for (int i = tid * 4; i < tile; i += nthreads * 4) {
            const int64_t g = origin + i;
            if (g >= a.n) continue;
            const int q = pad_idx(i);
            float4 v = make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]);
            v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale;
            flip4(v, a, g);
            *reinterpret_cast<float4 *>(x + g) = v;
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + i;
            if (g >= a.n) continue;
            x[g] = flip1(lds[pad_idx(i)] * a.scale, a, g);
        }
    }
}

constexpr int kPrefTileBits = 13; // 32 KiB tiles: eight waves, one run each, several workgroups per CU

struct Geometry {
    RhtTileArgs a;
    unsigned grid, threads;
    size_t lds_floats;
};

Geometry geometry(const float *vec, const void *sign, int sign_bits, int64_t n, int64_t block, float scale)
{
    Geometry g;
    const int kb = ilog2(block);
    int kt = kb < kPrefTileBits ? kPrefTileBits : kb;
    // short vectors: smaller tiles until there are two workgroups per CU (a tile is at least one run of 1024)
    while (kt > kb && kt > 10 && (n >> kt) < 512) kt--;
    while (kt > kb && kt > 8 && ((int64_t)1 << kt) > n) kt--;
    g.a.sign = sign; g.a.sign_bits = sign_bits; g.a.n = n; g.a.kt = kt; g.a.kb = kb; g.a.scale = scale;
    g.a.vec = aligned16(vec) && (sign == nullptr || sign_bits || aligned16(sign)) ? 1 : 0;
    const int tile = 1 << kt;
    int threads = tile / 16;
    g.threads = (unsigned)(threads < 64 ? 64 : (threads > 1024 ? 1024 : threads));
    g.grid = (unsigned)((n + tile - 1) >> kt);
    g.lds_floats = (size_t)padded_tile_floats(kt);
    return g;
}

template <class K> hipError_t allow_lds(K kernel, size_t bytes)
{
    if (bytes <= 48 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <int RDT, int NBITS, bool MEE>
hipError_t run_compress(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int64_t n, int64_t block,
                        float scale, const MeeParams &mp, RandKey key, hipStream_t stream)
{
    const Geometry g = geometry(src, sign, sign_bits, n, block, scale);
    const size_t lds = g.lds_floats * sizeof(float) + (size_t)(g.threads / 64) * Rec<NBITS>::WIN;
    auto kernel = rht_compress_kernel<RDT, NBITS, MEE>;
    hipError_t e = allow_lds(kernel, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(g.grid), dim3(g.threads), lds, stream, src, dst, rnd, g.a, aligned16(rnd) ? 1 : 0, key,
                       make_arg<NBITS, MEE>(mp));
    return hipGetLastError();
}

template <int PRE, int NBITS, bool MEE>
hipError_t run_decompress(const uint8_t *src, const void *sign, int sign_bits, float *dst, int64_t n, int64_t block, float scale,
                          const MeeParams &mp, hipStream_t stream)
{
    const Geometry g = geometry(dst, sign, sign_bits, n, block, scale);
    const size_t lds = g.lds_floats * sizeof(float) + (size_t)(g.threads / 64) * Rec<NBITS>::WIN +
                       (MEE ? (sizeof(float) << NBITS) : 0);
    auto kernel = irht_decompress_kernel<NBITS, MEE>;
    hipError_t e = allow_lds(kernel, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(g.grid), dim3(g.threads), lds, stream, src, dst, g.a, make_arg<NBITS, MEE>(mp));
    return hipGetLastError();
}

} // namespace

// rand_kind: DQ_F32 or DQ_BF16 pool, or DQ_PHILOX (rnd ignored)
hipError_t launch_rht_compress(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int rand_kind, int64_t n,
                               int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, uint64_t seed,
                               uint64_t step, hipStream_t stream)
{
    const RandKey key{seed, step};
    if (rand_kind == DQ_PHILOX) {
        DQ_NBITS_MEE(run_compress, DQ_PHILOX, src, sign, sign_bits, dst, nullptr, n, block, scale, mp, key, stream)
    } else if (rand_kind == DQ_BF16) {
        DQ_NBITS_MEE(run_compress, DQ_BF16, src, sign, sign_bits, dst, rnd, n, block, scale, mp, key, stream)
    } else {
        DQ_NBITS_MEE(run_compress, DQ_F32, src, sign, sign_bits, dst, rnd, n, block, scale, mp, key, stream)
    }
}

hipError_t launch_irht_decompress(const uint8_t *src, const void *sign, int sign_bits, float *dst, int64_t n, int64_t block, float scale,
                                  int nbits, bool mee, const MeeParams &mp, hipStream_t stream)
{
    DQ_NBITS_MEE(run_decompress, 0, src, sign, sign_bits, dst, n, block, scale, mp, stream)
}

} // namespace dq
