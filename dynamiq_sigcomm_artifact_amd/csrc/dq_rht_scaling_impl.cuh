// Blocked randomized Hadamard transform fused with the hierarchical chunk-16 quantiser, and -- with the same lane = chunk
// structure -- the passes of the transform alone (rht_tile_kernel, rht_tile_split_kernel, rht_strided_kernel), with or
// without THC's / EDEN's quantisers at the ends; dq_hadamard.hip plans which passes a transform takes.
//
// rht_blocked followed by scaling_compress moves every element through HBM three times (read, write the
// rotated vector, read it again); the inverse pair likewise.  Here the rotated tile never leaves the
// workgroup: a workgroup owns a tile of 2^kt consecutive floats (whole transform blocks of up to 2^15) in
// LDS.  One lane owns one chunk of 16 consecutive floats at both ends: it loads the chunk (64 bytes), flips
// the signs and does the stages of strides 1..8 on its registers, the remaining stages run as LDS passes of
// up to five stages each, and the lane then reads its chunk back and quantises it.  The LDS index is padded by
// one float per 32 (dq_fwht.cuh): the chunk-wise accesses, the passes and the coalesced stores are then all free
// of bank conflicts.  The inverse kernel decodes records into registers, does the first
// stages there, finishes in LDS and stores fp32 with coalesced 16-byte stores.
//
// Results are bit for bit those of the two-call sequences: the butterflies run in the same order
// (dq_fwht.cuh), the scale is applied by the same single multiplication, and the quantiser is the tile body
// of the hier16 kernels (dq_hier16_tiles.cuh).  Numerics of the quantiser: csrc/cuda_hierarchical_mee.cu:203-505;
// of the transform: csrc/cuda_hadamard.cu:66-157,534-605 with the sign flip and 1/sqrt(block) of
// testbed_evaluation/new_comm_hooks/thc_hooks.py:95-107 folded in.
//
// This file is the body of several translation units (the kernel templates have a few hundred instantiations between
// them, and one compiler run over all of them takes minutes): each .hip file that includes it defines DQ_RHT_PART as the
// set of entry points it emits --
//   DQ_RHT_TRANSFORM          launch_rht_tile, launch_rht_strided, launch_rht_compress (the dispatcher), the matrix-core variant
//   DQ_RHT_COMPRESS_PHILOX    launch_rht_compress_philox      (dq_rht_compress_philox.hip)
//   DQ_RHT_COMPRESS_BF16      launch_rht_compress_bf16_pool   (dq_rht_compress_bf16.hip)
//   DQ_RHT_COMPRESS_F32       launch_rht_compress_f32_pool    (dq_rht_compress_f32.hip)
//   DQ_RHT_DECOMPRESS         launch_irht_decompress          (dq_rht_decompress.hip)
// -- and only the templates those use are instantiated there.
#pragma once

#include <algorithm>

#include "dq_fwht.cuh"
#include "dq_hier16_tiles.cuh"
#include "dq_launch.h"

#define DQ_RHT_TRANSFORM 1
#define DQ_RHT_COMPRESS_PHILOX 2
#define DQ_RHT_COMPRESS_BF16 4
#define DQ_RHT_COMPRESS_F32 8
#define DQ_RHT_DECOMPRESS 16
#ifndef DQ_RHT_PART
#error "define DQ_RHT_PART before including dq_rht_scaling_impl.cuh"
#endif

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
__host__ __device__ constexpr int padded_tile_floats(int kt) { return padded_floats(1 << kt); }

// The stages of strides 1..8 of 64 chunks as one matrix product on the matrix cores: Y = X H16, X the wave's 64 x 16
// block of chunks, H16[i][j] = (-1)^popcount(i & j).  v_mfma_f32_16x16x4_f32 takes a 16 x 4 slice of X (lane l: row
// l % 16, column l / 16 of the slice) against a 4 x 16 slice of H16 (lane l: row l / 16, column l % 16) and leaves a
// 16 x 16 block of Y with lane l holding rows 4 (l / 16) .. + 3 of column l % 16.  With slice j made of the columns
// 4 (l / 16) + j of X, a lane's four slice operands are one aligned float4 of its row.  The sums of a product are not
// formed in the butterfly order, so the last bits differ from the stage-by-stage transform (the reference's own
// tolerance for the transform is 1e-5 relative): a measurement variant, not the default.
typedef float mfma_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void chunk_stages_mfma16(const float *__restrict__ x, const RhtTileArgs &a, int64_t origin, int chunk0,
                                                    int lane, float *lds)
{
    const int m = lane & 15, kk = lane >> 4;
    float h[4];
#pragma unroll
    for (int j = 0; j < 4; j++) h[j] = (__builtin_popcount((4 * kk + j) & m) & 1) ? -1.0f : 1.0f;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int64_t g = origin + (int64_t)(chunk0 + 16 * b + m) * 16 + 4 * kk;
        float4 q = *reinterpret_cast<const float4 *>(x + g);
        flip4(q, a, g);
        mfma_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(q.x, h[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(q.y, h[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(q.z, h[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(q.w, h[3], acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) lds[chunk_word(chunk0 + 16 * b + 4 * kk + i) + m] = acc[i];
    }
}

template <int RDT, int NBITS, bool MEE, bool MFMA16 = false>
__global__ __attribute__((amdgpu_waves_per_eu(8, 8))) void rht_compress_kernel(const float *__restrict__ x, uint8_t *__restrict__ dst, const void *__restrict__ rnd,
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
    if constexpr (MFMA16) {
        // whole tiles, 16-byte aligned, blocks of at least 16 (checked by the launcher)
        for (int c0 = (tid >> 6) * 64; c0 < nchunks; c0 += nthreads) chunk_stages_mfma16(x, a, origin, c0, tid & 63, lds);
    } else {
    for (int c = tid; c < nchunks; c += nthreads) {
        float v[16];
        load_chunk(v, x, a, origin + c * 16);
        chunk_stages(v, a.kb);
        float *mine = lds + chunk_word(c);
#pragma unroll
        for (int i = 0; i < 16; i++) mine[i] = v[i];
    }
    }
    fwht_lds_stages_after4(lds, a.kt, a.kb, tid, nthreads);

    // quantise: the tile holds one run of 64 chunks (4 superchunks, one contiguous run of records) per wave.
    // Every wave first takes its chunks into registers; after the barrier the tile is dead and the record
    // windows reuse its LDS.
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t nsc_total = a.n >> 8, sc_origin = origin >> 8;
    const int tile_sc = max(1, tile >> 8);
    const int64_t sc0 = sc_origin + wave * kRowsPerWave;
    const int rows_here = (wave * kRowsPerWave < tile_sc && sc0 < nsc_total)
                              ? (int)min((int64_t)min(kRowsPerWave, tile_sc - wave * kRowsPerWave), nsc_total - sc0)
                              : 0;
    Raw16<DQ_F32> v;
    Raw16<RDT> r;
    if ((lane >> 4) < rows_here) {
        if constexpr (RDT == DQ_PHILOX)
            r.generate(key, sc0 * 16 + lane);
        else
            r.load(rnd, (sc0 * 16 + lane) * 16, rvec);
        const float *mine = lds + chunk_word(wave * 64 + lane);
#pragma unroll
        for (int i = 0; i < 16; i++) v.w[i] = __float_as_uint(mine[i] * a.scale);
    } else {
        v.zero();
        r.zero();
    }
    __syncthreads();
    if (rows_here > 0)
        encode_store_run<NBITS, MEE, kRowsPerWave, false>(v, r, mp, dst + sc0 * RC::REC, rows_here, reinterpret_cast<uint8_t *>(lds) + wave * RC::WIN, threadIdx.x & 63);
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
    // the record windows and the MEE table use the tile's LDS before the tile itself does
    uint8_t *windows = reinterpret_cast<uint8_t *>(lds);
    uint8_t *win_in = windows + wave * RC::WIN;
    float *table = reinterpret_cast<float *>(windows + nwaves * RC::WIN);
    if (MEE) {
        for (int k = tid; k < (1 << NBITS); k += nthreads) table[k] = f16_bits_to_f32(mp.table[k]);
        __syncthreads();
    }

    // decode the wave's run of records into registers, one lane per chunk; chunks beyond n become zeros
    const int64_t nsc_total = a.n >> 8, sc_origin = origin >> 8;
    const int tile_sc = max(1, tile >> 8);
    const int64_t sc0 = sc_origin + wave * kRowsPerWave;
    const int rows_here = (wave * kRowsPerWave < tile_sc && sc0 < nsc_total)
                              ? (int)min((int64_t)min(kRowsPerWave, tile_sc - wave * kRowsPerWave), nsc_total - sc0)
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
    }
    __syncthreads(); // windows and table are done with: the tile takes the LDS
    {
        const int c = wave * 64 + lane;
        if (c * 16 < tile) {
            chunk_stages(t, a.kb);
            float *mine = lds + chunk_word(c);
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
            stream_store(reinterpret_cast<float4 *>(x + g), v);
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + i;
            if (g >= a.n) continue;
            x[g] = flip1(lds[pad_idx(i)] * a.scale, a, g);
        }
    }
}

// ---- quantisers folded into the ends of the plain transform (TransformEnds) ------------------------------------

// the sign flip of a chunk that is already in registers (g a multiple of 16; 16-byte accesses to a float sign vector)
__device__ __forceinline__ void flip16(float (&v)[16], const RhtTileArgs &a, int64_t g)
{
    if (!a.sign) return;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float4 q = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
        flip4(q, a, g + 4 * k);
        v[4 * k] = q.x; v[4 * k + 1] = q.y; v[4 * k + 2] = q.z; v[4 * k + 3] = q.w;
    }
}

// The chunk at g (a multiple of 16; n is a multiple of 32, so the chunk is inside the vector or outside) as the first
// pass sees it: the floats of x, or THC's levels times step plus lo (thc_hooks.py:176-178: two roundings), or the
// centroids of EDEN's bins, read from the bit planes (srrcomp.py:343-354); then the sign flip of a forward transform.
// cen: the centroid table in LDS.
template <bool ENDS>
__device__ __forceinline__ void fetch_chunk(float (&v)[16], const float *__restrict__ x, const RhtTileArgs &in,
                                            const TransformEnds &e, const float *cen, int64_t g)
{
    if (!ENDS || (!e.in_levels && !e.in_planes)) {
        load_chunk(v, x, in, g);
        return;
    }
    if (g >= in.n) {
#pragma unroll
        for (int i = 0; i < 16; i++) v[i] = 0.0f;
        return;
    }
    if (e.in_levels) {
        const uint4 *p = reinterpret_cast<const uint4 *>(e.in_levels + g);
        const uint4 l0 = p[0], l1 = p[1];
        const uint32_t w[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
        const float step = *e.in_step, lo = *e.in_lo;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float p0 = bf16_bits_to_f32(w[k] & 0xffffu) * step, p1 = bf16_bits_to_f32(w[k] >> 16) * step;
            v[2 * k] = p0 + lo;
            v[2 * k + 1] = p1 + lo;
        }
    } else {
        // sixteen consecutive bins from the thread's half word of every plane (two 8 x 8 bit transposes)
        const uint16_t *half = reinterpret_cast<const uint16_t *>(e.in_planes) + (g >> 4);
        const int64_t words = in.n >> 5;
        uint64_t lo8 = 0, hi8 = 0;
        for (int p = 0; p < e.in_nbits; p++) {
            const uint32_t h = half[(int64_t)p * words * 2];
            lo8 |= (uint64_t)(h & 0xffu) << (8 * p);
            hi8 |= (uint64_t)(h >> 8) << (8 * p);
        }
        lo8 = transpose8x8(lo8);
        hi8 = transpose8x8(hi8);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[k] = cen[(lo8 >> (8 * k)) & 0xffu];
            v[8 + k] = cen[(hi8 >> (8 * k)) & 0xffu];
        }
    }
    flip16(v, in, g);
}

// four consecutive elements of the last pass on their way out: scale, sign flip of an inverse transform, EDEN's scale,
// then the float store or THC's quantiser (thc_hooks.py:161-166) and a bf16 store
template <bool ENDS>
__device__ __forceinline__ void store4(float *__restrict__ x, float4 v, const RhtTileArgs &a, const TransformEnds &e, int sign_mode,
                                       int apply_scale, int64_t g)
{
    if (apply_scale) { v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale; }
    if (sign_mode == 2) flip4(v, a, g);
    if (ENDS && e.post_scale) {
        const float ps = *e.post_scale;
        v.x *= ps; v.y *= ps; v.z *= ps; v.w *= ps;
    }
    if (ENDS && e.out_levels) {
        const float4 u = *reinterpret_cast<const float4 *>(e.uniform + g);
        const float lo = *e.out_lo, delta = *e.out_delta;
        uint2 o;
        o.x = f32x2_to_bf16x2(thc_level(v.x, u.x, lo, delta, e.out_top), thc_level(v.y, u.y, lo, delta, e.out_top));
        o.y = f32x2_to_bf16x2(thc_level(v.z, u.z, lo, delta, e.out_top), thc_level(v.w, u.w, lo, delta, e.out_top));
        *reinterpret_cast<uint2 *>(e.out_levels + g) = o;
    } else {
        *reinterpret_cast<float4 *>(x + g) = v;
    }
}

// The transform alone (dq_rht_blocked, the first pass of a long dq_hadamard) with the structure of the two kernels
// above: a lane loads its chunk of 16 consecutive floats, does the stages of strides 1..8 on its registers, the rest
// runs as LDS passes of up to five stages, and the tile leaves as coalesced 16-byte stores with the scale and (inverse
// direction) the sign flip.  Against the all-in-LDS kernel of dq_hadamard.hip: two or three LDS passes instead of four,
// and a thread's loads issued together.  In place: a workgroup reads and writes only its own tile.
// sign_mode: 0 no flip, 1 flip on load, 2 flip on store
// ENDS: a quantiser may sit at either end (TransformEnds; 16-byte accesses only: a.vec is set)
template <bool ENDS>
__global__ void rht_tile_kernel(float *__restrict__ x, RhtTileArgs a, int sign_mode, int apply_scale, TransformEnds e)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int tile = 1 << a.kt;
    const int64_t origin = (int64_t)blockIdx.x << a.kt;
    RhtTileArgs in = a;
    if (sign_mode != 1) in.sign = nullptr;
    const float *cen = lds + padded_tile_floats(a.kt); // EDEN's centroids sit behind the tile
    if (ENDS && e.in_planes) {
        for (int k = tid; k < (1 << e.in_nbits); k += nthreads) lds[padded_tile_floats(a.kt) + k] = e.in_centroids[k];
        __syncthreads();
    }
    const int nchunks = tile >> 4;
    if (nchunks == 2 * nthreads) {
        // 2^15 tiles: both chunks of a thread are loaded before either is used
        float v[16], w[16];
        fetch_chunk<ENDS>(v, x, in, e, cen, origin + tid * 16);
        fetch_chunk<ENDS>(w, x, in, e, cen, origin + (tid + nthreads) * 16);
        chunk_stages(v, a.kb);
        chunk_stages(w, a.kb);
        float *mine = lds + chunk_word(tid), *other = lds + chunk_word(tid + nthreads);
#pragma unroll
        for (int i = 0; i < 16; i++) mine[i] = v[i];
#pragma unroll
        for (int i = 0; i < 16; i++) other[i] = w[i];
    } else {
        for (int c = tid; c < nchunks; c += nthreads) {
            float v[16];
            fetch_chunk<ENDS>(v, x, in, e, cen, origin + c * 16);
            chunk_stages(v, a.kb);
            float *mine = lds + chunk_word(c);
#pragma unroll
            for (int i = 0; i < 16; i++) mine[i] = v[i];
        }
    }
    fwht_lds_stages_after4(lds, a.kt, a.kb, tid, nthreads);
    if (a.vec) {
        for (int i = tid * 4; i < tile; i += nthreads * 4) {
            const int64_t g = origin + i;
            if (g >= a.n) continue;
            const int q = pad_idx(i);
            store4<ENDS>(x, make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]), a, e, sign_mode, apply_scale, g);
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + i;
            if (g >= a.n) continue;
            float v = lds[pad_idx(i)];
            if (apply_scale) v *= a.scale;
            x[g] = sign_mode == 2 ? flip1(v, a, g) : v;
        }
    }
}

// A later pass of a transform longer than one tile: index bits [sbits, sbits + rbits) of the vector.  A tile is
// 2^rbits rows of 32 consecutive floats (128 bytes), row stride 2^sbits elements; in LDS it is row-major, so row bit b
// is tile bit b + 5.  A thread owns column tid % 32 of sixteen consecutive rows: it loads them (every load instruction of
// a wave covers two whole 128-byte row segments), does the four lowest row stages on its registers and leaves the other
// rbits - 4 (at most 6) to one or two LDS passes.  sign_mode: 0, or 2 = flip on store (the last pass of an inverse).
template <bool ENDS>
__global__ void rht_strided_kernel(float *__restrict__ x, RhtTileArgs a, int rbits, int sbits, int sign_mode, int apply_scale,
                                   TransformEnds e)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int tile = 1 << (rbits + 5);
    // (shift and mask: written as a quotient and remainder by the power of two, the compiler expands a 64-bit
    // division in front of the kernel's first loads)
    const int64_t hi = (int64_t)(blockIdx.x >> (sbits - 5)), mid = (int64_t)(blockIdx.x & ((1u << (sbits - 5)) - 1u));
    const int64_t origin = (hi << (sbits + rbits)) + (mid << 5);
    const int col = tid & 31;
    const int groups = tile >> 9; // groups of sixteen rows
    if (groups == 2 * (nthreads >> 5)) {
        // 1024 rows: both groups of a thread are loaded before either is used
        const int r0 = (tid >> 5) * 16, r1 = r0 + (nthreads >> 5) * 16;
        float v[16], w[16];
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = x[origin + ((int64_t)(r0 + j) << sbits) + col];
#pragma unroll
        for (int j = 0; j < 16; j++) w[j] = x[origin + ((int64_t)(r1 + j) << sbits) + col];
        butterflies<4>(v);
        butterflies<4>(w);
#pragma unroll
        for (int j = 0; j < 16; j++) lds[pad_idx((r0 + j) * 32 + col)] = v[j];
#pragma unroll
        for (int j = 0; j < 16; j++) lds[pad_idx((r1 + j) * 32 + col)] = w[j];
    } else {
        for (int grp = tid >> 5; grp < groups; grp += nthreads >> 5) {
            float v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = x[origin + ((int64_t)(grp * 16 + j) << sbits) + col];
            butterflies<4>(v);
#pragma unroll
            for (int j = 0; j < 16; j++) lds[pad_idx((grp * 16 + j) * 32 + col)] = v[j];
        }
    }
    __syncthreads();
#define DQ_PASS(P, M)                                  \
    lds_pass<P, M>(lds, rbits + 5, tid, nthreads);     \
    __syncthreads();
    switch (rbits - 4) {
    case 1: DQ_PASS(9, 1) break;
    case 2: DQ_PASS(9, 2) break;
    case 3: DQ_PASS(9, 3) break;
    case 4: DQ_PASS(9, 4) break;
    case 5: DQ_PASS(9, 5) break;
    case 6: DQ_PASS(9, 3) DQ_PASS(12, 3) break;
    default: break;
    }
#undef DQ_PASS
    if (a.vec) {
        for (int i = tid * 4; i < tile; i += nthreads * 4) {
            const int64_t g = origin + ((int64_t)(i >> 5) << sbits) + (i & 31);
            const int q = pad_idx(i);
            store4<ENDS>(x, make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]), a, e, sign_mode, apply_scale, g);
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + ((int64_t)(i >> 5) << sbits) + (i & 31);
            float v = lds[pad_idx(i)];
            if (apply_scale) v *= a.scale;
            x[g] = sign_mode == 2 ? flip1(v, a, g) : v;
        }
    }
}

// ---- blocks of 2^15: the tile in two halves -----------------------------------------------------------
//
// A 2^15 tile with its padding needs 135 KB of LDS: one workgroup per CU, whose load, butterfly and
// quantise phases cannot overlap with a neighbour's.  Here thread t owns chunk t of both halves of the
// block: the stages of strides 1..8 run on registers, the stages of strides 16 .. 2^13 run in LDS one half
// after the other (68 KB: two workgroups per CU), and the last stage (stride 2^14) pairs the thread's own
// two chunks.  In the inverse kernel and the plain transform the record windows (and the MEE table) share the
// LDS with the tile: they are used only before the first half enters it or after the second has left.  The
// forward kernel keeps its second half in the LDS through the pairing stage and the quantiser of the first
// (see rht_compress_split_kernel).  All of them ask for eight waves per SIMD (64 registers): two resident
// workgroups are worth more than anything the register file could hold instead.
constexpr int kSplitBits = 15, kHalfBits = 14, kSplitThreads = 1024;

// stages of strides 16 .. 2^13 of the half block whose chunk t the thread holds in v (in and out)
template <int HB = kHalfBits>
__device__ __forceinline__ void half_block_stages(float (&v)[16], float *lds, int tid)
{
    float *mine = lds + chunk_word(tid);
#pragma unroll
    for (int i = 0; i < 16; i++) mine[i] = v[i];
    fwht_lds_stages_after4(lds, HB, HB, tid, 1 << (HB - 4));
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = mine[i];
    __syncthreads(); // the half has left the LDS
}

// The forward kernel takes blocks of 2^(HB + 1) in two halves of 2^HB, one chunk of each half per thread: HB = 14 for
// blocks of 2^15 (1024 threads; a CU holds at most two such workgroups), HB = 13 for blocks of 2^14 (512 threads, up to
// four per CU; as one tile those blocks need 1024 threads of which half sit idle in both LDS passes), ... HB = 10 for
// blocks of 2^11 on one wave.
//
// LDS: the half tile, in which the second half is parked through the quantiser of the first, and the record windows of
// the waves behind it.  For HB = 14 the sum must leave room for two workgroups per CU (80 KB each).
// records per window: four (one run per wave) where two workgroups of 2^15-element blocks still fit a CU with the parked half,
// two for the wider codes (7 and 8 bits), whose runs then leave in two pieces
template <int NBITS, int HB> __host__ __device__ constexpr int split_window_rows()
{
    return HB < kHalfBits || (size_t)padded_tile_floats(HB) * sizeof(float) + ((1 << (HB - 4)) / 64) * window_bytes<NBITS>(4) <= 80 * 1024 ? 4 : 2;
}
template <int NBITS, int HB> __host__ __device__ constexpr size_t split_lds_bytes()
{
    return (size_t)padded_tile_floats(HB) * sizeof(float) + ((1 << (HB - 4)) / 64) * window_bytes<NBITS>(split_window_rows<NBITS, HB>());
}

// PAIR = false: the two halves are two whole blocks of 2^HB (no pairing stage): blocks of 2^10 on one wave.
template <int RDT, int NBITS, bool MEE, int HB, bool PAIR = true>
__global__ __launch_bounds__(1 << (HB - 4), 8) void rht_compress_split_kernel(
    const float *__restrict__ x, uint8_t *__restrict__ dst, const void *__restrict__ rnd, RhtTileArgs a, int rvec, RandKey key,
    MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    constexpr int kThreads = 1 << (HB - 4), kWaves = kThreads / 64;
    constexpr int kWinRows = split_window_rows<NBITS, HB>();
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t origin = (int64_t)blockIdx.x << (HB + 1);
    float va[16], vb[16];
    load_chunk(va, x, a, origin + tid * 16);
    load_chunk(vb, x, a, origin + (1 << HB) + tid * 16);
    butterflies<4>(va);
    butterflies<4>(vb);
    half_block_stages<HB>(va, lds, tid);
    // The second half stays in the LDS after its stages: the thread pairs its two chunks there, keeps the sums and
    // leaves the differences in its own slot until the sums are quantised.  With both halves in registers through the
    // quantiser the kernel needs more than its 64 registers, and what it spills travels to memory and back (measured
    // at 2^28 elements in blocks of 2^15: 757 MB written and 1.52 GB read for 153 MB of records and 1.11 GB of input).
    // The record windows then lie behind the tile instead of inside it.
    float *mine = lds + chunk_word(tid);
#pragma unroll
    for (int i = 0; i < 16; i++) mine[i] = vb[i];
    fwht_lds_stages_after4(lds, HB, HB, tid, kThreads); // ends with a barrier; own slot only from here on
    if constexpr (PAIR) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float p = va[i], q = mine[i];
            va[i] = p + q;
            mine[i] = p - q;
        }
    }
    uint8_t *win_out = reinterpret_cast<uint8_t *>(lds + padded_tile_floats(HB)) + wave * window_bytes<NBITS>(kWinRows);
    // quantise: the wave's 64 chunks of a half are 4 superchunks, one run of records
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int64_t sc0 = (origin >> 8) + h * (kWaves * kRowsPerWave) + wave * kRowsPerWave;
        Raw16<DQ_F32> v;
        Raw16<RDT> r;
        if constexpr (RDT == DQ_PHILOX)
            r.generate(key, sc0 * 16 + lane);
        else
            r.load(rnd, (sc0 * 16 + lane) * 16, rvec);
#pragma unroll
        for (int i = 0; i < 16; i++) v.w[i] = __float_as_uint((h ? mine[i] : va[i]) * a.scale);
        encode_store_run<NBITS, MEE, kWinRows, false>(v, r, mp, dst + sc0 * RC::REC, kRowsPerWave, win_out, threadIdx.x & 63);
        wave_lds_sync(); // the window is reused for the other half
    }
}

// the inverse: blocks of 2^(HB + 1) in two halves (PAIR), or two blocks of 2^HB per workgroup (PAIR = false)
template <int NBITS, bool MEE, int HB, bool PAIR = true>
__global__ __launch_bounds__(1 << (HB - 4), 8) void irht_decompress_split_kernel(const uint8_t *__restrict__ src,
                                                                             float *__restrict__ x, RhtTileArgs a,
                                                                             MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    constexpr int kThreads = 1 << (HB - 4), kWaves = kThreads / 64;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane >> 4, j = lane & 15;
    const int64_t origin = (int64_t)blockIdx.x << (HB + 1);
    uint8_t *win_in = reinterpret_cast<uint8_t *>(lds) + wave * RC::WIN;
    float *table = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(lds) + kWaves * RC::WIN);
    if (MEE) {
        for (int k = tid; k < (1 << NBITS); k += kThreads) table[k] = f16_bits_to_f32(mp.table[k]);
        __syncthreads();
    }
    float va[16], vb[16];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int64_t sc0 = (origin >> 8) + h * (kWaves * kRowsPerWave) + wave * kRowsPerWave;
        const int total = kRowsPerWave * RC::REC;
        const uint8_t *g = src + sc0 * RC::REC;
        const WinRegs wr = window_fetch(g, total, lane);
        const int mis = window_commit(win_in, wr, g, total, lane);
        wave_lds_sync();
        const uint8_t *rec = win_in + mis + row * RC::REC;
        uint32_t cw[RC::WORDS], cq;
        chunk_read<NBITS>(rec + j * RC::CB, cw, cq);
        const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
        float t[16];
        chunk_decode<NBITS, MEE, false>(cw, cq, ub, table, t);
#pragma unroll
        for (int i = 0; i < 16; i++) (h ? vb[i] : va[i]) = t[i];
        wave_lds_sync(); // the window is reused for the other half
    }
    __syncthreads(); // windows and table are done with: the tile takes the LDS
    butterflies<4>(va);
    butterflies<4>(vb);
    half_block_stages<HB>(va, lds, tid);
    half_block_stages<HB>(vb, lds, tid);
    if constexpr (PAIR) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float p = va[i], q = vb[i];
            va[i] = p + q;
            vb[i] = p - q;
        }
    }
    // store one half after the other through the LDS, so that every store instruction covers 1 KiB contiguously
    float *mine = lds + chunk_word(tid);
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int i = 0; i < 16; i++) mine[i] = h ? vb[i] : va[i];
        __syncthreads();
        const int64_t half_origin = origin + ((int64_t)h << HB);
        if (a.vec) {
            for (int i = tid * 4; i < (1 << HB); i += kThreads * 4) {
                const int q = pad_idx(i);
                float4 v = make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]);
                v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale;
                flip4(v, a, half_origin + i);
                stream_store(reinterpret_cast<float4 *>(x + half_origin + i), v);
            }
        } else {
            for (int i = tid; i < (1 << HB); i += kThreads)
                x[half_origin + i] = flip1(lds[pad_idx(i)] * a.scale, a, half_origin + i);
        }
        __syncthreads();
    }
}

// the transform alone on blocks of 2^15, the tile in two halves as above
__global__ __launch_bounds__(kSplitThreads, 8) void rht_tile_split_kernel(float *__restrict__ x, RhtTileArgs a, int sign_mode,
                                                                      int apply_scale)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x;
    const int64_t origin = (int64_t)blockIdx.x << kSplitBits;
    RhtTileArgs in = a;
    if (sign_mode != 1) in.sign = nullptr;
    float va[16], vb[16];
    load_chunk(va, x, in, origin + tid * 16);
    load_chunk(vb, x, in, origin + (1 << kHalfBits) + tid * 16);
    butterflies<4>(va);
    butterflies<4>(vb);
    half_block_stages(va, lds, tid);
    half_block_stages(vb, lds, tid);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float p = va[i], q = vb[i];
        va[i] = p + q;
        vb[i] = p - q;
    }
    // store one half after the other through the LDS, so that every store instruction covers 1 KiB contiguously
    float *mine = lds + chunk_word(tid);
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int i = 0; i < 16; i++) mine[i] = h ? vb[i] : va[i];
        __syncthreads();
        const int64_t half_origin = origin + ((int64_t)h << kHalfBits);
        if (a.vec) {
            for (int i = tid * 4; i < (1 << kHalfBits); i += kSplitThreads * 4) {
                const int q = pad_idx(i);
                float4 v = make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]);
                if (apply_scale) { v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale; }
                if (sign_mode == 2) flip4(v, a, half_origin + i);
                *reinterpret_cast<float4 *>(x + half_origin + i) = v;
            }
        } else {
            for (int i = tid; i < (1 << kHalfBits); i += kSplitThreads) {
                float v = lds[pad_idx(i)];
                if (apply_scale) v *= a.scale;
                x[half_origin + i] = sign_mode == 2 ? flip1(v, a, half_origin + i) : v;
            }
        }
        __syncthreads();
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
    if (g.a.kb == 10 && (n & 2047) == 0) {
        // blocks of 2^10, two per wave
        auto kernel = rht_compress_split_kernel<RDT, NBITS, MEE, 10, false>;
        const size_t lds = split_lds_bytes<NBITS, 10>();
        hipLaunchKernelGGL(kernel, dim3((unsigned)(n >> 11)), dim3(64), lds, stream, src, dst, rnd, g.a, aligned16(rnd) ? 1 : 0, key,
                           make_arg<NBITS, MEE>(mp));
        return hipGetLastError();
    }
    if (g.a.kb >= kSplitBits - 4 && g.a.kb <= kSplitBits && (n & ((1 << g.a.kb) - 1)) == 0) {
        // blocks of 2^11 .. 2^15: two halves per workgroup
        auto launch = [&](auto kernel, size_t lds, int half_bits) -> hipError_t {
            hipError_t es = allow_lds(kernel, lds);
            if (es != hipSuccess) return es;
            hipLaunchKernelGGL(kernel, dim3((unsigned)(n >> (half_bits + 1))), dim3(1 << (half_bits - 4)), lds, stream, src, dst, rnd,
                               g.a, aligned16(rnd) ? 1 : 0, key, make_arg<NBITS, MEE>(mp));
            return hipGetLastError();
        };
        switch (g.a.kb) {
        case kSplitBits:
            return launch(rht_compress_split_kernel<RDT, NBITS, MEE, kHalfBits>, split_lds_bytes<NBITS, kHalfBits>(), kHalfBits);
        case kSplitBits - 1:
            return launch(rht_compress_split_kernel<RDT, NBITS, MEE, kHalfBits - 1>, split_lds_bytes<NBITS, kHalfBits - 1>(), kHalfBits - 1);
        case kSplitBits - 2:
            return launch(rht_compress_split_kernel<RDT, NBITS, MEE, kHalfBits - 2>, split_lds_bytes<NBITS, kHalfBits - 2>(), kHalfBits - 2);
        case kSplitBits - 3:
            return launch(rht_compress_split_kernel<RDT, NBITS, MEE, kHalfBits - 3>, split_lds_bytes<NBITS, kHalfBits - 3>(), kHalfBits - 3);
        default:
            return launch(rht_compress_split_kernel<RDT, NBITS, MEE, kHalfBits - 4>, split_lds_bytes<NBITS, kHalfBits - 4>(), kHalfBits - 4);
        }
    }
    if (g.a.kt >= kSplitBits) return hipErrorInvalidValue; // one run of records per wave needs tiles of at most 2^14
    const size_t windows = (size_t)(g.threads / 64) * Rec<NBITS>::WIN;
    const size_t lds = std::max(g.lds_floats * sizeof(float), windows);
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
    if (g.a.kb >= 10 && g.a.kb <= kSplitBits && (n & ((g.a.kb == 10 ? 2048 : (1 << g.a.kb)) - 1)) == 0) {
        // blocks of 2^11 .. 2^15 in two halves per workgroup, blocks of 2^10 two per wave
        auto launch = [&](auto kernel, int half_bits) -> hipError_t {
            const size_t tile = (size_t)padded_tile_floats(half_bits) * sizeof(float);
            const size_t windows = (size_t)((1 << (half_bits - 4)) / 64) * Rec<NBITS>::WIN + (MEE ? (sizeof(float) << NBITS) : 0);
            const size_t lds = std::max(tile, windows);
            hipError_t es = allow_lds(kernel, lds);
            if (es != hipSuccess) return es;
            hipLaunchKernelGGL(kernel, dim3((unsigned)(n >> (half_bits + 1))), dim3(1 << (half_bits - 4)), lds, stream, src, dst, g.a,
                               make_arg<NBITS, MEE>(mp));
            return hipGetLastError();
        };
        switch (g.a.kb) {
        case 15: return launch(irht_decompress_split_kernel<NBITS, MEE, 14>, 14);
        case 14: return launch(irht_decompress_split_kernel<NBITS, MEE, 13>, 13);
        case 13: return launch(irht_decompress_split_kernel<NBITS, MEE, 12>, 12);
        case 12: return launch(irht_decompress_split_kernel<NBITS, MEE, 11>, 11);
        case 11: return launch(irht_decompress_split_kernel<NBITS, MEE, 10>, 10);
        default: return launch(irht_decompress_split_kernel<NBITS, MEE, 10, false>, 10);
        }
    }
    if (g.a.kt >= kSplitBits) return hipErrorInvalidValue;
    const size_t windows = (size_t)(g.threads / 64) * Rec<NBITS>::WIN + (MEE ? (sizeof(float) << NBITS) : 0);
    const size_t lds = std::max(g.lds_floats * sizeof(float), windows);
    auto kernel = irht_decompress_kernel<NBITS, MEE>;
    hipError_t e = allow_lds(kernel, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(g.grid), dim3(g.threads), lds, stream, src, dst, g.a, make_arg<NBITS, MEE>(mp));
    return hipGetLastError();
}

} // namespace

// one entry point per rounding source, each in a translation unit of its own
hipError_t launch_rht_compress_philox(const float *src, const void *sign, int sign_bits, uint8_t *dst, int64_t n, int64_t block, float scale,
                                      int nbits, bool mee, const MeeParams &mp, RandKey key, hipStream_t stream);
hipError_t launch_rht_compress_bf16_pool(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int64_t n,
                                         int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, hipStream_t stream);
hipError_t launch_rht_compress_f32_pool(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int64_t n,
                                        int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, hipStream_t stream);

#if DQ_RHT_PART & DQ_RHT_COMPRESS_PHILOX
hipError_t launch_rht_compress_philox(const float *src, const void *sign, int sign_bits, uint8_t *dst, int64_t n, int64_t block, float scale,
                                      int nbits, bool mee, const MeeParams &mp, RandKey key, hipStream_t stream)
{
    DQ_NBITS_MEE(run_compress, DQ_PHILOX, src, sign, sign_bits, dst, nullptr, n, block, scale, mp, key, stream)
}
#endif

#if DQ_RHT_PART & DQ_RHT_COMPRESS_BF16
hipError_t launch_rht_compress_bf16_pool(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int64_t n,
                                         int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, hipStream_t stream)
{
    const RandKey key{0, 0};
    DQ_NBITS_MEE(run_compress, DQ_BF16, src, sign, sign_bits, dst, rnd, n, block, scale, mp, key, stream)
}
#endif

#if DQ_RHT_PART & DQ_RHT_COMPRESS_F32
hipError_t launch_rht_compress_f32_pool(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int64_t n,
                                        int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, hipStream_t stream)
{
    const RandKey key{0, 0};
    DQ_NBITS_MEE(run_compress, DQ_F32, src, sign, sign_bits, dst, rnd, n, block, scale, mp, key, stream)
}
#endif

#if DQ_RHT_PART & DQ_RHT_TRANSFORM
// rand_kind: DQ_F32 or DQ_BF16 pool, or DQ_PHILOX (rnd ignored)
hipError_t launch_rht_compress(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int rand_kind, int64_t n,
                               int64_t block, float scale, int nbits, bool mee, const MeeParams &mp, uint64_t seed,
                               uint64_t step, hipStream_t stream)
{
    if (rand_kind == DQ_PHILOX)
        return launch_rht_compress_philox(src, sign, sign_bits, dst, n, block, scale, nbits, mee, mp, RandKey{seed, step}, stream);
    if (rand_kind == DQ_BF16) return launch_rht_compress_bf16_pool(src, sign, sign_bits, dst, rnd, n, block, scale, nbits, mee, mp, stream);
    return launch_rht_compress_f32_pool(src, sign, sign_bits, dst, rnd, n, block, scale, nbits, mee, mp, stream);
}

// the 4-bit AEE kernel with the in-kernel rounding stream and the first four stages on the matrix cores (measurement variant)
hipError_t launch_rht_compress_mfma16(const float *src, const void *sign, int sign_bits, uint8_t *dst, int64_t n, int64_t block,
                                      float scale, const MeeParams &mp, uint64_t seed, uint64_t step, hipStream_t stream)
{
    const Geometry g = geometry(src, sign, sign_bits, n, block, scale);
    if (g.a.kb < 4 || g.a.kb >= kSplitBits || g.a.kt >= kSplitBits || g.a.kt < 10 || !g.a.vec || (n & ((1 << g.a.kt) - 1)) != 0 || (g.threads & 63) != 0)
        return hipErrorInvalidValue;
    const size_t windows = (size_t)(g.threads / 64) * Rec<4>::WIN;
    const size_t lds = std::max(g.lds_floats * sizeof(float), windows);
    auto kernel = rht_compress_kernel<DQ_PHILOX, 4, false, true>;
    hipError_t e = allow_lds(kernel, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(g.grid), dim3(g.threads), lds, stream, src, dst, nullptr, g.a, 0, RandKey{seed, step},
                       make_arg<4, false>(mp));
    return hipGetLastError();
}

#endif // DQ_RHT_TRANSFORM (first part)

#if DQ_RHT_PART & DQ_RHT_DECOMPRESS
hipError_t launch_irht_decompress(const uint8_t *src, const void *sign, int sign_bits, float *dst, int64_t n, int64_t block, float scale,
                                  int nbits, bool mee, const MeeParams &mp, hipStream_t stream)
{
    DQ_NBITS_MEE(run_decompress, 0, src, sign, sign_bits, dst, n, block, scale, mp, stream)
}
#endif

#if DQ_RHT_PART & DQ_RHT_TRANSFORM

// stages [0, kb) of every aligned block of 2^kb elements, tiles of 2^kt contiguous elements (10 <= kt <= 15, kb <= kt);
// vec: 16-byte accesses to x (and to a float sign vector) are allowed; ends: needs vec, n a multiple of 32 and 16-byte
// aligned levels
hipError_t launch_rht_tile(float *x, const void *sign, int sign_bits, int64_t n, int kt, int kb, float scale, int apply_scale,
                           int sign_mode, int vec, const TransformEnds &ends, hipStream_t stream)
{
    if (kt < 10 || kt > 15 || kb > kt || kb < 0) return hipErrorInvalidValue;
    const bool plain = !ends.in_levels && !ends.in_planes && !ends.out_levels && !ends.post_scale;
    if (!plain && (!vec || (n & 31) != 0)) return hipErrorInvalidValue;
    RhtTileArgs a;
    a.sign = sign; a.sign_bits = sign_bits; a.n = n; a.kt = kt; a.kb = kb; a.scale = scale; a.vec = vec;
    const int tile = 1 << kt;
    if (plain && kt == kSplitBits && kb == kSplitBits && (n & (tile - 1)) == 0) {
        // whole blocks of 2^15: half the LDS, two workgroups per CU
        const size_t half_lds = (size_t)padded_tile_floats(kHalfBits) * sizeof(float);
        hipError_t es = allow_lds(rht_tile_split_kernel, half_lds);
        if (es != hipSuccess) return es;
        hipLaunchKernelGGL(rht_tile_split_kernel, dim3((unsigned)(n >> kSplitBits)), dim3(kSplitThreads), half_lds, stream, x, a,
                           sign ? sign_mode : 0, apply_scale);
        return hipGetLastError();
    }
    const unsigned threads = (unsigned)std::min(1024, tile / 16);
    const size_t lds = ((size_t)padded_tile_floats(kt) + (ends.in_planes ? 256 : 0)) * sizeof(float);
    const dim3 grid((unsigned)((n + tile - 1) >> kt));
    if (plain) {
        hipError_t e = allow_lds(rht_tile_kernel<false>, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(rht_tile_kernel<false>, grid, dim3(threads), lds, stream, x, a, sign ? sign_mode : 0, apply_scale, ends);
    } else {
        hipError_t e = allow_lds(rht_tile_kernel<true>, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(rht_tile_kernel<true>, grid, dim3(threads), lds, stream, x, a, sign ? sign_mode : 0, apply_scale, ends);
    }
    return hipGetLastError();
}

// stages of the index bits [sbits, sbits + rbits) of x[0 .. n), n a multiple of 2^(sbits + rbits); 4 <= rbits <= 10, sbits >= 5
hipError_t launch_rht_strided(float *x, const void *sign, int sign_bits, int64_t n, int rbits, int sbits, float scale,
                              int apply_scale, int sign_mode, int vec, const TransformEnds &ends, hipStream_t stream)
{
    if (rbits < 4 || rbits > 10 || sbits < 5 || (n & (((int64_t)1 << (sbits + rbits)) - 1)) != 0) return hipErrorInvalidValue;
    const bool plain = !ends.out_levels && !ends.post_scale;
    if (!plain && !vec) return hipErrorInvalidValue;
    RhtTileArgs a;
    a.sign = sign; a.sign_bits = sign_bits; a.n = n; a.kt = rbits + 5; a.kb = 0; a.scale = scale; a.vec = vec;
    const int tile = 1 << (rbits + 5);
    const unsigned threads = (unsigned)std::min(1024, tile / 16);
    const size_t lds = (size_t)padded_tile_floats(rbits + 5) * sizeof(float);
    const dim3 grid((unsigned)(n >> (rbits + 5)));
    if (plain) {
        hipError_t e = allow_lds(rht_strided_kernel<false>, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(rht_strided_kernel<false>, grid, dim3(threads), lds, stream, x, a, rbits, sbits, sign ? sign_mode : 0,
                           apply_scale, ends);
    } else {
        hipError_t e = allow_lds(rht_strided_kernel<true>, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(rht_strided_kernel<true>, grid, dim3(threads), lds, stream, x, a, rbits, sbits, sign ? sign_mode : 0,
                           apply_scale, ends);
    }
    return hipGetLastError();
}

#endif // DQ_RHT_TRANSFORM

} // namespace dq
