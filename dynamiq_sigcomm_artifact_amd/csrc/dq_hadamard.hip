// Fast Walsh-Hadamard transform (unnormalised, Sylvester order) and the blocked
// randomized transform built on it.
//
// A pass: a workgroup owns a tile of 2^kt floats in LDS and applies the butterfly
// stages of a contiguous range of index bits to it.
//   * contiguous pass: the tile is 2^kt consecutive floats and the stages are
//     strides 1 .. 2^(kt-1) (or fewer when the transform block is smaller than
//     the tile, so several small blocks share one tile);
//   * strided pass (vectors longer than one tile): the tile is 2^r "rows" of
//     2^c consecutive floats taken at stride 2^s, and the stages are the row
//     bits, i.e. strides 2^s .. 2^(s+r-1) of the vector.
// A whole-vector transform of n = 2^k is one contiguous pass plus
// ceil((k-kt)/r) strided passes; each pass is one read and one write of the
// vector.  Stages always run in ascending stride with butterflies (a+b, a-b),
// which is the order of csrc/cuda_hadamard.cu:66-157,205-274,534-605, so the
// result is bit-identical to a plain stage-by-stage FWHT.
//
// This file plans the passes.  Passes of at least 1024 elements go to the kernels of
// dq_rht_scaling_impl.cuh, which do the first four stages on the registers a lane loads
// into and need fewer LDS passes; the kernel here, fwht_tile_kernel, does the stages
// of a tile four at a time (radix 16) between LDS and registers and serves what is
// left: small tiles, strided passes over fewer than four bits, buffers without
// 16-byte alignment.  Either kind can take a quantiser at the ends of the transform
// (THC's levels, EDEN's bit planes and scale).  The LDS index is
// padded by one float per 32 (dq_fwht.cuh).
#include "dq_fwht.cuh"
#include "dq_launch.h"

namespace dq {

struct FwhtArgs {
    float *x;
    const float *sign;         // +-1 values, or null
    const uint32_t *sign_bits; // or: one bit per element, set where the sign is negative (dq_pack_signs)
    int64_t n;         // elements in the vector (for bounds of ragged tiles)
    int kt;            // log2 tile elements
    int b0, b1;        // tile-index bits to transform: [b0, b1)
    int cbits;         // low cbits of the tile index are contiguous in memory
    int sbits;         // vector stride of a tile row is 2^sbits (== cbits for a contiguous tile)
    float scale;
    int apply_scale;
    int sign_mode;     // 0 none, 1 multiply on load, 2 multiply on store
    int vec;           // 16-byte accesses allowed
    // THC's quantiser folded into the two ends of a transform (all null / unused otherwise):
    const uint16_t *in_levels; // the pass loads float(level) * *in_step + *in_lo instead of x
    const float *in_step, *in_lo;
    uint16_t *out_levels;      // the pass stores thc_level(value, uniform) as bf16 instead of the value
    const float *uniform, *out_lo, *out_delta;
    float out_top;
    // EDEN's dequantiser folded into the ends of an inverse transform (null / unused otherwise):
    const uint32_t *in_planes; // the pass loads centroids[bin] from the bit planes of the bins instead of x
    const float *in_centroids; // 2^in_nbits values
    int64_t in_words;          // words per plane (n / 32)
    int in_nbits;
    const float *post_scale;   // the last pass multiplies by *post_scale after scale and sign
};

// the diagonal of +-1 on four consecutive elements from g (a multiple of 4) / on element g: a multiplication by
// the float value, or a flip of the sign bit where the packed bit is set (the same thing for +-1)
__device__ __forceinline__ void apply_sign4(const FwhtArgs &a, float4 &v, int64_t g)
{
    if (a.sign_bits) {
        const uint32_t w = a.sign_bits[g >> 5] >> (g & 31);
        v.x = __uint_as_float(__float_as_uint(v.x) ^ ((w & 1u) << 31));
        v.y = __uint_as_float(__float_as_uint(v.y) ^ ((w & 2u) << 30));
        v.z = __uint_as_float(__float_as_uint(v.z) ^ ((w & 4u) << 29));
        v.w = __uint_as_float(__float_as_uint(v.w) ^ ((w & 8u) << 28));
    } else {
        const float4 s = *reinterpret_cast<const float4 *>(a.sign + g);
        v.x *= s.x; v.y *= s.y; v.z *= s.z; v.w *= s.w;
    }
}

__device__ __forceinline__ float apply_sign1(const FwhtArgs &a, float v, int64_t g)
{
    if (a.sign_bits) return __uint_as_float(__float_as_uint(v) ^ (((a.sign_bits[g >> 5] >> (g & 31)) & 1u) << 31));
    return v * a.sign[g];
}

__global__ void fwht_tile_kernel(FwhtArgs a)
{
    extern __shared__ float lds[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int tile = 1 << a.kt;
    const int cmask = (1 << a.cbits) - 1;
    const int rbits = a.kt - a.cbits;

    // tile -> position in the vector.  A contiguous tile (sbits == cbits) starts
    // at blockIdx * 2^kt.  A strided tile covers rows rho = 0..2^rbits-1 at
    // stride 2^sbits and columns [mid*2^cbits, +2^cbits):
    //   index = hi * 2^(sbits+rbits) + rho * 2^sbits + mid * 2^cbits + col
    int64_t origin;
    if (a.sbits == a.cbits) {
        origin = (int64_t)blockIdx.x << a.kt;
    } else {
        // (shift and mask, not quotient and remainder: see rht_strided_kernel)
        const int mbits = a.sbits - a.cbits;
        const int64_t hi = (int64_t)(blockIdx.x >> mbits), mid = (int64_t)(blockIdx.x & ((1u << mbits) - 1u));
        origin = (hi << (a.sbits + rbits)) + (mid << a.cbits);
    }

    // load (coalesced), optional sign flip
    if (a.in_planes) {
        // sixteen consecutive bins per thread from its half word of every plane (two 8 x 8 bit transposes), their
        // centroids into one padded group of the tile; the centroid table sits behind the tile
        float *cen = lds + padded_floats(tile);
        for (int k = tid; k < (1 << a.in_nbits); k += nthreads) cen[k] = a.in_centroids[k];
        __syncthreads();
        for (int i = tid * 16; i < tile; i += nthreads * 16) {
            const int64_t g = origin + i; // the first pass works on contiguous tiles
            uint64_t lo8 = 0, hi8 = 0;
            if (g < a.n) {
                const uint16_t *half = reinterpret_cast<const uint16_t *>(a.in_planes) + (g >> 4);
                for (int p = 0; p < a.in_nbits; p++) {
                    const uint32_t h = half[(int64_t)p * a.in_words * 2];
                    lo8 |= (uint64_t)(h & 0xffu) << (8 * p);
                    hi8 |= (uint64_t)(h >> 8) << (8 * p);
                }
                lo8 = transpose8x8(lo8);
                hi8 = transpose8x8(hi8);
            }
            const int q = pad_idx(i);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                lds[q + k] = g < a.n ? cen[(lo8 >> (8 * k)) & 0xffu] : 0.0f;
                lds[q + 8 + k] = g < a.n ? cen[(hi8 >> (8 * k)) & 0xffu] : 0.0f;
            }
        }
    } else if (a.vec) {
        for (int i = tid * 4; i < tile; i += nthreads * 4) {
            const int64_t g = origin + ((int64_t)(i >> a.cbits) << a.sbits) + (i & cmask);
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (g < a.n) {
                if (a.in_levels) {
                    const uint2 l = *reinterpret_cast<const uint2 *>(a.in_levels + g);
                    const float step = *a.in_step, lo = *a.in_lo;
                    const float p0 = bf16_bits_to_f32(l.x & 0xffffu) * step, p1 = bf16_bits_to_f32(l.x >> 16) * step;
                    const float p2 = bf16_bits_to_f32(l.y & 0xffffu) * step, p3 = bf16_bits_to_f32(l.y >> 16) * step;
                    v = make_float4(p0 + lo, p1 + lo, p2 + lo, p3 + lo);
                } else {
                    v = *reinterpret_cast<const float4 *>(a.x + g);
                }
                if (a.sign_mode == 1) apply_sign4(a, v, g);
            }
            const int q = pad_idx(i); // i % 4 == 0: the four floats stay inside one padded group
            lds[q] = v.x; lds[q + 1] = v.y; lds[q + 2] = v.z; lds[q + 3] = v.w;
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + ((int64_t)(i >> a.cbits) << a.sbits) + (i & cmask);
            float v = 0.0f;
            if (g < a.n) {
                if (a.in_levels) {
                    const float prod = bf16_bits_to_f32(a.in_levels[g]) * *a.in_step;
                    v = prod + *a.in_lo;
                } else {
                    v = a.x[g];
                }
                if (a.sign_mode == 1) v = apply_sign1(a, v, g);
            }
            lds[pad_idx(i)] = v;
        }
    }
    __syncthreads();

    // butterfly stages, four index bits at a time
    fwht_lds_stages(lds, a.kt, a.b0, a.b1, tid, nthreads);

    // store (coalesced), optional scale then sign flip
    if (a.vec) {
        for (int i = tid * 4; i < tile; i += nthreads * 4) {
            const int64_t g = origin + ((int64_t)(i >> a.cbits) << a.sbits) + (i & cmask);
            if (g >= a.n) continue;
            const int q = pad_idx(i);
            float4 v = make_float4(lds[q], lds[q + 1], lds[q + 2], lds[q + 3]);
            if (a.apply_scale) { v.x *= a.scale; v.y *= a.scale; v.z *= a.scale; v.w *= a.scale; }
            if (a.sign_mode == 2) apply_sign4(a, v, g);
            if (a.post_scale) {
                const float ps = *a.post_scale;
                v.x *= ps; v.y *= ps; v.z *= ps; v.w *= ps;
            }
            if (a.out_levels) {
                const float4 u = *reinterpret_cast<const float4 *>(a.uniform + g);
                const float lo = *a.out_lo, delta = *a.out_delta;
                uint2 o;
                o.x = f32x2_to_bf16x2(thc_level(v.x, u.x, lo, delta, a.out_top), thc_level(v.y, u.y, lo, delta, a.out_top));
                o.y = f32x2_to_bf16x2(thc_level(v.z, u.z, lo, delta, a.out_top), thc_level(v.w, u.w, lo, delta, a.out_top));
                *reinterpret_cast<uint2 *>(a.out_levels + g) = o;
            } else {
                *reinterpret_cast<float4 *>(a.x + g) = v;
            }
        }
    } else {
        for (int i = tid; i < tile; i += nthreads) {
            const int64_t g = origin + ((int64_t)(i >> a.cbits) << a.sbits) + (i & cmask);
            if (g >= a.n) continue;
            float v = lds[pad_idx(i)];
            if (a.apply_scale) v *= a.scale;
            if (a.sign_mode == 2) v = apply_sign1(a, v, g);
            if (a.post_scale) v *= *a.post_scale;
            if (a.out_levels)
                a.out_levels[g] = (uint16_t)f32_to_bf16_bits(thc_level(v, a.uniform[g], *a.out_lo, *a.out_delta, a.out_top));
            else
                a.x[g] = v;
        }
    }
}

static hipError_t launch_tile(const FwhtArgs &a, int64_t ntiles, hipStream_t stream)
{
    const int tile = 1 << a.kt;
    int threads = tile / 16;
    threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
    const size_t lds_bytes = (size_t)(padded_floats(tile) + (a.in_planes ? 256 : 0)) * sizeof(float);
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(fwht_tile_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(fwht_tile_kernel, dim3((unsigned)ntiles), dim3(threads), lds_bytes, stream, a);
    return hipGetLastError();
}

constexpr int kMaxTileBits = 15; // 2^15 floats = 128 KiB (+ padding) of the 160 KiB LDS
constexpr int kPrefTileBits = 13; // 32 KiB tiles keep several workgroups per CU in flight
constexpr int kStridedCols = 5;   // 32 consecutive floats (128 B) per row of a strided tile

// transform index bits [0, kb) of every aligned block of 2^kb elements of x[0..n); `thc`: quantisers at the ends
typedef TransformEnds ThcEnds;

// sign: float +-1 values, or (sign_packed) the bit vector of dq_pack_signs; may be null
static hipError_t fwht_blocks(float *x, const void *sign, bool sign_packed, int64_t n, int kb, float scale, int apply_scale,
                              int inverse, hipStream_t stream, const ThcEnds &thc = ThcEnds())
{
    const bool vec16 = (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                       (sign == nullptr || sign_packed || (reinterpret_cast<uintptr_t>(sign) & 15) == 0) &&
                       (reinterpret_cast<uintptr_t>(thc.in_levels) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(thc.out_levels) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(thc.uniform) & 15) == 0;
    FwhtArgs a;
    a.x = x; a.n = n; a.scale = scale;
    a.sign = sign_packed ? nullptr : static_cast<const float *>(sign);
    a.sign_bits = sign_packed ? static_cast<const uint32_t *>(sign) : nullptr;
    a.in_levels = nullptr; a.in_step = thc.in_step; a.in_lo = thc.in_lo;
    a.in_planes = nullptr; a.in_centroids = thc.in_centroids; a.in_words = n >> 5; a.in_nbits = thc.in_nbits;
    a.post_scale = nullptr;
    a.out_levels = nullptr; a.uniform = thc.uniform; a.out_lo = thc.out_lo; a.out_delta = thc.out_delta;
    a.out_top = thc.out_top;
    const int sign_fwd = (sign && !inverse) ? 1 : 0, sign_inv = (sign && inverse) ? 2 : 0;
    // Passes of at least 1024 elements run as the chunk-first kernels of dq_rht_scaling_impl.cuh; a quantiser at an end needs
    // the 16-byte paths there
    const bool plain = !thc.in_levels && !thc.in_planes && !thc.out_levels && !thc.post_scale;
    const bool ends_ok = plain || (vec16 && (n & 31) == 0 && (reinterpret_cast<uintptr_t>(thc.in_levels) & 15) == 0);
    TransformEnds first = thc, last = thc, none;
    first.out_levels = nullptr; first.post_scale = nullptr;
    last.in_levels = nullptr; last.in_planes = nullptr;

    if (kb <= kMaxTileBits) {
        // single pass; small blocks share a tile
        int kt = kb < kPrefTileBits ? kPrefTileBits : kb;
        while (kt > kb && kt > 10 && (n >> kt) < 512) kt--; // short vectors: two workgroups per CU before larger tiles
        while (kt > kb && ((int64_t)1 << kt) > n) kt--;
        a.kt = kt; a.b0 = 0; a.b1 = kb; a.cbits = kt; a.sbits = kt;
        a.apply_scale = apply_scale; a.sign_mode = sign_fwd | sign_inv;
        a.vec = vec16 && kt >= 2 && (n & 3) == 0;
        a.in_levels = thc.in_levels;
        a.out_levels = thc.out_levels;
        a.in_planes = thc.in_planes;
        a.post_scale = thc.post_scale;
        const int64_t ntiles = (n + ((int64_t)1 << kt) - 1) >> kt;
        if (ends_ok && kt >= 10)
            return launch_rht_tile(x, sign, sign_packed ? 1 : 0, n, kt, kb, scale, apply_scale, sign_fwd | sign_inv, a.vec, thc,
                                   stream);
        return launch_tile(a, ntiles, stream);
    }

    // long transform: contiguous pass over the low bits, strided passes above
    int kt = kPrefTileBits;
    a.kt = kt; a.b0 = 0; a.b1 = kt; a.cbits = kt; a.sbits = kt;
    a.apply_scale = 0; a.sign_mode = sign_fwd; a.vec = vec16;
    a.in_levels = thc.in_levels;
    a.in_planes = thc.in_planes;
    hipError_t e = ends_ok ? launch_rht_tile(x, sign, sign_packed ? 1 : 0, n, kt, kt, scale, 0, sign_fwd, a.vec, first, stream)
                           : launch_tile(a, n >> kt, stream);
    if (e != hipSuccess) return e;
    a.in_levels = nullptr;
    a.in_planes = nullptr;
    int s = kt;
    const int max_rows = kMaxTileBits - kStridedCols;
    while (s < kb) {
        // split the remaining bits evenly over as few passes as the LDS allows
        const int rem = kb - s;
        const int passes = (rem + max_rows - 1) / max_rows;
        const int r = (rem + passes - 1) / passes;
        a.kt = r + kStridedCols; a.b0 = kStridedCols; a.b1 = kStridedCols + r;
        a.cbits = kStridedCols; a.sbits = s;
        const bool last_pass = (s + r == kb);
        a.apply_scale = last_pass ? apply_scale : 0;
        a.sign_mode = last_pass ? sign_inv : 0;
        a.out_levels = last_pass ? thc.out_levels : nullptr;
        a.post_scale = last_pass ? thc.post_scale : nullptr;
        a.vec = vec16;
        if (r >= 4 && ends_ok && (n & (((int64_t)1 << (s + r)) - 1)) == 0)
            e = launch_rht_strided(x, sign, sign_packed ? 1 : 0, n, r, s, scale, a.apply_scale, a.sign_mode, a.vec,
                                   last_pass ? last : none, stream);
        else
            e = launch_tile(a, n >> a.kt, stream);
        if (e != hipSuccess) return e;
        s += r;
    }
    return hipSuccess;
}

hipError_t launch_hadamard(float *vec, int64_t n, hipStream_t stream)
{
    return fwht_blocks(vec, nullptr, false, n, ilog2(n), 1.0f, 0, 0, stream);
}

hipError_t launch_rht_blocked(float *vec, const void *sign, bool sign_packed, int64_t n, int64_t block, float scale,
                              int inverse, hipStream_t stream)
{
    return fwht_blocks(vec, sign, sign_packed, n, ilog2(block), scale, 1, inverse, stream);
}

// rotate (forward) and quantise: vec is read and left holding intermediate values
hipError_t launch_thc_rht_quantize(float *vec, const void *sign, bool sign_packed, const float *uniform, void *levels_out,
                                   int64_t n, int64_t block, float scale, const float *lo, const float *delta, int levels,
                                   hipStream_t stream)
{
    ThcEnds thc;
    thc.out_levels = static_cast<uint16_t *>(levels_out);
    thc.uniform = uniform; thc.out_lo = lo; thc.out_delta = delta; thc.out_top = (float)(levels - 1);
    return fwht_blocks(vec, sign, sign_packed, n, ilog2(block), scale, 1, 0, stream, thc);
}

// dequantise and rotate back into out
hipError_t launch_thc_dequantize_irht(const void *levels_in, const void *sign, bool sign_packed, float *out, int64_t n,
                                      int64_t block, float scale, const float *step, const float *lo, hipStream_t stream)
{
    ThcEnds thc;
    thc.in_levels = static_cast<const uint16_t *>(levels_in);
    thc.in_step = step; thc.in_lo = lo;
    return fwht_blocks(out, sign, sign_packed, n, ilog2(block), scale, 1, 1, stream, thc);
}

// EDEN: centroids of the packed bins, rotated back (inverse transform over the whole vector or per block) and,
// with post_scale, multiplied by EDEN's scale -- the dequantised vector never reaches memory
hipError_t launch_eden_dequantize_irht(const uint32_t *packed, const float *centroids, int nbits, const void *sign,
                                       bool sign_packed, float *out, int64_t n, int64_t block, float scale,
                                       const float *post_scale, hipStream_t stream)
{
    ThcEnds ends;
    ends.in_planes = packed;
    ends.in_centroids = centroids;
    ends.in_nbits = nbits;
    ends.post_scale = post_scale;
    return fwht_blocks(out, sign, sign_packed, n, ilog2(block), scale, 1, 1, stream, ends);
}

// ---- randDiag -----------------------------------------------------------------------

// the 32 random bits of column j: nibble k decides element k * s8 + j (+1 where the nibble is >= 8)
__device__ __forceinline__ uint64_t rand_diag_word(int64_t j, uint64_t ss)
{
    const uint64_t M = 0xffffffffull;
    uint64_t r = (uint64_t)j + ss;
    r = (1103515245ull * r + 12345ull + ss) & M;
    r = (1140671485ull * r + 12820163ull + ss) & M;
    r += 0x9e3779b9ull; // the carry into bit 32 is kept
    r = ((r ^ (r >> 16)) * 0x85ebca6bull) & M;
    r = ((r ^ (r >> 13)) * 0xc2b2ae35ull) & M;
    return (r ^ (r >> 16)) & M;
}

__global__ __launch_bounds__(256) void rand_diag_kernel(float *__restrict__ out, int64_t size, int64_t s8, uint64_t ss)
{
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (j >= s8) return;
    const uint64_t r = rand_diag_word(j, ss);
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int64_t idx = (int64_t)k * s8 + j;
        if (idx < size) out[idx] = ((r >> (4 * k)) & 15u) >= 8u ? 1.0f : -1.0f;
    }
}

// The same diagonal as the bit vector of pack_signs (bit set where the value is -1), for size = 8 s8 with s8 a
// multiple of 32: a wave holds 64 consecutive columns, and its ballot for nibble k is two whole words of segment k.
__global__ __launch_bounds__(256) void rand_diag_bits_kernel(uint32_t *__restrict__ bits, int64_t s8, uint64_t ss)
{
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const uint64_t r = j < s8 ? rand_diag_word(j, ss) : ~0ull; // columns past the end: +1, bit clear
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const uint64_t m = __builtin_amdgcn_ballot_w64(((r >> (4 * k)) & 15u) < 8u);
        // lanes 0 and 32 store the halves; a half that starts at or past s8 belongs to nobody
        if ((lane & 31) == 0 && j < s8) bits[((int64_t)k * s8 + j) >> 5] = (uint32_t)(m >> lane);
    }
}

// one bit per element of a +-1 vector, set where the value is negative; bit e % 32 of word e / 32
__global__ __launch_bounds__(256) void pack_signs_kernel(const float *__restrict__ sign, uint32_t *__restrict__ bits, int64_t n)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool neg = e < n && sign[e] < 0.0f;
    const uint64_t m = __builtin_amdgcn_ballot_w64(neg);
    const int lane = threadIdx.x & 63;
    if ((lane & 31) == 0 && e < n) bits[e >> 5] = (uint32_t)(m >> lane);
}

hipError_t launch_pack_signs(const float *sign, uint32_t *bits, int64_t n, hipStream_t stream)
{
    hipLaunchKernelGGL(pack_signs_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, sign, bits, n);
    return hipGetLastError();
}

static uint64_t rand_diag_seed(int64_t seed)
{
    const uint64_t M = 0xffffffffull;
    uint64_t ss = ((uint64_t)seed * 1664525ull + 1013904223ull) & M;
    return (ss * 8121ull + 28411ull) & M;
}

hipError_t launch_rand_diag(float *out, int64_t size, int64_t seed, hipStream_t stream)
{
    const int64_t s8 = size / 8 + (size % 8 != 0);
    hipLaunchKernelGGL(rand_diag_kernel, dim3((unsigned)((s8 + 255) / 256)), dim3(256), 0, stream, out, size, s8,
                       rand_diag_seed(seed));
    return hipGetLastError();
}

// size: a multiple of 256
hipError_t launch_rand_diag_bits(uint32_t *bits, int64_t size, int64_t seed, hipStream_t stream)
{
    const int64_t s8 = size / 8;
    hipLaunchKernelGGL(rand_diag_bits_kernel, dim3((unsigned)((s8 + 255) / 256)), dim3(256), 0, stream, bits, s8,
                       rand_diag_seed(seed));
    return hipGetLastError();
}

} // namespace dq
