// Building blocks shared by the vectorised chunk-16 kernels (dq_scaling_hier16.hip,
// dq_scaling_tile16.hip): one lane owns one chunk of 16 elements, one wave owns a tile of
// 64 chunks whose packed bytes form one contiguous run of the record stream.
#pragma once

#include <type_traits>
#include "dq_device.cuh"

namespace dq {

constexpr int kRowsPerWave = 4; // superchunks per tile

template <int NBITS> struct Rec {
    static constexpr int R = (1 << (NBITS - 1)) - 1;
    static constexpr int PB = 2 * NBITS;       // code bytes per chunk
    static constexpr int CB = PB + 1;          // + one scale byte
    static constexpr int REC = 16 * CB + 2;    // + bf16 unit
    static constexpr int WORDS = (PB + 3) / 4; // dwords holding one chunk's codes
    // LDS window: 4 records + up to 15 bytes of misalignment, padded to 16
    static constexpr int WIN = ((kRowsPerWave * REC + 15 + 15) / 16) * 16;
    static constexpr int WIN_VECS = WIN / 16;  // <= 70: at most two 128-bit registers per lane
};

template <int NBITS, bool MEE> struct MeeArg {
    float c, cmm, l2b;
    uint32_t pad;
    double inv_c, inv_cmm, inv_l2b; // correctly rounded double reciprocals
    uint16_t table[MEE ? (1 << NBITS) : 4];
};

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}

// ---- 16 raw elements of one lane ----------------------------------------------------

template <int DT> struct Raw16;

template <> struct Raw16<DQ_BF16> {
    uint32_t w[8];
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int k = 0; k < 8; k++) w[k] = 0;
    }
    __device__ __forceinline__ void load(const void *p, int64_t e, bool vec)
    {
        // the unaligned path goes through volatile accesses so that the compiler cannot fold the two
        // paths into one narrow-load sequence
        const volatile uint16_t *h = static_cast<const volatile uint16_t *>(p) + e;
        if (vec) {
            const uint4 *q = reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(p) + e);
            uint4 a = q[0], b = q[1];
            w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) w[k] = (uint32_t)h[2 * k] | ((uint32_t)h[2 * k + 1] << 16);
        }
    }
    __device__ __forceinline__ void store(void *p, int64_t e, bool vec) const
    {
        volatile uint16_t *h = static_cast<volatile uint16_t *>(p) + e;
        if (vec) {
            uint4 *q = reinterpret_cast<uint4 *>(static_cast<uint16_t *>(p) + e);
            q[0] = make_uint4(w[0], w[1], w[2], w[3]);
            q[1] = make_uint4(w[4], w[5], w[6], w[7]);
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) { h[2 * k] = (uint16_t)w[k]; h[2 * k + 1] = (uint16_t)(w[k] >> 16); }
        }
    }
    __device__ __forceinline__ float get(int i) const
    {
        return (i & 1) ? __uint_as_float(w[i >> 1] & 0xffff0000u) : __uint_as_float(w[i >> 1] << 16);
    }
    __device__ __forceinline__ void set(const float (&t)[16])
    {
#pragma unroll
        for (int k = 0; k < 8; k++) w[k] = f32x2_to_bf16x2(t[2 * k], t[2 * k + 1]);
    }
    // binary32 bit pattern of max |element| in integer order (a NaN sorts above infinity)
    __device__ __forceinline__ uint32_t absmax_bits() const
    {
        uint32_t m = w[0] & 0x7fff7fffu;
#pragma unroll
        for (int k = 1; k < 8; k++) m = pk_max_u16(m, w[k] & 0x7fff7fffu);
        return max(m << 16, m & 0xffff0000u);
    }
    // every element in [+0, 1]
    __device__ __forceinline__ bool unit_interval() const
    {
        uint32_t m = w[0];
#pragma unroll
        for (int k = 1; k < 8; k++) m = pk_max_u16(m, w[k]);
        return max(m & 0xffffu, m >> 16) <= 0x3f80u;
    }
    static constexpr int kSlots = 2; // 16-byte pieces per lane
    __device__ __forceinline__ uint4 slot(int j) const { return make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]); }
};

template <> struct Raw16<DQ_F32> {
    uint32_t w[16];
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int k = 0; k < 16; k++) w[k] = 0;
    }
    __device__ __forceinline__ void load(const void *p, int64_t e, bool vec)
    {
        const volatile uint32_t *f = static_cast<const volatile uint32_t *>(p) + e;
        if (vec) {
            const uint4 *q = reinterpret_cast<const uint4 *>(static_cast<const uint32_t *>(p) + e);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                uint4 t = q[k];
                w[4 * k] = t.x; w[4 * k + 1] = t.y; w[4 * k + 2] = t.z; w[4 * k + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) w[k] = f[k];
        }
    }
    __device__ __forceinline__ void store(void *p, int64_t e, bool vec) const
    {
        volatile uint32_t *f = static_cast<volatile uint32_t *>(p) + e;
        if (vec) {
            uint4 *q = reinterpret_cast<uint4 *>(static_cast<uint32_t *>(p) + e);
#pragma unroll
            for (int k = 0; k < 4; k++) q[k] = make_uint4(w[4 * k], w[4 * k + 1], w[4 * k + 2], w[4 * k + 3]);
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) f[k] = w[k];
        }
    }
    __device__ __forceinline__ float get(int i) const { return __uint_as_float(w[i]); }
    __device__ __forceinline__ void set(const float (&t)[16])
    {
#pragma unroll
        for (int k = 0; k < 16; k++) w[k] = __float_as_uint(t[k]);
    }
    __device__ __forceinline__ uint32_t absmax_bits() const
    {
        uint32_t m = w[0] & 0x7fffffffu;
#pragma unroll
        for (int k = 1; k < 16; k++) m = max(m, w[k] & 0x7fffffffu);
        return m;
    }
    __device__ __forceinline__ bool unit_interval() const
    {
        uint32_t m = w[0];
#pragma unroll
        for (int k = 1; k < 16; k++) m = max(m, w[k]);
        return m <= 0x3f800000u;
    }
    static constexpr int kSlots = 4;
    __device__ __forceinline__ uint4 slot(int j) const { return make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]); }
};

// binary16 elements: the storage and the moves of the bf16 case, other conversions
template <> struct Raw16<DQ_F16> : Raw16<DQ_BF16> {
    __device__ __forceinline__ float get(int i) const { return f16_bits_to_f32((w[i >> 1] >> (16 * (i & 1))) & 0xffffu); }
    __device__ __forceinline__ void set(const float (&t)[16])
    {
#pragma unroll
        for (int k = 0; k < 8; k++) w[k] = f32_to_f16_bits(t[2 * k]) | (f32_to_f16_bits(t[2 * k + 1]) << 16);
    }
    // binary16 bit pattern of max |element| in integer order (a NaN sorts above infinity)
    __device__ __forceinline__ uint32_t absmax_half_bits() const
    {
        uint32_t m = w[0] & 0x7fff7fffu;
#pragma unroll
        for (int k = 1; k < 8; k++) m = pk_max_u16(m, w[k] & 0x7fff7fffu);
        return max(m & 0xffffu, m >> 16);
    }
    // every element in [+0, 1]
    __device__ __forceinline__ bool unit_interval() const
    {
        uint32_t m = w[0];
#pragma unroll
        for (int k = 1; k < 8; k++) m = pk_max_u16(m, w[k]);
        return max(m & 0xffffu, m >> 16) <= 0x3c00u;
    }
};

// the 16 uniform values of a chunk drawn in the kernel (element type tag for the random operand)
constexpr int DQ_PHILOX = 3;

template <> struct Raw16<DQ_PHILOX> {
    uint32_t w[4]; // the generator's words with the lowest bit of every byte set
    __device__ __forceinline__ void zero() { w[0] = w[1] = w[2] = w[3] = 0x01010101u; }
    __device__ __forceinline__ void generate(const RandKey &key, int64_t chunk)
    {
        chunk_uniform_words(key, chunk, w);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            w[k] |= 0x01010101u;
            // (the compiler would otherwise push the OR back into every byte's extraction)
            asm("" : "+v"(w[k]));
        }
    }
    // the generator's arithmetic stays where generate() was called (behind the tile's loads, in front of whatever waits
    // for them) instead of sinking to the first use of its words
    __device__ __forceinline__ void pin() const { asm volatile("" ::"v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3])); }
    __device__ __forceinline__ void load(const void *, int64_t, bool) {}
    // (byte i | 1) as a float: one byte-to-float conversion
    __device__ __forceinline__ float odd_byte(int i) const { return (float)((w[i >> 2] >> (8 * (i & 3))) & 0xffu); }
    __device__ __forceinline__ float get(int i) const
    {
        return odd_byte(i) * 0.00390625f;
    }
    __device__ __forceinline__ bool unit_interval() const { return true; }
};

// ---- the MEE level table on its way into LDS -------------------------------------------------------
//
// The table comes with the kernel arguments as 2^NBITS binary16 patterns.  A lane fetches its pairs of entries with the
// other loads of its tile (one or two 4-byte loads, no wait in between) and converts and stores them as floats once the
// tile's own data has arrived.
template <int NBITS> struct TableRegs {
    static constexpr int kPairs = (1 << NBITS) / 2;
    static constexpr int kPerLane = (kPairs + 63) / 64;
    uint32_t pair[kPerLane];
};

template <int NBITS, class ARG> __device__ __forceinline__ TableRegs<NBITS> table_fetch(const ARG &mp, int lane)
{
    TableRegs<NBITS> t;
    const uint32_t *pairs = reinterpret_cast<const uint32_t *>(mp.table); // 4-byte aligned inside the argument block
#pragma unroll
    for (int j = 0; j < TableRegs<NBITS>::kPerLane; j++) {
        const int k = lane + 64 * j;
        t.pair[j] = k < TableRegs<NBITS>::kPairs ? pairs[k] : 0u;
    }
    return t;
}

template <int NBITS> __device__ __forceinline__ void table_commit(float *table, const TableRegs<NBITS> &t, int lane)
{
#pragma unroll
    for (int j = 0; j < TableRegs<NBITS>::kPerLane; j++) {
        const int k = lane + 64 * j;
        if (k < TableRegs<NBITS>::kPairs) {
            table[2 * k] = f16_bits_to_f32(t.pair[j] & 0xffffu);
            table[2 * k + 1] = f16_bits_to_f32(t.pair[j] >> 16);
        }
    }
}

// ---- record windows --------------------------------------------------------------------

// the (up to two) aligned 128-bit pieces of a packed run this lane moves
struct WinRegs {
    u32x4 a, b;
};

// every lane loads (indices are clamped into the run), so the registers are
// always defined and the prefetch is two plain vector loads
__device__ __forceinline__ WinRegs window_fetch(const uint8_t *g, int total, int lane)
{
    const int mis = (int)(reinterpret_cast<uintptr_t>(g) & 15);
    const u32x4 *ga = reinterpret_cast<const u32x4 *>(g - mis);
    const int nvec = (mis + total + 15) >> 4;
    WinRegs r;
    r.a = ga[min(lane, nvec - 1)];
    r.b = ga[min(lane + 64, nvec - 1)];
    return r;
}

// byte k of the run lands at win[(g & 15) + k]
__device__ __forceinline__ int window_commit(uint8_t *win, const WinRegs &r, const uint8_t *g, int total, int lane)
{
    const int mis = (int)(reinterpret_cast<uintptr_t>(g) & 15);
    const int nvec = (mis + total + 15) >> 4;
    if (lane < nvec) reinterpret_cast<u32x4 *>(win)[lane] = r.a;
    if (lane + 64 < nvec) reinterpret_cast<u32x4 *>(win)[lane + 64] = r.b;
    return mis;
}

// stream `total` bytes from win[mis ...] to g (g & 15 == mis).  STREAM: whole 128-byte lines leave with the streaming hint
// (for kernels that the memory system bounds; the address test per vector costs a kernel bound by its arithmetic 1-4 %).
template <bool STREAM = true>
__device__ __forceinline__ void window_flush(const uint8_t *win, uint8_t *g, int mis, int total, int lane)
{
    int head = (16 - mis) & 15;
    head = min(head, total);
    const int body = (total - head) & ~15;
    const int tail = total - head - body;
    if (lane < head) g[lane] = win[mis + lane];
    const uint4 *wv = reinterpret_cast<const uint4 *>(win + mis + head);
    uint4 *gv = reinterpret_cast<uint4 *>(g + head);
    // 128-byte lines that lie wholly inside [g, g + total) leave with the streaming hint: they go out while the kernel
    // runs instead of waiting in the L2 for the write-back at its end.  The ragged ends share their lines with the
    // neighbouring waves' runs and are stored plainly, so that the L2 merges the pieces (as streaming stores they
    // would reach memory as partial writes: measured slower than no hint at all).
    const uintptr_t first = (reinterpret_cast<uintptr_t>(g) + 127) & ~(uintptr_t)127;
    const uintptr_t last = (reinterpret_cast<uintptr_t>(g) + total) & ~(uintptr_t)127;
    for (int v = lane; v < (body >> 4); v += 64) {
        const uintptr_t at = reinterpret_cast<uintptr_t>(gv + v);
        if (STREAM && at >= first && at < last)
            stream_store(gv + v, wv[v]);
        else
            gv[v] = wv[v];
    }
    const int tl = lane - 32; // lanes 32.. store the tail so head and tail overlap in time
    if (tl >= 0 && tl < tail) g[head + body + tl] = win[mis + head + body + tl];
}

// ---- per-chunk code words -----------------------------------------------------------------

template <int NBITS> __device__ __forceinline__ void words_put(uint32_t (&w)[Rec<NBITS>::WORDS], int i, uint32_t code)
{
    const int bit = i * NBITS;
    w[bit >> 5] |= code << (bit & 31);
    if ((bit & 31) + NBITS > 32) w[(bit >> 5) + 1] |= code >> (32 - (bit & 31));
}

// replaces the code of element i
template <int NBITS> __device__ __forceinline__ void words_set(uint32_t (&w)[Rec<NBITS>::WORDS], int i, uint32_t code)
{
    constexpr uint32_t kMask = (1u << NBITS) - 1u;
    const int bit = i * NBITS;
    w[bit >> 5] = (w[bit >> 5] & ~(kMask << (bit & 31))) | (code << (bit & 31));
    if ((bit & 31) + NBITS > 32) {
        const int done = 32 - (bit & 31);
        w[(bit >> 5) + 1] = (w[(bit >> 5) + 1] & ~(kMask >> done)) | (code >> done);
    }
}

template <int NBITS> __device__ __forceinline__ uint32_t words_get(const uint32_t (&w)[Rec<NBITS>::WORDS], int i)
{
    const int bit = i * NBITS;
    uint32_t v = w[bit >> 5] >> (bit & 31);
    if ((bit & 31) + NBITS > 32) v |= w[(bit >> 5) + 1] << (32 - (bit & 31));
    return v & ((1u << NBITS) - 1u);
}

// one chunk's CB bytes (codes + scale byte) from / to a window
template <int NBITS>
__device__ __forceinline__ void chunk_read(const uint8_t *p, uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t &q)
{
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = 0;
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::PB; k++) w[k >> 2] |= (uint32_t)p[k] << (8 * (k & 3));
    q = p[Rec<NBITS>::PB];
}

template <int NBITS>
__device__ __forceinline__ void chunk_write(uint8_t *p, const uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t q)
{
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::PB; k++) p[k] = (uint8_t)(w[k >> 2] >> (8 * (k & 3)));
    p[Rec<NBITS>::PB] = (uint8_t)q;
}

// ---- exact division by a chunk constant ------------------------------------------------------

// 1/b in double to within one double ulp, b a normal binary32 in [2^-100, 2^100]
__device__ __forceinline__ double recip_f64(float b)
{
    const double bd = (double)b;
    double y = (double)__builtin_amdgcn_rcpf(b);
    double e = __builtin_fma(-bd, y, 1.0);
    y = __builtin_fma(y, e, y);
    e = __builtin_fma(-bd, y, 1.0);
    y = __builtin_fma(y, e, y);
    return y;
}

// binary32 quotient a / b given yb ~= 1/b in double.  The product carries a relative error below 2^-51, and a quotient of
// two binary32 numbers that is a normal number comes no closer than 2^-49 (relative) to a rounding boundary without being
// representable: for those this is the correctly rounded quotient.  A quotient in the subnormal range can lie exactly
// half-way between two subnormal numbers (a = m 2^-150 b with m odd, possible when b is an even multiple of a power of
// two), and there the error of the product decides the direction instead of the tie rule: where that can change a result,
// use div_exact.
__device__ __forceinline__ float div_by(float a, double yb) { return (float)((double)a * yb); }

// q is a subnormal number other than zero
__device__ __forceinline__ bool is_subnormal(float q) { return (__float_as_uint(q) & 0x7fffffffu) - 1u < 0x007fffffu; }

// correctly rounded binary32 quotient a / b for every finite a: the product form, and the division itself when the product
// comes out subnormal (a product that rounds to zero is below every tie, as is the quotient)
__device__ __forceinline__ float div_exact(float a, float b, double yb)
{
    float q = div_by(a, yb);
    if (__builtin_amdgcn_ballot_w64(is_subnormal(q)) != 0) {
        // a branch of the wave, and one the compiler keeps: the division is a dozen instructions, which it would otherwise
        // execute for every element and select from afterwards
        asm volatile("");
        if (is_subnormal(q)) q = a / b;
    }
    return q;
}

// log2_det() for a finite argument >= 1 (same operations, special cases dropped)
__device__ __forceinline__ float log2_det_ge1(float x)
{
    const uint32_t ix = __float_as_uint(x);
    const uint32_t t = ix - 0x3f3504f3u;
    const int k = (int)t >> 23;
    const float z = __uint_as_float(ix - (t & 0xff800000u));
    const float f = z - 1.0f;
    float q = -0x1.d0dd08p-4f;
    q = __builtin_fmaf(q, f, 0x1.7ad622p-3f);
    q = __builtin_fmaf(q, f, -0x1.831b24p-3f);
    q = __builtin_fmaf(q, f, 0x1.a33bdap-3f);
    q = __builtin_fmaf(q, f, -0x1.eb492p-3f);
    q = __builtin_fmaf(q, f, 0x1.277e38p-2f);
    q = __builtin_fmaf(q, f, -0x1.715762p-2f);
    q = __builtin_fmaf(q, f, 0x1.ec7092p-2f);
    q = __builtin_fmaf(q, f, -0x1.715476p-1f);
    const float p = (f * f) * q;
    float r = __builtin_fmaf(f, 0x1.4ae0cp-26f, p);
    r = __builtin_fmaf(f, 0x1.715476p+0f, r);
    return (float)k + r;
}

// One element of the fast quantiser, every operation as the reference orders them (three correctly rounded
// divisions and the deterministic log2 for MEE): the signed code before clamping.
template <bool MEE, class ARG>
__device__ __forceinline__ int exact_code_fast(float vi, float ri, float d, double yd, const ARG &mp)
{
    // (the divisions further down are by constants above 1 of arguments that are zero or normal numbers, and a
    // subnormal |x| / c disappears in the sum with 1)
    float x = MEE ? div_by(vi, yd) : div_exact(vi, d, yd);
    if (MEE) {
        const float arg = div_by(__builtin_fabsf(x), mp.inv_c) + 1.0f;
        const float lat = div_by(log2_det_ge1(arg), mp.inv_l2b);
        x = __builtin_copysignf(lat, x);
    }
    const float fl = __builtin_floorf(x);
    const float c = __builtin_ceilf((x - fl) - ri);
    return (int)(fl + c); // |fl| <= R + 1 and c in {-1, 0, 1}: exact
}

// The code of an element is clamp(ceil(L - r), -R, R) + R for the coordinate L the exact chain computes -- v / d (AEE)
// or +-log2(|v / d| / c + 1) / log2(base) (MEE) -- because floor(L) + ceil(frac(L) - r) is that integer; and it is
// min(floor(L - r + R + 1), 2R) (nothing below zero) as long as L - r is not an integer.  A cheap estimate of
// T = L - r + R + 1 that is within e < kDelta of it decides the code unless T comes within kDelta of an integer; such
// elements (one in a few thousand) are redone with the exact chain, so the bytes are those of the exact chain
// throughout.  The estimate is formed as T' = estimate + kDelta (kDelta is part of the constant the random value is
// subtracted from): frac(T') >= 2 kDelta then puts T' - kDelta - e above floor(T') and T' - kDelta + e below
// floor(T') + 1, so floor(T) = floor(T'), and the guard is one fraction and one comparison.
//   AEE: estimate = fma(v, rcp(d), (R + 1 + kDelta) - r).  The hardware reciprocal is good to 1 ulp
//        (|v rcp(d) - v / d| < (R + 1) 2^-23), the constant minus r is exact for the in-kernel random bytes and within
//        (R + 1) 2^-26 otherwise, and the fma rounds a value below 2 (R + 1): e stays below 0.27 (R + 1) 2^-20.
//   MEE: estimate = fma(v_log_f32(fma(|v rcp(d)|, 1 / c, 1)), +-1 / log2(base), (R + 1 + kDelta) - r), v_log_f32 being
//        good to 1 ulp; estimate and exact chain both approximate log2(|v| / (d c) + 1) / log2(base), their distance is
//        bounded by (1.44 * 5e-7 + 2.7 ulp(log)) / log2(base) + 2 ulp(2 R): < 6.9e-5 for 6..8 bits (log2(base) = 0.0286,
//        log < 4) and < 1.2e-5 below (log2(base) >= 0.09, log < 1.5); measured over 4e9 random operands per width: 1.5e-5
//        and 4.8e-6 (without the constant in the last fma, which adds at most 3.8e-6 and 1e-6).
template <int NBITS, bool MEE> struct EstimateGuard {
    static constexpr float kDelta = MEE ? (NBITS >= 6 ? 0x1p-12f : 0x1p-14f) : (float)(1 << (NBITS - 1)) * 0x1p-20f;
};

// bias - r_i; exact for the in-kernel random bytes ((256 bias - odd byte) / 256 needs 16 bits)
template <class RR> __device__ __forceinline__ float below(const RR &r, int i, float bias)
{
    if constexpr (std::is_same<RR, Raw16<DQ_PHILOX>>::value)
        return __builtin_fmaf(r.odd_byte(i), -0.00390625f, bias);
    else
        return bias - r.get(i);
}

template <int NBITS, bool MEE, class RV, class RR>
__device__ __forceinline__ float estimate_coordinate(const RV &v, const RR &r, int i, float rd, float rc, float rl2b)
{
    const float vi = v.get(i);
    const float off = below(r, i, (float)(Rec<NBITS>::R + 1) + EstimateGuard<NBITS, MEE>::kDelta); // the constant is exact: <= 21 bits
    if (MEE) {
        const float est = __builtin_amdgcn_logf(__builtin_fmaf(__builtin_fabsf(vi * rd), rc, 1.0f));
        return __builtin_fmaf(est, __builtin_copysignf(rl2b, vi), off);
    }
    return __builtin_fmaf(vi, rd, off);
}

// Upper clamp of the packed codes of a chunk, for widths that divide 32: a field of an estimate_codes() word holds
// floor(T) <= 2 R + 1 = all ones, and only that value is above 2 R.  A field is all ones when its low NBITS - 1 bits
// carry into the top bit and the top bit is set; such fields lose their lowest bit.  A few integer instructions per
// word instead of one clamp per element.
template <int NBITS> __device__ __forceinline__ uint32_t clamp_fields(uint32_t w)
{
    static_assert(NBITS == 2 || NBITS == 4 || NBITS == 8, "fields must not straddle words");
    if (NBITS == 2) return w ^ (w & (w >> 1) & 0x55555555u);
    constexpr uint32_t one = NBITS == 4 ? 0x11111111u : 0x01010101u;
    constexpr uint32_t top = one << (NBITS - 1), low = top - one;
    const uint32_t full = ((w & low) + one) & w & top;
    return w - (full >> (NBITS - 1));
}

// The codes of one chunk against the step d (normal, 2^-100 <= d <= 2^100) for elements that are finite (a NaN would
// pass the guard unnoticed) with |v| <= (R + 1) d and random values in [0, 1]: estimate, guard, exact redo.  w must
// be zeroed.  -1 < T' < 2 R + 2, so the conversion to a signed integer (towards zero) is the lower clamp, and for the
// widths that divide 32 the upper clamp is done on the packed words (clamp_fields).
template <int NBITS, bool MEE, class RV, class RR, class ARG>
__device__ __forceinline__ void estimate_codes(const RV &v, const RR &r, float d, const ARG &mp, uint32_t (&w)[Rec<NBITS>::WORDS])
{
    constexpr int R = Rec<NBITS>::R;
    constexpr bool kFields = NBITS == 2 || NBITS == 4 || NBITS == 8;
    const float rd = __builtin_amdgcn_rcpf(d);
    const float rc = MEE ? (float)mp.inv_c : 0.0f, rl2b = MEE ? (float)mp.inv_l2b : 0.0f;
    constexpr float kDelta = EstimateGuard<NBITS, MEE>::kDelta;
    // (the wave-wide view of each flag is taken where the comparison is made: there it is the comparison's own lane mask, and
    // the tests further down are scalar)
    bool doubt[16];
    uint64_t lanes_in_doubt[16], any = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float t = estimate_coordinate<NBITS, MEE>(v, r, i, rd, rc, rl2b);
        doubt[i] = __builtin_amdgcn_fractf(t) < 2.0f * kDelta;
        lanes_in_doubt[i] = __builtin_amdgcn_ballot_w64(doubt[i]);
        any |= lanes_in_doubt[i];
        if (kFields)
            words_put<NBITS>(w, i, (uint32_t)(int)t);
        else
            words_put<NBITS>(w, i, (uint32_t)__builtin_amdgcn_fmed3f(t, 0.0f, (float)(2 * R))); // T < 2^20: exact
    }
    if (kFields) {
#pragma unroll
        for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = clamp_fields<kFields ? NBITS : 2>(w[k]);
    }
    if (any != 0) {
        const double yd = recip_f64(d);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (lanes_in_doubt[i] != 0) {
                // (among them the zero elements -- padding, sparse input -- whose random value is exactly 0 or 1: their
                // T is an integer, and the chain's ceil(-r) is 0, or -1 at r = 1)
                const int sv = exact_code_fast<MEE>(v.get(i), r.get(i), d, yd, mp);
                if (doubt[i]) words_set<NBITS>(w, i, (uint32_t)(min(max(sv, -R), R) + R));
            }
        }
    }
}

template <int NBITS, bool MEE> static MeeArg<NBITS, MEE> make_arg(const MeeParams &mp)
{
    MeeArg<NBITS, MEE> a;
    a.c = mp.c; a.cmm = mp.cmm; a.l2b = mp.l2b; a.pad = 0;
    a.inv_c = 1.0 / (double)mp.c; a.inv_cmm = 1.0 / (double)mp.cmm; a.inv_l2b = 1.0 / (double)mp.l2b;
    for (int k = 0; k < (MEE ? (1 << NBITS) : 4); k++) a.table[k] = mp.table[k];
    return a;
}


} // namespace dq
