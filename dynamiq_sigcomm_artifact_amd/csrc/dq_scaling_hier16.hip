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
#include "dq_device.cuh"
#include "dq_launch.h"

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

// ---- record windows --------------------------------------------------------------------

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// stream `total` bytes from win[mis ...] to g (g & 15 == mis)
__device__ __forceinline__ void window_flush(const uint8_t *win, uint8_t *g, int mis, int total, int lane)
{
    int head = (16 - mis) & 15;
    head = min(head, total);
    const int body = (total - head) & ~15;
    const int tail = total - head - body;
    if (lane < head) g[lane] = win[mis + lane];
    const uint4 *wv = reinterpret_cast<const uint4 *>(win + mis + head);
    uint4 *gv = reinterpret_cast<uint4 *>(g + head);
    for (int v = lane; v < (body >> 4); v += 64) gv[v] = wv[v];
    const int tl = lane - 32; // lanes 32.. store the tail so head and tail overlap in time
    if (tl >= 0 && tl < tail) g[head + body + tl] = win[mis + head + body + tl];
}

// LDS accesses of one wave execute in order; the fence only stops the compiler
// from moving them across the hand-over between lanes
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- per-chunk code words -----------------------------------------------------------------

template <int NBITS> __device__ __forceinline__ void words_put(uint32_t (&w)[Rec<NBITS>::WORDS], int i, uint32_t code)
{
    const int bit = i * NBITS;
    w[bit >> 5] |= code << (bit & 31);
    if ((bit & 31) + NBITS > 32) w[(bit >> 5) + 1] |= code >> (32 - (bit & 31));
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

// correctly rounded binary32 quotient a / b given yb ~= 1/b in double
__device__ __forceinline__ float div_by(float a, double yb) { return (float)((double)a * yb); }

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
                                                            MeeArg<NBITS, MEE> mp)
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

// 16-byte slot s of a wave's output tile lives at LDS slot s ^ ((s >> 3) & 7): both
// the per-lane writes (slots S*lane + j) and the lane-contiguous reads (slots
// 64*k + lane) then touch eight distinct bank groups per eight lanes
__device__ __forceinline__ int swz(int s) { return s ^ ((s >> 3) & 7); }

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

template <int NBITS, bool MEE> static MeeArg<NBITS, MEE> make_arg(const MeeParams &mp)
{
    MeeArg<NBITS, MEE> a;
    a.c = mp.c; a.cmm = mp.cmm; a.l2b = mp.l2b; a.pad = 0;
    a.inv_c = 1.0 / (double)mp.c; a.inv_cmm = 1.0 / (double)mp.cmm; a.inv_l2b = 1.0 / (double)mp.l2b;
    for (int k = 0; k < (MEE ? (1 << NBITS) : 4); k++) a.table[k] = mp.table[k];
    return a;
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// one single-wave workgroup per tile of 4 superchunks
static inline unsigned grid_for(int64_t nsc) { return (unsigned)((nsc + kRowsPerWave - 1) / kRowsPerWave); }

template <int DT, int RDT, int NBITS, bool MEE>
static hipError_t run_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd, const int32_t *rows,
                               int64_t nsc, bool fused, const MeeParams &mp, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    dim3 grid(grid_for(nsc)), block(64);
    const int vec = (aligned16(src) ? 1 : 0) | (aligned16(rnd) ? 2 : 0);
    if (fused)
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, true>), grid, block, 0, stream, src, recv, dst, rnd, rows, nsc, vec, arg);
    else
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, false>), grid, block, 0, stream, src, recv, dst, rnd, rows, nsc, vec, arg);
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
                                    const MeeParams &mp, hipStream_t stream)
{
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
    if (dtype == DQ_BF16) {
        DQ_NBITS_MEE(run_compress, DQ_BF16 DQ_COMMA DQ_BF16, src, recv, dst, rnd, rows, nsc, fused, mp, stream)
    } else if (rb16) {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_BF16, src, recv, dst, rnd, rows, nsc, fused, mp, stream)
    } else {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_F32, src, recv, dst, rnd, rows, nsc, fused, mp, stream)
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
