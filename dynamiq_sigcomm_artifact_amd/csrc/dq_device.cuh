// Device-side numeric primitives shared by the gfx950 kernels.
//
// Arithmetic contract (the kernels are checked byte-for-byte against a CPU
// restatement that follows the same rules): IEEE binary32, round to nearest
// even, denormals preserved, no implicit contraction (the translation units
// are compiled with -ffp-contract=off); a multiply-add is fused only where
// __builtin_fmaf is spelled out.  Half-precision operations are an fp32
// operation followed by one rounding to binary16.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dynamiq_eden.h"

namespace dq {

// ---- storage formats -------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    __bf16 b = (__bf16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi)
{
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {lo, hi};
    bf16x2 b = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f)
{
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// value of a binary16 result computed through fp32
__device__ __forceinline__ float rh(float x) { return (float)(_Float16)x; }
// value after a round trip through bfloat16
__device__ __forceinline__ float rb(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }

template <int DT> struct ElemIO;

template <> struct ElemIO<DQ_F16> {
    typedef uint16_t storage;
    static __device__ __forceinline__ float load(const void *p, int64_t i) { return f16_bits_to_f32(((const uint16_t *)p)[i]); }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) { ((uint16_t *)p)[i] = (uint16_t)f32_to_f16_bits(v); }
    static __device__ __forceinline__ float round(float v) { return rh(v); }
};
template <> struct ElemIO<DQ_BF16> {
    typedef uint16_t storage;
    static __device__ __forceinline__ float load(const void *p, int64_t i) { return bf16_bits_to_f32(((const uint16_t *)p)[i]); }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) { ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16_bits(v); }
    static __device__ __forceinline__ float round(float v) { return rb(v); }
};
template <> struct ElemIO<DQ_F32> {
    typedef float storage;
    static __device__ __forceinline__ float load(const void *p, int64_t i) { return ((const float *)p)[i]; }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) { ((float *)p)[i] = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};

// ---- conversions with saturating / wrapping device semantics ---------------

__device__ __forceinline__ int sat_i16(float x) // truncate, saturate, NaN -> 0
{
    int v = (int)x; // v_cvt_i32_f32: saturating, NaN -> 0
    return min(max(v, -32768), 32767);
}

__device__ __forceinline__ int sat_u16(float x)
{
    int v = (int)x;
    return min(max(v, 0), 65535);
}

__device__ __forceinline__ int wrap_i16(int x) { return (int)(int16_t)x; }

__device__ __forceinline__ int clamp_code(int signed_val, int range)
{
    return min(max(signed_val, -range), range) + range;
}

// ---- scale guards (fp32 path) ---------------------------------------------

__device__ __forceinline__ float pos_scale(float v)
{
    v = __builtin_isfinite(v) ? v : 1.0e-30f;
    return __builtin_fmaxf(v, 1.0e-30f);
}

__device__ __forceinline__ float nonneg_scale(float v)
{
    v = __builtin_isfinite(v) ? v : 0.0f;
    return __builtin_fmaxf(v, 0.0f);
}

// ---- deterministic log2 ----------------------------------------------------
// x = 2^k * z, z in [sqrt(1/2), sqrt(2)); log2(z) = f*log2(e) + f^2*Q(f) with
// f = z - 1 and Q a fixed degree-8 polynomial evaluated by Horner with fused
// multiply-adds.  <= 1.7 ulp; identical on any IEEE machine.
__device__ __forceinline__ float log2_det(float x)
{
    uint32_t ix = __float_as_uint(x);
    int k = 0;
    if (ix >= 0x7f800000u) {
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x7fffffffu) > 0x7f800000u) return x + x;
        if ((ix << 1) == 0) return -__builtin_inff();
        return __uint_as_float(0x7fc00000u);
    }
    if (ix < 0x00800000u) {
        if (ix == 0) return -__builtin_inff();
        x *= 8388608.0f;
        ix = __float_as_uint(x);
        k = -23;
    }
    uint32_t t = ix - 0x3f3504f3u;
    k += (int)t >> 23;
    float z = __uint_as_float(ix - (t & 0xff800000u));
    float f = z - 1.0f;
    float q = -0x1.d0dd08p-4f;
    q = __builtin_fmaf(q, f, 0x1.7ad622p-3f);
    q = __builtin_fmaf(q, f, -0x1.831b24p-3f);
    q = __builtin_fmaf(q, f, 0x1.a33bdap-3f);
    q = __builtin_fmaf(q, f, -0x1.eb492p-3f);
    q = __builtin_fmaf(q, f, 0x1.277e38p-2f);
    q = __builtin_fmaf(q, f, -0x1.715762p-2f);
    q = __builtin_fmaf(q, f, 0x1.ec7092p-2f);
    q = __builtin_fmaf(q, f, -0x1.715476p-1f);
    float p = (f * f) * q;
    float r = __builtin_fmaf(f, 0x1.4ae0cp-26f, p);
    r = __builtin_fmaf(f, 0x1.715476p+0f, r);
    return (float)k + r;
}

// ---- stochastic rounding ----------------------------------------------------

// floor(x) + ceil(frac - r) in int16 arithmetic, no guards
__device__ __forceinline__ int sr_plain(float x, float r)
{
    float fl = __builtin_floorf(x);
    int s = sat_i16(fl);
    return wrap_i16(s + sat_i16(__builtin_ceilf((x - fl) - r)));
}

// non-finite and out-of-range inputs saturate to +-32767 (NaN -> 0); a
// non-finite random value counts as 0
__device__ __forceinline__ int sr_guarded(float x, float r)
{
    r = __builtin_isfinite(r) ? r : 0.0f;
    int s = sr_plain(x, r);
    if (!__builtin_isfinite(x)) s = (x > 0.0f) ? 32767 : ((x < 0.0f) ? -32767 : 0);
    else if (x >= 32767.0f) s = 32767;
    else if (x <= -32767.0f) s = -32767;
    return s;
}

__device__ __forceinline__ float mee_inverse_plain(float x, float c, float l2b)
{
    float a = __builtin_fabsf(x);
    if (!(a > 0.0f)) return 0.0f;
    float lat = log2_det(a / c + 1.0f) / l2b;
    return x < 0.0f ? -lat : lat;
}

__device__ __forceinline__ float mee_inverse_guarded(float x, float c, float l2b)
{
    if (!__builtin_isfinite(x)) return (x > 0.0f) ? 32767.0f : ((x < 0.0f) ? -32767.0f : 0.0f);
    return mee_inverse_plain(x, c, l2b);
}

// ---- half-precision op set (fp32 op, one rounding to binary16) --------------

__device__ __forceinline__ float h_add(float a, float b) { return rh(a + b); }
__device__ __forceinline__ float h_sub(float a, float b) { return rh(a - b); }
// The product passes through an empty asm: otherwise "round to binary16 of a * b" is selected as
// v_fma_mixlo_f16 a, b, +0, and (-0) + (+0) turns a negative-zero product into +0.
__device__ __forceinline__ float h_mul(float a, float b)
{
    float p = a * b;
    asm("" : "+v"(p));
    return rh(p);
}
__device__ __forceinline__ float h_div(float a, float b) { return rh(a / b); }
__device__ __forceinline__ float h_max(float a, float b)
{
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}

__device__ __forceinline__ int sr_half(float x, float r)
{
    float fl = __builtin_floorf(x);
    int s = sat_i16(fl);
    float frac = h_sub(x, fl);
    return wrap_i16(s + sat_i16(__builtin_ceilf(h_sub(frac, r))));
}

__device__ __forceinline__ float mee_inverse_half(float x, float c, float l2b)
{
    float a = __builtin_fabsf(x);
    if (!(a > 0.0f)) return 0.0f;
    float arg = h_add(h_div(a, c), 1.0f);
    float lat = h_div(rh(log2_det(arg)), l2b);
    return x < 0.0f ? -lat : lat;
}

// ---- DPP row helpers (row = 16 lanes) ---------------------------------------

template <int CTRL> __device__ __forceinline__ float dpp_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// maximum over the 16 lanes of a DPP row with the fmaxf rule (NaN dropped)
__device__ __forceinline__ float row16_max(float v)
{
    v = __builtin_fmaxf(v, dpp_f32<0xB1>(v));  // quad_perm [1,0,3,2]
    v = __builtin_fmaxf(v, dpp_f32<0x4E>(v));  // quad_perm [2,3,0,1]
    v = __builtin_fmaxf(v, dpp_f32<0x141>(v)); // row_half_mirror
    v = __builtin_fmaxf(v, dpp_f32<0x140>(v)); // row_mirror
    return v;
}

// the same maximum for values that are positive and finite: such floats are ordered like their bit patterns, and an
// integer maximum takes its DPP operand directly (one instruction per step; the float form needs the move and a
// canonicalising maximum in front of every step)
__device__ __forceinline__ float row16_max_pos(float v)
{
    uint32_t u = __float_as_uint(v);
    u = max(u, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)u, 0xB1, 0xf, 0xf, true));
    u = max(u, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)u, 0x4E, 0xf, 0xf, true));
    u = max(u, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)u, 0x141, 0xf, 0xf, true));
    u = max(u, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)u, 0x140, 0xf, 0xf, true));
    return __uint_as_float(u);
}

// parameters of the MEE lattice, built on the host and passed by value
struct MeeParams {
    float c;   // (1+e^2)/(2e^2), binary16 widened
    float cmm; // chunk_max_mee, binary16 widened
    float l2b; // log2(1+2e^2), binary16 widened
    uint32_t pad;
    uint16_t table[256]; // binary16 bit patterns
};

// ---- counter-based random stream ----------------------------------------------------

// Philox4x32-10 (Salmon et al., SC'11): counter c, key (k0, k1)
__host__ __device__ __forceinline__ void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1)
{
#pragma unroll
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// The in-kernel random stream of the scaling quantiser: key = seed, counter = (chunk index, step).
// One block gives the 16 uniform values of one 16-element chunk: element i takes byte i of the four
// output words (little endian), u = (byte | 1) * 2^-8, i.e. the 128 odd multiples of 1/256: centred in
// their cells (a value k/256 would round up with probability ceil(256 f)/256 > f, a bias of 1/512 of a
// step on every element) and exactly representable in binary16, bfloat16 and binary32.
struct RandKey {
    uint64_t seed;
    uint64_t step;
};

__host__ __device__ __forceinline__ void chunk_uniform_words(const RandKey &key, int64_t chunk, uint32_t (&w)[4])
{
    w[0] = (uint32_t)chunk;
    w[1] = (uint32_t)((uint64_t)chunk >> 32);
    w[2] = (uint32_t)key.step;
    w[3] = (uint32_t)(key.step >> 32);
    philox4x32_10(w, (uint32_t)key.seed, (uint32_t)(key.seed >> 32));
}

// v / world, correctly rounded: world = 2^k multiplies by the exact reciprocal; otherwise the product with
// the double reciprocal is within 2^-51 of the quotient, closer than a normal quotient of two binary32 numbers
// can come to a rounding boundary without lying on it.  A subnormal quotient can lie exactly half-way between two
// subnormal numbers (v = m 2^-150 world, m odd): `ties` says that this can happen for the element type and world size
// at hand -- binary32 elements with any world size that is not a power of two, 16-bit elements (multiples of 2^-133
// or 2^-24) only from world = 3 * 2^17 on -- and such quotients then take the division itself.
struct WorldDiv {
    float inv;
    double inv_d;
    int pow2;
    int fuse16; // world = 2^k with k <= 16
    int ties;
    float world;
    __device__ __forceinline__ static bool subnormal(float q) { return (__float_as_uint(q) & 0x7fffffffu) - 1u < 0x007fffffu; }
    __device__ __forceinline__ float operator()(float v) const
    {
        if (pow2) return v * inv;
        float q = (float)((double)v * inv_d);
        if (ties && subnormal(q)) q = v / world;
        return q;
    }
    // sixteen quotients at once when world is not a power of two; the divisions sit behind one branch of the wave (written
    // as a choice per element, both quotients would be computed for every element)
    __device__ __forceinline__ void divide16(float (&v)[16]) const
    {
        float q[16];
#pragma unroll
        for (int k = 0; k < 16; k++) q[k] = (float)((double)v[k] * inv_d);
        if (ties) {
            bool sub = false;
#pragma unroll
            for (int k = 0; k < 16; k++) sub |= __builtin_amdgcn_class(q[k], 0x90); // a subnormal number of either sign
            if (__builtin_amdgcn_ballot_w64(sub) != 0) {
#pragma unroll
                for (int k = 0; k < 16; k++) q[k] = subnormal(q[k]) ? v[k] / world : q[k];
            }
        }
#pragma unroll
        for (int k = 0; k < 16; k++) v[k] = q[k];
    }
    // With fuse16 set, (*this)(v) - mean for a v that came from a 16-bit element is fma(v, inv, -mean): the product with
    // 2^-k is then exact in binary32 (eight or eleven significant bits, no exponent below the binary32 range for world
    // sizes up to 2^16), so the fused operation rounds the same number once.
};

// elem_bytes: 2 or 4
inline WorldDiv make_world_div(int world, int elem_bytes)
{
    WorldDiv wd;
    wd.inv = 1.0f / (float)world;
    wd.inv_d = 1.0 / (double)world;
    wd.pow2 = (world & (world - 1)) == 0;
    wd.fuse16 = wd.pow2 && world <= 65536;
    wd.ties = !wd.pow2 && (elem_bytes == 4 || world >= (3 << 17));
    wd.world = (float)world;
    return wd;
}

// THC's uniform stochastic quantiser (testbed_evaluation/new_comm_hooks/thc_hooks.py:161-166):
// x = clamp((v - lo) / delta, 0, levels - 1); level = floor(x) + (u < x - floor(x))
__device__ __forceinline__ float thc_level(float v, float u, float lo, float delta, float top)
{
    float x = (v - lo) / delta;
    // torch.clamp_ keeps NaN
    if (x < 0.0f) x = 0.0f;
    if (x > top) x = top;
    const float fl = __builtin_floorf(x);
    const float prob = x - fl;
    return fl + ((u < prob) ? 1.0f : 0.0f);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// A 16-byte store of output that this kernel does not read again, with the non-temporal hint: the decoders' element
// stores run a fifth faster with it on a 25 MB bucket (fp32 7.7 -> 6.25 us, bf16 5.6 -> 4.5 us with every launch
// streaming to memory; 6.8 -> 6.0 and 5.4 -> 4.2 us replaying one bucket).  The same hint on the loads costs 15-20 %,
// and on the encoder's small record stream it is within noise either way: neither carries it.
__device__ __forceinline__ void stream_store(uint4 *p, uint4 v)
{
    const u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ void stream_store(float4 *p, float4 v)
{
    const u32x4 t = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4 *>(p));
}


// LDS accesses of one wave execute in order; the fence only stops the compiler
// from moving them across the hand-over between lanes
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// 16-byte slot s of a wave's output tile lives at LDS slot s ^ ((s >> 3) & 7): both
// the per-lane writes (slots S*lane + j) and the lane-contiguous reads (slots
// 64*k + lane) then touch eight distinct bank groups per eight lanes
__device__ __forceinline__ int swz(int s) { return s ^ ((s >> 3) & 7); }

// A wave holds 64 x 16 words, sixteen consecutive ones per lane; they leave as contiguous 16-byte pieces, lane
// after lane.  tile: the wave's 256 LDS slots; dst: where the wave's first word goes (16-byte aligned);
// valid_slots: how many of the 256 pieces lie inside the destination.  Every lane of the wave must call.
__device__ __forceinline__ void store_wave_words16(uint4 *tile, const uint32_t (&w)[16], uint4 *dst, int lane, int valid_slots)
{
#pragma unroll
    for (int j = 0; j < 4; j++) tile[swz(4 * lane + j)] = make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]);
    wave_lds_sync();
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int s = 64 * k + lane;
        if (s < valid_slots) stream_store(dst + s, tile[swz(s)]);
    }
}

// Transposes an 8 x 8 bit matrix held in a 64-bit word: bit 8 i + j becomes bit 8 j + i.  With byte i = the bin
// of element i, byte p of the result holds bit p of the eight bins, element 0 in its lowest bit.
__device__ __forceinline__ uint64_t transpose8x8(uint64_t x)
{
    uint64_t t;
    t = 0x0f0f0f0f00000000ull & (x ^ (x << 28)); x ^= t ^ (t >> 28);
    t = 0x3333000033330000ull & (x ^ (x << 14)); x ^= t ^ (t >> 14);
    t = 0x5500550055005500ull & (x ^ (x << 7));  x ^= t ^ (t >> 7);
    return x;
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// floor(log2(v)) for v >= 1
inline int ilog2(int64_t v)
{
    int k = 0;
    while (((int64_t)1 << (k + 1)) <= v) k++;
    return k;
}

} // namespace dq
