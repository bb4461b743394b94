/*
 * CPU oracle for the eden_utils gradient-compression path -- see dq_oracle.h.
 *
 * TEST INFRASTRUCTURE ONLY: never linked into, loaded by or called from the
 * shipped library.  Scalar C, one thread, written for clarity; it must be
 * compiled with -ffp-contract=off so that the only fused multiply-adds are
 * the explicit fmaf() calls.
 *
 * Pinned by (tests/test_oracle_*.py): closed-form layouts and sizes,
 * single-element probes, all-zero / saturating chunks, rand = 0 / rand = 1
 * rounding direction, unbiasedness of the stochastic rounding, lattice fixed
 * points of the MEE table, FWHT involution and the explicit Sylvester matrix,
 * pack/unpack round trips, an independent numpy restatement of the
 * reference's own functional-test oracle at its tolerances, and golden
 * vectors of randDiag / EdenBinsToBits.
 */
#include "dq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* bit casts and storage formats                                             */
/* ------------------------------------------------------------------------ */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float dqo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* round-to-nearest-even; NaN keeps its sign and top payload bits, quieted */
uint16_t dqo_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float dqo_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0)
            return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31)
        return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t dqo_f32_to_f16(float f)
{
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u)                     /* NaN */
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
    if (a >= 0x477ff000u)                    /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) {                   /* below the smallest normal half */
        /* value / 2^-24 rounded to nearest even integer, 0..1024 */
        float scaled = u2f(a) * 16777216.0f; /* exact: power of two scaling */
        float r = nearbyintf(scaled);        /* default rounding mode = RNE */
        return (uint16_t)(sign | (uint16_t)r);
    }
    uint32_t rounded = a + 0xfffu + ((a >> 13) & 1u);
    return (uint16_t)(sign | (uint16_t)((rounded - 0x38000000u) >> 13));
}

/* value of a half-precision result: one rounding of an fp32 intermediate */
static inline float rh(float x) { return dqo_f16_to_f32(dqo_f32_to_f16(x)); }

static inline float load_elem(const void *p, int dtype, int64_t i)
{
    switch (dtype) {
    case DQO_F16: return dqo_f16_to_f32(((const uint16_t *)p)[i]);
    case DQO_BF16: return dqo_bf16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

static inline void store_elem(void *p, int dtype, int64_t i, float v)
{
    switch (dtype) {
    case DQO_F16: ((uint16_t *)p)[i] = dqo_f32_to_f16(v); break;
    case DQO_BF16: ((uint16_t *)p)[i] = dqo_f32_to_bf16(v); break;
    default: ((float *)p)[i] = v; break;
    }
}

/* value after rounding to the element dtype */
static inline float round_elem(int dtype, float v)
{
    switch (dtype) {
    case DQO_F16: return rh(v);
    case DQO_BF16: return dqo_bf16_to_f32(dqo_f32_to_bf16(v));
    default: return v;
    }
}

/* ------------------------------------------------------------------------ */
/* integer conversions with the device semantics                             */
/* ------------------------------------------------------------------------ */

static inline int sat_i16(float x)   /* float -> int16: truncate, saturate, NaN -> 0 */
{
    if (x != x) return 0;
    if (x >= 32767.0f) return 32767;
    if (x <= -32768.0f) return -32768;
    return (int)x;
}

static inline int sat_u16(float x)
{
    if (x != x) return 0;
    if (x >= 65535.0f) return 65535;
    if (x <= 0.0f) return 0;
    return (int)x;
}

static inline int wrap_i16(int x) { return (int)(int16_t)(uint16_t)(unsigned)x; }

static inline int clamp_code(int signed_val, int range)
{
    if (signed_val < -range) signed_val = -range;
    if (signed_val > range) signed_val = range;
    return signed_val + range;
}

/* ------------------------------------------------------------------------ */
/* deterministic log2                                                        */
/* ------------------------------------------------------------------------ */

float dqo_log2f(float x)
{
    uint32_t ix = f2u(x);
    int k = 0;
    if (ix >= 0x7f800000u) {             /* inf, NaN or negative */
        if (ix == 0x7f800000u) return x;                 /* +inf */
        if ((ix & 0x7fffffffu) > 0x7f800000u) return x + x; /* NaN */
        if ((ix << 1) == 0) return -INFINITY;            /* -0 */
        return u2f(0x7fc00000u);                         /* x < 0 */
    }
    if (ix < 0x00800000u) {              /* zero or subnormal */
        if (ix == 0) return -INFINITY;
        x *= 8388608.0f;                 /* 2^23, exact */
        ix = f2u(x);
        k = -23;
    }
    /* x = 2^k * z with z in [sqrt(1/2), sqrt(2)) */
    uint32_t t = ix - 0x3f3504f3u;
    k += (int)((int32_t)t >> 23);
    float z = u2f(ix - (t & 0xff800000u));
    float f = z - 1.0f;
    /* log2(1+f) = f*log2(e) + f^2 * Q(f), Q of degree 8 */
    float q = -0x1.d0dd08p-4f;
    q = fmaf(q, f, 0x1.7ad622p-3f);
    q = fmaf(q, f, -0x1.831b24p-3f);
    q = fmaf(q, f, 0x1.a33bdap-3f);
    q = fmaf(q, f, -0x1.eb492p-3f);
    q = fmaf(q, f, 0x1.277e38p-2f);
    q = fmaf(q, f, -0x1.715762p-2f);
    q = fmaf(q, f, 0x1.ec7092p-2f);
    q = fmaf(q, f, -0x1.715476p-1f);
    float p = (f * f) * q;
    float r = fmaf(f, 0x1.4ae0cp-26f, p);
    r = fmaf(f, 0x1.715476p+0f, r);
    return (float)k + r;
}

/* ------------------------------------------------------------------------ */
/* sizes and validation                                                      */
/* ------------------------------------------------------------------------ */

int64_t dqo_scaling_required_bytes(int64_t n, int nbits, int chunk_size, int strategy)
{
    int64_t chunks = n / chunk_size;
    int64_t packed = ((int64_t)chunk_size * nbits) >> 3;
    if (strategy >= 2)
        return (chunks / 16) * (16 * (packed + 1) + 2);
    return chunks * (packed + 2);
}

int dqo_scaling_check(int64_t n, int nbits, int chunk_size, int strategy, int strict)
{
    if (!(n > 0)) return DQO_ERR_N;
    if (strict) {
        if (!(nbits == 2 || nbits == 4 || nbits == 8)) return DQO_ERR_NBITS;
    } else if (nbits < 2 || nbits > 8) {
        return DQO_ERR_NBITS;
    }
    if (strategy < 0 || strategy > 3) return DQO_ERR_STRATEGY;
    if (!(chunk_size > 0 && chunk_size <= 32)) return DQO_ERR_CHUNK_RANGE;
    if ((chunk_size & (chunk_size - 1)) != 0) return DQO_ERR_CHUNK_POW2;
    if ((chunk_size * nbits) % 8 != 0) return DQO_ERR_CHUNK_BITS;
    if (n % chunk_size != 0) return DQO_ERR_N_CHUNK;
    if (strategy >= 2 && (n / chunk_size) % 16 != 0) return DQO_ERR_N_SUPER;
    return DQO_OK;
}

/* ------------------------------------------------------------------------ */
/* MEE lookup table                                                          */
/* ------------------------------------------------------------------------ */

static const float k_mee_eps[9] = {0.0f, 0.23f, 0.23f, 0.18f, 0.18f, 0.18f, 0.1f, 0.1f, 0.1f};

void dqo_mee_lut(int nbits, uint16_t table[256], uint16_t params[4])
{
    memset(table, 0, 256 * sizeof(uint16_t));
    float eps = k_mee_eps[nbits];
    /* host fp32 arithmetic, left to right, no contraction */
    float two_eps2 = 2.0f * eps * eps;
    float one_plus_2eps2 = 1.0f + two_eps2;
    float one_plus_eps2 = 1.0f + eps * eps;
    params[0] = dqo_f32_to_f16(one_plus_2eps2);
    params[1] = dqo_f32_to_f16(one_plus_eps2 / two_eps2);
    /* the host build evaluates log2f with the C library */
    params[3] = dqo_f32_to_f16(log2f(one_plus_2eps2));

    int anchor = (1 << (nbits - 1)) - 1;
    float pw = 1.0f;
    table[anchor] = dqo_f32_to_f16(0.0f);
    for (int j = 1; j <= anchor; j++) {
        pw *= one_plus_2eps2;
        float rep = (pw - 1.0f) / two_eps2 * one_plus_eps2;
        table[anchor + j] = dqo_f32_to_f16(rep);
        table[anchor - j] = dqo_f32_to_f16(-rep);
    }
    params[2] = table[anchor * 2];
}

/* ------------------------------------------------------------------------ */
/* bf16 / fp32 arithmetic path (fp32 math)                                   */
/* ------------------------------------------------------------------------ */

static const float k_min_pos = 1.0e-30f;

static inline float pos_scale(float v)          /* cuda_hierarchical_mee.cu:28-31 */
{
    if (!isfinite(v)) v = k_min_pos;
    return fmaxf(v, k_min_pos);
}

static inline float nonneg_scale(float v)       /* cuda_hierarchical_mee.cu:33-36 */
{
    if (!isfinite(v)) v = 0.0f;
    return fmaxf(v, 0.0f);
}

/* cuda_hadamard.cu:750-755: no guards */
static inline int sr_float_plain(float x, float r)
{
    float fl = floorf(x);
    int s = sat_i16(fl);
    s = wrap_i16(s + sat_i16(ceilf((x - fl) - r)));
    return s;
}

/* cuda_hierarchical_mee.cu:117-138 */
static inline int sr_float_guarded(float x, float r)
{
    if (!isfinite(x)) {
        if (x > 0.0f) return 32767;
        if (x < 0.0f) return -32767;
        return 0;
    }
    if (x >= 32767.0f) return 32767;
    if (x <= -32767.0f) return -32767;
    if (!isfinite(r)) r = 0.0f;
    return sr_float_plain(x, r);
}

/* cuda_hadamard.cu:757-765 */
static inline float mee_inverse_plain(float x, float c, float l2b)
{
    float a = fabsf(x);
    if (!(a > 0.0f)) return 0.0f;
    float lat = dqo_log2f(a / c + 1.0f) / l2b;
    return x < 0.0f ? -lat : lat;
}

/* cuda_hierarchical_mee.cu:140-157 */
static inline float mee_inverse_guarded(float x, float c, float l2b)
{
    if (!isfinite(x)) {
        if (x > 0.0f) return 32767.0f;
        if (x < 0.0f) return -32767.0f;
        return 0.0f;
    }
    return mee_inverse_plain(x, c, l2b);
}

/* max |v| over a chunk with the fmaxf rule (a NaN operand is dropped) */
static inline float chunk_absmax_f32(const float *v, int c)
{
    float m = fabsf(v[0]);
    for (int i = 1; i < c; i++) m = fmaxf(m, fabsf(v[i]));
    return m;
}

static inline void put_code(uint8_t *chunk_bytes, int i, int nbits, int code)
{
    int bit = i * nbits;
    unsigned v = (unsigned)code << (bit & 7);
    chunk_bytes[bit >> 3] |= (uint8_t)v;
    if ((bit & 7) + nbits > 8)
        chunk_bytes[(bit >> 3) + 1] |= (uint8_t)(v >> 8);
}

static inline int get_code(const uint8_t *chunk_bytes, int i, int nbits)
{
    int bit = i * nbits;
    unsigned v = chunk_bytes[bit >> 3];
    if ((bit & 7) + nbits > 8)
        v |= (unsigned)chunk_bytes[(bit >> 3) + 1] << 8;
    return (int)((v >> (bit & 7)) & ((1u << nbits) - 1u));
}

typedef struct {
    int mee;
    float c;    /* one_plus_eps2_over_2eps2, half widened */
    float cmm;  /* chunk_max_mee, half widened            */
    float l2b;  /* log2_one_plus_2eps2, half widened      */
    float table[256];
    uint16_t table_h[256];
} mee_ctx;

static void mee_ctx_init(mee_ctx *m, int nbits, int mee)
{
    m->mee = mee;
    if (!mee) return;
    uint16_t params[4];
    dqo_mee_lut(nbits, m->table_h, params);
    m->c = dqo_f16_to_f32(params[1]);
    m->cmm = dqo_f16_to_f32(params[2]);
    m->l2b = dqo_f16_to_f32(params[3]);
    for (int i = 0; i < 256; i++) m->table[i] = dqo_f16_to_f32(m->table_h[i]);
}

/* one hierarchical superchunk, fp32 math; vals/rnd hold 16*C widened inputs */
static void hier_compress_f32(const float *vals, const float *rnd, uint8_t *rec,
                              int nbits, int C, const mee_ctx *m)
{
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int CB = PB + 1;
    float s[16];
    for (int j = 0; j < 16; j++) {
        float a = chunk_absmax_f32(vals + j * C, C);
        if (m->mee)
            s[j] = pos_scale(a / pos_scale(m->cmm) + 1e-7f);
        else
            s[j] = pos_scale(a / (float)R + 1e-7f);
    }
    float g = s[0];
    for (int j = 1; j < 16; j++) g = fmaxf(g, s[j]);
    g = pos_scale(g);
    uint16_t ustore = dqo_f32_to_bf16(pos_scale(g / 255.0f));
    float unit = pos_scale(dqo_bf16_to_f32(ustore));
    rec[16 * CB] = (uint8_t)(ustore & 0xff);
    rec[16 * CB + 1] = (uint8_t)(ustore >> 8);

    for (int j = 0; j < 16; j++) {
        float ratio = pos_scale(s[j]) / pos_scale(g) * 255.0f;
        if (!isfinite(ratio)) ratio = ratio > 0.0f ? 255.0f : 1.0f;
        int q = sat_u16(ceilf(ratio));
        if (q < 1) q = 1;
        if (q > 255) q = 255;
        uint8_t *cb = rec + j * CB;
        memset(cb, 0, (size_t)PB);
        cb[PB] = (uint8_t)q;
        float d = pos_scale((float)q * unit);
        float dd = pos_scale(d);
        for (int i = 0; i < C; i++) {
            float x = vals[j * C + i] / dd;
            if (m->mee) x = mee_inverse_guarded(x, m->c, m->l2b);
            int code = clamp_code(sr_float_guarded(x, rnd[j * C + i]), R);
            put_code(cb, i, nbits, code);
        }
    }
}

/* decode one hierarchical superchunk to fp32 values (fma with acc when add) */
static void hier_decode_f32(const uint8_t *rec, float *out, const float *acc,
                            int nbits, int C, const mee_ctx *m)
{
    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int CB = PB + 1;
    uint16_t ubits = (uint16_t)(rec[16 * CB] | ((uint16_t)rec[16 * CB + 1] << 8));
    float us = nonneg_scale(dqo_bf16_to_f32(ubits));
    for (int j = 0; j < 16; j++) {
        const uint8_t *cb = rec + j * CB;
        float sc = nonneg_scale((float)cb[PB] * us);
        for (int i = 0; i < C; i++) {
            int code = get_code(cb, i, nbits);
            float lev = m->mee ? m->table[code] : (float)(code - R);
            out[j * C + i] = acc ? fmaf(lev, sc, acc[j * C + i]) : lev * sc;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* fp16 arithmetic path (every intermediate rounded to binary16)             */
/* ------------------------------------------------------------------------ */

static inline float h_add(float a, float b) { return rh(a + b); }
static inline float h_sub(float a, float b) { return rh(a - b); }
static inline float h_mul(float a, float b) { return rh(a * b); }
static inline float h_div(float a, float b) { return rh(a / b); }
static inline float h_max(float a, float b)
{
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}
static inline float h_log2(float a) { return rh(dqo_log2f(a)); }

/* cuda_hadamard.cu:713-719 / cuda_hierarchical_mee.cu:80-86 */
static inline int sr_half(float x, float r)
{
    float fl = floorf(x);
    int s = sat_i16(fl);                     /* __half2short_rd of an integer */
    float frac = h_sub(x, fl);
    s = wrap_i16(s + sat_i16(ceilf(h_sub(frac, r))));   /* __half2short_ru */
    return s;
}

/* cuda_hadamard.cu:731-740 / cuda_hierarchical_mee.cu:98-107 */
static inline float mee_inverse_half(float x, float c, float l2b)
{
    float a = fabsf(x);
    if (!(a > 0.0f)) return 0.0f;
    float arg = h_add(h_div(a, c), 1.0f);
    float lat = h_div(h_log2(arg), l2b);
    return x < 0.0f ? -lat : lat;
}

static inline float chunk_absmax_half(const float *v, int c)
{
    float m = fabsf(v[0]);
    for (int i = 1; i < c; i++) m = h_max(m, fabsf(v[i]));
    return m;
}

/* ------------------------------------------------------------------------ */
/* scaling_compress                                                          */
/* ------------------------------------------------------------------------ */

int dqo_scaling_compress(const void *src, uint8_t *dst, const void *rand_pool,
                         int64_t n, int nbits, int C, int strategy, int dtype)
{
    int rc = dqo_scaling_check(n, nbits, C, strategy, 0);
    if (rc) return rc;
    if (dtype < DQO_F16 || dtype > DQO_F32) return DQO_ERR_DTYPE;

    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int mee = (strategy == 1 || strategy == 3);
    mee_ctx m;
    mee_ctx_init(&m, nbits, mee);
    const float eps_h = dqo_f16_to_f32(dqo_f32_to_f16(1e-7f));
    const float c_h = mee ? m.c : 0.0f, cmm_h = mee ? m.cmm : 0.0f, l2b_h = mee ? m.l2b : 0.0f;

    float vals[16 * 32], rnd[16 * 32];

    if (strategy >= 2) {
        const int CB = PB + 1;
        const int64_t REC = 16 * CB + 2;
        const int64_t nsc = n / (16 * (int64_t)C);
        for (int64_t S = 0; S < nsc; S++) {
            int64_t base = S * 16 * C;
            for (int i = 0; i < 16 * C; i++) {
                vals[i] = load_elem(src, dtype, base + i);
                rnd[i] = load_elem(rand_pool, dtype, base + i);
            }
            uint8_t *rec = dst + S * REC;
            if (dtype != DQO_F16) {
                hier_compress_f32(vals, rnd, rec, nbits, C, &m);
                continue;
            }
            /* fp16: cuda_hierarchical_mee.cu:698-774 (AEE), 844-930 (MEE) */
            float s[16];
            for (int j = 0; j < 16; j++) {
                float a = chunk_absmax_half(vals + j * C, C);
                float div = mee ? cmm_h : (float)R;      /* R exact in half */
                s[j] = h_add(h_div(a, div), eps_h);
            }
            float g = s[0];
            for (int j = 1; j < 16; j++) g = h_max(g, s[j]);
            float unit = h_div(g, 255.0f);
            uint16_t ub = dqo_f32_to_f16(unit);
            rec[16 * CB] = (uint8_t)(ub & 0xff);
            rec[16 * CB + 1] = (uint8_t)(ub >> 8);
            for (int j = 0; j < 16; j++) {
                int q = sat_u16(ceilf(h_mul(h_div(s[j], g), 255.0f)));
                if (q > 255) q = 255;
                float d = h_mul((float)q, unit);       /* q <= 255 exact in half */
                uint8_t *cb = rec + j * CB;
                memset(cb, 0, (size_t)PB);
                cb[PB] = (uint8_t)q;
                for (int i = 0; i < C; i++) {
                    float x = h_div(vals[j * C + i], d);
                    if (mee) x = mee_inverse_half(x, c_h, l2b_h);
                    put_code(cb, i, nbits, clamp_code(sr_half(x, rnd[j * C + i]), R));
                }
            }
        }
        return DQO_OK;
    }

    /* flat layout: PB code bytes then a 2-byte scale per chunk */
    const int64_t nchunks = n / C;
    for (int64_t k = 0; k < nchunks; k++) {
        int64_t base = k * C;
        for (int i = 0; i < C; i++) {
            vals[i] = load_elem(src, dtype, base + i);
            rnd[i] = load_elem(rand_pool, dtype, base + i);
        }
        uint8_t *cb = dst + k * (PB + 2);
        memset(cb, 0, (size_t)PB);
        if (dtype == DQO_F16) {
            /* cuda_hadamard.cu:768-817 (AEE), 941-997 (MEE) */
            float a = chunk_absmax_half(vals, C);
            float scale = h_add(h_div(a, mee ? cmm_h : (float)R), eps_h);
            uint16_t sb = dqo_f32_to_f16(scale);
            cb[PB] = (uint8_t)(sb & 0xff);
            cb[PB + 1] = (uint8_t)(sb >> 8);
            for (int i = 0; i < C; i++) {
                float x = h_div(vals[i], scale);
                if (mee) x = mee_inverse_half(x, c_h, l2b_h);
                put_code(cb, i, nbits, clamp_code(sr_half(x, rnd[i]), R));
            }
        } else {
            /* cuda_hadamard.cu:1055-1094 (AEE), 1138-1178 (MEE) */
            float a = chunk_absmax_f32(vals, C);
            uint16_t sb = dqo_f32_to_bf16(a / (mee ? m.cmm : (float)R) + 1e-7f);
            float scale = dqo_bf16_to_f32(sb);
            cb[PB] = (uint8_t)(sb & 0xff);
            cb[PB + 1] = (uint8_t)(sb >> 8);
            for (int i = 0; i < C; i++) {
                float x = vals[i] / scale;
                if (mee) x = mee_inverse_plain(x, m.c, m.l2b);
                put_code(cb, i, nbits, clamp_code(sr_float_plain(x, rnd[i]), R));
            }
        }
    }
    return DQO_OK;
}

/* ------------------------------------------------------------------------ */
/* scaling_decompress / scaling_decompress_add                               */
/* ------------------------------------------------------------------------ */

int dqo_scaling_decompress(const uint8_t *src, void *dst, int64_t n, int nbits,
                           int C, int strategy, int dtype, int add_original)
{
    int rc = dqo_scaling_check(n, nbits, C, strategy, 0);
    if (rc) return rc;
    if (dtype < DQO_F16 || dtype > DQO_F32) return DQO_ERR_DTYPE;

    const int R = (1 << (nbits - 1)) - 1;
    const int PB = (C * nbits) >> 3;
    const int mee = (strategy == 1 || strategy == 3);
    mee_ctx m;
    mee_ctx_init(&m, nbits, mee);
    float out[16 * 32], acc[16 * 32];

    if (strategy >= 2) {
        const int CB = PB + 1;
        const int64_t REC = 16 * CB + 2;
        const int64_t nsc = n / (16 * (int64_t)C);
        for (int64_t S = 0; S < nsc; S++) {
            const uint8_t *rec = src + S * REC;
            int64_t base = S * 16 * C;
            if (dtype != DQO_F16) {
                if (add_original)
                    for (int i = 0; i < 16 * C; i++) acc[i] = load_elem(dst, dtype, base + i);
                hier_decode_f32(rec, out, add_original ? acc : NULL, nbits, C, &m);
                for (int i = 0; i < 16 * C; i++) store_elem(dst, dtype, base + i, out[i]);
                continue;
            }
            /* fp16: cuda_hierarchical_mee.cu:776-842 (AEE), 932-1014 (MEE) */
            uint16_t ub = (uint16_t)(rec[16 * CB] | ((uint16_t)rec[16 * CB + 1] << 8));
            float unit = dqo_f16_to_f32(ub);
            for (int j = 0; j < 16; j++) {
                const uint8_t *cb = rec + j * CB;
                float sc = h_mul((float)cb[PB], unit);
                for (int i = 0; i < C; i++) {
                    int code = get_code(cb, i, nbits);
                    float lev = mee ? m.table[code] : (float)(code - R);
                    float v = h_mul(lev, sc);
                    if (add_original) v = h_add(load_elem(dst, dtype, base + j * C + i), v);
                    store_elem(dst, dtype, base + j * C + i, v);
                }
            }
        }
        return DQO_OK;
    }

    const int64_t nchunks = n / C;
    for (int64_t k = 0; k < nchunks; k++) {
        const uint8_t *cb = src + k * (PB + 2);
        uint16_t sb = (uint16_t)(cb[PB] | ((uint16_t)cb[PB + 1] << 8));
        int64_t base = k * C;
        if (dtype == DQO_F16) {
            /* cuda_hadamard.cu:819-861 (AEE), 999-1053 (MEE) */
            float sc = dqo_f16_to_f32(sb);
            for (int i = 0; i < C; i++) {
                int code = get_code(cb, i, nbits);
                float lev = mee ? m.table[code] : (float)(code - R);
                float v = h_mul(lev, sc);
                if (add_original) v = h_add(load_elem(dst, dtype, base + i), v);
                store_elem(dst, dtype, base + i, v);
            }
        } else {
            /* cuda_hadamard.cu:1096-1136 (AEE), 1180-1234 (MEE): no guards */
            float sc = dqo_bf16_to_f32(sb);
            for (int i = 0; i < C; i++) {
                int code = get_code(cb, i, nbits);
                float lev = mee ? m.table[code] : (float)(code - R);
                float v = add_original ? fmaf(lev, sc, load_elem(dst, dtype, base + i)) : lev * sc;
                store_elem(dst, dtype, base + i, v);
            }
        }
    }
    return DQO_OK;
}

/* ------------------------------------------------------------------------ */
/* scaling_dec_comp                                                          */
/* ------------------------------------------------------------------------ */

int dqo_scaling_dec_comp(const uint8_t *recv, void *inp, uint8_t *send, const void *rand_pool,
                         int64_t n, int nbits, int C, int strategy, int dtype)
{
    int rc = dqo_scaling_check(n, nbits, C, strategy, 0);
    if (rc) return rc;
    if (dtype < DQO_F16 || dtype > DQO_F32) return DQO_ERR_DTYPE;

    if (dtype != DQO_F16 && C == 16 && strategy >= 2) {
        /* fused: cuda_hierarchical_mee.cu:526-696; inp is read-only */
        const int PB = (C * nbits) >> 3;
        const int64_t REC = 16 * (PB + 1) + 2;
        const int64_t nsc = n / 256;
        mee_ctx m;
        mee_ctx_init(&m, nbits, strategy == 3);
        float acc[256], t[256], rnd[256];
        for (int64_t S = 0; S < nsc; S++) {
            for (int i = 0; i < 256; i++) {
                acc[i] = load_elem(inp, dtype, S * 256 + i);
                rnd[i] = load_elem(rand_pool, dtype, S * 256 + i);
            }
            hier_decode_f32(recv + S * REC, t, acc, nbits, C, &m);
            for (int i = 0; i < 256; i++) t[i] = round_elem(dtype, t[i]);
            hier_compress_f32(t, rnd, send + S * REC, nbits, C, &m);
        }
        return DQO_OK;
    }
    /* split: eden_utils.cpp:212-214, cuda_hadamard.cu:1744-1747 (writes inp) */
    rc = dqo_scaling_decompress(recv, inp, n, nbits, C, strategy, dtype, 1);
    if (rc) return rc;
    return dqo_scaling_compress(inp, send, rand_pool, n, nbits, C, strategy, dtype);
}

/* ------------------------------------------------------------------------ */
/* superchunk mean-centre / add-mean                                         */
/* ------------------------------------------------------------------------ */

static void mean_center_impl(const void *src, void *residual, uint16_t *stats, float *mean_out,
                             int64_t n, int world_size, int dtype)
{
    const int64_t nsc = (n + 255) / 256;
    float sum[256], sq[256], val[256];
    for (int64_t b = 0; b < nsc; b++) {
        int64_t start = b * 256;
        int64_t valid = n - start;
        if (valid > 256) valid = 256;
        if (valid < 0) valid = 0;
        for (int l = 0; l < 256; l++) {
            float v = 0.0f;
            if (l < valid) v = load_elem(src, dtype, start + l) / (float)world_size;
            val[l] = v;
            sum[l] = v;
            sq[l] = v * v;
        }
        for (int stride = 128; stride > 0; stride >>= 1)
            for (int l = 0; l < stride; l++) {
                sum[l] += sum[l + stride];
                sq[l] += sq[l + stride];
            }
        float mean = valid > 0 ? sum[0] / (float)valid : 0.0f;
        if (residual)
            for (int l = 0; l < 256; l++)
                store_elem(residual, dtype, start + l, l < valid ? val[l] - mean : 0.0f);
        stats[2 * b] = dqo_f32_to_bf16(mean);
        stats[2 * b + 1] = dqo_f32_to_bf16(sq[0]);
        if (mean_out) mean_out[b] = mean;
    }
}

void dqo_superchunk_mean_center(const void *src, void *residual, uint16_t *stats,
                                int64_t n, int world_size, int dtype)
{
    mean_center_impl(src, residual, stats, NULL, n, world_size, dtype);
}

void dqo_superchunk_stats(const void *src, uint16_t *stats, float *mean, int64_t n, int world_size, int dtype)
{
    mean_center_impl(src, NULL, stats, mean, n, world_size, dtype);
}

void dqo_superchunk_add_mean_copy(const void *residual, void *dst, const uint16_t *stats,
                                  int64_t n, int dtype)
{
    for (int64_t i = 0; i < n; i++) {
        float mean = dqo_bf16_to_f32(stats[2 * (i >> 8)]);
        store_elem(dst, dtype, i, load_elem(residual, dtype, i) + mean);
    }
}

/* ------------------------------------------------------------------------ */
/* Walsh-Hadamard                                                            */
/* ------------------------------------------------------------------------ */

void dqo_fwht(float *x, int64_t n)
{
    for (int64_t h = 1; h < n; h <<= 1)
        for (int64_t i = 0; i < n; i += h << 1)
            for (int64_t j = i; j < i + h; j++) {
                float a = x[j], b = x[j + h];
                x[j] = a + b;
                x[j + h] = a - b;
            }
}

void dqo_rht_blocked(float *x, const float *sign, int64_t n, int64_t block, float scale, int inverse)
{
    for (int64_t b = 0; b + block <= n; b += block) {
        float *v = x + b;
        const float *s = sign + b;
        if (!inverse)
            for (int64_t i = 0; i < block; i++) v[i] = v[i] * s[i];
        dqo_fwht(v, block);
        for (int64_t i = 0; i < block; i++) v[i] = v[i] * scale;
        if (inverse)
            for (int64_t i = 0; i < block; i++) v[i] = v[i] * s[i];
    }
}

/* ------------------------------------------------------------------------ */
/* randDiag                                                                  */
/* ------------------------------------------------------------------------ */

void dqo_rand_diag(float *out, int64_t size, int64_t seed)
{
    const int64_t M = 0xffffffffLL;
    const int64_t s8 = size / 8 + (size % 8 != 0);
    /* int64 wrap-around arithmetic, as torch/python-int then & mask */
    uint64_t ss = ((uint64_t)seed * 1664525u + 1013904223u) & (uint64_t)M;
    ss = (ss * 8121u + 28411u) & (uint64_t)M;
    for (int64_t j = 0; j < s8; j++) {
        uint64_t r = (uint64_t)j + ss;
        r = (1103515245u * r + 12345u + ss) & (uint64_t)M;
        r = (1140671485u * r + 12820163u + ss) & (uint64_t)M;
        r += 0x9e3779b9u;                     /* may carry into bit 32 */
        r = ((r ^ (r >> 16)) * 0x85ebca6bu) & (uint64_t)M;
        r = ((r ^ (r >> 13)) * 0xc2b2ae35u) & (uint64_t)M;
        r = (r ^ (r >> 16)) & (uint64_t)M;
        for (int k = 0; k < 8; k++) {
            int64_t idx = (int64_t)k * s8 + j;
            if (idx < size)
                out[idx] = ((r >> (4 * k)) & 15u) >= 8u ? 1.0f : -1.0f;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* EDEN bit-plane packing                                                    */
/* ------------------------------------------------------------------------ */

void dqo_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int nbits)
{
    const int64_t words = nbins >> 5;
    for (int p = 0; p < nbits; p++)
        for (int64_t w = 0; w < words; w++) {
            uint32_t acc = 0;
            for (int t = 0; t < 32; t++)
                acc |= (((uint32_t)bins[32 * w + t] >> p) & 1u) << t;
            arr[(int64_t)p * words + w] = acc;
        }
}

void dqo_bits_to_bins(const uint32_t *arr, int64_t narr, int32_t *bins, int nbits)
{
    const int64_t words = narr / nbits;
    for (int64_t w = 0; w < words; w++)
        for (int t = 0; t < 32; t++) {
            int32_t v = 0;
            for (int p = 0; p < nbits; p++)
                if (arr[(int64_t)p * words + w] & (1u << t)) v += 1 << p;
            bins[32 * w + t] = v;
        }
}

/* ------------------------------------------------------------------------ */
/* counter-based random stream of the in-kernel rounding                     */
/* ------------------------------------------------------------------------ */

/* Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11) */
void dqo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* element e: block with key = seed, counter = (chunk e / 16, step); u = (byte e % 16 of the four output
 * words, little endian, with its low bit set) * 2^-8: the odd multiples of 1/256 */
void dqo_philox_uniform(float *out, int64_t n, uint64_t seed, uint64_t step)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    for (int64_t chunk = 0; chunk * 16 < n; chunk++) {
        const uint32_t ctr[4] = {(uint32_t)chunk, (uint32_t)((uint64_t)chunk >> 32), (uint32_t)step, (uint32_t)(step >> 32)};
        uint32_t w[4];
        dqo_philox4x32_10(ctr, key, w);
        for (int i = 0; i < 16 && chunk * 16 + i < n; i++)
            out[chunk * 16 + i] = (float)(((w[i >> 2] >> (8 * (i & 3))) & 0xffu) | 1u) * 0.00390625f;
    }
}

/* the same stream for a list of superchunks: out[256 k + e] = the value of element 256 rows[k] + e */
void dqo_philox_uniform_rows(float *out, const int64_t *rows, int64_t nrows, uint64_t seed, uint64_t step)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    for (int64_t k = 0; k < nrows; k++) {
        for (int j = 0; j < 16; j++) {
            const int64_t chunk = rows[k] * 16 + j;
            const uint32_t ctr[4] = {(uint32_t)chunk, (uint32_t)((uint64_t)chunk >> 32), (uint32_t)step, (uint32_t)(step >> 32)};
            uint32_t w[4];
            dqo_philox4x32_10(ctr, key, w);
            for (int i = 0; i < 16; i++)
                out[k * 256 + j * 16 + i] = (float)(((w[i >> 2] >> (8 * (i & 3))) & 0xffu) | 1u) * 0.00390625f;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* EDEN Lloyd-Max quantiser, THC uniform quantiser                           */
/* ------------------------------------------------------------------------ */

/* sum of term(i), i < n, in double: tiles of 4096 indices, inside a tile 256 lanes that add
 * indices lane + 256 k (k ascending), a halving tree over the lanes (stride 128 .. 1); the tile
 * sums are folded the same way (lane adds tiles lane + 256 k, then the tree).  torch leaves the
 * order of its reductions unspecified; this is the order the library documents for itself. */
typedef double (*dqo_term_fn)(int64_t i, void *ctx);

static double halve256(double *lane)
{
    for (int stride = 128; stride > 0; stride >>= 1)
        for (int l = 0; l < stride; l++) lane[l] += lane[l + stride];
    return lane[0];
}

/* consecutive == 0: lane l of a tile adds elements l + 256 k; otherwise elements 16 l + k (k ascending either way) */
static double tiled_sum(int64_t n, dqo_term_fn term, void *ctx, int consecutive)
{
    const int64_t tiles = (n + 4095) / 4096;
    double *tile_sum = (double *)malloc((size_t)tiles * sizeof(double));
    double lane[256];
    for (int64_t b = 0; b < tiles; b++) {
        for (int l = 0; l < 256; l++) {
            double acc = 0.0;
            for (int k = 0; k < 16; k++) {
                int64_t i = b * 4096 + (consecutive ? 16 * l + k : l + 256 * k);
                if (i < n) acc += term(i, ctx);
            }
            lane[l] = acc;
        }
        tile_sum[b] = halve256(lane);
    }
    for (int l = 0; l < 256; l++) {
        double acc = 0.0;
        for (int64_t i = l; i < tiles; i += 256) acc += tile_sum[i];
        lane[l] = acc;
    }
    free(tile_sum);
    return halve256(lane);
}

struct eden_ctx { const float *vec; const float *cen; const int32_t *bins; };
static double term_sq(int64_t i, void *c) { double v = (double)((struct eden_ctx *)c)->vec[i]; return v * v; }
static double term_dot(int64_t i, void *c)
{
    struct eden_ctx *e = (struct eden_ctx *)c;
    return (double)e->cen[e->bins[i]] * (double)e->vec[i];
}

/* srrcomp.py:356-361: bins = bucketize(vec * sqrt(n) / ||vec||, boundaries) with right=False, i.e. the
 * number of boundaries strictly below the value (a NaN value, 0/0 of an all-zero slice, lands in the last bin as in
 * torch's lower-bound search); scale = ||vec||^2 / <centroids[bins], vec>.
 * result = {sum of squares, dot, scale, norm}. */
void dqo_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids, int nbits,
                       int32_t *bins, float *result)
{
    const int nb = (1 << nbits) - 1;
    struct eden_ctx ctx = {vec, centroids, bins};
    const float sumsq = (float)tiled_sum(n, term_sq, &ctx, 0);
    const float norm = sqrtf(sumsq);
    const float sqrt_n = (float)sqrt((double)n);
    for (int64_t i = 0; i < n; i++) {
        const float x = (vec[i] * sqrt_n) / norm;
        int b = 0;
        while (b < nb && !(boundaries[b] >= x)) b++; /* torch's lower bound: NaN passes every boundary */
        bins[i] = b;
    }
    const float dot = (float)tiled_sum(n, term_dot, &ctx, 1);
    result[0] = sumsq;
    result[1] = dot;
    result[2] = (norm * norm) / dot;
    result[3] = norm;
}

/* srrcomp.py:343-345 */
void dqo_eden_dequantize(const int32_t *bins, int64_t n, const float *centroids, float *out)
{
    for (int64_t i = 0; i < n; i++) out[i] = centroids[bins[i]];
}

/* thc_hooks.py:161-166 with the Bernoulli draw given as a uniform value: 1 when uniform < probability */
void dqo_thc_quantize(const float *rotated, const float *uniform, uint16_t *levels_bf16, int64_t n, float lo,
                      float delta, int levels)
{
    const float top = (float)(levels - 1);
    for (int64_t i = 0; i < n; i++) {
        float x = (rotated[i] - lo) / delta;
        if (x < 0.0f) x = 0.0f;
        if (x > top) x = top;
        const float fl = floorf(x);
        const float prob = x - fl;
        levels_bf16[i] = dqo_f32_to_bf16(fl + (uniform[i] < prob ? 1.0f : 0.0f));
    }
}

/* thc_hooks.py:176-178 */
void dqo_thc_dequantize(const uint16_t *levels_bf16, float *out, int64_t n, float step, float lo)
{
    for (int64_t i = 0; i < n; i++) {
        const float prod = dqo_bf16_to_f32(levels_bf16[i]) * step;
        out[i] = prod + lo;
    }
}

/* ------------------------------------------------------------------------ */
/* dynamic bit-width rule                                                    */
/* ------------------------------------------------------------------------ */

static inline float rb(float x) { return dqo_bf16_to_f32(dqo_f32_to_bf16(x)); }

void dqo_dynamic_bitrate_qbits(const uint16_t *norms_bf16, int64_t stride, int64_t count,
                               double u, int64_t *qbits)
{
    const float eps = 1e-20f;
    const float norm_scale = (float)(4.0 / (512.0 / 17.0));
    for (int64_t i = 0; i < count; i++) {
        float x = dqo_bf16_to_f32(norms_bf16[i * stride]);
        x = (x != x) ? x : rb(x > eps ? x : eps);          /* clamp(min=eps)  */
        x = rb(dqo_log2f(x));                              /* log2            */
        x = rb(x * norm_scale);                            /* mul             */
        x = rb(x + (float)u);                              /* add             */
        x = (x != x) ? x : rb(x > eps ? x : eps);          /* clamp(min=eps)  */
        x = rb(dqo_log2f(x));                              /* log2            */
        x = floorf(x);                                     /* floor           */
        /* .to(torch.int64) on the device saturates (+inf -> INT64_MAX) and sends NaN below the clamp */
        int64_t z = (x != x) ? 1 : (x < 1.0f ? 1 : (x > 3.0f ? 3 : (int64_t)x));
        qbits[i] = (int64_t)1 << z;
    }
}

/* ------------------------------------------------------------------------ */
/* fixed-proportion groups                                                   */
/* ------------------------------------------------------------------------ */

/* torch.sort's order on floats, descending: NaN above every number, then the usual >; equal values
 * (including -0 and +0) are ties */
static int sorts_before(float a, float b)
{
    const int an = a != a, bn = b != b;
    if (an || bn) return an && !bn;
    return a > b;
}

/* testbed_evaluation/new_comm_hooks/comm_hooks.py:718: torch.argsort(norms, descending=True, stable=True)
 * on the bf16 norms widened to float, as a bottom-up merge sort on the comparison itself (ties keep the
 * left run's element first = ascending index). */
void dqo_argsort_descending_stable(const uint16_t *norms_bf16, int64_t stride, int64_t count, int64_t *order)
{
    if (count <= 0) return;
    int64_t *a = order, *b = (int64_t *)malloc(sizeof(int64_t) * (size_t)count);
    for (int64_t i = 0; i < count; i++) a[i] = i;
    for (int64_t width = 1; width < count; width *= 2) {
        for (int64_t lo = 0; lo < count; lo += 2 * width) {
            const int64_t mid = lo + width < count ? lo + width : count;
            const int64_t hi = lo + 2 * width < count ? lo + 2 * width : count;
            int64_t l = lo, r = mid, k = lo;
            while (l < mid && r < hi) {
                const float vl = dqo_bf16_to_f32(norms_bf16[a[l] * stride]);
                const float vr = dqo_bf16_to_f32(norms_bf16[a[r] * stride]);
                b[k++] = sorts_before(vr, vl) ? a[r++] : a[l++];
            }
            while (l < mid) b[k++] = a[l++];
            while (r < hi) b[k++] = a[r++];
        }
        int64_t *t = a; a = b; b = t;
    }
    if (a != order) {
        memcpy(order, a, sizeof(int64_t) * (size_t)count);
        free(a);
    } else {
        free(b);
    }
}

/* ------------------------------------------------------------------------ */
/* quantization_compression                                                  */
/* ------------------------------------------------------------------------ */

/* csrc/cuda_hadamard.cu:607-627: t = clamp(v / div_factor, +-tensor_max); v = floor(t) + (u < t - floor(t)).
 * The reference draws u from curand states that it never initialises (:669-686), so its stream is
 * undefined ("parity unpinned"); the library defines u for element e as the top 24 bits of word e % 4 of
 * the Philox4x32-10 block with key = seed and counter = (e / 4, 0), times 2^-24. */
void dqo_quantization(float *vec, int64_t n, float div_factor, float tensor_max, uint64_t seed)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    for (int64_t g = 0; g * 4 < n; g++) {
        const uint32_t ctr[4] = {(uint32_t)g, (uint32_t)((uint64_t)g >> 32), 0u, 0u};
        uint32_t w[4];
        dqo_philox4x32_10(ctr, key, w);
        for (int k = 0; k < 4 && g * 4 + k < n; k++) {
            float t = vec[g * 4 + k] / div_factor;
            t = t < tensor_max ? t : tensor_max;
            t = t > -tensor_max ? t : -tensor_max;
            const float fl = floorf(t);
            const float prob = t - fl;
            const float u = (float)(w[k] >> 8) * 5.9604644775390625e-08f;
            vec[g * 4 + k] = fl + (u < prob ? 1.0f : 0.0f);
        }
    }
}
