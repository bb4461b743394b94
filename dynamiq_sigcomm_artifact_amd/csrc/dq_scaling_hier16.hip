// Vectorised hierarchical scaling-quantisation kernels for the production
// shape: chunk 16, superchunk 16 chunks (256 elements), bf16 or fp32 elements,
// strategies 2 (AEE) and 3 (MEE), code widths 2..8.
//
// Work decomposition (wave64):
//   * one lane owns one chunk: 16 consecutive elements = 32 B (bf16) / 64 B
//     (fp32) of 128-bit loads, so the chunk maximum needs no cross-lane
//     traffic and every per-chunk scalar is computed once per 16 elements;
//   * one 16-lane DPP row owns one superchunk: the superchunk maximum is four
//     v_max_f32_dpp steps, no LDS, no barrier;
//   * one wave owns 4 consecutive superchunks = one contiguous run of 4
//     records (328..1096 bytes) in the packed stream.  Records are 82/146/274
//     bytes and never 16-byte aligned, so the run is assembled in a per-wave
//     LDS window whose offset equals the global address modulo 16 and then
//     streamed out with aligned 128-bit stores (ragged head / tail bytes are
//     stored singly).  The receive side of the fused kernel and the decoder
//     pull their run of records through the same kind of window with aligned
//     128-bit loads.
//   Waves never synchronise with each other.
//
// Numerics: csrc/cuda_hierarchical_mee.cu:203-343 (compress), 345-505
// (decompress) and 526-696 (fused decompress-accumulate-recompress).
#include "dq_device.cuh"
#include "dq_launch.h"

namespace dq {

constexpr int kWavesPerBlock = 4;
constexpr int kRowsPerWave = 4; // superchunks per wave

template <int NBITS> struct Rec {
    static constexpr int R = (1 << (NBITS - 1)) - 1;
    static constexpr int PB = 2 * NBITS;          // code bytes per chunk
    static constexpr int CB = PB + 1;             // + one scale byte
    static constexpr int REC = 16 * CB + 2;       // + bf16 unit
    static constexpr int WORDS = (PB + 3) / 4;    // dwords holding one chunk's codes
    // per-wave LDS window: 4 records + up to 15 bytes of misalignment, padded
    static constexpr int WIN = ((kRowsPerWave * REC + 15 + 15) / 16) * 16;
};

template <int NBITS, bool MEE> struct MeeArg {
    float c, cmm, l2b;
    uint16_t table[MEE ? (1 << NBITS) : 2];
};

// ---- element vectors -----------------------------------------------------------

template <int DT> struct Vec16;

template <> struct Vec16<DQ_BF16> {
    static __device__ __forceinline__ void load(const void *p, int64_t e, float (&v)[16], bool vec)
    {
        const uint16_t *h = static_cast<const uint16_t *>(p) + e;
        uint32_t w[8];
        if (vec) {
            const uint4 *q = reinterpret_cast<const uint4 *>(h);
            uint4 a = q[0], b = q[1];
            w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) w[k] = (uint32_t)h[2 * k] | ((uint32_t)h[2 * k + 1] << 16);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[2 * k] = __uint_as_float(w[k] << 16);
            v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(void *p, int64_t e, const float (&v)[16], bool vec)
    {
        uint32_t w[8];
#pragma unroll
        for (int k = 0; k < 8; k++) w[k] = f32x2_to_bf16x2(v[2 * k], v[2 * k + 1]);
        uint16_t *h = static_cast<uint16_t *>(p) + e;
        if (vec) {
            uint4 *q = reinterpret_cast<uint4 *>(h);
            q[0] = make_uint4(w[0], w[1], w[2], w[3]);
            q[1] = make_uint4(w[4], w[5], w[6], w[7]);
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) { h[2 * k] = (uint16_t)w[k]; h[2 * k + 1] = (uint16_t)(w[k] >> 16); }
        }
    }
    static __device__ __forceinline__ float round(float x) { return rb(x); }
};

template <> struct Vec16<DQ_F32> {
    static __device__ __forceinline__ void load(const void *p, int64_t e, float (&v)[16], bool vec)
    {
        const float *f = static_cast<const float *>(p) + e;
        if (vec) {
            const float4 *q = reinterpret_cast<const float4 *>(f);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float4 t = q[k];
                v[4 * k] = t.x; v[4 * k + 1] = t.y; v[4 * k + 2] = t.z; v[4 * k + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) v[k] = f[k];
        }
    }
    static __device__ __forceinline__ void store(void *p, int64_t e, const float (&v)[16], bool vec)
    {
        float *f = static_cast<float *>(p) + e;
        if (vec) {
            float4 *q = reinterpret_cast<float4 *>(f);
#pragma unroll
            for (int k = 0; k < 4; k++) q[k] = make_float4(v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) f[k] = v[k];
        }
    }
    static __device__ __forceinline__ float round(float x) { return x; }
};

// ---- record windows --------------------------------------------------------------

// pull `total` bytes starting at g (any alignment) into the window so that
// byte k of the run sits at win[(g & 15) + k]
__device__ __forceinline__ int window_fill(uint8_t *win, const uint8_t *g, int total, int lane)
{
    const int mis = (int)(reinterpret_cast<uintptr_t>(g) & 15);
    const uint4 *ga = reinterpret_cast<const uint4 *>(g - mis);
    const int nvec = (mis + total + 15) >> 4;
    for (int v = lane; v < nvec; v += 64) reinterpret_cast<uint4 *>(win)[v] = ga[v];
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

__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- per-chunk code words ---------------------------------------------------------

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

// read one chunk's CB bytes (codes + scale byte) from a window
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

// ---- the math of one chunk ---------------------------------------------------------

// decode 16 levels of one chunk and accumulate: t = round(lev*sc + acc)
template <int DT, int NBITS, bool MEE, bool ADD>
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

// quantise one chunk held in v[] against the superchunk (row) it belongs to
template <int NBITS, bool MEE>
__device__ __forceinline__ void chunk_encode(const float (&v)[16], const float (&r)[16], float c, float cmm, float l2b,
                                             uint32_t (&w)[Rec<NBITS>::WORDS], uint32_t &q, uint32_t &unit_bits)
{
    constexpr int R = Rec<NBITS>::R;
    float a = __builtin_fabsf(v[0]);
#pragma unroll
    for (int i = 1; i < 16; i++) a = __builtin_fmaxf(a, __builtin_fabsf(v[i]));
    const float s = pos_scale(MEE ? a / pos_scale(cmm) + 1e-7f : a / (float)R + 1e-7f);
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
        float x = v[i] / d;
        if (MEE) x = mee_inverse_guarded(x, c, l2b);
        words_put<NBITS>(w, i, (uint32_t)clamp_code(sr_guarded(x, r[i]), R));
    }
}

// ---- kernels ------------------------------------------------------------------------

// compress (FUSED = false) or decode-accumulate-recompress (FUSED = true)
template <int DT, int RDT, int NBITS, bool MEE, bool FUSED>
__global__ __launch_bounds__(kWavesPerBlock * 64) void hier16_compress_kernel(
    const void *__restrict__ src, const uint8_t *__restrict__ recv, uint8_t *__restrict__ dst,
    const void *__restrict__ rnd, int64_t nsc, int vec, MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    __shared__ __attribute__((aligned(16))) uint8_t win_out[kWavesPerBlock][RC::WIN];
    __shared__ __attribute__((aligned(16))) uint8_t win_in[FUSED ? kWavesPerBlock : 1][FUSED ? RC::WIN : 16];
    __shared__ float table[(MEE && FUSED) ? (1 << NBITS) : 1];

    if (MEE && FUSED) {
        for (int k = threadIdx.x; k < (1 << NBITS); k += kWavesPerBlock * 64) table[k] = f16_bits_to_f32(mp.table[k]);
        __syncthreads();
    }

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t sc0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const int row = lane >> 4, j = lane & 15;
    const bool active = row < rows;
    const int64_t e = (sc0 * 16 + lane) * 16;
    const int total = rows * RC::REC;

    float v[16], r[16];
    if (active) {
        Vec16<DT>::load(src, e, v, vec & 1);
        Vec16<RDT>::load(rnd, e, r, vec & 2);
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) { v[i] = 0.0f; r[i] = 0.0f; }
    }

    if (FUSED) {
        const int mis_in = window_fill(win_in[wave], recv + sc0 * RC::REC, total, lane);
        wave_lds_sync();
        if (active) {
            const uint8_t *rec = win_in[wave] + mis_in + row * RC::REC;
            uint32_t w[RC::WORDS], q;
            chunk_read<NBITS>(rec + j * RC::CB, w, q);
            const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
            chunk_decode<DT, NBITS, MEE, true>(w, q, ub, table, v);
#pragma unroll
            for (int i = 0; i < 16; i++) v[i] = Vec16<DT>::round(v[i]);
        }
    }

    uint32_t w[RC::WORDS], q, ub;
    chunk_encode<NBITS, MEE>(v, r, mp.c, mp.cmm, mp.l2b, w, q, ub);

    uint8_t *gout = dst + sc0 * RC::REC;
    const int mis = (int)(reinterpret_cast<uintptr_t>(gout) & 15);
    if (active) {
        uint8_t *rec = win_out[wave] + mis + row * RC::REC;
        chunk_write<NBITS>(rec + j * RC::CB, w, q);
        if (j == 0) {
            rec[16 * RC::CB] = (uint8_t)ub;
            rec[16 * RC::CB + 1] = (uint8_t)(ub >> 8);
        }
    }
    wave_lds_sync();
    window_flush(win_out[wave], gout, mis, total, lane);
}

template <int DT, int NBITS, bool MEE, bool ADD>
__global__ __launch_bounds__(kWavesPerBlock * 64) void hier16_decompress_kernel(
    const uint8_t *__restrict__ src, void *__restrict__ dst, int64_t nsc, int vec, MeeArg<NBITS, MEE> mp)
{
    typedef Rec<NBITS> RC;
    __shared__ __attribute__((aligned(16))) uint8_t win_in[kWavesPerBlock][RC::WIN];
    __shared__ float table[MEE ? (1 << NBITS) : 1];

    if (MEE) {
        for (int k = threadIdx.x; k < (1 << NBITS); k += kWavesPerBlock * 64) table[k] = f16_bits_to_f32(mp.table[k]);
        __syncthreads();
    }

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t sc0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const int row = lane >> 4, j = lane & 15;
    const bool active = row < rows;
    const int64_t e = (sc0 * 16 + lane) * 16;
    const int total = rows * RC::REC;

    float t[16];
    if (ADD && active) Vec16<DT>::load(dst, e, t, vec);

    const int mis_in = window_fill(win_in[wave], src + sc0 * RC::REC, total, lane);
    wave_lds_sync();
    if (!active) return;

    const uint8_t *rec = win_in[wave] + mis_in + row * RC::REC;
    uint32_t w[RC::WORDS], q;
    chunk_read<NBITS>(rec + j * RC::CB, w, q);
    const uint32_t ub = (uint32_t)rec[16 * RC::CB] | ((uint32_t)rec[16 * RC::CB + 1] << 8);
    chunk_decode<DT, NBITS, MEE, ADD>(w, q, ub, table, t);
    Vec16<DT>::store(dst, e, t, vec);
}

// ---- launchers ------------------------------------------------------------------------

template <int NBITS, bool MEE> static MeeArg<NBITS, MEE> make_arg(const MeeParams &mp)
{
    MeeArg<NBITS, MEE> a;
    a.c = mp.c; a.cmm = mp.cmm; a.l2b = mp.l2b;
    for (int k = 0; k < (MEE ? (1 << NBITS) : 2); k++) a.table[k] = mp.table[k];
    return a;
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static inline unsigned grid_for(int64_t nsc)
{
    const int64_t per_block = (int64_t)kWavesPerBlock * kRowsPerWave;
    return (unsigned)((nsc + per_block - 1) / per_block);
}

template <int DT, int RDT, int NBITS, bool MEE>
static hipError_t run_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd, int64_t nsc,
                               bool fused, const MeeParams &mp, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    dim3 grid(grid_for(nsc)), block(kWavesPerBlock * 64);
    const int vec = (aligned16(src) ? 1 : 0) | (aligned16(rnd) ? 2 : 0);
    if (fused)
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, true>), grid, block, 0, stream, src, recv, dst, rnd, nsc, vec, arg);
    else
        hipLaunchKernelGGL((hier16_compress_kernel<DT, RDT, NBITS, MEE, false>), grid, block, 0, stream, src, recv, dst, rnd, nsc, vec, arg);
    return hipGetLastError();
}

template <int DT, int NBITS, bool MEE>
static hipError_t run_decompress(const uint8_t *src, void *dst, int64_t nsc, int add, const MeeParams &mp, hipStream_t stream)
{
    auto arg = make_arg<NBITS, MEE>(mp);
    dim3 grid(grid_for(nsc)), block(kWavesPerBlock * 64);
    const int vec = aligned16(dst) ? 1 : 0;
    if (add)
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, true>), grid, block, 0, stream, src, dst, nsc, vec, arg);
    else
        hipLaunchKernelGGL((hier16_decompress_kernel<DT, NBITS, MEE, false>), grid, block, 0, stream, src, dst, nsc, vec, arg);
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

static hipError_t dispatch_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd, int64_t nsc,
                                    bool fused, int nbits, int dtype, bool mee, const MeeParams &mp, hipStream_t stream)
{
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
    if (dtype == DQ_BF16) {
        DQ_NBITS_MEE(run_compress, DQ_BF16 DQ_COMMA DQ_BF16, src, recv, dst, rnd, nsc, fused, mp, stream)
    } else if (rb16) {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_BF16, src, recv, dst, rnd, nsc, fused, mp, stream)
    } else {
        DQ_NBITS_MEE(run_compress, DQ_F32 DQ_COMMA DQ_F32, src, recv, dst, rnd, nsc, fused, mp, stream)
    }
}

hipError_t launch_hier16_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n, int nbits, int dtype,
                                  bool mee, const MeeParams &mp, hipStream_t stream)
{
    return dispatch_compress(src, nullptr, dst, rnd, n / 256, false, nbits, dtype, mee, mp, stream);
}

hipError_t launch_hier16_dec_comp(const uint8_t *recv, const void *inp, uint8_t *send, const void *rnd, int64_t n,
                                  int nbits, int dtype, bool mee, const MeeParams &mp, hipStream_t stream)
{
    return dispatch_compress(inp, recv, send, rnd, n / 256, true, nbits, dtype, mee, mp, stream);
}

hipError_t launch_hier16_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int dtype, bool mee,
                                    const MeeParams &mp, int add, hipStream_t stream)
{
    const int64_t nsc = n / 256;
    if ((dtype & 0xf) == DQ_BF16) {
        DQ_NBITS_MEE(run_decompress, DQ_BF16, src, dst, nsc, add, mp, stream)
    } else {
        DQ_NBITS_MEE(run_decompress, DQ_F32, src, dst, nsc, add, mp, stream)
    }
}

} // namespace dq
