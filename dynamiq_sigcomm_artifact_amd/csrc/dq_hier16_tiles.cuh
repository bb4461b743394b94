// Tile bodies of the hierarchical chunk-16 kernels: the work of one wave on one tile of four
// superchunks, shared by the single-width kernels (dq_scaling_hier16.hip) and the kernels that
// serve all bit-width groups of a bucket in one launch (dq_scaling_mixed.hip).
//
// Numerics: csrc/cuda_hierarchical_mee.cu:203-343 (compress), 345-505 (decompress) and 526-696
// (fused decompress-accumulate-recompress).
#pragma once

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
    const float g = row16_max_pos(s); // s >= 1e-7, finite
    unit_bits = f32_to_bf16_bits(div_by(g, 1.0 / 255.0));
    const float unit = bf16_bits_to_f32(unit_bits);
    const float ratio = div_by(s, recip_f64(g)) * 255.0f;
    int qi = (int)__builtin_ceilf(ratio);
    qi = min(max(qi, 1), 255);
    q = (uint32_t)qi;
    const float d = (float)qi * unit; // exact: 8 x 8 significant bits
#pragma unroll
    for (int k = 0; k < Rec<NBITS>::WORDS; k++) w[k] = 0;
    estimate_codes<NBITS, MEE>(v, r, d, mp, w);
}

constexpr uint32_t kFastMaxBits = 0x71800000u; // 2^100


// Mean-centring applied to the source elements as they are loaded (csrc/cuda_hadamard.cu:1304-1349):
// element e of superchunk b becomes T(f32(src[e]) / world - mean[b]) with mean in binary32, zero at and
// beyond n_valid.  mean == nullptr switches it off.
struct Center {
    const float *mean;
    int64_t n_valid;
    WorldDiv wd;
};

// v holds the chunk's 16 elements as loaded when `whole` (the chunk lies inside [0, n_valid)), else they are read here
template <int DT>
__device__ __forceinline__ void center_chunk(Raw16<DT> &v, const void *src, int64_t e0, const Center &ctr, float mean, bool whole)
{
    float t[16];
    if (whole) {
        // one branch for the wave on the kind of world size, not one select per element between the two quotients
        if (DT != DQ_F32 && ctr.wd.fuse16) {
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = __builtin_fmaf(v.get(i), ctr.wd.inv, -mean); // exact: see WorldDiv
        } else if (ctr.wd.pow2) {
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = v.get(i) * ctr.wd.inv - mean;
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] = v.get(i);
            ctr.wd.divide16(t);
#pragma unroll
            for (int i = 0; i < 16; i++) t[i] -= mean;
        }
    } else {
        // the ragged end of the vector: nothing at or beyond n_valid is read
#pragma unroll
        for (int i = 0; i < 16; i++) t[i] = e0 + i < ctr.n_valid ? ctr.wd(ElemIO<DT>::load(src, e0 + i)) - mean : 0.0f;
    }
    v.set(t);
}

// Quantise the wave's chunks (lane = chunk, 16 values in v, 16 uniform values in r; lanes of rows at or beyond
// rows_here hold zeros) and stream the run of rows_here records to gout.  win_out: Rec<NBITS>::WIN bytes of LDS,
// 16-byte aligned, owned by this wave.
// WROWS < 4: the window holds WROWS records and the run leaves in 4 / WROWS pieces (win_out: window_bytes<NBITS>(WROWS)),
// for kernels that cannot spare the LDS of a four-record window.
template <int NBITS> __host__ __device__ constexpr int window_bytes(int rows)
{
    return ((rows * Rec<NBITS>::REC + 15 + 15) / 16) * 16;
}

template <int NBITS, bool MEE, int WROWS = kRowsPerWave, bool STREAM = true, class RV, class RR>
__device__ __forceinline__ void encode_store_run(const RV &v, const RR &r, const MeeArg<NBITS, MEE> &mp, uint8_t *gout,
                                                 int rows_here, uint8_t *win_out, int lane)
{
    typedef Rec<NBITS> RC;
    static_assert(WROWS == 1 || WROWS == 2 || WROWS == 4, "the window holds 1, 2 or 4 records");
    const int row = lane >> 4, j = lane & 15;

    uint32_t w[RC::WORDS], q, ub;
    const uint32_t amax = v.absmax_bits();
    const bool lane_fast = amax <= kFastMaxBits && r.unit_interval();
    if (__builtin_amdgcn_ballot_w64(!lane_fast) == 0)
        chunk_encode_fast<NBITS, MEE>(v, r, amax, mp, w, q, ub);
    else
        chunk_encode_guarded<NBITS, MEE>(v, r, mp, w, q, ub);

#pragma unroll
    for (int p = 0; p < kRowsPerWave; p += WROWS) {
        if (p >= rows_here) break;
        uint8_t *g = gout + p * RC::REC;
        const int rows_now = min(WROWS, rows_here - p);
        const int mis = (int)(reinterpret_cast<uintptr_t>(g) & 15);
        if (row >= p && row < p + rows_now) {
            uint8_t *rec = win_out + mis + (row - p) * RC::REC;
            chunk_write<NBITS>(rec + j * RC::CB, w, q);
            if (j == 0) {
                rec[16 * RC::CB] = (uint8_t)ub;
                rec[16 * RC::CB + 1] = (uint8_t)(ub >> 8);
            }
        }
        wave_lds_sync();
        window_flush<STREAM>(win_out, g, mis, rows_now * RC::REC, lane);
        if (WROWS < kRowsPerWave) wave_lds_sync(); // the window is written again
    }
}

// The row list of the tiles a wave works through.  A wave that takes several tiles fetches their entries with one load
// (lane l holds entry first + l) and hands them out by a lane shuffle: the dependent load in front of a tile's element
// loads is then paid once per wave instead of once per tile, which is what keeps the row-list kernels from the rate of
// the plain ones on long buckets.  With a single tile per wave the entries are loaded where they are used, as before.
struct RowIds {
    const int32_t *rows; // null: the identity
    int64_t first;       // entry held by lane 0
    int32_t held;
    bool prefetched;
};

__device__ __forceinline__ RowIds row_ids_plain(const int32_t *rows)
{
    RowIds ids;
    ids.rows = rows; ids.first = 0; ids.held = 0; ids.prefetched = false;
    return ids;
}

// entries [first, first + count) of rows (count <= 64, clipped to the list's length nsc)
__device__ __forceinline__ RowIds row_ids_prefetch(const int32_t *rows, int64_t first, int count, int64_t nsc, int lane)
{
    RowIds ids = row_ids_plain(rows);
    if (rows && count > kRowsPerWave) {
        ids.first = first;
        ids.held = (lane < count && first + lane < nsc) ? rows[first + lane] : 0;
        ids.prefetched = true;
    }
    return ids;
}

// entry k of the list (k the entry itself when there is no list).  Called by every lane of the wave with k inside
// the list: a prefetched entry comes out of another lane's register.
__device__ __forceinline__ int64_t row_id(const RowIds &ids, int64_t k)
{
    if (!ids.rows) return k;
    if (ids.prefetched) return (int64_t)__shfl(ids.held, (int)(k - ids.first), 64);
    return (int64_t)ids.rows[k];
}

// compress (FUSED = false) or decode-accumulate-recompress (FUSED = true) of tile `tile` of a run of nsc
// records.  Record k of the packed streams (and row k of rnd) belongs to superchunk rows[k] of src
// (to superchunk k when rows is null).  win_out / win_in: Rec<NBITS>::WIN bytes of LDS each, 16-byte
// aligned (win_in only when FUSED); table: 2^NBITS floats of LDS (only when MEE && FUSED).
template <int DT, int RDT, int NBITS, bool MEE, bool FUSED>
__device__ __forceinline__ void compress_tile(const void *__restrict__ src, const uint8_t *__restrict__ recv,
                                              uint8_t *__restrict__ dst, const void *__restrict__ rnd,
                                              const RowIds &rows, int64_t nsc, int64_t tile, int vec,
                                              const RandKey &key, const Center &ctr, const MeeArg<NBITS, MEE> &mp,
                                              uint8_t *win_out, uint8_t *win_in, float *table, int lane)
{
    typedef Rec<NBITS> RC;
    const int row = lane >> 4, j = lane & 15;
    const int64_t sc0 = tile * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows_here = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const bool active = row < rows_here;
    const int total = rows_here * RC::REC;

    // all global loads of the tile are issued before anything waits on them: the received records and the level
    // table first (they do not depend on the row list), then the row index, the random values, the mean and the chunk
    WinRegs wr;
    if (FUSED) wr = window_fetch(recv + sc0 * RC::REC, total, lane);
    TableRegs<NBITS> tr;
    if (MEE && FUSED) tr = table_fetch<NBITS>(mp, lane);
    Raw16<DT> v;
    Raw16<RDT> r;
    v.zero();
    r.zero();
    const int64_t sc_src = row_id(rows, sc0 + min(row, rows_here - 1)); // every lane asks, for an entry of the list
    int64_t e0 = 0;
    float mean = 0.0f;
    bool whole = true;
    if (active) {
        if constexpr (RDT != DQ_PHILOX) r.load(rnd, (sc0 * 16 + lane) * 16, vec & 2);
        e0 = (sc_src * 16 + j) * 16;
        if (ctr.mean) {
            mean = ctr.mean[sc_src];
            whole = e0 + 16 <= ctr.n_valid;
        }
        if (whole) v.load(src, e0, vec & 1);
    }
    if (active) {
        if constexpr (RDT == DQ_PHILOX) {
            r.generate(key, sc_src * 16 + j); // keyed by the chunk's place in the source vector
            if (ctr.mean) r.pin();            // (the centring below is the first to wait for the loads)
        }
        if (ctr.mean) center_chunk<DT>(v, src, e0, ctr, mean, whole);
    }

    if (FUSED) {
        const int mis_in = window_commit(win_in, wr, recv + sc0 * RC::REC, total, lane);
        if (MEE) table_commit<NBITS>(table, tr, lane);
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

    encode_store_run<NBITS, MEE>(v, r, mp, dst + sc0 * RC::REC, rows_here, win_out, lane & 63);
}

// Tile `tile` of a run of nsc records: record k decodes into superchunk rows[k] of dst (superchunk k when
// rows is null).  With stats (interleaved bf16 pairs, the mean first) the stored value is
// T(float(T(decoded)) + mean of the destination superchunk); elements at or beyond `limit` are not
// written.  win_in: Rec<NBITS>::WIN bytes of LDS, 16-byte aligned; tile_out: 64 * Raw16<DT>::kSlots
// 16-byte slots of LDS; table: 2^NBITS floats of LDS (only when MEE).
template <int DT, int NBITS, bool MEE, bool ADD>
__device__ __forceinline__ void decompress_tile(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                const RowIds &rows, const uint16_t *__restrict__ stats,
                                                int64_t limit, int64_t nsc, int64_t tile, int vec,
                                                const MeeArg<NBITS, MEE> &mp, uint8_t *win_in, uint4 *tile_out, float *table)
{
    typedef Rec<NBITS> RC;
    constexpr int S = Raw16<DT>::kSlots;
    constexpr int ESZ = DT == DQ_F32 ? 4 : 2;
    constexpr int EP = 16 / ESZ; // elements per 16-byte slot

    const int lane = threadIdx.x;
    const int row = lane >> 4, j = lane & 15;
    const int64_t sc0 = tile * kRowsPerWave;
    if (sc0 >= nsc) return;
    const int rows_here = (int)min((int64_t)kRowsPerWave, nsc - sc0);
    const bool active = row < rows_here;
    const int total = rows_here * RC::REC;

    const WinRegs wr = window_fetch(src + sc0 * RC::REC, total, lane);
    // destination superchunk of this lane's chunk, and of the slots this lane stores after the transpose
    const int64_t d_own = row_id(rows, sc0 + min(row, rows_here - 1)); // every lane asks, for an entry of the list
    int64_t d_slot[S];
#pragma unroll
    for (int k = 0; k < S; k++) d_slot[k] = row_id(rows, sc0 + min((64 * k + lane) / (16 * S), rows_here - 1));
    Raw16<DT> acc;
    if (ADD && active) acc.load(dst, d_own * 256 + j * 16, vec);
    uint32_t mean_bits = 0; // widened where it is used, so that nothing waits for this load here
    if (stats && active) mean_bits = stats[2 * d_own];
    TableRegs<NBITS> tr;
    if (MEE) tr = table_fetch<NBITS>(mp, lane);

    const int mis_in = window_commit(win_in, wr, src + sc0 * RC::REC, total, lane);
    if (MEE) table_commit<NBITS>(table, tr, lane);
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
            const float mean = bf16_bits_to_f32(mean_bits);
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
                    // (the accumulating variant writes the lines it has just read: no streaming hint there)
                    if (ADD)
                        *reinterpret_cast<uint4 *>(dbytes + e * ESZ) = val;
                    else
                        stream_store(reinterpret_cast<uint4 *>(dbytes + e * ESZ), val);
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

} // namespace dq

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
