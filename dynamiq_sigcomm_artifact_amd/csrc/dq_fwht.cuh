// Butterfly stages of the Walsh-Hadamard transform on a tile held in LDS, shared by the transform kernels
// (dq_hadamard.hip) and the kernels that quantise the rotated tile before it leaves the workgroup
// (dq_rht_scaling_impl.cuh).  Stages run in ascending stride with butterflies (a+b, a-b), the order of
// csrc/cuda_hadamard.cu:66-157,205-274, four or five index bits at a time on registers.
//
// Layout.  The LDS serves 32 lanes per cycle from 32 banks of one word, so an access of a wave is free of bank
// conflicts when each half of the wave touches 32 different banks.  Element i of the tile lives at word
// i + i / 32 (one word of padding per 32):
//   * lanes on consecutive elements (every pass over index bits >= 5, the coalesced loads and stores): 32 lanes
//     starting at a multiple of 32 stay inside one group, consecutive words;
//   * a lane that owns 16 consecutive elements (one chunk of the quantiser) and reads or writes its k-th one: chunk c
//     starts at word 16 c + c / 2, so 32 consecutive chunks fall on (16 (c % 2) + c / 2 + k) mod 32, all different;
//   * the first pass in LDS (index bits from 4 on, lanes = 16 low index values x tuples): the lanes of a half wave are
//     16 consecutive words twice, and the two runs are 16 banks apart when the two tuples differ in index bit 9
//     (2^9 + 2^4 words): the tuples are numbered so that they do (tuple_base).
// A padding of one word per 16 -- the layout this replaced -- puts lane 0 and lane 31 of every run of 32 consecutive
// elements on one bank (a second cycle for every such access: 19.5 % of the LDS cycles of the fused kernels were
// conflicts) and the two runs of the first pass on the same 16 banks.
#pragma once

#include "dq_device.cuh"

namespace dq {

__device__ __forceinline__ int pad_idx(int i) { return i + (i >> 5); }

// words of LDS for a padded tile of `tile` floats, rounded up to a multiple of four (what follows stays 16-byte aligned)
__host__ __device__ constexpr int padded_floats(int tile) { return (tile + (tile >> 5) + 1 + 3) & ~3; }

// where the 16 consecutive elements of chunk c start: pad_idx(16 c + k) = 16 c + c / 2 + k for k < 16
__device__ __forceinline__ int chunk_word(int c) { return 16 * c + (c >> 1); }

template <int M> __device__ __forceinline__ void butterflies(float (&v)[1 << M])
{
#pragma unroll
    for (int h = 1; h < (1 << M); h <<= 1) {
#pragma unroll
        for (int i = 0; i < (1 << M); i++) {
            if ((i & h) == 0) {
                float a = v[i], b = v[i + h];
                v[i] = a + b;
                v[i + h] = a - b;
            }
        }
    }
}

// word offset of element j of a tuple of pass <P, M> from the tuple's first element: the index grows by j 2^P
template <int P> __device__ __forceinline__ constexpr int tuple_step(int j)
{
    if constexpr (P == 0)
        return j;
    else if constexpr (P >= 5)
        return j * ((1 << P) + (1 << (P - 5)));
    else
        return 16 * j + (j >> 1); // P == 4: bit 4 of the index is bit 0 of j
}

// Index of the first element of tuple u of a pass over index bits [P, P + M): the low P bits of u are the low P index
// bits, the rest of u fills the index bits from P + M on.  For P = 4 and M < 5 the first of those bits of u goes to
// index bit 9 instead of bit 4 + M (and the bits in between move down by one), so that lanes 0..15 and 16..31 of a wave
// sit 16 banks apart; `spare` = number of index bits above the tuple's (kt - P - M).
template <int P, int M> __device__ __forceinline__ int tuple_base(int u, int spare)
{
    const int lo = u & ((1 << P) - 1);
    int hi = u >> P;
    if constexpr (P == 4 && M < 5) {
        constexpr int t = 5 - M; // index bit 9 is bit t of the field above the tuple
        if (spare > t) hi = ((hi & 1) << t) | ((hi >> 1) & ((1 << t) - 1)) | ((hi >> (t + 1)) << (t + 1));
    }
    return (hi << (P + M)) | lo;
}

// stages for index bits [P, P+M) of a tile of 2^kt floats.  With P a compile-time constant the 2^M floats of a tuple
// sit at fixed distances from the first one (tuple_step), so every access is one address register plus an immediate
// offset.
template <int P, int M> __device__ __forceinline__ void lds_pass(float *lds, int kt, int tid, int nthreads)
{
    static_assert(P == 0 || P >= 4, "a tuple must not straddle padding groups irregularly");
    static_assert(P != 0 || M <= 5, "a tuple of consecutive elements must stay inside one padding group");
    const int ntuples = 1 << (kt - M);
    for (int u = tid; u < ntuples; u += nthreads) {
        float *q = lds + pad_idx(tuple_base<P, M>(u, kt - P - M));
        float v[1 << M];
#pragma unroll
        for (int j = 0; j < (1 << M); j++) v[j] = q[tuple_step<P>(j)];
        butterflies<M>(v);
#pragma unroll
        for (int j = 0; j < (1 << M); j++) q[tuple_step<P>(j)] = v[j];
    }
}

template <int P> __device__ __forceinline__ void lds_pass_m(float *lds, int m, int kt, int tid, int nthreads)
{
    switch (m) {
    case 4: lds_pass<P, 4>(lds, kt, tid, nthreads); break;
    case 3: lds_pass<P, 3>(lds, kt, tid, nthreads); break;
    case 2: lds_pass<P, 2>(lds, kt, tid, nthreads); break;
    default: lds_pass<P, 1>(lds, kt, tid, nthreads); break;
    }
}

// stages for the tile-index bits [b0, b1) of a tile of 2^kt floats, four at a time; b0 is 0 or >= 4;
// ends with a barrier
__device__ __forceinline__ void fwht_lds_stages(float *lds, int kt, int b0, int b1, int tid, int nthreads)
{
    for (int p = b0; p < b1; p += 4) {
        const int m = min(4, b1 - p);
        switch (p) {
        case 0: lds_pass_m<0>(lds, m, kt, tid, nthreads); break;
        case 4: lds_pass_m<4>(lds, m, kt, tid, nthreads); break;
        case 5: lds_pass_m<5>(lds, m, kt, tid, nthreads); break;
        case 8: lds_pass_m<8>(lds, m, kt, tid, nthreads); break;
        case 9: lds_pass_m<9>(lds, m, kt, tid, nthreads); break;
        case 12: lds_pass_m<12>(lds, m, kt, tid, nthreads); break;
        default: lds_pass_m<13>(lds, m, kt, tid, nthreads); break; // p == 13
        }
        __syncthreads();
    }
}

// ---- tiles whose first stages are done in registers -------------------------------------------------
//
// A lane that holds 16 consecutive elements (one chunk of the quantiser) does the stages of strides 1..8 on
// its registers before the tile ever touches LDS; the remaining kb - 4 stages then take as few LDS passes
// as possible, up to five stages (32 registers) per pass.  Regrouping stages does not change any addition:
// every stage still forms (a + b, a - b) of the same pairs, in ascending stride.

// stages [0, min(4, kb)) on the 16 consecutive elements of a lane
__device__ __forceinline__ void chunk_stages(float (&v)[16], int kb)
{
#pragma unroll
    for (int h = 1; h < 16; h <<= 1) {
        if (h < (1 << kb)) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if ((i & h) == 0) {
                    const float a = v[i], b = v[i + h];
                    v[i] = a + b;
                    v[i + h] = a - b;
                }
            }
        }
    }
}

// stages [4, kb) of a tile of 2^kt floats (padded layout) whose stages [0, 4) are done.  Starts with the barrier
// that makes the chunks written by other lanes visible; a barrier follows every pass.
__device__ __forceinline__ void fwht_lds_stages_after4(float *lds, int kt, int kb, int tid, int nthreads)
{
    __syncthreads();
#define DQ_PASS(P, M)                           \
    lds_pass<P, M>(lds, kt, tid, nthreads);     \
    __syncthreads();
    switch (kb - 4) {
    case 1: DQ_PASS(4, 1) break;
    case 2: DQ_PASS(4, 2) break;
    case 3: DQ_PASS(4, 3) break;
    case 4: DQ_PASS(4, 4) break;
    case 5: DQ_PASS(4, 5) break;
    case 6: DQ_PASS(4, 3) DQ_PASS(7, 3) break;
    case 7: DQ_PASS(4, 4) DQ_PASS(8, 3) break;
    case 8: DQ_PASS(4, 4) DQ_PASS(8, 4) break;
    case 9: DQ_PASS(4, 5) DQ_PASS(9, 4) break;
    case 10: DQ_PASS(4, 5) DQ_PASS(9, 5) break;
    case 11: DQ_PASS(4, 4) DQ_PASS(8, 4) DQ_PASS(12, 3) break;
    default: break; // kb <= 4: nothing left
    }
#undef DQ_PASS
}

} // namespace dq
