// Butterfly stages of the Walsh-Hadamard transform on a tile held in LDS, shared by the transform kernels
// (dq_hadamard.hip) and the kernels that quantise the rotated tile before it leaves the workgroup
// (dq_rht_scaling.hip).  Stages run in ascending stride with butterflies (a+b, a-b), the order of
// csrc/cuda_hadamard.cu:66-157,205-274, four index bits at a time on registers.  The LDS index is padded
// by one float per 16 (i + i/16): every access pattern used here is then free of bank conflicts, and a
// lane that owns 16 consecutive floats (one chunk of the quantiser) sits 17 words from its neighbour.
#pragma once

#include "dq_device.cuh"

namespace dq {

__device__ __forceinline__ int pad_idx(int i) { return i + (i >> 4); }

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

// stages for index bits [P, P+M) of the tile.  With P a compile-time constant the 2^M floats of a tuple sit at
// fixed distances from the first one -- pad_idx(base + j 2^P) = pad_idx(base) + j (2^P + 2^(P-4)) for P >= 4, and
// pad_idx(base) + j inside one group of 16 for P = 0 -- so every access is one address register plus an
// immediate offset.
template <int P, int M> __device__ __forceinline__ void lds_pass(float *lds, int ntuples, int tid, int nthreads)
{
    static_assert(P == 0 || P >= 4, "a tuple must not straddle padding groups irregularly");
    constexpr int step = P == 0 ? 1 : (1 << P) + (1 << (P - 4));
    for (int u = tid; u < ntuples; u += nthreads) {
        const int lo = u & ((1 << P) - 1);
        const int base = ((u >> P) << (P + M)) | lo;
        float *q = lds + pad_idx(base);
        float v[1 << M];
#pragma unroll
        for (int j = 0; j < (1 << M); j++) v[j] = q[j * step];
        butterflies<M>(v);
#pragma unroll
        for (int j = 0; j < (1 << M); j++) q[j * step] = v[j];
    }
}

template <int P> __device__ __forceinline__ void lds_pass_m(float *lds, int m, int tile, int tid, int nthreads)
{
    const int ntuples = tile >> m;
    switch (m) {
    case 4: lds_pass<P, 4>(lds, ntuples, tid, nthreads); break;
    case 3: lds_pass<P, 3>(lds, ntuples, tid, nthreads); break;
    case 2: lds_pass<P, 2>(lds, ntuples, tid, nthreads); break;
    default: lds_pass<P, 1>(lds, ntuples, tid, nthreads); break;
    }
}

// stages for the tile-index bits [b0, b1) of a tile of 2^kt floats, four at a time; b0 is 0 or >= 4;
// ends with a barrier
__device__ __forceinline__ void fwht_lds_stages(float *lds, int kt, int b0, int b1, int tid, int nthreads)
{
    const int tile = 1 << kt;
    for (int p = b0; p < b1; p += 4) {
        const int m = min(4, b1 - p);
        switch (p) {
        case 0: lds_pass_m<0>(lds, m, tile, tid, nthreads); break;
        case 4: lds_pass_m<4>(lds, m, tile, tid, nthreads); break;
        case 5: lds_pass_m<5>(lds, m, tile, tid, nthreads); break;
        case 8: lds_pass_m<8>(lds, m, tile, tid, nthreads); break;
        case 9: lds_pass_m<9>(lds, m, tile, tid, nthreads); break;
        case 12: lds_pass_m<12>(lds, m, tile, tid, nthreads); break;
        default: lds_pass_m<13>(lds, m, tile, tid, nthreads); break; // p == 13
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
    const int tile = 1 << kt;
    __syncthreads();
#define DQ_PASS(P, M)                                     \
    lds_pass<P, M>(lds, tile >> M, tid, nthreads);        \
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
