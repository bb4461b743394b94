// All bit-width groups of a bucket in one launch.
//
// The reference's dynamic-bitrate all-reduce splits a bucket's superchunks into the groups that got 8, 4
// and 2 bits, gathers each group into a tensor of its own and runs the ring three times
// (testbed_evaluation/new_comm_hooks/comm_hooks.py:963-1018).  Here one launch serves the three groups:
// the partition (`order`, group sizes `counts`, written by the plan kernels of dq_grouping.hip) stays in
// device memory, every workgroup works out from the three counts which group and which tile of it it
// owns, and runs the tile body of that width.  The host never learns the group sizes, so the whole
// bucket pipeline is a fixed sequence of launches without a read-back (and can be replayed as a graph).
//
// Ring chunk c of `world` (the reference's split of a group into world pieces of whole superchunks,
// ceil(n_g / world) each) is served as one stream of records:
//     [8-bit records of chunk c | 4-bit records of chunk c | 2-bit records of chunk c]
// The record formats are those of the single-width kernels, so each of the three runs is byte for byte
// what dq_scaling_compress_rows writes for the same superchunks and random values.
//
// Rounding randomness: row k of rand_pool (256 values) belongs to the k-th superchunk of the concatenation
// 8-bit group | 4-bit group | 2-bit group; the in-kernel stream is keyed by the chunk's index in the source
// vector.
#include "dq_hier16_tiles.cuh"
#include "dq_launch.h"

namespace dq {

namespace {

// the decoder's waves take one tile of a run, or four in a row when the ring chunk is long
constexpr int kSpanLong = 4;
constexpr int64_t kLongChunk = 262144; // superchunks per ring chunk

struct MixedPlan {
    const int32_t *order;  // superchunk indices: the 8-bit group from entry 0, the 4-bit group from nsc, the 2-bit group from 2 nsc
    const int32_t *counts; // n8, n4, n2
    int chunk, world;
    int nsc;               // the counts are clamped so that their sum cannot exceed it
    uint64_t inv40;        // ceil(2^40 / world) when world <= 2^16 and nsc + world < 2^24 (see divide_by_world), else 0
    const uint64_t *step_dev; // null, or a value in device memory that the encoder adds to the step of its random stream
};

// world > 1.  With inv40 set, x / world for 0 <= x < 2^24 is (x * inv40) >> 40: inv40 = (2^40 + e) / world with
// 0 <= e < world <= 2^16, so the product exceeds x / world * 2^40 by x e < 2^40, less than the 2^40 / world that
// separate x / world from the next integer; and it stays below 2^64.  One scalar multiply instead of the expansion
// of an integer division, which stands in front of the kernel's first load.
__device__ __forceinline__ int divide_by_world(int x, const MixedPlan &p, bool magic)
{
    return magic ? (int)(((uint64_t)(uint32_t)x * p.inv40) >> 40) : x / p.world;
}

static MixedPlan make_plan(const int32_t *order, const int32_t *counts, int ring_chunk, int ring_world, int64_t nsc)
{
    MixedPlan p{order, counts, ring_chunk, ring_world, (int)nsc, 0, nullptr};
    if (ring_world > 1 && ring_world <= 65536 && nsc + ring_world < (1 << 24))
        p.inv40 = ((uint64_t)1 << 40) / (uint64_t)ring_world + (((uint64_t)1 << 40) % (uint64_t)ring_world ? 1 : 0);
    return p;
}

struct Segment {
    int cls;          // 0: 8-bit, 1: 4-bit, 2: 2-bit, 3: nothing to do
    int tile;         // first tile inside the run
    int cnt;          // records in the run
    int64_t row0;     // entry of `order` holding the run's first superchunk
    int64_t pos0;     // rank of that superchunk in the concatenation 8 | 4 | 2 (row of the random pool)
    int64_t byte_off; // where the run starts in the packed stream
};

// block -> the run (bit-width group of the ring chunk) it works in and its first tile there; a block takes `span` tiles.
// MODE 0: a ring of one rank (the whole bucket is the chunk: nothing to divide); 1: division by the world size as a
// multiplication (divide_by_world); 2: as a division.
template <int MODE> __device__ __forceinline__ Segment locate_in(const MixedPlan &p, int block, int span)
{
    constexpr bool SINGLE = MODE == 0;
    constexpr int kRec[3] = {Rec<8>::REC, Rec<4>::REC, Rec<2>::REC};
    Segment s;
    s.cls = 3; s.tile = 0; s.cnt = 0; s.row0 = 0; s.pos0 = 0; s.byte_off = 0;
    int64_t pos = 0, off = 0;
    int t = block;
    // the three loads leave together, ahead of the arithmetic (taken one by one inside the loop, each waited for its own)
    const int counts[3] = {p.counts[0], p.counts[1], p.counts[2]};
#pragma unroll
    for (int g = 0; g < 3; g++) {
        const int n = min(max(counts[g], 0), p.nsc - (int)pos); // a corrupt count cannot lead outside a region or the pool
        const int per = SINGLE ? n : divide_by_world(n + p.world - 1, p, MODE == 1);
        const int begin = SINGLE ? 0 : (int)min((int64_t)per * p.chunk, (int64_t)n);
        const int cnt = min(per, n - begin);
        const int tiles = ((cnt + kRowsPerWave - 1) / kRowsPerWave + span - 1) / span; // blocks of this run
        if (s.cls == 3 && t < tiles) {
            s.cls = g; s.tile = t * span; s.cnt = cnt; s.row0 = (int64_t)g * p.nsc + begin; s.pos0 = pos + begin; s.byte_off = off;
        }
        t -= tiles;
        pos += n;
        off += (int64_t)cnt * kRec[g];
    }
    return s;
}

__device__ __forceinline__ Segment locate(const MixedPlan &p, int block, int span)
{
    if (p.world == 1) return locate_in<0>(p, block, span);
    if (p.inv40 != 0) return locate_in<1>(p, block, span);
    return locate_in<2>(p, block, span);
}

template <int DT, int RDT, bool MEE, bool FUSED>
__global__ __launch_bounds__(64) void mixed_compress_kernel(const void *__restrict__ src, const uint8_t *__restrict__ recv,
                                                           uint8_t *__restrict__ dst, const void *__restrict__ rnd,
                                                           MixedPlan plan, int vec, RandKey key, Center ctr,
                                                           MeeArg<8, MEE> m8, MeeArg<4, MEE> m4, MeeArg<2, MEE> m2)
{
    __shared__ __attribute__((aligned(16))) uint8_t win_out[Rec<8>::WIN];
    __shared__ __attribute__((aligned(16))) uint8_t win_in[FUSED ? Rec<8>::WIN : 16];
    __shared__ float table[(MEE && FUSED) ? 256 : 1];
    constexpr int RESZ = RDT == DQ_F32 ? 4 : 2;

    // the step's addend leaves with the three counts and is used behind them: added here, its round trip would stand in
    // front of theirs
    const uint64_t step_add = (RDT == DQ_PHILOX && plan.step_dev) ? *plan.step_dev : 0;
    const Segment s = locate(plan, blockIdx.x, 1);
    if (s.cls == 3) return;
    key.step += step_add;
    const RowIds rows = row_ids_plain(plan.order + s.row0);
    const void *r = RDT == DQ_PHILOX ? nullptr : static_cast<const char *>(rnd) + s.pos0 * 256 * RESZ;
    const uint8_t *in = FUSED ? recv + s.byte_off : nullptr;
    uint8_t *out = dst + s.byte_off;
    const int lane = threadIdx.x;
    switch (s.cls) {
    case 0:
        compress_tile<DT, RDT, 8, MEE, FUSED>(src, in, out, r, rows, s.cnt, s.tile, vec, key, ctr, m8, win_out, win_in, table, lane);
        break;
    case 1:
        compress_tile<DT, RDT, 4, MEE, FUSED>(src, in, out, r, rows, s.cnt, s.tile, vec, key, ctr, m4, win_out, win_in, table, lane);
        break;
    default:
        compress_tile<DT, RDT, 2, MEE, FUSED>(src, in, out, r, rows, s.cnt, s.tile, vec, key, ctr, m2, win_out, win_in, table, lane);
        break;
    }
}

// LONG: a wave takes kSpanLong consecutive tiles of its run and fetches their row-list entries with one load (RowIds);
// a variant of its own because the loop costs registers (about 50 instead of 20).  The encoder stays with one tile per
// wave: its time on long buckets goes into arithmetic (the centring above all), not into the wait for the row list, and
// looped it holds every literal of its tile body in a register of its own (over 100 registers).
template <int DT, bool MEE, bool LONG>
__global__ __launch_bounds__(64) void mixed_decompress_kernel(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                             MixedPlan plan, const uint16_t *__restrict__ stats,
                                                             int64_t limit, int vec, MeeArg<8, MEE> m8, MeeArg<4, MEE> m4,
                                                             MeeArg<2, MEE> m2)
{
    constexpr int span = LONG ? kSpanLong : 1;
    __shared__ __attribute__((aligned(16))) uint8_t win_in[Rec<8>::WIN];
    __shared__ __attribute__((aligned(16))) uint4 tile_out[64 * Raw16<DT>::kSlots];
    __shared__ float table[MEE ? 256 : 1];

    const Segment s = locate(plan, blockIdx.x, span);
    if (s.cls == 3) return;
    const RowIds rows = LONG ? row_ids_prefetch(plan.order + s.row0, (int64_t)s.tile * kRowsPerWave, span * kRowsPerWave, s.cnt, threadIdx.x)
                             : row_ids_plain(plan.order + s.row0);
    const uint8_t *in = src + s.byte_off;
#define DQ_MIXED_TILES(NBITS, ARG)                                                                                         \
    _Pragma("unroll 1") for (int t = 0; t < span; t++)                                                                     \
    {                                                                                                                      \
        decompress_tile<DT, NBITS, MEE, false>(in, dst, rows, stats, limit, s.cnt, s.tile + t, vec, ARG, win_in, tile_out, \
                                               table);                                                                     \
        wave_lds_sync(); /* window, table and output tile are reused by the next tile */                                   \
    }
    switch (s.cls) {
    case 0: DQ_MIXED_TILES(8, m8) break;
    case 1: DQ_MIXED_TILES(4, m4) break;
    default: DQ_MIXED_TILES(2, m2) break;
    }
#undef DQ_MIXED_TILES
}

inline int span_for(int64_t nsc, int world) { return nsc / world >= kLongChunk ? kSpanLong : 1; }

// every group rounds its share of a ring chunk up to whole superchunks, its superchunks up to whole tiles and its tiles
// up to whole blocks of `span`: at most nsc / world + 3 records and nsc / (4 span world) + 3 blocks
inline unsigned grid_for(int64_t nsc, int world, int span)
{
    return (unsigned)(nsc / ((int64_t)kRowsPerWave * span * world) + 4);
}

template <int DT, int RDT, bool MEE>
hipError_t run_compress(const void *src, const uint8_t *recv, uint8_t *dst, const void *rnd, const MixedPlan &plan,
                        int64_t nsc, const Center &ctr, const RandKey &key, const MeeParams *mp, hipStream_t stream)
{
    const auto m8 = make_arg<8, MEE>(mp[0]);
    const auto m4 = make_arg<4, MEE>(mp[1]);
    const auto m2 = make_arg<2, MEE>(mp[2]);
    dim3 grid(grid_for(nsc, plan.world, 1)), block(64);
    const int vec = (aligned16(src) ? 1 : 0) | (aligned16(rnd) ? 2 : 0);
    if (recv)
        hipLaunchKernelGGL((mixed_compress_kernel<DT, RDT, MEE, true>), grid, block, 0, stream, src, recv, dst, rnd, plan, vec,
                           key, ctr, m8, m4, m2);
    else
        hipLaunchKernelGGL((mixed_compress_kernel<DT, RDT, MEE, false>), grid, block, 0, stream, src, recv, dst, rnd, plan, vec,
                           key, ctr, m8, m4, m2);
    return hipGetLastError();
}

template <int DT, bool MEE>
hipError_t run_decompress(const uint8_t *src, void *dst, const MixedPlan &plan, int64_t nsc, const uint16_t *stats,
                          int64_t limit, const MeeParams *mp, hipStream_t stream)
{
    const auto m8 = make_arg<8, MEE>(mp[0]);
    const auto m4 = make_arg<4, MEE>(mp[1]);
    const auto m2 = make_arg<2, MEE>(mp[2]);
    const int span = span_for(nsc, plan.world);
    if (span > 1)
        hipLaunchKernelGGL((mixed_decompress_kernel<DT, MEE, true>), dim3(grid_for(nsc, plan.world, span)), dim3(64), 0, stream, src,
                           dst, plan, stats, limit, aligned16(dst) ? 1 : 0, m8, m4, m2);
    else
        hipLaunchKernelGGL((mixed_decompress_kernel<DT, MEE, false>), dim3(grid_for(nsc, plan.world, 1)), dim3(64), 0, stream, src,
                           dst, plan, stats, limit, aligned16(dst) ? 1 : 0, m8, m4, m2);
    return hipGetLastError();
}

} // namespace

int64_t mixed_stream_bytes(int64_t nsc, int world) { return (nsc / world + 3) * Rec<8>::REC; }

// mp: the MEE parameters of 8, 4 and 2 bits, in this order
hipError_t launch_mixed_compress(const void *src, const float *center_mean, int center_world, int64_t n_valid,
                                 const int32_t *order, const int32_t *counts, int ring_chunk, int ring_world,
                                 const uint8_t *recv, uint8_t *dst, const void *rnd, const RandKey *philox, int64_t nsc,
                                 int dtype, bool mee, const MeeParams *mp, hipStream_t stream, const uint64_t *step_dev)
{
    MixedPlan plan = make_plan(order, counts, ring_chunk, ring_world, nsc);
    plan.step_dev = philox ? step_dev : nullptr;
    Center ctr;
    ctr.mean = center_mean;
    ctr.n_valid = n_valid;
    ctr.wd = make_world_div(center_world, (dtype & 0xf) == DQ_F32 ? 4 : 2);
    const RandKey key = philox ? *philox : RandKey{0, 0};
    const bool rb16 = (dtype & DQ_RAND_BF16) != 0;
    dtype &= 0xf;
#define DQ_MIXED(DT, RDT)                                                                                              \
    return mee ? run_compress<DT, RDT, true>(src, recv, dst, rnd, plan, nsc, ctr, key, mp, stream)                     \
               : run_compress<DT, RDT, false>(src, recv, dst, rnd, plan, nsc, ctr, key, mp, stream)
    if (dtype == DQ_BF16) {
        if (philox) { DQ_MIXED(DQ_BF16, DQ_PHILOX); }
        DQ_MIXED(DQ_BF16, DQ_BF16);
    }
    if (philox) { DQ_MIXED(DQ_F32, DQ_PHILOX); }
    if (rb16) { DQ_MIXED(DQ_F32, DQ_BF16); }
    DQ_MIXED(DQ_F32, DQ_F32);
#undef DQ_MIXED
}

hipError_t launch_mixed_decompress(const uint8_t *src, void *dst, const int32_t *order, const int32_t *counts,
                                   int ring_chunk, int ring_world, const void *stats, int64_t limit, int64_t nsc,
                                   int dtype, bool mee, const MeeParams *mp, hipStream_t stream)
{
    const MixedPlan plan = make_plan(order, counts, ring_chunk, ring_world, nsc);
    const uint16_t *st = static_cast<const uint16_t *>(stats);
    if ((dtype & 0xf) == DQ_BF16)
        return mee ? run_decompress<DQ_BF16, true>(src, dst, plan, nsc, st, limit, mp, stream)
                   : run_decompress<DQ_BF16, false>(src, dst, plan, nsc, st, limit, mp, stream);
    return mee ? run_decompress<DQ_F32, true>(src, dst, plan, nsc, st, limit, mp, stream)
               : run_decompress<DQ_F32, false>(src, dst, plan, nsc, st, limit, mp, stream);
}

} // namespace dq
