// Stable partition of the superchunks of a bucket by their bit width: what three
// torch.nonzero(qbits == w) calls produce in the reference
// (testbed_evaluation/new_comm_hooks/comm_hooks.py:964-966), without host synchronisation.
//
//   order[0 .. n8)                 indices i with qbits[i] == 8, ascending
//   order[nsc .. nsc + n4)         indices with qbits[i] == 4, ascending
//   order[2 nsc .. 2 nsc + n2)     indices with qbits[i] == 2, ascending
//   work[0..2] = n8, n4, n2;  work[3] = superchunks of any other width (in no group)
//   work[4..6]                     thresholds kept between launches (widths from statistics): u's bits, the two patterns in
//                                  one word, and a seal
//   work[8 ...]                    per-tile counts of the two-launch path (tile b = superchunks
//                                  [1024 b, 1024 b + 1024)), four per tile; behind them the totals of every 64 tiles
//
// Every group has a region of its own, so where an index goes depends only on the superchunks before it.
// Buckets of up to 65536 superchunks (64 tiles) take ONE launch: the workgroup of tile b counts the
// classes of all tiles before it itself (at most 63 K superchunks, eight coalesced loads in flight per
// thread: cheaper than a second launch, and nothing waits on another workgroup), scans its own tile and places it; the
// workgroup of the last tile also writes the group sizes.  What makes the recount cheap is that the width
// is a monotone step function of the bf16 norm pattern (every operation of the rule is monotone, and
// neighbouring bf16 values are 2^-8 apart, far more than the error of the log2 polynomial): two waves
// first find the two patterns at which the width becomes 4 and 8 by a 64-way search with the exact rule,
// and a superchunk is then classified by two integer compares.
// Longer vectors take two launches: count per tile, then every tile sums the counts of the tiles before it
// and places its indices.
#include "dq_bitwidth.cuh"
#include "dq_launch.h"

#include <type_traits>

namespace dq {

namespace {

constexpr int kTile = 1024; // superchunks per workgroup
constexpr int kThreads = 256;
constexpr int kPer = kTile / kThreads;
static_assert(64 * kPer < 1024, "the wave scan of the placing kernel packs three counters of ten bits");

__device__ __forceinline__ int width_class(int64_t q) { return q == 8 ? 0 : q == 4 ? 1 : q == 2 ? 2 : 3; }

// three 21-bit counters in one word
__device__ __forceinline__ uint64_t one_of(int cls) { return cls < 3 ? (uint64_t)1 << (21 * cls) : 0; }
__device__ __forceinline__ int field(uint64_t p, int cls) { return (int)((p >> (21 * cls)) & 0x1fffff); }

// where the widths come from: an int64 array, or the norm column of the interleaved bf16 stats.
//   operator()(i)           the width of superchunk i by the rule itself (two-launch path)
//   prepare / load / cls    the one-launch path: prepare() fills thr[2] (no barrier inside), load() only
//                           loads, cls() turns a loaded value into the class 0 (8 bits) .. 3 (no group)
struct WidthsFromArray {
    const int64_t *qbits;
    typedef int64_t Raw;
    __device__ __forceinline__ int64_t operator()(int64_t i) const { return qbits[i]; }
    __device__ __forceinline__ int64_t width(int64_t i) const { return qbits[i]; }
    bool word_aligned() const { return true; }
    // the recount's loads: two widths per 16 bytes (i even), counted without branches; a width whose high half is
    // set is outside what the three compares see, and whoever finds one counts the batch again with cls()
    static constexpr int kPerLoad = 2;
    bool quad_aligned() const { return (reinterpret_cast<uintptr_t>(qbits) & 15) == 0; }
    __device__ __forceinline__ uint4 load_quad(int i) const { return *reinterpret_cast<const uint4 *>(qbits + i); }
    struct Tally {
        uint32_t n8, n4, n2, high;
    };
    __device__ __forceinline__ Tally tally_begin(const int *) const { return Tally{0u, 0u, 0u, 0u}; }
    __device__ __forceinline__ void tally_one(Tally &t, uint32_t lo, uint32_t hi) const
    {
        t.n8 += lo == 8u ? 1u : 0u;
        t.n4 += lo == 4u ? 1u : 0u;
        t.n2 += lo == 2u ? 1u : 0u;
        t.high |= hi;
    }
    __device__ __forceinline__ void tally_load(Tally &t, uint4 q) const
    {
        tally_one(t, q.x, q.y);
        tally_one(t, q.z, q.w);
    }
    __device__ __forceinline__ bool tally_beyond(const Tally &t) const { return t.high != 0u; }
    __device__ __forceinline__ uint32_t tally_n8(const Tally &t) const { return t.n8; }
    __device__ __forceinline__ uint32_t tally_n4(const Tally &t) const { return t.n4; }
    __device__ __forceinline__ uint32_t tally_n2(const Tally &t, uint32_t) const { return t.n2; }
    __device__ __forceinline__ uint64_t count_slow(uint4 q, const int *thr) const
    {
        return one_of(cls((int64_t)(((uint64_t)q.y << 32) | q.x), thr)) + one_of(cls((int64_t)(((uint64_t)q.w << 32) | q.z), thr));
    }
    __device__ __forceinline__ const uint16_t *norm_stats() const { return nullptr; }
    const void *norm_stats_host() const { return nullptr; }
    __device__ __forceinline__ void resolve() {}
    __device__ __forceinline__ void prepare(int *, int, int) const {}
    __device__ __forceinline__ uint32_t u_key() const { return 0u; }
    __host__ __device__ __forceinline__ bool known(int (&t)[2]) const // nothing to search for
    {
        t[0] = t[1] = 0;
        return true;
    }
    __device__ __forceinline__ Raw load(int i) const { return qbits[i]; }
    __device__ __forceinline__ int cls(Raw q, const int *) const { return width_class(q); }
};

struct WidthsFromStats {
    const uint16_t *stats;
    float u;
    const double *u_dev;  // when set, the offset is read from device memory (the search for u leaves it there)
    int thr_host[2];      // the two thresholds of prepare(), found on the host when u is a number (else -1)
    typedef uint32_t Raw; // a (mean, norm) pair: the norm pattern is the high half
    __device__ __forceinline__ const uint16_t *norm_stats() const { return stats; }
    const void *norm_stats_host() const { return stats; }
    __device__ __forceinline__ void resolve()
    {
        if (u_dev) u = (float)*u_dev;
    }
    __device__ __forceinline__ int64_t operator()(int64_t i) const { return qbits_of_norm(stats[2 * i + 1], u); }
    // the same by two compares when the host has found the thresholds
    __device__ __forceinline__ int64_t width(int64_t i) const
    {
        const uint32_t r = stats[2 * i + 1];
        if (thr_host[0] < 0 || r > (uint32_t)kMaxPattern) return qbits_of_norm(r, u);
        return (int)r >= thr_host[1] ? 8 : ((int)r >= thr_host[0] ? 4 : 2);
    }
    __device__ __forceinline__ void prepare(int *thr, int wave, int lane) const { width_thresholds(u, thr, wave, lane); }
    __device__ __forceinline__ uint32_t u_key() const { return __float_as_uint(u); } // what the thresholds depend on
    __host__ __device__ __forceinline__ bool known(int (&t)[2]) const
    {
        t[0] = thr_host[0];
        t[1] = thr_host[1];
        return thr_host[0] >= 0;
    }
    bool word_aligned() const { return (reinterpret_cast<uintptr_t>(stats) & 3) == 0; } // load() reads pairs as one word
    bool quad_aligned() const { return (reinterpret_cast<uintptr_t>(stats) & 15) == 0; } // load_quad(): four pairs, i % 4 == 0
    __device__ __forceinline__ Raw load(int i) const { return reinterpret_cast<const uint32_t *>(stats)[i]; }
    __device__ __forceinline__ uint4 load_quad(int i) const { return *reinterpret_cast<const uint4 *>(stats + 2 * (int64_t)i); }
    __device__ __forceinline__ int cls(Raw pair, const int *thr) const
    {
        const uint32_t r = pair >> 16;
        if (r <= (uint32_t)kMaxPattern) return (int)r >= thr[1] ? 0 : ((int)r >= thr[0] ? 1 : 2);
        return width_class(qbits_of_norm(r, u)); // negative or NaN norms: the rule itself
    }
    // the recount's form of cls(): counters without a branch.  The pattern is the high half of the pair, so r >= t is
    // pair >= t << 16 for 0 <= t <= 0x8000 whatever the low half holds: `ge8` counts the pairs at or above the 8-bit
    // threshold, `ge4` those at or above the 4-bit one, `top` keeps the largest pair seen (a pattern above kMaxPattern
    // -- a negative or NaN norm -- is outside the thresholds' range, and whoever finds one counts the batch again with cls())
    struct Tally {
        uint32_t t8, t4, ge8, ge4, top;
    };
    __device__ __forceinline__ Tally tally_begin(const int *thr) const
    {
        return Tally{(uint32_t)min(max(thr[1], 0), 0x8000) << 16, (uint32_t)min(max(thr[0], 0), 0x8000) << 16, 0u, 0u, 0u};
    }
    __device__ __forceinline__ void tally(Tally &t, Raw pair) const
    {
        t.ge8 += pair >= t.t8 ? 1u : 0u;
        t.ge4 += pair >= t.t4 ? 1u : 0u;
        t.top = max(t.top, pair);
    }
    __device__ __forceinline__ bool tally_beyond(const Tally &t) const { return t.top >= ((uint32_t)kMaxPattern + 1u) << 16; }
    // superchunks of the 8-bit and of the 4-bit class among those tallied (cls() asks for the 8-bit threshold first)
    __device__ __forceinline__ uint32_t tally_n8(const Tally &t) const { return t.ge8; }
    __device__ __forceinline__ uint32_t tally_n4(const Tally &t) const { return t.t4 <= t.t8 ? t.ge4 - t.ge8 : 0u; }
    __device__ __forceinline__ uint32_t tally_n2(const Tally &t, uint32_t seen) const { return seen - tally_n8(t) - tally_n4(t); }
    static constexpr int kPerLoad = 4; // (mean, norm) pairs per 16 bytes
    __device__ __forceinline__ void tally_load(Tally &t, uint4 q) const
    {
        tally(t, q.x);
        tally(t, q.y);
        tally(t, q.z);
        tally(t, q.w);
    }
    __device__ __forceinline__ uint64_t count_slow(uint4 q, const int *thr) const
    {
        return one_of(cls(q.x, thr)) + one_of(cls(q.y, thr)) + one_of(cls(q.z, thr)) + one_of(cls(q.w, thr));
    }
};


// Inclusive scan over the wave's 64 lanes with data-parallel-primitive moves (shifts by 1, 2, 4, 8 inside the rows of
// sixteen lanes, then lane 15 of a row into the next row, lane 31 into the upper half): a dozen register-to-register
// instructions where six rounds of cross-lane permutes through the LDS pipeline took about half a microsecond.  The
// operand packs small counters into one word; no field may overflow into the next one.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ uint32_t dpp_from(uint32_t x)
{
    // lanes without a source, and rows outside ROW_MASK, receive 0
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, 0xf, false);
}

__device__ __forceinline__ uint32_t wave_scan_inclusive(uint32_t x)
{
    x += dpp_from<0x111, 0xf>(x); // row_shr:1
    x += dpp_from<0x112, 0xf>(x); // row_shr:2
    x += dpp_from<0x114, 0xf>(x); // row_shr:4
    x += dpp_from<0x118, 0xf>(x); // row_shr:8
    x += dpp_from<0x142, 0xa>(x); // row_bcast:15 into rows 1 and 3
    x += dpp_from<0x143, 0xc>(x); // row_bcast:31 into rows 2 and 3
    return x;
}

// ---- one launch (up to 64 tiles) ----------------------------------------------------------------------

constexpr int kOneThreads = kTile; // one superchunk per thread while placing
constexpr int kOneMaxTiles = 64;
constexpr int kOneBatch = 8;       // loads in flight per thread while recounting the tiles before

// HIST: the launch has a few workgroups more than tiles (one per 8192 superchunks); they add the norm patterns of the
// bucket to `hist` (what the search for the next step's u works on) while the others plan, so the histogram costs no
// launch of its own.
// QUAD: the recount of the tiles before reads 16 bytes per load, four (mean, norm) pairs or two widths (a late tile's recount is a string of dependent
// round trips to the L2, and a quarter as many requests make it a quarter as long).
// SEARCH: the thresholds are not among the arguments (u is read from device memory) and two waves search for them; a
// variant of its own, because with the choice left to run time the compiler moves the loop-invariant part of that search
// (a hundred instructions) in front of the recount of every launch.  The search is a chain of its own behind the load of u
// -- three dependent rounds of the rule, then a barrier -- and a training step plans a thousand buckets with one u: the
// workgroup of tile 0 leaves what it found in work[4..6] (the bits of u, the two patterns in one word, and a seal, the
// exclusive-or of the two with a constant), and a later launch on the same work buffer whose u has the same bits and whose
// seal holds takes the thresholds from there.  Anything else in those words -- a buffer never planned on, the two patterns
// the long-bucket kernels leave there, an entry caught half written -- fails the seal, and the launch searches.
constexpr uint32_t kThresholdSeal = 0x9e3779b9u;
template <class W, bool HIST, bool QUAD, bool SEARCH>
__global__ __launch_bounds__(kOneThreads) void plan_one_kernel(W widths, int64_t *__restrict__ qbits_out, int nsc,
                                                              int32_t *__restrict__ order, int32_t *__restrict__ work,
                                                              uint32_t *__restrict__ hist)
{
    static_assert(kOneThreads == kHistThreads, "the histogram workgroup has the shape of the others");
    __shared__ uint32_t local[HIST ? kHistWords : 1];
    __shared__ int thr[2];
    __shared__ uint64_t before_sum[kOneThreads / 64], scan_sum[kOneThreads / 64];
    if (HIST && (int)blockIdx.x >= (nsc + kTile - 1) / kTile) {
        const int64_t h = (int)blockIdx.x - (nsc + kTile - 1) / kTile; // one batch each
        count_norm_patterns(widths.norm_stats(), nsc, h * kHistBatch, (int64_t)gridDim.x * kHistBatch, hist, local);
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nbefore = (int)blockIdx.x * kTile; // superchunks of the tiles before this one
    const int own = nbefore + (int)threadIdx.x;

    // this tile's load and the first batch of the recount are in flight while u arrives and the thresholds are searched
    // (u is first looked at below, behind those loads: read at the top of the kernel, its round trip stood in front of them)
    typename W::Raw own_raw = typename W::Raw();
    if (own < nsc) own_raw = widths.load(own);
    uint64_t mine = 0;
    int t2[2]; // the thresholds: from the kernel arguments, or searched by two waves and handed over through LDS
    bool ready = widths.known(t2) || !SEARCH;
    const bool keeps = SEARCH && (reinterpret_cast<uintptr_t>(work) & 15) == 0;
    bool searched = false, settled = false;
    uint4 kept = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (SEARCH) {
        if (keeps) kept = *reinterpret_cast<const uint4 *>(work + 4);
    }
    // u, and the thresholds kept from an earlier launch with the same u
    auto settle = [&]() {
        if (settled) return;
        settled = true;
        widths.resolve();
        if constexpr (SEARCH) {
            if (keeps && kept.x == widths.u_key() && kept.z == (kept.x ^ kept.y ^ kThresholdSeal)) {
                t2[0] = (int)(kept.y & 0xffffu);
                t2[1] = (int)(kept.y >> 16);
                ready = true;
            }
        }
    };
    constexpr int kStep = QUAD ? W::kPerLoad : 1; // superchunks per load; nbefore is a whole number of tiles
    for (int i0 = 0; i0 < nbefore; i0 += kOneBatch * kOneThreads * kStep) {
        typename W::Raw raw[QUAD ? 1 : kOneBatch];
        uint4 quad[QUAD ? kOneBatch : 1];
#pragma unroll
        for (int j = 0; j < kOneBatch; j++) {
            const int i = i0 + (j * kOneThreads + (int)threadIdx.x) * kStep;
            if (i < nbefore) {
                if constexpr (QUAD)
                    quad[j] = widths.load_quad(i);
                else
                    raw[j] = widths.load(i);
            }
        }
        settle();
        if constexpr (SEARCH) {
            if (!ready) {
                widths.prepare(thr, wave, lane);
                __syncthreads();
                t2[0] = thr[0];
                t2[1] = thr[1];
                ready = true;
                searched = true;
            }
        }
        if constexpr (QUAD) {
            // a late tile's recount is a few dozen classifications per thread on a compute unit that holds sixteen such
            // waves: counted without branches, and once more the long way in the rare batch with a pattern outside the
            // thresholds' range (a negative or NaN norm)
            typename W::Tally tl = widths.tally_begin(t2);
            uint32_t seen = 0;
#pragma unroll
            for (int j = 0; j < kOneBatch; j++) {
                const int i = i0 + (j * kOneThreads + (int)threadIdx.x) * kStep;
                if (i < nbefore) {
                    widths.tally_load(tl, quad[j]);
                    seen += kStep;
                }
            }
            if (__builtin_amdgcn_ballot_w64(widths.tally_beyond(tl)) == 0) {
                const uint32_t n8 = widths.tally_n8(tl), n4 = widths.tally_n4(tl);
                mine += (uint64_t)n8 | ((uint64_t)n4 << 21) | ((uint64_t)widths.tally_n2(tl, seen) << 42);
            } else {
#pragma unroll // (a loop would index the loaded values by a variable: they would live in scratch memory)
                for (int j = 0; j < kOneBatch; j++) {
                    const int i = i0 + (j * kOneThreads + (int)threadIdx.x) * kStep;
                    if (i < nbefore) mine += widths.count_slow(quad[j], t2);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < kOneBatch; j++) {
                const int i = i0 + (j * kOneThreads + (int)threadIdx.x) * kStep;
                if (i < nbefore) mine += one_of(widths.cls(raw[j], t2));
            }
        }
    }
    settle();
    if constexpr (SEARCH) {
        if (!ready) {
            widths.prepare(thr, wave, lane);
            __syncthreads();
            t2[0] = thr[0];
            t2[1] = thr[1];
            searched = true;
        }
        if (searched && keeps && blockIdx.x == 0 && threadIdx.x == 0) {
            const uint32_t both = (uint32_t)t2[0] | ((uint32_t)t2[1] << 16); // patterns: at most 0x7f81 each
            *reinterpret_cast<uint4 *>(work + 4) = make_uint4(widths.u_key(), both, widths.u_key() ^ both ^ kThresholdSeal, 0u);
        }
    }
    // the wave's total of the recount: a thread has counted at most 64 superchunks, a wave at most 4096 per class, so
    // two classes share a word (lane 63 of the scan holds the total)
    const uint32_t mine01 = wave_scan_inclusive((uint32_t)field(mine, 0) | ((uint32_t)field(mine, 1) << 16));
    const uint32_t mine2 = wave_scan_inclusive((uint32_t)field(mine, 2));

    // this tile: class of the thread's superchunk, inclusive scan over the wave (at most 64 per class: a byte each)
    const int c = own < nsc ? widths.cls(own_raw, t2) : 3;
    if (qbits_out && own < nsc) qbits_out[own] = c == 0 ? 8 : (c == 1 ? 4 : (c == 2 ? 2 : (int64_t)widths(own)));
    const uint64_t cnt = one_of(c);
    const uint32_t scanned = wave_scan_inclusive(c < 3 ? 1u << (8 * c) : 0u);
    const uint64_t incl = (uint64_t)(scanned & 0xffu) | ((uint64_t)((scanned >> 8) & 0xffu) << 21) |
                          ((uint64_t)((scanned >> 16) & 0xffu) << 42);
    if (lane == 63) {
        before_sum[wave] = (uint64_t)(mine01 & 0xffffu) | ((uint64_t)(mine01 >> 16) << 21) | ((uint64_t)mine2 << 42);
        scan_sum[wave] = incl;
    }
    __syncthreads();
    uint64_t before = 0, excl = incl - cnt, tile_all = 0;
#pragma unroll
    for (int k = 0; k < kOneThreads / 64; k++) {
        before += before_sum[k];
        if (k < wave) excl += scan_sum[k];
        tile_all += scan_sum[k];
    }
    if (c < 3) order[(int64_t)c * nsc + field(before, c) + field(excl, c)] = own;
    if ((int)blockIdx.x == (nsc + kTile - 1) / kTile - 1 && threadIdx.x == 0) { // the last tile (a histogram workgroup may follow)
        const uint64_t all = before + tile_all;
        work[0] = field(all, 0);
        work[1] = field(all, 1);
        work[2] = field(all, 2);
        work[3] = nsc - field(all, 0) - field(all, 1) - field(all, 2);
    }
}

// ---- two launches (any length) ------------------------------------------------------------------------

template <class W>
__global__ __launch_bounds__(kThreads) void plan_count_kernel(W widths, int64_t nsc, int32_t *__restrict__ work)
{
    __shared__ int cnt[4];
    widths.resolve();
    if (threadIdx.x < 4) cnt[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x * kPer;
    int c[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        if (base + k < nsc) c[width_class(widths.width(base + k))]++;
    }
#pragma unroll
    for (int w = 0; w < 4; w++) {
        if (c[w]) atomicAdd(&cnt[w], c[w]);
    }
    __syncthreads();
    if (threadIdx.x < 4) work[8 + 4 * blockIdx.x + threadIdx.x] = cnt[threadIdx.x];
}

template <class W>
__global__ __launch_bounds__(kThreads) void plan_place_kernel(W widths, int64_t *__restrict__ qbits_out, int64_t nsc,
                                                              int ntiles, int32_t *__restrict__ order,
                                                              int32_t *__restrict__ work)
{
    __shared__ int before[4], total[4];
    __shared__ uint64_t wave_sum[kThreads / 64];
    widths.resolve();
    if (threadIdx.x < 4) {
        before[threadIdx.x] = 0;
        total[threadIdx.x] = 0;
    }
    __syncthreads();
    {
        int t[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
        for (int tile = threadIdx.x; tile < ntiles; tile += kThreads) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const int c = work[8 + 4 * tile + w];
                t[w] += c;
                if (tile < (int)blockIdx.x) b[w] += c;
            }
        }
#pragma unroll
        for (int w = 0; w < 4; w++) {
            if (t[w]) atomicAdd(&total[w], t[w]);
            if (b[w]) atomicAdd(&before[w], b[w]);
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x < 4) work[threadIdx.x] = total[threadIdx.x];

    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x * kPer;
    int cls[kPer];
    uint64_t mine = 0;
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        cls[k] = 3;
        if (base + k < nsc) {
            const int64_t q = widths.width(base + k);
            if (qbits_out) qbits_out[base + k] = q;
            cls[k] = width_class(q);
        }
        mine += one_of(cls[k]);
    }
    // inclusive scan over the wave, then over the waves of the workgroup
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // (a thread holds at most kPer = 4 superchunks, a wave at most 256 per class: ten bits each)
    const uint32_t scanned = wave_scan_inclusive((uint32_t)field(mine, 0) | ((uint32_t)field(mine, 1) << 10) |
                                                 ((uint32_t)field(mine, 2) << 20));
    const uint64_t incl = (uint64_t)(scanned & 0x3ffu) | ((uint64_t)((scanned >> 10) & 0x3ffu) << 21) |
                          ((uint64_t)((scanned >> 20) & 0x3ffu) << 42);
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint64_t excl = incl - mine;
    for (int w = 0; w < wave; w++) excl += wave_sum[w];

    int64_t pos[3];
#pragma unroll
    for (int w = 0; w < 3; w++) pos[w] = (int64_t)w * nsc + before[w] + field(excl, w);
#pragma unroll
    for (int k = 0; k < kPer; k++) {
#pragma unroll
        for (int w = 0; w < 3; w++) {
            if (cls[k] == w) order[pos[w]++] = (int32_t)(base + k);
        }
    }
}

// ---- two launches, widths from statistics (long buckets) ----------------------------------------------
//
// The kernels above let every workgroup of the second launch add up the counts of all tiles (four 4-byte loads per
// tile): with T tiles that is T * T * 16 bytes of L2 reads -- 0.9 GB at the 7,630 tiles of a 2 * 10^9-element bucket,
// 100 us for a plan whose own traffic is 60 MB.  Here the first launch takes a group of tiles per workgroup and leaves,
// beside the count of every tile, the total of its group; a workgroup of the second launch then reads the totals of
// the groups before its own and the counts of the tiles before it inside its group: at most 256 + 31 entries of 16
// bytes (groups of 8 or 32 tiles, see group_tiles_for).  The first launch also leaves the two threshold patterns in work[4..6] (found on the host, or searched
// by two waves of every workgroup when u is read from device memory), so the second neither searches nor evaluates
// the rule; both classify four superchunks per 16-byte load.  Needs stats and work 16-byte aligned.

// tiles per workgroup of the first launch: 8 (one per wave) up to 1,024 tiles, 32 (two per wave) beyond -- at most 256
// groups up to 8,192 tiles, the 2^31 elements an int32 index reaches
constexpr int kFewTiles = 1024;
inline int group_tiles_for(int64_t ntiles) { return ntiles <= kFewTiles ? 8 : 32; }

// the classes of up to four superchunks of a quad, counted into n[0..2]
__device__ __forceinline__ void count_quad_slow(const WidthsFromStats &widths, uint4 q, int valid, const int *t2, uint32_t (&n)[3])
{
    const uint32_t v[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (k < valid) {
            const int c = widths.cls(v[k], t2);
#pragma unroll
            for (int w = 0; w < 3; w++) n[w] += c == w ? 1u : 0u;
        }
    }
}

// superchunks [i, i + 4) of the statistics as four pairs; those at and beyond nsc read as zero pairs
__device__ __forceinline__ uint4 load_quad_guarded(const WidthsFromStats &widths, int64_t i, int64_t nsc, int &valid)
{
    valid = (int)min((int64_t)4, max((int64_t)0, nsc - i));
    if (valid == 4) return widths.load_quad((int)i);
    uint4 q = make_uint4(0, 0, 0, 0);
    if (valid > 0) q.x = widths.load((int)i);
    if (valid > 1) q.y = widths.load((int)i + 1);
    if (valid > 2) q.z = widths.load((int)i + 2);
    return q;
}

template <bool SEARCH, int G, int THREADS>
__global__ __launch_bounds__(THREADS) void plan_count_stats_kernel(WidthsFromStats widths, int64_t nsc, int ntiles,
                                                                  int32_t *__restrict__ work)
{
    constexpr int kSuperTiles = G, kCountThreads = THREADS;
    __shared__ int thr[2];
    __shared__ uint32_t group_total[4];
    const uint4 kept = *reinterpret_cast<const uint4 *>(work + 4); // (work is 16-byte aligned on this path)
    widths.resolve();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int t2[2];
    bool ready = widths.known(t2);
    if (threadIdx.x < 4) group_total[threadIdx.x] = 0;
    if constexpr (SEARCH) {
        // the thresholds an earlier plan on this work buffer found for the same u (see plan_one_kernel), or a search
        if (kept.x == widths.u_key() && kept.z == (kept.x ^ kept.y ^ kThresholdSeal)) {
            t2[0] = (int)(kept.y & 0xffffu);
            t2[1] = (int)(kept.y >> 16);
            ready = true;
        }
        if (!ready) widths.prepare(thr, wave, lane);
    }
    __syncthreads();
    if constexpr (SEARCH) {
        if (!ready) {
            t2[0] = thr[0];
            t2[1] = thr[1];
        }
    }
    // for the second launch, and for the next plan on this buffer: u's bits, both patterns (at most 0x7f81 each), the seal
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        const uint32_t both = (uint32_t)t2[0] | ((uint32_t)t2[1] << 16);
        *reinterpret_cast<uint4 *>(work + 4) = make_uint4(widths.u_key(), both, widths.u_key() ^ both ^ kThresholdSeal, 0u);
    }
    int4 *tile_counts = reinterpret_cast<int4 *>(work + 8);
    const int tile0 = (int)blockIdx.x * kSuperTiles;
    for (int k = wave; k < kSuperTiles && tile0 + k < ntiles; k += kCountThreads / 64) { // the bounds are the wave's own
        const int tile = tile0 + k;
        const int64_t base = (int64_t)tile * kTile + lane * 4;
        uint4 q[4];
        int valid[4];
#pragma unroll
        for (int j = 0; j < 4; j++) q[j] = load_quad_guarded(widths, base + j * 256, nsc, valid[j]);
        WidthsFromStats::Tally tl = widths.tally_begin(t2);
        uint32_t seen = 0;
        bool ragged = false;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (valid[j] == 4) {
                widths.tally(tl, q[j].x);
                widths.tally(tl, q[j].y);
                widths.tally(tl, q[j].z);
                widths.tally(tl, q[j].w);
                seen += 4;
            } else if (valid[j] > 0) {
                ragged = true;
            }
        }
        uint32_t n[3];
        if (__builtin_amdgcn_ballot_w64(ragged || widths.tally_beyond(tl)) == 0) {
            n[0] = widths.tally_n8(tl);
            n[1] = widths.tally_n4(tl);
            n[2] = seen - n[0] - n[1];
        } else { // the bucket's last tile, or a negative or NaN norm somewhere in this one: class by class
            n[0] = n[1] = n[2] = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) count_quad_slow(widths, q[j], valid[j], t2, n);
        }
        // a lane has counted at most 16 superchunks, the wave 1024: two classes share a word
        const uint32_t s01 = wave_scan_inclusive(n[0] | (n[1] << 16));
        const uint32_t s2 = wave_scan_inclusive(n[2]);
        if (lane == 63) {
            const int c8 = (int)(s01 & 0xffffu), c4 = (int)(s01 >> 16), c2 = (int)s2;
            tile_counts[tile] = make_int4(c8, c4, c2, 0);
            atomicAdd(&group_total[0], (uint32_t)c8);
            atomicAdd(&group_total[1], (uint32_t)c4);
            atomicAdd(&group_total[2], (uint32_t)c2);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0)
        tile_counts[ntiles + blockIdx.x] = make_int4((int)group_total[0], (int)group_total[1], (int)group_total[2], 0);
}

__global__ __launch_bounds__(kThreads) void plan_place_stats_kernel(WidthsFromStats widths, int64_t *__restrict__ qbits_out,
                                                                   int64_t nsc, int ntiles, int kSuperTiles,
                                                                   int32_t *__restrict__ order, int32_t *__restrict__ work)
{
    __shared__ int before[4], total[4];
    __shared__ uint64_t wave_sum[kThreads / 64];
    widths.resolve(); // (cls() evaluates the rule itself for a negative or NaN norm)
    if (threadIdx.x < 4) {
        before[threadIdx.x] = 0;
        total[threadIdx.x] = 0;
    }
    __syncthreads();
    const int t2[2] = {(int)((uint32_t)work[5] & 0xffffu), (int)((uint32_t)work[5] >> 16)}; // as the first launch left them
    const int4 *tile_counts = reinterpret_cast<const int4 *>(work + 8);
    const int group = (int)blockIdx.x / kSuperTiles, inside = (int)blockIdx.x % kSuperTiles;
    const int ngroups = (ntiles + kSuperTiles - 1) / kSuperTiles;
    {
        // entries [0, group): the totals of the groups before; [group, group + inside): the tiles before inside the group
        int b[3] = {0, 0, 0};
        for (int e = threadIdx.x; e < group + inside; e += kThreads) {
            const int4 c = e < group ? tile_counts[ntiles + e] : tile_counts[group * kSuperTiles + (e - group)];
            b[0] += c.x;
            b[1] += c.y;
            b[2] += c.z;
        }
#pragma unroll
        for (int w = 0; w < 3; w++) {
            if (b[w]) atomicAdd(&before[w], b[w]);
        }
        if (blockIdx.x == 0) { // the group sizes of the whole bucket
            int t[3] = {0, 0, 0};
            for (int e = threadIdx.x; e < ngroups; e += kThreads) {
                const int4 c = tile_counts[ntiles + e];
                t[0] += c.x;
                t[1] += c.y;
                t[2] += c.z;
            }
#pragma unroll
            for (int w = 0; w < 3; w++) {
                if (t[w]) atomicAdd(&total[w], t[w]);
            }
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x < 4) work[threadIdx.x] = threadIdx.x < 3 ? total[threadIdx.x] : 0;

    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x * kPer;
    static_assert(kPer == 4, "a thread places the four superchunks of one 16-byte load");
    int valid;
    const uint4 q = load_quad_guarded(widths, base, nsc, valid);
    const uint32_t v[4] = {q.x, q.y, q.z, q.w};
    int cls[kPer];
    uint64_t mine = 0;
#pragma unroll
    for (int k = 0; k < kPer; k++) {
        cls[k] = 3;
        if (k < valid) {
            cls[k] = widths.cls(v[k], t2);
            if (qbits_out) qbits_out[base + k] = cls[k] == 0 ? 8 : (cls[k] == 1 ? 4 : 2);
        }
        mine += one_of(cls[k]);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t scanned = wave_scan_inclusive((uint32_t)field(mine, 0) | ((uint32_t)field(mine, 1) << 10) |
                                                 ((uint32_t)field(mine, 2) << 20));
    const uint64_t incl = (uint64_t)(scanned & 0x3ffu) | ((uint64_t)((scanned >> 10) & 0x3ffu) << 21) |
                          ((uint64_t)((scanned >> 20) & 0x3ffu) << 42);
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint64_t excl = incl - mine;
    for (int w = 0; w < wave; w++) excl += wave_sum[w];
    int64_t pos[3];
#pragma unroll
    for (int w = 0; w < 3; w++) pos[w] = (int64_t)w * nsc + before[w] + field(excl, w);
#pragma unroll
    for (int k = 0; k < kPer; k++) {
#pragma unroll
        for (int w = 0; w < 3; w++) {
            if (cls[k] == w) order[pos[w]++] = (int32_t)(base + k);
        }
    }
}

// ---- fixed-proportion groups: the stable descending sort of the norms in one launch -------------------
//
// testbed_evaluation/new_comm_hooks/comm_hooks.py:710-721: sorted = argsort(norms, descending, stable); the first
// `top` entries of sorted are the 8-bit group, the last `bottom` the 2-bit group, the rest the 4-bit group, each **in
// sorted order**.  The norms are bf16 values, so the sort key has 16 bits and the position of superchunk i is
//     G(key_i) + E(i),   G = superchunks with a key that sorts earlier,   E = superchunks j < i with the same key
// -- a counting sort.  As in plan_one_kernel no workgroup waits for another: the workgroup of tile b (256
// superchunks) counts the keys of the whole bucket itself, in an LDS histogram (128 KB, 144 KB with its padding),
// in two steps: first the superchunks before its tile (the counter of key_i is then the part of E(i) that lies in
// earlier tiles), then the rest; an in-place exclusive scan of the histogram gives G.  The part of E inside the tile
// comes from comparing the tile's keys with each other.  nsc <= 65535, so no counter overflows.
//
// Sort key (ascending key = descending norm, as torch.sort orders floats): NaN (either sign) first, then +inf ...
// +0 = -0 ... -inf.
constexpr int kSortThreads = 1024;
constexpr int kSortTile = 256;
constexpr int kSortWords = 32768;                          // words of the histogram
constexpr int kSortLdsWords = kSortWords + kSortWords / 8; // stored with 4 words of padding after every 32
constexpr int kSortBatch = 32;                             // loads in flight per thread: 32768 superchunks in one round trip

// Word w of the histogram lives at w + 4 (w / 32): in the scan thread t owns the 32 words [32 t, 32 t + 32), and with a
// lane stride of 36 words instead of 32 the 16-byte accesses of neighbouring lanes fall into different banks (unpadded,
// all lanes of a wave hit the same four banks).
__device__ __forceinline__ int hist_slot(uint32_t word) { return (int)(word + ((word >> 5) << 2)); }

// Two layouts.  Sums of squares are not negative, so normally every pattern is one of 0 .. 0x7f80 or a NaN: then a key
// takes 15 bits, NaN -> 0, +inf -> 1, ..., +0 -> 0x7f81, and every counter has a word of its own (narrow).  A bucket that
// holds a negative pattern (-0 included) takes the general key, 16 bits, with two 16-bit counters per word (wide); its
// counting and its scan cost about twice the narrow ones.
__device__ __forceinline__ uint32_t narrow_key(uint32_t pattern)
{
    return pattern <= (uint32_t)kMaxPattern ? (uint32_t)kMaxPattern + 1u - pattern : 0u; // NaN (sign bit clear) -> 0
}

__device__ __forceinline__ uint32_t wide_key(uint32_t pattern)
{
    const uint32_t mag = pattern & 0x7fffu;
    if (mag > (uint32_t)kMaxPattern) return 0u;             // NaN
    if (pattern & 0x8000u) return 0x7fffu + mag;            // -0 -> 0x7fff (the key of +0), -inf -> 0xff7f
    return 0x7fffu - mag;                                   // +inf -> 0x7f, +0 -> 0x7fff
}

template <bool WIDE> __device__ __forceinline__ uint32_t sort_key(uint32_t pattern) { return WIDE ? wide_key(pattern) : narrow_key(pattern); }

template <bool WIDE> __device__ __forceinline__ void count_one(uint32_t *hist, uint32_t pattern)
{
    const uint32_t k = sort_key<WIDE>(pattern);
    if (WIDE)
        atomicAdd(&hist[hist_slot(k >> 1)], 1u << (16 * (k & 1)));
    else
        atomicAdd(&hist[hist_slot(k)], 1u);
}

template <bool WIDE> __device__ __forceinline__ int counter_of(const uint32_t *hist, uint32_t k)
{
    return WIDE ? (int)((hist[hist_slot(k >> 1)] >> (16 * (k & 1))) & 0xffffu) : (int)hist[hist_slot(k)];
}

// adds the keys of the superchunks [begin, end) to the histogram; cached: the (mean, norm) pairs of the first
// kSortBatch * kSortThreads superchunks, already in registers (pair j of thread t = superchunk j * kSortThreads + t)
template <bool WIDE>
__device__ __forceinline__ void count_keys(const uint32_t *__restrict__ pairs, int begin, int end, uint32_t *hist,
                                           const uint32_t (&cached)[kSortBatch])
{
#pragma unroll
    for (int j = 0; j < kSortBatch; j++) {
        const int i = j * kSortThreads + (int)threadIdx.x;
        if (i >= begin && i < end) count_one<WIDE>(hist, cached[j] >> 16);
    }
    for (int i0 = max(begin, kSortBatch * kSortThreads) / (kSortBatch * kSortThreads) * (kSortBatch * kSortThreads); i0 < end;
         i0 += kSortBatch * kSortThreads) {
        uint32_t raw[kSortBatch];
#pragma unroll
        for (int j = 0; j < kSortBatch; j++) {
            const int i = i0 + j * kSortThreads + (int)threadIdx.x;
            if (i >= begin && i < end) raw[j] = pairs[i];
        }
#pragma unroll
        for (int j = 0; j < kSortBatch; j++) {
            const int i = i0 + j * kSortThreads + (int)threadIdx.x;
            if (i >= begin && i < end) count_one<WIDE>(hist, raw[j] >> 16);
        }
    }
}

// exclusive scan of the counters in place; thread t owns the words [32 t, 32 t + 32)
template <bool WIDE> __device__ __forceinline__ void scan_counters(uint32_t *hist, uint32_t *wave_sum)
{
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    uint4 *mine = reinterpret_cast<uint4 *>(hist + 36 * t); // hist_slot(32 t)
    uint4 v[8];
    uint32_t sum = 0;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        v[q] = mine[q];
        const uint32_t w[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
        for (int h = 0; h < 4; h++) sum += WIDE ? (w[h] & 0xffffu) + (w[h] >> 16) : w[h];
    }
    const uint32_t incl = wave_scan_inclusive(sum);
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum;
    for (int k = 0; k < wave; k++) run += wave_sum[k];
#pragma unroll
    for (int q = 0; q < 8; q++) {
        uint32_t w[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
        for (int h = 0; h < 4; h++) {
            if (WIDE) {
                const uint32_t lo = w[h] & 0xffffu, hi = w[h] >> 16;
                w[h] = (run & 0xffffu) | ((run + lo) << 16); // an exclusive prefix is at most nsc - 1 < 65536
                run += lo + hi;
            } else {
                const uint32_t c = w[h];
                w[h] = run;
                run += c;
            }
        }
        mine[q] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

template <bool WIDE>
__device__ __forceinline__ void sorted_plan_body(const uint32_t *__restrict__ pairs, int nsc, int top, int bottom,
                                                 int64_t *__restrict__ qbits_out, int32_t *__restrict__ order,
                                                 const uint32_t (&cached)[kSortBatch], uint32_t own_pattern, uint32_t *hist,
                                                 uint16_t *tile_key, int (*part_rank)[kSortTile], uint32_t *wave_sum)
{
    const int t = threadIdx.x;
    const int nbefore = (int)blockIdx.x * kSortTile;
    const int e = t & (kSortTile - 1), part = t / kSortTile; // element of the tile, quarter of its predecessors
    const int own = nbefore + e;
    const int valid = min(kSortTile, nsc - nbefore);
    const uint32_t key = e < valid ? sort_key<WIDE>(own_pattern) : 0u;
    if (part == 0) tile_key[e] = (uint16_t)key;
    __syncthreads(); // the zeroed histogram and the tile's keys are in place

    // superchunks of the tile with the same key and a smaller index: quarter `part` of the candidates (the quarters
    // behind the element's own hold none)
    {
        int r = 0;
        const int j0 = part * (kSortTile / 4);
        if (j0 <= e) {
            const uint4 *k4 = reinterpret_cast<const uint4 *>(tile_key + j0);
#pragma unroll
            for (int q = 0; q < kSortTile / 4 / 8; q++) {
                const uint4 v = k4[q]; // the same address in every lane: a broadcast
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int h = 0; h < 8; h++) {
                    const int j = j0 + 8 * q + h;
                    const uint32_t kj = (w[h >> 1] >> (16 * (h & 1))) & 0xffffu;
                    r += (kj == key && j < e) ? 1 : 0;
                }
            }
        }
        part_rank[part][e] = r;
    }
    count_keys<WIDE>(pairs, 0, nbefore, hist, cached);
    __syncthreads();
    int same_before = 0;
    if (part == 0 && e < valid) {
        same_before = counter_of<WIDE>(hist, key);
#pragma unroll
        for (int q = 0; q < kSortThreads / kSortTile; q++) same_before += part_rank[q][e];
    }
    __syncthreads();
    count_keys<WIDE>(pairs, nbefore, nsc, hist, cached);
    __syncthreads();
    scan_counters<WIDE>(hist, wave_sum);
    __syncthreads();

    if (part == 0 && e < valid) {
        const int pos = counter_of<WIDE>(hist, key) + same_before;
        const int mid_end = nsc - bottom;
        int region, at;
        if (pos < top) region = 0, at = pos;
        else if (pos < mid_end) region = 1, at = pos - top;
        else region = 2, at = pos - mid_end;
        order[(int64_t)region * nsc + at] = own;
        if (qbits_out) qbits_out[own] = region == 0 ? 8 : (region == 1 ? 4 : 2);
    }
}

__global__ __launch_bounds__(kSortThreads) void sorted_plan_kernel(const uint32_t *__restrict__ pairs, int nsc, int top,
                                                                  int bottom, int64_t *__restrict__ qbits_out,
                                                                  int32_t *__restrict__ order, int32_t *__restrict__ work)
{
    __shared__ __align__(16) uint32_t hist[kSortLdsWords];
    __shared__ __align__(16) uint16_t tile_key[kSortTile];
    __shared__ int part_rank[kSortThreads / kSortTile][kSortTile];
    __shared__ uint32_t wave_sum[kSortThreads / 64];
    __shared__ int any_negative;
    const int t = threadIdx.x;
    if (t == 0) any_negative = 0;
    // the first kSortBatch * kSortThreads pairs stay in registers for all three passes over them
    uint32_t cached[kSortBatch];
#pragma unroll
    for (int j = 0; j < kSortBatch; j++) {
        const int i = j * kSortThreads + t;
        cached[j] = i < nsc ? pairs[i] : 0u;
    }
    const int own = (int)blockIdx.x * kSortTile + (t & (kSortTile - 1));
    const uint32_t own_pattern = own < nsc ? pairs[own] >> 16 : 0u;
    {
        uint4 *h4 = reinterpret_cast<uint4 *>(hist);
        for (int w = t; w < kSortLdsWords / 4; w += kSortThreads) h4[w] = make_uint4(0u, 0u, 0u, 0u);
    }
    __syncthreads();
    // any pattern with the sign bit set that is not a NaN (a NaN is key 0 in both layouts)
    bool negative = false;
#pragma unroll
    for (int j = 0; j < kSortBatch; j++) negative |= (cached[j] >> 31) != 0 && (cached[j] & 0x7fff0000u) <= ((uint32_t)kMaxPattern << 16);
    for (int i = kSortBatch * kSortThreads + t; i < nsc; i += kSortThreads) {
        const uint32_t p = pairs[i];
        negative |= (p >> 31) != 0 && (p & 0x7fff0000u) <= ((uint32_t)kMaxPattern << 16);
    }
    if (__builtin_amdgcn_ballot_w64(negative) != 0 && (t & 63) == 0) any_negative = 1;
    __syncthreads();
    if (any_negative)
        sorted_plan_body<true>(pairs, nsc, top, bottom, qbits_out, order, cached, own_pattern, hist, tile_key, part_rank, wave_sum);
    else
        sorted_plan_body<false>(pairs, nsc, top, bottom, qbits_out, order, cached, own_pattern, hist, tile_key, part_rank, wave_sum);
    if (blockIdx.x == 0 && t == 0) {
        work[0] = top;
        work[1] = nsc - top - bottom;
        work[2] = bottom;
        work[3] = 0;
    }
}

} // namespace

hipError_t launch_group_plan_sorted(const void *stats, int64_t nsc, int64_t top, int64_t bottom, int64_t *qbits_out,
                                    int32_t *order, int32_t *work, hipStream_t stream)
{
    const int ntiles = (int)((nsc + kSortTile - 1) / kSortTile);
    hipLaunchKernelGGL(sorted_plan_kernel, dim3(ntiles), dim3(kSortThreads), 0, stream,
                       static_cast<const uint32_t *>(stats), (int)nsc, (int)top, (int)bottom, qbits_out, order, work);
    return hipGetLastError();
}

// header, four counts per tile, four per group of tiles
int64_t group_plan_work_ints(int64_t nsc)
{
    const int64_t ntiles = (nsc + kTile - 1) / kTile;
    const int64_t g = group_tiles_for(ntiles);
    return 8 + 4 * ntiles + 4 * ((ntiles + g - 1) / g);
}

// hist (only with widths from statistics): the bucket's norm patterns are added to it
template <class W>
static hipError_t run_plan(W widths, int64_t *qbits_out, int64_t nsc, int32_t *order, int32_t *work, uint32_t *hist,
                           hipStream_t stream)
{
    const int ntiles = (int)((nsc + kTile - 1) / kTile);
    if (ntiles <= kOneMaxTiles && widths.word_aligned()) {
        const dim3 grid(hist ? ntiles + (int)((nsc + kHistBatch - 1) / kHistBatch) : ntiles), block(kOneThreads);
        const bool quad = widths.quad_aligned();
        int t2[2];
        const bool search = !widths.known(t2);
#define DQ_PLAN_ONE(HIST, QUAD)                                                                                            \
    do {                                                                                                                   \
        if (search)                                                                                                        \
            hipLaunchKernelGGL((plan_one_kernel<W, HIST, QUAD, true>), grid, block, 0, stream, widths, qbits_out, (int)nsc, \
                               order, work, hist);                                                                         \
        else                                                                                                               \
            hipLaunchKernelGGL((plan_one_kernel<W, HIST, QUAD, false>), grid, block, 0, stream, widths, qbits_out,          \
                               (int)nsc, order, work, hist);                                                               \
    } while (0)
        if (hist) {
            if (quad) DQ_PLAN_ONE(true, true); else DQ_PLAN_ONE(true, false);
        } else {
            if (quad) DQ_PLAN_ONE(false, true); else DQ_PLAN_ONE(false, false);
        }
#undef DQ_PLAN_ONE
        return hipGetLastError();
    }
    if (hist) {
        const hipError_t eh = launch_norm_histogram(widths.norm_stats_host(), nsc, hist, stream);
        if (eh != hipSuccess) return eh;
    }
    if constexpr (std::is_same<W, WidthsFromStats>::value) {
        if (widths.quad_aligned() && (reinterpret_cast<uintptr_t>(work) & 15) == 0) {
            int t2[2];
            const bool search = !widths.known(t2);
            const int g = group_tiles_for(ntiles);
            const dim3 groups((unsigned)((ntiles + g - 1) / g));
#define DQ_PLAN_COUNT(SEARCH)                                                                                              \
    do {                                                                                                                   \
        if (g == 8)                                                                                                        \
            hipLaunchKernelGGL((plan_count_stats_kernel<SEARCH, 8, 512>), groups, dim3(512), 0, stream, widths, nsc, ntiles, \
                               work);                                                                                      \
        else                                                                                                               \
            hipLaunchKernelGGL((plan_count_stats_kernel<SEARCH, 32, 1024>), groups, dim3(1024), 0, stream, widths, nsc,     \
                               ntiles, work);                                                                              \
    } while (0)
            if (search) DQ_PLAN_COUNT(true); else DQ_PLAN_COUNT(false);
#undef DQ_PLAN_COUNT
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(plan_place_stats_kernel, dim3(ntiles), dim3(kThreads), 0, stream, widths, qbits_out, nsc, ntiles, g,
                               order, work);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL(plan_count_kernel<W>, dim3(ntiles), dim3(kThreads), 0, stream, widths, nsc, work);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(plan_place_kernel<W>, dim3(ntiles), dim3(kThreads), 0, stream, widths, qbits_out, nsc, ntiles, order, work);
    return hipGetLastError();
}

hipError_t launch_group_plan(const int64_t *qbits, int64_t nsc, int32_t *order, int32_t *work, hipStream_t stream)
{
    return run_plan(WidthsFromArray{qbits}, nullptr, nsc, order, work, nullptr, stream);
}

// ---- the thresholds of the width rule on the host ------------------------------------------------------
//
// The rule (dq_bitwidth.cuh: qbits_of_norm) is binary32 arithmetic with every result rounded to bf16 and the
// library's polynomial log2: the same operations in the same order give the same bits on the host, so when u comes
// as a number the two patterns at which the width becomes 4 and 8 are found here and travel with the kernel
// arguments, and the plan kernel neither searches nor waits for the two waves that would.

static inline uint32_t host_bits(float f) { uint32_t u; __builtin_memcpy(&u, &f, 4); return u; }
static inline float host_float(uint32_t u) { float f; __builtin_memcpy(&f, &u, 4); return f; }

static inline float host_round_bf16(float x) // round to nearest even, as v_cvt_pk_bf16_f32
{
    uint32_t b = host_bits(x);
    if ((b & 0x7fffffffu) > 0x7f800000u) return host_float((b | 0x00400000u) & 0xffff0000u); // NaN stays NaN
    b += 0x7fffu + ((b >> 16) & 1u);
    return host_float(b & 0xffff0000u);
}

static float host_log2_det(float x) // log2_det of dq_device.cuh, operation by operation
{
    uint32_t ix = host_bits(x);
    int k = 0;
    if (ix >= 0x7f800000u) {
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x7fffffffu) > 0x7f800000u) return x + x;
        if ((ix << 1) == 0) return -__builtin_inff();
        return host_float(0x7fc00000u);
    }
    if (ix < 0x00800000u) {
        if (ix == 0) return -__builtin_inff();
        x *= 8388608.0f;
        ix = host_bits(x);
        k = -23;
    }
    const uint32_t t = ix - 0x3f3504f3u;
    k += (int)t >> 23;
    const float z = host_float(ix - (t & 0xff800000u));
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

static int host_qbits_of_norm(uint32_t norm_bits, float u) // qbits_of_norm of dq_bitwidth.cuh
{
    const float eps = 1e-20f;
    float x = host_float(norm_bits << 16);
    x = (x != x) ? x : host_round_bf16(x > eps ? x : eps);
    x = host_round_bf16(host_log2_det(x));
    x = host_round_bf16(x * (float)(4.0 / (512.0 / 17.0)));
    x = host_round_bf16(x + u);
    x = (x != x) ? x : host_round_bf16(x > eps ? x : eps);
    x = host_round_bf16(host_log2_det(x));
    x = __builtin_floorf(x);
    const int z = (x != x) ? 1 : (x < 1.0f ? 1 : (x > 3.0f ? 3 : (int)x));
    return 1 << z;
}

// the smallest pattern in [0, kMaxPattern] whose width is >= target, kMaxPattern + 1 if none (the width is a
// monotone step function of the pattern: width_thresholds() on the device relies on the same)
static int host_width_threshold(float u, int target)
{
    int lo = 0, hi = kMaxPattern + 1; // the answer lies in [lo, hi]
    while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (host_qbits_of_norm((uint32_t)mid, u) >= target)
            hi = mid;
        else
            lo = mid + 1;
    }
    return lo;
}

// u_dev != nullptr: the offset is *u_dev at the time the kernels run, u is ignored
hipError_t launch_group_plan_stats(const void *stats, float u, const double *u_dev, int64_t nsc, int64_t *qbits_out,
                                   int32_t *order, int32_t *work, uint32_t *hist, hipStream_t stream)
{
    WidthsFromStats widths{static_cast<const uint16_t *>(stats), u, u_dev, {-1, -1}};
    if (!u_dev && u == u) { // (a NaN offset: every width is 2, and the device search says so itself)
        widths.thr_host[0] = host_width_threshold(u, 4);
        widths.thr_host[1] = host_width_threshold(u, 8);
    }
    return run_plan(widths, qbits_out, nsc, order, work, hist, stream);
}

} // namespace dq
