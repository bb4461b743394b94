// The consumers of the rotated vector: EDEN's Lloyd-Max quantiser with its bit-plane packer
// (cuda_kernels/src/srrcomp/srrcomp.py:293-361) and THC's uniform stochastic quantiser
// (testbed_evaluation/new_comm_hooks/thc_hooks.py:149-181), which the reference runs as chains of
// torch element-wise ops and reductions around eden_utils.Hadamard.
//
// EDEN quantise, four launches (three for vectors of up to 2^22 elements, where every workgroup of `bins` folds the
// partial sums of `sumsq` itself instead of waiting for a launch of one workgroup to do it), no host synchronisation:
//   sumsq   tile b = elements [4096 b, 4096 b + 4096): thread t adds v^2 of elements t + 256 k (k ascending)
//           in double, the 256 sums are halved (stride 128 .. 1) -> work[b]
//   norm    one workgroup folds work[] the same way -> sumsq (double); norm = sqrtf((float)sumsq)
//   bins    x = (v * (float)sqrt(n)) / norm; bin = number of boundaries b with !(b >= x) (torch.bucketize, right=False: NaN -> last bin);
//           bit plane p of 32 consecutive bins -> packed[p * n/32 + w]; the products centroid[bin] * v are
//           summed in double, thread t adding elements 16 t + k of the tile (k ascending), then halved -> work[b]
//   scale   dot = fold(work[]); scale = (norm * norm) / (float)dot
// The sums are in double with a fixed association, so the result does not depend on the launch geometry
// and the CPU restatement reproduces it bit for bit.
#include <mutex>

#include "dq_launch.h"
#include "dq_tile16.cuh"

namespace dq {

namespace {

constexpr int kEdenThreads = 256;
constexpr int kEdenPerThread = 16;
constexpr int kEdenTile = kEdenThreads * kEdenPerThread; // 4096 elements

// sum[l] += sum[l + stride], stride 128 .. 1; returns the total in every thread
__device__ __forceinline__ double fold256(double v, double *lds)
{
    const int t = threadIdx.x;
    lds[t] = v;
    __syncthreads();
#pragma unroll
    for (int stride = 128; stride > 0; stride >>= 1) {
        if (t < stride) lds[t] += lds[t + stride];
        __syncthreads();
    }
    const double total = lds[0];
    __syncthreads();
    return total;
}

__global__ __launch_bounds__(kEdenThreads) void eden_sumsq_kernel(const float *__restrict__ vec, int64_t n,
                                                                 double *__restrict__ work)
{
    __shared__ double lds[kEdenThreads];
    const int64_t base = (int64_t)blockIdx.x * kEdenTile;
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < kEdenPerThread; k++) {
        const int64_t i = base + threadIdx.x + (int64_t)kEdenThreads * k;
        if (i < n) {
            const double v = (double)vec[i];
            acc += v * v;
        }
    }
    const double total = fold256(acc, lds);
    if (threadIdx.x == 0) work[blockIdx.x] = total;
}

// folds work[0 .. count): thread t adds entries t + 256 k (k ascending), then the halving tree
__device__ __forceinline__ double fold_array(const double *work, int64_t count, double *lds)
{
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += kEdenThreads) acc += work[i];
    return fold256(acc, lds);
}

// result[0] = (float)sumsq, result[3] = norm
__global__ __launch_bounds__(kEdenThreads) void eden_norm_kernel(const double *__restrict__ work, int64_t count,
                                                                float *__restrict__ result)
{
    __shared__ double lds[kEdenThreads];
    const double sumsq = fold_array(work, count, lds);
    if (threadIdx.x == 0) {
        const float s = (float)sumsq;
        result[0] = s;
        result[3] = __builtin_sqrtf(s);
    }
}

// Every thread owns sixteen consecutive elements (four 16-byte loads), so that it builds its half word of every
// bit plane in registers.  The boundaries sit in LDS in breadth-first order of the search tree (node 1 = the
// middle boundary, children of node i at 2 i and 2 i + 1): the lanes of a wave read one level of the tree at a
// time, consecutive words, where the sorted layout puts a whole level into a few banks.
// FOLD: the norm is not in result[3] yet; the workgroup folds the `tiles` partial sums in `sums` the way eden_norm_kernel
// does (the same association: the same bits), and workgroup 0 leaves result[0] and result[3] as that kernel would.  `work`
// (the products) is then a region of its own: other workgroups are still reading `sums`.
template <int NBITS, bool FOLD>
__global__ __launch_bounds__(kEdenThreads) void eden_bins_kernel(const float *__restrict__ vec, int64_t n,
                                                                const float *__restrict__ boundaries,
                                                                const float *__restrict__ centroids,
                                                                float *__restrict__ result, float sqrt_n,
                                                                uint32_t *__restrict__ packed, double *__restrict__ work,
                                                                const double *__restrict__ sums, int64_t tiles)
{
    constexpr int L = 1 << NBITS;
    __shared__ double lds[kEdenThreads];
    __shared__ float tree[L], cen[L];
    for (int k = threadIdx.x; k < L; k += kEdenThreads) {
        cen[k] = centroids[k];
        if (k < L - 1) {
            // sorted position k = (2 r + 1) 2^(NBITS - 1 - level) - 1 is node 2^level + r
            const int tz = __builtin_ctz(k + 1);
            tree[(1 << (NBITS - 1 - tz)) + ((k + 1) >> (tz + 1))] = boundaries[k];
        }
    }
    __syncthreads();
    float norm;
    if constexpr (FOLD) {
        const float s = (float)fold_array(sums, tiles, lds);
        norm = __builtin_sqrtf(s);
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            result[0] = s;
            result[3] = norm;
        }
    } else {
        norm = result[3];
    }
    const uint32_t nb = __float_as_uint(norm);
    const bool ordinary = nb >= 0x0d800000u && nb <= 0x71800000u; // uniform over the grid
    const double yn = ordinary ? recip_f64(norm) : 0.0;
    const int64_t words = n >> 5;
    const int64_t first = (int64_t)blockIdx.x * kEdenTile + (int64_t)threadIdx.x * kEdenPerThread;
    // n is a multiple of 32: the sixteen elements are all inside the vector or all outside
    const bool in = first < n;
    float v[kEdenPerThread], x[kEdenPerThread];
    int node[kEdenPerThread];
    if (in) {
        if ((reinterpret_cast<uintptr_t>(vec) & 15) == 0) { // uniform over the grid
#pragma unroll
            for (int q = 0; q < kEdenPerThread / 4; q++) {
                const float4 f = *reinterpret_cast<const float4 *>(vec + first + 4 * q);
                v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < kEdenPerThread; k++) v[k] = vec[first + k];
        }
    } else {
#pragma unroll
        for (int k = 0; k < kEdenPerThread; k++) v[k] = 0.0f;
    }
    if (ordinary) {
#pragma unroll
        for (int k = 0; k < kEdenPerThread; k++) x[k] = div_exact(v[k] * sqrt_n, norm, yn);
    } else {
#pragma unroll
        for (int k = 0; k < kEdenPerThread; k++) x[k] = (v[k] * sqrt_n) / norm;
    }
    // the sixteen searches advance level by level: sixteen independent LDS reads per level; node[] holds the
    // node's byte offset into the table
#pragma unroll
    for (int k = 0; k < kEdenPerThread; k++) node[k] = 4;
#pragma unroll
    for (int level = 0; level < NBITS; level++) {
#pragma unroll
        for (int k = 0; k < kEdenPerThread; k++) {
            const float b = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(tree) + node[k]);
            node[k] = 2 * node[k] + (!(b >= x[k]) ? 4 : 0); // torch's lower bound: a NaN goes right at every level
        }
    }
    // the product of two floats is exact in double, so the fused multiply-add rounds like multiply, then add;
    // threads past the end hold zeros and drop their sum below
    double acc = 0.0;
    uint32_t four[kEdenPerThread / 4];
#pragma unroll
    for (int q = 0; q < kEdenPerThread / 4; q++) four[q] = 0;
#pragma unroll
    for (int k = 0; k < kEdenPerThread; k++) {
        const uint32_t off = (uint32_t)(node[k] - 4 * L); // 4 * bin
        const float c = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(cen) + off);
        acc = __builtin_fma((double)c, (double)v[k], acc);
        four[k >> 2] |= (k & 3) ? off << (8 * (k & 3) - 2) : off >> 2;
    }
    if (!in) acc = 0.0;
    if (in) {
        const uint64_t lo8 = transpose8x8((uint64_t)four[0] | ((uint64_t)four[1] << 32));
        const uint64_t hi8 = transpose8x8((uint64_t)four[2] | ((uint64_t)four[3] << 32));
        // plane p, word (first >> 5), half (first >> 4) & 1
        uint16_t *half = reinterpret_cast<uint16_t *>(packed) + (first >> 4);
#pragma unroll
        for (int p = 0; p < NBITS; p++)
            half[(int64_t)p * words * 2] = (uint16_t)(((lo8 >> (8 * p)) & 0xffu) | (((hi8 >> (8 * p)) & 0xffu) << 8));
    }
    const double total = fold256(acc, lds);
    if (threadIdx.x == 0) work[blockIdx.x] = total;
}

// result[1] = (float)dot, result[2] = scale
__global__ __launch_bounds__(kEdenThreads) void eden_scale_kernel(const double *__restrict__ work, int64_t count,
                                                                 float *__restrict__ result)
{
    __shared__ double lds[kEdenThreads];
    const double dot = fold_array(work, count, lds);
    if (threadIdx.x == 0) {
        const float d = (float)dot;
        const float norm = result[3];
        result[1] = d;
        result[2] = (norm * norm) / d;
    }
}

// sixteen consecutive elements per thread: its half word of every bit plane, transposed back into sixteen bins;
// the centroids leave through a per-wave LDS tile so that the lanes store contiguous 16-byte pieces
template <int NBITS>
__global__ __launch_bounds__(256) void eden_dequantize_kernel(const uint32_t *__restrict__ packed, int64_t n,
                                                              const float *__restrict__ centroids, float *__restrict__ out)
{
    constexpr int L = 1 << NBITS;
    __shared__ float cen[L];
    __shared__ __attribute__((aligned(16))) uint4 tiles[4][256];
    for (int k = threadIdx.x; k < L; k += 256) cen[k] = centroids[k];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t first = g * 16, wave_first = (g - lane) * 16;
    if (wave_first >= n) return; // the whole wave
    const int64_t words = n >> 5;
    uint64_t lo = 0, hi = 0;
    if (first < n) { // n is a multiple of 32
        const uint16_t *half = reinterpret_cast<const uint16_t *>(packed) + g;
#pragma unroll
        for (int p = 0; p < NBITS; p++) {
            const uint32_t h = half[(int64_t)p * words * 2];
            lo |= (uint64_t)(h & 0xffu) << (8 * p);
            hi |= (uint64_t)(h >> 8) << (8 * p);
        }
    }
    lo = transpose8x8(lo);
    hi = transpose8x8(hi);
    uint32_t w[16];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        w[k] = __float_as_uint(cen[(lo >> (8 * k)) & 0xffu]);
        w[8 + k] = __float_as_uint(cen[(hi >> (8 * k)) & 0xffu]);
    }
    store_wave_words16(tiles[wave], w, reinterpret_cast<uint4 *>(out + wave_first), lane,
                       (int)min((int64_t)256, (n - wave_first) >> 2));
}

// ---- THC ------------------------------------------------------------------------------------------

// levels stored as bf16; VEC: four elements per thread through 16-byte loads and one 8-byte store
template <bool VEC>
__global__ __launch_bounds__(256) void thc_quantize_kernel(const float *__restrict__ rotated, const float *__restrict__ uniform,
                                                           uint16_t *__restrict__ out, int64_t begin, int64_t n,
                                                           const float *__restrict__ lo_p, const float *__restrict__ delta_p,
                                                           float top)
{
    const float lo = *lo_p, delta = *delta_p;
    if (VEC) {
        const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
        if (i + 4 > n) return;
        const float4 v = *reinterpret_cast<const float4 *>(rotated + i);
        const float4 u = *reinterpret_cast<const float4 *>(uniform + i);
        uint2 o;
        o.x = f32x2_to_bf16x2(thc_level(v.x, u.x, lo, delta, top), thc_level(v.y, u.y, lo, delta, top));
        o.y = f32x2_to_bf16x2(thc_level(v.z, u.z, lo, delta, top), thc_level(v.w, u.w, lo, delta, top));
        *reinterpret_cast<uint2 *>(out + i) = o;
    } else {
        const int64_t i = begin + (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (i >= n) return;
        out[i] = (uint16_t)f32_to_bf16_bits(thc_level(rotated[i], uniform[i], lo, delta, top));
    }
}

// v = float(level sum) * step + lo, two roundings
template <bool VEC>
__global__ __launch_bounds__(256) void thc_dequantize_kernel(const uint16_t *__restrict__ levels, float *__restrict__ out,
                                                             int64_t begin, int64_t n, const float *__restrict__ step_p,
                                                             const float *__restrict__ lo_p)
{
    const float step = *step_p, lo = *lo_p;
    if (VEC) {
        const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
        if (i + 4 > n) return;
        const uint2 l = *reinterpret_cast<const uint2 *>(levels + i);
        float4 o;
        float p0 = bf16_bits_to_f32(l.x & 0xffffu) * step, p1 = bf16_bits_to_f32(l.x >> 16) * step;
        float p2 = bf16_bits_to_f32(l.y & 0xffffu) * step, p3 = bf16_bits_to_f32(l.y >> 16) * step;
        o.x = p0 + lo; o.y = p1 + lo; o.z = p2 + lo; o.w = p3 + lo;
        stream_store(reinterpret_cast<float4 *>(out + i), o);
    } else {
        const int64_t i = begin + (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (i >= n) return;
        const float prod = bf16_bits_to_f32(levels[i]) * step;
        out[i] = prod + lo;
    }
}

inline int64_t eden_tiles(int64_t n) { return (n + kEdenTile - 1) / kEdenTile; }

} // namespace

// vectors of up to kEdenFoldTiles tiles take three launches and keep the two kinds of partial sums apart
constexpr int64_t kEdenFoldTiles = 1024;

int64_t eden_work_doubles(int64_t n)
{
    const int64_t tiles = eden_tiles(n);
    return tiles <= kEdenFoldTiles ? 2 * tiles : tiles;
}

hipError_t launch_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids, int nbits,
                                uint32_t *packed, float *result, double *work, hipStream_t stream)
{
    const int64_t tiles = eden_tiles(n);
    const float sqrt_n = (float)sqrt((double)n);
    dim3 grid((unsigned)tiles), block(kEdenThreads);
    const bool fold = tiles <= kEdenFoldTiles;
    double *products = fold ? work + tiles : work;
    hipLaunchKernelGGL(eden_sumsq_kernel, grid, block, 0, stream, vec, n, work);
    if (!fold) hipLaunchKernelGGL(eden_norm_kernel, dim3(1), block, 0, stream, work, tiles, result);
#define DQ_EDEN_BINS(B)                                                                                                   \
    do {                                                                                                                  \
        if (fold)                                                                                                         \
            hipLaunchKernelGGL((eden_bins_kernel<B, true>), grid, block, 0, stream, vec, n, boundaries, centroids, result, \
                               sqrt_n, packed, products, work, tiles);                                                    \
        else                                                                                                              \
            hipLaunchKernelGGL((eden_bins_kernel<B, false>), grid, block, 0, stream, vec, n, boundaries, centroids, result, \
                               sqrt_n, packed, products, work, tiles);                                                    \
    } while (0)
    switch (nbits) {
    case 1: DQ_EDEN_BINS(1); break;
    case 2: DQ_EDEN_BINS(2); break;
    case 3: DQ_EDEN_BINS(3); break;
    case 4: DQ_EDEN_BINS(4); break;
    case 5: DQ_EDEN_BINS(5); break;
    case 6: DQ_EDEN_BINS(6); break;
    case 7: DQ_EDEN_BINS(7); break;
    default: DQ_EDEN_BINS(8); break;
    }
#undef DQ_EDEN_BINS
    hipLaunchKernelGGL(eden_scale_kernel, dim3(1), block, 0, stream, products, tiles, result);
    return hipGetLastError();
}

} // namespace dq

// ---- EDEN quantise without any allocation ------------------------------------------------------
// The per-tile partial sums of launch_eden_quantize live in this array instead of a caller's buffer.
// Every device the library runs on holds its own copy for the life of the process (512 KiB).  The
// array's name is only a host-side handle: its device address comes from hipGetSymbolAddress, once
// per device, and that pointer is what the kernels receive.
static constexpr int64_t kEdenStaticMaxTiles = 65536; // 2^28 elements of 4096-element tiles
static __device__ __align__(256) double eden_static_scratch[kEdenStaticMaxTiles];

namespace dq {

int64_t eden_static_max_n() { return kEdenStaticMaxTiles * (int64_t)kEdenTile; }

namespace {
constexpr int kMaxDevices = 64;
std::mutex static_lock;
double *static_scratch_of[kMaxDevices]; // device address of eden_static_scratch, per device
} // namespace

// Resolves the address of the static array on `device` (which the caller has made current), once per device.  Called
// by the library's first call on a device, so that the entry point below has nothing left to look up when it runs
// (e.g. under stream capture).
hipError_t eden_static_prepare(int device)
{
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> g(static_lock);
    if (!static_scratch_of[device]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(eden_static_scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        static_scratch_of[device] = static_cast<double *>(p);
    }
    return hipSuccess;
}

hipError_t launch_eden_quantize_static(const float *vec, int64_t n, const float *boundaries, const float *centroids,
                                       int nbits, uint32_t *packed, float *result, int device, hipStream_t stream)
{
    if (eden_tiles(n) > kEdenStaticMaxTiles) return hipErrorInvalidValue;
    const hipError_t e = eden_static_prepare(device);
    if (e != hipSuccess) return e;
    double *scratch;
    {
        std::lock_guard<std::mutex> g(static_lock);
        scratch = static_scratch_of[device];
    }
    // every word of scratch that a kernel reads has been written by an earlier kernel of this same
    // call (sumsq -> norm or bins, bins -> scale), so nothing has to be cleared between calls; the array
    // holds the two regions of a short vector (2 * 1024 doubles) as it holds the one of a long vector
    return launch_eden_quantize(vec, n, boundaries, centroids, nbits, packed, result, scratch, stream);
}

hipError_t launch_eden_dequantize(const uint32_t *packed, int64_t n, const float *centroids, int nbits, float *out,
                                  hipStream_t stream)
{
    // n is a multiple of 32 and out 16-byte aligned: a thread's sixteen elements are half a word of every plane
    dim3 grid((unsigned)((n / 16 + 255) / 256)), block(256);
    switch (nbits) {
#define DQ_EDEN_CASE(B)                                                                                      \
    case B: hipLaunchKernelGGL(eden_dequantize_kernel<B>, grid, block, 0, stream, packed, n, centroids, out); break;
        DQ_EDEN_CASE(1) DQ_EDEN_CASE(2) DQ_EDEN_CASE(3) DQ_EDEN_CASE(4) DQ_EDEN_CASE(5) DQ_EDEN_CASE(6) DQ_EDEN_CASE(7)
    default: hipLaunchKernelGGL(eden_dequantize_kernel<8>, grid, block, 0, stream, packed, n, centroids, out); break;
#undef DQ_EDEN_CASE
    }
    return hipGetLastError();
}

hipError_t launch_thc_quantize(const float *rotated, const float *uniform, void *out, int64_t n, const float *lo,
                               const float *delta, int levels, hipStream_t stream)
{
    uint16_t *o = static_cast<uint16_t *>(out);
    const float top = (float)(levels - 1);
    const bool aligned = ((reinterpret_cast<uintptr_t>(rotated) | reinterpret_cast<uintptr_t>(uniform)) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 7) == 0;
    int64_t done = 0;
    if (aligned && n >= 4) {
        done = n / 4 * 4;
        hipLaunchKernelGGL(thc_quantize_kernel<true>, dim3((unsigned)((done / 4 + 255) / 256)), dim3(256), 0, stream, rotated,
                           uniform, o, (int64_t)0, done, lo, delta, top);
    }
    if (done < n)
        hipLaunchKernelGGL(thc_quantize_kernel<false>, dim3((unsigned)((n - done + 255) / 256)), dim3(256), 0, stream, rotated,
                           uniform, o, done, n, lo, delta, top);
    return hipGetLastError();
}

hipError_t launch_thc_dequantize(const void *levels, float *out, int64_t n, const float *step, const float *lo,
                                 hipStream_t stream)
{
    const uint16_t *l = static_cast<const uint16_t *>(levels);
    const bool aligned = (reinterpret_cast<uintptr_t>(levels) & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    int64_t done = 0;
    if (aligned && n >= 4) {
        done = n / 4 * 4;
        hipLaunchKernelGGL(thc_dequantize_kernel<true>, dim3((unsigned)((done / 4 + 255) / 256)), dim3(256), 0, stream, l, out,
                           (int64_t)0, done, step, lo);
    }
    if (done < n)
        hipLaunchKernelGGL(thc_dequantize_kernel<false>, dim3((unsigned)((n - done + 255) / 256)), dim3(256), 0, stream, l, out,
                           done, n, step, lo);
    return hipGetLastError();
}

} // namespace dq
