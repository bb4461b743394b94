// What does a launch of the codec's shape cost when the arithmetic is taken away?  A measurement aid, not part of the codec.
//
// The chunk-16 encoders and decoders run one wave per tile of 1,024 elements: a lane reads its chunk of 16 elements (and of
// the rounding pool) as 16-byte pieces, the wave writes its four records as one unaligned run.  A 25 MB bucket is 6,400 such
// waves, a launch a few microseconds long, and how close such a launch can come to the HBM rate is a property of the launch
// (its ramp, the unaligned record runs, the write-back at its end) as much as of the kernel's instructions.  The kernel here
// moves the same bytes with the same access pattern and does nothing else: every lane folds what it loaded into one word with
// exclusive-ors (so that no load can be dropped and every store waits for every load) and the stores carry that word.  Timed
// over the same buffers, it is the floor a codec kernel of this shape can be held against.
//
//   direction 0 (encoder shape): per tile read `a_bytes` from `a` and `b_bytes` from `b` (lane l owns bytes [l*bytes/64, +bytes/64)
//       as 16-byte pieces), write `run_bytes` to `run` (8-byte pieces, piece j by lane j % 64; the tile's run starts at
//       tile * run_bytes, 8-byte aligned, not line aligned -- as the records are);
//   direction 1 (decoder shape): per tile read `run_bytes` from `run` the same way, optionally `b_bytes` from `b`, write `a_bytes`
//       to `a` as the decoders do after their transposition through the LDS: 16-byte pieces, piece 64 k + l by lane l, with the
//       streaming hint.
#include "dq_device.cuh"
#include "dq_launch.h"

#include <hip/hip_runtime.h>

namespace dq {

namespace {

__device__ __forceinline__ uint32_t fold(uint4 v) { return v.x ^ v.y ^ v.z ^ v.w; }

template <int A16, int B16, int DIR>
__global__ __launch_bounds__(64) void tile_io_floor_kernel(uint4 *__restrict__ a, const uint4 *__restrict__ b, uint2 *__restrict__ run,
                                                           int run_pieces)
{
    const int lane = threadIdx.x;
    const int64_t tile = blockIdx.x;
    uint32_t x = (uint32_t)lane;
    uint4 vb[B16 > 0 ? B16 : 1];
    if (B16 > 0) {
        const uint4 *pb = b + (tile * 64 + lane) * B16;
#pragma unroll
        for (int k = 0; k < B16; k++) vb[k] = pb[k];
    }
    if (DIR == 0) {
        uint4 va[A16];
        const uint4 *pa = a + (tile * 64 + lane) * A16;
#pragma unroll
        for (int k = 0; k < A16; k++) va[k] = pa[k];
#pragma unroll
        for (int k = 0; k < A16; k++) x ^= fold(va[k]);
        if (B16 > 0) {
#pragma unroll
            for (int k = 0; k < B16; k++) x ^= fold(vb[k]);
        }
        uint2 *out = run + tile * run_pieces;
        for (int j = lane; j < run_pieces; j += 64) out[j] = make_uint2(x, x + (uint32_t)(j >> 6));
    } else {
        const uint2 *in = run + tile * run_pieces;
        for (int j = lane; j < run_pieces; j += 64) {
            const uint2 v = in[j];
            x ^= v.x ^ v.y;
        }
        if (B16 > 0) {
#pragma unroll
            for (int k = 0; k < B16; k++) x ^= fold(vb[k]);
        }
        uint4 *pa = a + tile * 64 * A16 + lane;
#pragma unroll
        for (int k = 0; k < A16; k++) stream_store(pa + 64 * k, make_uint4(x, x + 1u, x + 2u, x + 3u + (uint32_t)k));
    }
}

template <int A16, int B16>
void launch_dir(int direction, void *a, const void *b, void *run, int run_pieces, int64_t tiles, hipStream_t stream)
{
    const dim3 grid((unsigned)tiles), block(64);
    if (direction == 0)
        hipLaunchKernelGGL((tile_io_floor_kernel<A16, B16, 0>), grid, block, 0, stream, static_cast<uint4 *>(a),
                           static_cast<const uint4 *>(b), static_cast<uint2 *>(run), run_pieces);
    else
        hipLaunchKernelGGL((tile_io_floor_kernel<A16, B16, 1>), grid, block, 0, stream, static_cast<uint4 *>(a),
                           static_cast<const uint4 *>(b), static_cast<uint2 *>(run), run_pieces);
}

} // namespace

bool tile_io_floor_shape_ok(int a_bytes, int b_bytes, int run_bytes)
{
    return (a_bytes == 2048 || a_bytes == 4096) && (b_bytes == 0 || b_bytes == 2048 || b_bytes == 4096) && run_bytes > 0 &&
           run_bytes % 8 == 0 && run_bytes <= 8192;
}

hipError_t launch_tile_io_floor(int direction, void *a, int a_bytes, const void *b, int b_bytes, void *run, int run_bytes, int64_t tiles,
                                hipStream_t stream)
{
    const int pieces = run_bytes / 8;
    const int a16 = a_bytes / 1024, b16 = b_bytes / 1024;
#define DQ_FLOOR_CASE(A, B)                                                    \
    if (a16 == A && b16 == B) {                                                \
        launch_dir<A, B>(direction, a, b, run, pieces, tiles, stream);         \
        return hipGetLastError();                                              \
    }
    DQ_FLOOR_CASE(2, 0)
    DQ_FLOOR_CASE(2, 2)
    DQ_FLOOR_CASE(2, 4)
    DQ_FLOOR_CASE(4, 0)
    DQ_FLOOR_CASE(4, 2)
    DQ_FLOOR_CASE(4, 4)
#undef DQ_FLOOR_CASE
    return hipErrorInvalidValue;
}

} // namespace dq
