// Host-side launcher declarations shared by the translation units of
// libdynamiq_eden.so.  Each launcher enqueues on `stream` and returns the
// launch status; argument validation happens in the C ABI layer (dq_api.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dq_device.cuh"

namespace dq {

// scaling quantisation, catch-all kernels (dq_scaling_generic.hip)
hipError_t launch_generic_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n,
                                   int nbits, int C, int dtype, int strategy, const MeeParams &mp,
                                   hipStream_t stream);
hipError_t launch_generic_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int C,
                                     int dtype, int strategy, const MeeParams &mp, int add,
                                     hipStream_t stream);

// scaling quantisation, vectorised chunk-16 hierarchical kernels
// (dq_scaling_hier16.hip); dtype BF16 or F32, element pointers 16-byte aligned
hipError_t launch_hier16_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n,
                                  int nbits, int dtype, bool mee, const MeeParams &mp,
                                  hipStream_t stream);
hipError_t launch_hier16_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int dtype,
                                    bool mee, const MeeParams &mp, int add, hipStream_t stream);
// compress (recv == null) or the fused ring step with the uniform values drawn in the kernel
hipError_t launch_hier16_compress_philox(const void *src, const uint8_t *recv, uint8_t *dst, int64_t n,
                                         int nbits, int dtype, bool mee, const MeeParams &mp,
                                         uint64_t seed, uint64_t step, hipStream_t stream);
hipError_t launch_hier16_dec_comp(const uint8_t *recv, const void *inp, uint8_t *send,
                                  const void *rnd, int64_t n, int nbits, int dtype, bool mee,
                                  const MeeParams &mp, hipStream_t stream);

// vectorised chunk-16 kernels for the remaining shapes (dq_scaling_tile16.hip): binary16 elements
// with any strategy, bf16 / fp32 elements with the flat strategies 0 / 1
hipError_t launch_tile16_compress(const void *src, uint8_t *dst, const void *rnd, int64_t n, int nbits,
                                  int dtype, int strategy, const MeeParams &mp, hipStream_t stream,
                                  const RandKey *philox = nullptr);
// the in-kernel random stream (dq_device.cuh: chunk_uniform_words) written out as a tensor
hipError_t launch_philox_uniform(void *out, int64_t n, int dtype, uint64_t seed, uint64_t step,
                                 hipStream_t stream);
hipError_t launch_tile16_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int dtype,
                                    int strategy, const MeeParams &mp, int add, hipStream_t stream);

// the same kernels over a list of superchunk indices: record k <-> superchunk rows[k] of the
// element buffer; recv != null makes compress the fused decode-accumulate-recompress step;
// stats != null adds the destination superchunk's mean after decoding; elements >= limit are
// not written
hipError_t launch_hier16_compress_rows(const void *src, const uint8_t *recv, const int32_t *rows,
                                       uint8_t *dst, const void *rnd, int64_t nrows, int nbits,
                                       int dtype, bool mee, const MeeParams &mp, hipStream_t stream);
hipError_t launch_hier16_decompress_rows(const uint8_t *src, void *dst, const int32_t *rows,
                                         const void *stats, int64_t limit, int64_t nrows, int nbits,
                                         int dtype, bool mee, const MeeParams &mp, int add,
                                         hipStream_t stream);

// stable partition of superchunk indices by bit width (dq_grouping.hip)
int64_t group_plan_work_ints(int64_t nsc);
hipError_t launch_group_plan(const int64_t *qbits, int64_t nsc, int32_t *order, int32_t *work,
                             hipStream_t stream);
// the same with the widths computed from the norm column of the bf16 stats and the offset u
// fixed-proportion groups (stable descending sort of the bf16 norms); nsc <= 65535, stats 4-byte aligned
hipError_t launch_group_plan_sorted(const void *stats, int64_t nsc, int64_t top, int64_t bottom, int64_t *qbits_out,
                                    int32_t *order, int32_t *work, hipStream_t stream);
int64_t group_plan_sorted_large_work_ints(int64_t nsc);
hipError_t launch_group_plan_sorted_large(const void *stats, int64_t nsc, int64_t top, int64_t bottom, int64_t *qbits_out,
                                          int32_t *order, int32_t *work, int64_t work_ints, hipStream_t stream);
hipError_t launch_group_plan_stats(const void *stats, float u, const double *u_dev, int64_t nsc, int64_t *qbits_out,
                                   int32_t *order, int32_t *work, uint32_t *hist, hipStream_t stream);

// the offset u of the bit-width rule from a histogram of the norm patterns (dq_bitrate.hip)
int64_t bitrate_hist_ints();
hipError_t launch_norm_histogram(const void *stats, int64_t nsc, uint32_t *hist, hipStream_t stream);
hipError_t launch_bitrate_search(uint32_t *hist, int mode, double prev_u, const double *prev_u_dev, double target, double *out,
                                 hipStream_t stream);

// all bit-width groups of a planned bucket in one launch (dq_scaling_mixed.hip); mp: the MEE
// parameters of 8, 4 and 2 bits in this order; step_dev (nullable, device memory): a value the kernel adds to
// philox->step when it runs, so that a recorded launch can draw fresh rounding randomness on every replay
int64_t mixed_stream_bytes(int64_t nsc, int world);
hipError_t launch_mixed_compress(const void *src, const float *center_mean, int center_world, int64_t n_valid,
                                 const int32_t *order, const int32_t *counts, int ring_chunk, int ring_world,
                                 const uint8_t *recv, uint8_t *dst, const void *rnd, const RandKey *philox,
                                 int64_t nsc, int dtype, bool mee, const MeeParams *mp, hipStream_t stream,
                                 const uint64_t *step_dev = nullptr);
hipError_t launch_mixed_decompress(const uint8_t *src, void *dst, const int32_t *order, const int32_t *counts,
                                   int ring_chunk, int ring_world, const void *stats, int64_t limit, int64_t nsc,
                                   int dtype, bool mee, const MeeParams *mp, hipStream_t stream);

// superchunk mean-centring (dq_superchunk.hip)
// residual == nullptr: statistics only; mean_out (nullable) receives the binary32 means
hipError_t launch_mean_center(const void *src, void *residual, void *stats, float *mean_out, int64_t n,
                              int world_size, int dtype, hipStream_t stream);
hipError_t launch_add_mean_copy(const void *residual, void *dst, const void *stats, int64_t n,
                                int dtype, hipStream_t stream);

// Walsh-Hadamard (dq_hadamard.hip)
hipError_t launch_hadamard(float *vec, int64_t n, hipStream_t stream);
// sign: float +-1 values, or (sign_packed) the bit vector of launch_pack_signs; may be null
hipError_t launch_rht_blocked(float *vec, const void *sign, bool sign_packed, int64_t n, int64_t block, float scale,
                              int inverse, hipStream_t stream);
// EDEN's dequantiser folded into the first pass of the inverse transform, EDEN's scale (device scalar, may be null)
// into the last
hipError_t launch_eden_dequantize_irht(const uint32_t *packed, const float *centroids, int nbits, const void *sign,
                                       bool sign_packed, float *out, int64_t n, int64_t block, float scale,
                                       const float *post_scale, hipStream_t stream);
hipError_t launch_rand_diag(float *out, int64_t size, int64_t seed, hipStream_t stream);
// the same diagonal as packed bits (set where the value is -1); size a multiple of 256
hipError_t launch_rand_diag_bits(uint32_t *bits, int64_t size, int64_t seed, hipStream_t stream);
// THC's quantiser folded into the last pass of the forward transform / the first pass of the inverse one
hipError_t launch_thc_rht_quantize(float *vec, const void *sign, bool sign_packed, const float *uniform, void *levels_out,
                                   int64_t n, int64_t block, float scale, const float *lo, const float *delta, int levels,
                                   hipStream_t stream);
hipError_t launch_thc_dequantize_irht(const void *levels_in, const void *sign, bool sign_packed, float *out, int64_t n,
                                      int64_t block, float scale, const float *step, const float *lo, hipStream_t stream);

// blocked randomized Hadamard transform fused with the hierarchical chunk-16 quantiser (dq_rht_scaling_impl.cuh and the translation units that include it);
// rand_kind: DQ_F32 or DQ_BF16 pool, or 3 for the in-kernel stream (rnd ignored)
hipError_t launch_pack_signs(const float *sign, uint32_t *bits, int64_t n, hipStream_t stream);
// sign: fp32 +-1 values, or with sign_bits one bit per element (launch_pack_signs); may be null
hipError_t launch_rht_compress(const float *src, const void *sign, int sign_bits, uint8_t *dst, const void *rnd, int rand_kind,
                               int64_t n, int64_t block, float scale, int nbits, bool mee, const MeeParams &mp,
                               uint64_t seed, uint64_t step, hipStream_t stream);
hipError_t launch_rht_compress_mfma16(const float *src, const void *sign, int sign_bits, uint8_t *dst, int64_t n, int64_t block,
                                      float scale, const MeeParams &mp, uint64_t seed, uint64_t step, hipStream_t stream);
hipError_t launch_irht_decompress(const uint8_t *src, const void *sign, int sign_bits, float *dst, int64_t n, int64_t block,
                                  float scale, int nbits, bool mee, const MeeParams &mp, hipStream_t stream);
// Quantisers folded into the two ends of a transform (all null: the plain transform).  `in_*` replace the load of the
// first pass, `out_*` / `post_scale` act on the store of the last one.
struct TransformEnds {
    // THC: the pass loads float(level) * *in_step + *in_lo instead of x
    const uint16_t *in_levels = nullptr;
    const float *in_step = nullptr, *in_lo = nullptr;
    // THC: the pass stores thc_level(value, uniform) as bf16 instead of the value
    uint16_t *out_levels = nullptr;
    const float *uniform = nullptr, *out_lo = nullptr, *out_delta = nullptr;
    float out_top = 0.0f;
    // EDEN: the pass loads centroids[bin] from the bit planes of the bins; the last pass multiplies by *post_scale
    const uint32_t *in_planes = nullptr;
    const float *in_centroids = nullptr;
    int in_nbits = 0;
    const float *post_scale = nullptr;
};

hipError_t launch_rht_tile(float *x, const void *sign, int sign_bits, int64_t n, int kt, int kb, float scale, int apply_scale,
                           int sign_mode, int vec, const TransformEnds &ends, hipStream_t stream);
hipError_t launch_rht_strided(float *x, const void *sign, int sign_bits, int64_t n, int rbits, int sbits, float scale,
                              int apply_scale, int sign_mode, int vec, const TransformEnds &ends, hipStream_t stream);

// EDEN Lloyd-Max quantiser + packer, THC uniform quantiser (dq_eden.hip)
int64_t eden_work_doubles(int64_t n);
hipError_t launch_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids,
                                int nbits, uint32_t *packed, float *result, double *work,
                                hipStream_t stream);
// *overlap = 1 when kernels enqueued on a and b run side by side, 0 when the two streams take turns (they share a
// hardware queue, or are the same stream).  Synchronises with both streams: a set-up call, not for stream capture.
hipError_t probe_streams_overlap(hipStream_t a, hipStream_t b, int *overlap);
// `stream` waits for the work enqueued on `after` so far (pooled event, no allocation after the first 64 calls per device)
hipError_t stream_order_after(hipStream_t stream, hipStream_t after, int device);
// a kernel with the access pattern of the chunk-16 codec on `tiles` tiles and no arithmetic (dq_io_floor.hip); direction 0
// reads a and b and writes run, direction 1 reads run (and b) and writes a
bool tile_io_floor_shape_ok(int a_bytes, int b_bytes, int run_bytes);
hipError_t launch_tile_io_floor(int direction, void *a, int a_bytes, const void *b, int b_bytes, void *run, int run_bytes, int64_t tiles,
                                hipStream_t stream);

// the same launches with the partial sums in the library's own static device array (no allocation anywhere);
// `device` must be current
int64_t eden_static_max_n();
hipError_t eden_static_prepare(int device);
hipError_t launch_eden_quantize_static(const float *vec, int64_t n, const float *boundaries, const float *centroids,
                                       int nbits, uint32_t *packed, float *result, int device,
                                       hipStream_t stream);
hipError_t launch_eden_dequantize(const uint32_t *packed, int64_t n, const float *centroids, int nbits,
                                  float *out, hipStream_t stream);
hipError_t launch_thc_quantize(const float *rotated, const float *uniform, void *out, int64_t n,
                               const float *lo, const float *delta, int levels, hipStream_t stream);
hipError_t launch_thc_dequantize(const void *levels, float *out, int64_t n, const float *step,
                                 const float *lo, hipStream_t stream);

// EDEN bit-plane packing and THC rounding (dq_packing.hip)
hipError_t launch_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int nbits,
                               hipStream_t stream);
hipError_t launch_bits_to_bins(int32_t *bins, int64_t nbins, const uint32_t *arr, int nbits,
                               hipStream_t stream);
hipError_t launch_quantization(float *vec, int64_t n, float div_factor, float tensor_max,
                               uint64_t seed, hipStream_t stream);

} // namespace dq
