/*
 * CPU oracle for the eden_utils gradient-compression path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a scalar, single-threaded restatement of
 * the reference algorithm used to check the HIP kernels byte-for-byte.  The
 * shipped library never links, loads or calls anything in this directory;
 * only tests/, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function cites the reference source it restates (paths are relative
 * to the reference checkout, cuda_kernels/src/srrcomp/eden_utils unless the
 * path says otherwise).
 *
 * Arithmetic conventions (these define "bit-exact" for the GPU kernels):
 *   - all fp32 operations are IEEE-754 binary32, round-to-nearest-even, with
 *     denormals preserved and NO implicit contraction; a multiply feeding an
 *     add is fused only where this file calls fmaf() explicitly (the decode
 *     "code*scale + accumulator" step, which the reference's compiler fuses);
 *   - half-precision ops of the fp16 path are evaluated as fp32 op followed
 *     by one round-to-nearest-even to binary16 (exactly the correctly rounded
 *     half result for + - * /);
 *   - log2 is dqo_log2f(), a fixed polynomial evaluated with explicit fmaf
 *     (<= 1.7 ulp); it replaces the device log2f/hlog2 so that MEE codes are
 *     reproducible on any IEEE machine;
 *   - float -> int16 conversions saturate and map NaN to 0, int16 additions
 *     wrap (what the reference's cvt/add instructions do).
 *
 * What pins this file (tests/test_oracle_*.py): the reference's golden vectors
 * for randDiag, the bit-plane packer, the torch butterfly and 50 Eden
 * compress / decompress runs (the .npz files under tests/golden, written by the reference's own
 * CPU code); closed forms, special cases and invariants of the reference's
 * functional test for the scaling quantiser; an independently written numpy
 * model of the bf16 / fp16 arithmetic.
 *
 * Parity unpinned (no reference output can exist or be reproduced):
 *   - bit patterns of MEE codes on the reference's own GPU (device log2f under
 *     fast-math); pinned to dqo_log2f instead;
 *   - the last bits of dqo_eden_quantize's scale and bins within rounding error
 *     of a boundary (torch's reduction order is unspecified); tolerance-pinned;
 *   - dqo_thc_quantize's individual roundings (torch's bernoulli_ stream); the
 *     uniform draws are an input here;
 *   - fp32-element and 3/5/6/7-bit scaling modes (extensions of the reference's
 *     formulas, checked against the numpy model only).
 * quantization_compression has no restatement at all: the reference's curand
 * states are never initialised (csrc/cuda_hadamard.cu:669-686).
 */
#ifndef DQ_ORACLE_H
#define DQ_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { DQO_F16 = 0, DQO_BF16 = 1, DQO_F32 = 2 };

/* status codes shared by the scaling entry points (0 = ok) */
enum {
    DQO_OK = 0,
    DQO_ERR_N = 1,          /* n must be positive                        */
    DQO_ERR_NBITS = 2,      /* nbits not in the accepted set             */
    DQO_ERR_STRATEGY = 3,   /* strategy not in [0,3]                     */
    DQO_ERR_CHUNK_RANGE = 4,/* chunk_size not in [1,32]                  */
    DQO_ERR_CHUNK_POW2 = 5, /* chunk_size not a power of two             */
    DQO_ERR_CHUNK_BITS = 6, /* chunk_size*nbits not divisible by 8       */
    DQO_ERR_N_CHUNK = 7,    /* n not a multiple of chunk_size            */
    DQO_ERR_N_SUPER = 8,    /* hierarchical: chunks not a multiple of 16 */
    DQO_ERR_DTYPE = 9
};

/* eden_utils.cpp:33-40 */
int64_t dqo_scaling_required_bytes(int64_t n, int nbits, int chunk_size, int strategy);
/* eden_utils.cpp:42-53; strict != 0 keeps nbits in {2,4,8}, otherwise 2..8 */
int dqo_scaling_check(int64_t n, int nbits, int chunk_size, int strategy, int strict);

/* csrc/cuda_hadamard.cu:873-899.  table: 256 binary16 bit patterns; params:
 * {one_plus_2eps2, one_plus_eps2_over_2eps2, chunk_max_mee, log2_one_plus_2eps2}
 * as binary16 bit patterns. nbits in 1..8. */
void dqo_mee_lut(int nbits, uint16_t table[256], uint16_t params[4]);

/* deterministic log2 used by the MEE inverse lattice */
float dqo_log2f(float x);

/* conversions (exposed so tests can pin them against numpy/torch) */
float    dqo_bf16_to_f32(uint16_t h);
uint16_t dqo_f32_to_bf16(float f);
float    dqo_f16_to_f32(uint16_t h);
uint16_t dqo_f32_to_f16(float f);

/* csrc/cuda_hadamard.cu:768-817,941-997,1055-1094,1138-1178 (flat) and
 * csrc/cuda_hierarchical_mee.cu:203-343,698-774,844-930,1016-1089,1149-1222 */
int dqo_scaling_compress(const void *src, uint8_t *dst, const void *rand_pool,
                         int64_t n, int nbits, int chunk_size, int strategy, int dtype);

/* csrc/cuda_hadamard.cu:819-861,999-1053,1096-1136,1180-1234 and
 * csrc/cuda_hierarchical_mee.cu:345-505,776-842,932-1014,1091-1147,1224-1294 */
int dqo_scaling_decompress(const uint8_t *src, void *dst, int64_t n, int nbits,
                           int chunk_size, int strategy, int dtype, int add_original);

/* eden_utils.cpp:191-219 + csrc/cuda_hadamard.cu:1710-1753 +
 * csrc/cuda_hierarchical_mee.cu:526-696.  Fused (inp untouched) for
 * bf16/f32 with chunk 16 and strategy 2/3; otherwise decompress_add into inp
 * followed by compress, exactly like the reference dispatch. */
int dqo_scaling_dec_comp(const uint8_t *recv, void *inp, uint8_t *send, const void *rand_pool,
                         int64_t n, int nbits, int chunk_size, int strategy, int dtype);

/* csrc/cuda_hadamard.cu:1257-1349; stats is bf16 [2*ceil(n/256)] */
void dqo_superchunk_mean_center(const void *src, void *residual, uint16_t *stats,
                                int64_t n, int world_size, int dtype);
/* the same statistics without the residual, plus the unrounded binary32 mean of every superchunk
 * (the value the residual is formed with) */
void dqo_superchunk_stats(const void *src, uint16_t *stats, float *mean, int64_t n, int world_size,
                          int dtype);
/* csrc/cuda_hadamard.cu:1351-1369 */
void dqo_superchunk_add_mean_copy(const void *residual, void *dst, const uint16_t *stats,
                                  int64_t n, int dtype);

/* csrc/cuda_hadamard.cu:66-157,205-274,534-605: unnormalised FWHT, stages in
 * ascending stride, butterflies (a+b, a-b). n must be a power of two. */
void dqo_fwht(float *x, int64_t n);
/* Blocked randomized transform (extension): per block of `block` elements
 * y = FWHT(sign .* x) * scale (forward) or y = sign .* (FWHT(x) * scale)
 * (inverse).  On one block equals thc_hooks.py:95-107 / srrcomp.py:317-319. */
void dqo_rht_blocked(float *x, const float *sign, int64_t n, int64_t block, float scale, int inverse);

/* srrcomp.py:61-106 (torchRNG=False branch) */
void dqo_rand_diag(float *out, int64_t size, int64_t seed);

/* csrc/cuda_packing.cu:11-29 / 76-95 and srrcomp.py:124-167 */
void dqo_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int nbits);
void dqo_bits_to_bins(const uint32_t *arr, int64_t narr, int32_t *bins, int nbits);

/* The random stream of the library's in-kernel rounding mode (no counterpart in the reference, whose
 * random values are an input tensor): Philox4x32-10, pinned by the published known-answer vectors. */
void dqo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
void dqo_philox_uniform(float *out, int64_t n, uint64_t seed, uint64_t step);
void dqo_philox_uniform_rows(float *out, const int64_t *rows, int64_t nrows, uint64_t seed, uint64_t step);

/* cuda_kernels/src/srrcomp/srrcomp.py:356-361 (Eden._quantize) and :343-345; sums in double in the
 * library's documented order (torch's reduction order is unspecified: "parity unpinned" for the
 * last bits of `scale`, pinned within tolerance by the reference's own outputs in
 * tests/golden/eden_golden.npz).  result = {sum of squares, dot, scale, norm}. */
void dqo_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids,
                       int nbits, int32_t *bins, float *result);
void dqo_eden_dequantize(const int32_t *bins, int64_t n, const float *centroids, float *out);

/* testbed_evaluation/new_comm_hooks/thc_hooks.py:161-166 and :176-178; the Bernoulli draw is an
 * input (uniform < probability): torch's bernoulli_ stream is "parity unpinned". */
void dqo_thc_quantize(const float *rotated, const float *uniform, uint16_t *levels_bf16, int64_t n,
                      float lo, float delta, int levels);
void dqo_thc_dequantize(const uint16_t *levels_bf16, float *out, int64_t n, float step, float lo);

/* testbed_evaluation/new_comm_hooks/comm_hooks.py:64-70 evaluated on bf16
 * norms with bf16 rounding after every tensor op (what torch does for a bf16
 * tensor); qbits out as int64. */
void dqo_dynamic_bitrate_qbits(const uint16_t *norms_bf16, int64_t stride, int64_t count,
                               double u, int64_t *qbits);

/* testbed_evaluation/new_comm_hooks/comm_hooks.py:718: torch.argsort(norms, descending=True,
 * stable=True) of bf16 norms (NaN first, ties by ascending index); order: int64 [count]. */
void dqo_argsort_descending_stable(const uint16_t *norms_bf16, int64_t stride, int64_t count,
                                   int64_t *order);

/* csrc/cuda_hadamard.cu:607-627 with the library's Philox stream in place of the reference's
 * uninitialised curand states ("parity unpinned" for the stream, the arithmetic is the reference's). */
void dqo_quantization(float *vec, int64_t n, float div_factor, float tensor_max, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif
