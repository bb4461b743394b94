/*
 * C ABI of libdynamiq_eden.so -- the MI355X (gfx950) implementation of the
 * on-GPU gradient-compression path behind DynamiQ's `eden_utils` module.
 *
 * Every entry point takes plain device pointers, sizes, a HIP device index and
 * a HIP stream handle (hipStream_t passed as void*; NULL = the null stream).
 * All work is enqueued asynchronously on that stream; nothing synchronises,
 * nothing allocates device memory, no state is kept between calls, and the
 * functions are re-entrant (they may be called concurrently from several host
 * threads on distinct streams with sub-buffer pointers at record-aligned
 * offsets, as ring_allreduce_backend.cu:1262-1289 does).
 *
 * Return value: DQ_OK (0) or a dq_status code.  Argument errors carry the same
 * message text as the TORCH_CHECKs of the reference binding
 * (eden_utils.cpp:42-53); dq_last_error() returns the text for the calling
 * thread.  Unlike the reference (which only prints launch failures,
 * cuda_hadamard.cu:1496-1499) a failed launch is reported as DQ_ERR_LAUNCH.
 *
 * "reference" paths below are relative to
 * cuda_kernels/src/srrcomp/eden_utils/ of the DynamiQ artifact.
 */
#ifndef DYNAMIQ_EDEN_H
#define DYNAMIQ_EDEN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *dq_stream_t; /* hipStream_t */

/* element type of gradient / random buffers */
enum dq_dtype {
    DQ_F16 = 0,  /* reference __half path: every intermediate in binary16   */
    DQ_BF16 = 1, /* reference __nv_bfloat16 path: fp32 math, bf16 storage   */
    DQ_F32 = 2   /* extension: the bf16 path's math on fp32 storage         */
};
/* OR-ed into the dtype argument of dq_scaling_compress / dq_scaling_dec_comp:
 * rand_pool holds bfloat16 values although the gradient elements are DQ_F32
 * (the reference's pools are bf16, utils_aggregation.py:384-389; this saves
 * 2 bytes per element of HBM traffic for fp32 gradients). */
#define DQ_RAND_BF16 0x10

enum dq_status {
    DQ_OK = 0,
    DQ_ERR_N = 1,
    DQ_ERR_NBITS = 2,
    DQ_ERR_STRATEGY = 3,
    DQ_ERR_CHUNK_RANGE = 4,
    DQ_ERR_CHUNK_POW2 = 5,
    DQ_ERR_CHUNK_BITS = 6,
    DQ_ERR_N_CHUNK = 7,
    DQ_ERR_N_SUPER = 8,
    DQ_ERR_DTYPE = 9,
    DQ_ERR_NULL = 10,
    DQ_ERR_SUPERCHUNK_SIZE = 11,
    DQ_ERR_WORLD_SIZE = 12,
    DQ_ERR_POW2 = 13,
    DQ_ERR_SIZE = 14,
    DQ_ERR_DEVICE = 15,
    DQ_ERR_LAUNCH = 16
};

const char *dq_status_string(int status);
const char *dq_last_error(void);
/* library build identification: "dynamiq_eden <version> gfx950" */
const char *dq_version(void);

/* ---- sizes and validation -------------------------------------------- */

/* eden_utils.cpp:33-40 (scaling_required_bytes) */
int64_t dq_scaling_required_bytes(int64_t n, int nbits, int chunk_size, int strategy);
/* eden_utils.cpp:42-53 (scaling_check_common).  nbits in {2,4,8} when
 * strict != 0; strict == 0 also admits the 3/5/6/7-bit extension codes. */
int dq_scaling_check_common(int64_t n, int nbits, int chunk_size, int strategy, int strict);

/* ---- MEE lookup table ------------------------------------------------- */

/* csrc/cuda_hadamard.cu:935-939 (init_lookup_table).  The table is built on
 * the host once per process and travels to the kernels as launch arguments,
 * so this call is optional and never touches the device. */
int dq_init_lookup_table(void);
/* csrc/cuda_hadamard.cu:873-899: copies the 256 binary16 table entries and the
 * four binary16 parameters {1+2e^2, (1+e^2)/(2e^2), chunk_max_mee,
 * log2(1+2e^2)} for nbits in 1..8. */
int dq_mee_lookup_table(int nbits, uint16_t table[256], uint16_t params[4]);

/* ---- scaling quantisation -------------------------------------------- */

/* csrc/cuda_hadamard.h:18,20 (scaling_compress_with_cuda, both overloads).
 * src, rand_pool: `dtype` elements [>= n]; dst: packed records
 * [>= dq_scaling_required_bytes].  strategy 0 AEE, 1 MEE, 2/3 hierarchical. */
int dq_scaling_compress(const void *src, uint8_t *dst, const void *rand_pool, int64_t n,
                        int nbits, int chunk_size, int dtype, int device, int strategy,
                        dq_stream_t stream);

/* csrc/cuda_hadamard.h:19,21 (scaling_decompress_with_cuda).  add_original
 * != 0 accumulates into dst (scaling_decompress_add). */
int dq_scaling_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int chunk_size,
                          int dtype, int device, int strategy, dq_stream_t stream,
                          int add_original);

/* csrc/cuda_hadamard.h:22 (scaling_dec_comp_with_cuda) plus the fp16 split of
 * eden_utils.cpp:212-214.  send = compress(round(inp + decode(recv))).  With
 * bf16/f32, chunk_size 16 and strategy 2/3 this is one fused kernel and inp is
 * left untouched; every other combination decodes INTO inp first, exactly like
 * the reference dispatch (csrc/cuda_hadamard.cu:1744-1747). */
int dq_scaling_dec_comp(const uint8_t *recv, void *inp, uint8_t *send, const void *rand_pool,
                        int64_t n, int nbits, int chunk_size, int dtype, int device,
                        int strategy, dq_stream_t stream);

/* ---- in-kernel random stream -------------------------------------------
 *
 * No counterpart in the reference, whose random values always arrive as the
 * rand_pool tensor (utils_aggregation.py:384-397).  Here the uniform values of
 * the stochastic rounding are drawn inside the kernel from Philox4x32-10:
 * key = seed, counter = (chunk index, step); the 16 bytes of one block are the
 * 16 values of one chunk, u = (byte | 1) / 256 (the odd multiples of 1/256:
 * unbiased rounding, exact in all three element types).  This removes the 2 (4) bytes per
 * element the pool costs in HBM reads.  chunk_size must be 16; every dtype and
 * strategy.  The result equals dq_scaling_compress / dq_scaling_dec_comp fed
 * with the tensor dq_philox_uniform writes for the same (seed, step). */
int dq_scaling_compress_philox(const void *src, uint8_t *dst, int64_t n, int nbits, int chunk_size,
                               int dtype, int device, int strategy, uint64_t seed, uint64_t step,
                               dq_stream_t stream);
int dq_scaling_dec_comp_philox(const uint8_t *recv, void *inp, uint8_t *send, int64_t n, int nbits,
                               int chunk_size, int dtype, int device, int strategy, uint64_t seed,
                               uint64_t step, dq_stream_t stream);
/* out: `dtype` elements [n]; element e = (byte e % 16 of the block of chunk e / 16, low bit set) * 2^-8 */
int dq_philox_uniform(void *out, int64_t n, int dtype, int device, uint64_t seed, uint64_t step,
                      dq_stream_t stream);

/* ---- dynamic-bitrate groups: gather / scatter folded into the codec ----
 *
 * The reference's dynamic-bitrate hook builds, per bit width w in {8, 4, 2}, the
 * list of superchunks with that width (three torch.nonzero calls,
 * testbed_evaluation/new_comm_hooks/comm_hooks.py:964-966), copies them into a
 * contiguous group tensor (index_select, :1001), runs the compressed ring on the
 * group, copies the result back (index_copy_, :1011) and finally adds the means
 * (superchunk_add_mean_copy, :1019).  The entry points below produce the same
 * bytes without the group tensor: record k of a packed stream stands for
 * superchunk rows[k] of the full residual / output buffer.  chunk_size is 16,
 * strategy 2 or 3, dtype DQ_BF16 or DQ_F32 (DQ_RAND_BF16 allowed on the
 * compress side); other combinations return DQ_ERR_DTYPE / DQ_ERR_STRATEGY. */

/* number of int32 the `work` argument of dq_group_plan must hold */
int64_t dq_group_plan_work_ints(int64_t nsc);

/* comm_hooks.py:964-966.  qbits: int64 [nsc] on the device (the output of
 * _dynamic_bitrate_qbits, :48-66).  order: int32 [3 * nsc], one region of nsc
 * entries per width; on return order[0..n8) lists, ascending, the superchunks
 * with qbits == 8, order[nsc..nsc+n4) those with 4 and order[2*nsc..2*nsc+n2)
 * those with 2 (torch.nonzero order); the rest of order is not written.
 * work[0..2] = n8, n4, n2 and work[3] = superchunks of any other width (they
 * appear in no group); the rest of work is scratch.  One launch on `stream`
 * for nsc <= 65536, two beyond; no host synchronisation. */
int dq_group_plan(const int64_t *qbits, int64_t nsc, int32_t *order, int32_t *work,
                  int64_t work_ints, int device, dq_stream_t stream);

/* comm_hooks.py:48-70 (_dynamic_bitrate_qbits on the bf16 norms, every torch op
 * rounding its result to bf16) + :964-966 in one call: the width of superchunk
 * i is computed from stats[2 * i + 1] (the reduced sum of squares written by
 * dq_superchunk_mean_center) and the offset u, log2 being the library's fixed
 * polynomial.  qbits_out: int64 [nsc] or NULL. */
int dq_group_plan_stats(const void *stats, double u, int64_t nsc, int64_t *qbits_out,
                        int32_t *order, int32_t *work, int64_t work_ints, int device,
                        dq_stream_t stream);

/* comm_hooks.py:710-721, the fixed-proportion allocation of the non-dynamic
 * P2P_dynamiQ hook: sorted = argsort(norms, descending=True, stable=True) over
 * the reduced sums of squares stats[2 * i + 1]; its first top_count entries are
 * the 8-bit group, its last bottom_count entries the 2-bit group, the rest the
 * 4-bit group (the caller derives the two counts from the method's fractions,
 * :713-716, :842-856).  order / work as written by dq_group_plan, except that
 * every list is in **sorted order** (descending norm, equal norms by ascending
 * index, NaN before every number, -0 == +0: torch's documented order and what
 * its CPU sort does; torch's radix sort on a device orders NaNs by payload and
 * puts a NaN with the sign bit set behind -inf, patterns that sums of squares
 * computed on a device do not take), which is the order in which the hook
 * gathers a group and pairs it with rand_pool rows.  qbits_out: int64
 * [nsc] or NULL.  No host synchronisation.  Up to 65535 superchunks: one
 * launch, no sort passes (the key is a 16-bit pattern: counting sort in LDS),
 * work holds 4 ints.  Longer buckets (the reference's training scripts give
 * DDP a 4000 MB bucket cap, testbed_evaluation/train_llm_causal.py:416): a
 * stable radix sort of the 16-bit keys inside `work`, which must then hold
 * dq_group_plan_sorted_work_ints(nsc) ints (about 12.2 bytes per superchunk; the
 * figure includes the scratch the sort library asks for on the current device,
 * so call it with the device selected that will run the plan).  The long path
 * runs the library's sort, whose launches include memset nodes: only the
 * one-launch path (nsc <= 65535) may be captured into a HIP graph.
 * stats 4-byte aligned. */
int64_t dq_group_plan_sorted_work_ints(int64_t nsc);
int dq_group_plan_sorted(const void *stats, int64_t nsc, int64_t top_count, int64_t bottom_count,
                         int64_t *qbits_out, int32_t *order, int32_t *work, int64_t work_ints,
                         int device, dq_stream_t stream);

/* the same with the offset read from device memory when the kernels run
 * (u_dev: one float64, e.g. result[0] of dq_bitrate_search): a training step
 * then needs no read-back of u at all.  hist (may be NULL; dq_bitrate_hist_ints()
 * uint32): the bucket's norm patterns are also added to it, as by
 * dq_norm_histogram, by a few more workgroups of the same launch (for nsc <= 65536).
 * The launch leaves the two width thresholds it derived from u in work[4..6]
 * (with the bits of u and a check word); the next call on the same work buffer
 * with the same u takes them from there instead of searching again, so a
 * caller that plans many buckets per step does well to keep one work buffer
 * per stream.  Whatever else those words hold is recognised and ignored.
 * No counterpart in the reference, which keeps u on the host. */
int dq_group_plan_stats_dev_u(const void *stats, const double *u_dev, int64_t nsc,
                              int64_t *qbits_out, int32_t *order, int32_t *work,
                              int64_t work_ints, uint32_t *hist, int64_t hist_ints, int device,
                              dq_stream_t stream);

/* ---- the offset u of the bit-width rule (comm_hooks.py:73-139) -----------
 *
 * The reference probes the average width at up to 33 values of u per search,
 * each probe being ten torch ops and a reduction over the norms of every bucket
 * with a read-back.  The width depends on a norm only through its bf16 pattern,
 * so the library counts the patterns once and searches on the counts. */

/* number of uint32 the `hist` argument below must hold (zeroed before the first
 * dq_norm_histogram of a training step) */
int64_t dq_bitrate_hist_ints(void);

/* adds the norm patterns stats[2 * i + 1], i < nsc (the reduced sums of squares
 * written by dq_superchunk_mean_center / dq_superchunk_stats, after the
 * all-reduce) to hist; call once per bucket.  At most 2^32 - 1 norms in all. */
int dq_norm_histogram(const void *stats, int64_t nsc, uint32_t *hist, int64_t hist_ints,
                      int device, dq_stream_t stream);

/* mode 0: _dynamic_bitrate_binary_search_u (comm_hooks.py:94-114); mode 1:
 * _dynamic_bitrate_adjust_u from prev_u (:117-139).  One launch, the whole
 * search on the device.  result: float64 [4] on the device = u, the average
 * width at u, target_avg_bits minus that average, the number of probes; the
 * first three are what the reference's function returns for the same norms.
 * hist is consumed: on return it is all zero, ready for the next step.
 * prev_u_dev (may be NULL): when set, mode 1 starts from the float64 it points
 * to on the device instead of prev_u; it may be result itself, so that the u of
 * one step feeds the correction of the next without leaving the device. */
int dq_bitrate_search(uint32_t *hist, int64_t hist_ints, int mode, double prev_u,
                      const double *prev_u_dev, double target_avg_bits, double *result,
                      int device, dq_stream_t stream);

/* comm_hooks.py:1001 + scaling_compress: dst record k (and rand_pool row k,
 * 256 elements) encodes superchunk rows[k] of src.  rows: int32 [nrows] on the
 * device, every entry in [0, src superchunks).  rows == NULL means rows[k] = k. */
int dq_scaling_compress_rows(const void *src, const int32_t *rows, uint8_t *dst,
                             const void *rand_pool, int64_t nrows, int nbits, int dtype,
                             int device, int strategy, dq_stream_t stream);

/* the ring's fused step on a group: send record k =
 * compress(round(inp[rows[k]] + decode(recv record k))); inp is not modified. */
int dq_scaling_dec_comp_rows(const uint8_t *recv, const void *inp, const int32_t *rows,
                             uint8_t *send, const void *rand_pool, int64_t nrows, int nbits,
                             int dtype, int device, int strategy, dq_stream_t stream);

/* scaling_decompress + comm_hooks.py:1011 (+ :1019 when stats != NULL): record
 * k decodes into superchunk rows[k] of dst.  With stats (bf16 pairs
 * (mean, sum of squares) per superchunk of dst, as written by
 * dq_superchunk_mean_center) the value stored is
 * T(float(T(decoded)) + float(stats[2 * rows[k]])) -- what decompress into the
 * residual followed by superchunk_add_mean_copy stores.  Elements at index >=
 * n_limit of dst are not written (n_limit = the unpadded element count when dst
 * is the final output; pass the padded count for a residual buffer).
 * add_original != 0 accumulates into dst (stats must then be NULL). */
int dq_scaling_decompress_rows(const uint8_t *src, void *dst, const int32_t *rows,
                               const void *stats, int64_t n_limit, int64_t nrows, int nbits,
                               int dtype, int device, int strategy, dq_stream_t stream,
                               int add_original);

/* ---- the three bit-width groups of a bucket in one launch ----------------
 *
 * comm_hooks.py:963-1018 runs gather -> ring all-reduce -> scatter once per
 * bit-width group (8, 4, 2), with the group sizes known on the host.  The
 * calls below take the partition from device memory instead -- `order` and the
 * first three ints of `work` as written by dq_group_plan / dq_group_plan_stats
 * (n8, n4, n2) -- and serve all three groups with one launch and no host
 * synchronisation.
 *
 * Ring chunk `ring_chunk` of `ring_world` is, per group, superchunks
 * [per * ring_chunk, min(per * (ring_chunk + 1), n_g)) of the group with
 * per = ceil(n_g / ring_world) (the split of ring_rdma.py:590-631 applied to a
 * gathered group).  Its packed stream is the 8-bit records, then the 4-bit
 * records, then the 2-bit records, each run byte for byte what
 * dq_scaling_compress_rows writes for the same superchunks and random values;
 * dq_mixed_required_bytes(nsc, ring_world) bounds its size.  ring_world = 1,
 * ring_chunk = 0 addresses whole groups.
 *
 * Rounding randomness: rand_pool != NULL -> row k (256 values, element type of
 * src, or bf16 with DQ_RAND_BF16) belongs to the k-th superchunk of the
 * concatenation 8-bit group | 4-bit group | 2-bit group, so the pool holds
 * >= 256 * nsc values; rand_pool == NULL -> the in-kernel Philox
 * stream of dq_scaling_compress_philox, keyed by (seed, step, index of the
 * chunk in src).
 *
 * center_mean != NULL folds superchunk_mean_center into the load: element e
 * of src is replaced by T(float(src[e]) / center_world - center_mean[e / 256]),
 * and by zero at e >= n; nothing at or beyond n is read.  center_mean is the
 * binary32 mean array written by dq_superchunk_stats.  With center_mean ==
 * NULL src is a residual buffer of 256 * nsc elements and n is ignored.
 * recv != NULL makes the call the ring's fused step (decode recv, add the
 * centred source, re-encode into dst; recv and dst share one layout).
 * strategy 2 or 3, dtype DQ_BF16 or DQ_F32. */
int64_t dq_mixed_required_bytes(int64_t nsc, int ring_world);
int dq_mixed_compress(const void *src, const float *center_mean, int center_world, int64_t n,
                      const int32_t *order, const int32_t *counts, int ring_chunk, int ring_world,
                      const uint8_t *recv, uint8_t *dst, const void *rand_pool, uint64_t seed,
                      uint64_t step, int64_t nsc, int dtype, int device, int strategy,
                      dq_stream_t stream);

/* decode ring chunk `ring_chunk` of all three groups into their superchunks of
 * dst; stats / n_limit as in dq_scaling_decompress_rows. */
int dq_mixed_decompress(const uint8_t *src, void *dst, const int32_t *order, const int32_t *counts,
                        int ring_chunk, int ring_world, const void *stats, int64_t n_limit,
                        int64_t nsc, int dtype, int device, int strategy, dq_stream_t stream);

/* cuda_hadamard.cu:1304-1349 without the residual: stats as written by
 * dq_superchunk_mean_center, plus (mean != NULL) the unrounded binary32 mean
 * of every superchunk, float [ceil(n / 256)]. */
int dq_superchunk_stats(const void *src, void *stats, float *mean, int64_t n, int world_size,
                        int dtype, int device, dq_stream_t stream);

/* ---- one bucket of the dynamic-bitrate path in one host call --------------
 *
 * The reference's hook runs a bucket as a sequence of Python-level steps
 * (comm_hooks.py:932-1024: superchunk_mean_center, the stats all-reduce, the
 * width rule, three nonzero / index_select / ring / index_copy_ rounds,
 * superchunk_add_mean_copy).  With the calls above the same bucket is four
 * launches -- dq_superchunk_stats, dq_group_plan_stats(_dev_u),
 * dq_mixed_compress, dq_mixed_decompress -- and on a 25 MB bucket the host's
 * cost of four calls is as long as the kernels.  dq_dynamic_bitrate_bucket
 * enqueues any run of these stages for one bucket with one call; the stages,
 * their arguments and their results are exactly those of the four calls.
 *
 *   DQ_STAGE_STATS       src -> stats (bf16 pairs), mean (binary32)   [dq_superchunk_stats, world = center_world]
 *   DQ_STAGE_PLAN        reduced_stats (or stats when NULL), u or *u_dev -> order, work[0..3] (+ hist)
 *   DQ_STAGE_COMPRESS    src centred on load with mean -> packed: ring chunk ring_chunk of ring_world, recv != NULL =
 *                        the fused ring step; in-kernel rounding stream (seed, step + *step_dev)
 *   DQ_STAGE_DECOMPRESS  packed -> out (+ the mean of reduced_stats), elements below n
 *
 * A ring of one rank (or a rank's local round trip) runs all four at once; in
 * a ring of several ranks the stats all-reduce sits between STATS and PLAN and
 * the exchanges between the codec stages, so a rank calls it once per run of
 * consecutive stages.  step_dev (may be NULL): one uint64 in device memory that
 * the encoder adds to `step` when it runs -- a launch recorded into a HIP graph
 * then draws fresh rounding randomness on every replay if the owner advances
 * that counter between replays.  No counterpart in the reference. */
enum { DQ_STAGE_STATS = 1, DQ_STAGE_PLAN = 2, DQ_STAGE_COMPRESS = 4, DQ_STAGE_DECOMPRESS = 8 };

typedef struct dq_bucket {
    const void *src;            /* n elements of dtype (DQ_BF16 or DQ_F32) */
    int64_t n;
    int32_t dtype, strategy;    /* strategy 2 (AEE) or 3 (MEE) */
    int32_t center_world;       /* the divisor of superchunk_mean_center */
    int32_t ring_chunk, ring_world;
    int32_t reserved;
    double u;                   /* offset of the width rule, used when u_dev == NULL */
    const double *u_dev;        /* ... or read from device memory when the plan runs */
    void *stats;                /* bf16 [nsc, 2], nsc = ceil(n / 256): written by STATS */
    float *mean;                /* float [nsc]: written by STATS, read by COMPRESS */
    const void *reduced_stats;  /* the stats after the all-reduce; NULL = stats */
    int32_t *order;             /* int32 [3 nsc] */
    int32_t *work;              /* int32 [work_ints], work_ints >= dq_group_plan_work_ints(nsc) */
    int64_t work_ints;
    const uint8_t *recv;        /* may be NULL */
    uint8_t *packed;            /* packed_bytes >= dq_mixed_required_bytes(nsc, ring_world) */
    int64_t packed_bytes;
    void *out;                  /* n elements of dtype: written by DECOMPRESS */
    uint32_t *hist;             /* may be NULL; with u_dev only (see dq_group_plan_stats_dev_u) */
    int64_t hist_ints;
    uint64_t seed, step;
    const uint64_t *step_dev;   /* may be NULL */
} dq_bucket_t;

int dq_dynamic_bitrate_bucket(const dq_bucket_t *bucket, int stages, int device, dq_stream_t stream);

/* No counterpart in the reference (its hooks run every bucket on one stream).
 * A caller that keeps several buckets in flight, each on a stream of its own,
 * gains from it only when the streams run side by side: the runtime maps the
 * streams of a process onto a few hardware queues (4 by default) at their
 * first use, and two streams on one queue take turns.  *overlap = 1 when
 * kernels enqueued on a and b overlap, 0 when they are serialised (or a == b).
 * Measured with a 0.1 ms single-wave kernel on each stream; synchronises with
 * both streams and creates events: a set-up call, not for stream capture. */
int dq_streams_overlap(dq_stream_t a, dq_stream_t b, int device, int *overlap);

/* No counterpart in the reference.  `stream` waits for everything enqueued on
 * `after` so far (what a framework's wait_stream does), through an event taken
 * from a ring the library keeps per device: nothing is created after the first
 * 64 calls on a device, and the call costs the host two runtime calls.  A
 * caller that hands each bucket to a worker stream as it becomes ready uses
 * it in place of creating an event per bucket.  Not for stream capture. */
int dq_stream_order_after(dq_stream_t stream, dq_stream_t after, int device);

/* No counterpart in the reference: a measurement aid.  Launches a kernel with
 * the launch shape and the memory accesses of the chunk-16 codec kernels -- one
 * wave per tile of 1,024 elements, each lane reading its chunk as 16-byte
 * pieces, each wave writing one unaligned run of record bytes -- and no
 * arithmetic beyond an exclusive-or of everything a lane loaded, which its
 * stores carry.  Timed over the same buffers as a codec call, it tells how
 * much of that call's time the launch itself and its memory traffic account
 * for.  direction 0 (encoder shape): per tile read a_bytes_per_tile from `a`
 * and b_bytes_per_tile from `b`, write run_bytes_per_tile to `run`.
 * direction 1 (decoder shape): per tile read the run (and `b` when
 * b_bytes_per_tile > 0), write `a` with streaming stores.  a_bytes_per_tile
 * is 2048 or 4096 (1,024 bf16 or fp32 elements), b_bytes_per_tile 0, 2048 or
 * 4096, run_bytes_per_tile a multiple of 8 up to 8192 (4 * record bytes).
 * What it writes has no meaning; it overwrites `run` (direction 0) or `a`
 * (direction 1) over tiles * bytes_per_tile bytes. */
int dq_tile_io_floor(int direction, void *a, int a_bytes_per_tile, const void *b, int b_bytes_per_tile,
                     void *run, int run_bytes_per_tile, int64_t tiles, int device, dq_stream_t stream);

/* ---- consumers of the rotated vector: EDEN and THC ----------------------
 *
 * "reference" here: cuda_kernels/src/srrcomp/srrcomp.py (EDEN) and
 * testbed_evaluation/new_comm_hooks/thc_hooks.py (THC); both run these steps
 * as chains of torch ops around eden_utils.Hadamard. */

/* number of doubles the `work` argument of dq_eden_quantize must hold */
int64_t dq_eden_work_doubles(int64_t n);

/* srrcomp.py:356-361 (Eden._quantize) + :124-145 (EdenBinsToBits) in one call.
 * vec: float32 [n], n a positive multiple of 32 (the caller pads, :300-309).
 * boundaries: float32 [2^nbits - 1] ascending, centroids: float32 [2^nbits]
 * (Eden.boundaries[nbits], Eden.centroids[nbits]); nbits 1..8.
 *   bin_i   = #{ b in boundaries : !(b >= x_i) },  x_i = (vec_i * (float)sqrt(n)) / ||vec||
 *             (torch.bucketize, right=False; a NaN x_i -- an all-zero vec -- lands in the last bin)
 *   packed  = bit planes of the bins, uint32 [n / 32 * nbits]
 *   result  = float32 [4] on the device: sum of squares, <centroids[bin], vec>,
 *             scale = ||vec||^2 / <centroids[bin], vec>, ||vec||
 * Sums are accumulated in double in a fixed order (4096-element tiles, 256
 * partial sums per tile -- of elements t + 256 k for the sum of squares, of
 * elements 16 t + k for the dot product, k ascending -- then halving trees), so
 * the result is independent of the launch shape; torch's own reduction order is
 * not specified, hence `scale` agrees with the reference to rounding error, not
 * bit for bit. */
int dq_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids,
                     int nbits, uint32_t *packed, float *result, double *work,
                     int64_t work_doubles, int device, dq_stream_t stream);

/* No counterpart in the reference.  dq_eden_quantize for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same launches and the same results, with
 * the per-tile partial sums in a static device array inside the library
 * (512 KiB per GPU, held until the process ends) instead of a caller's `work`.
 * Neither this call nor anything it runs allocates or frees memory.  The
 * array's device address is looked up once per GPU by the first call of any
 * function of this library on that GPU; under stream capture, make one such
 * call (any, e.g. this one as a warm-up) before the capture begins.
 * n is limited to dq_eden_quantize_static_max_n() = 2^28 elements; a larger n
 * is refused with DQ_ERR_SIZE.  All calls on one GPU share the array: calls
 * that may overlap on one GPU (two streams, two threads) race -- serialise them
 * or use dq_eden_quantize with separate work buffers. */
int64_t dq_eden_quantize_static_max_n(void);
int dq_eden_quantize_static(const float *vec, int64_t n, const float *boundaries,
                            const float *centroids, int nbits, uint32_t *packed, float *result,
                            int device, dq_stream_t stream);

/* srrcomp.py:343-345: out_i = centroids[bin_i] from the bit planes.  out must be
 * 16-byte aligned. */
int dq_eden_dequantize(const uint32_t *packed, int64_t n, const float *centroids, int nbits,
                       float *out, int device, dq_stream_t stream);

/* thc_hooks.py:161-166: level = floor(x) + (uniform < x - floor(x)) with
 * x = clamp((rotated - *lo) / *delta, 0, levels - 1), stored as bfloat16.
 * lo, delta: device scalars (they derive from the all-reduced norm,
 * thc_hooks.py:143-147).  uniform: float32 [n] in [0, 1) -- the caller draws it
 * (torch's bernoulli_ stream cannot be reproduced outside torch). */
int dq_thc_quantize(const float *rotated, const float *uniform, void *levels_bf16, int64_t n,
                    const float *lo, const float *delta, int levels, int device,
                    dq_stream_t stream);

/* srrcomp.py:343-354 in one call per rotation: dq_eden_dequantize folded into
 * the first pass of the inverse transform of dq_rht_blocked (sign, sign_packed,
 * block, scale as there; block >= 16), so that the dequantised vector never
 * reaches memory; out (fp32 [n]) receives the rotated vector.  post_scale (a
 * float32 on the device, e.g. result + 2 of dq_eden_quantize; may be NULL)
 * multiplies every element last, which is the reference's `scale * vec`.
 * Same bits as dq_eden_dequantize, dq_rht_blocked(inverse) and the product. */
int dq_eden_dequantize_irht(const uint32_t *packed, int64_t n, const float *centroids, int nbits,
                            const void *sign, int sign_packed, float *out, int64_t block,
                            float scale, const float *post_scale, int device,
                            dq_stream_t stream);

/* thc_hooks.py:176-178: out = float(levels) * *step + *lo (two roundings). */
int dq_thc_dequantize(const void *levels_bf16, float *out, int64_t n, const float *step,
                      const float *lo, int device, dq_stream_t stream);

/* thc_hooks.py:95-100 + :161-166 in one call: the forward transform of
 * dq_rht_blocked (sign flip, FWHT per block of `block` = 2^k, scale) whose last
 * pass stores dq_thc_quantize's levels instead of the rotated values.  work
 * (fp32 [n]) is the vector on entry and holds intermediate values on return
 * (the reference's work buffer is scratch as well, thc_hooks.py:152-158). */
int dq_thc_rht_quantize(float *work, const void *sign, int sign_packed, const float *uniform,
                        void *levels_bf16, int64_t n, int64_t block, float scale, const float *lo,
                        const float *delta, int levels, int device, dq_stream_t stream);

/* thc_hooks.py:176-181: dq_thc_dequantize folded into the first pass of the
 * inverse transform of dq_rht_blocked; the result lands in out (fp32 [n]). */
int dq_thc_dequantize_irht(const void *levels_bf16, const void *sign, int sign_packed, float *out,
                           int64_t n, int64_t block, float scale, const float *step,
                           const float *lo, int device, dq_stream_t stream);

/* ---- superchunk mean-centring ---------------------------------------- */

/* csrc/cuda_hadamard.h:23-24 (superchunk_mean_center_with_cuda).  residual
 * [>= 256*ceil(n/256)] (padded tail zero-filled), stats bf16
 * [>= 2*ceil(n/256)] interleaved (mean, sum of squares).  dtype F16 or BF16
 * (F32 accepted as an extension). */
int dq_superchunk_mean_center(const void *src, void *residual, void *stats, int64_t n,
                              int world_size, int superchunk_size, int dtype, int device,
                              dq_stream_t stream);
/* csrc/cuda_hadamard.h:25-26 (superchunk_add_mean_copy_with_cuda) */
int dq_superchunk_add_mean_copy(const void *residual, void *dst, const void *stats, int64_t n,
                                int superchunk_size, int dtype, int device, dq_stream_t stream);

/* ---- Walsh-Hadamard --------------------------------------------------- */

/* csrc/cuda_hadamard.h:14 (HadamardWithCuda): in-place unnormalised FWHT of
 * n = 2^k floats; depth is accepted and ignored as in the reference. */
int dq_hadamard(float *vec, int64_t n, int device, dq_stream_t stream, int depth);
/* Extension (no reference entry point; fuses thc_hooks.py:95-107 /
 * srrcomp.py:317-319): per block of `block` = 2^k floats, in place,
 *   forward: y = FWHT(sign .* x) * scale,   inverse: y = sign .* (FWHT(x) * scale).
 * sign: fp32 [n] of +-1 values, or (sign_packed != 0) the bit vector written by
 * dq_pack_signs -- 1/32 of the traffic, same result; NULL means all +1.
 * n must be a multiple of block.  dq_thc_rht_quantize / dq_thc_dequantize_irht
 * take sign the same way. */
int dq_rht_blocked(float *vec, const void *sign, int sign_packed, int64_t n, int64_t block,
                   float scale, int inverse, int device, dq_stream_t stream);
/* Extension: dq_rht_blocked (forward) followed by dq_scaling_compress of the
 * rotated vector, without the rotated vector ever reaching memory -- a
 * workgroup keeps whole transform blocks in LDS and quantises them there.  src
 * (fp32 [n]) is not modified; dst receives the hierarchical chunk-16 records
 * (strategy 2 or 3, nbits 2..8), byte for byte those of the two calls.
 * block = 2^k <= 32768; n a multiple of block and of 256.  sign: NULL, fp32
 * +-1 values [n] (sign_packed = 0), or one bit per element as written by
 * dq_pack_signs (sign_packed = 1: 4 bytes less traffic per element).
 * rand_pool: fp32 or bf16 [n] (rand_dtype DQ_F32 / DQ_BF16), or NULL for the
 * in-kernel Philox stream of dq_scaling_compress_philox keyed by (seed, step,
 * chunk). */
int dq_rht_scaling_compress(const float *src, const void *sign, int sign_packed, uint8_t *dst,
                            const void *rand_pool, int rand_dtype, int64_t n, int64_t block,
                            float scale, int nbits, int device, int strategy, uint64_t seed,
                            uint64_t step, dq_stream_t stream);
/* Measurement variant, no counterpart in the reference: dq_rht_scaling_compress
 * for 4-bit AEE codes with the in-kernel rounding stream, the transform's first
 * four stages (H16 on 16 consecutive elements) computed as a product with the
 * +-1 matrix on the matrix cores (v_mfma_f32_16x16x4_f32) instead of add /
 * subtract butterflies.  A product sums in another order than the butterflies,
 * so the rotated values agree with dq_rht_blocked to rounding error (1e-5
 * relative, the reference's tolerance for its transform) and a small share of
 * the codes differ by one step; it is also slower (16 multiply-adds per element
 * on the matrix pipe against 4 additions).  Kept to answer that question with a
 * number; use dq_rht_scaling_compress.  block 16 .. 16384, 16-byte aligned
 * buffers, n a multiple of the kernel's tile. */
int dq_rht_scaling_compress_mfma16(const float *src, const void *sign, int sign_packed, uint8_t *dst,
                                   int64_t n, int64_t block, float scale, int device,
                                   uint64_t seed, uint64_t step, dq_stream_t stream);
/* the way back: dq_scaling_decompress into fp32 followed by dq_rht_blocked
 * (inverse), the decoded vector staying in LDS. */
int dq_scaling_decompress_irht(const uint8_t *src, const void *sign, int sign_packed, float *dst,
                               int64_t n, int64_t block, float scale, int nbits, int device,
                               int strategy, dq_stream_t stream);
/* bits: uint32 [ceil(n / 32)]; bit e % 32 of word e / 32 is set where sign[e] < 0 */
int dq_pack_signs(const float *sign, uint32_t *bits, int64_t n, int device, dq_stream_t stream);
/* srrcomp.py:61-106 (SRRCompUtils.randDiag, torchRNG=False) computed on the
 * device: out[size] of +-1.0f. */
int dq_rand_diag(float *out, int64_t size, int64_t seed, int device, dq_stream_t stream);
/* the same diagonal written as the bit vector dq_pack_signs would make of it
 * (uint32 [size / 32], bit set where the value is -1), without the float vector:
 * size a positive multiple of 256. */
int dq_rand_diag_bits(uint32_t *bits, int64_t size, int64_t seed, int device, dq_stream_t stream);

/* ---- EDEN bit-plane packing ------------------------------------------ */

/* csrc/cuda_packing.h:10 (BinsToBits).  arr[p*(nbins/32) + w] bit t = bit p of
 * bins[32*w + t]; nbins % 32 == 0; narr == nbins/32*nbits.  Unlike the
 * reference launch (cuda_packing.cu:58-65) every bin is processed, also when
 * nbins is not a multiple of 1024, and the caller's stream is honoured. */
int dq_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int64_t narr, int nbits,
                    int device, dq_stream_t stream);
/* csrc/cuda_packing.h:11 (BitsToBins); bins must be 16-byte aligned */
int dq_bits_to_bins(int32_t *bins, int64_t nbins, const uint32_t *arr, int64_t narr, int nbits,
                    int device, dq_stream_t stream);

/* ---- THC-style stochastic rounding ------------------------------------ */

/* csrc/cuda_hadamard.h:16 (quantization_with_cuda): in place
 *   t = clamp(v / div_factor, +-tensor_max); v = floor(t) + (u < t - floor(t)).
 * The reference draws u from curand states it never initialises
 * (cuda_hadamard.cu:669-686); here u is a counter-based Philox4x32-10 uniform
 * keyed by (seed, element index). */
int dq_quantization(float *vec, int64_t n, int device, float div_factor, float tensor_max,
                    uint64_t seed, dq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
