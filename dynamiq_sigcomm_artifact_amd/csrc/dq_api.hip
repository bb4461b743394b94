// C ABI of libdynamiq_eden.so: argument validation, MEE table, kernel dispatch.
// Declarations and the reference entry point each function replaces are in
// include/dynamiq_eden.h.
#include <math.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <string>

#include "dq_device.cuh"
#include "dq_launch.h"

namespace {

thread_local std::string g_last_error;

const char *status_text(int s)
{
    switch (s) {
    case DQ_OK: return "ok";
    case DQ_ERR_N: return "n must be positive";
    case DQ_ERR_NBITS: return "nbits must be one of {2, 4, 8}";
    case DQ_ERR_STRATEGY: return "strategy must be 0 (AEE), 1 (MEE), 2 (hierarchical AEE), or 3 (hierarchical MEE)";
    case DQ_ERR_CHUNK_RANGE: return "chunk_size must be in [1, 32]";
    case DQ_ERR_CHUNK_POW2: return "chunk_size must be a power of two";
    case DQ_ERR_CHUNK_BITS: return "chunk_size * nbits must be divisible by 8";
    case DQ_ERR_N_CHUNK: return "n must be a multiple of chunk_size";
    case DQ_ERR_N_SUPER: return "hierarchical mode requires n to contain a whole number of 16-chunk superchunks";
    case DQ_ERR_DTYPE: return "unsupported element dtype";
    case DQ_ERR_NULL: return "null pointer argument";
    case DQ_ERR_SUPERCHUNK_SIZE: return "superchunk_size must be 256";
    case DQ_ERR_WORLD_SIZE: return "world_size must be positive";
    case DQ_ERR_POW2: return "input size must be a power of 2";
    case DQ_ERR_SIZE: return "size mismatch";
    case DQ_ERR_DEVICE: return "could not select the HIP device";
    case DQ_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
    }
}

int fail(int status, const char *detail = nullptr)
{
    g_last_error = status_text(status);
    if (detail) {
        g_last_error += ": ";
        g_last_error += detail;
    }
    return status;
}

int ok()
{
    g_last_error.clear();
    return DQ_OK;
}

int finish(hipError_t e)
{
    if (e != hipSuccess) return fail(DQ_ERR_LAUNCH, hipGetErrorString(e));
    return ok();
}

int select_device(int device)
{
    int cur = -1;
    if (!(hipGetDevice(&cur) == hipSuccess && cur == device) && hipSetDevice(device) != hipSuccess) return fail(DQ_ERR_DEVICE);
    // the first call on a device also resolves the address of the static scratch array of dq_eden_quantize_static,
    // so that that entry point itself never has to (it may run under stream capture); a failure here is reported by
    // that entry point, not by the caller at hand
    static std::atomic<uint64_t> prepared{0};
    if (device >= 0 && device < 64 && !(prepared.load(std::memory_order_acquire) >> device & 1)) {
        if (dq::eden_static_prepare(device) != hipSuccess) (void)hipGetLastError();
        prepared.fetch_or((uint64_t)1 << device, std::memory_order_release);
    }
    return DQ_OK;
}

// ---- MEE lookup tables (host, built once) -----------------------------------------

// binary32 -> binary16 bits, round to nearest even (host side)
uint16_t host_f32_to_f16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) {
        float mag;
        memcpy(&mag, &a, 4);
        return (uint16_t)(sign | (uint16_t)nearbyintf(mag * 16777216.0f));
    }
    const uint32_t rounded = a + 0xfffu + ((a >> 13) & 1u);
    return (uint16_t)(sign | (uint16_t)((rounded - 0x38000000u) >> 13));
}

float host_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

struct Lut {
    uint16_t table[9][256];
    uint16_t params[9][4];
    dq::MeeParams mp[9];
};

Lut g_lut;
std::once_flag g_lut_once;

void build_lut()
{
    // csrc/cuda_hadamard.cu:873-899: fp32 host arithmetic, results kept as binary16
    static const float epses[9] = {0.0f, 0.23f, 0.23f, 0.18f, 0.18f, 0.18f, 0.1f, 0.1f, 0.1f};
    memset(&g_lut, 0, sizeof(g_lut));
    for (int b = 1; b < 9; b++) {
        const float eps = epses[b];
        volatile float two_eps2 = 2.0f * eps * eps;
        volatile float base = 1.0f + two_eps2;
        volatile float one_plus_eps2 = 1.0f + eps * eps;
        g_lut.params[b][0] = host_f32_to_f16(base);
        g_lut.params[b][1] = host_f32_to_f16(one_plus_eps2 / two_eps2);
        g_lut.params[b][3] = host_f32_to_f16(log2f(base));
        const int anchor = (1 << (b - 1)) - 1;
        volatile float pw = 1.0f;
        for (int j = 1; j <= anchor; j++) {
            pw = pw * base;
            volatile float num = pw - 1.0f;
            volatile float quo = num / two_eps2;
            volatile float rep = quo * one_plus_eps2;
            g_lut.table[b][anchor + j] = host_f32_to_f16(rep);
            g_lut.table[b][anchor - j] = host_f32_to_f16(-rep);
        }
        g_lut.params[b][2] = g_lut.table[b][anchor * 2];
        dq::MeeParams &m = g_lut.mp[b];
        m.c = host_f16_to_f32(g_lut.params[b][1]);
        m.cmm = host_f16_to_f32(g_lut.params[b][2]);
        m.l2b = host_f16_to_f32(g_lut.params[b][3]);
        m.pad = 0;
        memcpy(m.table, g_lut.table[b], sizeof(m.table));
    }
}

const dq::MeeParams &mee_params(int nbits)
{
    std::call_once(g_lut_once, build_lut);
    return g_lut.mp[nbits];
}

int check_common(int64_t n, int nbits, int chunk_size, int strategy, int strict)
{
    if (!(n > 0)) return DQ_ERR_N;
    if (strict) {
        if (!(nbits == 2 || nbits == 4 || nbits == 8)) return DQ_ERR_NBITS;
    } else if (nbits < 2 || nbits > 8) {
        return DQ_ERR_NBITS;
    }
    if (strategy < 0 || strategy > 3) return DQ_ERR_STRATEGY;
    if (!(chunk_size > 0 && chunk_size <= 32)) return DQ_ERR_CHUNK_RANGE;
    if ((chunk_size & (chunk_size - 1)) != 0) return DQ_ERR_CHUNK_POW2;
    if ((chunk_size * nbits) % 8 != 0) return DQ_ERR_CHUNK_BITS;
    if (n % chunk_size != 0) return DQ_ERR_N_CHUNK;
    if (strategy >= 2 && (n / chunk_size) % 16 != 0) return DQ_ERR_N_SUPER;
    return DQ_OK;
}

inline bool dtype_ok(int dtype) { return dtype == DQ_F16 || dtype == DQ_BF16 || dtype == DQ_F32; }
// compress-side dtype: the DQ_RAND_BF16 flag is only meaningful with DQ_F32 elements
inline bool dtype_rand_ok(int dtype)
{
    if (dtype & ~(0xf | DQ_RAND_BF16)) return false;
    if ((dtype & DQ_RAND_BF16) && (dtype & 0xf) != DQ_F32) return false;
    return dtype_ok(dtype & 0xf);
}

// the production shape: one fused-capable vectorised kernel family
inline bool hier16_shape(int dtype, int chunk_size, int strategy)
{
    return (dtype == DQ_BF16 || dtype == DQ_F32) && chunk_size == 16 && strategy >= 2;
}
// every other chunk-16 shape: binary16 elements, flat strategies
inline bool tile16_shape(int dtype, int chunk_size, int strategy)
{
    return chunk_size == 16 && !hier16_shape(dtype, chunk_size, strategy);
}

} // namespace

extern "C" {

const char *dq_status_string(int status) { return status_text(status); }
const char *dq_last_error(void) { return g_last_error.c_str(); }
const char *dq_version(void) { return "dynamiq_eden 0.1 gfx950"; }

int64_t dq_scaling_required_bytes(int64_t n, int nbits, int chunk_size, int strategy)
{
    if (chunk_size <= 0) return 0;
    const int64_t chunks = n / chunk_size;
    const int64_t packed = ((int64_t)chunk_size * nbits) >> 3;
    if (strategy >= 2) return (chunks / 16) * (16 * (packed + 1) + 2);
    return chunks * (packed + 2);
}

int dq_scaling_check_common(int64_t n, int nbits, int chunk_size, int strategy, int strict)
{
    const int rc = check_common(n, nbits, chunk_size, strategy, strict);
    return rc ? fail(rc) : ok();
}

int dq_init_lookup_table(void)
{
    (void)mee_params(2);
    return ok();
}

int dq_mee_lookup_table(int nbits, uint16_t table[256], uint16_t params[4])
{
    if (nbits < 1 || nbits > 8) return fail(DQ_ERR_NBITS);
    if (!table || !params) return fail(DQ_ERR_NULL);
    (void)mee_params(nbits);
    memcpy(table, g_lut.table[nbits], 256 * sizeof(uint16_t));
    memcpy(params, g_lut.params[nbits], 4 * sizeof(uint16_t));
    return ok();
}

int dq_scaling_compress(const void *src, uint8_t *dst, const void *rand_pool, int64_t n, int nbits, int chunk_size,
                        int dtype, int device, int strategy, dq_stream_t stream)
{
    int rc = check_common(n, nbits, chunk_size, strategy, 0);
    if (rc) return fail(rc);
    if (!dtype_rand_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!src || !dst || !rand_pool) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dq::MeeParams &mp = mee_params(nbits);
    if (hier16_shape(dtype & 0xf, chunk_size, strategy))
        return finish(dq::launch_hier16_compress(src, dst, rand_pool, n, nbits, dtype, strategy == 3, mp, s));
    if (tile16_shape(dtype & 0xf, chunk_size, strategy))
        return finish(dq::launch_tile16_compress(src, dst, rand_pool, n, nbits, dtype, strategy, mp, s));
    return finish(dq::launch_generic_compress(src, dst, rand_pool, n, nbits, chunk_size, dtype, strategy, mp, s));
}

int dq_scaling_decompress(const uint8_t *src, void *dst, int64_t n, int nbits, int chunk_size, int dtype, int device,
                          int strategy, dq_stream_t stream, int add_original)
{
    int rc = check_common(n, nbits, chunk_size, strategy, 0);
    if (rc) return fail(rc);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dq::MeeParams &mp = mee_params(nbits);
    if (hier16_shape(dtype, chunk_size, strategy))
        return finish(dq::launch_hier16_decompress(src, dst, n, nbits, dtype, strategy == 3, mp, add_original, s));
    if (tile16_shape(dtype, chunk_size, strategy))
        return finish(dq::launch_tile16_decompress(src, dst, n, nbits, dtype, strategy, mp, add_original, s));
    return finish(dq::launch_generic_decompress(src, dst, n, nbits, chunk_size, dtype, strategy, mp, add_original, s));
}

int dq_scaling_dec_comp(const uint8_t *recv, void *inp, uint8_t *send, const void *rand_pool, int64_t n, int nbits,
                        int chunk_size, int dtype, int device, int strategy, dq_stream_t stream)
{
    int rc = check_common(n, nbits, chunk_size, strategy, 0);
    if (rc) return fail(rc);
    if (!dtype_rand_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!recv || !inp || !send || !rand_pool) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dq::MeeParams &mp = mee_params(nbits);
    if (hier16_shape(dtype & 0xf, chunk_size, strategy))
        return finish(dq::launch_hier16_dec_comp(recv, inp, send, rand_pool, n, nbits, dtype, strategy == 3, mp, s));
    // every other combination: decode into inp, then compress inp (two kernels, inp is modified)
    if (tile16_shape(dtype & 0xf, chunk_size, strategy)) {
        hipError_t e = dq::launch_tile16_decompress(recv, inp, n, nbits, dtype & 0xf, strategy, mp, 1, s);
        if (e != hipSuccess) return finish(e);
        return finish(dq::launch_tile16_compress(inp, send, rand_pool, n, nbits, dtype, strategy, mp, s));
    }
    hipError_t e = dq::launch_generic_decompress(recv, inp, n, nbits, chunk_size, dtype & 0xf, strategy, mp, 1, s);
    if (e != hipSuccess) return finish(e);
    return finish(dq::launch_generic_compress(inp, send, rand_pool, n, nbits, chunk_size, dtype, strategy, mp, s));
}

int64_t dq_group_plan_work_ints(int64_t nsc) { return nsc > 0 ? dq::group_plan_work_ints(nsc) : 4; }

int dq_group_plan(const int64_t *qbits, int64_t nsc, int32_t *order, int32_t *work, int64_t work_ints, int device,
                  dq_stream_t stream)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return fail(DQ_ERR_N, "nsc must be in [1, 2^31)");
    if (!qbits || !order || !work) return fail(DQ_ERR_NULL);
    if (work_ints < dq::group_plan_work_ints(nsc)) return fail(DQ_ERR_SIZE, "work buffer is too small");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_group_plan(qbits, nsc, order, work, static_cast<hipStream_t>(stream)));
}

int dq_group_plan_stats(const void *stats, double u, int64_t nsc, int64_t *qbits_out, int32_t *order, int32_t *work,
                        int64_t work_ints, int device, dq_stream_t stream)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return fail(DQ_ERR_N, "nsc must be in [1, 2^31)");
    if (!stats || !order || !work) return fail(DQ_ERR_NULL);
    if (work_ints < dq::group_plan_work_ints(nsc)) return fail(DQ_ERR_SIZE, "work buffer is too small");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_group_plan_stats(stats, (float)u, nullptr, nsc, qbits_out, order, work, nullptr, static_cast<hipStream_t>(stream)));
}

// up to here the one-launch counting sort in LDS, beyond it the radix sort in the caller's workspace
static constexpr int64_t kSortedPlanOneLaunch = 65535;

int64_t dq_group_plan_sorted_work_ints(int64_t nsc)
{
    return nsc > kSortedPlanOneLaunch ? dq::group_plan_sorted_large_work_ints(nsc) : 4;
}

int dq_group_plan_sorted(const void *stats, int64_t nsc, int64_t top_count, int64_t bottom_count, int64_t *qbits_out,
                         int32_t *order, int32_t *work, int64_t work_ints, int device, dq_stream_t stream)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return fail(DQ_ERR_N, "nsc must be in [1, 2^31)");
    if (top_count < 0 || bottom_count < 0 || top_count + bottom_count > nsc)
        return fail(DQ_ERR_SIZE, "top_count and bottom_count must be non-negative and sum to at most nsc");
    if (!stats || !order || !work) return fail(DQ_ERR_NULL);
    if (reinterpret_cast<uintptr_t>(stats) & 3) return fail(DQ_ERR_SIZE, "stats must be 4-byte aligned");
    if (work_ints < dq_group_plan_sorted_work_ints(nsc))
        return fail(DQ_ERR_SIZE, "work buffer is too small (dq_group_plan_sorted_work_ints)");
    int rc;
    if ((rc = select_device(device))) return rc;
    if (nsc > kSortedPlanOneLaunch)
        return finish(dq::launch_group_plan_sorted_large(stats, nsc, top_count, bottom_count, qbits_out, order, work, work_ints,
                                                         static_cast<hipStream_t>(stream)));
    return finish(dq::launch_group_plan_sorted(stats, nsc, top_count, bottom_count, qbits_out, order, work,
                                               static_cast<hipStream_t>(stream)));
}

int dq_group_plan_stats_dev_u(const void *stats, const double *u_dev, int64_t nsc, int64_t *qbits_out, int32_t *order,
                              int32_t *work, int64_t work_ints, uint32_t *hist, int64_t hist_ints, int device,
                              dq_stream_t stream)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return fail(DQ_ERR_N, "nsc must be in [1, 2^31)");
    if (!stats || !u_dev || !order || !work) return fail(DQ_ERR_NULL);
    if (work_ints < dq::group_plan_work_ints(nsc)) return fail(DQ_ERR_SIZE, "work buffer is too small");
    if (hist && hist_ints < dq::bitrate_hist_ints()) return fail(DQ_ERR_SIZE, "hist buffer is too small");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_group_plan_stats(stats, 0.0f, u_dev, nsc, qbits_out, order, work, hist, static_cast<hipStream_t>(stream)));
}

int64_t dq_bitrate_hist_ints(void) { return dq::bitrate_hist_ints(); }

int dq_norm_histogram(const void *stats, int64_t nsc, uint32_t *hist, int64_t hist_ints, int device, dq_stream_t stream)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return fail(DQ_ERR_N, "nsc must be in [1, 2^31)");
    if (!stats || !hist) return fail(DQ_ERR_NULL);
    if (hist_ints < dq::bitrate_hist_ints()) return fail(DQ_ERR_SIZE, "hist buffer is too small");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_norm_histogram(stats, nsc, hist, static_cast<hipStream_t>(stream)));
}

int dq_bitrate_search(uint32_t *hist, int64_t hist_ints, int mode, double prev_u, const double *prev_u_dev,
                      double target_avg_bits, double *result, int device, dq_stream_t stream)
{
    if (mode != 0 && mode != 1) return fail(DQ_ERR_SIZE, "mode must be 0 (bisection) or 1 (correction from prev_u)");
    if (!hist || !result) return fail(DQ_ERR_NULL);
    if (hist_ints < dq::bitrate_hist_ints()) return fail(DQ_ERR_SIZE, "hist buffer is too small");
    if (prev_u != prev_u || target_avg_bits != target_avg_bits) return fail(DQ_ERR_SIZE, "prev_u and target_avg_bits must be numbers");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_bitrate_search(hist, mode, prev_u, prev_u_dev, target_avg_bits, result, static_cast<hipStream_t>(stream)));
}

static int check_rows(int64_t nrows, int nbits, int dtype, int strategy, bool rand)
{
    if (!(nrows > 0) || nrows > (int64_t)0x7fffffff) return DQ_ERR_N;
    if (nbits < 2 || nbits > 8) return DQ_ERR_NBITS;
    if (strategy != 2 && strategy != 3) return DQ_ERR_STRATEGY;
    if (rand ? !dtype_rand_ok(dtype) : !dtype_ok(dtype)) return DQ_ERR_DTYPE;
    if ((dtype & 0xf) == DQ_F16) return DQ_ERR_DTYPE;
    return DQ_OK;
}

int dq_scaling_compress_rows(const void *src, const int32_t *rows, uint8_t *dst, const void *rand_pool, int64_t nrows,
                             int nbits, int dtype, int device, int strategy, dq_stream_t stream)
{
    int rc = check_rows(nrows, nbits, dtype, strategy, true);
    if (rc) return fail(rc);
    if (!src || !dst || !rand_pool) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_hier16_compress_rows(src, nullptr, rows, dst, rand_pool, nrows, nbits, dtype, strategy == 3,
                                                  mee_params(nbits), static_cast<hipStream_t>(stream)));
}

int dq_scaling_dec_comp_rows(const uint8_t *recv, const void *inp, const int32_t *rows, uint8_t *send,
                             const void *rand_pool, int64_t nrows, int nbits, int dtype, int device, int strategy,
                             dq_stream_t stream)
{
    int rc = check_rows(nrows, nbits, dtype, strategy, true);
    if (rc) return fail(rc);
    if (!recv || !inp || !send || !rand_pool) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_hier16_compress_rows(inp, recv, rows, send, rand_pool, nrows, nbits, dtype, strategy == 3,
                                                  mee_params(nbits), static_cast<hipStream_t>(stream)));
}

int dq_scaling_decompress_rows(const uint8_t *src, void *dst, const int32_t *rows, const void *stats, int64_t n_limit,
                               int64_t nrows, int nbits, int dtype, int device, int strategy, dq_stream_t stream,
                               int add_original)
{
    int rc = check_rows(nrows, nbits, dtype, strategy, false);
    if (rc) return fail(rc);
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if (!(n_limit > 0)) return fail(DQ_ERR_N, "n_limit");
    if (add_original && stats) return fail(DQ_ERR_SIZE, "stats cannot be combined with add_original");
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_hier16_decompress_rows(src, dst, rows, stats, n_limit, nrows, nbits, dtype, strategy == 3,
                                                    mee_params(nbits), add_original, static_cast<hipStream_t>(stream)));
}

static int check_mixed(int64_t nsc, int ring_chunk, int ring_world, int dtype, int strategy, bool rand)
{
    if (!(nsc > 0) || nsc > (int64_t)0x7fffffff) return DQ_ERR_N;
    if (!(ring_world > 0) || ring_chunk < 0 || ring_chunk >= ring_world) return DQ_ERR_WORLD_SIZE;
    if (strategy != 2 && strategy != 3) return DQ_ERR_STRATEGY;
    if (rand ? !dtype_rand_ok(dtype) : !dtype_ok(dtype)) return DQ_ERR_DTYPE;
    if ((dtype & 0xf) == DQ_F16) return DQ_ERR_DTYPE;
    return DQ_OK;
}

int64_t dq_mixed_required_bytes(int64_t nsc, int ring_world)
{
    return (nsc > 0 && ring_world > 0) ? dq::mixed_stream_bytes(nsc, ring_world) : 0;
}

int dq_mixed_compress(const void *src, const float *center_mean, int center_world, int64_t n, const int32_t *order,
                      const int32_t *counts, int ring_chunk, int ring_world, const uint8_t *recv, uint8_t *dst,
                      const void *rand_pool, uint64_t seed, uint64_t step, int64_t nsc, int dtype, int device, int strategy,
                      dq_stream_t stream)
{
    int rc = check_mixed(nsc, ring_chunk, ring_world, dtype, strategy, rand_pool != nullptr);
    if (rc) return fail(rc);
    if (!src || !order || !counts || !dst) return fail(DQ_ERR_NULL);
    if (center_mean) {
        if (!(center_world > 0)) return fail(DQ_ERR_WORLD_SIZE);
        if (!(n > 0) || (n + 255) / 256 > nsc) return fail(DQ_ERR_N, "n must lie in [1, 256 * nsc]");
    }
    if ((rc = select_device(device))) return rc;
    const dq::MeeParams mp[3] = {mee_params(8), mee_params(4), mee_params(2)};
    const dq::RandKey key{seed, step};
    return finish(dq::launch_mixed_compress(src, center_mean, center_mean ? center_world : 1, n, order, counts, ring_chunk,
                                            ring_world, recv, dst, rand_pool, rand_pool ? nullptr : &key, nsc, dtype,
                                            strategy == 3, mp, static_cast<hipStream_t>(stream)));
}

int dq_mixed_decompress(const uint8_t *src, void *dst, const int32_t *order, const int32_t *counts, int ring_chunk,
                        int ring_world, const void *stats, int64_t n_limit, int64_t nsc, int dtype, int device,
                        int strategy, dq_stream_t stream)
{
    int rc = check_mixed(nsc, ring_chunk, ring_world, dtype, strategy, false);
    if (rc) return fail(rc);
    if (!src || !dst || !order || !counts) return fail(DQ_ERR_NULL);
    if (!(n_limit > 0)) return fail(DQ_ERR_N, "n_limit");
    if ((rc = select_device(device))) return rc;
    const dq::MeeParams mp[3] = {mee_params(8), mee_params(4), mee_params(2)};
    return finish(dq::launch_mixed_decompress(src, dst, order, counts, ring_chunk, ring_world, stats, n_limit, nsc, dtype,
                                              strategy == 3, mp, static_cast<hipStream_t>(stream)));
}

int dq_streams_overlap(dq_stream_t a, dq_stream_t b, int device, int *overlap)
{
    if (!overlap) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::probe_streams_overlap(static_cast<hipStream_t>(a), static_cast<hipStream_t>(b), overlap));
}

int dq_stream_order_after(dq_stream_t stream, dq_stream_t after, int device)
{
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::stream_order_after(static_cast<hipStream_t>(stream), static_cast<hipStream_t>(after), device));
}

int dq_tile_io_floor(int direction, void *a, int a_bytes_per_tile, const void *b, int b_bytes_per_tile, void *run, int run_bytes_per_tile,
                     int64_t tiles, int device, dq_stream_t stream)
{
    if (direction != 0 && direction != 1) return fail(DQ_ERR_SIZE, "direction must be 0 (encoder shape) or 1 (decoder shape)");
    if (!dq::tile_io_floor_shape_ok(a_bytes_per_tile, b_bytes_per_tile, run_bytes_per_tile))
        return fail(DQ_ERR_SIZE, "a_bytes_per_tile must be 2048 or 4096, b_bytes_per_tile 0, 2048 or 4096, run_bytes_per_tile a multiple of 8 up to 8192");
    if (!(tiles > 0) || tiles > 0x7fffffff) return fail(DQ_ERR_N);
    if (!a || !run || (b_bytes_per_tile > 0 && !b)) return fail(DQ_ERR_NULL);
    if ((reinterpret_cast<uintptr_t>(a) & 15) || (reinterpret_cast<uintptr_t>(b) & 15) || (reinterpret_cast<uintptr_t>(run) & 7))
        return fail(DQ_ERR_SIZE, "a and b must be 16-byte aligned, run 8-byte aligned");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_tile_io_floor(direction, a, a_bytes_per_tile, b, b_bytes_per_tile, run, run_bytes_per_tile, tiles,
                                           static_cast<hipStream_t>(stream)));
}

int dq_dynamic_bitrate_bucket(const dq_bucket_t *b, int stages, int device, dq_stream_t stream)
{
    if (!b) return fail(DQ_ERR_NULL);
    if (stages <= 0 || stages > 15) return fail(DQ_ERR_SIZE, "stages must be a combination of DQ_STAGE_*");
    if (!(b->n > 0)) return fail(DQ_ERR_N);
    const int64_t nsc = (b->n + 255) / 256;
    const bool s_stats = stages & DQ_STAGE_STATS, s_plan = stages & DQ_STAGE_PLAN, s_comp = stages & DQ_STAGE_COMPRESS,
               s_dec = stages & DQ_STAGE_DECOMPRESS;
    // everything is checked before the first launch
    int rc = check_mixed(nsc, b->ring_chunk, b->ring_world, b->dtype, b->strategy, false);
    if (rc) return fail(rc);
    if (!(b->center_world > 0)) return fail(DQ_ERR_WORLD_SIZE);
    const void *reduced = b->reduced_stats ? b->reduced_stats : b->stats;
    if (!b->src && (s_stats || s_comp)) return fail(DQ_ERR_NULL);
    if (s_stats && (!b->stats || !b->mean)) return fail(DQ_ERR_NULL);
    if (s_plan) {
        if (!reduced || !b->order || !b->work) return fail(DQ_ERR_NULL);
        if (b->work_ints < dq::group_plan_work_ints(nsc)) return fail(DQ_ERR_SIZE, "work buffer is too small");
        if (b->hist && !b->u_dev) return fail(DQ_ERR_SIZE, "hist is filled by the plan only when u is read from device memory");
        if (b->hist && b->hist_ints < dq::bitrate_hist_ints()) return fail(DQ_ERR_SIZE, "hist buffer is too small");
        if (!b->u_dev && b->u != b->u) return fail(DQ_ERR_SIZE, "u must be a number");
    }
    if (s_comp || s_dec) {
        if (!b->order || !b->work || !b->packed) return fail(DQ_ERR_NULL);
        if (b->packed_bytes < dq::mixed_stream_bytes(nsc, b->ring_world))
            return fail(DQ_ERR_SIZE, "packed buffer is too small (dq_mixed_required_bytes)");
    }
    if (s_comp && !b->mean) return fail(DQ_ERR_NULL);
    if (s_dec && (!b->out || !reduced)) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipSuccess;
    if (s_stats) e = dq::launch_mean_center(b->src, nullptr, b->stats, b->mean, b->n, b->center_world, b->dtype, s);
    if (e == hipSuccess && s_plan)
        e = dq::launch_group_plan_stats(reduced, (float)b->u, b->u_dev, nsc, nullptr, b->order, b->work, b->hist, s);
    if (e == hipSuccess && (s_comp || s_dec)) {
        const dq::MeeParams mp[3] = {mee_params(8), mee_params(4), mee_params(2)};
        const dq::RandKey key{b->seed, b->step};
        if (s_comp)
            e = dq::launch_mixed_compress(b->src, b->mean, b->center_world, b->n, b->order, b->work, b->ring_chunk, b->ring_world,
                                          b->recv, b->packed, nullptr, &key, nsc, b->dtype, b->strategy == 3, mp, s, b->step_dev);
        if (e == hipSuccess && s_dec)
            e = dq::launch_mixed_decompress(b->packed, b->out, b->order, b->work, b->ring_chunk, b->ring_world, reduced, b->n, nsc,
                                            b->dtype, b->strategy == 3, mp, s);
    }
    return finish(e);
}

int dq_scaling_compress_philox(const void *src, uint8_t *dst, int64_t n, int nbits, int chunk_size, int dtype, int device,
                               int strategy, uint64_t seed, uint64_t step, dq_stream_t stream)
{
    int rc = check_common(n, nbits, chunk_size, strategy, 0);
    if (rc) return fail(rc);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (chunk_size != 16) return fail(DQ_ERR_CHUNK_RANGE, "the in-kernel random stream is defined for chunk_size 16");
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dq::MeeParams &mp = mee_params(nbits);
    if (hier16_shape(dtype, chunk_size, strategy))
        return finish(dq::launch_hier16_compress_philox(src, nullptr, dst, n, nbits, dtype, strategy == 3, mp, seed, step, s));
    const dq::RandKey key{seed, step};
    return finish(dq::launch_tile16_compress(src, dst, nullptr, n, nbits, dtype, strategy, mp, s, &key));
}

int dq_scaling_dec_comp_philox(const uint8_t *recv, void *inp, uint8_t *send, int64_t n, int nbits, int chunk_size, int dtype,
                               int device, int strategy, uint64_t seed, uint64_t step, dq_stream_t stream)
{
    int rc = check_common(n, nbits, chunk_size, strategy, 0);
    if (rc) return fail(rc);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (chunk_size != 16) return fail(DQ_ERR_CHUNK_RANGE, "the in-kernel random stream is defined for chunk_size 16");
    if (!recv || !inp || !send) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dq::MeeParams &mp = mee_params(nbits);
    if (hier16_shape(dtype, chunk_size, strategy))
        return finish(dq::launch_hier16_compress_philox(inp, recv, send, n, nbits, dtype, strategy == 3, mp, seed, step, s));
    hipError_t e = dq::launch_tile16_decompress(recv, inp, n, nbits, dtype, strategy, mp, 1, s);
    if (e != hipSuccess) return finish(e);
    const dq::RandKey key{seed, step};
    return finish(dq::launch_tile16_compress(inp, send, nullptr, n, nbits, dtype, strategy, mp, s, &key));
}

int dq_philox_uniform(void *out, int64_t n, int dtype, int device, uint64_t seed, uint64_t step, dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!out) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_philox_uniform(out, n, dtype, seed, step, static_cast<hipStream_t>(stream)));
}

int dq_superchunk_mean_center(const void *src, void *residual, void *stats, int64_t n, int world_size,
                              int superchunk_size, int dtype, int device, dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!(world_size > 0)) return fail(DQ_ERR_WORLD_SIZE);
    if (superchunk_size != 256) return fail(DQ_ERR_SUPERCHUNK_SIZE);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!src || !residual || !stats) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_mean_center(src, residual, stats, nullptr, n, world_size, dtype, static_cast<hipStream_t>(stream)));
}

int dq_superchunk_stats(const void *src, void *stats, float *mean, int64_t n, int world_size, int dtype, int device,
                        dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!(world_size > 0)) return fail(DQ_ERR_WORLD_SIZE);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!src || !stats) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_mean_center(src, nullptr, stats, mean, n, world_size, dtype, static_cast<hipStream_t>(stream)));
}

int dq_superchunk_add_mean_copy(const void *residual, void *dst, const void *stats, int64_t n, int superchunk_size,
                                int dtype, int device, dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (superchunk_size != 256) return fail(DQ_ERR_SUPERCHUNK_SIZE);
    if (!dtype_ok(dtype)) return fail(DQ_ERR_DTYPE);
    if (!residual || !dst || !stats) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_add_mean_copy(residual, dst, stats, n, dtype, static_cast<hipStream_t>(stream)));
}

int dq_hadamard(float *vec, int64_t n, int device, dq_stream_t stream, int depth)
{
    (void)depth;
    if (!(n > 0) || (n & (n - 1)) != 0) return fail(DQ_ERR_POW2);
    if (!vec) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_hadamard(vec, n, static_cast<hipStream_t>(stream)));
}

int dq_rht_blocked(float *vec, const void *sign, int sign_packed, int64_t n, int64_t block, float scale, int inverse,
                   int device, dq_stream_t stream)
{
    if (!(block > 0) || (block & (block - 1)) != 0) return fail(DQ_ERR_POW2, "block");
    if (!(n > 0) || n % block != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of block");
    if (!vec) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_rht_blocked(vec, sign, sign_packed != 0, n, block, scale, inverse, static_cast<hipStream_t>(stream)));
}

static int check_rht_scaling(int64_t n, int64_t block, int nbits, int strategy)
{
    if (!(block > 0) || (block & (block - 1)) != 0) return fail(DQ_ERR_POW2, "block");
    if (block > 32768) return fail(DQ_ERR_SIZE, "block must not exceed 32768 (one workgroup holds a whole transform block)");
    if (!(n > 0) || n % block != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of block");
    if (n % 256 != 0) return fail(DQ_ERR_N_SUPER);
    if (nbits < 2 || nbits > 8) return fail(DQ_ERR_NBITS);
    if (strategy != 2 && strategy != 3) return fail(DQ_ERR_STRATEGY);
    return DQ_OK;
}

int dq_rht_scaling_compress(const float *src, const void *sign, int sign_packed, uint8_t *dst, const void *rand_pool, int rand_dtype,
                            int64_t n, int64_t block, float scale, int nbits, int device, int strategy, uint64_t seed,
                            uint64_t step, dq_stream_t stream)
{
    int rc = check_rht_scaling(n, block, nbits, strategy);
    if (rc) return rc;
    if (rand_pool && rand_dtype != DQ_F32 && rand_dtype != DQ_BF16) return fail(DQ_ERR_DTYPE);
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_rht_compress(src, sign, sign_packed ? 1 : 0, dst, rand_pool, rand_pool ? rand_dtype : 3, n, block, scale, nbits,
                                          strategy == 3, mee_params(nbits), seed, step, static_cast<hipStream_t>(stream)));
}

int dq_rht_scaling_compress_mfma16(const float *src, const void *sign, int sign_packed, uint8_t *dst, int64_t n, int64_t block,
                                   float scale, int device, uint64_t seed, uint64_t step, dq_stream_t stream)
{
    int rc = check_rht_scaling(n, block, 4, 2);
    if (rc) return rc;
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if (block < 16 || block > 16384) return fail(DQ_ERR_SIZE, "the matrix-core variant takes blocks of 16 .. 16384");
    if ((reinterpret_cast<uintptr_t>(src) & 15) || (sign && !sign_packed && (reinterpret_cast<uintptr_t>(sign) & 15)))
        return fail(DQ_ERR_SIZE, "the matrix-core variant needs 16-byte aligned vectors");
    if ((rc = select_device(device))) return rc;
    const hipError_t e = dq::launch_rht_compress_mfma16(src, sign, sign_packed ? 1 : 0, dst, n, block, scale, mee_params(4), seed, step,
                                                        static_cast<hipStream_t>(stream));
    if (e == hipErrorInvalidValue) return fail(DQ_ERR_SIZE, "the matrix-core variant needs n to be a multiple of its tile (8192 elements or the block)");
    return finish(e);
}

int dq_scaling_decompress_irht(const uint8_t *src, const void *sign, int sign_packed, float *dst, int64_t n, int64_t block, float scale,
                               int nbits, int device, int strategy, dq_stream_t stream)
{
    int rc = check_rht_scaling(n, block, nbits, strategy);
    if (rc) return rc;
    if (!src || !dst) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_irht_decompress(src, sign, sign_packed ? 1 : 0, dst, n, block, scale, nbits, strategy == 3, mee_params(nbits),
                                             static_cast<hipStream_t>(stream)));
}

int dq_pack_signs(const float *sign, uint32_t *bits, int64_t n, int device, dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!sign || !bits) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_pack_signs(sign, bits, n, static_cast<hipStream_t>(stream)));
}

int dq_rand_diag(float *out, int64_t size, int64_t seed, int device, dq_stream_t stream)
{
    if (!(size > 0)) return fail(DQ_ERR_N);
    if (!out) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_rand_diag(out, size, seed, static_cast<hipStream_t>(stream)));
}

int dq_rand_diag_bits(uint32_t *bits, int64_t size, int64_t seed, int device, dq_stream_t stream)
{
    if (!(size > 0) || size % 256 != 0) return fail(DQ_ERR_SIZE, "size must be a positive multiple of 256");
    if (!bits) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_rand_diag_bits(bits, size, seed, static_cast<hipStream_t>(stream)));
}

int dq_bins_to_bits(const int32_t *bins, int64_t nbins, uint32_t *arr, int64_t narr, int nbits, int device,
                    dq_stream_t stream)
{
    if (nbits < 1 || nbits > 32) return fail(DQ_ERR_NBITS, "nbits must be in [1, 32]");
    if (!(nbins > 0) || (nbins & 31) != 0) return fail(DQ_ERR_SIZE, "bins size must be a multiple of 32");
    if (narr != (nbins >> 5) * nbits) return fail(DQ_ERR_SIZE, "narr must equal nbins / 32 * nbits");
    if (!bins || !arr) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_bins_to_bits(bins, nbins, arr, nbits, static_cast<hipStream_t>(stream)));
}

int dq_bits_to_bins(int32_t *bins, int64_t nbins, const uint32_t *arr, int64_t narr, int nbits, int device,
                    dq_stream_t stream)
{
    if (nbits < 1 || nbits > 32) return fail(DQ_ERR_NBITS, "nbits must be in [1, 32]");
    if (!(nbins > 0) || (nbins & 31) != 0) return fail(DQ_ERR_SIZE, "bins size must be a multiple of 32");
    if (narr != (nbins >> 5) * nbits) return fail(DQ_ERR_SIZE, "narr must equal nbins / 32 * nbits");
    if (!bins || !arr) return fail(DQ_ERR_NULL);
    if (reinterpret_cast<uintptr_t>(bins) & 15) return fail(DQ_ERR_SIZE, "bins must be 16-byte aligned");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_bits_to_bins(bins, nbins, arr, nbits, static_cast<hipStream_t>(stream)));
}

int64_t dq_eden_work_doubles(int64_t n) { return n > 0 ? dq::eden_work_doubles(n) : 1; }

int dq_eden_quantize(const float *vec, int64_t n, const float *boundaries, const float *centroids, int nbits,
                     uint32_t *packed, float *result, double *work, int64_t work_doubles, int device, dq_stream_t stream)
{
    if (!(n > 0) || (n & 31) != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of 32");
    if (nbits < 1 || nbits > 8) return fail(DQ_ERR_NBITS, "nbits must be in [1, 8]");
    if (!vec || !boundaries || !centroids || !packed || !result || !work) return fail(DQ_ERR_NULL);
    if (work_doubles < dq::eden_work_doubles(n)) return fail(DQ_ERR_SIZE, "work buffer is too small");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_eden_quantize(vec, n, boundaries, centroids, nbits, packed, result, work,
                                           static_cast<hipStream_t>(stream)));
}

int64_t dq_eden_quantize_static_max_n(void) { return dq::eden_static_max_n(); }

int dq_eden_quantize_static(const float *vec, int64_t n, const float *boundaries, const float *centroids, int nbits,
                            uint32_t *packed, float *result, int device, dq_stream_t stream)
{
    if (!(n > 0) || (n & 31) != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of 32");
    if (n > dq::eden_static_max_n())
        return fail(DQ_ERR_SIZE, "n exceeds the static scratch array (dq_eden_quantize_static_max_n); use dq_eden_quantize");
    if (nbits < 1 || nbits > 8) return fail(DQ_ERR_NBITS, "nbits must be in [1, 8]");
    if (!vec || !boundaries || !centroids || !packed || !result) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_eden_quantize_static(vec, n, boundaries, centroids, nbits, packed, result, device,
                                                  static_cast<hipStream_t>(stream)));
}

int dq_eden_dequantize(const uint32_t *packed, int64_t n, const float *centroids, int nbits, float *out, int device,
                       dq_stream_t stream)
{
    if (!(n > 0) || (n & 31) != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of 32");
    if (nbits < 1 || nbits > 8) return fail(DQ_ERR_NBITS, "nbits must be in [1, 8]");
    if (!packed || !centroids || !out) return fail(DQ_ERR_NULL);
    if (reinterpret_cast<uintptr_t>(out) & 15) return fail(DQ_ERR_SIZE, "out must be 16-byte aligned");
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_eden_dequantize(packed, n, centroids, nbits, out, static_cast<hipStream_t>(stream)));
}

int dq_thc_quantize(const float *rotated, const float *uniform, void *levels_bf16, int64_t n, const float *lo,
                    const float *delta, int levels, int device, dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (levels < 2 || levels > 256) return fail(DQ_ERR_SIZE, "levels must be in [2, 256]");
    if (!rotated || !uniform || !levels_bf16 || !lo || !delta) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_thc_quantize(rotated, uniform, levels_bf16, n, lo, delta, levels, static_cast<hipStream_t>(stream)));
}

static int check_thc_rht(int64_t n, int64_t block)
{
    if (!(block > 0) || (block & (block - 1)) != 0) return fail(DQ_ERR_POW2, "block");
    if (!(n > 0) || n % block != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of block");
    return DQ_OK;
}

int dq_thc_rht_quantize(float *work, const void *sign, int sign_packed, const float *uniform, void *levels_bf16, int64_t n,
                        int64_t block, float scale, const float *lo, const float *delta, int levels, int device,
                        dq_stream_t stream)
{
    int rc = check_thc_rht(n, block);
    if (rc) return rc;
    if (levels < 2 || levels > 256) return fail(DQ_ERR_SIZE, "levels must be in [2, 256]");
    if (!work || !uniform || !levels_bf16 || !lo || !delta) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_thc_rht_quantize(work, sign, sign_packed != 0, uniform, levels_bf16, n, block, scale, lo, delta, levels,
                                              static_cast<hipStream_t>(stream)));
}

int dq_thc_dequantize_irht(const void *levels_bf16, const void *sign, int sign_packed, float *out, int64_t n, int64_t block,
                           float scale, const float *step, const float *lo, int device, dq_stream_t stream)
{
    int rc = check_thc_rht(n, block);
    if (rc) return rc;
    if (!levels_bf16 || !out || !step || !lo) return fail(DQ_ERR_NULL);
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_thc_dequantize_irht(levels_bf16, sign, sign_packed != 0, out, n, block, scale, step, lo,
                                                 static_cast<hipStream_t>(stream)));
}

int dq_eden_dequantize_irht(const uint32_t *packed, int64_t n, const float *centroids, int nbits, const void *sign,
                            int sign_packed, float *out, int64_t block, float scale, const float *post_scale, int device,
                            dq_stream_t stream)
{
    if (nbits < 1 || nbits > 8) return fail(DQ_ERR_NBITS, "nbits must be in [1, 8]");
    if (!(n > 0) || (n & 31) != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of 32");
    if (!(block >= 16) || (block & (block - 1)) != 0) return fail(DQ_ERR_POW2, "block (at least 16)");
    if (n % block != 0) return fail(DQ_ERR_SIZE, "n must be a positive multiple of block");
    if (!packed || !centroids || !out) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_eden_dequantize_irht(packed, centroids, nbits, sign, sign_packed != 0, out, n, block, scale,
                                                  post_scale, static_cast<hipStream_t>(stream)));
}

int dq_thc_dequantize(const void *levels_bf16, float *out, int64_t n, const float *step, const float *lo, int device,
                      dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!levels_bf16 || !out || !step || !lo) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_thc_dequantize(levels_bf16, out, n, step, lo, static_cast<hipStream_t>(stream)));
}

int dq_quantization(float *vec, int64_t n, int device, float div_factor, float tensor_max, uint64_t seed,
                    dq_stream_t stream)
{
    if (!(n > 0)) return fail(DQ_ERR_N);
    if (!vec) return fail(DQ_ERR_NULL);
    int rc;
    if ((rc = select_device(device))) return rc;
    return finish(dq::launch_quantization(vec, n, div_factor, tensor_max, seed, static_cast<hipStream_t>(stream)));
}

} // extern "C"
