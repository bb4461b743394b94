// Python module `eden_utils`: the binding layer of the reference
// (cuda_kernels/src/srrcomp/eden_utils/eden_utils.cpp:417-433) re-created on
// top of the C ABI of libdynamiq_eden.so.  Same function names, argument order,
// keyword names, defaults, dtypes, ownership rules and TORCH_CHECK messages, so
// testbed_evaluation/new_comm_hooks/utils_aggregation.py, thc_hooks.py and
// srrcomp.py import it unchanged.  On ROCm builds of PyTorch a HIP device
// reports itself as torch::kCUDA, which is what the checks below test.
//
// Additions (not in the reference): the *_ex variants accept float32 buffers
// and 3/5/6/7-bit codes, plus rht_blocked, rand_diag, scaling_required_bytes,
// set_quantization_seed and abi_version.
#include <torch/extension.h>
#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPStream.h>

#include <atomic>
#include <cstring>
#include <vector>

#include "dynamiq_eden.h"

namespace {

std::atomic<uint64_t> g_quant_seed{0x243F6A8885A308D3ull};

bool is_supported_data_dtype(c10::ScalarType dtype, bool extended)
{
    if (dtype == torch::kFloat16 || dtype == torch::kBFloat16) return true;
    return extended && dtype == torch::kFloat32;
}

int dq_dtype_of(c10::ScalarType dtype)
{
    if (dtype == torch::kFloat16) return DQ_F16;
    if (dtype == torch::kBFloat16) return DQ_BF16;
    return DQ_F32;
}

int64_t superchunk_num_chunks(int n, int superchunk_size)
{
    return (static_cast<int64_t>(n) + superchunk_size - 1) / superchunk_size;
}

// eden_utils.cpp:42-53, same order and wording
void scaling_check_common(int n, int nbits, int chunk_size, int strategy, bool extended)
{
    TORCH_CHECK(n > 0, "n must be positive");
    if (extended) {
        TORCH_CHECK(nbits >= 2 && nbits <= 8, "nbits must be in [2, 8]");
    } else {
        TORCH_CHECK(nbits == 2 || nbits == 4 || nbits == 8, "nbits must be one of {2, 4, 8}");
    }
    TORCH_CHECK(strategy >= 0 && strategy <= 3, "strategy must be 0 (AEE), 1 (MEE), 2 (hierarchical AEE), or 3 (hierarchical MEE)");
    TORCH_CHECK(chunk_size > 0 && chunk_size <= 32, "chunk_size must be in [1, 32]");
    TORCH_CHECK((chunk_size & (chunk_size - 1)) == 0, "chunk_size must be a power of two");
    TORCH_CHECK((chunk_size * nbits) % 8 == 0, "chunk_size * nbits must be divisible by 8");
    TORCH_CHECK(n % chunk_size == 0, "n must be a multiple of chunk_size");
    if (strategy >= 2) {
        TORCH_CHECK((n / chunk_size) % 16 == 0, "hierarchical mode requires n to contain a whole number of 16-chunk superchunks");
    }
}

void check_status(int status, const char *what)
{
    TORCH_CHECK(status == DQ_OK, what, ": ", dq_last_error());
}

dq_stream_t as_stream(uint64_t stream_p) { return reinterpret_cast<dq_stream_t>(static_cast<uintptr_t>(stream_p)); }

// A tensor allocated here belongs to torch's current stream; the kernels that use it run on the caller's stream_p (the
// reference's functions have the same split).  When the two differ the caching allocator is told, so that the block is
// not handed out again (once the tensor is released) before the work queued on stream_p has finished with it.
torch::Tensor on_stream(torch::Tensor t, uint64_t stream_p)
{
    if (!t.defined() || t.numel() == 0) return t;
    const auto dev = t.device().index();
    const hipStream_t s = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(stream_p));
    if (c10::hip::getCurrentHIPStream(dev).stream() != s) {
        const auto user = s == nullptr ? c10::hip::getDefaultHIPStream(dev) : c10::hip::getStreamFromExternal(s, dev);
        c10::hip::HIPCachingAllocator::recordStream(t.storage().data_ptr(), user);
    }
    return t;
}

// ---- Hadamard --------------------------------------------------------------------

torch::Tensor Hadamard(torch::Tensor vec, uint64_t stream_p = 0, int depth = 0)
{
    TORCH_CHECK(vec.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(vec.dtype() == torch::kFloat32, "input must be a torch.float32 CUDA tensor");
    auto n = vec.size(-1);
    TORCH_CHECK(n == vec.numel(), "input must be 1D");
    TORCH_CHECK((n & (n - 1)) == 0 && n > 0, "input size must be a power of 2");
    auto output = vec.clone(); // contiguous copy, as in the reference
    check_status(dq_hadamard(output.data_ptr<float>(), n, output.device().index(), as_stream(stream_p), depth), "Hadamard");
    return output;
}

void Hadamard_inplace(torch::Tensor vec, uint64_t stream_p = 0, int depth = 0)
{
    TORCH_CHECK(vec.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(vec.dtype() == torch::kFloat32, "input must be a torch.float32 CUDA tensor");
    auto n = vec.size(-1);
    TORCH_CHECK(n == vec.numel(), "input must be 1D");
    TORCH_CHECK((n & (n - 1)) == 0 && n > 0, "input size must be a power of 2");
    check_status(dq_hadamard(vec.data_ptr<float>(), n, vec.device().index(), as_stream(stream_p), depth), "Hadamard_inplace");
}

void Hadamard_inplace_ptr(long long vec, int n, int device, uint64_t stream_p = 0, int depth = 0)
{
    check_status(dq_hadamard(reinterpret_cast<float *>(vec), n, device, as_stream(stream_p), depth), "Hadamard_inplace_ptr");
}

// The reference stores the pointer as curand state storage and launches
// nothing (cuda_hadamard.cu:674-686).  Randomness here is counter based, so
// there is no state to place in the caller's buffer: both calls are no-ops.
void Hadamard_init(torch::Tensor vec) { (void)vec.data_ptr<int>(); }
void Hadamard_init_ptr(long long vec, int device = 0) { (void)vec; (void)device; }

void quantization_compression(torch::Tensor vec, float div_factor, float tensor_max, uint64_t stream_p = 0)
{
    TORCH_CHECK(vec.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(vec.dtype() == torch::kFloat32, "input must be a torch.float32 CUDA tensor");
    auto n = vec.size(-1);
    const uint64_t seed = g_quant_seed.fetch_add(0x9E3779B97F4A7C15ull);
    check_status(dq_quantization(vec.data_ptr<float>(), n, vec.device().index(), div_factor, tensor_max, seed, as_stream(stream_p)),
                 "quantization_compression");
}

void set_quantization_seed(uint64_t seed) { g_quant_seed.store(seed); }

static const void *sign_arg(const c10::optional<torch::Tensor> &sign, const torch::Tensor &vec, int64_t n, int *packed);

torch::Tensor rht_blocked(torch::Tensor vec, c10::optional<torch::Tensor> sign, int64_t block, double scale, bool inverse,
                          uint64_t stream_p = 0)
{
    TORCH_CHECK(vec.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(vec.dtype() == torch::kFloat32, "input must be a torch.float32 CUDA tensor");
    TORCH_CHECK(vec.is_contiguous(), "input must be contiguous");
    int packed = 0;
    const void *sp = sign_arg(sign, vec, vec.numel(), &packed);
    check_status(dq_rht_blocked(vec.data_ptr<float>(), sp, packed, vec.numel(), block, (float)scale, inverse ? 1 : 0,
                                vec.device().index(), as_stream(stream_p)),
                 "rht_blocked");
    return vec;
}

// sign for the fused transform + quantiser calls: float32 +-1 values or the int32 bit vector of pack_signs
static const void *sign_arg(const c10::optional<torch::Tensor> &sign, const torch::Tensor &vec, int64_t n, int *packed)
{
    *packed = 0;
    if (!sign.has_value()) return nullptr;
    TORCH_CHECK(sign->device() == vec.device(), "sign must be on the same device as the vector");
    TORCH_CHECK(sign->is_contiguous(), "sign must be contiguous");
    if (sign->dtype() == torch::kInt32) {
        TORCH_CHECK(sign->numel() >= (n + 31) / 32, "packed sign has fewer than n bits");
        *packed = 1;
    } else {
        TORCH_CHECK(sign->dtype() == torch::kFloat32, "sign must be torch.float32 (+-1 values) or torch.int32 (packed bits)");
        TORCH_CHECK(sign->numel() >= n, "sign has fewer elements than the vector");
    }
    return sign->data_ptr();
}

torch::Tensor rand_diag_bits(int64_t size, int64_t seed, torch::Device device, uint64_t stream_p = 0)
{
    TORCH_CHECK(device.type() == torch::kCUDA, "device must be a CUDA device");
    TORCH_CHECK(size > 0 && size % 256 == 0, "size must be a positive multiple of 256");
    auto bits = on_stream(torch::empty({size / 32}, torch::TensorOptions().dtype(torch::kInt32).device(device)), stream_p);
    check_status(dq_rand_diag_bits(reinterpret_cast<uint32_t *>(bits.data_ptr<int32_t>()), size, seed, bits.device().index(),
                                   as_stream(stream_p)),
                 "rand_diag_bits");
    return bits;
}

torch::Tensor pack_signs(torch::Tensor sign, uint64_t stream_p = 0)
{
    TORCH_CHECK(sign.device().type() == torch::kCUDA && sign.dtype() == torch::kFloat32 && sign.is_contiguous(),
                "sign must be a contiguous torch.float32 CUDA tensor");
    TORCH_CHECK(sign.numel() > 0, "sign must not be empty");
    auto bits = on_stream(torch::empty({(sign.numel() + 31) / 32}, sign.options().dtype(torch::kInt32)), stream_p);
    check_status(dq_pack_signs(sign.data_ptr<float>(), reinterpret_cast<uint32_t *>(bits.data_ptr<int32_t>()), sign.numel(),
                               sign.device().index(), as_stream(stream_p)),
                 "pack_signs");
    return bits;
}

void rht_scaling_compress(torch::Tensor src, c10::optional<torch::Tensor> sign, torch::Tensor dst, int64_t block, double scale,
                          int nbits, c10::optional<torch::Tensor> rand_pool, uint64_t seed = 0, uint64_t step = 0,
                          uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA && src.dtype() == torch::kFloat32 && src.is_contiguous(),
                "input must be a contiguous torch.float32 CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA && dst.dtype() == torch::kUInt8 && dst.is_contiguous(),
                "output must be a contiguous torch.uint8 CUDA tensor");
    const int64_t n = src.numel();
    TORCH_CHECK(n > 0 && n % 256 == 0, "the element count must be a positive multiple of 256");
    TORCH_CHECK(dst.numel() >= dq_scaling_required_bytes(n, nbits, 16, strategy), "output buffer is too small");
    int packed = 0;
    const void *sp = sign_arg(sign, src, n, &packed);
    const void *rp = nullptr;
    int rcode = DQ_F32;
    if (rand_pool.has_value()) {
        TORCH_CHECK(rand_pool->device() == src.device() && rand_pool->is_contiguous(), "rand_pool must be a contiguous tensor on the input's device");
        TORCH_CHECK(rand_pool->dtype() == torch::kFloat32 || rand_pool->dtype() == torch::kBFloat16, "rand_pool must be torch.float32 or torch.bfloat16");
        TORCH_CHECK(rand_pool->numel() >= n, "rand_pool has fewer elements than the input");
        rcode = dq_dtype_of(rand_pool->scalar_type());
        rp = rand_pool->data_ptr();
    }
    check_status(dq_rht_scaling_compress(src.data_ptr<float>(), sp, packed, dst.data_ptr<uint8_t>(), rp, rcode, n, block,
                                         (float)scale, nbits, src.device().index(), strategy, seed, step, as_stream(stream_p)),
                 "rht_scaling_compress");
}

void scaling_decompress_irht(torch::Tensor src, c10::optional<torch::Tensor> sign, torch::Tensor dst, int64_t block, double scale,
                             int nbits, uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA && src.dtype() == torch::kUInt8 && src.is_contiguous(),
                "input must be a contiguous torch.uint8 CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA && dst.dtype() == torch::kFloat32 && dst.is_contiguous(),
                "output must be a contiguous torch.float32 CUDA tensor");
    const int64_t n = dst.numel();
    TORCH_CHECK(n > 0 && n % 256 == 0, "the element count must be a positive multiple of 256");
    TORCH_CHECK(src.numel() >= dq_scaling_required_bytes(n, nbits, 16, strategy), "input buffer is too small");
    int packed = 0;
    const void *sp = sign_arg(sign, dst, n, &packed);
    check_status(dq_scaling_decompress_irht(src.data_ptr<uint8_t>(), sp, packed, dst.data_ptr<float>(), n, block, (float)scale,
                                            nbits, dst.device().index(), strategy, as_stream(stream_p)),
                 "scaling_decompress_irht");
}

torch::Tensor rand_diag(int64_t size, int64_t seed, torch::Device device, uint64_t stream_p = 0)
{
    TORCH_CHECK(device.type() == torch::kCUDA, "device must be a CUDA device");
    auto out = on_stream(torch::empty({size}, torch::TensorOptions().device(device).dtype(torch::kFloat32)), stream_p);
    check_status(dq_rand_diag(out.data_ptr<float>(), size, seed, out.device().index(), as_stream(stream_p)), "rand_diag");
    return out;
}

// ---- scaling quantisation ---------------------------------------------------------

void scaling_compress_impl(torch::Tensor src, torch::Tensor dst, torch::Tensor rand_pool, int n, int nbits, int chunk_size,
                           uint64_t stream_p, int strategy, bool ex)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(rand_pool.device().type() == torch::kCUDA, "rand_pool must be a CUDA tensor");
    TORCH_CHECK(is_supported_data_dtype(src.scalar_type(), ex), "input must be torch.float16 or torch.bfloat16");
    TORCH_CHECK(dst.dtype() == torch::kUInt8, "output must be torch.uint8");
    // extended calls also take a bf16 pool next to float32 gradients (the reference's pools are bf16)
    const bool mixed = ex && src.scalar_type() == torch::kFloat32 && rand_pool.scalar_type() == torch::kBFloat16;
    TORCH_CHECK(mixed || rand_pool.dtype() == src.dtype(), "rand_pool dtype must match input dtype");
    TORCH_CHECK(src.is_contiguous(), "input must be contiguous");
    TORCH_CHECK(dst.is_contiguous(), "output must be contiguous");
    TORCH_CHECK(rand_pool.is_contiguous(), "rand_pool must be contiguous");
    scaling_check_common(n, nbits, chunk_size, strategy, ex);
    TORCH_CHECK(src.numel() >= n, "input has fewer than n elements");
    TORCH_CHECK(rand_pool.numel() >= n, "rand_pool has fewer than n elements");
    TORCH_CHECK(dst.numel() >= dq_scaling_required_bytes(n, nbits, chunk_size, strategy), "output buffer is too small");
    check_status(dq_scaling_compress(src.data_ptr(), dst.data_ptr<uint8_t>(), rand_pool.data_ptr(), n, nbits, chunk_size,
                                     dq_dtype_of(src.scalar_type()) | (mixed ? DQ_RAND_BF16 : 0), src.device().index(), strategy,
                                     as_stream(stream_p)),
                 "scaling_compress");
}

void scaling_decompress_impl(torch::Tensor src, torch::Tensor dst, int n, int nbits, int chunk_size, uint64_t stream_p,
                             int strategy, bool ex, int add)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(src.dtype() == torch::kUInt8, "input must be torch.uint8");
    TORCH_CHECK(is_supported_data_dtype(dst.scalar_type(), ex), "output must be torch.float16 or torch.bfloat16");
    TORCH_CHECK(src.is_contiguous(), "input must be contiguous");
    TORCH_CHECK(dst.is_contiguous(), "output must be contiguous");
    scaling_check_common(n, nbits, chunk_size, strategy, ex);
    TORCH_CHECK(src.numel() >= dq_scaling_required_bytes(n, nbits, chunk_size, strategy), "input buffer is too small");
    TORCH_CHECK(dst.numel() >= n, "output has fewer than n elements");
    check_status(dq_scaling_decompress(src.data_ptr<uint8_t>(), dst.data_ptr(), n, nbits, chunk_size,
                                       dq_dtype_of(dst.scalar_type()), src.device().index(), strategy, as_stream(stream_p), add),
                 add ? "scaling_decompress_add" : "scaling_decompress");
}

void scaling_dec_comp_impl(torch::Tensor recv, torch::Tensor inp, torch::Tensor send, torch::Tensor rand_pool, int n, int nbits,
                           int chunk_size, uint64_t stream_p, int strategy, bool ex)
{
    TORCH_CHECK(recv.device().type() == torch::kCUDA, "recv must be a CUDA tensor");
    TORCH_CHECK(inp.device().type() == torch::kCUDA, "inp must be a CUDA tensor");
    TORCH_CHECK(send.device().type() == torch::kCUDA, "send must be a CUDA tensor");
    TORCH_CHECK(rand_pool.device().type() == torch::kCUDA, "rand_pool must be a CUDA tensor");
    TORCH_CHECK(recv.dtype() == torch::kUInt8, "recv must be torch.uint8");
    TORCH_CHECK(is_supported_data_dtype(inp.scalar_type(), ex), "inp must be torch.float16 or torch.bfloat16");
    TORCH_CHECK(send.dtype() == torch::kUInt8, "send must be torch.uint8");
    const bool mixed = ex && inp.scalar_type() == torch::kFloat32 && rand_pool.scalar_type() == torch::kBFloat16;
    TORCH_CHECK(mixed || rand_pool.dtype() == inp.dtype(), "rand_pool dtype must match inp dtype");
    TORCH_CHECK(recv.is_contiguous(), "recv must be contiguous");
    TORCH_CHECK(inp.is_contiguous(), "inp must be contiguous");
    TORCH_CHECK(send.is_contiguous(), "send must be contiguous");
    TORCH_CHECK(rand_pool.is_contiguous(), "rand_pool must be contiguous");
    scaling_check_common(n, nbits, chunk_size, strategy, ex);
    const int64_t required_bytes = dq_scaling_required_bytes(n, nbits, chunk_size, strategy);
    TORCH_CHECK(recv.numel() >= required_bytes, "recv buffer is too small");
    TORCH_CHECK(send.numel() >= required_bytes, "send buffer is too small");
    TORCH_CHECK(inp.numel() >= n, "inp has fewer than n elements");
    TORCH_CHECK(rand_pool.numel() >= n, "rand_pool has fewer than n elements");
    check_status(dq_scaling_dec_comp(recv.data_ptr<uint8_t>(), inp.data_ptr(), send.data_ptr<uint8_t>(), rand_pool.data_ptr(), n,
                                     nbits, chunk_size, dq_dtype_of(inp.scalar_type()) | (mixed ? DQ_RAND_BF16 : 0),
                                     recv.device().index(), strategy, as_stream(stream_p)),
                 "scaling_dec_comp");
}

void scaling_compress(torch::Tensor src, torch::Tensor dst, torch::Tensor rand_pool, int n, int nbits, int chunk_size,
                      uint64_t stream_p = 0, int strategy = 0)
{
    scaling_compress_impl(src, dst, rand_pool, n, nbits, chunk_size, stream_p, strategy, false);
}
void scaling_compress_ex(torch::Tensor src, torch::Tensor dst, torch::Tensor rand_pool, int n, int nbits, int chunk_size,
                         uint64_t stream_p = 0, int strategy = 0)
{
    scaling_compress_impl(src, dst, rand_pool, n, nbits, chunk_size, stream_p, strategy, true);
}
void scaling_decompress(torch::Tensor src, torch::Tensor dst, int n, int nbits, int chunk_size, uint64_t stream_p = 0, int strategy = 0)
{
    scaling_decompress_impl(src, dst, n, nbits, chunk_size, stream_p, strategy, false, 0);
}
void scaling_decompress_ex(torch::Tensor src, torch::Tensor dst, int n, int nbits, int chunk_size, uint64_t stream_p = 0, int strategy = 0)
{
    scaling_decompress_impl(src, dst, n, nbits, chunk_size, stream_p, strategy, true, 0);
}
void scaling_decompress_add(torch::Tensor src, torch::Tensor dst, int n, int nbits, int chunk_size, uint64_t stream_p = 0, int strategy = 0)
{
    scaling_decompress_impl(src, dst, n, nbits, chunk_size, stream_p, strategy, false, 1);
}
void scaling_decompress_add_ex(torch::Tensor src, torch::Tensor dst, int n, int nbits, int chunk_size, uint64_t stream_p = 0,
                               int strategy = 0)
{
    scaling_decompress_impl(src, dst, n, nbits, chunk_size, stream_p, strategy, true, 1);
}
void scaling_dec_comp(torch::Tensor recv, torch::Tensor inp, torch::Tensor send, torch::Tensor rand_pool, int n, int nbits,
                      int chunk_size, uint64_t stream_p = 0, int strategy = 0)
{
    scaling_dec_comp_impl(recv, inp, send, rand_pool, n, nbits, chunk_size, stream_p, strategy, false);
}
void scaling_dec_comp_ex(torch::Tensor recv, torch::Tensor inp, torch::Tensor send, torch::Tensor rand_pool, int n, int nbits,
                         int chunk_size, uint64_t stream_p = 0, int strategy = 0)
{
    scaling_dec_comp_impl(recv, inp, send, rand_pool, n, nbits, chunk_size, stream_p, strategy, true);
}

int64_t scaling_required_bytes(int64_t n, int nbits, int chunk_size, int strategy)
{
    return dq_scaling_required_bytes(n, nbits, chunk_size, strategy);
}

// ---- dynamic-bitrate groups (additions; see include/dynamiq_eden.h) -----------------

void check_rows_tensor(const torch::Tensor &rows, int64_t nrows)
{
    TORCH_CHECK(rows.device().type() == torch::kCUDA, "rows must be a CUDA tensor");
    TORCH_CHECK(rows.dtype() == torch::kInt32, "rows must be torch.int32");
    TORCH_CHECK(rows.is_contiguous(), "rows must be contiguous");
    TORCH_CHECK(rows.numel() >= nrows, "rows has fewer than nrows entries");
}

void check_rows_common(int64_t nrows, int nbits, int strategy)
{
    TORCH_CHECK(nrows > 0, "nrows must be positive");
    TORCH_CHECK(nbits >= 2 && nbits <= 8, "nbits must be in [2, 8]");
    TORCH_CHECK(strategy == 2 || strategy == 3, "strategy must be 2 (hierarchical AEE) or 3 (hierarchical MEE)");
}

torch::Tensor group_plan(torch::Tensor qbits, torch::Tensor order, uint64_t stream_p = 0)
{
    TORCH_CHECK(qbits.device().type() == torch::kCUDA, "qbits must be a CUDA tensor");
    TORCH_CHECK(order.device().type() == torch::kCUDA, "order must be a CUDA tensor");
    TORCH_CHECK(qbits.dtype() == torch::kInt64, "qbits must be torch.int64");
    TORCH_CHECK(order.dtype() == torch::kInt32, "order must be torch.int32");
    TORCH_CHECK(qbits.is_contiguous() && order.is_contiguous(), "qbits and order must be contiguous");
    const int64_t nsc = qbits.numel();
    TORCH_CHECK(nsc > 0, "qbits must not be empty");
    TORCH_CHECK(order.numel() >= 3 * nsc, "order has fewer than 3 * nsc entries");
    auto work = on_stream(torch::empty({dq_group_plan_work_ints(nsc)}, order.options()), stream_p);
    check_status(dq_group_plan(qbits.data_ptr<int64_t>(), nsc, order.data_ptr<int32_t>(), work.data_ptr<int32_t>(),
                               work.numel(), qbits.device().index(), as_stream(stream_p)),
                 "group_plan");
    return work.slice(0, 0, 4);
}

torch::Tensor group_plan_stats(torch::Tensor stats, double u, torch::Tensor order, c10::optional<torch::Tensor> qbits_out,
                               uint64_t stream_p = 0)
{
    TORCH_CHECK(stats.device().type() == torch::kCUDA, "stats must be a CUDA tensor");
    TORCH_CHECK(order.device().type() == torch::kCUDA, "order must be a CUDA tensor");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(order.dtype() == torch::kInt32, "order must be torch.int32");
    TORCH_CHECK(stats.is_contiguous() && order.is_contiguous(), "stats and order must be contiguous");
    const int64_t nsc = stats.numel() / 2;
    TORCH_CHECK(nsc > 0 && stats.numel() == 2 * nsc, "stats must hold (mean, norm) pairs");
    TORCH_CHECK(order.numel() >= 3 * nsc, "order has fewer than 3 * nsc entries");
    int64_t *qptr = nullptr;
    if (qbits_out.has_value()) {
        TORCH_CHECK(qbits_out->device().type() == torch::kCUDA && qbits_out->dtype() == torch::kInt64 &&
                        qbits_out->is_contiguous() && qbits_out->numel() >= nsc,
                    "qbits_out must be a contiguous torch.int64 CUDA tensor with one entry per superchunk");
        qptr = qbits_out->data_ptr<int64_t>();
    }
    auto work = on_stream(torch::empty({dq_group_plan_work_ints(nsc)}, order.options()), stream_p);
    check_status(dq_group_plan_stats(stats.data_ptr(), u, nsc, qptr, order.data_ptr<int32_t>(), work.data_ptr<int32_t>(),
                                     work.numel(), stats.device().index(), as_stream(stream_p)),
                 "group_plan_stats");
    return work.slice(0, 0, 4);
}

torch::Tensor group_plan_sorted(torch::Tensor stats, int64_t top_count, int64_t bottom_count, torch::Tensor order,
                                c10::optional<torch::Tensor> qbits_out, uint64_t stream_p = 0)
{
    TORCH_CHECK(stats.device().type() == torch::kCUDA, "stats must be a CUDA tensor");
    TORCH_CHECK(order.device().type() == torch::kCUDA, "order must be a CUDA tensor");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(order.dtype() == torch::kInt32, "order must be torch.int32");
    TORCH_CHECK(stats.is_contiguous() && order.is_contiguous(), "stats and order must be contiguous");
    const int64_t nsc = stats.numel() / 2;
    TORCH_CHECK(nsc > 0 && stats.numel() == 2 * nsc, "stats must hold (mean, norm) pairs");
    TORCH_CHECK(order.numel() >= 3 * nsc, "order has fewer than 3 * nsc entries");
    int64_t *qptr = nullptr;
    if (qbits_out.has_value()) {
        TORCH_CHECK(qbits_out->device().type() == torch::kCUDA && qbits_out->dtype() == torch::kInt64 &&
                        qbits_out->is_contiguous() && qbits_out->numel() >= nsc,
                    "qbits_out must be a contiguous torch.int64 CUDA tensor with one entry per superchunk");
        qptr = qbits_out->data_ptr<int64_t>();
    }
    auto work = on_stream(torch::empty({dq_group_plan_sorted_work_ints(nsc)}, order.options()), stream_p);
    check_status(dq_group_plan_sorted(stats.data_ptr(), nsc, top_count, bottom_count, qptr, order.data_ptr<int32_t>(),
                                      work.data_ptr<int32_t>(), work.numel(), stats.device().index(), as_stream(stream_p)),
                 "group_plan_sorted");
    return work.slice(0, 0, 4);
}

torch::Tensor group_plan_stats_dev_u(torch::Tensor stats, torch::Tensor u, torch::Tensor order,
                                     c10::optional<torch::Tensor> qbits_out, c10::optional<torch::Tensor> hist,
                                     uint64_t stream_p = 0)
{
    TORCH_CHECK(stats.device().type() == torch::kCUDA, "stats must be a CUDA tensor");
    TORCH_CHECK(order.device().type() == torch::kCUDA, "order must be a CUDA tensor");
    TORCH_CHECK(u.device() == stats.device() && u.dtype() == torch::kFloat64 && u.numel() >= 1,
                "u must be a torch.float64 tensor on the device of stats");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(order.dtype() == torch::kInt32, "order must be torch.int32");
    TORCH_CHECK(stats.is_contiguous() && order.is_contiguous(), "stats and order must be contiguous");
    const int64_t nsc = stats.numel() / 2;
    TORCH_CHECK(nsc > 0 && stats.numel() == 2 * nsc, "stats must hold (mean, norm) pairs");
    TORCH_CHECK(order.numel() >= 3 * nsc, "order has fewer than 3 * nsc entries");
    int64_t *qptr = nullptr;
    if (qbits_out.has_value()) {
        TORCH_CHECK(qbits_out->device().type() == torch::kCUDA && qbits_out->dtype() == torch::kInt64 &&
                        qbits_out->is_contiguous() && qbits_out->numel() >= nsc,
                    "qbits_out must be a contiguous torch.int64 CUDA tensor with one entry per superchunk");
        qptr = qbits_out->data_ptr<int64_t>();
    }
    auto work = on_stream(torch::empty({dq_group_plan_work_ints(nsc)}, order.options()), stream_p);
    uint32_t *hptr = nullptr;
    int64_t hlen = 0;
    if (hist.has_value()) {
        TORCH_CHECK(hist->device() == stats.device() && hist->dtype() == torch::kInt32 && hist->is_contiguous() &&
                        hist->numel() >= dq_bitrate_hist_ints(),
                    "hist must be a contiguous torch.int32 tensor of bitrate_hist_ints() entries on the device of stats");
        hptr = reinterpret_cast<uint32_t *>(hist->data_ptr<int32_t>());
        hlen = hist->numel();
    }
    check_status(dq_group_plan_stats_dev_u(stats.data_ptr(), u.data_ptr<double>(), nsc, qptr, order.data_ptr<int32_t>(),
                                           work.data_ptr<int32_t>(), work.numel(), hptr, hlen, stats.device().index(),
                                           as_stream(stream_p)),
                 "group_plan_stats_dev_u");
    return work.slice(0, 0, 4);
}

int64_t bitrate_hist_ints() { return dq_bitrate_hist_ints(); }

void norm_histogram(torch::Tensor stats, torch::Tensor hist, uint64_t stream_p = 0)
{
    TORCH_CHECK(stats.device().type() == torch::kCUDA && hist.device().type() == torch::kCUDA, "stats and hist must be CUDA tensors");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(hist.dtype() == torch::kInt32, "hist must be torch.int32");
    TORCH_CHECK(stats.is_contiguous() && hist.is_contiguous(), "stats and hist must be contiguous");
    const int64_t nsc = stats.numel() / 2;
    TORCH_CHECK(nsc > 0 && stats.numel() == 2 * nsc, "stats must hold (mean, norm) pairs");
    TORCH_CHECK(hist.numel() >= dq_bitrate_hist_ints(), "hist has fewer than bitrate_hist_ints() entries");
    check_status(dq_norm_histogram(stats.data_ptr(), nsc, reinterpret_cast<uint32_t *>(hist.data_ptr<int32_t>()), hist.numel(),
                                   stats.device().index(), as_stream(stream_p)),
                 "norm_histogram");
}

torch::Tensor bitrate_search(torch::Tensor hist, int mode, double prev_u, double target_avg_bits, uint64_t stream_p = 0)
{
    TORCH_CHECK(hist.device().type() == torch::kCUDA, "hist must be a CUDA tensor");
    TORCH_CHECK(hist.dtype() == torch::kInt32 && hist.is_contiguous(), "hist must be a contiguous torch.int32 tensor");
    TORCH_CHECK(hist.numel() >= dq_bitrate_hist_ints(), "hist has fewer than bitrate_hist_ints() entries");
    TORCH_CHECK(mode == 0 || mode == 1, "mode must be 0 (bisection) or 1 (correction from prev_u)");
    auto result = on_stream(torch::empty({4}, hist.options().dtype(torch::kFloat64)), stream_p);
    check_status(dq_bitrate_search(reinterpret_cast<uint32_t *>(hist.data_ptr<int32_t>()), hist.numel(), mode, prev_u, nullptr,
                                   target_avg_bits, result.data_ptr<double>(), hist.device().index(), as_stream(stream_p)),
                 "bitrate_search");
    return result;
}

void scaling_compress_rows(torch::Tensor src, torch::Tensor rows, torch::Tensor dst, torch::Tensor rand_pool, int64_t nrows,
                           int nbits, uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(rand_pool.device().type() == torch::kCUDA, "rand_pool must be a CUDA tensor");
    TORCH_CHECK(src.scalar_type() == torch::kBFloat16 || src.scalar_type() == torch::kFloat32, "input must be torch.bfloat16 or torch.float32");
    TORCH_CHECK(dst.dtype() == torch::kUInt8, "output must be torch.uint8");
    const bool mixed = src.scalar_type() == torch::kFloat32 && rand_pool.scalar_type() == torch::kBFloat16;
    TORCH_CHECK(mixed || rand_pool.dtype() == src.dtype(), "rand_pool dtype must match input dtype");
    TORCH_CHECK(src.is_contiguous() && dst.is_contiguous() && rand_pool.is_contiguous(), "buffers must be contiguous");
    check_rows_common(nrows, nbits, strategy);
    check_rows_tensor(rows, nrows);
    TORCH_CHECK(dst.numel() >= dq_scaling_required_bytes(nrows * 256, nbits, 16, strategy), "output buffer is too small");
    TORCH_CHECK(rand_pool.numel() >= nrows * 256, "rand_pool has fewer than 256 * nrows elements");
    check_status(dq_scaling_compress_rows(src.data_ptr(), rows.data_ptr<int32_t>(), dst.data_ptr<uint8_t>(), rand_pool.data_ptr(),
                                          nrows, nbits, dq_dtype_of(src.scalar_type()) | (mixed ? DQ_RAND_BF16 : 0),
                                          src.device().index(), strategy, as_stream(stream_p)),
                 "scaling_compress_rows");
}

void scaling_dec_comp_rows(torch::Tensor recv, torch::Tensor inp, torch::Tensor rows, torch::Tensor send, torch::Tensor rand_pool,
                           int64_t nrows, int nbits, uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(recv.device().type() == torch::kCUDA && inp.device().type() == torch::kCUDA &&
                    send.device().type() == torch::kCUDA && rand_pool.device().type() == torch::kCUDA,
                "all buffers must be CUDA tensors");
    TORCH_CHECK(recv.dtype() == torch::kUInt8, "recv must be torch.uint8");
    TORCH_CHECK(send.dtype() == torch::kUInt8, "send must be torch.uint8");
    TORCH_CHECK(inp.scalar_type() == torch::kBFloat16 || inp.scalar_type() == torch::kFloat32, "inp must be torch.bfloat16 or torch.float32");
    const bool mixed = inp.scalar_type() == torch::kFloat32 && rand_pool.scalar_type() == torch::kBFloat16;
    TORCH_CHECK(mixed || rand_pool.dtype() == inp.dtype(), "rand_pool dtype must match inp dtype");
    TORCH_CHECK(recv.is_contiguous() && inp.is_contiguous() && send.is_contiguous() && rand_pool.is_contiguous(), "buffers must be contiguous");
    check_rows_common(nrows, nbits, strategy);
    check_rows_tensor(rows, nrows);
    const int64_t required_bytes = dq_scaling_required_bytes(nrows * 256, nbits, 16, strategy);
    TORCH_CHECK(recv.numel() >= required_bytes, "recv buffer is too small");
    TORCH_CHECK(send.numel() >= required_bytes, "send buffer is too small");
    TORCH_CHECK(rand_pool.numel() >= nrows * 256, "rand_pool has fewer than 256 * nrows elements");
    check_status(dq_scaling_dec_comp_rows(recv.data_ptr<uint8_t>(), inp.data_ptr(), rows.data_ptr<int32_t>(), send.data_ptr<uint8_t>(),
                                          rand_pool.data_ptr(), nrows, nbits,
                                          dq_dtype_of(inp.scalar_type()) | (mixed ? DQ_RAND_BF16 : 0), inp.device().index(),
                                          strategy, as_stream(stream_p)),
                 "scaling_dec_comp_rows");
}

void scaling_decompress_rows(torch::Tensor src, torch::Tensor dst, torch::Tensor rows, c10::optional<torch::Tensor> stats,
                             int64_t n_limit, int64_t nrows, int nbits, uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(src.dtype() == torch::kUInt8, "input must be torch.uint8");
    TORCH_CHECK(dst.scalar_type() == torch::kBFloat16 || dst.scalar_type() == torch::kFloat32, "output must be torch.bfloat16 or torch.float32");
    TORCH_CHECK(src.is_contiguous() && dst.is_contiguous(), "buffers must be contiguous");
    check_rows_common(nrows, nbits, strategy);
    check_rows_tensor(rows, nrows);
    TORCH_CHECK(src.numel() >= dq_scaling_required_bytes(nrows * 256, nbits, 16, strategy), "input buffer is too small");
    TORCH_CHECK(n_limit > 0 && n_limit <= dst.numel(), "n_limit must be in (0, output elements]");
    const void *stats_ptr = nullptr;
    if (stats.has_value()) {
        TORCH_CHECK(stats->device().type() == torch::kCUDA, "stats must be a CUDA tensor");
        TORCH_CHECK(stats->dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
        TORCH_CHECK(stats->is_contiguous(), "stats must be contiguous");
        TORCH_CHECK(stats->numel() >= 2 * ((n_limit + 255) / 256), "stats buffer is too small");
        stats_ptr = stats->data_ptr();
    }
    check_status(dq_scaling_decompress_rows(src.data_ptr<uint8_t>(), dst.data_ptr(), rows.data_ptr<int32_t>(), stats_ptr, n_limit,
                                            nrows, nbits, dq_dtype_of(dst.scalar_type()), dst.device().index(), strategy,
                                            as_stream(stream_p), 0),
                 "scaling_decompress_rows");
}

// ---- all bit-width groups of a planned bucket in one launch ---------------------------------

int64_t mixed_required_bytes(int64_t nsc, int ring_world = 1) { return dq_mixed_required_bytes(nsc, ring_world); }

static void check_plan_tensors(const torch::Tensor &order, const torch::Tensor &counts, int64_t nsc)
{
    TORCH_CHECK(nsc > 0, "nsc must be positive");
    TORCH_CHECK(order.device().type() == torch::kCUDA && counts.device().type() == torch::kCUDA, "order and counts must be CUDA tensors");
    TORCH_CHECK(order.dtype() == torch::kInt32 && counts.dtype() == torch::kInt32, "order and counts must be torch.int32");
    TORCH_CHECK(order.is_contiguous() && counts.is_contiguous(), "order and counts must be contiguous");
    TORCH_CHECK(order.numel() >= 3 * nsc, "order has fewer than 3 * nsc entries");
    TORCH_CHECK(counts.numel() >= 3, "counts must hold the three group sizes");
}

void mixed_compress(torch::Tensor src, torch::Tensor order, torch::Tensor counts, torch::Tensor dst, int64_t nsc,
                    c10::optional<torch::Tensor> rand_pool, c10::optional<torch::Tensor> recv,
                    c10::optional<torch::Tensor> center_mean, int center_world = 1, int64_t n = 0, int ring_chunk = 0,
                    int ring_world = 1, uint64_t seed = 0, uint64_t step = 0, uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(src.scalar_type() == torch::kBFloat16 || src.scalar_type() == torch::kFloat32, "input must be torch.bfloat16 or torch.float32");
    TORCH_CHECK(dst.dtype() == torch::kUInt8, "output must be torch.uint8");
    TORCH_CHECK(src.is_contiguous() && dst.is_contiguous(), "buffers must be contiguous");
    TORCH_CHECK(strategy == 2 || strategy == 3, "strategy must be 2 or 3");
    TORCH_CHECK(ring_world > 0 && ring_chunk >= 0 && ring_chunk < ring_world, "ring_chunk must lie in [0, ring_world)");
    check_plan_tensors(order, counts, nsc);
    const int64_t need = dq_mixed_required_bytes(nsc, ring_world);
    TORCH_CHECK(dst.numel() >= need, "output buffer is smaller than mixed_required_bytes(nsc, ring_world)");
    int code = dq_dtype_of(src.scalar_type());
    const void *rand_ptr = nullptr, *recv_ptr = nullptr;
    const float *mean_ptr = nullptr;
    if (rand_pool.has_value()) {
        TORCH_CHECK(rand_pool->device().type() == torch::kCUDA && rand_pool->is_contiguous(), "rand_pool must be a contiguous CUDA tensor");
        const bool mixed = src.scalar_type() == torch::kFloat32 && rand_pool->scalar_type() == torch::kBFloat16;
        TORCH_CHECK(mixed || rand_pool->dtype() == src.dtype(), "rand_pool dtype must match input dtype");
        TORCH_CHECK(rand_pool->numel() >= nsc * 256, "rand_pool has fewer than 256 * nsc elements");
        if (mixed) code |= DQ_RAND_BF16;
        rand_ptr = rand_pool->data_ptr();
    }
    if (recv.has_value()) {
        TORCH_CHECK(recv->device().type() == torch::kCUDA && recv->dtype() == torch::kUInt8 && recv->is_contiguous(),
                    "recv must be a contiguous torch.uint8 CUDA tensor");
        TORCH_CHECK(recv->numel() >= need, "recv buffer is smaller than mixed_required_bytes(nsc, ring_world)");
        recv_ptr = recv->data_ptr();
    }
    if (center_mean.has_value()) {
        TORCH_CHECK(center_mean->device().type() == torch::kCUDA && center_mean->dtype() == torch::kFloat32 &&
                        center_mean->is_contiguous() && center_mean->numel() >= nsc,
                    "center_mean must be a contiguous torch.float32 CUDA tensor with one entry per superchunk");
        TORCH_CHECK(center_world > 0, "center_world must be positive");
        TORCH_CHECK(n > 0 && (n + 255) / 256 <= nsc, "n must lie in [1, 256 * nsc]");
        TORCH_CHECK(src.numel() >= n, "input has fewer than n elements");
        mean_ptr = center_mean->data_ptr<float>();
    } else {
        TORCH_CHECK(src.numel() >= nsc * 256, "input has fewer than 256 * nsc elements");
    }
    check_status(dq_mixed_compress(src.data_ptr(), mean_ptr, center_world, n, order.data_ptr<int32_t>(), counts.data_ptr<int32_t>(),
                                   ring_chunk, ring_world, static_cast<const uint8_t *>(recv_ptr), dst.data_ptr<uint8_t>(), rand_ptr,
                                   seed, step, nsc, code, src.device().index(), strategy, as_stream(stream_p)),
                 "mixed_compress");
}

void mixed_decompress(torch::Tensor src, torch::Tensor dst, torch::Tensor order, torch::Tensor counts, int64_t nsc,
                      c10::optional<torch::Tensor> stats, int64_t n_limit, int ring_chunk = 0, int ring_world = 1,
                      uint64_t stream_p = 0, int strategy = 2)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(src.dtype() == torch::kUInt8, "input must be torch.uint8");
    TORCH_CHECK(dst.scalar_type() == torch::kBFloat16 || dst.scalar_type() == torch::kFloat32, "output must be torch.bfloat16 or torch.float32");
    TORCH_CHECK(src.is_contiguous() && dst.is_contiguous(), "buffers must be contiguous");
    TORCH_CHECK(strategy == 2 || strategy == 3, "strategy must be 2 or 3");
    TORCH_CHECK(ring_world > 0 && ring_chunk >= 0 && ring_chunk < ring_world, "ring_chunk must lie in [0, ring_world)");
    check_plan_tensors(order, counts, nsc);
    TORCH_CHECK(src.numel() >= dq_mixed_required_bytes(nsc, ring_world), "input buffer is smaller than mixed_required_bytes(nsc, ring_world)");
    TORCH_CHECK(n_limit > 0 && n_limit <= dst.numel() && n_limit <= nsc * 256, "n_limit must be in (0, min(output elements, 256 * nsc)]");
    const void *stats_ptr = nullptr;
    if (stats.has_value()) {
        TORCH_CHECK(stats->device().type() == torch::kCUDA && stats->dtype() == torch::kBFloat16 && stats->is_contiguous(),
                    "stats must be a contiguous torch.bfloat16 CUDA tensor");
        TORCH_CHECK(stats->numel() >= 2 * nsc, "stats buffer is too small");
        stats_ptr = stats->data_ptr();
    }
    check_status(dq_mixed_decompress(src.data_ptr<uint8_t>(), dst.data_ptr(), order.data_ptr<int32_t>(), counts.data_ptr<int32_t>(),
                                     ring_chunk, ring_world, stats_ptr, n_limit, nsc, dq_dtype_of(dst.scalar_type()),
                                     dst.device().index(), strategy, as_stream(stream_p)),
                 "mixed_decompress");
}

void superchunk_stats(torch::Tensor src, torch::Tensor stats, c10::optional<torch::Tensor> mean, int64_t n, int world_size,
                      uint64_t stream_p = 0)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA && stats.device().type() == torch::kCUDA, "src and stats must be CUDA tensors");
    TORCH_CHECK(is_supported_data_dtype(src.scalar_type(), true), "src must be torch.float16, torch.bfloat16 or torch.float32");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(src.is_contiguous() && stats.is_contiguous(), "buffers must be contiguous");
    TORCH_CHECK(n > 0, "n must be positive");
    TORCH_CHECK(world_size > 0, "world_size must be positive");
    TORCH_CHECK(src.numel() >= n, "src has fewer than n elements");
    const int64_t nsc = (n + 255) / 256;
    TORCH_CHECK(stats.numel() >= 2 * nsc, "stats buffer is too small");
    float *mean_ptr = nullptr;
    if (mean.has_value()) {
        TORCH_CHECK(mean->device().type() == torch::kCUDA && mean->dtype() == torch::kFloat32 && mean->is_contiguous() &&
                        mean->numel() >= nsc,
                    "mean must be a contiguous torch.float32 CUDA tensor with one entry per superchunk");
        mean_ptr = mean->data_ptr<float>();
    }
    check_status(dq_superchunk_stats(src.data_ptr(), stats.data_ptr(), mean_ptr, n, world_size, dq_dtype_of(src.scalar_type()),
                                     src.device().index(), as_stream(stream_p)),
                 "superchunk_stats");
}

// One bucket of the dynamic-bitrate path as one call: any run of the stages statistics (1) -> plan (2) -> mixed
// compress (4) -> mixed decompress (8).  The arguments of a stage that is not asked for are not looked at.
void dynamic_bitrate_bucket(torch::Tensor src, int64_t n, torch::Tensor stats, torch::Tensor mean, torch::Tensor order,
                            torch::Tensor work, torch::Tensor packed, c10::optional<torch::Tensor> out, double u,
                            c10::optional<torch::Tensor> u_dev, int stages = 15, c10::optional<torch::Tensor> reduced_stats = c10::nullopt,
                            int center_world = 1, int ring_chunk = 0, int ring_world = 1,
                            c10::optional<torch::Tensor> recv = c10::nullopt, c10::optional<torch::Tensor> hist = c10::nullopt,
                            uint64_t seed = 0, uint64_t step = 0, c10::optional<torch::Tensor> step_dev = c10::nullopt,
                            uint64_t stream_p = 0, int strategy = 2)
{
    auto dev_ok = [&](const torch::Tensor &t) { return t.device() == src.device() && t.is_contiguous(); };
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(src.scalar_type() == torch::kBFloat16 || src.scalar_type() == torch::kFloat32, "input must be torch.bfloat16 or torch.float32");
    TORCH_CHECK(src.is_contiguous(), "buffers must be contiguous");
    TORCH_CHECK(n > 0 && src.numel() >= n, "n must be positive and at most the number of input elements");
    TORCH_CHECK(strategy == 2 || strategy == 3, "strategy must be 2 or 3");
    TORCH_CHECK(stages > 0 && stages <= 15, "stages must be a combination of 1 (statistics), 2 (plan), 4 (compress), 8 (decompress)");
    TORCH_CHECK(ring_world > 0 && ring_chunk >= 0 && ring_chunk < ring_world, "ring_chunk must lie in [0, ring_world)");
    TORCH_CHECK(center_world > 0, "center_world must be positive");
    const int64_t nsc = (n + 255) / 256;
    TORCH_CHECK(dev_ok(stats) && stats.dtype() == torch::kBFloat16 && stats.numel() >= 2 * nsc, "stats must be a contiguous torch.bfloat16 tensor with a (mean, norm) pair per superchunk on the device of the input");
    TORCH_CHECK(dev_ok(mean) && mean.dtype() == torch::kFloat32 && mean.numel() >= nsc, "mean must be a contiguous torch.float32 tensor with one entry per superchunk on the device of the input");
    TORCH_CHECK(dev_ok(order) && order.dtype() == torch::kInt32 && order.numel() >= 3 * nsc, "order must be a contiguous torch.int32 tensor with 3 * nsc entries on the device of the input");
    TORCH_CHECK(dev_ok(work) && work.dtype() == torch::kInt32 && work.numel() >= dq_group_plan_work_ints(nsc), "work must be a contiguous torch.int32 tensor with group_plan_work_ints(nsc) entries on the device of the input");
    TORCH_CHECK(dev_ok(packed) && packed.dtype() == torch::kUInt8 && packed.numel() >= dq_mixed_required_bytes(nsc, ring_world), "packed must be a contiguous torch.uint8 tensor of mixed_required_bytes(nsc, ring_world) bytes on the device of the input");
    dq_bucket_t b;
    memset(&b, 0, sizeof(b));
    b.src = src.data_ptr();
    b.n = n;
    b.dtype = dq_dtype_of(src.scalar_type());
    b.strategy = strategy;
    b.center_world = center_world;
    b.ring_chunk = ring_chunk;
    b.ring_world = ring_world;
    b.u = u;
    if (u_dev.has_value()) {
        TORCH_CHECK(dev_ok(*u_dev) && u_dev->dtype() == torch::kFloat64 && u_dev->numel() >= 1, "u_dev must be a torch.float64 tensor on the device of the input");
        b.u_dev = u_dev->data_ptr<double>();
    }
    b.stats = stats.data_ptr();
    b.mean = mean.data_ptr<float>();
    if (reduced_stats.has_value()) {
        TORCH_CHECK(dev_ok(*reduced_stats) && reduced_stats->dtype() == torch::kBFloat16 && reduced_stats->numel() >= 2 * nsc, "reduced_stats must be a contiguous torch.bfloat16 tensor like stats");
        b.reduced_stats = reduced_stats->data_ptr();
    }
    b.order = order.data_ptr<int32_t>();
    b.work = work.data_ptr<int32_t>();
    b.work_ints = work.numel();
    if (recv.has_value()) {
        TORCH_CHECK(dev_ok(*recv) && recv->dtype() == torch::kUInt8 && recv->numel() >= dq_mixed_required_bytes(nsc, ring_world), "recv must be a contiguous torch.uint8 tensor of mixed_required_bytes(nsc, ring_world) bytes");
        b.recv = recv->data_ptr<uint8_t>();
    }
    b.packed = packed.data_ptr<uint8_t>();
    b.packed_bytes = packed.numel();
    if (out.has_value()) {
        TORCH_CHECK(dev_ok(*out) && out->dtype() == src.dtype() && out->numel() >= n, "out must be a contiguous tensor of the input's dtype with at least n elements");
        b.out = out->data_ptr();
    }
    TORCH_CHECK(!(stages & 8) || out.has_value(), "the decompress stage needs out");
    if (hist.has_value()) {
        TORCH_CHECK(dev_ok(*hist) && hist->dtype() == torch::kInt32 && hist->numel() >= dq_bitrate_hist_ints(), "hist must be a contiguous torch.int32 tensor with bitrate_hist_ints() entries");
        b.hist = reinterpret_cast<uint32_t *>(hist->data_ptr<int32_t>());
        b.hist_ints = hist->numel();
    }
    b.seed = seed;
    b.step = step;
    if (step_dev.has_value()) {
        TORCH_CHECK(dev_ok(*step_dev) && step_dev->dtype() == torch::kInt64 && step_dev->numel() >= 1, "step_dev must be a torch.int64 tensor on the device of the input");
        b.step_dev = reinterpret_cast<const uint64_t *>(step_dev->data_ptr<int64_t>());
    }
    check_status(dq_dynamic_bitrate_bucket(&b, stages, src.device().index(), as_stream(stream_p)), "dynamic_bitrate_bucket");
}

// ---- superchunk ops ---------------------------------------------------------------

void superchunk_mean_center(torch::Tensor src, torch::Tensor residual, torch::Tensor stats, int n, int world_size,
                            int superchunk_size = 256, uint64_t stream_p = 0)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "src must be a CUDA tensor");
    TORCH_CHECK(residual.device().type() == torch::kCUDA, "residual must be a CUDA tensor");
    TORCH_CHECK(stats.device().type() == torch::kCUDA, "stats must be a CUDA tensor");
    TORCH_CHECK(residual.device() == src.device(), "residual must be on the same CUDA device as src");
    TORCH_CHECK(stats.device() == src.device(), "stats must be on the same CUDA device as src");
    TORCH_CHECK(is_supported_data_dtype(src.scalar_type(), false), "src must be torch.float16 or torch.bfloat16");
    TORCH_CHECK(residual.scalar_type() == src.scalar_type(), "residual dtype must match src dtype");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(src.is_contiguous(), "src must be contiguous");
    TORCH_CHECK(residual.is_contiguous(), "residual must be contiguous");
    TORCH_CHECK(stats.is_contiguous(), "stats must be contiguous");
    TORCH_CHECK(n > 0, "n must be positive");
    TORCH_CHECK(world_size > 0, "world_size must be positive");
    TORCH_CHECK(superchunk_size == 256, "superchunk_size must be 256");
    TORCH_CHECK(src.numel() >= n, "src has fewer than n elements");
    const int64_t num_superchunks = superchunk_num_chunks(n, superchunk_size);
    TORCH_CHECK(residual.numel() >= num_superchunks * superchunk_size, "residual buffer is too small");
    TORCH_CHECK(stats.numel() >= num_superchunks * 2, "stats buffer is too small");
    check_status(dq_superchunk_mean_center(src.data_ptr(), residual.data_ptr(), stats.data_ptr(), n, world_size, superchunk_size,
                                           dq_dtype_of(src.scalar_type()), src.device().index(), as_stream(stream_p)),
                 "superchunk_mean_center");
}

void superchunk_add_mean_copy(torch::Tensor residual, torch::Tensor dst, torch::Tensor stats, int n, int superchunk_size = 256,
                              uint64_t stream_p = 0)
{
    TORCH_CHECK(residual.device().type() == torch::kCUDA, "residual must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "dst must be a CUDA tensor");
    TORCH_CHECK(stats.device().type() == torch::kCUDA, "stats must be a CUDA tensor");
    TORCH_CHECK(dst.device() == residual.device(), "dst must be on the same CUDA device as residual");
    TORCH_CHECK(stats.device() == residual.device(), "stats must be on the same CUDA device as residual");
    TORCH_CHECK(is_supported_data_dtype(residual.scalar_type(), false), "residual must be torch.float16 or torch.bfloat16");
    TORCH_CHECK(dst.scalar_type() == residual.scalar_type(), "dst dtype must match residual dtype");
    TORCH_CHECK(stats.dtype() == torch::kBFloat16, "stats must be torch.bfloat16");
    TORCH_CHECK(residual.is_contiguous(), "residual must be contiguous");
    TORCH_CHECK(dst.is_contiguous(), "dst must be contiguous");
    TORCH_CHECK(stats.is_contiguous(), "stats must be contiguous");
    TORCH_CHECK(n > 0, "n must be positive");
    TORCH_CHECK(superchunk_size == 256, "superchunk_size must be 256");
    TORCH_CHECK(dst.numel() >= n, "dst has fewer than n elements");
    const int64_t num_superchunks = superchunk_num_chunks(n, superchunk_size);
    TORCH_CHECK(residual.numel() >= num_superchunks * superchunk_size, "residual buffer is too small");
    TORCH_CHECK(stats.numel() >= num_superchunks * 2, "stats buffer is too small");
    check_status(dq_superchunk_add_mean_copy(residual.data_ptr(), dst.data_ptr(), stats.data_ptr(), n, superchunk_size,
                                             dq_dtype_of(residual.scalar_type()), residual.device().index(), as_stream(stream_p)),
                 "superchunk_add_mean_copy");
}

// ---- EDEN bit-plane packing (default stream, fresh outputs, as the reference) -------

torch::Tensor EdenBinsToBits(torch::Tensor bins, int nbits)
{
    TORCH_CHECK(bins.device().type() == torch::kCUDA, "bins must be a CUDA tensor");
    TORCH_CHECK(bins.dtype() == torch::kInt32, "bins must be a torch.int32 CUDA tensor");
    auto nbins = bins.size(-1);
    TORCH_CHECK(nbins == bins.numel(), "bins must be 1D");
    TORCH_CHECK((nbins & 31) == 0, "bins size must be a multiple of 32");
    auto cbins = on_stream(bins.clone(), 0);
    const int device = cbins.device().index();
    auto opts = torch::TensorOptions().device(bins.device().type(), device).dtype(torch::kInt32);
    torch::Tensor carr = on_stream(torch::zeros({(nbins >> 5) * nbits}, opts), 0);
    if (nbins > 0)
        check_status(dq_bins_to_bits(cbins.data_ptr<int32_t>(), nbins, reinterpret_cast<uint32_t *>(carr.data_ptr<int32_t>()),
                                     (nbins >> 5) * nbits, nbits, device, nullptr),
                     "EdenBinsToBits");
    return carr;
}

torch::Tensor EdenBitsToBins(torch::Tensor arr, int nbits)
{
    TORCH_CHECK(arr.device().type() == torch::kCUDA, "arr must be a CUDA tensor");
    TORCH_CHECK(arr.dtype() == torch::kInt32, "arr must be a torch.int32 CUDA tensor");
    auto narr = arr.size(-1);
    TORCH_CHECK(narr == arr.numel(), "arr must be 1D");
    auto carr = on_stream(arr.clone(), 0);
    const int device = carr.device().index();
    auto opts = torch::TensorOptions().device(arr.device().type(), device).dtype(torch::kInt32);
    const int64_t nbins = (narr / nbits) << 5;
    torch::Tensor cbins = on_stream(torch::zeros({nbins}, opts), 0);
    if (nbins > 0)
        check_status(dq_bits_to_bins(cbins.data_ptr<int32_t>(), nbins, reinterpret_cast<const uint32_t *>(carr.data_ptr<int32_t>()),
                                     (nbins >> 5) * nbits, nbits, device, nullptr),
                     "EdenBitsToBins");
    return cbins;
}

// ---- in-kernel random stream (additions; see include/dynamiq_eden.h) ------------------------

void scaling_compress_philox(torch::Tensor src, torch::Tensor dst, int64_t n, int nbits, int chunk_size, uint64_t seed,
                             uint64_t step, uint64_t stream_p = 0, int strategy = 0)
{
    TORCH_CHECK(src.device().type() == torch::kCUDA, "input must be a CUDA tensor");
    TORCH_CHECK(dst.device().type() == torch::kCUDA, "output must be a CUDA tensor");
    TORCH_CHECK(is_supported_data_dtype(src.scalar_type(), true), "input must be torch.float16, torch.bfloat16 or torch.float32");
    TORCH_CHECK(dst.dtype() == torch::kUInt8, "output must be torch.uint8");
    TORCH_CHECK(src.is_contiguous(), "input must be contiguous");
    TORCH_CHECK(dst.is_contiguous(), "output must be contiguous");
    scaling_check_common((int)n, nbits, chunk_size, strategy, true);
    TORCH_CHECK(chunk_size == 16, "the in-kernel random stream is defined for chunk_size 16");
    TORCH_CHECK(src.numel() >= n, "input has fewer than n elements");
    TORCH_CHECK(dst.numel() >= dq_scaling_required_bytes(n, nbits, chunk_size, strategy), "output buffer is too small");
    check_status(dq_scaling_compress_philox(src.data_ptr(), dst.data_ptr<uint8_t>(), n, nbits, chunk_size,
                                            dq_dtype_of(src.scalar_type()), src.device().index(), strategy, seed, step,
                                            as_stream(stream_p)),
                 "scaling_compress_philox");
}

void scaling_dec_comp_philox(torch::Tensor recv, torch::Tensor inp, torch::Tensor send, int64_t n, int nbits, int chunk_size,
                             uint64_t seed, uint64_t step, uint64_t stream_p = 0, int strategy = 0)
{
    TORCH_CHECK(recv.device().type() == torch::kCUDA && inp.device().type() == torch::kCUDA && send.device().type() == torch::kCUDA,
                "all buffers must be CUDA tensors");
    TORCH_CHECK(recv.dtype() == torch::kUInt8, "recv must be torch.uint8");
    TORCH_CHECK(send.dtype() == torch::kUInt8, "send must be torch.uint8");
    TORCH_CHECK(is_supported_data_dtype(inp.scalar_type(), true), "inp must be torch.float16, torch.bfloat16 or torch.float32");
    TORCH_CHECK(recv.is_contiguous() && inp.is_contiguous() && send.is_contiguous(), "buffers must be contiguous");
    scaling_check_common((int)n, nbits, chunk_size, strategy, true);
    TORCH_CHECK(chunk_size == 16, "the in-kernel random stream is defined for chunk_size 16");
    const int64_t required_bytes = dq_scaling_required_bytes(n, nbits, chunk_size, strategy);
    TORCH_CHECK(recv.numel() >= required_bytes, "recv buffer is too small");
    TORCH_CHECK(send.numel() >= required_bytes, "send buffer is too small");
    TORCH_CHECK(inp.numel() >= n, "inp has fewer than n elements");
    check_status(dq_scaling_dec_comp_philox(recv.data_ptr<uint8_t>(), inp.data_ptr(), send.data_ptr<uint8_t>(), n, nbits, chunk_size,
                                            dq_dtype_of(inp.scalar_type()), inp.device().index(), strategy, seed, step,
                                            as_stream(stream_p)),
                 "scaling_dec_comp_philox");
}

void philox_uniform(torch::Tensor out, uint64_t seed, uint64_t step, uint64_t stream_p = 0)
{
    TORCH_CHECK(out.device().type() == torch::kCUDA, "out must be a CUDA tensor");
    TORCH_CHECK(is_supported_data_dtype(out.scalar_type(), true), "out must be torch.float16, torch.bfloat16 or torch.float32");
    TORCH_CHECK(out.is_contiguous() && out.numel() > 0, "out must be contiguous and not empty");
    check_status(dq_philox_uniform(out.data_ptr(), out.numel(), dq_dtype_of(out.scalar_type()), out.device().index(), seed, step,
                                   as_stream(stream_p)),
                 "philox_uniform");
}

// ---- EDEN / THC consumers (additions; see include/dynamiq_eden.h) --------------------------

void check_f32_cuda(const torch::Tensor &t, const char *name)
{
    TORCH_CHECK(t.device().type() == torch::kCUDA, name, " must be a CUDA tensor");
    TORCH_CHECK(t.dtype() == torch::kFloat32, name, " must be torch.float32");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// returns (packed int32 [n / 32 * nbits], result float32 [4] = sum of squares, dot, scale, norm)
std::vector<torch::Tensor> eden_quantize(torch::Tensor vec, torch::Tensor boundaries, torch::Tensor centroids, int nbits,
                                         uint64_t stream_p = 0)
{
    check_f32_cuda(vec, "vec");
    check_f32_cuda(boundaries, "boundaries");
    check_f32_cuda(centroids, "centroids");
    TORCH_CHECK(nbits >= 1 && nbits <= 8, "nbits must be in [1, 8]");
    const int64_t n = vec.numel();
    TORCH_CHECK(n > 0 && (n & 31) == 0, "vec size must be a positive multiple of 32");
    TORCH_CHECK(boundaries.numel() == (1 << nbits) - 1, "boundaries must hold 2^nbits - 1 values");
    TORCH_CHECK(centroids.numel() == (1 << nbits), "centroids must hold 2^nbits values");
    auto packed = on_stream(torch::empty({n / 32 * nbits}, vec.options().dtype(torch::kInt32)), stream_p);
    auto result = on_stream(torch::empty({4}, vec.options()), stream_p);
    auto work = on_stream(torch::empty({dq_eden_work_doubles(n)}, vec.options().dtype(torch::kFloat64)), stream_p);
    check_status(dq_eden_quantize(vec.data_ptr<float>(), n, boundaries.data_ptr<float>(), centroids.data_ptr<float>(), nbits,
                                  reinterpret_cast<uint32_t *>(packed.data_ptr<int32_t>()), result.data_ptr<float>(),
                                  work.data_ptr<double>(), work.numel(), vec.device().index(), as_stream(stream_p)),
                 "eden_quantize");
    return {packed, result};
}

torch::Tensor eden_dequantize(torch::Tensor packed, torch::Tensor centroids, int nbits, uint64_t stream_p = 0)
{
    TORCH_CHECK(packed.device().type() == torch::kCUDA && packed.dtype() == torch::kInt32 && packed.is_contiguous(),
                "packed must be a contiguous torch.int32 CUDA tensor");
    check_f32_cuda(centroids, "centroids");
    TORCH_CHECK(nbits >= 1 && nbits <= 8, "nbits must be in [1, 8]");
    TORCH_CHECK(packed.numel() > 0 && packed.numel() % nbits == 0, "packed size must be a multiple of nbits");
    TORCH_CHECK(centroids.numel() == (1 << nbits), "centroids must hold 2^nbits values");
    const int64_t n = packed.numel() / nbits * 32;
    auto out = on_stream(torch::empty({n}, centroids.options()), stream_p);
    check_status(dq_eden_dequantize(reinterpret_cast<const uint32_t *>(packed.data_ptr<int32_t>()), n, centroids.data_ptr<float>(),
                                    nbits, out.data_ptr<float>(), packed.device().index(), as_stream(stream_p)),
                 "eden_dequantize");
    return out;
}

torch::Tensor eden_dequantize_irht(torch::Tensor packed, torch::Tensor centroids, int nbits, c10::optional<torch::Tensor> sign,
                                   int64_t block, double scale, c10::optional<torch::Tensor> post_scale, uint64_t stream_p = 0)
{
    TORCH_CHECK(packed.device().type() == torch::kCUDA && packed.dtype() == torch::kInt32 && packed.is_contiguous(),
                "packed must be a contiguous torch.int32 CUDA tensor");
    check_f32_cuda(centroids, "centroids");
    TORCH_CHECK(nbits >= 1 && nbits <= 8, "nbits must be in [1, 8]");
    TORCH_CHECK(packed.numel() > 0 && packed.numel() % nbits == 0, "packed size must be a multiple of nbits");
    TORCH_CHECK(centroids.numel() == (1 << nbits), "centroids must hold 2^nbits values");
    const int64_t n = packed.numel() / nbits * 32;
    auto out = on_stream(torch::empty({n}, centroids.options()), stream_p);
    int sign_packed = 0;
    const void *sp = sign_arg(sign, out, n, &sign_packed);
    const float *ps = nullptr;
    if (post_scale.has_value()) {
        check_f32_cuda(*post_scale, "post_scale");
        TORCH_CHECK(post_scale->numel() == 1, "post_scale must hold one value");
        ps = post_scale->data_ptr<float>();
    }
    check_status(dq_eden_dequantize_irht(reinterpret_cast<const uint32_t *>(packed.data_ptr<int32_t>()), n, centroids.data_ptr<float>(),
                                         nbits, sp, sign_packed, out.data_ptr<float>(), block, (float)scale, ps,
                                         packed.device().index(), as_stream(stream_p)),
                 "eden_dequantize_irht");
    return out;
}

torch::Tensor thc_quantize(torch::Tensor rotated, torch::Tensor uniform, torch::Tensor lo, torch::Tensor delta, int levels,
                           uint64_t stream_p = 0)
{
    check_f32_cuda(rotated, "rotated");
    check_f32_cuda(uniform, "uniform");
    check_f32_cuda(lo, "lo");
    check_f32_cuda(delta, "delta");
    TORCH_CHECK(uniform.numel() >= rotated.numel(), "uniform has fewer elements than rotated");
    TORCH_CHECK(lo.numel() == 1 && delta.numel() == 1, "lo and delta must hold one value");
    TORCH_CHECK(levels >= 2 && levels <= 256, "levels must be in [2, 256]");
    auto out = on_stream(torch::empty({rotated.numel()}, rotated.options().dtype(torch::kBFloat16)), stream_p);
    check_status(dq_thc_quantize(rotated.data_ptr<float>(), uniform.data_ptr<float>(), out.data_ptr(), rotated.numel(),
                                 lo.data_ptr<float>(), delta.data_ptr<float>(), levels, rotated.device().index(),
                                 as_stream(stream_p)),
                 "thc_quantize");
    return out;
}

void thc_dequantize(torch::Tensor levels, torch::Tensor out, torch::Tensor step, torch::Tensor lo, uint64_t stream_p = 0)
{
    TORCH_CHECK(levels.device().type() == torch::kCUDA && levels.dtype() == torch::kBFloat16 && levels.is_contiguous(),
                "levels must be a contiguous torch.bfloat16 CUDA tensor");
    check_f32_cuda(out, "out");
    check_f32_cuda(step, "step");
    check_f32_cuda(lo, "lo");
    TORCH_CHECK(out.numel() >= levels.numel(), "out has fewer elements than levels");
    TORCH_CHECK(step.numel() == 1 && lo.numel() == 1, "step and lo must hold one value");
    check_status(dq_thc_dequantize(levels.data_ptr(), out.data_ptr<float>(), levels.numel(), step.data_ptr<float>(),
                                   lo.data_ptr<float>(), levels.device().index(), as_stream(stream_p)),
                 "thc_dequantize");
}

void thc_rht_quantize(torch::Tensor work, c10::optional<torch::Tensor> sign, torch::Tensor uniform, torch::Tensor levels_out,
                      int64_t block, double scale, torch::Tensor lo, torch::Tensor delta, int levels, uint64_t stream_p = 0)
{
    check_f32_cuda(work, "work");
    check_f32_cuda(uniform, "uniform");
    check_f32_cuda(lo, "lo");
    check_f32_cuda(delta, "delta");
    TORCH_CHECK(levels_out.device().type() == torch::kCUDA && levels_out.dtype() == torch::kBFloat16 && levels_out.is_contiguous(),
                "levels_out must be a contiguous torch.bfloat16 CUDA tensor");
    const int64_t n = work.numel();
    TORCH_CHECK(uniform.numel() >= n && levels_out.numel() >= n, "uniform or levels_out has fewer elements than work");
    TORCH_CHECK(lo.numel() == 1 && delta.numel() == 1, "lo and delta must hold one value");
    int packed = 0;
    const void *sp = sign_arg(sign, work, n, &packed);
    check_status(dq_thc_rht_quantize(work.data_ptr<float>(), sp, packed, uniform.data_ptr<float>(), levels_out.data_ptr(), n,
                                     block, (float)scale, lo.data_ptr<float>(), delta.data_ptr<float>(), levels,
                                     work.device().index(), as_stream(stream_p)),
                 "thc_rht_quantize");
}

void thc_dequantize_irht(torch::Tensor levels, c10::optional<torch::Tensor> sign, torch::Tensor out, int64_t block, double scale,
                         torch::Tensor step, torch::Tensor lo, uint64_t stream_p = 0)
{
    TORCH_CHECK(levels.device().type() == torch::kCUDA && levels.dtype() == torch::kBFloat16 && levels.is_contiguous(),
                "levels must be a contiguous torch.bfloat16 CUDA tensor");
    check_f32_cuda(out, "out");
    check_f32_cuda(step, "step");
    check_f32_cuda(lo, "lo");
    const int64_t n = out.numel();
    TORCH_CHECK(levels.numel() >= n, "levels has fewer elements than out");
    TORCH_CHECK(step.numel() == 1 && lo.numel() == 1, "step and lo must hold one value");
    int packed = 0;
    const void *sp = sign_arg(sign, out, n, &packed);
    check_status(dq_thc_dequantize_irht(levels.data_ptr(), sp, packed, out.data_ptr<float>(), n, block, (float)scale,
                                        step.data_ptr<float>(), lo.data_ptr<float>(), out.device().index(), as_stream(stream_p)),
                 "thc_dequantize_irht");
}

void init_lookup_table() { check_status(dq_init_lookup_table(), "init_lookup_table"); }

std::string abi_version() { return dq_version(); }

} // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, modul)
{
    modul.def("Hadamard", &Hadamard, "fast Hadamard transform", py::arg("vec"), py::arg("stream_p") = 0, py::arg("depth") = 0);
    modul.def("EdenBinsToBits", &EdenBinsToBits, "EDEN's packing bins to bits");
    modul.def("EdenBitsToBins", &EdenBitsToBins, "EDEN's unpacking bits to bins");
    modul.def("Hadamard_init", &Hadamard_init, "hadamard init", py::arg("vec"));
    modul.def("Hadamard_init_ptr", &Hadamard_init_ptr, "hadamard init", py::arg("vec"), py::arg("device") = 0);
    modul.def("Hadamard_inplace", &Hadamard_inplace, "fast Hadamard transform", py::arg("vec"), py::arg("stream_p") = 0, py::arg("depth") = 0);
    modul.def("Hadamard_inplace_ptr", &Hadamard_inplace_ptr, "fast Hadamard transform", py::arg("vec"), py::arg("n"), py::arg("device"), py::arg("stream_p") = 0, py::arg("depth") = 0);
    modul.def("quantization_compression", &quantization_compression, "quantization compression", py::arg("vec"), py::arg("div_factor"), py::arg("tensor_max"), py::arg("stream_p") = 0);
    modul.def("scaling_compress", &scaling_compress, "scaling compress", py::arg("src"), py::arg("dst"), py::arg("rand_pool"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_decompress", &scaling_decompress, "scaling decompress", py::arg("src"), py::arg("dst"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_decompress_add", &scaling_decompress_add, "scaling decompress and add", py::arg("src"), py::arg("dst"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_dec_comp", &scaling_dec_comp, "scaling decompress and compress", py::arg("recv"), py::arg("inp"), py::arg("send"), py::arg("rand_pool"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("superchunk_mean_center", &superchunk_mean_center, "mean-center 256-element superchunks and write per-superchunk mean/norm stats", py::arg("src"), py::arg("residual"), py::arg("stats"), py::arg("n"), py::arg("world_size"), py::arg("superchunk_size") = 256, py::arg("stream_p") = 0);
    modul.def("superchunk_add_mean_copy", &superchunk_add_mean_copy, "add reduced per-superchunk means to residuals and copy back valid elements", py::arg("residual"), py::arg("dst"), py::arg("stats"), py::arg("n"), py::arg("superchunk_size") = 256, py::arg("stream_p") = 0);
    modul.def("init_lookup_table", &init_lookup_table, "init lookup table");

    // additions
    modul.def("scaling_compress_ex", &scaling_compress_ex, "scaling compress (also float32 buffers, 2..8-bit codes)", py::arg("src"), py::arg("dst"), py::arg("rand_pool"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_decompress_ex", &scaling_decompress_ex, "scaling decompress (also float32 buffers, 2..8-bit codes)", py::arg("src"), py::arg("dst"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_decompress_add_ex", &scaling_decompress_add_ex, "scaling decompress and add (also float32 buffers, 2..8-bit codes)", py::arg("src"), py::arg("dst"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_dec_comp_ex", &scaling_dec_comp_ex, "scaling decompress and compress (also float32 buffers, 2..8-bit codes)", py::arg("recv"), py::arg("inp"), py::arg("send"), py::arg("rand_pool"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_required_bytes", &scaling_required_bytes, "packed size in bytes", py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("strategy"));
    modul.def("rht_blocked", &rht_blocked, "in-place blocked randomized Hadamard transform", py::arg("vec"), py::arg("sign"), py::arg("block"), py::arg("scale"), py::arg("inverse") = false, py::arg("stream_p") = 0);
    modul.def("pack_signs", &pack_signs, "+-1 float32 vector -> int32 bit vector (bit set where negative)", py::arg("sign"), py::arg("stream_p") = 0);
    modul.def("rht_scaling_compress", &rht_scaling_compress, "blocked randomized Hadamard transform + hierarchical chunk-16 compress in one launch (the rotated vector never reaches memory)", py::arg("src"), py::arg("sign"), py::arg("dst"), py::arg("block"), py::arg("scale"), py::arg("nbits"), py::arg("rand_pool") = py::none(), py::arg("seed") = 0, py::arg("step") = 0, py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("scaling_decompress_irht", &scaling_decompress_irht, "hierarchical chunk-16 decompress + inverse blocked randomized Hadamard transform in one launch", py::arg("src"), py::arg("sign"), py::arg("dst"), py::arg("block"), py::arg("scale"), py::arg("nbits"), py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("rand_diag", &rand_diag, "EDEN's seeded +-1 diagonal", py::arg("size"), py::arg("seed"), py::arg("device"), py::arg("stream_p") = 0);
    modul.def("rand_diag_bits", &rand_diag_bits, "EDEN's seeded +-1 diagonal as the int32 bit vector of pack_signs (bit set where the value is -1)", py::arg("size"), py::arg("seed"), py::arg("device"), py::arg("stream_p") = 0);
    modul.def("set_quantization_seed", &set_quantization_seed, "seed of quantization_compression's random stream", py::arg("seed"));
    modul.def("group_plan", &group_plan, "stable partition of superchunk indices by bit width into the three regions of order (8-bit rows from 0, 4-bit from nsc, 2-bit from 2 nsc); returns int32 [4] = counts of 8/4/2/other", py::arg("qbits"), py::arg("order"), py::arg("stream_p") = 0);
    modul.def("group_plan_stats", &group_plan_stats, "bit widths from the reduced bf16 norms and the offset u, and the partition by width, in one call; returns int32 [4] = counts of 8/4/2/other", py::arg("stats"), py::arg("u"), py::arg("order"), py::arg("qbits_out") = py::none(), py::arg("stream_p") = 0);
    modul.def("group_plan_sorted", &group_plan_sorted, "fixed-proportion groups: the first top_count superchunks of the stable descending sort of the norms in the 8-bit region of order, the last bottom_count in the 2-bit region, the rest in the 4-bit region, each in sorted order; returns int32 [4] = counts of 8/4/2/other", py::arg("stats"), py::arg("top_count"), py::arg("bottom_count"), py::arg("order"), py::arg("qbits_out") = py::none(), py::arg("stream_p") = 0);
    modul.def("group_plan_stats_dev_u", &group_plan_stats_dev_u, "group_plan_stats with the offset u read from a float64 device tensor when the kernels run; hist also gets the bucket's norm patterns", py::arg("stats"), py::arg("u"), py::arg("order"), py::arg("qbits_out") = py::none(), py::arg("hist") = py::none(), py::arg("stream_p") = 0);
    modul.def("bitrate_hist_ints", &bitrate_hist_ints, "int32 entries of the norm-pattern histogram");
    modul.def("norm_histogram", &norm_histogram, "adds the bf16 norm patterns of a bucket's statistics to the histogram", py::arg("stats"), py::arg("hist"), py::arg("stream_p") = 0);
    modul.def("bitrate_search", &bitrate_search, "the reference's search for the offset u (mode 0: bisection, 1: correction from prev_u) on the histogram, one launch; returns float64 [4] = u, average width, target - average, probes and leaves hist zeroed", py::arg("hist"), py::arg("mode"), py::arg("prev_u"), py::arg("target_avg_bits"), py::arg("stream_p") = 0);
    modul.def("scaling_compress_rows", &scaling_compress_rows, "compress the superchunks rows[k] of src into consecutive records", py::arg("src"), py::arg("rows"), py::arg("dst"), py::arg("rand_pool"), py::arg("nrows"), py::arg("nbits"), py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("scaling_dec_comp_rows", &scaling_dec_comp_rows, "fused ring step over the superchunks rows[k] of inp", py::arg("recv"), py::arg("inp"), py::arg("rows"), py::arg("send"), py::arg("rand_pool"), py::arg("nrows"), py::arg("nbits"), py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("scaling_decompress_rows", &scaling_decompress_rows, "decode consecutive records into the superchunks rows[k] of dst, optionally adding the per-superchunk mean", py::arg("src"), py::arg("dst"), py::arg("rows"), py::arg("stats"), py::arg("n_limit"), py::arg("nrows"), py::arg("nbits"), py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("mixed_required_bytes", &mixed_required_bytes, "upper bound of the packed stream of one ring chunk over the three bit-width groups", py::arg("nsc"), py::arg("ring_world") = 1);
    modul.def("mixed_compress", &mixed_compress, "compress (or, with recv, decode-accumulate-recompress) ring chunk ring_chunk of all three bit-width groups of a planned bucket in one launch", py::arg("src"), py::arg("order"), py::arg("counts"), py::arg("dst"), py::arg("nsc"), py::arg("rand_pool") = py::none(), py::arg("recv") = py::none(), py::arg("center_mean") = py::none(), py::arg("center_world") = 1, py::arg("n") = 0, py::arg("ring_chunk") = 0, py::arg("ring_world") = 1, py::arg("seed") = 0, py::arg("step") = 0, py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("mixed_decompress", &mixed_decompress, "decode ring chunk ring_chunk of all three bit-width groups into their superchunks of dst, optionally adding the per-superchunk mean", py::arg("src"), py::arg("dst"), py::arg("order"), py::arg("counts"), py::arg("nsc"), py::arg("stats"), py::arg("n_limit"), py::arg("ring_chunk") = 0, py::arg("ring_world") = 1, py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("dynamic_bitrate_bucket", &dynamic_bitrate_bucket, "one bucket of the dynamic-bitrate path in one call: any run of the stages statistics (1), plan (2), mixed compress (4), mixed decompress (8)", py::arg("src"), py::arg("n"), py::arg("stats"), py::arg("mean"), py::arg("order"), py::arg("work"), py::arg("packed"), py::arg("out"), py::arg("u") = 0.0, py::arg("u_dev") = py::none(), py::arg("stages") = 15, py::arg("reduced_stats") = py::none(), py::arg("center_world") = 1, py::arg("ring_chunk") = 0, py::arg("ring_world") = 1, py::arg("recv") = py::none(), py::arg("hist") = py::none(), py::arg("seed") = 0, py::arg("step") = 0, py::arg("step_dev") = py::none(), py::arg("stream_p") = 0, py::arg("strategy") = 2);
    modul.def("superchunk_stats", &superchunk_stats, "the statistics of superchunk_mean_center without the residual, plus the unrounded float32 means", py::arg("src"), py::arg("stats"), py::arg("mean"), py::arg("n"), py::arg("world_size"), py::arg("stream_p") = 0);
    modul.def("scaling_compress_philox", &scaling_compress_philox, "scaling compress with the uniform values drawn in the kernel (Philox: key = seed, counter = chunk, step)", py::arg("src"), py::arg("dst"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("seed"), py::arg("step"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("scaling_dec_comp_philox", &scaling_dec_comp_philox, "scaling decompress and compress with the uniform values drawn in the kernel", py::arg("recv"), py::arg("inp"), py::arg("send"), py::arg("n"), py::arg("nbits"), py::arg("chunk_size"), py::arg("seed"), py::arg("step"), py::arg("stream_p") = 0, py::arg("strategy") = 0);
    modul.def("philox_uniform", &philox_uniform, "the uniform values of that stream written out as a tensor", py::arg("out"), py::arg("seed"), py::arg("step"), py::arg("stream_p") = 0);
    modul.def("eden_quantize", &eden_quantize, "EDEN: normalise, bucketize against the Lloyd-Max boundaries, pack bit planes, scale; returns [packed, result]", py::arg("vec"), py::arg("boundaries"), py::arg("centroids"), py::arg("nbits"), py::arg("stream_p") = 0);
    modul.def("eden_dequantize", &eden_dequantize, "EDEN: centroids of the packed bins", py::arg("packed"), py::arg("centroids"), py::arg("nbits"), py::arg("stream_p") = 0);
    modul.def("eden_dequantize_irht", &eden_dequantize_irht, "EDEN: centroids of the packed bins rotated back (inverse blocked transform) and multiplied by post_scale, without the dequantised vector reaching memory", py::arg("packed"), py::arg("centroids"), py::arg("nbits"), py::arg("sign"), py::arg("block"), py::arg("scale"), py::arg("post_scale") = py::none(), py::arg("stream_p") = 0);
    modul.def("thc_quantize", &thc_quantize, "THC: uniform stochastic quantiser of the rotated vector, bfloat16 levels", py::arg("rotated"), py::arg("uniform"), py::arg("lo"), py::arg("delta"), py::arg("levels"), py::arg("stream_p") = 0);
    modul.def("thc_dequantize", &thc_dequantize, "THC: out = float(levels) * step + lo", py::arg("levels"), py::arg("out"), py::arg("step"), py::arg("lo"), py::arg("stream_p") = 0);
    modul.def("thc_rht_quantize", &thc_rht_quantize, "THC: blocked randomized Hadamard transform whose last pass stores the quantiser's levels (work is scratch afterwards)", py::arg("work"), py::arg("sign"), py::arg("uniform"), py::arg("levels_out"), py::arg("block"), py::arg("scale"), py::arg("lo"), py::arg("delta"), py::arg("levels"), py::arg("stream_p") = 0);
    modul.def("thc_dequantize_irht", &thc_dequantize_irht, "THC: inverse transform whose first pass loads float(levels) * step + lo", py::arg("levels"), py::arg("sign"), py::arg("out"), py::arg("block"), py::arg("scale"), py::arg("step"), py::arg("lo"), py::arg("stream_p") = 0);
    modul.def("abi_version", &abi_version, "version string of libdynamiq_eden.so");
}
