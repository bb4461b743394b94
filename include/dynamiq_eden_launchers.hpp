/*
 * C++ launchers with the names and argument lists that the DynamiQ artifact declares in
 * cuda_kernels/src/srrcomp/eden_utils/csrc/cuda_hadamard.h:13-28 and csrc/cuda_packing.h:10-11, on a
 * hipStream_t, as inline forwards to the C ABI of libdynamiq_eden.so (dynamiq_eden.h).
 *
 * This is the second boundary of the compression path: the reference's transport extension
 * (rdma_comm_compress/ring_allreduce_ext/ring_allreduce_backend.cu:1255-1301,1678-1721) includes
 * cuda_hadamard.h and calls these overloads per record-aligned tile, from two host threads on distinct
 * streams.  A ROCm build of such a caller includes this header instead and links libdynamiq_eden.so;
 * the call sites stay as they are (cudaStream_t -> hipStream_t, __nv_bfloat16 -> __hip_bfloat16).
 *
 * Error behaviour: the reference's launchers return void and print a failed launch to stderr
 * (cuda_hadamard.cu:1496-1499).  These do the same with the library's message for any non-zero
 * status -- which here also covers the argument checks that the reference leaves to its Python
 * binding -- and additionally keep the status: dynamiq_launchers_last_status() returns the last
 * non-zero status of the calling thread and clears it.  Compile with DYNAMIQ_LAUNCHERS_THROW to get a
 * std::runtime_error instead of the print.
 *
 * Nothing here allocates or synchronises; every call enqueues on the given stream.
 */
#ifndef DYNAMIQ_EDEN_LAUNCHERS_HPP
#define DYNAMIQ_EDEN_LAUNCHERS_HPP

#include <hip/hip_runtime_api.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <cstdint>
#include <cstdio>
#ifdef DYNAMIQ_LAUNCHERS_THROW
#include <stdexcept>
#include <string>
#endif

#include "dynamiq_eden.h"

namespace dynamiq_launchers_detail {
inline int &last_status()
{
    static thread_local int status = 0;
    return status;
}
inline void report(int status, const char *what)
{
    if (status == 0) return;
    last_status() = status;
#ifdef DYNAMIQ_LAUNCHERS_THROW
    throw std::runtime_error(std::string(what) + ": " + dq_last_error());
#else
    std::fprintf(stderr, "%s: %s\n", what, dq_last_error());
#endif
}
} // namespace dynamiq_launchers_detail

/* the last non-zero dq_status seen by a launcher on the calling thread (0 if none); reading clears it */
inline int dynamiq_launchers_last_status()
{
    int &s = dynamiq_launchers_detail::last_status();
    const int v = s;
    s = 0;
    return v;
}

/* csrc/cuda_hadamard.h:14; `depth` is ignored there (cuda_hadamard.cu:534-605) and here */
inline void HadamardWithCuda(float *vec, int n, int device, hipStream_t stream, int depth)
{
    dynamiq_launchers_detail::report(dq_hadamard(vec, n, device, stream, depth), "HadamardWithCuda");
}

/* csrc/cuda_hadamard.h:13: the same transform (the two differ only in how the reference stages it) */
inline void HadamardWithCudaNoSharedMemory(float *vec, int n, int device, hipStream_t stream)
{
    dynamiq_launchers_detail::report(dq_hadamard(vec, n, device, stream, 0), "HadamardWithCudaNoSharedMemory");
}

/* csrc/cuda_hadamard.h:18,20 */
inline void scaling_compress_with_cuda(__half *src, uint8_t *dst, __half *rand_pool, int n, int nbits, int chunk_size,
                                       int device, int strategy, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_scaling_compress(src, dst, rand_pool, n, nbits, chunk_size, DQ_F16, device, strategy, stream),
        "scaling_compress_with_cuda");
}
inline void scaling_compress_with_cuda(__hip_bfloat16 *src, uint8_t *dst, __hip_bfloat16 *rand_pool, int n, int nbits,
                                       int chunk_size, int device, int strategy, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_scaling_compress(src, dst, rand_pool, n, nbits, chunk_size, DQ_BF16, device, strategy, stream),
        "scaling_compress_with_cuda");
}

/* csrc/cuda_hadamard.h:19,21 */
inline void scaling_decompress_with_cuda(uint8_t *src, __half *dst, int n, int nbits, int chunk_size, int device,
                                         int strategy, hipStream_t stream, int add_original)
{
    dynamiq_launchers_detail::report(
        dq_scaling_decompress(src, dst, n, nbits, chunk_size, DQ_F16, device, strategy, stream, add_original),
        "scaling_decompress_with_cuda");
}
inline void scaling_decompress_with_cuda(uint8_t *src, __hip_bfloat16 *dst, int n, int nbits, int chunk_size, int device,
                                         int strategy, hipStream_t stream, int add_original)
{
    dynamiq_launchers_detail::report(
        dq_scaling_decompress(src, dst, n, nbits, chunk_size, DQ_BF16, device, strategy, stream, add_original),
        "scaling_decompress_with_cuda");
}

/* csrc/cuda_hadamard.h:22: bfloat16 only, as in the reference */
inline void scaling_dec_comp_with_cuda(uint8_t *recv, __hip_bfloat16 *inp, uint8_t *send, __hip_bfloat16 *rand_pool,
                                       int n, int nbits, int chunk_size, int device, int strategy, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_scaling_dec_comp(recv, inp, send, rand_pool, n, nbits, chunk_size, DQ_BF16, device, strategy, stream),
        "scaling_dec_comp_with_cuda");
}

/* csrc/cuda_hadamard.h:23-24: the statistics are bfloat16 for both element types */
inline void superchunk_mean_center_with_cuda(__half *src, __half *residual, __hip_bfloat16 *stats, int n,
                                             int world_size, int superchunk_size, int device, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_superchunk_mean_center(src, residual, stats, n, world_size, superchunk_size, DQ_F16, device, stream),
        "superchunk_mean_center_with_cuda");
}
inline void superchunk_mean_center_with_cuda(__hip_bfloat16 *src, __hip_bfloat16 *residual, __hip_bfloat16 *stats, int n,
                                             int world_size, int superchunk_size, int device, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_superchunk_mean_center(src, residual, stats, n, world_size, superchunk_size, DQ_BF16, device, stream),
        "superchunk_mean_center_with_cuda");
}

/* csrc/cuda_hadamard.h:25-26 */
inline void superchunk_add_mean_copy_with_cuda(__half *residual, __half *dst, __hip_bfloat16 *stats, int n,
                                               int superchunk_size, int device, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_superchunk_add_mean_copy(residual, dst, stats, n, superchunk_size, DQ_F16, device, stream),
        "superchunk_add_mean_copy_with_cuda");
}
inline void superchunk_add_mean_copy_with_cuda(__hip_bfloat16 *residual, __hip_bfloat16 *dst, __hip_bfloat16 *stats, int n,
                                               int superchunk_size, int device, hipStream_t stream)
{
    dynamiq_launchers_detail::report(
        dq_superchunk_add_mean_copy(residual, dst, stats, n, superchunk_size, DQ_BF16, device, stream),
        "superchunk_add_mean_copy_with_cuda");
}

/* csrc/cuda_hadamard.h:28 */
inline void init_lookup_table() { dynamiq_launchers_detail::report(dq_init_lookup_table(), "init_lookup_table"); }

/* csrc/cuda_packing.h:10-11.  The reference launches on the legacy default stream (cuda_packing.cu:58-65,
 * 119-126); so do these. */
inline void BinsToBits(int *bins, int nbins, uint32_t *arr, int narr, int nbits, int device)
{
    dynamiq_launchers_detail::report(dq_bins_to_bits(bins, nbins, arr, narr, nbits, device, nullptr), "BinsToBits");
}
inline void BitsToBins(int *bins, int nbins, uint32_t *arr, int narr, int nbits, int device)
{
    dynamiq_launchers_detail::report(dq_bits_to_bins(bins, nbins, arr, narr, nbits, device, nullptr), "BitsToBins");
}

/* csrc/cuda_hadamard.h:16 declares quantization_with_cuda(vec, n, device, div_factor, tensor_max, curandState_t*, stream):
 * its random states are a cuRAND type that the reference never initialises (cuda_hadamard.cu:669-686).  The
 * counterpart takes the seed of a counter-based stream in their place. */
inline void quantization_with_hip(float *vec, int n, int device, float div_factor, float tensor_max, uint64_t seed,
                                  hipStream_t stream)
{
    dynamiq_launchers_detail::report(dq_quantization(vec, n, device, div_factor, tensor_max, seed, stream),
                                     "quantization_with_hip");
}

#endif
