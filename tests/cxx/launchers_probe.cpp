// Test helper: a translation unit that uses include/dynamiq_eden_launchers.hpp the way the reference's transport
// extension uses csrc/cuda_hadamard.h (ring_allreduce_backend.cu:1255-1301): it takes every launcher through a
// function pointer of exactly the declared type (cuda_hadamard.h:13-28, cuda_packing.h:10-11, with hipStream_t for
// cudaStream_t and __hip_bfloat16 for __nv_bfloat16), so a drifted argument list fails to compile, and exports plain-C
// wrappers that the GPU tests call through ctypes.
#include "dynamiq_eden_launchers.hpp"

typedef __hip_bfloat16 bf16;

static void (*const p_hadamard)(float *, int, int, hipStream_t, int) = &HadamardWithCuda;
static void (*const p_hadamard_nsm)(float *, int, int, hipStream_t) = &HadamardWithCudaNoSharedMemory;
static void (*const p_comp_h)(__half *, uint8_t *, __half *, int, int, int, int, int, hipStream_t) = &scaling_compress_with_cuda;
static void (*const p_comp_b)(bf16 *, uint8_t *, bf16 *, int, int, int, int, int, hipStream_t) = &scaling_compress_with_cuda;
static void (*const p_dec_h)(uint8_t *, __half *, int, int, int, int, int, hipStream_t, int) = &scaling_decompress_with_cuda;
static void (*const p_dec_b)(uint8_t *, bf16 *, int, int, int, int, int, hipStream_t, int) = &scaling_decompress_with_cuda;
static void (*const p_dc)(uint8_t *, bf16 *, uint8_t *, bf16 *, int, int, int, int, int, hipStream_t) = &scaling_dec_comp_with_cuda;
static void (*const p_mc_h)(__half *, __half *, bf16 *, int, int, int, int, hipStream_t) = &superchunk_mean_center_with_cuda;
static void (*const p_mc_b)(bf16 *, bf16 *, bf16 *, int, int, int, int, hipStream_t) = &superchunk_mean_center_with_cuda;
static void (*const p_am_h)(__half *, __half *, bf16 *, int, int, int, hipStream_t) = &superchunk_add_mean_copy_with_cuda;
static void (*const p_am_b)(bf16 *, bf16 *, bf16 *, int, int, int, hipStream_t) = &superchunk_add_mean_copy_with_cuda;
static void (*const p_init)() = &init_lookup_table;
static void (*const p_b2b)(int *, int, uint32_t *, int, int, int) = &BinsToBits;
static void (*const p_b2n)(int *, int, uint32_t *, int, int, int) = &BitsToBins;

extern "C" {

int probe_last_status() { return dynamiq_launchers_last_status(); }

void probe_hadamard(float *vec, int n, int device, void *stream, int shared)
{
    if (shared)
        p_hadamard(vec, n, device, (hipStream_t)stream, 0);
    else
        p_hadamard_nsm(vec, n, device, (hipStream_t)stream);
}

// half: 1 = binary16 elements, 0 = bfloat16
void probe_compress(int half, void *src, uint8_t *dst, void *rand_pool, int n, int nbits, int chunk_size, int device, int strategy,
                    void *stream)
{
    if (half)
        p_comp_h((__half *)src, dst, (__half *)rand_pool, n, nbits, chunk_size, device, strategy, (hipStream_t)stream);
    else
        p_comp_b((bf16 *)src, dst, (bf16 *)rand_pool, n, nbits, chunk_size, device, strategy, (hipStream_t)stream);
}

void probe_decompress(int half, uint8_t *src, void *dst, int n, int nbits, int chunk_size, int device, int strategy, void *stream,
                      int add_original)
{
    if (half)
        p_dec_h(src, (__half *)dst, n, nbits, chunk_size, device, strategy, (hipStream_t)stream, add_original);
    else
        p_dec_b(src, (bf16 *)dst, n, nbits, chunk_size, device, strategy, (hipStream_t)stream, add_original);
}

void probe_dec_comp(uint8_t *recv, void *inp, uint8_t *send, void *rand_pool, int n, int nbits, int chunk_size, int device,
                    int strategy, void *stream)
{
    p_dc(recv, (bf16 *)inp, send, (bf16 *)rand_pool, n, nbits, chunk_size, device, strategy, (hipStream_t)stream);
}

void probe_mean_center(int half, void *src, void *residual, void *stats, int n, int world_size, int superchunk_size, int device,
                       void *stream)
{
    if (half)
        p_mc_h((__half *)src, (__half *)residual, (bf16 *)stats, n, world_size, superchunk_size, device, (hipStream_t)stream);
    else
        p_mc_b((bf16 *)src, (bf16 *)residual, (bf16 *)stats, n, world_size, superchunk_size, device, (hipStream_t)stream);
}

void probe_add_mean_copy(int half, void *residual, void *dst, void *stats, int n, int superchunk_size, int device, void *stream)
{
    if (half)
        p_am_h((__half *)residual, (__half *)dst, (bf16 *)stats, n, superchunk_size, device, (hipStream_t)stream);
    else
        p_am_b((bf16 *)residual, (bf16 *)dst, (bf16 *)stats, n, superchunk_size, device, (hipStream_t)stream);
}

void probe_init_lookup_table() { p_init(); }

void probe_bins_to_bits(int *bins, int nbins, uint32_t *arr, int narr, int nbits, int device) { p_b2b(bins, nbins, arr, narr, nbits, device); }

void probe_bits_to_bins(int *bins, int nbins, uint32_t *arr, int narr, int nbits, int device) { p_b2n(bins, nbins, arr, narr, nbits, device); }

void probe_quantization(float *vec, int n, int device, float div_factor, float tensor_max, uint64_t seed, void *stream)
{
    quantization_with_hip(vec, n, device, div_factor, tensor_max, seed, (hipStream_t)stream);
}
}
