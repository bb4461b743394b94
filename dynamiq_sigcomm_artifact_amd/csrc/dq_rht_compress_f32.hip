// Blocked randomized Hadamard transform fused with the quantiser: the fused forward kernels with a float32 random pool
// (one translation unit of dq_rht_scaling_impl.cuh; the value is that file's DQ_RHT_COMPRESS_F32).
#define DQ_RHT_PART 8
#include "dq_rht_scaling_impl.cuh"
