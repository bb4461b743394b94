// Blocked randomized Hadamard transform fused with the quantiser: the fused forward kernels with a bfloat16 random pool
// (one translation unit of dq_rht_scaling_impl.cuh; the value is that file's DQ_RHT_COMPRESS_BF16).
#define DQ_RHT_PART 4
#include "dq_rht_scaling_impl.cuh"
