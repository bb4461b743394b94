// Blocked randomized Hadamard transform fused with the quantiser: the fused inverse kernels
// (one translation unit of dq_rht_scaling_impl.cuh; the value is that file's DQ_RHT_DECOMPRESS).
#define DQ_RHT_PART 16
#include "dq_rht_scaling_impl.cuh"
