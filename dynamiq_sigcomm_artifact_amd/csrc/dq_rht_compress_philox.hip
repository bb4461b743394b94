// Blocked randomized Hadamard transform fused with the quantiser: the fused forward kernels with the in-kernel rounding stream
// (one translation unit of dq_rht_scaling_impl.cuh; the value is that file's DQ_RHT_COMPRESS_PHILOX).
#define DQ_RHT_PART 2
#include "dq_rht_scaling_impl.cuh"
