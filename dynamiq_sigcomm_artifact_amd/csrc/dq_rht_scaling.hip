// Blocked randomized Hadamard transform fused with the quantiser: the transform passes, the dispatcher of the fused forward call and its matrix-core variant
// (one translation unit of dq_rht_scaling_impl.cuh; the value is that file's DQ_RHT_TRANSFORM).
#define DQ_RHT_PART 1
#include "dq_rht_scaling_impl.cuh"
