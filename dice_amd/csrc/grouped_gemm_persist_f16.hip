// The persistent expert GEMMs for fp16 activations and weights: the same source
// as the bf16 kernels with the element type, the MFMA instruction and the fp8
// widening switched (see the head of grouped_gemm_persist.hip).
#define DICE_PERSIST_F16 1
#include "grouped_gemm_persist.hip"
