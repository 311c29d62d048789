// The permutation-addressed expert GEMMs for fp32 activations and weights on the
// fp32 MFMA: the same source as the bf16 kernels with the element type, the k
// step and the inner loop switched (see the head of grouped_gemm_bf16.hip).
#define DICE_GEMM_F32 1
#include "grouped_gemm_bf16.hip"
