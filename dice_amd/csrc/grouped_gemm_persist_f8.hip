// The persistent expert GEMM with fp8 (e4m3) activations AND weights: the fp8
// kernel of grouped_gemm_persist.hip, compiled on its own (bf16 output).
#define DICE_PERSIST_F8 1
#include "grouped_gemm_persist.hip"
