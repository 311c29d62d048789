// fp32 grouped expert GEMM (the module-dtype float path, e.g. DiT-S/2).
//
// Same scheduling and fused prologue/epilogue as the bf16 MFMA kernel (row
// gather through the permutation, SwiGLU / GELU, scatter to slot rows) but on
// plain fp32 FMAs so results stay within fp32 round-off of the reference
// (MoeMLP.forward, models.py:252-273).  64x64 output tile per workgroup, a 4x4
// micro-tile per thread, operands staged k-major in LDS.
#include "gemm_common.h"

namespace dice {
namespace {

constexpr int kBM = 64, kBN = 64, kBK = 16, kPad = 4;

template <int MODE>
__global__ __launch_bounds__(256) void grouped_gemm_f32_kernel(GemmParams p) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  __shared__ float As[kBK][kBM + kPad];
  __shared__ float Bs[SWIGLU ? 2 : 1][kBK][kBN + kPad];

  const TileCoord t = locate_tile<kBM, kBN>(p);
  if (!t.active) return;
  const int tid = threadIdx.x;
  const int ld_row = tid >> 2;        // 0..63
  const int ld_k = (tid & 3) * 4;     // 0,4,8,12
  const float *a = (const float *)p.a;
  const float *w = (const float *)p.w + (size_t)t.expert * p.w_rows * p.k;

  int grow = t.row_begin + (ld_row < t.rows_valid ? ld_row : t.rows_valid - 1);
  const int64_t src = p.a_perm ? p.a_perm[grow] / p.a_div : grow;
  const float *a_ptr = a + src * p.lda + ld_k;
  int ncol = t.n0 + ld_row;
  if (ncol >= p.n) ncol = p.n - 1;
  const float *b_ptr0 = w + (size_t)ncol * p.k + ld_k;
  const float *b_ptr1 = SWIGLU ? w + (size_t)(p.up_offset + ncol) * p.k + ld_k : nullptr;

  const int tm = (tid >> 4) * 4;  // micro-tile origin
  const int tn = (tid & 15) * 4;
  float acc0[4][4], acc1[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc0[i][j] = acc1[i][j] = 0.f;

  for (int k0 = 0; k0 < p.k; k0 += kBK) {
    const f32x4_t av = *(const f32x4_t *)(a_ptr + k0);
    const f32x4_t bv0 = *(const f32x4_t *)(b_ptr0 + k0);
    f32x4_t bv1 = {0.f, 0.f, 0.f, 0.f};
    if (SWIGLU) bv1 = *(const f32x4_t *)(b_ptr1 + k0);
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      As[ld_k + q][ld_row] = av[q];
      Bs[0][ld_k + q][ld_row] = bv0[q];
      if (SWIGLU) Bs[1][ld_k + q][ld_row] = bv1[q];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kBK; ++kk) {
      const f32x4_t ar = *(const f32x4_t *)&As[kk][tm];
      const f32x4_t br0 = *(const f32x4_t *)&Bs[0][kk][tn];
      f32x4_t br1 = {0.f, 0.f, 0.f, 0.f};
      if (SWIGLU) br1 = *(const f32x4_t *)&Bs[1][kk][tn];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc0[i][j] = fmaf(ar[i], br0[j], acc0[i][j]);
          if (SWIGLU) acc1[i][j] = fmaf(ar[i], br1[j], acc1[i][j]);
        }
    }
  }

  float *c = (float *)p.c;
  const float *bias = p.bias ? p.bias + (size_t)t.expert * p.n : nullptr;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = tm + i;
    if (m >= t.rows_valid) continue;
    const int gr = t.row_begin + m;
    const int64_t orow = p.c_perm ? p.c_perm[gr] : gr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = t.n0 + tn + j;
      if (n >= p.n) continue;
      float v = acc0[i][j];
      if (MODE == kFc1Swiglu) {
        v = silu_f(v) * acc1[i][j];
      } else {
        if (bias) v += bias[n];
        if (MODE == kFc1Gelu) v = gelu_tanh_f(v);
      }
      c[orow * p.ldc + n] = v;
    }
  }
}

}  // namespace

int launch_grouped_gemm_f32(const GemmParams &p, int mode, int64_t max_rows, hipStream_t s) {
  if (p.k % kBK != 0) return fail(DICE_ERR_UNSUPPORTED, "fp32 expert GEMM: k %d %% %d != 0", p.k, kBK);
  const int64_t grid = max_tiles(max_rows, p.n_experts, p.n, kBM, kBN);
  if (grid <= 0) return DICE_OK;
  if (grid >= (1ll << 31)) return fail(DICE_ERR_UNSUPPORTED, "fp32 expert GEMM: grid too large");
  switch (mode) {
    case kFc1Swiglu:
      hipLaunchKernelGGL(grouped_gemm_f32_kernel<kFc1Swiglu>, dim3((unsigned)grid), dim3(256), 0, s, p);
      break;
    case kFc1Gelu:
      hipLaunchKernelGGL(grouped_gemm_f32_kernel<kFc1Gelu>, dim3((unsigned)grid), dim3(256), 0, s, p);
      break;
    default:
      hipLaunchKernelGGL(grouped_gemm_f32_kernel<kFc2>, dim3((unsigned)grid), dim3(256), 0, s, p);
  }
  return launch_status("grouped_gemm_f32");
}

}  // namespace dice
