// Per-output-channel fp8 (OCP e4m3fn) quantiser for expert weights.
//
// The reference has no fp8 path; the scheme is defined here:
//   scale[r] = amax(|w[r,:]|) / 448   (1 when the row is all zero)
//   q[r,c]   = e4m3fn(round-to-nearest-even(w[r,c] / scale[r]))
// One workgroup per row: a max-reduction pass, then a conversion pass with the
// hardware v_cvt_pk_fp8_f32 (inputs are already inside +-448, so saturation
// never triggers).  HBM-bound: reads the row twice (second time from cache),
// writes one byte per element.
#include "common.h"

namespace dice {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const T *__restrict__ w, int64_t cols,
                                                            uint8_t *__restrict__ q,
                                                            float *__restrict__ scale) {
  __shared__ float wave_max_s[4];
  const int64_t r = blockIdx.x;
  const T *row = w + r * cols;
  float m = 0.f;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) m = fmaxf(m, fabsf(to_f32(row[c])));
  m = wave_max(m);
  if ((threadIdx.x & (kWave - 1)) == 0) wave_max_s[threadIdx.x / kWave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(wave_max_s[0], wave_max_s[1]), fmaxf(wave_max_s[2], wave_max_s[3]));
  const float sc = m > 0.f ? m / 448.0f : 1.0f;
  if (threadIdx.x == 0) scale[r] = sc;
  uint8_t *qrow = q + r * cols;
  // Pairs of elements -> one packed conversion; cols is even (checked on the host).
  for (int64_t c = (int64_t)threadIdx.x * 2; c < cols; c += (int64_t)blockDim.x * 2) {
    float a = to_f32(row[c]) / sc;
    float b = to_f32(row[c + 1]) / sc;
    a = fminf(fmaxf(a, -448.f), 448.f);
    b = fminf(fmaxf(b, -448.f), 448.f);
    const uint32_t packed = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    *reinterpret_cast<uint16_t *>(qrow + c) = (uint16_t)(packed & 0xffffu);
  }
}

}  // namespace
}  // namespace dice

extern "C" int dice_quantize_fp8_rowwise(const void *w, int in_dtype, int64_t rows, int64_t cols,
                                         uint8_t *q, float *scale, void *stream) {
  using namespace dice;
  DICE_REQUIRE(w && q && scale, DICE_ERR_BAD_ARG, "dice_quantize_fp8_rowwise: null pointer");
  DICE_REQUIRE(rows >= 0 && cols > 0 && cols % 2 == 0, DICE_ERR_BAD_ARG,
               "dice_quantize_fp8_rowwise: cols %lld must be positive and even", (long long)cols);
  if (rows == 0) return DICE_OK;
  DICE_REQUIRE(rows < (1ll << 31), DICE_ERR_BAD_ARG, "dice_quantize_fp8_rowwise: too many rows");
  hipStream_t s = (hipStream_t)stream;
  if (in_dtype == DICE_BF16) {
    hipLaunchKernelGGL(quantize_rows_kernel<bf16_t>, dim3((unsigned)rows), dim3(256), 0, s,
                       (const bf16_t *)w, cols, q, scale);
  } else if (in_dtype == DICE_F16) {
    hipLaunchKernelGGL(quantize_rows_kernel<f16_t>, dim3((unsigned)rows), dim3(256), 0, s,
                       (const f16_t *)w, cols, q, scale);
  } else if (in_dtype == DICE_F32) {
    hipLaunchKernelGGL(quantize_rows_kernel<float>, dim3((unsigned)rows), dim3(256), 0, s,
                       (const float *)w, cols, q, scale);
  } else {
    return fail(DICE_ERR_UNSUPPORTED, "dice_quantize_fp8_rowwise: in_dtype %d", in_dtype);
  }
  return launch_status("dice_quantize_fp8_rowwise");
}
