// fp8 (OCP e4m3fn) quantisers: per output channel for expert weights, per row
// (token) for the activations of the fp8 expert GEMMs.
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

// Activation rows -> e4m3 with one scale per row, for the expert GEMMs that
// multiply on the fp8 matrix pipe (build-defined, like the weight quantiser):
//   amax = max |x[r,:]|;  scale[r] = amax / 448 (1 when the row is all zero)
//   q[r,c] = e4m3fn(rne(x[r,c] * (448 / amax)))
// (a multiplication by the reciprocal, not a division: one rounding of the
// reciprocal, one of the product, both reproducible in fp32 anywhere).
// One wavefront per output row; the row stays in registers between the max and
// the conversion (CHUNKS 16-byte pieces per lane), so x is read once.  With a
// row table the source row of output row r is perm[r] / slots_per_token: the
// gather of the dispatch fused into the quantiser, output in grouped order.
// Rows at and beyond *n_rows_dev (the device-side row count) are left alone.
template <typename T, int CHUNKS>
__global__ __launch_bounds__(256) void quantize_act_rows_kernel(const T *__restrict__ x, const int32_t *__restrict__ perm,
                                                                int slots_per_token, const int32_t *__restrict__ n_rows_dev,
                                                                int64_t max_rows, int cols, uint8_t *__restrict__ q,
                                                                float *__restrict__ scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (r >= max_rows) return;
  if (n_rows_dev && r >= *n_rows_dev) return;
  int64_t src = r;
  if (perm) {
    const int slot = perm[r];
    if (slot < 0) return;
    src = slot / slots_per_token;
  }
  const u32x4_t *row = reinterpret_cast<const u32x4_t *>(x + src * cols);
  const int n_chunks = cols / 8;  // 16-byte pieces of a row
  u32x4_t v[CHUNKS];
  float m = 0.f;
  bool finite = true;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = c * kWave + lane;
    v[c] = u32x4_t{0, 0, 0, 0};
    if (i < n_chunks) v[c] = row[i];
    const T *e = reinterpret_cast<const T *>(&v[c]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = fabsf(to_f32(e[j]));
      finite = finite && a < __builtin_inff();   // (false for NaN as well; fmaxf would drop a NaN)
      m = fmaxf(m, a);
    }
  }
  m = wave_max(m);
  // A row with a NaN or an infinity stays visible: its scale is NaN, which the
  // GEMM's epilogue multiplies into every output of the row (a 16-bit row would
  // carry it through the products likewise); its bytes are zeros.
  const bool row_finite = __ballot(!finite) == 0;
  const float inv = !row_finite ? 0.f : m > 0.f ? 448.0f / m : 1.0f;
  if (lane == 0) scale[r] = !row_finite ? __builtin_nanf("") : m > 0.f ? m / 448.0f : 1.0f;
  u32x2_t *qrow = reinterpret_cast<u32x2_t *>(q + r * cols);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = c * kWave + lane;
    const T *e = reinterpret_cast<const T *>(&v[c]);
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = row_finite ? fminf(fmaxf(to_f32(e[j]) * inv, -448.f), 448.f) : 0.f;
    u32x2_t o;
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
    o[0] = (uint32_t)w;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w, true);
    o[1] = (uint32_t)w;
    if (i < n_chunks) qrow[i] = o;
  }
}

template <typename T>
int launch_quantize_act(const void *x, const int32_t *perm, int slots_per_token, const int32_t *n_rows_dev,
                        int64_t max_rows, int cols, uint8_t *q, float *scale, hipStream_t s) {
  const unsigned grid = (unsigned)((max_rows + 3) / 4);
  const int per_lane = (cols / 8 + kWave - 1) / kWave;
#define DICE_QA(C)                                                                                        \
  hipLaunchKernelGGL((quantize_act_rows_kernel<T, C>), dim3(grid), dim3(256), 0, s, (const T *)x, perm, \
                     slots_per_token, n_rows_dev, max_rows, cols, q, scale)
  if (per_lane <= 2) DICE_QA(2);
  else if (per_lane <= 4) DICE_QA(4);
  else if (per_lane <= 8) DICE_QA(8);
  else DICE_QA(16);
#undef DICE_QA
  return launch_status("dice_quantize_fp8_act");
}

}  // namespace

int quantize_act_impl(const void *x, int in_dtype, const int32_t *perm, int slots_per_token,
                      const int32_t *n_rows_dev, int64_t max_rows, int cols, uint8_t *q, float *scale,
                      void *stream) {
  DICE_REQUIRE(x && q && scale, DICE_ERR_BAD_ARG, "dice_quantize_fp8_act: null pointer");
  DICE_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), DICE_ERR_BAD_ARG, "dice_quantize_fp8_act: max_rows %lld",
               (long long)max_rows);
  DICE_REQUIRE(cols > 0 && cols % 8 == 0 && cols <= 16 * 8 * kWave, DICE_ERR_UNSUPPORTED,
               "dice_quantize_fp8_act: cols %d must be a positive multiple of 8, at most %d", cols, 16 * 8 * kWave);
  DICE_REQUIRE(!perm || slots_per_token >= 1, DICE_ERR_BAD_ARG, "dice_quantize_fp8_act: slots_per_token %d",
               slots_per_token);
  if (max_rows == 0) return DICE_OK;
  hipStream_t s = (hipStream_t)stream;
  if (in_dtype == DICE_BF16)
    return launch_quantize_act<bf16_t>(x, perm, slots_per_token, n_rows_dev, max_rows, cols, q, scale, s);
  if (in_dtype == DICE_F16)
    return launch_quantize_act<f16_t>(x, perm, slots_per_token, n_rows_dev, max_rows, cols, q, scale, s);
  return fail(DICE_ERR_UNSUPPORTED, "dice_quantize_fp8_act: in_dtype %d (BF16 or F16)", in_dtype);
}

}  // namespace dice

extern "C" int dice_quantize_fp8_act(const void *x, int in_dtype, const int32_t *perm, int slots_per_token,
                                     const int32_t *n_rows_dev, int64_t max_rows, int cols, uint8_t *q,
                                     float *scale, void *stream) {
  return dice::quantize_act_impl(x, in_dtype, perm, slots_per_token, n_rows_dev, max_rows, cols, q, scale, stream);
}

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
