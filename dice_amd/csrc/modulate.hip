// Prologue of the layer's caller: LayerNorm without affine parameters followed
// by the adaLN modulation, h = LN(x) * (1 + scale[b]) + shift[b].
//
// Replaces modulate(self.norm2(x), shift_mlp, scale_mlp) of DiTBlock.forward
// (reference models.py:75-76,497,519), which the reference runs as one
// LayerNorm kernel plus three elementwise kernels (four round trips over
// [N, D]); here x is read once and h written once.
//
// HBM-bound.  One wavefront per token row: the row stays in registers (up to
// kMaxChunks 16-byte chunks per lane), mean and variance are two exact passes
// over those registers in fp32 (variance around the mean, biased, eps inside
// the square root, as torch.nn.LayerNorm), and the result is rounded once.
#include "modulate_row.h"

namespace dice {
namespace {

constexpr int kModWaves = 4;

template <typename T, int MAXC>
__global__ __launch_bounds__(kModWaves *kWave) void ln_modulate_kernel(
    const Chunk<T> *__restrict__ x, const Chunk<T> *__restrict__ shift,
    const Chunk<T> *__restrict__ scale, Chunk<T> *__restrict__ out, int64_t n_tokens,
    int chunks_per_row, int64_t tokens_per_sample, float inv_hidden, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (int64_t t = (int64_t)blockIdx.x * kModWaves + wave; t < n_tokens;
       t += (int64_t)gridDim.x * kModWaves) {
    const Chunk<T> *row = x + t * chunks_per_row;
    const int64_t b = t / tokens_per_sample;
    const Chunk<T> *sh = shift + b * chunks_per_row;
    const Chunk<T> *sc = scale + b * chunks_per_row;
    // Everything the row needs is requested at once (the sample's shift and
    // scale rows with the token row): one memory round trip per token, not two.
    Chunk<T> v[MAXC], ms[MAXC], mh[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + i * kWave;
      if (c < chunks_per_row) {
        v[i] = row[c];
        ms[i] = sc[c];
        mh[i] = sh[c];
      }
    }
    ln_modulate_row<T, MAXC>(v, ms, mh, lane, chunks_per_row, inv_hidden, eps);
    Chunk<T> *dst = out + t * chunks_per_row;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + i * kWave;
      if (c < chunks_per_row) dst[c] = v[i];
    }
  }
}

template <typename T>
int launch_modulate(const void *x, const void *shift, const void *scale, void *out, int64_t n_tokens,
                    int hidden, int64_t tokens_per_sample, float eps, hipStream_t s) {
  const int chunks = hidden / Chunk<T>::kN;
  int64_t blocks = (n_tokens + kModWaves - 1) / kModWaves;
  if (blocks > 8192) blocks = 8192;
  const float inv_hidden = 1.0f / (float)hidden;
#define DICE_MOD_LAUNCH(MAXC)                                                                      \
  hipLaunchKernelGGL((ln_modulate_kernel<T, MAXC>), dim3((unsigned)blocks), dim3(kModWaves *kWave), 0, s, \
                     (const Chunk<T> *)x, (const Chunk<T> *)shift, (const Chunk<T> *)scale,        \
                     (Chunk<T> *)out, n_tokens, chunks, tokens_per_sample, inv_hidden, eps)
  if (chunks <= 2 * kWave) {
    DICE_MOD_LAUNCH(2);
  } else if (chunks <= 4 * kWave) {
    DICE_MOD_LAUNCH(4);
  } else if (chunks <= 8 * kWave) {
    DICE_MOD_LAUNCH(8);
  } else if (chunks <= 16 * kWave) {
    DICE_MOD_LAUNCH(16);
  } else {
    return fail(DICE_ERR_UNSUPPORTED, "dice_ln_modulate: hidden %d exceeds %d elements", hidden,
                16 * kWave * Chunk<T>::kN);
  }
#undef DICE_MOD_LAUNCH
  return launch_status("dice_ln_modulate");
}

}  // namespace

int ln_modulate_impl(const void *x, const void *shift, const void *scale, void *out, int dtype,
                     int64_t n_tokens, int hidden, int64_t tokens_per_sample, float eps, void *stream) {
  DICE_REQUIRE(x && shift && scale && out, DICE_ERR_BAD_ARG, "dice_ln_modulate: null pointer");
  DICE_REQUIRE(n_tokens >= 0, DICE_ERR_BAD_ARG, "dice_ln_modulate: n_tokens %lld < 0", (long long)n_tokens);
  DICE_REQUIRE(tokens_per_sample >= 1, DICE_ERR_BAD_ARG, "dice_ln_modulate: tokens_per_sample %lld < 1",
               (long long)tokens_per_sample);
  DICE_REQUIRE(eps >= 0.f, DICE_ERR_BAD_ARG, "dice_ln_modulate: eps %g < 0", (double)eps);
  const size_t es = dtype_size(dtype);
  DICE_REQUIRE(es == 2 || es == 4, DICE_ERR_UNSUPPORTED, "dice_ln_modulate: dtype %d", dtype);
  DICE_REQUIRE(hidden > 0 && ((size_t)hidden * es) % 16 == 0, DICE_ERR_BAD_ARG,
               "dice_ln_modulate: hidden %d rows are not a multiple of 16 bytes", hidden);
  if (n_tokens == 0) return DICE_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DICE_F32:
      return launch_modulate<float>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, s);
    case DICE_BF16:
      return launch_modulate<bf16_t>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, s);
    case DICE_F16:
      return launch_modulate<f16_t>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, s);
  }
  return fail(DICE_ERR_UNSUPPORTED, "dice_ln_modulate: dtype %d", dtype);
}

}  // namespace dice

extern "C" int dice_ln_modulate(const void *x, const void *shift, const void *scale, void *out,
                                int dtype, int64_t n_tokens, int hidden, int64_t tokens_per_sample,
                                float eps, void *stream) {
  return dice::ln_modulate_impl(x, shift, scale, out, dtype, n_tokens, hidden, tokens_per_sample, eps,
                                stream);
}
