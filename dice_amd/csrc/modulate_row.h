// LayerNorm without affine parameters plus the adaLN modulation of one token
// row held in the registers of one wavefront, h = LN(x) * (1 + scale) + shift
// (reference models.py:75-76,497,519).  Shared by the stand-alone prologue
// kernel and by the prologue that also routes, so both round every element the
// same way: mean and variance are two exact fp32 passes over the registers
// (variance around the mean, biased, eps inside the square root, as
// torch.nn.LayerNorm), the result is rounded once.
#pragma once

#include "common.h"

namespace dice {

template <typename T> struct Chunk;  // 16 bytes of a row
template <> struct Chunk<float> {
  static constexpr int kN = 4;
  f32x4_t v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = f; }
};
template <> struct Chunk<bf16_t> {
  static constexpr int kN = 8;
  bf16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (bf16_t)f; }
};
template <> struct Chunk<f16_t> {
  static constexpr int kN = 8;
  f16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (f16_t)f; }
};

// Lane l holds chunks l, l + 64, ... (< chunks_per_row) of the token row in v,
// of the sample's scale row in ms and of its shift row in mh; v becomes the
// modulated row.
template <typename T, int MAXC>
__device__ __forceinline__ void ln_modulate_row(Chunk<T> (&v)[MAXC], const Chunk<T> (&ms)[MAXC],
                                                const Chunk<T> (&mh)[MAXC], int lane, int chunks_per_row,
                                                float inv_hidden, float eps) {
  constexpr int N = Chunk<T>::kN;
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    if (lane + i * kWave < chunks_per_row) {
#pragma unroll
      for (int e = 0; e < N; ++e) sum += v[i].get(e);
    }
  }
  const float mean = wave_sum(sum) * inv_hidden;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    if (lane + i * kWave < chunks_per_row) {
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float d = v[i].get(e) - mean;
        sq = fmaf(d, d, sq);
      }
    }
  }
  const float rstd = 1.0f / sqrtf(wave_sum(sq) * inv_hidden + eps);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    if (lane + i * kWave < chunks_per_row) {
      const Chunk<T> s = ms[i], h = mh[i];
      Chunk<T> o;
#pragma unroll
      for (int e = 0; e < N; ++e)
        o.set(e, fmaf((v[i].get(e) - mean) * rstd, 1.0f + s.get(e), h.get(e)));
      v[i] = o;
    }
  }
}

}  // namespace dice
