// Router: fp32 logits -> softmax -> top-k, one wavefront per token.
//
// Replaces MoEGate.forward, inference branch (reference models.py:179-196).
// HBM-bound: the only large operand is x, read exactly once (n_tokens*hidden
// elements); the router matrix is staged once per workgroup in LDS.  Each wave
// keeps TOK tokens in flight so one LDS read of a router chunk feeds TOK
// dot-product updates.
#include "common.h"

namespace dice {

namespace {

template <typename T> struct Vec8;  // 8 consecutive elements of a row
template <> struct Vec8<float> {
  f32x4_t a, b;
  __device__ __forceinline__ float get(int i) const { return i < 4 ? a[i] : b[i - 4]; }
};
template <> struct Vec8<bf16_t> {
  bf16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};
template <> struct Vec8<f16_t> {
  f16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};

template <typename T>
__device__ __forceinline__ Vec8<T> load8(const T *p) {
  return *reinterpret_cast<const Vec8<T> *>(p);
}

constexpr int kGateWaves = 4;

// EP = experts padded to a compile-time bound so accumulators stay in
// registers; TOK = tokens per wave per pass.
template <typename XT, typename WT, int EP, int TOK, bool W_IN_LDS>
__global__ __launch_bounds__(kGateWaves *kWave) void gate_topk_kernel(
    const XT *__restrict__ x, const WT *__restrict__ w, const float *__restrict__ bias,
    int64_t n_tokens, int hidden, int n_experts, int top_k, int norm_topk,
    int32_t *__restrict__ topk_idx, int64_t *__restrict__ topk_idx64,
    float *__restrict__ topk_weight, float *__restrict__ logits_out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int chunks = hidden / 8;

  const WT *wsrc = w;
  if (W_IN_LDS) {
    WT *wl = reinterpret_cast<WT *>(lds_raw);
    const int total = n_experts * chunks;
    for (int c = threadIdx.x; c < total; c += blockDim.x)
      *reinterpret_cast<Vec8<WT> *>(wl + (size_t)c * 8) = load8(w + (size_t)c * 8);
    __syncthreads();
    wsrc = wl;
  }

  const int64_t groups = (n_tokens + TOK - 1) / TOK;
  for (int64_t g = (int64_t)blockIdx.x * kGateWaves + wave; g < groups;
       g += (int64_t)gridDim.x * kGateWaves) {
    const int64_t t0 = g * TOK;
    float acc[TOK][EP];
#pragma unroll
    for (int t = 0; t < TOK; ++t)
#pragma unroll
      for (int e = 0; e < EP; ++e) acc[t][e] = 0.f;

    const XT *xrow[TOK];
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      int64_t tt = t0 + t < n_tokens ? t0 + t : n_tokens - 1;
      xrow[t] = x + tt * hidden;
    }

    for (int c = lane; c < chunks; c += kWave) {
      Vec8<XT> xv[TOK];
#pragma unroll
      for (int t = 0; t < TOK; ++t) xv[t] = load8(xrow[t] + c * 8);
#pragma unroll
      for (int e = 0; e < EP; ++e) {
        if (e < n_experts) {
          Vec8<WT> wv = load8(wsrc + ((size_t)e * chunks + c) * 8);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float wf = wv.get(i);
#pragma unroll
            for (int t = 0; t < TOK; ++t) acc[t][e] = fmaf(xv[t].get(i), wf, acc[t][e]);
          }
        }
      }
    }

#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      // Lane e ends up owning expert e's logit.
      float logit = -INFINITY;
#pragma unroll
      for (int e = 0; e < EP; ++e) {
        float s = wave_sum(acc[t][e]);
        if (lane == e) logit = s;
      }
      const bool live = lane < n_experts;
      if (live && bias) logit += bias[lane];
      if (!live) logit = -INFINITY;
      const int64_t tok = t0 + t;
      if (tok >= n_tokens) continue;  // uniform across the wave
      if (logits_out && live) logits_out[tok * n_experts + lane] = logit;

      const float m = wave_max(logit);
      const float p = live ? expf(logit - m) : 0.f;
      const float denom = wave_sum(p);
      float score = live ? p / denom : -1.f;

      float sel_w = 0.f;  // lane j < top_k keeps the j-th pick
      int sel_i = 0;
      float picked_sum = 0.f;
      for (int j = 0; j < top_k; ++j) {
        float bv = score;
        int bi = lane;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          float ov = __shfl_xor(bv, o, kWave);
          int oi = __shfl_xor(bi, o, kWave);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
        if (lane == j) {
          sel_w = bv;
          sel_i = bi;
        }
        picked_sum += bv;
        if (lane == bi) score = -1.f;
      }
      if (norm_topk && top_k > 1) sel_w = sel_w / (picked_sum + 1e-20f);
      if (lane < top_k) {
        topk_idx[tok * top_k + lane] = sel_i;
        if (topk_idx64) topk_idx64[tok * top_k + lane] = sel_i;
        topk_weight[tok * top_k + lane] = sel_w;
      }
    }
  }
}

template <typename XT, typename WT, int EP, int TOK>
int launch_gate(const void *x, const void *w, const float *bias, int64_t n_tokens, int hidden,
                int n_experts, int top_k, int norm, int32_t *idx, int64_t *idx64, float *wt,
                float *logits, hipStream_t stream) {
  const size_t w_bytes = (size_t)n_experts * hidden * sizeof(WT);
  const int64_t groups = (n_tokens + TOK - 1) / TOK;
  int64_t blocks = (groups + kGateWaves - 1) / kGateWaves;
  if (blocks > 512) blocks = 512;
  if (blocks < 1) blocks = 1;
  if (w_bytes <= 160 * 1024 - 1024) {
    auto kern = gate_topk_kernel<XT, WT, EP, TOK, true>;
    if (w_bytes > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)w_bytes);
      if (e != hipSuccess) return fail(DICE_ERR_LAUNCH, "gate: LDS attribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kGateWaves * kWave), w_bytes, stream,
                       (const XT *)x, (const WT *)w, bias, n_tokens, hidden, n_experts, top_k, norm,
                       idx, idx64, wt, logits);
  } else {
    auto kern = gate_topk_kernel<XT, WT, EP, TOK, false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kGateWaves * kWave), 0, stream,
                       (const XT *)x, (const WT *)w, bias, n_tokens, hidden, n_experts, top_k, norm,
                       idx, idx64, wt, logits);
  }
  return launch_status("dice_gate_topk");
}

template <typename XT, typename WT>
int dispatch_experts(const void *x, const void *w, const float *bias, int64_t n_tokens, int hidden,
                     int n_experts, int top_k, int norm, int32_t *idx, int64_t *idx64, float *wt,
                     float *logits, hipStream_t s) {
  if (n_experts <= 8)
    return launch_gate<XT, WT, 8, 4>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  if (n_experts <= 16)
    return launch_gate<XT, WT, 16, 4>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  if (n_experts <= 32)
    return launch_gate<XT, WT, 32, 2>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  return launch_gate<XT, WT, 64, 1>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
}

// The router matrix is either fp32 or stored in the activation dtype.
template <typename XT>
int dispatch_wtype(int x_dtype, int w_dtype, const void *x, const void *w, const float *bias,
                   int64_t n_tokens, int hidden, int n_experts, int top_k, int norm, int32_t *idx,
                   int64_t *idx64, float *wt, float *logits, hipStream_t s) {
  if (w_dtype == DICE_F32)
    return dispatch_experts<XT, float>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  if (w_dtype == x_dtype)
    return dispatch_experts<XT, XT>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  return fail(DICE_ERR_UNSUPPORTED, "dice_gate_topk: w_dtype %d must be F32 or equal x_dtype %d", w_dtype, x_dtype);
}

}  // namespace
}  // namespace dice

extern "C" int dice_gate_topk(const void *x, int x_dtype, const void *w, int w_dtype,
                              const float *bias, int64_t n_tokens, int hidden, int n_experts,
                              int top_k, int norm_topk_prob, int32_t *topk_idx,
                              int64_t *topk_idx64, float *topk_weight, float *logits,
                              void *stream) {
  using namespace dice;
  DICE_REQUIRE(x && w && topk_idx && topk_weight, DICE_ERR_BAD_ARG, "dice_gate_topk: null pointer");
  DICE_REQUIRE(n_tokens >= 0, DICE_ERR_BAD_ARG, "dice_gate_topk: n_tokens %lld < 0", (long long)n_tokens);
  DICE_REQUIRE(hidden > 0 && hidden % 8 == 0, DICE_ERR_BAD_ARG,
               "dice_gate_topk: hidden %d must be a positive multiple of 8", hidden);
  DICE_REQUIRE(n_experts >= 1 && n_experts <= 64, DICE_ERR_UNSUPPORTED,
               "dice_gate_topk: n_experts %d outside [1, 64]", n_experts);
  DICE_REQUIRE(top_k >= 1 && top_k <= 8 && top_k <= n_experts, DICE_ERR_BAD_ARG,
               "dice_gate_topk: top_k %d outside [1, min(8, n_experts)]", top_k);
  if (n_tokens == 0) return DICE_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (x_dtype) {
    case DICE_F32:
      return dispatch_wtype<float>(x_dtype, w_dtype, x, w, bias, n_tokens, hidden, n_experts, top_k,
                                   norm_topk_prob, topk_idx, topk_idx64, topk_weight, logits, s);
    case DICE_BF16:
      return dispatch_wtype<bf16_t>(x_dtype, w_dtype, x, w, bias, n_tokens, hidden, n_experts, top_k,
                                    norm_topk_prob, topk_idx, topk_idx64, topk_weight, logits, s);
    case DICE_F16:
      return dispatch_wtype<f16_t>(x_dtype, w_dtype, x, w, bias, n_tokens, hidden, n_experts, top_k,
                                   norm_topk_prob, topk_idx, topk_idx64, topk_weight, logits, s);
  }
  return fail(DICE_ERR_UNSUPPORTED, "dice_gate_topk: unsupported x_dtype %d", x_dtype);
}
