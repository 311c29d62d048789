// Router: fp32 logits -> softmax -> top-k.
//
// Replaces MoEGate.forward, inference branch (reference models.py:179-196).
// HBM-bound: the only large operand is x, read exactly once (n_tokens*hidden
// elements).  Two kernels: 16-bit activations with a router matrix of the same
// type and at most 32 experts (every DiT-MoE size) multiply on the matrix pipe,
// 32 tokens per workgroup (gate_topk_mfma_kernel, below); everything else -
// fp32, an fp32 router matrix for 16-bit activations, more experts, odd hidden
// sizes - takes gate_topk_kernel, one wavefront per 64 / E tokens, where the
// router matrix comes from the vector cache, or, when it is too large for
// that, from LDS, and each wave keeps 64/E tokens in flight so one read of a
// router chunk feeds that many dot-product updates.  A third kernel
// (ln_modulate_route_kernel) runs the caller's LayerNorm + modulation prologue
// and the matrix-pipe router in one launch.
#include <type_traits>

#include "modulate_row.h"

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

// 8-element dot product accumulate.  bf16 x bf16 uses the packed
// v_dot2_f32_bf16 (exact products, fp32 accumulation); everything else widens
// to fp32 FMAs.
template <typename XT, typename WT>
__device__ __forceinline__ float dot8(const Vec8<XT> &x, const Vec8<WT> &w, float acc) {
#pragma unroll
  for (int i = 0; i < 8; ++i) acc = fmaf(x.get(i), w.get(i), acc);
  return acc;
}
template <>
__device__ __forceinline__ float dot8<bf16_t, bf16_t>(const Vec8<bf16_t> &x, const Vec8<bf16_t> &w,
                                                      float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16x2_t a = {x.v[2 * i], x.v[2 * i + 1]};
    const bf16x2_t b = {w.v[2 * i], w.v[2 * i + 1]};
    acc = __builtin_amdgcn_fdot2_f32_bf16(a, b, acc, false);
  }
  return acc;
}

// Sums v[0..V-1] across the 64 lanes; lane l returns the total of v[l % V].
// Each step halves the values a lane keeps (the partner takes the other half),
// so the reduction over the low log2(V) lane bits costs V - 1 lane exchanges
// instead of V x log2(V); the remaining lane bits (V < 64) take one plain
// butterfly each.  The summation order is fixed.
template <int HALF, int V>
__device__ __forceinline__ void reduce_transpose_step(float (&v)[V], int lane) {
  const bool upper = lane & HALF;  // partner distance == number of values kept
#pragma unroll
  for (int i = 0; i < HALF; ++i) {
    const float keep = upper ? v[i + HALF] : v[i];
    const float send = upper ? v[i] : v[i + HALF];
    v[i] = keep + __shfl_xor(send, HALF, kWave);
  }
}
template <int HALF, int V>
__device__ __forceinline__ void reduce_transpose_from(float (&v)[V], int lane) {
  if constexpr (HALF >= 1) {
    reduce_transpose_step<HALF, V>(v, lane);
    reduce_transpose_from<HALF / 2, V>(v, lane);
  }
}
template <int V>
__device__ __forceinline__ float reduce_transpose(float (&v)[V], int lane) {
  reduce_transpose_from<V / 2, V>(v, lane);
  float r = v[0];
#pragma unroll
  for (int o = V; o < kWave; o <<= 1) r += __shfl_xor(r, o, kWave);
  return r;
}

// One wavefront routes TOK <= 64 / EP tokens at a time: lanes split the hidden
// dimension, every lane accumulates all TOK x EP dot products, the transposing
// reduction leaves lane t*EP + e (and, for TOK x EP < 64, its copies further up)
// with logit (t, e), and softmax / top-k then run inside each group of EP lanes
// for all TOK tokens at once.  (TOK = 64 / EP in every launch: a quarter of that
// per wave, four times the waves, measured slower.)
template <typename XT, typename WT, int EP, int TOK, bool W_IN_LDS>
__global__ __launch_bounds__(kGateWaves *kWave) void gate_topk_kernel(
    const XT *__restrict__ x, const WT *__restrict__ w, const float *__restrict__ bias,
    int64_t n_tokens, int hidden, int n_experts, int top_k, int norm_topk,
    int32_t *__restrict__ topk_idx, int64_t *__restrict__ topk_idx64,
    float *__restrict__ topk_weight, float *__restrict__ logits_out) {
  constexpr int V = TOK * EP;  // dot products per lane
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int chunks = hidden / 8;

  const int my_tok = (lane % V) / EP, my_e = lane % EP;
  const bool live = my_e < n_experts;
  const int64_t groups = (n_tokens + TOK - 1) / TOK;
  // A lane's share of a token row is every 64th 16-byte chunk.  Up to kBatch of
  // them per token are requested at once (a whole 16-bit row up to hidden = 2048), so a
  // group costs one memory round trip, not one per chunk; the first group's
  // loads are issued before the router matrix is staged, the next group's before
  // this group's reduction and softmax.
  constexpr int kBatch = sizeof(XT) == 4 ? 2 : 4;  // (fp32 rows take twice the registers per chunk)
  Vec8<XT> xv[kBatch][TOK];
  auto load_batch = [&](int64_t g, int c0) {
    const int64_t t0 = g * TOK;
#pragma unroll
    for (int r = 0; r < kBatch; ++r) {
      const int c = c0 + r * kWave + lane;
      if (c < chunks) {
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
          const int64_t tt = t0 + t < n_tokens ? t0 + t : n_tokens - 1;
          xv[r][t] = load8(x + tt * hidden + (size_t)c * 8);
        }
      }
    }
  };
  int64_t g = (int64_t)blockIdx.x * kGateWaves + wave;
  if (g < groups) load_batch(g, 0);

  const WT *wsrc = w;
  if (W_IN_LDS) {
    WT *wl = reinterpret_cast<WT *>(lds_raw);
    const int total = n_experts * chunks;
    for (int c = threadIdx.x; c < total; c += blockDim.x)
      *reinterpret_cast<Vec8<WT> *>(wl + (size_t)c * 8) = load8(w + (size_t)c * 8);
    __syncthreads();
    wsrc = wl;
  }

  for (; g < groups; g += (int64_t)gridDim.x * kGateWaves) {
    const int64_t t0 = g * TOK;
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    for (int c0 = 0; c0 < chunks; c0 += kBatch * kWave) {
      if (c0 > 0) load_batch(g, c0);  // rows longer than one batch: the next piece, after the last was consumed
#pragma unroll
      for (int r = 0; r < kBatch; ++r) {
        const int c = c0 + r * kWave + lane;
        if (c < chunks) {
          // Router rows eight experts at a time: the eight reads are issued together
          // and waited for once (experts past n_experts re-read the last row; their
          // logits are discarded below), no branch per expert.
          constexpr int EB = EP < 8 ? EP : 8;
#pragma unroll
          for (int e0 = 0; e0 < EP; e0 += EB) {
            Vec8<WT> wv[EB];
#pragma unroll
            for (int e = 0; e < EB; ++e) {
              const int row = e0 + e < n_experts ? e0 + e : n_experts - 1;
              wv[e] = load8(wsrc + ((size_t)row * chunks + c) * 8);
            }
#pragma unroll
            for (int e = 0; e < EB; ++e)
#pragma unroll
              for (int t = 0; t < TOK; ++t) acc[t * EP + e0 + e] = dot8<XT, WT>(xv[r][t], wv[e], acc[t * EP + e0 + e]);
          }
        }
      }
    }
    const int64_t g_next = g + (int64_t)gridDim.x * kGateWaves;
    if (g_next < groups) load_batch(g_next, 0);
    float logit = reduce_transpose<V>(acc, lane);
    if (live && bias) logit += bias[my_e];
    if (!live) logit = -INFINITY;
    const int64_t tok = t0 + my_tok;
    const bool tok_ok = tok < n_tokens && lane < V;  // (lanes from V on hold copies)
    if (logits_out && live && tok_ok) logits_out[tok * n_experts + my_e] = logit;

    // softmax inside the EP-lane group
    float m = logit;
#pragma unroll
    for (int o = EP / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, kWave));
    const float p = live ? expf(logit - m) : 0.f;
    float denom = p;
#pragma unroll
    for (int o = EP / 2; o > 0; o >>= 1) denom += __shfl_xor(denom, o, kWave);
    float score = live ? p / denom : -1.f;

    float sel_w = 0.f;  // lane j of the group keeps the j-th pick
    int sel_i = 0;
    float picked_sum = 0.f;
    for (int j = 0; j < top_k; ++j) {
      float bv = score;
      int bi = my_e;
#pragma unroll
      for (int o = EP / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, kWave);
        const int oi = __shfl_xor(bi, o, kWave);
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (my_e == j) {
        sel_w = bv;
        sel_i = bi;
      }
      picked_sum += bv;
      if (my_e == bi) score = -1.f;
    }
    if (norm_topk && top_k > 1) sel_w = sel_w / (picked_sum + 1e-20f);
    if (tok_ok && my_e < top_k) {
      topk_idx[tok * top_k + my_e] = sel_i;
      if (topk_idx64) topk_idx64[tok * top_k + my_e] = sel_i;
      topk_weight[tok * top_k + my_e] = sel_w;
    }
  }
}

template <typename XT, typename WT, int EP>
int launch_gate(const void *x, const void *w, const float *bias, int64_t n_tokens, int hidden,
                int n_experts, int top_k, int norm, int32_t *idx, int64_t *idx64, float *wt,
                float *logits, hipStream_t stream) {
  constexpr int TOK = kWave / EP;
  const size_t w_bytes = (size_t)n_experts * hidden * sizeof(WT);
  const int64_t groups = (n_tokens + TOK - 1) / TOK;
  int64_t blocks = (groups + kGateWaves - 1) / kGateWaves;
  if (blocks > 512) blocks = 512;
  if (blocks < 1) blocks = 1;
  // A router matrix that fits the compute unit's vector cache beside the token
  // rows streaming through it is read from there: staging it in LDS first puts a
  // load, a store and a workgroup barrier in front of the first product.
  if (w_bytes > 24 * 1024 && w_bytes <= 160 * 1024 - 1024) {
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


// ---------------------------------------------------------------------------
// The router on the matrix pipe (16-bit activations and router matrix, at most
// 32 experts).  The kernel above spends its time issuing instructions - about
// 3000 per wave for eight tokens - not waiting for memory; here a workgroup
// routes 32 tokens with v_mfma_f32_32x32x16: the experts are the 32 rows of the
// left operand (rows past n_experts repeat the last one and are ignored), the
// tokens the 32 columns of the right one, so lane l supplies 16 bytes of token
// l % 32 per step - straight from memory, no LDS staging.  The hidden dimension
// is cut into WPB contiguous segments, one per wave, of which the two lane
// halves take alternate 16-byte chunks (a load then touches 32 bytes of 32
// lines; with a segment per lane half it was 16 bytes of 64 lines and the
// launch 0.8 us longer): a wave
// requests its whole share (at most kRouterMaxSteps x 2 loads of 1 KB) before
// the first product, the WPB partial logit tiles are added in wave order
// through LDS, and the first wave finishes softmax and top-k with all of a
// token's logits in one lane.  Summation order is fixed (per lane half, per
// wave, then over the waves), so results do not depend on timing.
constexpr int kRouterMaxSteps = 18;
template <typename T> struct RouterMfma;
template <> struct RouterMfma<bf16_t> {
  static __device__ __forceinline__ f32x16_t mul(bf16x8_t a, bf16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct RouterMfma<f16_t> {
  static __device__ __forceinline__ f32x16_t mul(f16x8_t a, f16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// Second half of the matrix-pipe router, run by one wave: adds the `waves`
// partial logit tiles in `part` ([waves][EP / 2][64] floats in LDS, lane (col,
// half), register a = expert 8 (a / 4) + 4 half + a % 4 of token col) in wave
// order, then softmax and top-k with all of a token's logits in one lane.
template <int EP>
__device__ __forceinline__ void router_mfma_finish(
    const float *part, int waves, int lane, int64_t tok, const float *__restrict__ bias, int64_t n_tokens,
    int n_experts, int top_k, int norm_topk, int32_t *__restrict__ topk_idx, int64_t *__restrict__ topk_idx64,
    float *__restrict__ topk_weight, float *__restrict__ logits_out) {
  constexpr int NR = EP / 2;
  const int half = lane >> 5;
  float mine[NR], other[NR];
#pragma unroll
  for (int a = 0; a < NR; ++a) {
    float v = part[a * kWave + lane];
    for (int q = 1; q < waves; ++q) v += part[(q * NR + a) * kWave + lane];
    mine[a] = v;
  }
#pragma unroll
  for (int a = 0; a < NR; ++a) other[a] = __shfl_xor(mine[a], 32, kWave);
  float score[EP];
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    const int a = (e / 8) * 4 + e % 4;
    float logit = ((e % 8) / 4 == half) ? mine[a] : other[a];
    if (e < n_experts) {
      if (bias) logit += bias[e];
      if (logits_out && half == 0 && tok < n_tokens) logits_out[tok * n_experts + e] = logit;
    } else {
      logit = -INFINITY;
    }
    score[e] = logit;
    m = fmaxf(m, logit);
  }
  float denom = 0.f;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    score[e] = e < n_experts ? expf(score[e] - m) : 0.f;
    denom += score[e];
  }
#pragma unroll
  for (int e = 0; e < EP; ++e) score[e] = e < n_experts ? score[e] / denom : -1.f;
  // top-k: repeated arg-max, ties to the lower expert id (ascending scan, strict compare)
  float sel_w[8];
  int sel_i[8];
  float picked_sum = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    sel_w[j] = 0.f;
    sel_i[j] = 0;
    if (j < top_k) {
      float bv = -2.f;
      int bi = 0;
#pragma unroll
      for (int e = 0; e < EP; ++e)
        if (score[e] > bv) {
          bv = score[e];
          bi = e;
        }
#pragma unroll
      for (int e = 0; e < EP; ++e)
        if (e == bi) score[e] = -1.f;
      sel_w[j] = bv;
      sel_i[j] = bi;
      picked_sum += bv;
    }
  }
  if (half != 0 || tok >= n_tokens) return;
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (j < top_k) {
      const float wgt = (norm_topk && top_k > 1) ? sel_w[j] / (picked_sum + 1e-20f) : sel_w[j];
      topk_idx[tok * top_k + j] = sel_i[j];
      if (topk_idx64) topk_idx64[tok * top_k + j] = sel_i[j];
      topk_weight[tok * top_k + j] = wgt;
    }
}
template <typename T, int EP, int WPB>
__device__ __forceinline__ void gate_topk_mfma_body(
    const T *__restrict__ x, const T *__restrict__ w, const float *__restrict__ bias, int64_t n_tokens,
    int hidden, int n_experts, int top_k, int norm_topk, int32_t *__restrict__ topk_idx,
    int64_t *__restrict__ topk_idx64, float *__restrict__ topk_weight, float *__restrict__ logits_out) {
  constexpr int NR = EP / 2;  // accumulator registers of a lane that hold experts below EP
  __shared__ float part[WPB][NR][kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int col = lane & 31, half = lane >> 5;
  const int64_t tok = (int64_t)blockIdx.x * 32 + col;
  const int64_t tok_c = tok < n_tokens ? tok : n_tokens - 1;   // (columns past the end repeat the last token)
  const int steps = hidden / 16 / WPB;                         // per wave; at most kRouterMaxSteps
  // A wave's segment of the hidden dimension is 2 x steps chunks of 16 bytes; the
  // two lane halves take alternate chunks, so that a load instruction touches 32
  // bytes of each of its 32 rows' lines, not 16 bytes of 64 lines.
  const int seg = (wave * 2 * steps + half) * 8;
  const T *xp = x + tok_c * hidden + seg;
  const T *wp = w + (size_t)(col < n_experts ? col : n_experts - 1) * hidden + seg;
  Vec8<T> xv[kRouterMaxSteps], wv[kRouterMaxSteps];
#pragma unroll
  for (int s = 0; s < kRouterMaxSteps; ++s) {
    const int at = s < steps ? s : 0;   // (no branch around a load: steps past the end re-read the first chunk)
    xv[s] = load8(xp + at * 16);
    wv[s] = load8(wp + at * 16);
  }
  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
  for (int s = 0; s < kRouterMaxSteps; ++s)
    if (s < steps) acc = RouterMfma<T>::mul(wv[s].v, xv[s].v, acc);
  // lane (col, half), register a: logit of expert 8 (a / 4) + 4 half + a % 4 for token col
#pragma unroll
  for (int a = 0; a < NR; ++a) part[wave][a][lane] = acc[a];
  __syncthreads();
  if (wave != 0) return;
  router_mfma_finish<EP>(&part[0][0][0], WPB, lane, tok, bias, n_tokens, n_experts, top_k, norm_topk, topk_idx,
                         topk_idx64, topk_weight, logits_out);
}
// (builtins that only exist for the device stay out of the __global__ template's own body)
template <typename T, int EP, int WPB>
__global__ __launch_bounds__(WPB *kWave) void gate_topk_mfma_kernel(
    const T *__restrict__ x, const T *__restrict__ w, const float *__restrict__ bias, int64_t n_tokens,
    int hidden, int n_experts, int top_k, int norm_topk, int32_t *__restrict__ topk_idx,
    int64_t *__restrict__ topk_idx64, float *__restrict__ topk_weight, float *__restrict__ logits_out) {
  gate_topk_mfma_body<T, EP, WPB>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm_topk, topk_idx, topk_idx64,
                                  topk_weight, logits_out);
}

// Waves per 32-token workgroup of the matrix-pipe router for this hidden size
// (0: it does not apply).
inline int router_mfma_waves(int hidden) {
  if (hidden % 64 != 0) return 0;
  const int steps = hidden / 16;
  if (steps / 4 <= kRouterMaxSteps) return 4;
  if (steps % 8 == 0 && steps / 8 <= kRouterMaxSteps) return 8;
  return 0;
}
template <typename T, int EP>
int launch_gate_mfma(const void *x, const void *w, const float *bias, int64_t n_tokens, int hidden, int n_experts,
                     int top_k, int norm, int32_t *idx, int64_t *idx64, float *wt, float *logits,
                     hipStream_t stream) {
  const int wpb = router_mfma_waves(hidden);
  const unsigned blocks = (unsigned)((n_tokens + 31) / 32);
  if (wpb == 4)
    hipLaunchKernelGGL((gate_topk_mfma_kernel<T, EP, 4>), dim3(blocks), dim3(4 * kWave), 0, stream, (const T *)x,
                       (const T *)w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits);
  else
    hipLaunchKernelGGL((gate_topk_mfma_kernel<T, EP, 8>), dim3(blocks), dim3(8 * kWave), 0, stream, (const T *)x,
                       (const T *)w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits);
  return launch_status("dice_gate_topk");
}

// ---------------------------------------------------------------------------
// The caller's prologue and the router in one launch: a workgroup of 16 waves
// takes 32 tokens.  Each wave normalises and modulates two rows in registers
// (both requested up front: one memory round trip), writes them to the layer
// input in HBM and to LDS; after one barrier the first `wpb` waves multiply the
// LDS copy with the router matrix exactly as gate_topk_mfma_body multiplies the
// rows it loads from memory (same segments of the hidden dimension per wave and
// lane half, same order of products and sums: bit-identical logits), and the
// first wave finishes.  Against the two separate launches the modulated rows
// are not read back from memory and one launch ramp goes away.  LDS rows are
// one 16-byte chunk longer than the row, so the 32 lanes of a half-wave, which
// read the same chunk of 32 different rows, fall into different banks.
constexpr int kRouteWaves = 16;
constexpr int kRouteChunks = 3;   // 16-byte chunks of a row per lane: rows up to 1536 16-bit elements

template <typename T, int EP>
__device__ __forceinline__ void ln_modulate_route_body(
    const Chunk<T> *__restrict__ x, const Chunk<T> *__restrict__ shift, const Chunk<T> *__restrict__ scale,
    Chunk<T> *__restrict__ out, int64_t n_tokens, int chunks_per_row, int64_t tokens_per_sample, float inv_hidden,
    float eps, const T *__restrict__ w, const float *__restrict__ bias, int n_experts, int top_k, int norm_topk,
    int wpb, int32_t *__restrict__ topk_idx, float *__restrict__ topk_weight) {
  constexpr int NR = EP / 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int pitch = chunks_per_row + 1;                         // LDS row pitch in chunks
  Chunk<T> *rows = reinterpret_cast<Chunk<T> *>(lds_raw);       // [32][pitch]
  float *part = reinterpret_cast<float *>(lds_raw + (size_t)32 * pitch * sizeof(Chunk<T>));  // [wpb][NR][64]
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t t_base = (int64_t)blockIdx.x * 32;

  Chunk<T> v[2][kRouteChunks], ms[2][kRouteChunks], mh[2][kRouteChunks];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t t = t_base + wave * 2 + j;
    const int64_t tt = t < n_tokens ? t : n_tokens - 1;         // (rows past the end repeat the last token)
    const int64_t b = tt / tokens_per_sample;
    const Chunk<T> *row = x + tt * chunks_per_row;
    const Chunk<T> *sc = scale + b * chunks_per_row;
    const Chunk<T> *sh = shift + b * chunks_per_row;
#pragma unroll
    for (int i = 0; i < kRouteChunks; ++i) {
      const int c = lane + i * kWave;
      if (c < chunks_per_row) {
        v[j][i] = row[c];
        ms[j][i] = sc[c];
        mh[j][i] = sh[c];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 2; ++j)
    ln_modulate_row<T, kRouteChunks>(v[j], ms[j], mh[j], lane, chunks_per_row, inv_hidden, eps);

  // The router matrix is requested before the rows are stored: the wait for it
  // behind the barrier then does not wait for the stores as well (one counter
  // covers both, in issue order).
  const int col = lane & 31, half = lane >> 5;
  const int steps = chunks_per_row / 2 / wpb;                   // per wave; at most kRouterMaxSteps
  const int seg = wave * 2 * steps + half;                      // this lane's first chunk; it takes every other one
  Vec8<T> wv[kRouterMaxSteps];
  if (wave < wpb) {
    const T *wp = w + ((size_t)(col < n_experts ? col : n_experts - 1) * chunks_per_row + seg) * 8;
#pragma unroll
    for (int s = 0; s < kRouterMaxSteps; ++s) wv[s] = load8(wp + (s < steps ? s : 0) * 16);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t t = t_base + wave * 2 + j;
    Chunk<T> *dst = out + t * chunks_per_row;
    Chunk<T> *lrow = rows + (wave * 2 + j) * pitch;
#pragma unroll
    for (int i = 0; i < kRouteChunks; ++i) {
      const int c = lane + i * kWave;
      if (c < chunks_per_row) {
        lrow[c] = v[j][i];
        if (t < n_tokens) dst[c] = v[j][i];
      }
    }
  }
  block_lds_barrier();   // (LDS only: the rows' way to memory is not waited for)
  if (wave < wpb) {
    const Chunk<T> *xp = rows + col * pitch + seg;
    f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    // LDS reads six at a time in front of their products (no branch around a read:
    // steps past the end re-read the first chunk)
    constexpr int kReads = 6;
#pragma unroll
    for (int s0 = 0; s0 < kRouterMaxSteps; s0 += kReads) {
      Chunk<T> xb[kReads];
#pragma unroll
      for (int i = 0; i < kReads; ++i) xb[i] = xp[s0 + i < steps ? 2 * (s0 + i) : 0];
#pragma unroll
      for (int i = 0; i < kReads; ++i)
        if (s0 + i < steps) acc = RouterMfma<T>::mul(wv[s0 + i].v, xb[i].v, acc);
    }
#pragma unroll
    for (int a = 0; a < NR; ++a) part[(wave * NR + a) * kWave + lane] = acc[a];
  }
  block_lds_barrier();
  if (wave != 0) return;
  router_mfma_finish<EP>(part, wpb, lane, t_base + col, bias, n_tokens, n_experts, top_k, norm_topk, topk_idx,
                         nullptr, topk_weight, nullptr);
}
template <typename T, int EP>
__global__ __launch_bounds__(kRouteWaves *kWave) void ln_modulate_route_kernel(
    const Chunk<T> *__restrict__ x, const Chunk<T> *__restrict__ shift, const Chunk<T> *__restrict__ scale,
    Chunk<T> *__restrict__ out, int64_t n_tokens, int chunks_per_row, int64_t tokens_per_sample, float inv_hidden,
    float eps, const T *__restrict__ w, const float *__restrict__ bias, int n_experts, int top_k, int norm_topk,
    int wpb, int32_t *__restrict__ topk_idx, float *__restrict__ topk_weight) {
  ln_modulate_route_body<T, EP>(x, shift, scale, out, n_tokens, chunks_per_row, tokens_per_sample, inv_hidden, eps,
                                w, bias, n_experts, top_k, norm_topk, wpb, topk_idx, topk_weight);
}

template <typename T, int EP>
int launch_ln_modulate_route(const void *x, const void *shift, const void *scale, void *out, int64_t n_tokens,
                             int hidden, int64_t tokens_per_sample, float eps, const void *w, const float *bias,
                             int n_experts, int top_k, int norm, int32_t *idx, float *wt, hipStream_t stream) {
  const int chunks = hidden / 8;
  const int wpb = router_mfma_waves(hidden);
  const size_t lds = (size_t)32 * (chunks + 1) * 16 + (size_t)wpb * (EP / 2) * kWave * sizeof(float);
  auto kern = ln_modulate_route_kernel<T, EP>;
  // More than 64 KB of dynamic LDS has to be allowed per kernel and device, once.
  constexpr int kMaxDevices = 64;
  static size_t lds_allowed[kMaxDevices] = {};   // (per instantiation)
  int dev = 0;
  DICE_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices || lds > lds_allowed[dev]) {
    DICE_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 (int)lds));
    if (dev >= 0 && dev < kMaxDevices) lds_allowed[dev] = lds;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((n_tokens + 31) / 32)), dim3(kRouteWaves * kWave), lds, stream,
                     (const Chunk<T> *)x, (const Chunk<T> *)shift, (const Chunk<T> *)scale, (Chunk<T> *)out, n_tokens,
                     chunks, tokens_per_sample, 1.0f / (float)hidden, eps, (const T *)w, bias, n_experts, top_k, norm,
                     wpb, idx, wt);
  return launch_status("dice_moe_forward_modulated");
}
template <typename T>
int ln_modulate_route_experts(const void *x, const void *shift, const void *scale, void *out, int64_t n_tokens,
                              int hidden, int64_t tokens_per_sample, float eps, const void *w, const float *bias,
                              int n_experts, int top_k, int norm, int32_t *idx, float *wt, hipStream_t s) {
  if (n_experts <= 8)
    return launch_ln_modulate_route<T, 8>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, w, bias,
                                          n_experts, top_k, norm, idx, wt, s);
  if (n_experts <= 16)
    return launch_ln_modulate_route<T, 16>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, w, bias,
                                           n_experts, top_k, norm, idx, wt, s);
  return launch_ln_modulate_route<T, 32>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, w, bias,
                                         n_experts, top_k, norm, idx, wt, s);
}

template <typename XT, typename WT>
int dispatch_experts(const void *x, const void *w, const float *bias, int64_t n_tokens, int hidden,
                     int n_experts, int top_k, int norm, int32_t *idx, int64_t *idx64, float *wt,
                     float *logits, hipStream_t s) {
  if constexpr (std::is_same<XT, WT>::value && sizeof(XT) == 2) {
    if (n_experts <= 32 && n_tokens < (1ll << 31) / 32 && router_mfma_waves(hidden) != 0) {
      if (n_experts <= 8)
        return launch_gate_mfma<XT, 8>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
      if (n_experts <= 16)
        return launch_gate_mfma<XT, 16>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
      return launch_gate_mfma<XT, 32>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
    }
  }
  if (n_experts <= 8)
    return launch_gate<XT, WT, 8>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  if (n_experts <= 16)
    return launch_gate<XT, WT, 16>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  if (n_experts <= 32)
    return launch_gate<XT, WT, 32>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
  return launch_gate<XT, WT, 64>(x, w, bias, n_tokens, hidden, n_experts, top_k, norm, idx, idx64, wt, logits, s);
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

bool ln_modulate_route_applies(int act_dtype, int gate_w_dtype, int64_t n_tokens, int hidden, int n_experts) {
  return (act_dtype == DICE_BF16 || act_dtype == DICE_F16) && gate_w_dtype == act_dtype && n_experts <= 32 &&
         n_tokens >= 1 && n_tokens < (1ll << 31) / 32 && hidden <= kRouteChunks * kWave * 8 &&
         router_mfma_waves(hidden) != 0;
}

int ln_modulate_route_impl(const void *x, const void *shift, const void *scale, void *out, int dtype,
                           int64_t n_tokens, int hidden, int64_t tokens_per_sample, float eps, const void *gate_w,
                           const float *gate_bias, int n_experts, int top_k, int norm_topk_prob, int32_t *topk_idx,
                           float *topk_weight, void *stream) {
  DICE_REQUIRE(ln_modulate_route_applies(dtype, dtype, n_tokens, hidden, n_experts), DICE_ERR_UNSUPPORTED,
               "ln_modulate + router: dtype %d, hidden %d, %d experts are outside the fused kernel", dtype, hidden,
               n_experts);
  DICE_REQUIRE(x && shift && scale && out && gate_w && topk_idx && topk_weight, DICE_ERR_BAD_ARG,
               "ln_modulate + router: null pointer");
  DICE_REQUIRE(tokens_per_sample >= 1 && eps >= 0.f, DICE_ERR_BAD_ARG,
               "ln_modulate + router: tokens_per_sample %lld, eps %g", (long long)tokens_per_sample, (double)eps);
  DICE_REQUIRE(top_k >= 1 && top_k <= 8 && top_k <= n_experts, DICE_ERR_BAD_ARG,
               "ln_modulate + router: top_k %d outside [1, min(8, n_experts)]", top_k);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DICE_BF16)
    return ln_modulate_route_experts<bf16_t>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, gate_w,
                                             gate_bias, n_experts, top_k, norm_topk_prob, topk_idx, topk_weight, s);
  return ln_modulate_route_experts<f16_t>(x, shift, scale, out, n_tokens, hidden, tokens_per_sample, eps, gate_w,
                                          gate_bias, n_experts, top_k, norm_topk_prob, topk_idx, topk_weight, s);
}

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
