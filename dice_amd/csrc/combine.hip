// Combine: routing-weighted sum of a token's k expert rows, the shared-expert
// add, and the staleness-cache blend / put, in one pass.
//
// Replaces mul_ + scatter_reduce_ of SparseMoeBlock.moe_infer (reference
// models.py:377-381) = final.mul_(w).view(N,k,h).sum(1) of moe_infer_ep
// (expertpara/ep_fwd.py:190-195), `y + shared_experts(identity)`
// (models.py:355-357) and the skip blend / put (ep_fwd.py:176-188).
//
// HBM-bound.  Each thread owns one 16-byte column chunk of one token: it reads
// the k slot rows (or the cached row for the skipped slot), the shared row,
// and writes y (and the cache row on a "put" step).  Accumulation is fp32 in
// slot order with a single rounding, no atomics, so the result is
// deterministic.
//
// Optionally also the caller's epilogue, out = resid + gate[b] * y
// (x + gate_mlp.unsqueeze(1) * self.moe(...) of DiTBlock.forward, reference
// models.py:519; b = token / tokens_per_sample), applied to the fp32 sum before
// the one rounding: two more reads per element instead of the reference's two
// extra elementwise kernels over [N, D].
#include "common.h"

namespace dice {
namespace {

template <typename T> struct Pack;  // 16 bytes of T
template <> struct Pack<float> {
  static constexpr int kN = 4;
  f32x4_t v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = f; }
};
template <> struct Pack<bf16_t> {
  static constexpr int kN = 8;
  bf16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (bf16_t)f; }
};
template <> struct Pack<f16_t> {
  static constexpr int kN = 8;
  f16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (f16_t)f; }
};

constexpr int kMaxTopK = 8;

// What one routing slot of a token contributes: its weight and where its row
// comes from (the cache, the slot rows, or nowhere: a zero row).
template <typename T>
struct SlotSource {
  float w;
  const Pack<T> *row;   // nullptr: a zero row
  bool put;             // the row also goes to cache_out
};
template <typename T>
__device__ __forceinline__ SlotSource<T> slot_source(
    int64_t s, int64_t chunk_of_token, int c, int vec_per_row, const Pack<T> *__restrict__ slot_out,
    const int32_t *__restrict__ inv_perm, const float *__restrict__ topk_weight,
    const uint8_t *__restrict__ skip_mask, const Pack<T> *__restrict__ cache_in, bool have_cache_out) {
  SlotSource<T> r;
  r.w = topk_weight[s];
  const bool skipped = skip_mask && skip_mask[s];
  if (skipped && cache_in) {
    r.row = cache_in + chunk_of_token;
    r.put = false;
  } else {
    // A slot the dispatch left out (masked, or an expert id outside the
    // table: inv_perm = -1) contributes a zero row, as the zero-initialised
    // buffer of the reference's _local_combine does (ep_fwd.py:350-354).
    const int64_t src = inv_perm ? (int64_t)inv_perm[s] : s;
    r.row = src >= 0 ? slot_out + src * vec_per_row + c : nullptr;
    r.put = skipped && have_cache_out;
  }
  return r;
}

// K > 0: top_k known at compile time - the routing tables of all K slots are read
// first, then all K rows are requested, then they are added in slot order (two
// memory round trips per thread instead of two per slot; same arithmetic).
// K = 0: any top_k, slot by slot.
template <typename T, int K>
__global__ __launch_bounds__(256) void combine_kernel(
    const Pack<T> *__restrict__ slot_out, const int32_t *__restrict__ inv_perm,
    const float *__restrict__ topk_weight, const Pack<T> *__restrict__ shared_out,
    const uint8_t *__restrict__ skip_mask, const Pack<T> *__restrict__ cache_in,
    Pack<T> *__restrict__ cache_out, Pack<T> *__restrict__ y, int64_t n_tokens, int top_k,
    int vec_per_row, const Pack<T> *__restrict__ resid, const Pack<T> *__restrict__ gate,
    int64_t tokens_per_sample) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_tokens * vec_per_row) return;
  const int64_t t = i / vec_per_row;
  const int c = (int)(i - t * vec_per_row);
  float acc[Pack<T>::kN];
#pragma unroll
  for (int e = 0; e < Pack<T>::kN; ++e) acc[e] = 0.f;
  // (the rows that do not depend on the routing tables are requested first, so
  // that they travel while the slot rows' addresses are still being looked up)
  Pack<T> sh{}, res{}, gt{};
  if (shared_out) sh = shared_out[i];
  if (resid) {
    res = resid[i];
    gt = gate[(t / tokens_per_sample) * vec_per_row + c];
  }
  if constexpr (K > 0) {
    SlotSource<T> src[K];
#pragma unroll
    for (int j = 0; j < K; ++j)
      src[j] = slot_source<T>(t * K + j, i, c, vec_per_row, slot_out, inv_perm, topk_weight, skip_mask, cache_in,
                              cache_out != nullptr);
    Pack<T> row[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
      row[j] = Pack<T>{};
      if (src[j].row) row[j] = *src[j].row;
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if (src[j].put) cache_out[i] = row[j];
#pragma unroll
      for (int e = 0; e < Pack<T>::kN; ++e) acc[e] = fmaf(src[j].w, row[j].get(e), acc[e]);
    }
  } else {
    for (int j = 0; j < top_k; ++j) {
      const SlotSource<T> src = slot_source<T>(t * top_k + j, i, c, vec_per_row, slot_out, inv_perm, topk_weight,
                                               skip_mask, cache_in, cache_out != nullptr);
      Pack<T> row{};
      if (src.row) row = *src.row;
      if (src.put) cache_out[i] = row;
#pragma unroll
      for (int e = 0; e < Pack<T>::kN; ++e) acc[e] = fmaf(src.w, row.get(e), acc[e]);
    }
  }
  if (shared_out) {
#pragma unroll
    for (int e = 0; e < Pack<T>::kN; ++e) acc[e] += sh.get(e);
  }
  if (resid) {
#pragma unroll
    for (int e = 0; e < Pack<T>::kN; ++e) acc[e] = fmaf(gt.get(e), acc[e], res.get(e));
  }
  Pack<T> o;
#pragma unroll
  for (int e = 0; e < Pack<T>::kN; ++e) o.set(e, acc[e]);
  y[i] = o;
}

template <typename T>
int launch_combine(const void *slot_out, const int32_t *inv_perm, const float *w,
                   const void *shared_out, const uint8_t *skip, const void *cache_in,
                   void *cache_out, void *y, int64_t n_tokens, int top_k, int hidden,
                   const void *resid, const void *gate, int64_t tokens_per_sample, hipStream_t s) {
  const int vec_per_row = hidden / Pack<T>::kN;
  const int64_t total = n_tokens * vec_per_row;
  const int64_t blocks = (total + 255) / 256;
#define DICE_COMBINE_LAUNCH(K)                                                                      \
  hipLaunchKernelGGL((combine_kernel<T, K>), dim3((unsigned)blocks), dim3(256), 0, s,               \
                     (const Pack<T> *)slot_out, inv_perm, w, (const Pack<T> *)shared_out, skip,     \
                     (const Pack<T> *)cache_in, (Pack<T> *)cache_out, (Pack<T> *)y, n_tokens, top_k, \
                     vec_per_row, (const Pack<T> *)resid, (const Pack<T> *)gate, tokens_per_sample)
  switch (top_k) {
    case 1: DICE_COMBINE_LAUNCH(1); break;
    case 2: DICE_COMBINE_LAUNCH(2); break;
    case 4: DICE_COMBINE_LAUNCH(4); break;
    default: DICE_COMBINE_LAUNCH(0); break;
  }
#undef DICE_COMBINE_LAUNCH
  return launch_status("dice_combine");
}

}  // namespace

int combine_impl(const void *slot_out, const int32_t *inv_perm, const float *topk_weight,
                 const void *shared_out, const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                 void *y, int dtype, int64_t n_tokens, int top_k, int hidden, const void *resid,
                 const void *gate, int64_t tokens_per_sample, void *stream) {
  DICE_REQUIRE(slot_out && topk_weight && y, DICE_ERR_BAD_ARG, "dice_combine: null pointer");
  DICE_REQUIRE(top_k >= 1 && top_k <= kMaxTopK, DICE_ERR_BAD_ARG, "dice_combine: top_k %d outside [1, %d]",
               top_k, kMaxTopK);
  DICE_REQUIRE(!(cache_in || cache_out) || skip_mask, DICE_ERR_BAD_ARG,
               "dice_combine: a cache pointer needs skip_mask");
  DICE_REQUIRE(!(cache_in && cache_out), DICE_ERR_BAD_ARG,
               "dice_combine: a step either reads (skip) or writes (put) the cache, not both");
  DICE_REQUIRE(!resid == !gate, DICE_ERR_BAD_ARG, "dice_combine: residual and gate come together");
  DICE_REQUIRE(!resid || tokens_per_sample >= 1, DICE_ERR_BAD_ARG,
               "dice_combine: tokens_per_sample %lld < 1", (long long)tokens_per_sample);
  const size_t es = dtype_size(dtype);
  DICE_REQUIRE(es == 2 || es == 4, DICE_ERR_UNSUPPORTED, "dice_combine: dtype %d", dtype);
  DICE_REQUIRE(hidden > 0 && ((size_t)hidden * es) % 16 == 0, DICE_ERR_BAD_ARG,
               "dice_combine: hidden %d rows are not a multiple of 16 bytes", hidden);
  if (n_tokens <= 0) return DICE_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DICE_F32:
      return launch_combine<float>(slot_out, inv_perm, topk_weight, shared_out, skip_mask, cache_in,
                                   cache_out, y, n_tokens, top_k, hidden, resid, gate, tokens_per_sample, s);
    case DICE_BF16:
      return launch_combine<bf16_t>(slot_out, inv_perm, topk_weight, shared_out, skip_mask, cache_in,
                                    cache_out, y, n_tokens, top_k, hidden, resid, gate, tokens_per_sample, s);
    case DICE_F16:
      return launch_combine<f16_t>(slot_out, inv_perm, topk_weight, shared_out, skip_mask, cache_in,
                                   cache_out, y, n_tokens, top_k, hidden, resid, gate, tokens_per_sample, s);
  }
  return fail(DICE_ERR_UNSUPPORTED, "dice_combine: dtype %d", dtype);
}

}  // namespace dice

extern "C" int dice_combine(const void *slot_out, const int32_t *inv_perm,
                            const float *topk_weight, const void *shared_out,
                            const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                            void *y, int dtype, int64_t n_tokens, int top_k, int hidden,
                            void *stream) {
  return dice::combine_impl(slot_out, inv_perm, topk_weight, shared_out, skip_mask, cache_in, cache_out, y,
                            dtype, n_tokens, top_k, hidden, nullptr, nullptr, 1, stream);
}

extern "C" int dice_combine_residual(const void *slot_out, const int32_t *inv_perm,
                                     const float *topk_weight, const void *shared_out,
                                     const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                                     const void *resid, const void *gate, int64_t tokens_per_sample,
                                     void *out, int dtype, int64_t n_tokens, int top_k, int hidden,
                                     void *stream) {
  using namespace dice;
  DICE_REQUIRE(resid && gate, DICE_ERR_BAD_ARG, "dice_combine_residual: null pointer");
  return combine_impl(slot_out, inv_perm, topk_weight, shared_out, skip_mask, cache_in, cache_out, out, dtype,
                      n_tokens, top_k, hidden, resid, gate, tokens_per_sample, stream);
}
