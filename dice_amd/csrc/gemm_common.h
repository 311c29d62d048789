// Problem description and tile scheduling shared by the grouped expert GEMMs.
//
// One launch covers every expert: grouped rows [offsets[e], offsets[e+1]) of
// the activation matrix multiply expert e's weight matrix.  The row counts
// live on the device, so the host sizes the grid from an upper bound and each
// workgroup derives its own (expert, m-tile, n-tile) from the offset table;
// surplus workgroups exit at once.  No host synchronisation is needed, unlike
// the reference's bincount().cpu() (models.py:366).
#pragma once

#include "common.h"

namespace dice {

enum GemmMode { kFc1Swiglu = 0, kFc1Gelu = 1, kFc2 = 2 };

struct GemmParams {
  const void *a;           // activations, row stride lda elements
  const int32_t *a_perm;   // grouped row -> slot; source row = slot / a_div.  NULL: identity
  int a_div;
  int lda;
  const int32_t *offsets;  // [n_experts + 1] grouped row ranges
  int n_experts;
  const void *w;           // [n_experts, w_rows, k]
  int w_rows;              // weight rows per expert (2*n for SwiGLU fc1, else n)
  int up_offset;           // SwiGLU: first up_proj row inside an expert's block (= n)
  const float *bias;       // [n_experts, n] or NULL
  const float *w_scale;    // [n_experts, w_rows] or NULL (fp8 weights)
  void *c;                 // output, row stride ldc elements
  int ldc;
  const int32_t *c_perm;   // grouped row -> output row.  NULL: identity
  int n;                   // output columns
  int k;                   // reduction length
};

struct TileCoord {
  int expert;
  int row_begin;   // first grouped row of the tile
  int rows_valid;  // rows of the tile that belong to the expert (1..BM)
  int n0;          // first output column
  bool active;
};

constexpr int kNumXcd = 8;

// Upper bound on the grid for `max_rows` grouped rows.
inline int64_t max_tiles(int64_t max_rows, int n_experts, int n, int bm, int bn_out) {
  const int64_t m_tiles = (max_rows + bm - 1) / bm + n_experts;
  const int64_t n_tiles = (n + bn_out - 1) / bn_out;
  const int64_t total = m_tiles * n_tiles;
  return (total + kNumXcd - 1) / kNumXcd * kNumXcd;
}

// Maps blockIdx.x to a tile.  Hardware hands consecutive workgroup ids to the
// eight XCDs round-robin; the remap gives each XCD one contiguous run of the
// logical tile order (expert-major, then n-tile, m-tile fastest), so the
// workgroups that share an L2 work on the same expert's weights and re-use
// the same weight tile across neighbouring m-tiles.
template <int BM, int BN_OUT>
__device__ __forceinline__ TileCoord locate_tile(const GemmParams &p) {
  // Every wave works this out for itself, 64 experts at a time: lane l reads the
  // row range of expert e0 + l (two loads per lane instead of a scalar loop of
  // dependent loads over the experts, which costs microseconds before a tile of
  // a small batch can start).
  TileCoord t;
  t.active = false;
  const int lane = threadIdx.x & (kWave - 1);
  const int n_tiles = (p.n + BN_OUT - 1) / BN_OUT;
  const bool one_pass = p.n_experts <= kWave;
  int begin = 0, cnt = 0, mt = 0, total_mt = 0;
  for (int e0 = 0; e0 < p.n_experts; e0 += kWave) {
    const int e = e0 + lane;
    begin = e < p.n_experts ? p.offsets[e] : 0;
    cnt = e < p.n_experts ? p.offsets[e + 1] - begin : 0;
    mt = (cnt + BM - 1) / BM;
    total_mt += wave_sum_i32(mt);
  }
  const int total = total_mt * n_tiles;
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const int xcd = blockIdx.x % kNumXcd;
  const int j = blockIdx.x / kNumXcd;
  const int logical = xcd * per_xcd + j;
  if (j >= per_xcd || logical >= total) return t;
  int base_mt = 0;  // m-tiles of the experts before this chunk
  for (int e0 = 0; e0 < p.n_experts; e0 += kWave) {
    if (!one_pass) {  // (a single chunk still holds its row ranges from the first loop)
      const int e = e0 + lane;
      begin = e < p.n_experts ? p.offsets[e] : 0;
      cnt = e < p.n_experts ? p.offsets[e + 1] - begin : 0;
      mt = (cnt + BM - 1) / BM;
    }
    int inc = mt;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(inc, o, kWave);
      if (lane >= o) inc += up;
    }
    inc += base_mt;
    const int span_begin = (inc - mt) * n_tiles, span_end = inc * n_tiles;
    const uint64_t hit = __ballot(mt > 0 && logical >= span_begin && logical < span_end);
    if (hit) {
      const int g = __builtin_ctzll(hit);
      const int g_begin = __shfl(begin, g, kWave), g_cnt = __shfl(cnt, g, kWave);
      const int g_mt = __shfl(mt, g, kWave), g_base = __shfl(span_begin, g, kWave);
      const int r = logical - g_base;
      const int n_tile = r / g_mt;
      const int m_tile = r - n_tile * g_mt;
      t.expert = __builtin_amdgcn_readfirstlane(e0 + g);
      t.row_begin = __builtin_amdgcn_readfirstlane(g_begin + m_tile * BM);
      const int left = g_cnt - m_tile * BM;
      t.rows_valid = __builtin_amdgcn_readfirstlane(left < BM ? left : BM);
      t.n0 = __builtin_amdgcn_readfirstlane(n_tile * BN_OUT);
      t.active = true;
      return t;
    }
    base_mt = __shfl(inc, kWave - 1, kWave);
  }
  return t;
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

// tanh-approximate GELU, the closed form of torch gelu(approximate="tanh").
__device__ __forceinline__ float gelu_tanh_f(float x) {
  const float k0 = 0.7978845608028654f;  // sqrt(2/pi)
  const float k1 = 0.044715f;
  const float inner = k0 * (x + k1 * x * x * x);
  return 0.5f * x * (1.0f + tanhf(inner));
}

// Hardware-transcendental forms for the bf16 kernels (v_exp_f32 / v_rcp_f32,
// about 1 ulp each, far below bf16 resolution): sigmoid(z) = 1/(1 + 2^(-z log2 e)).
__device__ __forceinline__ float sigmoid_fast(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
}
__device__ __forceinline__ float silu_fast(float g) { return g * sigmoid_fast(g); }
// 0.5 x (1 + tanh(u)) = x sigmoid(2u), u = k0 (x + k1 x^3): the exponent of the
// sigmoid is x (c0 + c1 x^2) with the constants folded (three multiplies and one
// fused multiply-add per value beside the two transcendentals).
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  constexpr float k0 = 0.7978845608028654f, k1 = 0.044715f;
  constexpr float c0 = -2.0f * k0 * 1.4426950408889634f, c1 = c0 * k1;
  const float z = x * __builtin_fmaf(x * x, c1, c0);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z));
}

// One grouped GEMM of a persistent launch: grouped activation rows (row r of
// expert e = a + (offsets[e] + r) * lda, or, with a_rows, the source row
// a_rows[offsets[e] + r] / a_div of a), bf16 (or, with w_scale, fp8) weights
// [n_experts, w_rows, k], output rows in grouped order.
struct PersistProblem {
  const void *a;
  int lda;
  const int32_t *offsets;  // [n_experts + 1], device
  int n_experts;
  const void *w;
  int w_rows;
  int up_offset;           // SwiGLU: first up_proj row of an expert's block
  const float *bias;       // [n_experts, n] or NULL
  void *c;
  int ldc;
  int n, k;
  int max_rows;            // host-side upper bound on the grouped rows (offsets live on the device)
  const int32_t *a_rows;   // grouped row -> slot (the dispatch permutation), or NULL: rows are contiguous
  int a_div;               // slots per source row (top-k)
  int a_src_rows;          // rows of the source matrix (range check of the gather)
  const float *w_scale;    // [n_experts, w_rows] per-output-channel scales: the weights are fp8 (e4m3) bytes; NULL: bf16
  const float *a_scale;    // [max_rows] per-row scales in grouped order: the activations too are fp8 (e4m3) bytes
                           // (lda then counts bytes) and the products run on the fp8 matrix pipe; NULL: 16-bit rows
  // Block scales (fp8 kernels only): one power of two per row and 32 columns, as a byte (the exponent biased by 127,
  // what the scaled MFMA takes), laid out [columns / 128][max_rows][4]: the four scales of a row's 128 columns - one
  // step of the fp8 kernel - are one dword, the dwords of consecutive rows are adjacent (a tile's scales of a step are
  // 1 KB of contiguous memory), and within a dword the bytes are ordered 0, 2, 1, 3 (block_scale_pos).
  const uint8_t *a_block_scale;  // the activations are e4m3 bytes with these scales instead of a_scale (fc2)
  uint8_t *c_block_scale;        // the output is written as e4m3 bytes (ldc counts bytes) with these scales (fc1)
};
// Byte of the scale of 32-column block `cb` within its dword: the fp8 kernel's lane half h reads the scales of both
// 64-k blocks of a 128-k step as two adjacent bytes.
__host__ __device__ inline int block_scale_pos(int cb) { return ((cb & 1) << 1) | ((cb >> 1) & 1); }
constexpr int kMaxPersistProblems = 3;
struct PersistBatch {
  int n_problems;
  PersistProblem prob[kMaxPersistProblems];
  int band_tiles;  // tile order: m-tiles per band (a group with more is cut into bands); 0 = the default rule
  int xcd_split;   // how the tiles are shared out over the XCDs (set by the launcher; see TileWalker)
  // Partial-tile slots (persist_split_ws_bytes() bytes) or NULL.  With slots, a
  // single-problem fc2 launch whose tiles do not fill the workgroups' last turn
  // cuts that turn's tiles along k, one piece per workgroup, and a second small
  // launch adds the pieces up; without, every tile is multiplied whole.
  void *split_ws;
};
constexpr int kPersistSplitSlots = 320;  // partial-tile slots: one per workgroup of a launch (one per compute unit)
size_t persist_split_ws_bytes();         // kPersistSplitSlots tiles of 256 x 256 16-bit values
bool persist_supported(const PersistBatch &b, int mode);
bool persist_fits_table(const PersistBatch &b, int mode);  // at most kTableTurns tiles per workgroup: no kernel has to rebuild its tile table
int persist_cu_count();  // compute units of the current device
int persist_band_tiles(int mode);  // tuning hook state: band height of the tile order for this stage (0 = default rule)
int persist_slim_choice(int mode);  // tuning hook state: 128-row weight tiles for launches of this stage that can take them: 1 = always, -1 = never, 0 = by the model
int shared_fc2_launch_choice();   // tuning hook state: 1 = the shared expert's fc2 as a launch of its own, -1 = never, 0 = by size
bool persist_split_allowed();      // tuning hook state: fc2 launches of the layer call may cut their last turn along k
bool route_in_prologue_allowed();   // tuning hook state: the modulated layer call may route inside its prologue kernel
bool gemm_config_is_default(int mode);  // tuning hook state: nothing is set for this stage
bool gemm_config_allows_persistent(int mode);  // tuning hook state: no tiling of the permutation-addressed kernels is forced for this stage
int launch_grouped_gemm_persist(const PersistBatch &b, int mode, hipStream_t s);      // bf16
int launch_grouped_gemm_persist_f16(const PersistBatch &b, int mode, hipStream_t s);  // fp16
// fp8 activations (a_scale) and weights (w_scale) on the fp8 matrix pipe, bf16 output
bool persist_f8_supported(const PersistBatch &b, int mode);
int launch_grouped_gemm_persist_f8(const PersistBatch &b, int mode, hipStream_t s);

// Few rows per group (at most 128 on average): a 256-row tile of the persistent
// kernels is then mostly padding - its matrix-pipe time is that of a full tile -
// and a launch a single short turn, while the permutation-addressed kernels
// with 64-row tiles only stream the weights (DiT-XL width, 8 experts: 63 against
// 117 us for both stages at 128 slots, 98 against 120 at 1024, 155 against 135
// at 2048).
inline bool few_rows_per_group(int64_t max_rows, int n_groups) { return max_rows <= 128ll * n_groups; }

// LayerNorm + adaLN modulation in front of the layer, and the combine with the
// caller's residual / gate epilogue behind it (modulate.hip, combine.hip).
int ln_modulate_impl(const void *x, const void *shift, const void *scale, void *out, int dtype,
                     int64_t n_tokens, int hidden, int64_t tokens_per_sample, float eps, void *stream);
// The same prologue with the router in the same launch (gate.hip): writes the
// modulated rows and their top-k routing; `applies` says whether the shape is
// one the kernel takes (16-bit rows of at most 1536 elements, a router matrix
// of the same type, at most 32 experts).
bool ln_modulate_route_applies(int act_dtype, int gate_w_dtype, int64_t n_tokens, int hidden, int n_experts);
int ln_modulate_route_impl(const void *x, const void *shift, const void *scale, void *out, int dtype,
                           int64_t n_tokens, int hidden, int64_t tokens_per_sample, float eps, const void *gate_w,
                           const float *gate_bias, int n_experts, int top_k, int norm_topk_prob, int32_t *topk_idx,
                           float *topk_weight, void *stream);
int combine_impl(const void *slot_out, const int32_t *inv_perm, const float *topk_weight,
                 const void *shared_out, const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                 void *y, int dtype, int64_t n_tokens, int top_k, int hidden, const void *resid,
                 const void *gate, int64_t tokens_per_sample, void *stream);

int dispatch_impl(const int32_t *flat_idx, const uint8_t *skip_mask, int64_t n_slots, int n_experts,
                  int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv_perm, void *workspace,
                  size_t workspace_bytes, int32_t *range_out, int32_t range_n, void *stream);
int gather_rows_impl(const void *x, int dtype, const int32_t *perm, int slots_per_token,
                     int64_t n_rows, int hidden, void *out, int32_t *range_out, int32_t range_n,
                     void *stream);

// Rows of x (row perm[r] / slots_per_token when perm is given) -> e4m3 rows and one scale per row (quant.hip).
int quantize_act_impl(const void *x, int in_dtype, const int32_t *perm, int slots_per_token,
                      const int32_t *n_rows_dev, int64_t max_rows, int cols, uint8_t *q, float *scale,
                      void *stream);

int launch_grouped_gemm_bf16(const GemmParams &p, int mode, int w_dtype, int64_t max_rows,
                             hipStream_t s);
int launch_grouped_gemm_f16(const GemmParams &p, int mode, int w_dtype, int64_t max_rows, hipStream_t s);
int launch_grouped_gemm_f32(const GemmParams &p, int mode, int w_dtype, int64_t max_rows, hipStream_t s);

}  // namespace dice
