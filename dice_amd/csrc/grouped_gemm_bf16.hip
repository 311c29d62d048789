// bf16 grouped expert GEMM on CDNA4 matrix cores (v_mfma_f32_32x32x16_bf16).
//
// Computes, for every expert e and its grouped rows r,
//   fc1 (SwiGLU): h[r, n] = silu(A[r] . Wg[e, n]) * (A[r] . Wu[e, n])
//   fc1 (GELU)  : h[r, n] = gelu_tanh(A[r] . W1[e, n] + b1[e, n])
//   fc2         : out[dst(r), n] = h[r] . W2[e, n] (+ b2[e, n])
// i.e. MoeMLP.forward of the reference (models.py:252-273) for all experts of
// moe_infer's loop (models.py:368-377) in one launch.  fp32 accumulation, one
// rounding to bf16 at the end.
//
// Layout.  Activations and weights are both k-contiguous ("NT" GEMM), which is
// the layout the MFMA operands want: a lane supplies 8 consecutive k values of
// one row.  A BMxBK activation tile and a BNxBK weight tile are staged in LDS
// (double buffered); rows are 128 bytes = eight 16-byte chunks and the chunk
// index is XOR-swizzled with the row so that the 16-byte fragment reads of a
// wave spread over all banks.  The weight tile is the MFMA "A" operand and the
// activation tile the "B" operand, which leaves every lane with 4 consecutive
// output columns of one row: packed 8-byte stores, and gate/up values of the
// same (row, column) in the same lane for the SwiGLU epilogue.
//
// fc1 reads its rows through the dispatch permutation (no gathered copy of x
// is ever written) and fc2 writes each row straight to its slot position (the
// un-permute of the reference's _local_combine, expertpara/ep_fwd.py:350-354).
//
// fp8 (e4m3) weights are widened to bf16 while they are copied into LDS, so
// the MFMA loop is unchanged; the per-output-channel scale is applied to the
// fp32 accumulator in the epilogue.
//
// Compiled twice, like the persistent kernels: as it stands for bf16, and with
// DICE_GEMM_F16 (through grouped_gemm_f16.hip) for fp16 activations and weights.
#include "gemm_common.h"

#ifndef DICE_GEMM_F16
#define DICE_GEMM_F16 0
#endif
// ... and with DICE_GEMM_F32 (through grouped_gemm_f32.hip) for fp32
// activations and weights, the type the reference serves its S and B models in
// (sample_ddp.py:82-85): 32 k per step (still 128-byte LDS rows), the fp32
// MFMA v_mfma_f32_32x32x2_f32 (fp32 products and sums), no fp8 weights.
#ifndef DICE_GEMM_F32
#define DICE_GEMM_F32 0
#endif

namespace dice {
namespace {

#if DICE_GEMM_F32
typedef float h16_t;
typedef f32x4_t h16x4_t;
#define DICE_GEMM_LAUNCH launch_grouped_gemm_f32
#elif DICE_GEMM_F16
typedef f16_t h16_t;
typedef f16x8_t h16x8_t;
typedef _Float16 h16x4_t __attribute__((ext_vector_type(4)));
#define DICE_MFMA_32X32X16 __builtin_amdgcn_mfma_f32_32x32x16_f16
#define DICE_WIDEN_FP8 __builtin_amdgcn_cvt_scalef32_pk_f16_fp8
#define DICE_GEMM_LAUNCH launch_grouped_gemm_f16
#else
typedef bf16_t h16_t;
typedef bf16x8_t h16x8_t;
typedef bf16x4_t h16x4_t;
#define DICE_MFMA_32X32X16 __builtin_amdgcn_mfma_f32_32x32x16_bf16
#define DICE_WIDEN_FP8 __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8
#define DICE_GEMM_LAUNCH launch_grouped_gemm_bf16
#endif

constexpr int kChunkElems = 16 / (int)sizeof(h16_t);  // elements per 16-byte chunk
constexpr int kBK = 8 * kChunkElems;                  // elements per k step = 128 bytes per LDS row

__device__ __forceinline__ int swizzle(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Element offset of 16-byte chunk `chunk` of row `row` inside a [rows][kBK] tile.
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * kBK + ((chunk ^ swizzle(row)) * kChunkElems);
}

// DEPTH: register stages between global memory and LDS.  The loads of step
// kt + DEPTH are issued while step kt is multiplied and reach LDS DEPTH - 1
// steps later; a 64 x 64 tile multiplies a step in 0.2 - 0.4 us, a load takes a
// microsecond or more, and with few rows there is one wave per SIMD: nothing
// else hides the difference.
template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, bool W_FP8, int DEPTH>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWave) void grouped_gemm_bf16_kernel(GemmParams p) {
  static_assert(DEPTH == 2 || DEPTH == 4, "an even number of register stages: the LDS stage of a step is its parity");
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold at least one 32x32 block");
  static_assert(!SWIGLU || TN % 2 == 0, "SwiGLU needs gate and up blocks in the same wave");
  static_assert(!(DICE_GEMM_F32 && W_FP8), "fp8 weights go with 16-bit activations");
  constexpr int A_ROWS_PER_PASS = NT / 8;
  constexpr int A_PASSES = BM / A_ROWS_PER_PASS;
  // bf16 weights: 8 threads x 16 B per row; fp8: 4 threads x 16 B per row.
  constexpr int B_THREADS_PER_ROW = W_FP8 ? 4 : 8;
  constexpr int B_ROWS_PER_PASS = NT / B_THREADS_PER_ROW;
  constexpr int B_PASSES = BN / B_ROWS_PER_PASS;
  static_assert(A_PASSES >= 1 && B_PASSES >= 1, "tile too small for the workgroup");
  constexpr int A_STAGE = BM * kBK, B_STAGE = BN * kBK;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  h16_t *As = reinterpret_cast<h16_t *>(lds_raw);
  h16_t *Bs = As + 2 * A_STAGE;

  const TileCoord t = locate_tile<BM, BN_OUT>(p);
  if (!t.active) return;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- global -> register -> LDS copy assignment ----
  const int a_chunk = tid & 7, a_row0 = tid >> 3;
  const h16_t *a_base = (const h16_t *)p.a;
  uint32_t a_src[A_PASSES];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i) {
    const int rt = a_row0 + i * A_ROWS_PER_PASS;
    const int gr = t.row_begin + (rt < t.rows_valid ? rt : t.rows_valid - 1);
    const int src = p.a_perm ? p.a_perm[gr] / p.a_div : gr;
    a_src[i] = (uint32_t)src * (uint32_t)p.lda + a_chunk * kChunkElems;
  }
  const int b_chunk = tid % B_THREADS_PER_ROW, b_row0 = tid / B_THREADS_PER_ROW;
  const size_t w_expert = (size_t)t.expert * p.w_rows * p.k;
  uint32_t b_src[B_PASSES];
#pragma unroll
  for (int i = 0; i < B_PASSES; ++i) {
    const int rt = b_row0 + i * B_ROWS_PER_PASS;
    int col = t.n0 + (SWIGLU ? (rt % (BN / 2)) : rt);
    if (col >= p.n) col = t.n0;
    const int wrow = (SWIGLU && rt >= BN / 2) ? p.up_offset + col : col;
    b_src[i] = (uint32_t)wrow * (uint32_t)p.k + b_chunk * (W_FP8 ? 16 : kChunkElems);
  }

  u32x4_t a_reg[DEPTH][A_PASSES], b_reg[DEPTH][B_PASSES];
  // (`r`, the register stage, is a compile-time constant wherever this is called)
  auto load_global = [&](int k0, int r) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i)
      a_reg[r][i] = *reinterpret_cast<const u32x4_t *>(a_base + a_src[i] + k0);
    if (W_FP8) {
      const uint8_t *wb = (const uint8_t *)p.w + w_expert;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i)
        b_reg[r][i] = *reinterpret_cast<const u32x4_t *>(wb + b_src[i] + k0);
    } else {
      const h16_t *wb = (const h16_t *)p.w + w_expert;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i)
        b_reg[r][i] = *reinterpret_cast<const u32x4_t *>(wb + b_src[i] + k0);
    }
  };
  auto store_lds = [&](int stage, int r) {
    h16_t *as = As + stage * A_STAGE;
    h16_t *bs = Bs + stage * B_STAGE;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const int rt = a_row0 + i * A_ROWS_PER_PASS;
      *reinterpret_cast<u32x4_t *>(as + lds_off(rt, a_chunk)) = a_reg[r][i];
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      const int rt = b_row0 + i * B_ROWS_PER_PASS;
#if !DICE_GEMM_F32
      if (W_FP8) {
        // 16 e4m3 bytes -> 16 bf16 = chunks 2c and 2c+1 of the row.
        u32x4_t lo, hi;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          auto c0 = DICE_WIDEN_FP8(b_reg[r][i][q], 1.0f, false);
          auto c1 = DICE_WIDEN_FP8(b_reg[r][i][q], 1.0f, true);
          lo[2 * q] = __builtin_bit_cast(uint32_t, c0);
          lo[2 * q + 1] = __builtin_bit_cast(uint32_t, c1);
          auto d0 = DICE_WIDEN_FP8(b_reg[r][i][q + 2], 1.0f, false);
          auto d1 = DICE_WIDEN_FP8(b_reg[r][i][q + 2], 1.0f, true);
          hi[2 * q] = __builtin_bit_cast(uint32_t, d0);
          hi[2 * q + 1] = __builtin_bit_cast(uint32_t, d1);
        }
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, 2 * b_chunk)) = lo;
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, 2 * b_chunk + 1)) = hi;
      } else
#endif
      {
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, b_chunk)) = b_reg[r][i];
      }
    }
  };

  // LDS row of 32-row block j of this wave's weight operand.
  auto w_block_row = [&](int j) {
    if (SWIGLU) {
      constexpr int HALF = TN / 2;
      return j < HALF ? wn * (WTN / 2) + j * 32 : BN / 2 + wn * (WTN / 2) + (j - HALF) * 32;
    }
    return wn * WTN + j * 32;
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int kt_count = p.k / kBK;

  // Step kt sits in register stage kt % DEPTH until it is written to LDS stage
  // kt % 2.  Loads past the last step re-read the last one (every step issues the
  // same number of loads, so the wait for a stage's data may leave exactly the
  // younger stages' loads in flight); their data is never written to LDS.
  const int k_last = (kt_count - 1) * kBK;
  auto k_of = [&](int kt) { return kt < kt_count ? kt * kBK : k_last; };
#pragma unroll
  for (int r = 0; r < DEPTH; ++r) load_global(k_of(r), r);
  store_lds(0, 0);
  __syncthreads();
  for (int kt0 = 0; kt0 < kt_count; kt0 += DEPTH) {
#pragma unroll
   for (int r = 0; r < DEPTH; ++r) {
    const int kt = kt0 + r;
    if (kt >= kt_count) break;
    constexpr int kStages = 2;
    const int cur = r % kStages;
    load_global(k_of(kt + DEPTH), r);  // stage r went to LDS one step ago
    const h16_t *as = As + cur * A_STAGE;
    const h16_t *bs = Bs + cur * B_STAGE;
#if DICE_GEMM_F32
    // v_mfma_f32_32x32x2_f32 takes one k per half-wave: lanes 0..31 supply k = c,
    // lanes 32..63 k = 16 + c of the step's 32, for c = 0..15 (any pairing of the
    // k values is a valid order of the sum as long as both operands use it).
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int chunk = frag_half * 4 + cc;
      f32x4_t wf[TN], af[TM];
#pragma unroll
      for (int j = 0; j < TN; ++j)
        wf[j] = *reinterpret_cast<const f32x4_t *>(bs + lds_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const f32x4_t *>(as + lds_off(wm * WTM + i * 32 + frag_row, chunk));
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int i = 0; i < TM; ++i) {
            const int ii = (j & 1) ? TM - 1 - i : i;
            acc[ii][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[j][e], af[ii][e], acc[ii][j], 0, 0, 0);
          }
    }
#else
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      const int chunk = kk * 2 + frag_half;
      h16x8_t wf[TN], af[TM];
#pragma unroll
      for (int j = 0; j < TN; ++j)
        wf[j] = *reinterpret_cast<const h16x8_t *>(bs + lds_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const h16x8_t *>(as + lds_off(wm * WTM + i * 32 + frag_row, chunk));
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          // weight block by weight block, the row blocks up and down in turn: one operand
          // changes per product, the left one every fourth time (same sums as any order)
          const int ii = (j & 1) ? TM - 1 - i : i;
          acc[ii][j] = DICE_MFMA_32X32X16(wf[j], af[ii], acc[ii][j], 0, 0, 0);
        }
    }
#endif
    if (kt + 1 < kt_count) store_lds(cur ^ 1, (r + 1) % DEPTH);
    __syncthreads();
   }
  }

  // ---- epilogue: lane holds row (lane&31), columns 8*q + 4*(lane>>5) + {0..3} of each block ----
  h16_t *c = (h16_t *)p.c;
  const float *bias = p.bias ? p.bias + (size_t)t.expert * p.n : nullptr;
  const float *scale = p.w_scale ? p.w_scale + (size_t)t.expert * p.w_rows : nullptr;
  constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = wm * WTM + i * 32 + frag_row;
    if (m >= t.rows_valid) continue;
    const int gr = t.row_begin + m;
    const int64_t orow = p.c_perm ? p.c_perm[gr] : gr;
    h16_t *crow = c + orow * p.ldc;
#pragma unroll
    for (int j = 0; j < OUT_BLOCKS; ++j) {
      const int nb = t.n0 + (SWIGLU ? wn * (WTN / 2) : wn * WTN) + j * 32 + frag_half * 4;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = nb + q * 8;
        if (n >= p.n) continue;
        h16x4_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[i][j][q * 4 + r];
          if (scale) v *= scale[n + r];
          if (SWIGLU) {
            float u = acc[i][j + OUT_BLOCKS][q * 4 + r];
            if (scale) u *= scale[p.up_offset + n + r];
            v = silu_fast(v) * u;
          } else {
            if (bias) v += bias[n + r];
            if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);
          }
          o[r] = (h16_t)v;
        }
        *reinterpret_cast<h16x4_t *>(crow + n) = o;
      }
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, bool W_FP8>
int launch_cfg(const GemmParams &p, int64_t max_rows, hipStream_t s) {
  constexpr int DEPTH = BM * BN <= 64 * 128 ? 4 : 2;
  constexpr int BN_OUT = MODE == kFc1Swiglu ? BN / 2 : BN;
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr size_t lds = 2ull * (BM + BN) * kBK * sizeof(h16_t);
  const int64_t grid = max_tiles(max_rows, p.n_experts, p.n, BM, BN_OUT);
  if (grid <= 0) return DICE_OK;
  if (grid >= (1ll << 31)) return fail(DICE_ERR_UNSUPPORTED, "16-bit expert GEMM: grid too large");
  auto kern = grouped_gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, MODE, W_FP8, DEPTH>;
  if (lds > 48 * 1024) {
    static thread_local bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess)
        return fail(DICE_ERR_LAUNCH, "16-bit expert GEMM: LDS attribute: %s", hipGetErrorString(e));
      configured = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, s, p);
  return launch_status("grouped_gemm_bf16");
}

#if DICE_GEMM_F16 || DICE_GEMM_F32
}  // namespace
extern int g_cfg_fc1, g_cfg_fc2;
namespace {
#else
}  // namespace
int g_cfg_fc1 = 0, g_cfg_fc2 = 0;
namespace {
#endif

template <int MODE, bool W_FP8>
int launch_mode(const GemmParams &p, int cfg, int64_t max_rows, hipStream_t s) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  // Few rows (the reference's DiT-S batches: 1024 tokens): 128-row tiles would
  // leave most compute units without one and the rest with a long k loop each;
  // 64-row tiles with 64 output columns make four times as many.
  if (cfg == 0 && max_tiles(max_rows, p.n_experts, p.n, 128, SWIGLU ? 64 : 128) < 2 * persist_cu_count()) cfg = 3;
  switch (cfg) {
    case 1:
      return launch_cfg<256, 256, 2, 4, MODE, W_FP8>(p, max_rows, s);
    case 2:
      return launch_cfg<256, 128, 2, 2, MODE, W_FP8>(p, max_rows, s);
    case 3:
      return launch_cfg<64, SWIGLU ? 128 : 64, 2, 2, MODE, W_FP8>(p, max_rows, s);
    default:
      return launch_cfg<128, 128, 2, 2, MODE, W_FP8>(p, max_rows, s);
  }
}

}  // namespace

int DICE_GEMM_LAUNCH(const GemmParams &p, int mode, int w_dtype, int64_t max_rows, hipStream_t s) {
  if (p.k % kBK != 0) return fail(DICE_ERR_UNSUPPORTED, "16-bit expert GEMM: k %d %% %d != 0", p.k, kBK);
  if (p.n % 8 != 0) return fail(DICE_ERR_UNSUPPORTED, "16-bit expert GEMM: n %d %% 8 != 0", p.n);
  int cfg = mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1;
  if (cfg >= 20) cfg = 0;  // the hook's persistent-kernel values: this file picks its own tiling
#if DICE_GEMM_F32
  if (w_dtype != DICE_F32) return fail(DICE_ERR_UNSUPPORTED, "fp32 expert GEMM: w_dtype %d", w_dtype);
  switch (mode) {
    case kFc1Swiglu: return launch_mode<kFc1Swiglu, false>(p, cfg, max_rows, s);
    case kFc1Gelu: return launch_mode<kFc1Gelu, false>(p, cfg, max_rows, s);
    default: return launch_mode<kFc2, false>(p, cfg, max_rows, s);
  }
#else
  const bool fp8 = w_dtype == DICE_FP8_E4M3;
  switch (mode) {
    case kFc1Swiglu:
      return fp8 ? launch_mode<kFc1Swiglu, true>(p, cfg, max_rows, s)
                 : launch_mode<kFc1Swiglu, false>(p, cfg, max_rows, s);
    case kFc1Gelu:
      return fp8 ? launch_mode<kFc1Gelu, true>(p, cfg, max_rows, s)
                 : launch_mode<kFc1Gelu, false>(p, cfg, max_rows, s);
    default:
      return fp8 ? launch_mode<kFc2, true>(p, cfg, max_rows, s)
                 : launch_mode<kFc2, false>(p, cfg, max_rows, s);
  }
#endif
}

}  // namespace dice

#if !DICE_GEMM_F16 && !DICE_GEMM_F32
namespace dice {
constexpr int kCfgPersistent = 20;
extern int g_persist_waves;
bool gemm_config_allows_persistent(int mode) {
  const int cfg = mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1;
  return cfg == 0 || cfg >= kCfgPersistent;
}
int persist_band_tiles(int mode) {
  const int cfg = mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1;
  return cfg > 30 && cfg <= 46 ? cfg - 30 : 0;
}
int persist_slim_choice(int mode) {
  const int cfg = mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1;
  return cfg == 54 ? 1 : cfg == 55 ? -1 : 0;
}
bool persist_split_allowed() { return g_cfg_fc2 != 50; }
int shared_fc2_launch_choice() { return g_cfg_fc2 == 51 ? 1 : g_cfg_fc2 == 52 ? -1 : 0; }
bool route_in_prologue_allowed() { return g_cfg_fc1 != 50; }
bool gemm_config_is_default(int mode) { return (mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1) == 0; }
}  // namespace dice

// Tuning hook, per GEMM stage.  0 (default) and values >= 20: dice_grouped_mlp
// takes the persistent kernels where they apply and otherwise the
// permutation-addressed kernels of this file with 128x128 tiles / 4 waves, or
// 64-row tiles where those would be too few; 20 also restricts every persistent
// launch to the 32-k pipeline; 30 + b (b = 1 .. 16) orders the tiles of the
// persistent launches of that stage in bands of b m-tiles (each band taken
// through every n-tile before the next); 50 (fc2) has the layer call multiply every
// tile of its fc2 launches whole instead of cutting the tiles of a short last turn
// along k; 50 (fc1) has dice_moe_forward_modulated launch the router on its own
// instead of inside the prologue kernel; 51 / 52 (fc2) have the layer call launch
// the shared expert's fc2 on its own always / never (by default it does for small
// batches, where both launches then cut their tiles along k); 54 / 55 (either stage)
// have launches that can take 128-row weight tiles do so always / never (by default
// where the host's model says they shorten the launch).  Any value from 20 on also keeps a
// dice_grouped_mlp stage whose groups average at most 128 rows on the persistent
// kernels (21 does only that; by default such a stage takes this file's 64-row
// tiles).  1 .. 4 name a tiling of this file's kernels for
// dice_grouped_mlp whatever the shape (1: 256x256 / 8 waves; 2: 256x128 / 4
// waves; 3: 64x64 outputs / 4 waves; 4: 128x128).  Not part of the drop-in
// surface; used by the benchmark and the tests to compare kernels.
extern "C" int dice_set_gemm_config(int fc1_cfg, int fc2_cfg) {
  dice::g_cfg_fc1 = fc1_cfg;
  dice::g_cfg_fc2 = fc2_cfg;
  // 20: the 32-k eight-wave pipeline only; anything else: the 64-k pipeline where it applies (default)
  dice::g_persist_waves = fc1_cfg == dice::kCfgPersistent ? 8 : 4;
  return DICE_OK;
}
#endif  // bf16 compilation only
