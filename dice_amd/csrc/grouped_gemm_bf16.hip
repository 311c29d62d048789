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
#include "gemm_common.h"

namespace dice {
namespace {

constexpr int kBK = 64;  // bf16 elements per k step = 128 bytes per LDS row

__device__ __forceinline__ int swizzle(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Element offset of 16-byte chunk `chunk` of row `row` inside a [rows][64] tile.
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * kBK + ((chunk ^ swizzle(row)) << 3);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, bool W_FP8>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWave) void grouped_gemm_bf16_kernel(GemmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold at least one 32x32 block");
  static_assert(!SWIGLU || TN % 2 == 0, "SwiGLU needs gate and up blocks in the same wave");
  constexpr int A_ROWS_PER_PASS = NT / 8;
  constexpr int A_PASSES = BM / A_ROWS_PER_PASS;
  // bf16 weights: 8 threads x 16 B per row; fp8: 4 threads x 16 B per row.
  constexpr int B_THREADS_PER_ROW = W_FP8 ? 4 : 8;
  constexpr int B_ROWS_PER_PASS = NT / B_THREADS_PER_ROW;
  constexpr int B_PASSES = BN / B_ROWS_PER_PASS;
  static_assert(A_PASSES >= 1 && B_PASSES >= 1, "tile too small for the workgroup");
  constexpr int A_STAGE = BM * kBK, B_STAGE = BN * kBK;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t *As = reinterpret_cast<bf16_t *>(lds_raw);
  bf16_t *Bs = As + 2 * A_STAGE;

  const TileCoord t = locate_tile<BM, BN_OUT>(p);
  if (!t.active) return;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- global -> register -> LDS copy assignment ----
  const int a_chunk = tid & 7, a_row0 = tid >> 3;
  const bf16_t *a_base = (const bf16_t *)p.a;
  uint32_t a_src[A_PASSES];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i) {
    const int rt = a_row0 + i * A_ROWS_PER_PASS;
    const int gr = t.row_begin + (rt < t.rows_valid ? rt : t.rows_valid - 1);
    const int src = p.a_perm ? p.a_perm[gr] / p.a_div : gr;
    a_src[i] = (uint32_t)src * (uint32_t)p.lda + a_chunk * 8;
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
    b_src[i] = (uint32_t)wrow * (uint32_t)p.k + b_chunk * (W_FP8 ? 16 : 8);
  }

  u32x4_t a_reg[A_PASSES], b_reg[B_PASSES];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i)
      a_reg[i] = *reinterpret_cast<const u32x4_t *>(a_base + a_src[i] + k0);
    if (W_FP8) {
      const uint8_t *wb = (const uint8_t *)p.w + w_expert;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i)
        b_reg[i] = *reinterpret_cast<const u32x4_t *>(wb + b_src[i] + k0);
    } else {
      const bf16_t *wb = (const bf16_t *)p.w + w_expert;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i)
        b_reg[i] = *reinterpret_cast<const u32x4_t *>(wb + b_src[i] + k0);
    }
  };
  auto store_lds = [&](int stage) {
    bf16_t *as = As + stage * A_STAGE;
    bf16_t *bs = Bs + stage * B_STAGE;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const int rt = a_row0 + i * A_ROWS_PER_PASS;
      *reinterpret_cast<u32x4_t *>(as + lds_off(rt, a_chunk)) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      const int rt = b_row0 + i * B_ROWS_PER_PASS;
      if (W_FP8) {
        // 16 e4m3 bytes -> 16 bf16 = chunks 2c and 2c+1 of the row.
        u32x4_t lo, hi;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          bf16x2_t c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b_reg[i][q], 1.0f, false);
          bf16x2_t c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b_reg[i][q], 1.0f, true);
          lo[2 * q] = __builtin_bit_cast(uint32_t, c0);
          lo[2 * q + 1] = __builtin_bit_cast(uint32_t, c1);
          bf16x2_t d0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b_reg[i][q + 2], 1.0f, false);
          bf16x2_t d1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b_reg[i][q + 2], 1.0f, true);
          hi[2 * q] = __builtin_bit_cast(uint32_t, d0);
          hi[2 * q + 1] = __builtin_bit_cast(uint32_t, d1);
        }
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, 2 * b_chunk)) = lo;
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, 2 * b_chunk + 1)) = hi;
      } else {
        *reinterpret_cast<u32x4_t *>(bs + lds_off(rt, b_chunk)) = b_reg[i];
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

  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < kt_count; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < kt_count) load_global((kt + 1) * kBK);
    const bf16_t *as = As + cur * A_STAGE;
    const bf16_t *bs = Bs + cur * B_STAGE;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      const int chunk = kk * 2 + frag_half;
      bf16x8_t wf[TN], af[TM];
#pragma unroll
      for (int j = 0; j < TN; ++j)
        wf[j] = *reinterpret_cast<const bf16x8_t *>(bs + lds_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8_t *>(as + lds_off(wm * WTM + i * 32 + frag_row, chunk));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < kt_count) store_lds(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds row (lane&31), columns 8*q + 4*(lane>>5) + {0..3} of each block ----
  bf16_t *c = (bf16_t *)p.c;
  const float *bias = p.bias ? p.bias + (size_t)t.expert * p.n : nullptr;
  const float *scale = p.w_scale ? p.w_scale + (size_t)t.expert * p.w_rows : nullptr;
  constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = wm * WTM + i * 32 + frag_row;
    if (m >= t.rows_valid) continue;
    const int gr = t.row_begin + m;
    const int64_t orow = p.c_perm ? p.c_perm[gr] : gr;
    bf16_t *crow = c + orow * p.ldc;
#pragma unroll
    for (int j = 0; j < OUT_BLOCKS; ++j) {
      const int nb = t.n0 + (SWIGLU ? wn * (WTN / 2) : wn * WTN) + j * 32 + frag_half * 4;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = nb + q * 8;
        if (n >= p.n) continue;
        bf16x4_t o;
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
          o[r] = (bf16_t)v;
        }
        *reinterpret_cast<bf16x4_t *>(crow + n) = o;
      }
    }
  }
}

// Variant with direct global->LDS copies (global_load_lds_dwordx4): a wave-wide
// load drops 64 x 16 bytes = eight 128-byte tile rows straight into LDS, so no
// VGPRs or ds_write instructions are spent on staging.  The XOR swizzle moves
// to the global side: lane i owns LDS slot (row i/8, chunk i%8) and fetches
// the source chunk that belongs there.  One workgroup-wide barrier per k step;
// the next stage's copies and the next step's fragment reads are threaded
// between the MFMAs.  bf16 weights only.
template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWave, 1) void gemm_dl_kernel(GemmParams p) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_INSTR = BM / 8 / NW;   // 1 KB direct loads per wave per stage
  constexpr int B_INSTR = BN / 8 / NW;
  constexpr int STAGE_BYTES = (BM + BN) * kBK * 2;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

  const TileCoord t = locate_tile<BM, BN_OUT>(p);
  if (!t.active) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // per-lane source offsets (bytes) for each direct load
  const int lrow = lane >> 3, lchunk = lane & 7;
  uint32_t a_off[A_INSTR], b_off[B_INSTR];
#pragma unroll
  for (int i = 0; i < A_INSTR; ++i) {
    const int q = wave + NW * i;           // row group of 8
    const int rt = q * 8 + lrow;
    const int gr = t.row_begin + (rt < t.rows_valid ? rt : t.rows_valid - 1);
    const int src = p.a_perm ? p.a_perm[gr] / p.a_div : gr;
    const int c = lchunk ^ swizzle(rt);
    a_off[i] = ((uint32_t)src * (uint32_t)p.lda + c * 8) * 2;
  }
#pragma unroll
  for (int i = 0; i < B_INSTR; ++i) {
    const int q = wave + NW * i;
    const int rt = q * 8 + lrow;
    int col = t.n0 + (SWIGLU ? (rt % (BN / 2)) : rt);
    if (col >= p.n) col = t.n0;
    const int wrow = (SWIGLU && rt >= BN / 2) ? p.up_offset + col : col;
    const int c = lchunk ^ swizzle(rt);
    b_off[i] = ((uint32_t)wrow * (uint32_t)p.k + c * 8) * 2;
  }
  const unsigned char *a_base = (const unsigned char *)p.a;
  const unsigned char *w_base = (const unsigned char *)p.w + (size_t)t.expert * p.w_rows * p.k * 2;

  auto issue_loads = [&](int stage, int k0) {
    unsigned char *sa = lds_raw + stage * STAGE_BYTES;
    unsigned char *sb = sa + BM * kBK * 2;
#pragma unroll
    for (int i = 0; i < A_INSTR; ++i) {
      const int q = wave + NW * i;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(a_base + (size_t)k0 * 2 + a_off[i]),
          (__attribute__((address_space(3))) void *)(sa + q * 1024), 16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < B_INSTR; ++i) {
      const int q = wave + NW * i;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(w_base + (size_t)k0 * 2 + b_off[i]),
          (__attribute__((address_space(3))) void *)(sb + q * 1024), 16, 0, 0);
    }
  };

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

  constexpr int LOADS = A_INSTR + B_INSTR;
  constexpr int LOADS_PER_KK = (LOADS + 3) / 4;
  auto issue_one = [&](int stage, int k0, int idx) {
    unsigned char *sa = lds_raw + stage * STAGE_BYTES;
    unsigned char *sb = sa + BM * kBK * 2;
    if (idx < A_INSTR) {
      const int q = wave + NW * idx;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(a_base + (size_t)k0 * 2 + a_off[idx]),
          (__attribute__((address_space(3))) void *)(sa + q * 1024), 16, 0, 0);
    } else if (idx < LOADS) {
      const int q = wave + NW * (idx - A_INSTR);
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(w_base + (size_t)k0 * 2 + b_off[idx - A_INSTR]),
          (__attribute__((address_space(3))) void *)(sb + q * 1024), 16, 0, 0);
    }
  };
  issue_loads(0, 0);
  for (int kt = 0; kt < kt_count; ++kt) {
    const int cur = kt & 1;
    // The last step re-fetches its own tile into the idle stage: no branch in the loop body.
    const int k_next = (kt + 1 < kt_count ? kt + 1 : kt) * kBK;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const bf16_t *as = reinterpret_cast<const bf16_t *>(lds_raw + cur * STAGE_BYTES);
    const bf16_t *bs = as + BM * kBK;
    bf16x8_t wf[2][TN], af[2][TM];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      wf[0][j] = *reinterpret_cast<const bf16x8_t *>(bs + lds_off(w_block_row(j) + frag_row, frag_half));
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[0][i] = *reinterpret_cast<const bf16x8_t *>(as + lds_off(wm * WTM + i * 32 + frag_row, frag_half));
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int cb = kk & 1, nb = cb ^ 1;
#pragma unroll
      for (int l = 0; l < LOADS_PER_KK; ++l) issue_one(cur ^ 1, k_next, kk * LOADS_PER_KK + l);
      if (kk < 3) {
        const int chunk = (kk + 1) * 2 + frag_half;
#pragma unroll
        for (int j = 0; j < TN; ++j)
          wf[nb][j] = *reinterpret_cast<const bf16x8_t *>(bs + lds_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
        for (int i = 0; i < TM; ++i)
          af[nb][i] = *reinterpret_cast<const bf16x8_t *>(as + lds_off(wm * WTM + i * 32 + frag_row, chunk));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[cb][j], af[cb][i], acc[i][j], 0, 0, 0);
    }
    // Pin the issue order: fragment reads for step kk+1 and the next stage's
    // global->LDS loads are threaded between the MFMAs of step kk.
    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      constexpr int MF = TM * TN;
      constexpr int RD = TM + TN;
      constexpr int PER = MF / RD;          // MFMAs after each read
#pragma unroll
      for (int r = 0; r < RD; ++r) {
        if (kk < 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (r < LOADS_PER_KK) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
      }
      if (MF - PER * RD > 0) __builtin_amdgcn_sched_group_barrier(0x008, MF - PER * RD, 0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // epilogue
  bf16_t *c = (bf16_t *)p.c;
  const float *bias = p.bias ? p.bias + (size_t)t.expert * p.n : nullptr;
  constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = wm * WTM + i * 32 + frag_row;
    if (m >= t.rows_valid) continue;
    const int gr = t.row_begin + m;
    const int64_t orow = p.c_perm ? p.c_perm[gr] : gr;
    bf16_t *crow = c + orow * p.ldc;
#pragma unroll
    for (int j = 0; j < OUT_BLOCKS; ++j) {
      const int nb = t.n0 + (SWIGLU ? wn * (WTN / 2) : wn * WTN) + j * 32 + frag_half * 4;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = nb + q * 8;
        if (n >= p.n) continue;
        bf16x4_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[i][j][q * 4 + r];
          if (SWIGLU) {
            v = silu_fast(v) * acc[i][j + OUT_BLOCKS][q * 4 + r];
          } else {
            if (bias) v += bias[n + r];
            if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);
          }
          o[r] = (bf16_t)v;
        }
        *reinterpret_cast<bf16x4_t *>(crow + n) = o;
      }
    }
  }
}

// Ring-buffered variant: BK = 32 (64-byte LDS rows), STAGES slots, copies run
// STAGES-1 steps ahead of the MFMAs.
constexpr int kRingBK = 32;

__device__ __forceinline__ int swizzle32(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }
// Byte offset of 16-byte chunk `chunk` (0..3) of row `row` in a [rows][32] bf16 tile.
__device__ __forceinline__ int ring_off(int row, int chunk) {
  return row * 64 + ((chunk ^ swizzle32(row)) << 4);
}

// Issue-order template for half a k step of the ring kernel: two fragment
// reads behind each of the first MFMAs, then COPIES global->LDS copies spread
// evenly over the remaining MFMAs (the texture path takes 16 cycles per
// wave-wide 16-byte copy, so bursts issued by all waves at once would queue).
template <int I, int N, int RD>
__device__ __forceinline__ void schedule_reads() {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, (I == N - 1 && (RD & 1)) ? 1 : 2, 0);
    schedule_reads<I + 1, N, RD>();
  }
}
template <int I, int N, int GAP>
__device__ __forceinline__ void schedule_copies() {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, GAP, 0);
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    schedule_copies<I + 1, N, GAP>();
  }
}
template <int MF, int RD, int COPIES>
__device__ __forceinline__ void schedule_half() {
  constexpr int RDG = (RD + 1) / 2;
  static_assert(MF > RDG, "too few MFMAs to thread the fragment reads through");
  constexpr int REST = MF - RDG;
  constexpr int GAP = COPIES > 0 ? (REST / COPIES > 0 ? REST / COPIES : 1) : REST;
  schedule_reads<0, RDG, RD>();
  schedule_copies<0, COPIES, GAP>();
  constexpr int LEFT = REST - COPIES * GAP;
  if constexpr (LEFT > 0) __builtin_amdgcn_sched_group_barrier(0x008, LEFT, 0);
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, int STAGES>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWave, 1) void gemm_ring_kernel(GemmParams p) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_INSTR = BM / 16 / NW;  // 1 KB copies (16 rows x 64 B) per wave per step
  constexpr int B_INSTR = BN / 16 / NW;
  constexpr int LPS = A_INSTR + B_INSTR;
  constexpr int SLOT_BYTES = (BM + BN) * 64;
  constexpr int AHEAD = STAGES - 1;
  constexpr int PENDING_OK = (STAGES - 3) * LPS;  // copies that may still be in flight at a barrier
  static_assert(STAGES >= 3, "ring needs at least three slots");
  static_assert(A_INSTR >= 1 && B_INSTR >= 1, "tile too small for the workgroup");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

  const TileCoord t = locate_tile<BM, BN_OUT>(p);
  if (!t.active) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: LDS copy targets stay in SGPRs
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  const int lrow = lane >> 2, lchunk = lane & 3;
  uint32_t a_off[A_INSTR], b_off[B_INSTR];
#pragma unroll
  for (int i = 0; i < A_INSTR; ++i) {
    const int rt = (wave + NW * i) * 16 + lrow;
    const int gr = t.row_begin + (rt < t.rows_valid ? rt : t.rows_valid - 1);
    const int src = p.a_perm ? p.a_perm[gr] / p.a_div : gr;
    a_off[i] = ((uint32_t)src * (uint32_t)p.lda + ((lchunk ^ swizzle32(rt)) << 3)) * 2;
  }
#pragma unroll
  for (int i = 0; i < B_INSTR; ++i) {
    const int rt = (wave + NW * i) * 16 + lrow;
    int col = t.n0 + (SWIGLU ? (rt % (BN / 2)) : rt);
    if (col >= p.n) col = t.n0;
    const int wrow = (SWIGLU && rt >= BN / 2) ? p.up_offset + col : col;
    b_off[i] = ((uint32_t)wrow * (uint32_t)p.k + ((lchunk ^ swizzle32(rt)) << 3)) * 2;
  }
  const unsigned char *a_base = (const unsigned char *)p.a;
  const unsigned char *w_base = (const unsigned char *)p.w + (size_t)t.expert * p.w_rows * p.k * 2;
  const int kt_count = p.k / kRingBK;

  // Output rows this lane will store in the epilogue (-1 = past the group's end).
  // Fetched now: a load issued between the epilogue's stores would have to wait
  // for every earlier store to be acknowledged (loads and stores share vmcnt).
  constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
  constexpr int OUT_COLS = OUT_BLOCKS * 32;          // this wave's output columns
  constexpr int PITCH = OUT_COLS * 2 + 16;           // staging row pitch in bytes (16-byte aligned)
  constexpr int LANES_PER_ROW = OUT_COLS * 2 / 16;
  constexpr int ROWS_PER_PASS = kWave / LANES_PER_ROW;
  constexpr int PASSES = 32 / ROWS_PER_PASS;
  const int rd_row = lane / LANES_PER_ROW, rd_chunk = lane % LANES_PER_ROW;
  int out_row[TM][PASSES];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int m = wm * WTM + i * 32 + ps * ROWS_PER_PASS + rd_row;
      const int gr = t.row_begin + (m < t.rows_valid ? m : t.rows_valid - 1);
      const int orow = p.c_perm ? p.c_perm[gr] : gr;
      out_row[i][ps] = m < t.rows_valid ? orow : -1;
    }

  // Copies of k step `step` into ring slot `slot`; steps past the end re-fetch
  // the last step into a slot nobody reads, which keeps the in-flight count uniform.
  auto issue_step = [&](int step, int slot) {
    const int ks = step < kt_count ? step : kt_count - 1;
    const size_t kb = (size_t)ks * (kRingBK * 2);
    unsigned char *sa = lds_raw + slot * SLOT_BYTES;
    unsigned char *sb = sa + BM * 64;
#pragma unroll
    for (int i = 0; i < A_INSTR; ++i)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(a_base + kb + a_off[i]),
          (__attribute__((address_space(3))) void *)(sa + (wave + NW * i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < B_INSTR; ++i)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(w_base + kb + b_off[i]),
          (__attribute__((address_space(3))) void *)(sb + (wave + NW * i) * 1024), 16, 0, 0);
  };

  // Half of the copies of a step: part 0 = first LPS/2 copies, part 1 = the rest.
  auto issue_part = [&](int step, int slot, int part) {
    const int ks = step < kt_count ? step : kt_count - 1;
    const size_t kb = (size_t)ks * (kRingBK * 2);
    unsigned char *sa = lds_raw + slot * SLOT_BYTES;
    unsigned char *sb = sa + BM * 64;
    constexpr int HALF = LPS / 2;
#pragma unroll
    for (int l = 0; l < LPS; ++l) {
      if ((l < HALF) != (part == 0)) continue;
      if (l < A_INSTR)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(a_base + kb + a_off[l]),
            (__attribute__((address_space(3))) void *)(sa + (wave + NW * l) * 1024), 16, 0, 0);
      else
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(w_base + kb + b_off[l - A_INSTR]),
            (__attribute__((address_space(3))) void *)(sb + (wave + NW * (l - A_INSTR)) * 1024), 16, 0, 0);
    }
  };

  auto w_block_row = [&](int j) {
    if (SWIGLU) {
      constexpr int HALF = TN / 2;
      return j < HALF ? wn * (WTN / 2) + j * 32 : BN / 2 + wn * (WTN / 2) + (j - HALF) * 32;
    }
    return wn * WTN + j * 32;
  };
  const int frag_row = lane & 31, frag_half = lane >> 5;
  bf16x8_t wf[2][TN], af[2][TM];
  auto read_frags = [&](int slot, int kk, int buf) {
    const unsigned char *sa = lds_raw + slot * SLOT_BYTES;
    const unsigned char *sb = sa + BM * 64;
    const int chunk = kk * 2 + frag_half;
#pragma unroll
    for (int j = 0; j < TN; ++j)
      wf[buf][j] = *reinterpret_cast<const bf16x8_t *>(sb + ring_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[buf][i] = *reinterpret_cast<const bf16x8_t *>(sa + ring_off(wm * WTM + i * 32 + frag_row, chunk));
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

#pragma unroll
  for (int s = 0; s < AHEAD; ++s) issue_step(s, s);
  wait_vmcnt<PENDING_OK>();
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, 0);

  int slot = 0;  // slot of step kt
  for (int kt = 0; kt < kt_count; ++kt) {
    const int prev = slot == 0 ? STAGES - 1 : slot - 1;
    const int next = slot == STAGES - 1 ? 0 : slot + 1;
    wait_vmcnt<PENDING_OK>();        // this wave's copies for steps <= kt+1 have landed
    __builtin_amdgcn_s_barrier();    // ... everyone's have, and nobody still reads slot `prev`
    read_frags(slot, 1, 1);          // program order: reads, copies, MFMAs (copies are LDS writes
    issue_part(kt + AHEAD, prev, 0); // the compiler will not move reads across)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[0][j], af[0][i], acc[i][j], 0, 0, 0);
    read_frags(next, 0, 0);
    issue_part(kt + AHEAD, prev, 1);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[1][j], af[1][i], acc[i][j], 0, 0, 0);
    {
      // Issue order of the step.  kk = 0 starts at once on fragments fetched
      // before the barrier; the kk = 1 fragment reads, then the copies for step
      // kt + AHEAD, go between its MFMAs.  kk = 1 threads the reads of the next
      // step's first fragments early enough to land before the loop wraps.
      constexpr int MF = TM * TN, RD = TM + TN;
      schedule_half<MF, RD, LPS / 2>();
      schedule_half<MF, RD, LPS - LPS / 2>();
    }
    slot = next;
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();  // ring is dead from here on: every wave is past its last fragment read

  // ---- epilogue ----
  // A lane holds, per 32x32 block, one row and 4x4 consecutive columns.  Going
  // straight to memory would write 16-byte pieces of 32 different rows per
  // instruction; instead each wave transposes one 32-row band at a time
  // through its own LDS staging area and stores whole row segments.
  bf16_t *c = (bf16_t *)p.c;
  const float *bias = p.bias ? p.bias + (size_t)t.expert * p.n : nullptr;
  static_assert(NW * 32 * PITCH <= STAGES * SLOT_BYTES, "staging does not fit in the ring");
  unsigned char *stage = lds_raw + wave * (32 * PITCH);
  const int wave_col0 = t.n0 + (SWIGLU ? wn * (WTN / 2) : wn * WTN);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < OUT_BLOCKS; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = j * 32 + frag_half * 4 + q * 8;
        bf16x4_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[i][j][q * 4 + r];
          if (SWIGLU) {
            v = silu_fast(v) * acc[i][j + OUT_BLOCKS][q * 4 + r];
          } else {
            if (bias) v += bias[wave_col0 + col + r < p.n ? wave_col0 + col + r : 0];
            if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);
          }
          o[r] = (bf16_t)v;
        }
        *reinterpret_cast<u32x2_any_t *>(stage + frag_row * PITCH + col * 2) = __builtin_bit_cast(u32x2_t, o);
      }
    }
    wave_lds_sync();
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int r = ps * ROWS_PER_PASS + rd_row;
      const u32x4_t v = *reinterpret_cast<const u32x4_any_t *>(stage + r * PITCH + rd_chunk * 16);
      const int n = wave_col0 + rd_chunk * 8;
      if (out_row[i][ps] >= 0 && n < p.n)
        *reinterpret_cast<u32x4_t *>(c + (int64_t)out_row[i][ps] * p.ldc + n) = v;
    }
    wave_lds_sync();  // the next band overwrites the staging rows
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, bool W_FP8>
int launch_cfg(const GemmParams &p, int64_t max_rows, hipStream_t s) {
  constexpr int BN_OUT = MODE == kFc1Swiglu ? BN / 2 : BN;
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr size_t lds = 2ull * (BM + BN) * kBK * sizeof(bf16_t);
  const int64_t grid = max_tiles(max_rows, p.n_experts, p.n, BM, BN_OUT);
  if (grid <= 0) return DICE_OK;
  if (grid >= (1ll << 31)) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: grid too large");
  auto kern = grouped_gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, MODE, W_FP8>;
  if (lds > 48 * 1024) {
    static thread_local bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess)
        return fail(DICE_ERR_LAUNCH, "bf16 expert GEMM: LDS attribute: %s", hipGetErrorString(e));
      configured = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, s, p);
  return launch_status("grouped_gemm_bf16");
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE>
int launch_dl(const GemmParams &p, int64_t max_rows, hipStream_t s) {
  constexpr int BN_OUT = MODE == kFc1Swiglu ? BN / 2 : BN;
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr size_t lds = 2ull * (BM + BN) * kBK * sizeof(bf16_t);
  const int64_t grid = max_tiles(max_rows, p.n_experts, p.n, BM, BN_OUT);
  if (grid <= 0) return DICE_OK;
  if (grid >= (1ll << 31)) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: grid too large");
  auto kern = gemm_dl_kernel<BM, BN, WAVES_M, WAVES_N, MODE>;
  static thread_local bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return fail(DICE_ERR_LAUNCH, "bf16 expert GEMM: LDS attribute: %s", hipGetErrorString(e));
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, s, p);
  return launch_status("grouped_gemm_bf16");
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE, int STAGES>
int launch_ring(const GemmParams &p, int64_t max_rows, hipStream_t s) {
  constexpr int BN_OUT = MODE == kFc1Swiglu ? BN / 2 : BN;
  constexpr int NT = WAVES_M * WAVES_N * kWave;
  constexpr size_t lds = (size_t)STAGES * (BM + BN) * 64;
  static_assert(lds <= 160 * 1024, "ring does not fit the 160 KB LDS of a CU");
  if (p.k % kRingBK != 0) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: k %d %% 32 != 0", p.k);
  const int64_t grid = max_tiles(max_rows, p.n_experts, p.n, BM, BN_OUT);
  if (grid <= 0) return DICE_OK;
  if (grid >= (1ll << 31)) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: grid too large");
  auto kern = gemm_ring_kernel<BM, BN, WAVES_M, WAVES_N, MODE, STAGES>;
  static thread_local bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return fail(DICE_ERR_LAUNCH, "bf16 expert GEMM: LDS attribute: %s", hipGetErrorString(e));
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), lds, s, p);
  return launch_status("grouped_gemm_bf16");
}

int g_cfg_fc1 = 0, g_cfg_fc2 = 0;

template <int MODE, bool W_FP8>
int launch_mode(const GemmParams &p, int cfg, int64_t max_rows, hipStream_t s) {
  if (!W_FP8) {
    if (cfg == 3) return launch_dl<256, 256, 2, 2, MODE>(p, max_rows, s);
    if (cfg == 4) return launch_dl<256, 256, 2, 4, MODE>(p, max_rows, s);
    if (cfg == 5) return launch_dl<256, 128, 2, 2, MODE>(p, max_rows, s);
    if (cfg == 6) return launch_dl<128, 128, 2, 2, MODE>(p, max_rows, s);
    if (cfg == 7) return launch_ring<256, 256, 2, 2, MODE, 5>(p, max_rows, s);
    if (cfg == 8) return launch_ring<256, 256, 2, 2, MODE, 4>(p, max_rows, s);
    if (cfg == 9) return launch_ring<256, 256, 2, 4, MODE, 5>(p, max_rows, s);
    if (cfg == 10) return launch_ring<256, 128, 2, 2, MODE, 5>(p, max_rows, s);
    if (cfg == 11) return launch_ring<256, 256, 2, 2, MODE, 3>(p, max_rows, s);
  }
  switch (cfg) {
    case 1:
      return launch_cfg<256, 256, 2, 4, MODE, W_FP8>(p, max_rows, s);
    case 2:
      return launch_cfg<256, 128, 2, 2, MODE, W_FP8>(p, max_rows, s);
    default:
      return launch_cfg<128, 128, 2, 2, MODE, W_FP8>(p, max_rows, s);
  }
}

}  // namespace

int launch_grouped_gemm_bf16(const GemmParams &p, int mode, int w_dtype, int64_t max_rows,
                             hipStream_t s) {
  if (p.k % kBK != 0) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: k %d %% %d != 0", p.k, kBK);
  if (p.n % 8 != 0) return fail(DICE_ERR_UNSUPPORTED, "bf16 expert GEMM: n %d %% 8 != 0", p.n);
  const bool fp8 = w_dtype == DICE_FP8_E4M3;
  const int cfg = mode == kFc2 ? g_cfg_fc2 : g_cfg_fc1;
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
}

}  // namespace dice

namespace dice {
constexpr int kCfgPersistent = 20;
extern int g_persist_waves;
bool gemm_config_wants_persistent() { return g_cfg_fc1 >= kCfgPersistent && g_cfg_fc2 >= kCfgPersistent; }
}  // namespace dice

// Tuning hook: selects the tile configuration (0: 128x128x64 / 4 waves,
// 1: 256x256x64 / 8 waves, 2: 256x128x64 / 4 waves) per GEMM.  Not part of the
// drop-in surface; used by the benchmark to compare tilings.
extern "C" int dice_set_gemm_config(int fc1_cfg, int fc2_cfg) {
  dice::g_cfg_fc1 = fc1_cfg;
  dice::g_cfg_fc2 = fc2_cfg;
  // 20: the 32-k eight-wave pipeline only; anything else: the 64-k pipeline where it applies (default)
  dice::g_persist_waves = fc1_cfg == dice::kCfgPersistent ? 8 : 4;
  return DICE_OK;
}
