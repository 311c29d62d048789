// Persistent bf16 grouped GEMM for the expert MLPs (routed experts and the
// shared expert in ONE launch per GEMM stage).
//
// One workgroup per CU stays resident and walks a list of 256x256 output tiles;
// the k loop of consecutive tiles forms one continuous software pipeline:
//
//   * global -> LDS copies (buffer_load_dwordx4 ... lds) run AHEAD = 3 steps of
//     32 k ahead of the MFMAs in a ring of four 32 KB LDS slots and simply
//     carry on into the next tile while the current one finishes, so there is
//     no per-tile prologue and no workgroup re-launch between tiles;
//   * operands are addressed through buffer descriptors: the descriptor's
//     range check zero-fills rows past a group's end and past the last output
//     column, so ragged groups need no special code, and a tile switch only
//     rewrites a few SGPRs;
//   * eight waves (two per SIMD) each own a 128x64 block of the tile
//     (v_mfma_f32_32x32x16_bf16, fp32 accumulate); fragment reads of the next
//     half step and the copies are threaded between the MFMAs;
//   * the epilogue applies SwiGLU / GELU / bias, transposes through a small
//     LDS staging area and writes whole row segments with buffer stores (rows
//     past the group's end are dropped by the range check).
//
// Tiles are ordered problem-major, expert-major, then n-tile with the m-tile
// fastest; each XCD takes one contiguous run of that order so the 32 CUs that
// share an L2 work on the same expert's weights at the same time.
//
// Activations must be contiguous grouped rows (the dispatch kernel's gathered
// copy); weights are [experts, rows, k] bf16 as in the reference's nn.Linear
// layout (models.py:245-247).
#include "gemm_common.h"

namespace dice {
namespace {

constexpr int kPBM = 256, kPBN = 256, kPBK = 32;
constexpr int kPWavesM = 2, kPWavesN = 4, kPWaves = 8;
constexpr int kPStages = 4, kPAhead = 3;
constexpr int kPSlotBytes = (kPBM + kPBN) * 64;          // 32 KB
constexpr int kPRingBytes = kPStages * kPSlotBytes;      // 128 KB
constexpr int kPStageArea = 32 * 1024;                   // epilogue staging
constexpr int kPLdsBytes = kPRingBytes + kPStageArea;    // 160 KB
constexpr int kPCopiesA = kPBM / 16 / kPWaves;           // 1 KB copies per wave per step
constexpr int kPCopiesB = kPBN / 16 / kPWaves;
constexpr int kPCopies = kPCopiesA + kPCopiesB;
constexpr uint32_t kRsrcFlags = 0x00020000u;             // raw buffer, 32-bit elements
constexpr uint32_t kOutOfRange = 0x80000000u;            // voffset no descriptor covers

__device__ __forceinline__ int pswizzle(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }
__device__ __forceinline__ int pring_off(int row, int chunk) {
  return row * 64 + ((chunk ^ pswizzle(row)) << 4);
}

// Workgroup barrier that instructions may not be scheduled across.
__device__ __forceinline__ void phase_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

template <int N> __device__ __forceinline__ void pwait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int I, int N, int RD>
__device__ __forceinline__ void psched_reads() {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, (I == N - 1 && (RD & 1)) ? 1 : 2, 0);
    psched_reads<I + 1, N, RD>();
  }
}
template <int I, int N, int GAP>
__device__ __forceinline__ void psched_copies() {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, GAP, 0);
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    psched_copies<I + 1, N, GAP>();
  }
}
// Half a k step: two fragment reads behind each of the first MFMAs, then
// COPIES copies spread over the remaining MFMAs.
template <int MF, int RD, int COPIES>
__device__ __forceinline__ void psched_half() {
  constexpr int RDG = (RD + 1) / 2;
  static_assert(MF > RDG, "too few MFMAs to thread the fragment reads through");
  constexpr int REST = MF - RDG;
  constexpr int GAP = COPIES > 0 ? (REST / COPIES > 0 ? REST / COPIES : 1) : REST;
  psched_reads<0, RDG, RD>();
  psched_copies<0, COPIES, GAP>();
  constexpr int LEFT = REST - COPIES * GAP;
  if constexpr (LEFT > 0) __builtin_amdgcn_sched_group_barrier(0x008, LEFT, 0);
}

// Pins a wave-uniform value into SGPRs (the compiler cannot always prove uniformity
// of values derived from lane reads; a buffer descriptor held in VGPRs would
// cost a readfirstlane loop around every copy).
__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T> __device__ __forceinline__ T *uni(T *ptr) {
  const uint64_t v = reinterpret_cast<uint64_t>(ptr);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<T *>(((uint64_t)hi << 32) | lo);
}

// Everything a wave needs to know about one tile; all wave-uniform (SGPRs).
struct Tile {
  const unsigned char *a;    // first row of the tile
  uint32_t a_bytes;          // rows_valid * lda * 2
  uint32_t a_pitch;          // lda * 2
  const unsigned char *b0;   // weight rows of the tile (SwiGLU: gate rows)
  const unsigned char *b1;   // SwiGLU: up rows
  uint32_t b_bytes;          // valid weight rows * k * 2 (per half for SwiGLU)
  uint32_t b_pitch;          // k * 2
  unsigned char *c;          // first output row of the tile
  uint32_t c_bytes;          // rows_valid * ldc * 2
  uint32_t c_pitch;          // ldc * 2
  const float *bias;         // + expert * n, or NULL
  int n0, n;                 // first output column, output columns of the problem
  int steps;                 // k / 32
  bool valid;
};

// HAS_BIAS is a compile-time switch so that the bias-free (reference SwiGLU)
// instantiations carry no bias loads: a vector load in the epilogue makes the
// compiler wait for every outstanding copy and store.
template <int MODE, bool HAS_BIAS>
__global__ __launch_bounds__(kPWaves *kWave, 1) void gemm_persist_kernel(PersistBatch batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? kPBN / 2 : kPBN;
  constexpr int WTM = kPBM / kPWavesM, WTN = kPBN / kPWavesN;  // 128 x 64
  constexpr int TM = WTM / 32, TN = WTN / 32;                  // 4 x 2
  constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
  constexpr int OUT_COLS = OUT_BLOCKS * 32;
  constexpr int PITCH = OUT_COLS * 2 + 16;
  constexpr int BAND = (kPWaves * 32 * PITCH <= kPStageArea) ? 32 : 16;  // rows staged at a time
  static_assert(kPWaves * BAND * PITCH <= kPStageArea, "staging area too small");
  constexpr int LANES_PER_ROW = OUT_COLS * 2 / 16;
  constexpr int ROWS_PER_PASS = kWave / LANES_PER_ROW;
  constexpr int PASSES = BAND / ROWS_PER_PASS;
  static_assert(PASSES >= 1, "band smaller than one store pass");
  constexpr int STORES = (WTM / BAND) * PASSES;  // buffer stores per wave per tile
  constexpr int WAIT_STEADY = (kPAhead - 1) * kPCopies;  // copies of the two newest steps
  constexpr int WAIT_AFTER_EPILOGUE = WAIT_STEADY + STORES;
  static_assert(WAIT_AFTER_EPILOGUE < 64, "vmcnt is a 6-bit counter");

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / kPWavesN, wn = wave % kPWavesN;

  // ---- group table: lane g describes group g = (problem, expert) ----
  int g_prob = 0, g_expert = 0, g_row0 = 0, g_cnt = 0, g_mt = 0, g_nt = 0, g_base = 0;
  {
    int acc_groups = 0;
    for (int pi = 0; pi < batch.n_problems; ++pi) {
      const PersistProblem &pr = batch.prob[pi];
      const int local = lane - acc_groups;
      if (local >= 0 && local < pr.n_experts) {
        g_prob = pi;
        g_expert = local;
        g_row0 = pr.offsets[local];
        g_cnt = pr.offsets[local + 1] - g_row0;
        g_mt = (g_cnt + kPBM - 1) / kPBM;
        g_nt = (pr.n + BN_OUT - 1) / BN_OUT;
      }
      acc_groups += pr.n_experts;
    }
    int tiles = g_mt * g_nt, inc = tiles;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(inc, o, kWave);
      if (lane >= o) inc += up;
    }
    g_base = inc - tiles;
  }
  const int total_tiles = __shfl(g_base + g_mt * g_nt, kWave - 1, kWave);
  const int g_end = g_base + g_mt * g_nt;

  // This workgroup's share: XCD x (= blockIdx.x % 8) owns the x-th eighth of the
  // tile order; its workgroups take tiles of that run round-robin.
  const int per_xcd = (total_tiles + kNumXcd - 1) / kNumXcd;
  const int xcd = blockIdx.x % kNumXcd;
  const int wg_in_xcd = blockIdx.x / kNumXcd;
  const int wgs_per_xcd = gridDim.x / kNumXcd;
  const int run_begin = xcd * per_xcd;
  const int run_end = run_begin + per_xcd < total_tiles ? run_begin + per_xcd : total_tiles;

  auto decode = [&](int id) {
    Tile t;
    t.valid = id < run_end;
    const int idc = t.valid ? id : 0;
    const uint64_t hit = __ballot(idc >= g_base && idc < g_end);
    const int g = hit ? __builtin_ctzll(hit) : 0;
    const int pi = __builtin_amdgcn_readlane(g_prob, g);
    const int expert = __builtin_amdgcn_readlane(g_expert, g);
    const int row0 = __builtin_amdgcn_readlane(g_row0, g);
    const int cnt = __builtin_amdgcn_readlane(g_cnt, g);
    const int mt = __builtin_amdgcn_readlane(g_mt, g);
    const int base = __builtin_amdgcn_readlane(g_base, g);
    const PersistProblem &pr = batch.prob[pi];
    const int r = idc - base;
    const int n_tile = mt > 0 ? r / mt : 0;
    const int m_tile = r - n_tile * mt;
    const int left = cnt - m_tile * kPBM;
    const int rows = left < kPBM ? left : kPBM;
    t.n0 = n_tile * BN_OUT;
    t.n = pr.n;
    const int cols_left = pr.n - t.n0;
    const int wrows = cols_left < BN_OUT ? cols_left : BN_OUT;
    t.a_pitch = (uint32_t)pr.lda * 2;
    t.a = (const unsigned char *)pr.a + (size_t)(row0 + m_tile * kPBM) * t.a_pitch;
    t.a_bytes = t.valid ? (uint32_t)rows * t.a_pitch : 0;
    t.b_pitch = (uint32_t)pr.k * 2;
    const unsigned char *wexp = (const unsigned char *)pr.w + (size_t)expert * pr.w_rows * t.b_pitch;
    t.b0 = wexp + (size_t)t.n0 * t.b_pitch;
    t.b1 = wexp + (size_t)(pr.up_offset + t.n0) * t.b_pitch;
    t.b_bytes = t.valid ? (uint32_t)wrows * t.b_pitch : 0;
    t.c_pitch = (uint32_t)pr.ldc * 2;
    t.c = (unsigned char *)pr.c + (size_t)(row0 + m_tile * kPBM) * t.c_pitch;
    t.c_bytes = (uint32_t)rows * t.c_pitch;
    t.bias = pr.bias ? pr.bias + (size_t)expert * pr.n : nullptr;
    t.steps = pr.k / kPBK;
    t.a = uni(t.a); t.b0 = uni(t.b0); t.b1 = uni(t.b1); t.c = uni(t.c); t.bias = uni(t.bias);
    t.a_bytes = uni(t.a_bytes); t.a_pitch = uni(t.a_pitch);
    t.b_bytes = uni(t.b_bytes); t.b_pitch = uni(t.b_pitch);
    t.c_bytes = uni(t.c_bytes); t.c_pitch = uni(t.c_pitch);
    t.n0 = uni(t.n0); t.n = uni(t.n); t.steps = uni(t.steps);
    t.valid = uni((int)t.valid) != 0;
    return t;
  };

  // ---- per-lane copy offsets (row part depends on the tile's pitch) ----
  const int lrow = lane >> 2, lchunk = lane & 3;
  int cp_row[kPCopies];      // tile row (A) / weight row within its half (B)
  int cp_chunk[kPCopies];    // byte offset of the 16-byte chunk inside the 64-byte k slice
#pragma unroll
  for (int i = 0; i < kPCopiesA; ++i) {
    const int rt = (wave + kPWaves * i) * 16 + lrow;
    cp_row[i] = rt;
    cp_chunk[i] = (lchunk ^ pswizzle(rt)) << 4;
  }
#pragma unroll
  for (int i = 0; i < kPCopiesB; ++i) {
    const int rt = (wave + kPWaves * i) * 16 + lrow;  // row inside the 256-row weight tile
    cp_row[kPCopiesA + i] = SWIGLU ? rt % (kPBN / 2) : rt;
    cp_chunk[kPCopiesA + i] = (lchunk ^ pswizzle(rt)) << 4;
  }

  // Issues copy `l` of the step `kt` of tile `t` into ring slot `slot`.
  auto issue_copy = [&](const Tile &t, int kt, int slot, int l) {
    unsigned char *dst = lds_raw + slot * kPSlotBytes;
    if (l < kPCopiesA) {
      const __amdgpu_buffer_rsrc_t rs =
          __builtin_amdgcn_make_buffer_rsrc((void *)t.a, 0, t.a_bytes, kRsrcFlags);
      const uint32_t voff = (uint32_t)cp_row[l] * t.a_pitch + cp_chunk[l];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs, (__attribute__((address_space(3))) void *)(dst + (wave + kPWaves * l) * 1024), 16, voff,
          kt * 64, 0, 0);
    } else {
      const int i = l - kPCopiesA;
      const bool up_half = SWIGLU && (wave + kPWaves * i) * 16 >= kPBN / 2;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)(up_half ? t.b1 : t.b0), 0, t.b_bytes, kRsrcFlags);
      const uint32_t voff = (uint32_t)cp_row[l] * t.b_pitch + cp_chunk[l];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs,
          (__attribute__((address_space(3))) void *)(dst + kPBM * 64 + (wave + kPWaves * i) * 1024), 16,
          voff, kt * 64, 0, 0);
    }
  };

  auto w_block_row = [&](int j) {
    if (SWIGLU) {
      constexpr int HALF = TN / 2;
      return j < HALF ? wn * (WTN / 2) + j * 32 : kPBN / 2 + wn * (WTN / 2) + (j - HALF) * 32;
    }
    return wn * WTN + j * 32;
  };
  const int frag_row = lane & 31, frag_half = lane >> 5;
  bf16x8_t wf[2][TN], af[2][TM];
  auto read_frags = [&](int slot, int kk, int buf) {
    const unsigned char *sa = lds_raw + slot * kPSlotBytes;
    const unsigned char *sb = sa + kPBM * 64;
    const int chunk = kk * 2 + frag_half;
#pragma unroll
    for (int j = 0; j < TN; ++j)
      wf[buf][j] = *reinterpret_cast<const bf16x8_t *>(sb + pring_off(w_block_row(j) + frag_row, chunk));
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[buf][i] = *reinterpret_cast<const bf16x8_t *>(sa + pring_off(wm * WTM + i * 32 + frag_row, chunk));
  };

  f32x16_t acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
  };

  // ---- pipeline state ----
  int next_id = run_begin + wg_in_xcd;           // next tile the copy side will open
  Tile ld = decode(next_id);                     // tile being copied
  next_id += wgs_per_xcd;
  if (!ld.valid) return;                         // nothing to do for this workgroup
  Tile cp = ld;                                  // tile being multiplied
  int ld_kt = 0;
  int cslot = 0;                                 // ring slot of the step being multiplied

  // Advances the copy side by one step (wave-uniform control flow only).
  auto advance_copy = [&]() {
    if (++ld_kt == ld.steps) {
      ld = decode(next_id);
      next_id += wgs_per_xcd;
      ld_kt = 0;
    }
  };

#pragma unroll
  for (int s = 0; s < kPAhead; ++s) {
#pragma unroll
    for (int l = 0; l < kPCopies; ++l) issue_copy(ld, ld_kt, s, l);
    advance_copy();
  }
  zero_acc();
  pwait_vmcnt<WAIT_STEADY>();
  phase_barrier();                      // everyone's copies of steps 0 and 1 have landed
  int since_epilogue = 2;

  const int stage_base = kPRingBytes + wave * (BAND * PITCH);
  const int rd_row = lane / LANES_PER_ROW, rd_chunk = lane % LANES_PER_ROW;
  const int wave_col0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;

  // Two groups of four waves (one wave of each group per SIMD) alternate between
  // a memory phase (fragment reads of one k step + this wave's share of the
  // copies three steps ahead) and a compute phase (the step's 16 MFMAs), one
  // phase apart: while one group multiplies the other one loads, so the matrix
  // pipe only idles for the barrier hand-over between phases.
  const int group = wm;
  // Waits until at most the copies of the two newest steps (plus the stores of an
  // epilogue that was issued in between) are still in flight.
  auto copies_landed = [&]() {
    if (since_epilogue < 2) pwait_vmcnt<WAIT_AFTER_EPILOGUE>();
    else pwait_vmcnt<WAIT_STEADY>();
    ++since_epilogue;
  };
  while (true) {  // one tile per iteration
    if (group == 1) phase_barrier();
    for (int s = 0; s < cp.steps; ++s) {
      // ---- memory phase ----
      const int lslot = (cslot + kPAhead) & (kPStages - 1);  // slot of the step before this one
      read_frags(cslot, 0, 0);
      read_frags(cslot, 1, 1);
#pragma unroll
      for (int l = 0; l < kPCopies; ++l) issue_copy(ld, ld_kt, lslot, l);
      advance_copy();
      // The first reader of step s+1 is the first group, right after the barrier
      // that ends this phase pair.  Each wave therefore confirms that its own
      // copies of step s+1 have landed at the last barrier before that point:
      // the second group at the end of its memory phase, the first group at the
      // end of its compute phase.  Copies get four to five phases to land.
      if (group == 1) copies_landed();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // slot fully read before anyone may refill it
      phase_barrier();
      // ---- compute phase ----
#ifndef DICE_PRIO_COMPUTE
#define DICE_PRIO_COMPUTE 0
#endif
#ifndef DICE_PRIO_MEMORY
#define DICE_PRIO_MEMORY 0
#endif
      __builtin_amdgcn_s_setprio(DICE_PRIO_COMPUTE);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[kk][j], af[kk][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_s_setprio(DICE_PRIO_MEMORY);
      if (group == 0) copies_landed();
      phase_barrier();
      cslot = (cslot + 1) & (kPStages - 1);
    }
    if (group == 0) phase_barrier();  // let the other group finish the tile's last step

    // ---- epilogue of tile `cp` ----
    {
      const __amdgpu_buffer_rsrc_t crs =
          __builtin_amdgcn_make_buffer_rsrc((void *)cp.c, 0, cp.c_bytes, kRsrcFlags);
      unsigned char *stage = lds_raw + stage_base;
      const int col_base = cp.n0 + wave_col0;
      // Bias of this lane's columns, fetched in one batch (one wait instead of one per element).
      float bias_v[OUT_BLOCKS][16];
      if (HAS_BIAS) {
#pragma unroll
        for (int j = 0; j < OUT_BLOCKS; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) bias_v[j][e] = 0.f;
        if (cp.bias) {
#pragma unroll
          for (int j = 0; j < OUT_BLOCKS; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int cn = col_base + j * 32 + frag_half * 4 + (e >> 2) * 8 + (e & 3);
              bias_v[j][e] = cp.bias[cn < cp.n ? cn : 0];
            }
        }
      }
#pragma unroll
      for (int band = 0; band < WTM / BAND; ++band) {
        const int i = band * BAND / 32;             // 32-row block the band lies in
        const int half = (band * BAND % 32) / 16;   // which 16 rows of it (BAND == 16 only)
        if (BAND == 32 || (frag_row >> 4) == half) {
          const int srow = BAND == 32 ? frag_row : (frag_row & 15);
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
                  if (HAS_BIAS) v += bias_v[j][q * 4 + r];
                  if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);
                }
                o[r] = (bf16_t)v;
              }
              *reinterpret_cast<u32x2_any_t *>(stage + srow * PITCH + col * 2) = __builtin_bit_cast(u32x2_t, o);
            }
          }
        }
        wave_lds_sync();
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
          const int r = ps * ROWS_PER_PASS + rd_row;
          const u32x4_t v = *reinterpret_cast<const u32x4_any_t *>(stage + r * PITCH + rd_chunk * 16);
          const int m = wm * WTM + band * BAND + r;
          const int n = col_base + rd_chunk * 8;
          const uint32_t voff = n < cp.n ? (uint32_t)m * cp.c_pitch + (uint32_t)n * 2 : kOutOfRange;
          __builtin_amdgcn_raw_buffer_store_b128(v, crs, voff, 0, 0);
        }
        wave_lds_sync();  // the next band overwrites the staging rows
      }
    }
    // Every tile has more than AHEAD steps, so the copy side is exactly one
    // tile ahead here: the tile it is working on is the one to multiply next.
    cp = ld;
    if (!cp.valid) break;
    since_epilogue = 0;
    zero_acc();
  }
  pwait_vmcnt<0>();
}

}  // namespace

bool persist_supported(const PersistBatch &b, int mode) {
  int groups = 0;
  for (int i = 0; i < b.n_problems; ++i) {
    const PersistProblem &p = b.prob[i];
    groups += p.n_experts;
    if (p.k % kPBK != 0 || p.k < kPBK * (kPAhead + 1)) return false;
    if (p.n % 8 != 0 || p.lda % 8 != 0 || p.ldc % 8 != 0) return false;
    if (mode == kFc1Swiglu && p.n % (kPBN / 2) != 0) return false;  // gate/up halves share one range check
    if ((size_t)kPBM * p.lda * 2 >= (1ull << 31) || (size_t)kPBN * p.k * 2 >= (1ull << 31)) return false;
  }
  return groups >= 1 && groups <= kWave;
}

int launch_grouped_gemm_persist(const PersistBatch &b, int mode, hipStream_t s) {
  if (!persist_supported(b, mode))
    return fail(DICE_ERR_UNSUPPORTED, "persistent expert GEMM: unsupported shape");
  static thread_local int grid = 0;
  if (grid == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < kNumXcd)
      return fail(DICE_ERR_LAUNCH, "persistent expert GEMM: cannot query the CU count");
    grid = cus / kNumXcd * kNumXcd;
  }
  bool has_bias = false;
  for (int i = 0; i < b.n_problems; ++i) has_bias = has_bias || b.prob[i].bias != nullptr;
  if (mode == kFc1Swiglu) has_bias = false;
  void (*kern)(PersistBatch) = nullptr;
  switch (mode) {
    case kFc1Swiglu: kern = gemm_persist_kernel<kFc1Swiglu, false>; break;
    case kFc1Gelu: kern = has_bias ? gemm_persist_kernel<kFc1Gelu, true> : gemm_persist_kernel<kFc1Gelu, false>; break;
    default: kern = has_bias ? gemm_persist_kernel<kFc2, true> : gemm_persist_kernel<kFc2, false>; break;
  }
  const int slot = mode * 2 + (has_bias ? 1 : 0);
  static thread_local bool configured[6] = {false, false, false, false, false, false};
  if (!configured[slot]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kPLdsBytes);
    if (e != hipSuccess)
      return fail(DICE_ERR_LAUNCH, "persistent expert GEMM: LDS attribute: %s", hipGetErrorString(e));
    configured[slot] = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kPWaves * kWave), kPLdsBytes, s, b);
  return launch_status("grouped_gemm_persist");
}

}  // namespace dice
