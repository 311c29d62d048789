// What the persistent expert GEMM kernels share (grouped_gemm_persist.hip for 16-bit
// operands, compiled for bf16 and for fp16; grouped_gemm_persist_f8.hip for fp8
// activations and weights): operand types, the batch description, the tile
// order and the tile table (TileWalker), the accumulation-register helpers, the
// epilogue, the LDS layout of the 64-k pipeline, and the cut last turn (the sum
// of its pieces, the launcher's planning).  Everything sits in an unnamed
// namespace: each translation unit has its own copy.
#pragma once
#include <type_traits>

#include <algorithm>
#include <vector>

#include "gemm_common.h"

#ifndef DICE_PERSIST_F16
#define DICE_PERSIST_F16 0
#endif
#ifndef DICE_MFMA_ROWS_OUTERMOST
#define DICE_MFMA_ROWS_OUTERMOST 0
#endif

namespace dice {
namespace {

#if DICE_PERSIST_F16
typedef f16_t h16_t;
typedef f16x8_t h16x8_t;
typedef _Float16 h16x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x16_t mfma_32x32x16(h16x8_t a, h16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// two fp8 (e4m3) bytes of `src` (the low or the high pair) -> two fp16, exactly
__device__ __forceinline__ uint32_t widen_fp8_pair(uint32_t src, bool high) {
  return __builtin_bit_cast(uint32_t, high ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(src, 1.0f, true)
                                           : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(src, 1.0f, false));
}
#else
typedef bf16_t h16_t;
typedef bf16x8_t h16x8_t;
typedef bf16x4_t h16x4_t;
__device__ __forceinline__ f32x16_t mfma_32x32x16(h16x8_t a, h16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
// two fp8 (e4m3) bytes of `src` (the low or the high pair) -> two bf16, exactly
__device__ __forceinline__ uint32_t widen_fp8_pair(uint32_t src, bool high) {
  return __builtin_bit_cast(uint32_t, high ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(src, 1.0f, true)
                                           : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(src, 1.0f, false));
}
#endif

constexpr int kPBM = 256, kPBN = 256, kPBK = 32;
constexpr int kPWavesM = 2;
constexpr int kPStages = 4, kPAhead = 3;
constexpr int kPSlotBytes = (kPBM + kPBN) * 64;          // 32 KB
constexpr int kPRingBytes = kPStages * kPSlotBytes;      // 128 KB
constexpr int kPStageArea = 32 * 1024;                   // epilogue staging
constexpr int kPLdsBytes = kPRingBytes + kPStageArea;    // 160 KB
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

template <int V> using template_int = std::integral_constant<int, V>;

// Calls f(template_int<I>{}) for I = 0 .. N - 1: a loop whose index is a
// compile-time constant in the body (register numbers of inline assembly).
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(template_int<I>{});
    static_for<N, I + 1>(f);
  }
}

// ---- accumulators on fixed registers ----
// The 64-k kernel keeps its sums in the accumulation registers a0 .. a255 by
// NAME: block b (32 x 32 sums, 16 per lane) is a[16 b : 16 b + 15].  The
// products, the reads and the writes of these registers are inline assembly,
// so the compiler neither sees nor allocates them - it cannot move them between
// register files where code paths join (a second copy of the k loop made it
// spill hundreds of registers when the sums were its own values), and the order
// of the statements in the source is the order of the instructions: a volatile
// asm statement is a barrier to the scheduler for every memory instruction.
// What the compiler does not know it cannot protect, so the hazards are covered
// by hand: fixed_acc_settle() after the last product of a tile and before the
// first read of a sum (the matrix pipe's result is not interlocked against
// vector-ALU reads), and nothing else may touch an accumulation register - the
// build checks the generated code for that (dice_amd/build.py).
#if DICE_PERSIST_F16
#define DICE_MFMA16 "v_mfma_f32_32x32x16_f16"
#else
#define DICE_MFMA16 "v_mfma_f32_32x32x16_bf16"
#endif
// sums of block BLK += w x a
template <int BLK>
__device__ __forceinline__ void mfma_fixed(const h16x8_t &w, const h16x8_t &a) {
  asm volatile(DICE_MFMA16 " a[%2:%3], %0, %1, a[%2:%3]" ::"v"(w), "v"(a), "n"(BLK * 16), "n"(BLK * 16 + 15));
}
// sums of block BLK = z x z + 0 for a fragment z of zeros: clears the block on the
// matrix pipe, which is idle during an epilogue, instead of with sixteen
// vector-ALU writes that the epilogue's arithmetic would have to wait for
template <int BLK>
__device__ __forceinline__ void mfma_fixed_clear(const h16x8_t &z) {
  asm volatile(DICE_MFMA16 " a[%1:%2], %0, %0, 0" ::"v"(z), "n"(BLK * 16), "n"(BLK * 16 + 15));
}
template <int REG>
__device__ __forceinline__ float fixed_acc_get() {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(REG));
  return v;
}
template <int REG>
__device__ __forceinline__ void fixed_acc_set(float v) {
  asm volatile("v_accvgpr_write_b32 a[%1], %0" ::"v"(v), "n"(REG));
}
template <int BLK>
__device__ __forceinline__ f32x16_t fixed_acc_block() {
  f32x16_t t;
  static_for<16>([&](auto q) { t[decltype(q)::value] = fixed_acc_get<BLK * 16 + decltype(q)::value>(); });
  return t;
}
// Clears the top REGS accumulation registers, a[256 - REGS] .. a255.  A kernel
// with fewer than sixteen blocks keeps them at the top: the registers below are
// the ones the compiler takes first when it runs out of vector registers (it
// parks values there instead of in scratch memory), and it must find them free.
// The clobber names the highest register the kernel uses, which is how the
// compiler learns how many to reserve for the wave.
template <int REGS>
__device__ __forceinline__ void fixed_acc_clear() {
  static_assert(REGS == 256 || REGS == 192, "sixteen or twelve blocks");
  if constexpr (REGS == 256)
    asm volatile(".set dice_acc_r, 0\n.rept 256\nv_accvgpr_write_b32 a[dice_acc_r], 0\n.set dice_acc_r, dice_acc_r + 1\n.endr" ::: "a255");
  else
    asm volatile(".set dice_acc_r, 64\n.rept 192\nv_accvgpr_write_b32 a[dice_acc_r], 0\n.set dice_acc_r, dice_acc_r + 1\n.endr" ::: "a255");
}
// Tells the compiler that the kernel uses accumulation registers up to a255 (it
// sizes the wave's register file from the registers it sees named).
__device__ __forceinline__ void fixed_acc_declare() { asm volatile("" ::: "a255", "v255"); }
// Wait states between a product and a vector-ALU access to its sums (19 for the
// longest matrix instruction), and between a vector-ALU write and a product.
__device__ __forceinline__ void fixed_acc_settle() { asm volatile("s_nop 7\ns_nop 7\ns_nop 7"); }

template <int N> __device__ __forceinline__ void pwait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
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
  int steps;                 // pipeline steps (k / step extent)
  bool valid;
  const int32_t *a_rows;     // gathered tiles: slot of the tile's first row (else NULL)
  uint32_t a_magic;          // gathered tiles: source row = mulhi(slot, a_magic) (= slot / a_div); 0: a_div == 1
  int rows;                  // rows of the tile that belong to its group
};

// A tile description parked in ONE vector register (lane f holds 32-bit word f),
// for descriptions that are not needed for a while: scalar registers are scarce
// and a description spilled by the compiler would come back as per-lane values,
// which buffer instructions cannot take without a loop over lanes.
struct PackedTile {
  uint32_t words;
};
constexpr int kTileWords = 24;   // pointers a, b0, b1, c, bias, ten 32-bit fields, then a_rows, a_magic, rows
constexpr int kTableTurns = 64;  // turns of one workgroup that the LDS tile table holds
__device__ __forceinline__ Tile unpack_tile(const PackedTile &pk) {
  auto word = [&](int i) { return (uint32_t)__builtin_amdgcn_readlane(pk.words, i); };
  auto ptr = [&](int i) { return ((uint64_t)word(2 * i + 1) << 32) | word(2 * i); };
  Tile t;
  t.a = (const unsigned char *)ptr(0);
  t.b0 = (const unsigned char *)ptr(1);
  t.b1 = (const unsigned char *)ptr(2);
  t.c = (unsigned char *)ptr(3);
  t.bias = (const float *)ptr(4);
  t.a_bytes = word(10); t.a_pitch = word(11); t.b_bytes = word(12); t.b_pitch = word(13);
  t.c_bytes = word(14); t.c_pitch = word(15);
  t.n0 = (int)word(16); t.n = (int)word(17); t.steps = (int)word(18);
  t.valid = word(19) != 0;
  t.a_rows = (const int32_t *)(((uint64_t)word(21) << 32) | word(20));
  t.a_magic = word(22);
  t.rows = (int)word(23);
  return t;
}

// The tile order of one launch and this workgroup's share of it.  Lane g of
// every wave describes group g = (problem, expert): its rows, its tile grid and
// the index of its first tile (at most 64 groups); a tile id is mapped back to
// its group with one ballot.  Tiles are ordered problem-major, expert-major,
// then n-tile with the m-tile fastest; callers list the problem with the longest
// k first.  XCD x (= blockIdx.x % 8) owns the x-th eighth of every problem's tiles
// and its workgroups take the tiles of that run in turns.
// Position of tile `r` inside one (problem, expert) group of mt x nt tiles.
// The m-tile runs fastest, so that the workgroups of an XCD that work side by
// side share weight tiles; a group with many m-tiles (large batches) is cut
// into bands of about eight m-tiles, each taken through all n-tiles before the
// next, or a round of 32 workgroups would touch 32 different activation tiles
// and every one of them again for each n-tile.
struct TilePos {
  int m_tile, n_tile;
};
// `band_tiles` > 0 (tuning hook) sets the band height for every group with more
// m-tiles than that.
__device__ __forceinline__ TilePos tile_pos(int r, int mt, int nt, int band_tiles) {
  const int kBandTiles = band_tiles > 0 ? band_tiles : 8, kBandFrom = band_tiles > 0 ? band_tiles : 12;
  const int bands = mt > kBandFrom ? (mt + kBandTiles - 1) / kBandTiles : 1;
  const int band_m = (mt + bands - 1) / bands;          // m-tiles per band (the last may have fewer)
  const int per_band = band_m * nt > 0 ? band_m * nt : 1;
  const int band = r / per_band;
  const int r2 = r - band * per_band;
  const int left = mt - band * band_m;
  const int width = left < band_m ? (left > 0 ? left : 1) : (band_m > 0 ? band_m : 1);
  TilePos p;
  p.n_tile = r2 / width;
  p.m_tile = band * band_m + (r2 - p.n_tile * width);
  return p;
}

// Split turn.  The tiles of an XCD's run rarely fill its last turn: with R tiles
// left for W workgroups, W - R of them would idle for a whole tile.  Where the
// launch allows it (PersistBatch::split_ws: a plain-epilogue launch, whose
// products are linear in k) and R <= W / 3, the W workgroups are dealt out over
// those R tiles - W / R of them per tile, one more for the first W % R tiles, at
// most kSplitMaxWays - and each multiplies one piece of its tile's k range: runs
// of an even number of steps, at least kSplitMinSteps, that differ by at most
// two steps.  A piece writes its partial products, in the output type, to the
// partial-tile slot of its workgroup, and persist_split_sum_kernel adds the slots
// of a tile in fp32, in piece order, into the output rows.
constexpr int kSplitMinSteps = 6;
constexpr int kSplitMaxWays = 8;
// One workgroup position of the split turn.
struct SplitPiece {
  int tile;    // index of the tile within the turn
  int piece;   // which piece of it, 0 .. ways - 1
  int ways;    // pieces of that tile; 0: this position idles
  int first;   // position of the tile's first piece (pieces sit side by side)
};
// Steps [begin, begin + count) of piece `piece` of `ways` of a tile of `steps` steps.
struct SplitRange {
  int begin, count;
};
__device__ __forceinline__ SplitRange split_range(int steps, int piece, int ways) {
  const int pairs = steps / 2, base = pairs / ways, rem = pairs % ways;
  SplitRange r;
  r.begin = 2 * (piece * base + (piece < rem ? piece : rem));
  r.count = 2 * (base + (piece < rem ? 1 : 0));
  return r;
}

template <int BN_OUT>
struct TileWalker {
  int g_prob = 0, g_expert = 0, g_row0 = 0, g_cnt = 0, g_mt = 0, g_base = 0, g_end = 0;
  // This XCD's tiles: of every problem the x-th eighth of its tiles (sub_first:
  // id of the first, sub_len: how many), taken problem after problem.
  int sub_first[kMaxPersistProblems], sub_len[kMaxPersistProblems], run_len;
  int wg_in_xcd, wgs_per_xcd, xcd_id;
  int split_turn, split_left;   // the XCD's last, short turn and its tiles
  int split_q, split_extra;     // positions per tile of that turn when it is cut: q + 1 for the first `extra` tiles, q for the rest
  int split_cap;                // most pieces a tile's length allows; 0: the turn is not cut

  __device__ __forceinline__ TileWalker(const PersistBatch &batch, int lane)
      : TileWalker(batch, lane, (int)(blockIdx.x % kNumXcd), (int)(blockIdx.x / kNumXcd), (int)(gridDim.x / kNumXcd)) {}
  // (as seen by workgroup `wg` of `wgs` of XCD `xcd` of the launch that multiplies)
  __device__ __forceinline__ TileWalker(const PersistBatch &batch, int lane, int xcd, int wg, int wgs) {
    int g_nt = 0, g_k32 = 1, acc_groups = 0;
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
        g_k32 = pr.k / 32;
      }
      acc_groups += pr.n_experts;
    }
    const int tiles = g_mt * g_nt;
    // Inclusive scans over the groups: tile counts, and cost in units of 32 k
    // (tiles of different problems differ in length).
    const int cost = tiles * g_k32;
    int inc = tiles, cinc = cost;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(inc, o, kWave), cup = __shfl_up(cinc, o, kWave);
      if (lane >= o) {
        inc += up;
        cinc += cup;
      }
    }
    g_base = inc - tiles;
    g_end = inc;
    xcd_id = uni(xcd);
    wg_in_xcd = uni(wg);
    wgs_per_xcd = uni(wgs);
    // Two ways to give every XCD the same amount of work (the launcher picks one
    // per shape, see persist_xcd_split):
    //  0: XCD x takes the tiles between the x-th and the (x+1)-th eighth of the
    //     total COST in problem order.  XCDs then differ in their mix - some get
    //     only long tiles, some only short ones - which spreads the tiles with the
    //     most bytes per step over the whole launch, but an XCD whose long tiles
    //     just spill into another turn waits a whole long tile for a few of them
    //     (a skip step's fc2: 39 tiles of 72 steps for 32 workgroups).
    //  1: XCD x takes the x-th eighth of the tiles of EVERY problem (the tiles of
    //     one problem cost the same): the same mix everywhere; a workgroup's turns
    //     run from the longest tiles to the shortest, and one that got a long tile
    //     less makes up for it with short ones.
    int run_begin = 0, run_end = 0x7fffffff;   // (split 0) the XCD's stretch of the tile order
    if (batch.xcd_split == 0) {
      const int total_tiles = __shfl(inc, kWave - 1, kWave);
      const int total_cost = __shfl(cinc, kWave - 1, kWave);
      auto boundary = [&](int x) {
        if (x >= kNumXcd) return total_tiles;
        const int target = (int)((long long)total_cost * x / kNumXcd);
        const uint64_t hit = __ballot(cost > 0 && target >= cinc - cost && target < cinc);
        if (!hit) return total_tiles;
        const int g = __builtin_ctzll(hit);
        const int base = __builtin_amdgcn_readlane(g_base, g);
        const int cbase = __builtin_amdgcn_readlane(cinc - cost, g);
        const int k32 = __builtin_amdgcn_readlane(g_k32, g);
        return base + (target - cbase + k32 / 2) / k32;
      };
      run_begin = uni(boundary(xcd));
      run_end = uni(boundary(xcd + 1));
    }
    run_len = 0;
    int first_group = 0;
#pragma unroll
    for (int pi = 0; pi < kMaxPersistProblems; ++pi) {
      sub_first[pi] = sub_len[pi] = 0;
      if (pi < batch.n_problems) {
        const int last_group = first_group + batch.prob[pi].n_experts - 1;
        const int p_base = __builtin_amdgcn_readlane(g_base, first_group);
        const int p_end = __builtin_amdgcn_readlane(g_end, last_group);
        int lo, hi;
        if (batch.xcd_split == 0) {   // the problem's part of the XCD's stretch
          lo = run_begin > p_base ? run_begin : p_base;
          hi = run_end < p_end ? run_end : p_end;
        } else {
          const int p_tiles = p_end - p_base;
          lo = p_base + (int)((long long)p_tiles * xcd / kNumXcd);
          hi = p_base + (int)((long long)p_tiles * (xcd + 1) / kNumXcd);
        }
        sub_first[pi] = uni(lo);
        sub_len[pi] = uni(hi > lo ? hi - lo : 0);
        run_len += sub_len[pi];
        first_group = last_group + 1;
      }
    }
    split_turn = run_len / wgs_per_xcd;
    split_left = run_len - split_turn * wgs_per_xcd;
    split_q = split_extra = split_cap = 0;
  }

  // The id of the i-th tile of this XCD's run (kNoTile past its end).
  static constexpr int kNoTile = 0x7fffffff;
  __device__ __forceinline__ int run_tile(int i) const {
    int id = kNoTile;
#pragma unroll
    for (int pi = kMaxPersistProblems - 1; pi >= 0; --pi) {
      int before = 0;
#pragma unroll
      for (int q = 0; q < pi; ++q) before += sub_len[q];
      if (i >= before && i < before + sub_len[pi]) id = sub_first[pi] + (i - before);
    }
    return i >= 0 ? id : kNoTile;
  }

  // Decides whether the last turn is cut (launches with partial-tile slots
  // carry one problem, so every tile has prob[0].k / bk steps).
  __device__ __forceinline__ void plan_split(const PersistBatch &batch, int bk) {
    split_q = split_extra = split_cap = 0;
    if (batch.split_ws == nullptr || split_left <= 0) return;
    const int q = wgs_per_xcd / split_left;
    const int cap = batch.prob[0].k / bk / kSplitMinSteps;   // pieces of at least kSplitMinSteps steps
    // (A cut turn has no operand reuse between its workgroups: it runs at the
    // rate at which the XCD can bring in its tiles' operands, about a twelfth of a
    // tile's multiply time per tile, whatever the number of pieces - 8 tiles per
    // XCD at 2048 x 8192 took 55 us where a whole tile takes 93.  With fewer
    // than three workgroups per tile the cut no longer pays for itself and the
    // sum of its pieces.)
    if (q < 3 || cap < 2) return;
    split_cap = cap < kSplitMaxWays ? cap : kSplitMaxWays;
    split_q = q;
    split_extra = wgs_per_xcd - q * split_left;
  }
  // What position `w` of the cut turn multiplies.
  __device__ __forceinline__ SplitPiece split_piece(int w) const {
    const int wide = split_extra * (split_q + 1);
    SplitPiece sp;
    int width;
    if (w < wide) {
      sp.tile = w / (split_q + 1);
      width = split_q + 1;
      sp.first = sp.tile * width;
    } else {
      const int t = (w - wide) / split_q;
      sp.tile = split_extra + t;
      width = split_q;
      sp.first = wide + t * width;
    }
    sp.piece = w - sp.first;
    sp.ways = width < split_cap ? width : split_cap;
    if (sp.tile >= split_left || sp.piece >= sp.ways) sp.ways = 0;
    return sp;
  }
  // Position of the first piece of the turn's j-th tile and its number of pieces.
  __device__ __forceinline__ SplitPiece split_tile(int j) const {
    return split_piece(j < split_extra ? j * (split_q + 1) : split_extra * (split_q + 1) + (j - split_extra) * split_q);
  }

  // Partial-tile slot of workgroup position `w` of this XCD (kPBM rows of BN_OUT
  // columns in the output type).
  __device__ __forceinline__ uint64_t split_slot(const PersistBatch &batch, int w) const {
    return (uint64_t)batch.split_ws + (uint64_t)(xcd_id * wgs_per_xcd + w) * (kPBM * BN_OUT * 2);
  }

  // Describes 64 of this workgroup's turns at once - lane r works out turn
  // turn0 + r - and leaves them in LDS, kTileWords dwords per turn in PackedTile order, so
  // that a tile switch inside the kernel is a single LDS read.  Turns past the
  // XCD's run give descriptions that cover no bytes.  Called by one wave.
  // a8: the activations are fp8 bytes (one byte per element; no row table) and
  // words 20/21 carry the address of the tile's per-row scales instead.
  __device__ __forceinline__ void build_table(const PersistBatch &batch, int lane, int bk,
                                              uint32_t *table, bool w8 = false, int turn0 = 0,
                                              bool a8 = false) {
    plan_split(batch, bk);
    const int turn = turn0 + lane;  // entry `lane` of the table describes this turn
    const int w = (turn & 1) ? wgs_per_xcd - 1 - wg_in_xcd : wg_in_xcd;
    // (the split turn: positions j S .. j S + S - 1 share the turn's j-th tile)
    const bool cut = split_cap != 0 && turn == split_turn;
    const SplitPiece sp = cut ? split_piece(w) : SplitPiece{0, 0, 0, 0};
    const int id = run_tile(turn * wgs_per_xcd + (cut ? sp.tile : w));
    const bool valid = id != kNoTile && (!cut || sp.ways != 0);
    const int idc = valid ? id : 0;
    int n_groups = 0;
    for (int pi = 0; pi < batch.n_problems; ++pi) n_groups += batch.prob[pi].n_experts;
    int grp = 0;
    for (int g = 0; g < n_groups; ++g) {
      const int b = __builtin_amdgcn_readlane(g_base, g), e = __builtin_amdgcn_readlane(g_end, g);
      grp = (idc >= b && idc < e) ? g : grp;
    }
    const int pi = __shfl(g_prob, grp, kWave), expert = __shfl(g_expert, grp, kWave);
    const int row0 = __shfl(g_row0, grp, kWave), cnt = __shfl(g_cnt, grp, kWave);
    const int mt = __shfl(g_mt, grp, kWave), base = __shfl(g_base, grp, kWave);
    // this lane's problem (a handful of selects instead of a divergent struct index)
    uint64_t pa = 0, pw = 0, pc = 0, pbias = 0, prows = 0, pascale = 0, pablock = 0;
    bool c8 = false;
    int max_rows = 0;
    int lda = 0, ldc = 0, w_rows = 0, up_offset = 0, n = 0, k = 0, a_div = 1, a_src_rows = 0;
    for (int q = 0; q < batch.n_problems; ++q) {
      const PersistProblem &pr = batch.prob[q];
      if (pi == q) {
        pa = (uint64_t)pr.a; pw = (uint64_t)pr.w; pc = (uint64_t)pr.c; pbias = (uint64_t)pr.bias;
        lda = pr.lda; ldc = pr.ldc; w_rows = pr.w_rows; up_offset = pr.up_offset; n = pr.n; k = pr.k;
        prows = (uint64_t)pr.a_rows; a_div = pr.a_div; a_src_rows = pr.a_src_rows;
        pascale = (uint64_t)pr.a_scale;
        pablock = (uint64_t)pr.a_block_scale;
        c8 = pr.c_block_scale != nullptr;
        max_rows = pr.max_rows;
      }
    }
    const int r = idc - base;
    const TilePos tp = tile_pos(r, mt, (n + BN_OUT - 1) / BN_OUT, batch.band_tiles);
    const int n_tile = tp.n_tile, m_tile = tp.m_tile;
    const int left = cnt - m_tile * kPBM;
    const int rows = left < kPBM ? left : kPBM;
    const int n0 = n_tile * BN_OUT;
    const int cols_left = n - n0;
    const int wrows = cols_left < BN_OUT ? cols_left : BN_OUT;
    // (fp8 weights: one byte per element, and word 22 carries the row of the
    // per-output-channel scale table instead of the gather's reciprocal, which a
    // single-problem launch takes from its arguments)
    const uint32_t a_pitch = (uint32_t)lda * (a8 ? 1 : 2), b_pitch = (uint32_t)k * (w8 ? 1 : 2);
    uint32_t c_pitch = (uint32_t)ldc * (c8 ? 1 : 2), c_extent = (uint32_t)rows * c_pitch;
    const uint64_t wexp = pw + (uint64_t)expert * w_rows * b_pitch;
    // Gathered rows are addressed from the start of the source matrix.
    uint64_t ptrs[5] = {prows ? pa : pa + (uint64_t)(row0 + m_tile * kPBM) * a_pitch, wexp + (uint64_t)n0 * b_pitch,
                        wexp + (uint64_t)(up_offset + n0) * b_pitch,
                        pc + (uint64_t)(row0 + m_tile * kPBM) * c_pitch,
                        pbias ? pbias + ((uint64_t)expert * n) * sizeof(float) : 0};
    int steps = k / bk;
    uint32_t k_first = 0;
    if (cut && sp.ways != 0) {
      // This position's piece of the tile: its run of steps (the k offset moves
      // the operands' base addresses; range checks look at row offsets only), and
      // the position's partial-tile slot as the output, addressed so that column
      // n0 is the slot's first.  The bias rides on the first piece.
      const SplitRange run = split_range(steps, sp.piece, sp.ways);
      steps = run.count;
      const uint32_t k0 = (uint32_t)(run.begin * bk);
      k_first = k0;
      ptrs[0] += (uint64_t)k0 * (a8 ? 1 : 2);
      ptrs[1] += (uint64_t)k0 * (w8 ? 1 : 2);
      ptrs[2] += (uint64_t)k0 * (w8 ? 1 : 2);
      c_pitch = BN_OUT * 2;
      c_extent = (uint32_t)rows * c_pitch + (uint32_t)n0 * 2;
      ptrs[3] = split_slot(batch, w) - (uint64_t)n0 * 2;
      if (sp.piece != 0) ptrs[4] = 0;
    }
    const uint32_t a_extent = prows ? (uint32_t)a_src_rows * a_pitch : (uint32_t)rows * a_pitch;
    const uint32_t words[10] = {valid ? a_extent : 0u, a_pitch, valid ? (uint32_t)wrows * b_pitch : 0u,
                                b_pitch, c_extent, c_pitch, (uint32_t)n0, (uint32_t)n,
                                (uint32_t)steps, valid ? 1u : 0u};
    uint32_t *entry = table + lane * kTileWords;
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      entry[2 * i] = (uint32_t)ptrs[i];
      entry[2 * i + 1] = (uint32_t)(ptrs[i] >> 32);
    }
#pragma unroll
    for (int i = 0; i < 10; ++i) entry[10 + i] = words[i];
    // (fp8 activations: the tile's first row scale, or the dword of its first row's block scales in the tile's
    // first step - the next step's lie max_rows dwords on)
    const uint64_t tile_rows = a8 ? (pablock ? pablock + ((uint64_t)(k_first / 128) * (uint32_t)max_rows +
                                                          (uint64_t)(row0 + m_tile * kPBM)) * 4
                                             : pascale + (uint64_t)(row0 + m_tile * kPBM) * sizeof(float))
                                  : (prows ? prows + (uint64_t)(row0 + m_tile * kPBM) * sizeof(int32_t) : 0);
    entry[20] = (uint32_t)tile_rows;
    entry[21] = (uint32_t)(tile_rows >> 32);
    entry[22] = w8 ? (uint32_t)(expert * w_rows + n0)
                   : (uint32_t)(0xffffffffull / (uint32_t)a_div + 1);  // mulhi(slot, .) = slot / a_div for slot < 2^28, a_div <= 16
    entry[23] = (uint32_t)(valid ? rows : 0);
  }

  // The id of the tile this workgroup takes in its `round`-th turn.  Turns
  // alternate direction over the XCD's workgroups (0..W-1, W-1..0, ...): the
  // order runs from the longest tiles to the shortest, so the workgroups that got
  // the last long tiles get the fewest short ones.
  __device__ __forceinline__ int tile_id(int round) const {
    const int w = (round & 1) ? wgs_per_xcd - 1 - wg_in_xcd : wg_in_xcd;
    return uni(run_tile(round * wgs_per_xcd + w));
  }

  // Tile `id` of the order (ids past this XCD's run give an invalid tile whose
  // descriptors cover no bytes); `bk` is the k extent of one pipeline step.
  __device__ __forceinline__ Tile decode(const PersistBatch &batch, int id, int bk) const {
    Tile t;
    id = uni(id);  // wave-uniform by construction; says so to the compiler (scalar arithmetic below)
    t.valid = id != kNoTile;
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
    const TilePos tp = tile_pos(r, mt, (pr.n + BN_OUT - 1) / BN_OUT, batch.band_tiles);
    const int n_tile = tp.n_tile, m_tile = tp.m_tile;
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
    t.steps = pr.k / bk;
    t.a_rows = nullptr;
    t.a_magic = 0;
    t.rows = rows;
    t.a = uni(t.a); t.b0 = uni(t.b0); t.b1 = uni(t.b1); t.c = uni(t.c); t.bias = uni(t.bias);
    t.a_bytes = uni(t.a_bytes); t.a_pitch = uni(t.a_pitch);
    t.b_bytes = uni(t.b_bytes); t.b_pitch = uni(t.b_pitch);
    t.c_bytes = uni(t.c_bytes); t.c_pitch = uni(t.c_pitch);
    t.n0 = uni(t.n0); t.n = uni(t.n); t.steps = uni(t.steps);
    t.valid = uni((int)t.valid) != 0;
    return t;
  }
};

// Geometry of one wave's epilogue: its TM x TN accumulator blocks become
// OUT_COLS output columns (SwiGLU folds gate and up blocks), staged BAND rows at
// a time through WAVE_BYTES of LDS and stored as whole 16-byte row chunks.
template <int MODE, int WAVES, int TM, int TN, int RESERVE = 0>
struct EpiGeom {
  static constexpr bool SWIGLU = MODE == kFc1Swiglu;
  static constexpr int OUT_BLOCKS = SWIGLU ? TN / 2 : TN;
  static constexpr int OUT_COLS = OUT_BLOCKS * 32;
  static constexpr int PITCH = OUT_COLS * 2 + 16;
  // rows staged at a time (RESERVE: bytes of the staging area that other tables take)
  static constexpr int BAND = (WAVES * 32 * PITCH + RESERVE <= kPStageArea) ? 32 : 16;
  static constexpr int LANES_PER_ROW = OUT_COLS * 2 / 16;
  static constexpr int ROWS_PER_PASS = kWave / LANES_PER_ROW;   // lanes past ROWS_PER_PASS rows idle
  static constexpr int PASSES = (BAND + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
  static constexpr bool EXACT = kWave % LANES_PER_ROW == 0 && BAND % ROWS_PER_PASS == 0;
  static constexpr int STORES = (TM * 32 / BAND) * PASSES;  // buffer stores per wave per tile
  static constexpr int WAVE_BYTES = BAND * PITCH;
  static_assert(WAVES * WAVE_BYTES <= kPStageArea, "staging area too small");
  static_assert(PASSES >= 1, "band smaller than one store pass");
};

// One 32x32 accumulator block for the epilogue's arithmetic.  With four waves the
// accumulators live in the accumulation registers; left to itself the compiler
// copies all of them out at the top of the epilogue and then spills, so the block
// is pulled into vector registers at the place where it is used (the empty asm
// statement demands a vector-register operand and cannot be moved).
template <bool FROM_ACC_REGS>
__device__ __forceinline__ f32x16_t acc_block(const f32x16_t &a) {
  f32x16_t t = a;
  if constexpr (FROM_ACC_REGS) asm volatile("" : "+v"(t));
  return t;
}

// Epilogue of tile `cp` for one wave: activation (and bias), transposition through
// the wave's LDS staging rows, row-segment stores.  Rows past the group's end are
// dropped by the descriptor's range check, columns past the problem's n by an
// offset no descriptor covers.
// HAS_SCALE: the weights were fp8; column c of the product is multiplied by
// scale_lds[c - n0] (SwiGLU: gate columns first, the up columns 128 floats on).
// HAS_ROW: the activations were fp8 with one scale per row; row m of the tile is
// multiplied by rowscale_lds[m] as well.
// BIAS_LDS: the bias of the tile's columns sits in LDS (bias_lds[c - n0]) and is
// read four values at a time where it is added, instead of being held in
// registers for the whole epilogue (HAS_BIAS) or folded into the accumulators.
// ACC_BLOCK0 >= 0: the sums are not in `acc` but in the accumulation registers by
// name (block (i, j) = a[16 (ACC_BLOCK0 + i TN + j) ..], see mfma_fixed); the
// caller has let the last products settle.  CLEAR_ACC: every block is cleared as
// soon as it has been read (mfma_fixed_clear), so the next tile's products can
// add to it at once.
// ROW_STRIDE: tile rows between a wave's consecutive 32-row blocks (32: the wave
// owns a solid band of the tile; 64: the two waves that share a tile's columns
// take alternate 32-row blocks).  live_blocks (wave-uniform): only the wave's
// first live_blocks row blocks hold rows of the group (a group's last tile);
// the others were not multiplied and are not touched.
template <int MODE, bool HAS_BIAS, int WAVES, int TM, int TN, bool HAS_SCALE = false, int RESERVE = 0,
          bool HAS_ROW = false, bool BIAS_LDS = false, int ACC_BLOCK0 = -1, bool CLEAR_ACC = false,
          int ROW_STRIDE = 32>
__device__ __forceinline__ void tile_epilogue(const Tile &cp, f32x16_t (&acc)[TM][TN], unsigned char *stage,
                                              int wave_row0, int wave_col0, int lane,
                                              const float *scale_lds = nullptr,
                                              const float *rowscale_lds = nullptr,
                                              const float *bias_lds = nullptr, int live_blocks = TM) {
  static_assert(!(HAS_BIAS && BIAS_LDS), "one source of the bias");
  using G = EpiGeom<MODE, WAVES, TM, TN, RESERVE>;
  constexpr bool SWIGLU = G::SWIGLU;
  constexpr int OUT_BLOCKS = G::OUT_BLOCKS, PITCH = G::PITCH, BAND = G::BAND;
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int rd_row = lane / G::LANES_PER_ROW, rd_chunk = lane % G::LANES_PER_ROW;
  const __amdgpu_buffer_rsrc_t crs =
      __builtin_amdgcn_make_buffer_rsrc((void *)uni(cp.c), 0, uni(cp.c_bytes), kRsrcFlags);
  const int col_base = cp.n0 + wave_col0;
  // (a fragment of zeros, made here and not ahead of the tile loop, where it
  // would hold four registers through the k-loop)
  h16x8_t zero_frag;
  if constexpr (CLEAR_ACC) {
    u32x4_t z;
    asm volatile("v_mov_b32 %0, 0\nv_mov_b32 %1, 0\nv_mov_b32 %2, 0\nv_mov_b32 %3, 0"
                 : "=v"(z[0]), "=v"(z[1]), "=v"(z[2]), "=v"(z[3]));
    zero_frag = __builtin_bit_cast(h16x8_t, z);
  }
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
#define DICE_EPI_SCALES(j, q)                                                                         \
  f32x4_t sg, su;                                                                                     \
  if (HAS_SCALE) {                                                                                    \
    const float *sp = scale_lds + wave_col0 + (j) * 32 + frag_half * 4 + (q) * 8;                       \
    sg = *reinterpret_cast<const f32x4_t *>(sp);                                                      \
    if (SWIGLU) su = *reinterpret_cast<const f32x4_t *>(sp + 128);                                    \
    if (HAS_ROW) {                                                                                    \
      sg *= row_scale;                                                                                \
      if (SWIGLU) su *= row_scale;                                                                    \
    }                                                                                                 \
  }                                                                                                   \
  f32x4_t sb;                                                                                         \
  if (BIAS_LDS) sb = *reinterpret_cast<const f32x4_t *>(bias_lds + wave_col0 + (j) * 32 + frag_half * 4 + (q) * 8);
#define DICE_EPI_VALUE(v, j, q, r)                          \
  do {                                                      \
    if (HAS_SCALE) v *= sg[r];                              \
    if (SWIGLU) {                                           \
      float u = up[(q) * 4 + (r)];                          \
      if (HAS_SCALE) u *= su[r];                            \
      v = silu_fast(v) * u;                                 \
    } else {                                                \
      if (HAS_BIAS) v += bias_v[j][(q) * 4 + (r)];          \
      if (BIAS_LDS) v += sb[r];                             \
      if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);          \
    }                                                       \
  } while (0)
#define DICE_EPI_STORE_BAND(row_off)                                                                        \
  do {                                                                                                     \
    wave_lds_sync();                                                                                       \
    _Pragma("unroll") for (int ps = 0; ps < G::PASSES; ++ps) {                                             \
      int r = ps * G::ROWS_PER_PASS + rd_row;                                                              \
      bool live = true;                                                                                    \
      if (!G::EXACT) {                                                                                     \
        live = rd_row < G::ROWS_PER_PASS && r < BAND;                                                      \
        r = live ? r : 0;                                                                                  \
      }                                                                                                    \
      const u32x4_t v = *reinterpret_cast<const u32x4_any_t *>(stage + r * PITCH + rd_chunk * 16);         \
      const int m = wave_row0 + (row_off) + r;                                                             \
      const int n = col_base + rd_chunk * 8;                                                               \
      const uint32_t voff = (live && n < cp.n) ? (uint32_t)m * cp.c_pitch + (uint32_t)n * 2 : kOutOfRange; \
      __builtin_amdgcn_raw_buffer_store_b128(v, crs, voff, 0, 0);                                          \
    }                                                                                                      \
    wave_lds_sync(); /* the next band overwrites the staging rows */                                       \
  } while (0)
  static_for<TM>([&](auto i_c) {
    constexpr int i = decltype(i_c)::value;
    if (i >= live_blocks) return;
    float row_scale = 1.0f;
    if (HAS_ROW) row_scale = rowscale_lds[wave_row0 + i * ROW_STRIDE + frag_row];
    if constexpr (BAND == 32) {
      static_for<OUT_BLOCKS>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        f32x16_t blk, up;
        if constexpr (ACC_BLOCK0 >= 0) {
          blk = fixed_acc_block<ACC_BLOCK0 + i * TN + j>();
          if constexpr (SWIGLU) up = fixed_acc_block<ACC_BLOCK0 + i * TN + j + OUT_BLOCKS>();
          if constexpr (CLEAR_ACC) {   // ready for the next tile's sums
            mfma_fixed_clear<ACC_BLOCK0 + i * TN + j>(zero_frag);
            if constexpr (SWIGLU) mfma_fixed_clear<ACC_BLOCK0 + i * TN + j + OUT_BLOCKS>(zero_frag);
          }
        } else {
          blk = acc_block<WAVES == 4>(acc[i][j]);
          if constexpr (SWIGLU) up = acc_block<WAVES == 4>(acc[i][j + OUT_BLOCKS]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = j * 32 + frag_half * 4 + q * 8;
          h16x4_t o;
          DICE_EPI_SCALES(j, q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = blk[q * 4 + r];
            DICE_EPI_VALUE(v, j, q, r);
            o[r] = (h16_t)v;
          }
          *reinterpret_cast<u32x2_any_t *>(stage + frag_row * PITCH + col * 2) = __builtin_bit_cast(u32x2_t, o);
        }
      });
      DICE_EPI_STORE_BAND(i * ROW_STRIDE);
    } else {
      // The staging rows hold 16 rows at a time.  The activation of the whole
      // 32-row block is worked out once, with every lane at work (per band only
      // half the lanes own rows), and kept packed while its two bands go out.
      h16x4_t packed[OUT_BLOCKS][4];
      static_for<OUT_BLOCKS>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        f32x16_t blk, up;
        if constexpr (ACC_BLOCK0 >= 0) {
          blk = fixed_acc_block<ACC_BLOCK0 + i * TN + j>();
          if constexpr (SWIGLU) up = fixed_acc_block<ACC_BLOCK0 + i * TN + j + OUT_BLOCKS>();
          if constexpr (CLEAR_ACC) {   // ready for the next tile's sums
            mfma_fixed_clear<ACC_BLOCK0 + i * TN + j>(zero_frag);
            if constexpr (SWIGLU) mfma_fixed_clear<ACC_BLOCK0 + i * TN + j + OUT_BLOCKS>(zero_frag);
          }
        } else {
          blk = acc_block<WAVES == 4>(acc[i][j]);
          if constexpr (SWIGLU) up = acc_block<WAVES == 4>(acc[i][j + OUT_BLOCKS]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          DICE_EPI_SCALES(j, q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = blk[q * 4 + r];
            DICE_EPI_VALUE(v, j, q, r);
            packed[j][q][r] = (h16_t)v;
          }
        }
      });
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if ((frag_row >> 4) == half) {
#pragma unroll
          for (int j = 0; j < OUT_BLOCKS; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int col = j * 32 + frag_half * 4 + q * 8;
              *reinterpret_cast<u32x2_any_t *>(stage + (frag_row & 15) * PITCH + col * 2) =
                  __builtin_bit_cast(u32x2_t, packed[j][q]);
            }
        }
        DICE_EPI_STORE_BAND(i * ROW_STRIDE + half * 16);
      }
    }
    // Keeps the 32-row blocks apart: hoisting the next block's accumulator reads
    // over this one's stores only lengthens live ranges (register spills cost far
    // more here than the lost overlap).
    __builtin_amdgcn_sched_barrier(0);
  });
#undef DICE_EPI_VALUE
#undef DICE_EPI_SCALES
#undef DICE_EPI_STORE_BAND
}

// The epilogue of an fp8 fc1 tile whose output goes out as e4m3 bytes with one
// power-of-two scale per row and 32 columns (what the scaled MFMA of the next
// GEMM takes), instead of 16-bit values that a quantiser launch would read
// back.  A lane holds 16 of the 32 columns of one row of a block; the other 16
// sit in the lane 32 on.  Per block, from the activation value rounded to the
// 16-bit type (so that the bytes are a function of the h the 16-bit epilogue
// would have written):
//   amax = max |h|;  t = amax * fp32(1 / 448);  e = exponent field of t, plus one
//   if t is not a power of two (2^(e - 127) >= amax / 448);  byte = e4m3(rne(h * 2^(127 - e)))
// A block that holds a NaN or an infinity becomes NaN bytes with scale 1.
// Scale bytes go to cscale[((column / 128) * scale_rows + row) * 4 + block_scale_pos(column / 32)]
// (cscale: the dword of the tile's first row in the first step).
// The sums are in the accumulation registers (block (i, j) = a[16 (i TN + j) ..]).
template <int MODE, int WAVES, int TN, int RESERVE>
struct BlockqGeom {
  static constexpr int OUT_BLOCKS = MODE == kFc1Swiglu ? TN / 2 : TN, OUT_COLS = OUT_BLOCKS * 32, PITCH = OUT_COLS + 16;
  // rows of a block staged at a time (RESERVE: bytes of the staging area that other tables take)
  static constexpr int BAND = (WAVES * 32 * PITCH + RESERVE <= kPStageArea) ? 32 : 16;
  static constexpr int WAVE_BYTES = BAND * PITCH;
  static_assert(WAVES * WAVE_BYTES + RESERVE <= kPStageArea, "staging area too small");
};
template <int MODE, int WAVES, int TM, int TN, bool BIAS_LDS, int ROW_STRIDE, int RESERVE>
__device__ __forceinline__ void tile_epilogue_blockq(const Tile &cp, unsigned char *stage, int wave_row0, int wave_col0,
                                                     int lane, const float *scale_lds, const float *rowscale_lds,
                                                     const float *bias_lds, int live_blocks, unsigned char *cscale,
                                                     uint32_t scale_rows) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  using G = BlockqGeom<MODE, WAVES, TN, RESERVE>;
  constexpr int OUT_BLOCKS = G::OUT_BLOCKS, OUT_COLS = G::OUT_COLS, PITCH = G::PITCH, BAND = G::BAND;
  constexpr int LANES_PER_ROW = OUT_COLS / 16, ROWS_PER_PASS = kWave / LANES_PER_ROW, PASSES = BAND / ROWS_PER_PASS;
  static_assert(PASSES >= 1 && BAND % ROWS_PER_PASS == 0, "whole store passes");
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int rd_row = lane / LANES_PER_ROW, rd_chunk = lane % LANES_PER_ROW;
  const __amdgpu_buffer_rsrc_t crs =
      __builtin_amdgcn_make_buffer_rsrc((void *)uni(cp.c), 0, uni(cp.c_bytes), kRsrcFlags);
  const __amdgpu_buffer_rsrc_t srs = __builtin_amdgcn_make_buffer_rsrc(
      (void *)uni(cscale), 0, uni((uint32_t)((cp.n + 127) >> 7) * scale_rows * 4u), kRsrcFlags);   // (rows are checked below)
  const int col_base = cp.n0 + wave_col0;
  static_for<TM>([&](auto i_c) {
    constexpr int i = decltype(i_c)::value;
    if (i >= live_blocks) return;
    const float row_scale = rowscale_lds[wave_row0 + i * ROW_STRIDE + frag_row];
    uint32_t packed[OUT_BLOCKS][4];
    static_for<OUT_BLOCKS>([&](auto j_c) {
      constexpr int j = decltype(j_c)::value;
      f32x16_t blk = fixed_acc_block<i * TN + j>(), up;
      if constexpr (SWIGLU) up = fixed_acc_block<i * TN + j + OUT_BLOCKS>();
      // (maxima of the magnitudes as packed 16-bit integers: non-negative values of the 16-bit type order like
      // their bits, NaN above all)
      typedef h16_t h16pair_t __attribute__((ext_vector_type(2)));
      typedef unsigned short u16pair_t __attribute__((ext_vector_type(2)));
      u16pair_t amax2 = {0, 0};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float *sp = scale_lds + wave_col0 + j * 32 + frag_half * 4 + q * 8;
        f32x4_t sg = *reinterpret_cast<const f32x4_t *>(sp), su, sb;
        sg *= row_scale;
        if (SWIGLU) su = *reinterpret_cast<const f32x4_t *>(sp + 128) * row_scale;
        if (BIAS_LDS) sb = *reinterpret_cast<const f32x4_t *>(bias_lds + wave_col0 + j * 32 + frag_half * 4 + q * 8);
        float vv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = blk[q * 4 + r] * sg[r];
          if (SWIGLU) {
            v = silu_fast(v) * (up[q * 4 + r] * su[r]);
          } else {
            if (BIAS_LDS) v += sb[r];
            if (MODE == kFc1Gelu) v = gelu_tanh_fast(v);
          }
          vv[r] = v;
        }
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          static_assert(MODE < 0 || !DICE_PERSIST_F16, "bf16 rows (the fp8 kernels take no other)");
          const h16pair_t hp = {(h16_t)vv[r], (h16_t)vv[r + 1]};
          const uint32_t pr = __builtin_bit_cast(uint32_t, hp);
          blk[q * 4 + r] = __uint_as_float(pr << 16);             // (bf16: the value is its bits, 16 up)
          blk[q * 4 + r + 1] = __uint_as_float(pr & 0xffff0000u);
          amax2 = __builtin_elementwise_max(amax2, __builtin_bit_cast(u16pair_t, pr & 0x7fff7fffu));
        }
      }
      uint32_t amax_bits = (uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1]) << 16;
      // (the row's other 16 columns sit in the lane 32 on: one swap of the lane halves of two copies, then
      // every lane holds both maxima)
      {
        const auto both = __builtin_amdgcn_permlane32_swap(amax_bits, amax_bits, false, false);
        amax_bits = both[0] > both[1] ? both[0] : both[1];
      }
      const bool bad = amax_bits >= 0x7f800000u;
      const uint32_t tb = __float_as_uint(__uint_as_float(amax_bits) * (1.0f / 448.0f));
      uint32_t e = (tb >> 23) + ((tb & 0x7fffffu) != 0 ? 1u : 0u);
      e = bad ? 127u : e;
      const float inv = __uint_as_float((254u - e) << 23);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float f[4];
#pragma unroll
        // (no clamp: the scale is at least amax / 448 for a 16-bit amax, so the products stay within +-448)
        for (int r = 0; r < 4; ++r) f[r] = blk[q * 4 + r] * inv;
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
        packed[j][q] = bad ? 0x7f7f7f7fu : (uint32_t)w;
      }
      const int n = col_base + j * 32;
      const int m = wave_row0 + i * ROW_STRIDE + frag_row;
      const uint32_t voff =
          (frag_half == 0 && n < cp.n && m < cp.rows) ? (uint32_t)m * 4u + (uint32_t)block_scale_pos(n >> 5) : kOutOfRange;
      __builtin_amdgcn_raw_buffer_store_b8((unsigned char)e, srs, voff, uni((uint32_t)(n >> 7) * scale_rows * 4u), 0);
    });
#pragma unroll
    for (int band = 0; band < 32 / BAND; ++band) {
      if (BAND == 32 || (frag_row >> 4) == band) {
#pragma unroll
        for (int j = 0; j < OUT_BLOCKS; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<uint32_t *>(stage + (frag_row & (BAND - 1)) * PITCH + j * 32 + q * 8 + frag_half * 4) =
                packed[j][q];
      }
      wave_lds_sync();
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        const int r = ps * ROWS_PER_PASS + rd_row;
        const u32x4_t v = *reinterpret_cast<const u32x4_any_t *>(stage + r * PITCH + rd_chunk * 16);
        const int m = wave_row0 + i * ROW_STRIDE + band * BAND + r;
        const int n = col_base + rd_chunk * 16;
        const uint32_t voff = n < cp.n ? (uint32_t)m * cp.c_pitch + (uint32_t)n : kOutOfRange;
        __builtin_amdgcn_raw_buffer_store_b128(v, crs, voff, 0, 0);
      }
      wave_lds_sync();   // the next rows overwrite the staging rows
    }
    __builtin_amdgcn_sched_barrier(0);
  });
}

// ---------------------------------------------------------------------------
// Geometry of the 64-k pipelines (see gemm_persist64_body).
constexpr int kQBK = 64;
constexpr int kQWaves = 4;
constexpr int kQSlotBytes = (kPBM + kPBN) * 128;   // 64 KB
constexpr int kQRingBytes = 2 * kQSlotBytes;       // staging area follows
constexpr int kQMinSteps = 6;                      // loads run four steps ahead, within the next tile
static_assert(kSplitMinSteps >= kQMinSteps && kSplitMinSteps % 2 == 0, "a piece of a cut tile is a tile of its own");
static_assert(kQRingBytes == kPRingBytes, "both pipelines share the LDS budget");

__device__ __forceinline__ int qswizzle(int row) { return (row >> 1) & 7; }
// Byte offset of 16-byte chunk `chunk` (0..7) of `row` inside a slot half: any
// 16 consecutive rows put one chunk index into 16 different bank groups.
__device__ __forceinline__ int qring_off(int row, int chunk) {
  return row * 128 + ((chunk ^ qswizzle(row)) << 4);
}

// A step's loads in four quarters: the two halves of the activation rows, then
// the two halves of the weight rows.  quarter_first(q) .. quarter_first(q + 1)
// are quarter q's indices into the register stage.
constexpr int quarter_first(int copies_a, int copies_b, int q) {
  return q <= 2 ? q * (copies_a / 2) : q == 3 ? copies_a + (copies_b + 1) / 2 : copies_a + copies_b;
}
// Where side work goes in a block of `mf` products: item `idx` of `n` follows
// the product with this index (`phase` quarters of an interval in: fragment
// reads 0, LDS writes 1, global loads 3, so that the three kinds alternate).
// For 16 products: reads behind every even one, a write behind products 1, 5, 9,
// 13 and a load behind 3, 7, 11, 15: one instruction per gap.  The LDS takes 16 cycles per 16-byte-per-lane
// write against 4 per read, so the writes of the four waves are spread over the
// whole block rather than bunched.
constexpr int side_slot(int idx, int n, int mf, int phase) { return ((4 * idx + phase) * mf) / (4 * n); }
// The item that follows product `i` (at most one of each kind: n <= mf), or -1.
constexpr int side_item(int i, int n, int mf, int phase) {
  for (int idx = 0; idx < n; ++idx)
    if (side_slot(idx, n, mf, phase) == i) return idx;
  return -1;
}

// Instruction order of one block of MF MFMAs: RD fragment reads, 4 LDS writes
// and 4 global loads spread evenly behind the MFMAs (reads from the first MFMA
// on, writes and loads offset against each other).  The LDS takes 16 cycles per
// 16-byte-per-lane write against 4 per read, so the writes of the four waves are
// spread over the whole block rather than bunched.
template <int I, int MF, int RD>
__device__ __forceinline__ void qsched_block() {
  if constexpr (I < MF) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    constexpr int reads = (I + 1) * RD / MF - I * RD / MF;
    if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);
    constexpr int Q = MF / 4;  // one write and one load per quarter of the block
    if constexpr (I % Q == Q / 4) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    if constexpr (I % Q == Q / 4 + Q / 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    qsched_block<I + 1, MF, RD>();
  }
}


// Adds up the pieces of the tiles that the launch before it cut along k (see
// TileWalker): workgroup (xcd, j, part) re-derives XCD xcd's split turn from the
// same batch, and adds the partial-tile slots of its j-th tile, 16 rows per
// workgroup, in fp32 and in piece order into the tile's output rows.  `wgs` is
// the multiplying launch's workgroups per XCD, `bk` its k extent per step.
// (Many small workgroups, every piece of a chunk requested at once: the kernel
// moves a few tens of MB and is over in the time of a few memory round trips.)
constexpr int kSplitSumParts = 16, kSplitSumRows = kPBM / kSplitSumParts;
template <int BN_OUT>
__device__ __forceinline__ void persist_split_sum_body(const PersistBatch &batch, int wgs, int bk) {
  const int lane = threadIdx.x & 63;
  const int part = blockIdx.x % kSplitSumParts;
  const int j = (blockIdx.x / kSplitSumParts) % (wgs / 2);
  const int xcd = blockIdx.x / kSplitSumParts / (wgs / 2);
  TileWalker<BN_OUT> walk(batch, lane, xcd, 0, wgs);
  walk.plan_split(batch, bk);
  if (walk.split_cap == 0 || j >= walk.split_left) return;
  const SplitPiece sp = walk.split_tile(j);
  const Tile t = walk.decode(batch, walk.run_tile(walk.split_turn * wgs + j), bk);
  if (!t.valid || sp.ways == 0) return;
  constexpr int kChunks = BN_OUT / 8;  // 16-byte chunks per slot row
  const int ways = sp.ways;
  const unsigned char *slot0 = (const unsigned char *)walk.split_slot(batch, sp.first);
  for (int idx = threadIdx.x; idx < kSplitSumRows * kChunks; idx += blockDim.x) {
    const int r = part * kSplitSumRows + idx / kChunks, c = (idx % kChunks) * 8;
    if (r >= t.rows || t.n0 + c >= t.n) continue;
    h16x8_t v[kSplitMaxWays];
#pragma unroll
    for (int p = 0; p < kSplitMaxWays; ++p)
      if (p < ways)
        v[p] = *reinterpret_cast<const h16x8_t *>(slot0 + (size_t)p * (kPBM * BN_OUT * 2) +
                                                  ((size_t)r * BN_OUT + c) * 2);
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.f;
#pragma unroll
    for (int p = 0; p < kSplitMaxWays; ++p)
      if (p < ways) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sum[e] += (float)v[p][e];
      }
    h16x8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (h16_t)sum[e];
    *reinterpret_cast<h16x8_t *>(t.c + (size_t)r * t.c_pitch + (size_t)(t.n0 + c) * 2) = o;
  }
}
template <int BN_OUT>
__global__ __launch_bounds__(256) void persist_split_sum_kernel(PersistBatch batch, int wgs, int bk) {
  persist_split_sum_body<BN_OUT>(batch, wgs, bk);
}
// Whether a launch of `grid` workgroups over batch `b` (one problem) can leave a
// short last turn at all: a single group of known height whose tiles fill
// every workgroup's turns exactly never does (the shared expert at round sizes).
bool split_may_apply(const PersistBatch &b, int grid, int bn_out) {
  const PersistProblem &p = b.prob[0];
  if (p.n_experts != 1) return true;   // group heights live on the device
  const int64_t tiles = ((int64_t)p.max_rows + kPBM - 1) / kPBM * ((p.n + bn_out - 1) / bn_out);
  return tiles % grid != 0;
}
// The order of a launch's problems and which of TileWalker's two ways of
// sharing the tiles out over the XCDs it takes.  The group heights live on the
// device, so the pick is made from a model: evenly loaded groups, every
// workgroup's load in k steps (same arithmetic as the device) for the caller's
// order and for longest-k-first, under both splits.  The caller's order with
// the cost split stands unless another arrangement shortens the longest
// workgroup by 7 % or more: with equal makespans it measures fastest (it does
// not start all the long tiles, which move the most bytes per step, at the same
// time on every XCD).  A launch of one problem has nothing to choose.  The model
// costs a few microseconds of host time, so the last few shapes are remembered.
struct PersistPlan {
  bool longest_first;   // sort the problems by k, longest first
  int xcd_split;
  int64_t makespan;     // the model's longest workgroup under this arrangement, in 32-k steps
};
int64_t model_makespan(const PersistProblem *prob, int n_problems, int bn_out, int wgs, int split) {
  int64_t tiles[kMaxPersistProblems], steps[kMaxPersistProblems], base[kMaxPersistProblems], total_cost = 0, total = 0;
  for (int p = 0; p < n_problems; ++p) {
    const PersistProblem &pr = prob[p];
    // Groups of a routed problem are ragged: every other one a little over, the
    // rest as much under the mean (1.5 standard deviations of a uniform routing) -
    // with the mean on a multiple of the tile height, as in a benchmark, half of
    // the groups then spill into one more m-tile, as they do on the device.
    const int64_t per = pr.max_rows / pr.n_experts;
    const int64_t swing = pr.n_experts > 1 ? std::min<int64_t>(kPBM / 2, (int64_t)(1.5 * std::sqrt((double)per))) : 0;
    int64_t m_tiles = 0;
    for (int e = 0; e < pr.n_experts; ++e)
      m_tiles += (std::max<int64_t>(0, per + ((e & 1) ? swing : -swing)) + kPBM - 1) / kPBM;
    tiles[p] = m_tiles * ((pr.n + bn_out - 1) / bn_out);
    steps[p] = pr.k / 32;
    base[p] = total;
    total += tiles[p];
    total_cost += tiles[p] * steps[p];
  }
  auto boundary = [&](int x) -> int64_t {   // (split 0) first tile of XCD x's stretch
    if (x >= kNumXcd) return total;
    const int64_t target = total_cost * x / kNumXcd;
    int64_t cbase = 0;
    for (int p = 0; p < n_problems; ++p) {
      const int64_t c = tiles[p] * steps[p];
      if (c > 0 && target >= cbase && target < cbase + c) return base[p] + (target - cbase + steps[p] / 2) / steps[p];
      cbase += c;
    }
    return total;
  };
  int64_t makespan = 0;
  std::vector<int64_t> load(wgs);
  for (int x = 0; x < kNumXcd; ++x) {
    std::fill(load.begin(), load.end(), 0);
    int64_t i = 0;   // position in the XCD's run
    for (int p = 0; p < n_problems; ++p) {
      int64_t lo, hi;
      if (split == 0) {
        lo = std::max(boundary(x), base[p]);
        hi = std::min(boundary(x + 1), base[p] + tiles[p]);
      } else {
        lo = base[p] + tiles[p] * x / kNumXcd;
        hi = base[p] + tiles[p] * (x + 1) / kNumXcd;
      }
      for (int64_t t = lo; t < hi; ++t, ++i) {
        const int turn = (int)(i / wgs), w = (int)(i % wgs);
        load[(turn & 1) ? wgs - 1 - w : w] += steps[p];
      }
    }
    makespan = std::max(makespan, *std::max_element(load.begin(), load.end()));
  }
  return makespan;
}
// The most turns any workgroup walks when every problem has its tallest
// possible groups (the row bound plus a ragged tile per expert), under one way
// of sharing the tiles out over the XCDs: the device's arithmetic, counted in
// tiles instead of steps.
int64_t worst_case_turns(const PersistProblem *prob, int n_problems, int bn_out_fc1, bool fc2, int wgs, int split) {
  int64_t tiles[kMaxPersistProblems], steps[kMaxPersistProblems], base[kMaxPersistProblems], total_cost = 0, total = 0;
  for (int p = 0; p < n_problems; ++p) {
    const PersistProblem &pr = prob[p];
    const int bn_out = !fc2 ? bn_out_fc1 : (pr.n % 192 == 0 && pr.n % 256 != 0 ? 192 : kPBN);
    const int64_t m_tiles = ((int64_t)pr.max_rows + kPBM - 1) / kPBM + pr.n_experts;
    tiles[p] = m_tiles * ((pr.n + bn_out - 1) / bn_out);
    steps[p] = pr.k / 32;
    base[p] = total;
    total += tiles[p];
    total_cost += tiles[p] * steps[p];
  }
  auto boundary = [&](int x) -> int64_t {
    if (x >= kNumXcd) return total;
    const int64_t target = total_cost * x / kNumXcd;
    int64_t cbase = 0;
    for (int p = 0; p < n_problems; ++p) {
      const int64_t c = tiles[p] * steps[p];
      if (c > 0 && target >= cbase && target < cbase + c) return base[p] + (target - cbase + steps[p] / 2) / steps[p];
      cbase += c;
    }
    return total;
  };
  int64_t worst = 0;
  for (int x = 0; x < kNumXcd; ++x) {
    int64_t run = 0;
    for (int p = 0; p < n_problems; ++p) {
      int64_t lo, hi;
      if (split == 0) {
        lo = std::max(boundary(x), base[p]);
        hi = std::min(boundary(x + 1), base[p] + tiles[p]);
      } else {
        lo = base[p] + tiles[p] * x / kNumXcd;
        hi = base[p] + tiles[p] * (x + 1) / kNumXcd;
      }
      run += std::max<int64_t>(0, hi - lo);
    }
    worst = std::max(worst, (run + wgs - 1) / wgs);
  }
  return worst;
}
PersistPlan persist_plan(const PersistBatch &b, int bn_out, int grid, bool fc2) {
  struct Shape {
    int n_problems, bn_out, grid, rows[kMaxPersistProblems], experts[kMaxPersistProblems], n[kMaxPersistProblems],
        k[kMaxPersistProblems];
    PersistPlan plan;
  };
  Shape key{};
  key.n_problems = b.n_problems;
  key.bn_out = fc2 ? -bn_out : bn_out;   // (the stage is part of the shape)
  key.grid = grid;
  for (int p = 0; p < b.n_problems; ++p) {
    key.rows[p] = b.prob[p].max_rows;
    key.experts[p] = b.prob[p].n_experts;
    key.n[p] = b.prob[p].n;
    key.k[p] = b.prob[p].k;
  }
  constexpr int kRemembered = 16;
  static thread_local Shape seen[kRemembered];
  static thread_local int n_seen = 0, next = 0;
  auto same = [](const Shape &a, const Shape &c) {
    if (a.n_problems != c.n_problems || a.bn_out != c.bn_out || a.grid != c.grid) return false;
    for (int p = 0; p < a.n_problems; ++p)
      if (a.rows[p] != c.rows[p] || a.experts[p] != c.experts[p] || a.n[p] != c.n[p] || a.k[p] != c.k[p]) return false;
    return true;
  };
  for (int i = 0; i < n_seen; ++i)
    if (same(seen[i], key)) return seen[i].plan;
  PersistProblem sorted[kMaxPersistProblems];
  std::copy(b.prob, b.prob + b.n_problems, sorted);
  std::stable_sort(sorted, sorted + b.n_problems,
                   [](const PersistProblem &x, const PersistProblem &y) { return x.k > y.k; });
  const int wgs = grid / kNumXcd;
  if (b.n_problems < 2) {
    key.plan = PersistPlan{false, 1, model_makespan(b.prob, b.n_problems, bn_out, wgs, 1)};
    seen[next] = key;
    next = (next + 1) % kRemembered;
    if (n_seen < kRemembered) ++n_seen;
    return key.plan;
  }
  // In order of preference.  The model assumes evenly loaded groups, and real ones
  // are ragged (at a multiple of 256 rows per group half of them spill into one
  // more m-tile), so what it cannot tell apart is decided by measurement.  fc2 with
  // the longer problem first and an eighth of every problem per XCD, against
  // contiguous eighths of the cost, on the layer call at DiT-XL width: 4096
  // tokens 386 -> 362 us, 3072 -1.5 %, 1024 / 8192 / 12288 / 16384 and the
  // Zipf-loaded 16384 -0.2 ... -0.4 %, 1536 / 2048 the same, 6144 +0.7 %; the
  // config-literal block -0.5 % at 8192 (the same split *without* the order is 6 %
  // behind there).  fc1 keeps contiguous eighths of the cost (the other split:
  // +0.3 % at 8192 and at the Zipf-loaded 16384, -0.3 ... -1.1 % between 2048 and
  // 6144 tokens).
  const PersistPlan fc1_plans[4] = {{false, 0, 0}, {true, 0, 0}, {false, 1, 0}, {true, 1, 0}};
  const PersistPlan fc2_plans[4] = {{true, 1, 0}, {false, 1, 0}, {true, 0, 0}, {false, 0, 0}};
  const PersistPlan *plans = fc2 ? fc2_plans : fc1_plans;
  PersistPlan pick = plans[0];
  int64_t best = model_makespan(plans[0].longest_first ? sorted : b.prob, b.n_problems, bn_out, wgs,
                                plans[0].xcd_split);
  for (int i = 1; i < 4; ++i) {
    const int64_t m = model_makespan(plans[i].longest_first ? sorted : b.prob, b.n_problems, bn_out, wgs,
                                     plans[i].xcd_split);
    if (m * 100 < best * 93) {
      best = m;
      pick = plans[i];
    }
  }
  pick.makespan = best;
  key.plan = pick;
  seen[next] = key;
  next = (next + 1) % kRemembered;
  if (n_seen < kRemembered) ++n_seen;
  return pick;
}
// Launches the sum for a multiplying launch of `grid` workgroups.
template <int BN_OUT>
void launch_split_sum(const PersistBatch &launch, int grid, int bk, hipStream_t s) {
  const int wgs = grid / kNumXcd;
  hipLaunchKernelGGL(persist_split_sum_kernel<BN_OUT>, dim3(kNumXcd * (wgs / 2) * kSplitSumParts), dim3(256), 0,
                     s, launch, wgs, bk);
}


// ---------------------------------------------------------------------------
// What the kernels whose k-loop is generated assembly share (gen_persist64_asm.py
// writes persist64_asm.inc into the build directory).
#define DICE_MFMA8 "v_mfma_f32_32x32x64_f8f6f4"
#define DICE_MFMA8_SCALED "v_mfma_scale_f32_32x32x64_f8f6f4"
// One global memory -> LDS instruction (16 bytes per lane, no register in
// between) as text.  A load the compiler knows of would have it wait for "its
// only load" with vmcnt(0) before the next LDS access of its own - which drains
// the 32 operand loads the assembly keeps in flight, once per tile.  M0 holds
// the LDS address for the instruction and is put back.  The data has landed
// once the wave has waited for a load issued later (vector loads complete in
// order).
__device__ __forceinline__ void lds_dma_x4_text(u32x4_t rs, uint32_t dst_lds, uint32_t voff) {
  const uint32_t dst = uni(dst_lds);
  uint32_t keep_m0;
  asm volatile("s_mov_b32 %[keep], m0\n\t"
               "s_mov_b32 m0, %[dst]\n\t"
               "s_nop 0\n\t"
               "buffer_load_dwordx4 %[voff], %[rs], 0 offen lds\n\t"
               "s_mov_b32 m0, %[keep]"
               : [keep] "=&s"(keep_m0)
               : [dst] "s"(dst), [voff] "v"(voff), [rs] "s"(rs)
               : "memory");
}
struct P64Addr {
  uint32_t wr[2];       // LDS address of this lane's chunk in slot 0 / 1 (writes)
  uint32_t ra[2][4];    // LDS address of this lane's activation fragment of 16-k block kk in slot 0 / 1
  uint32_t rb[2][4];    // ... of its weight fragment
  uint32_t va[8];       // byte offsets of this lane's eight activation rows in the tile being loaded
  uint32_t vb;          // ... of its first weight row (the others: scalar offsets, P64_PARAMS)
};
#define P64_PARAMS                                                                                        \
  f32x32_t &f0, f32x32_t &f1, const P64Addr &ad, u32x4_t dA, u32x4_t dB0, u32x4_t dB1, uint32_t koff,       \
      const uint32_t (&sb)[8]
#define P64_ARGS f0, f1, ad, dA, dB0, dB1, koff, sb
#define P64_CONSTRAINTS                                                                                         \
  : "+{v[0:31]}"(f0), "+{v[32:63]}"(f1)                                                                         \
  : [wr0] "v"(ad.wr[0]), [wr1] "v"(ad.wr[1]), [ra00] "v"(ad.ra[0][0]), [ra01] "v"(ad.ra[0][1]),                 \
    [ra02] "v"(ad.ra[0][2]), [ra03] "v"(ad.ra[0][3]), [ra10] "v"(ad.ra[1][0]), [ra11] "v"(ad.ra[1][1]),         \
    [ra12] "v"(ad.ra[1][2]), [ra13] "v"(ad.ra[1][3]), [rb00] "v"(ad.rb[0][0]), [rb01] "v"(ad.rb[0][1]),         \
    [rb02] "v"(ad.rb[0][2]), [rb03] "v"(ad.rb[0][3]), [rb10] "v"(ad.rb[1][0]), [rb11] "v"(ad.rb[1][1]),         \
    [rb12] "v"(ad.rb[1][2]), [rb13] "v"(ad.rb[1][3]), [va0] "v"(ad.va[0]), [va1] "v"(ad.va[1]),                 \
    [va2] "v"(ad.va[2]), [va3] "v"(ad.va[3]), [va4] "v"(ad.va[4]), [va5] "v"(ad.va[5]), [va6] "v"(ad.va[6]),    \
    [va7] "v"(ad.va[7]), [vb] "v"(ad.vb), [dA] "s"(dA), [dB0] "s"(dB0), [dB1] "s"(dB1), [koff] "s"(koff),       \
    [sb0] "s"(sb[0]), [sb1] "s"(sb[1]), [sb2] "s"(sb[2]), [sb3] "s"(sb[3]), [sb4] "s"(sb[4]), [sb5] "s"(sb[5]), \
    [sb6] "s"(sb[6]), [sb7] "s"(sb[7])                                                                          \
  : "memory"
// The kernel for block-scaled fp8 activations also passes: the byte offset of this lane's row of block scales in
// the tile being loaded (vs), the LDS address its scales go to (wrs; slot 1 lies 1 KB on) and the one it reads its
// rows' scales from (rs), the descriptor of the tile's scales (dS) and the step's offset in a row of them (kso).
// The text also names v117..v127 (the scales' register stage, the scales of the step's row blocks, the weights'
// scale), which the compiler must not use: it allocates from v0 upwards and parks scalar registers in the lanes of
// the first vector registers past those - the build-time check of the device assembly (check_acc_regs.py) fails an
// instantiation in which either reaches v117.  (A value pinned to these registers and passed through every
// statement does not keep them free: the compiler moves it out and back around the epilogue.)
struct P64ScaleAddr {
  uint32_t vs, wrs, rs;
};
#define P64S_PARAMS P64_PARAMS, const P64ScaleAddr &sa, u32x4_t dS, uint32_t kso
#define P64S_ARGS P64_ARGS, sa, dS, kso
#define P64S_CONSTRAINTS                                                                                        \
  : "+{v[0:31]}"(f0), "+{v[32:63]}"(f1)                                                                         \
  : [wr0] "v"(ad.wr[0]), [wr1] "v"(ad.wr[1]), [ra00] "v"(ad.ra[0][0]), [ra01] "v"(ad.ra[0][1]),                 \
    [ra02] "v"(ad.ra[0][2]), [ra03] "v"(ad.ra[0][3]), [ra10] "v"(ad.ra[1][0]), [ra11] "v"(ad.ra[1][1]),         \
    [ra12] "v"(ad.ra[1][2]), [ra13] "v"(ad.ra[1][3]), [rb00] "v"(ad.rb[0][0]), [rb01] "v"(ad.rb[0][1]),         \
    [rb02] "v"(ad.rb[0][2]), [rb03] "v"(ad.rb[0][3]), [rb10] "v"(ad.rb[1][0]), [rb11] "v"(ad.rb[1][1]),         \
    [rb12] "v"(ad.rb[1][2]), [rb13] "v"(ad.rb[1][3]), [va0] "v"(ad.va[0]), [va1] "v"(ad.va[1]),                 \
    [va2] "v"(ad.va[2]), [va3] "v"(ad.va[3]), [va4] "v"(ad.va[4]), [va5] "v"(ad.va[5]), [va6] "v"(ad.va[6]),    \
    [va7] "v"(ad.va[7]), [vb] "v"(ad.vb), [dA] "s"(dA), [dB0] "s"(dB0), [dB1] "s"(dB1), [koff] "s"(koff),       \
    [sb0] "s"(sb[0]), [sb1] "s"(sb[1]), [sb2] "s"(sb[2]), [sb3] "s"(sb[3]), [sb4] "s"(sb[4]), [sb5] "s"(sb[5]), \
    [sb6] "s"(sb[6]), [sb7] "s"(sb[7]), [vs] "v"(sa.vs), [wrs] "v"(sa.wrs), [rs] "v"(sa.rs), [dS] "s"(dS),      \
    [kso] "s"(kso)                                                                                              \
  : "memory"
typedef float f32x32_t __attribute__((ext_vector_type(32)));
#include "persist64_asm.inc"
}  // namespace
}  // namespace dice
