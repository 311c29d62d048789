// Persistent bf16 grouped GEMMs for the expert MLPs (routed experts and the
// shared expert in ONE launch per GEMM stage).
//
// One workgroup per CU stays resident and walks a list of 256-row output tiles;
// the k loop of consecutive tiles forms one continuous software pipeline, so
// there is no per-tile prologue and no workgroup re-launch between tiles.
// Operands are addressed through buffer descriptors: the range check zero-fills
// rows past a group's end and past the last output column, so ragged groups
// need no special code.  The epilogue applies SwiGLU / GELU / bias, transposes
// through a small LDS staging area and writes whole row segments with buffer
// stores (rows past the group's end are dropped by the range check).
//
// Two pipelines share the tile order and the epilogue; the launcher picks one
// per launch (persist_variant):
//
//   * 64 k per step, four waves (one per SIMD, 128x128 or 128x96 of the tile
//     each, accumulators in the accumulation registers), operands staged
//     through registers four steps ahead and written to one of two 64 KB LDS
//     slots; optional row table for the activations (the dispatch permutation).
//     The product path: see the comment above gemm_persist64_body.
//   * 32 k per step, eight waves (two per SIMD, 128x64 each), global -> LDS
//     copies (buffer_load_dwordx4 ... lds) three steps ahead in a ring of four
//     32 KB slots, the two wave groups alternating memory and MFMA phases.
//     Takes shorter k and any number of tiles per workgroup.
//
// Tiles are ordered problem-major (longest k first), expert-major, then n-tile
// with the m-tile fastest; each XCD takes one contiguous, equally expensive run
// of that order, so the 32 CUs that share an L2 work on the same expert's
// weights at the same time.
//
// Weights are [experts, rows, k] bf16 as in the reference's nn.Linear layout
// (models.py:245-247), or fp8 (e4m3) bytes of the same shape with one fp32
// scale per output channel (64-k pipeline only: widened to bf16 on the way into
// LDS, scale applied to the fp32 sums); activations are grouped rows
// (contiguous, or rows of the token matrix named by a row table).
//
// This file is compiled twice: as it stands for bf16 activations and weights,
// and with DICE_PERSIST_F16 (through grouped_gemm_persist_f16.hip) for fp16,
// which the reference serves its XL and G models in (sample_ddp.py:77-81,97-98).
// Only the element type of the operands, the MFMA instruction and the fp8
// widening differ; shared host-side helpers live in the bf16 compilation.
#include <type_traits>

#include <algorithm>
#include <vector>

#include "gemm_common.h"

#ifndef DICE_PERSIST_F16
#define DICE_PERSIST_F16 0
#endif
// A third compilation (grouped_gemm_persist_f8.hip, DICE_PERSIST_F8) holds the
// kernel whose activations are fp8 as well; it shares the tile order, the tile
// table and the epilogue with the others and writes bf16.
#ifndef DICE_MFMA_ROWS_OUTERMOST
#define DICE_MFMA_ROWS_OUTERMOST 0
#endif
#ifndef DICE_PERSIST_F8
#define DICE_PERSIST_F8 0
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
    uint64_t pa = 0, pw = 0, pc = 0, pbias = 0, prows = 0, pascale = 0;
    int lda = 0, ldc = 0, w_rows = 0, up_offset = 0, n = 0, k = 0, a_div = 1, a_src_rows = 0;
    for (int q = 0; q < batch.n_problems; ++q) {
      const PersistProblem &pr = batch.prob[q];
      if (pi == q) {
        pa = (uint64_t)pr.a; pw = (uint64_t)pr.w; pc = (uint64_t)pr.c; pbias = (uint64_t)pr.bias;
        lda = pr.lda; ldc = pr.ldc; w_rows = pr.w_rows; up_offset = pr.up_offset; n = pr.n; k = pr.k;
        prows = (uint64_t)pr.a_rows; a_div = pr.a_div; a_src_rows = pr.a_src_rows;
        pascale = (uint64_t)pr.a_scale;
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
    uint32_t c_pitch = (uint32_t)ldc * 2, c_extent = (uint32_t)rows * c_pitch;
    const uint64_t wexp = pw + (uint64_t)expert * w_rows * b_pitch;
    // Gathered rows are addressed from the start of the source matrix.
    uint64_t ptrs[5] = {prows ? pa : pa + (uint64_t)(row0 + m_tile * kPBM) * a_pitch, wexp + (uint64_t)n0 * b_pitch,
                        wexp + (uint64_t)(up_offset + n0) * b_pitch,
                        pc + (uint64_t)(row0 + m_tile * kPBM) * c_pitch,
                        pbias ? pbias + ((uint64_t)expert * n) * sizeof(float) : 0};
    int steps = k / bk;
    if (cut && sp.ways != 0) {
      // This position's piece of the tile: its run of steps (the k offset moves
      // the operands' base addresses; range checks look at row offsets only), and
      // the position's partial-tile slot as the output, addressed so that column
      // n0 is the slot's first.  The bias rides on the first piece.
      const SplitRange run = split_range(steps, sp.piece, sp.ways);
      steps = run.count;
      const uint32_t k0 = (uint32_t)(run.begin * bk);
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
    const uint64_t tile_rows = a8 ? pascale + (uint64_t)(row0 + m_tile * kPBM) * sizeof(float)
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

// HAS_BIAS is a compile-time switch so that the bias-free (reference SwiGLU)
// instantiations carry no bias loads: a vector load in the epilogue makes the
// compiler wait for every outstanding copy and store.
template <int MODE, bool HAS_BIAS, int kPWaves>
__device__ __forceinline__ void gemm_persist_body(const PersistBatch &batch) {
  static_assert(kPWaves == 4 || kPWaves == 8, "four or eight waves");
  constexpr int kPWavesN = kPWaves / kPWavesM;
  constexpr int kPCopiesA = kPBM / 16 / kPWaves;  // 1 KB copies per wave per step
  constexpr int kPCopiesB = kPBN / 16 / kPWaves;
  constexpr int kPCopies = kPCopiesA + kPCopiesB;
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int BN_OUT = SWIGLU ? kPBN / 2 : kPBN;
  constexpr int WTM = kPBM / kPWavesM, WTN = kPBN / kPWavesN;  // 128 x 64 (eight waves) or 128 x 128
  constexpr int TM = WTM / 32, TN = WTN / 32;
  using Epi = EpiGeom<MODE, kPWaves, TM, TN>;
  constexpr int WAIT_STEADY = (kPAhead - 1) * kPCopies;  // copies of the two newest steps

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / kPWavesN, wn = wave % kPWavesN;

  TileWalker<BN_OUT> walk(batch, lane);
  auto decode = [&](int id) { return walk.decode(batch, id, kPBK); };

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

  // Per-lane byte offsets of this wave's copies inside the tile being copied.
  // They depend on the tile's row pitches only, so they are worked out once per
  // tile; the asm statement keeps the compiler from re-deriving them (integer
  // multiplies) inside every k step, where vector ALU work competes with the
  // other group's MFMAs for the SIMD's issue slots.
  uint32_t ld_voff[kPCopies];
  auto set_copy_offsets = [&](const Tile &t) {
#pragma unroll
    for (int l = 0; l < kPCopies; ++l) {
      ld_voff[l] = (uint32_t)cp_row[l] * (l < kPCopiesA ? t.a_pitch : t.b_pitch) + cp_chunk[l];
      asm volatile("" : "+v"(ld_voff[l]));
    }
  };

  // Issues copy `l` of the step `kt` of tile `t` into ring slot `slot`.
  auto issue_copy = [&](const Tile &t, int kt, int slot, int l) {
    unsigned char *dst = lds_raw + slot * kPSlotBytes;
    if (l < kPCopiesA) {
      const __amdgpu_buffer_rsrc_t rs =
          __builtin_amdgcn_make_buffer_rsrc((void *)t.a, 0, t.a_bytes, kRsrcFlags);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs, (__attribute__((address_space(3))) void *)(dst + (wave + kPWaves * l) * 1024), 16,
          ld_voff[l], kt * 64, 0, 0);
    } else {
      const int i = l - kPCopiesA;
      const bool up_half = SWIGLU && kPWaves * i * 16 >= kPBN / 2;  // wave * 16 < 128 never crosses the halves
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)(up_half ? t.b1 : t.b0), 0, t.b_bytes, kRsrcFlags);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs,
          (__attribute__((address_space(3))) void *)(dst + kPBM * 64 + (wave + kPWaves * i) * 1024), 16,
          ld_voff[l], kt * 64, 0, 0);
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
  h16x8_t wf[2][TN], af[2][TM];
  // Lane part of the fragment addresses for the two 16-k halves of a step; the
  // 32-row block and the ring slot only add compile-time constants (the swizzle
  // uses row bits 1..3, which block offsets do not touch), so the reads of a
  // step need no address arithmetic.
  uint32_t rd_a[2], rd_b[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    rd_a[kk] = pring_off(wm * WTM + frag_row, kk * 2 + frag_half);
    rd_b[kk] = kPBM * 64 + pring_off(w_block_row(0) + frag_row, kk * 2 + frag_half);
    asm volatile("" : "+v"(rd_a[kk]), "+v"(rd_b[kk]));
  }
  auto read_frags = [&](auto slot_c, int kk, int buf) {
    constexpr int SLOT = decltype(slot_c)::value;
    const unsigned char *base = lds_raw + SLOT * kPSlotBytes;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      constexpr int HALF = TN / 2;
      const int joff = (SWIGLU && j >= HALF) ? (kPBN / 2 + (j - HALF) * 32) * 64 : j * 32 * 64;
      wf[buf][j] = *reinterpret_cast<const h16x8_t *>(base + rd_b[kk] + joff);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[buf][i] = *reinterpret_cast<const h16x8_t *>(base + rd_a[kk] + i * 32 * 64);
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
  int next_round = 0;                            // this workgroup's next turn
  Tile ld = decode(walk.tile_id(next_round++));  // tile being copied
  if (!ld.valid) return;                         // nothing to do for this workgroup
  Tile cp = ld;                                  // tile being multiplied
  int ld_kt = 0;

  // Advances the copy side by one step (wave-uniform control flow only).
  auto advance_copy = [&]() {
    if (++ld_kt == ld.steps) {
      ld = decode(walk.tile_id(next_round++));
      set_copy_offsets(ld);
      ld_kt = 0;
    }
  };
  set_copy_offsets(ld);

#pragma unroll
  for (int s = 0; s < kPAhead; ++s) {
#pragma unroll
    for (int l = 0; l < kPCopies; ++l) issue_copy(ld, ld_kt, s, l);
    advance_copy();
  }
  zero_acc();
  int since_epilogue = 2;
  const int stage_base = kPRingBytes + wave * Epi::WAVE_BYTES;
  const int wave_col0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;

  auto epilogue = [&]() {
    // Loads and stores may retire out of order with respect to each other, so
    // after the stores of the epilogue the counter no longer tells how many
    // copies are pending.  Drain the copies first (the next tile's first three
    // steps; the youngest were issued one step ago) and skip the waits of the
    // next tile's first two steps, whose operands are then known to have landed.
    pwait_vmcnt<0>();
    tile_epilogue<MODE, HAS_BIAS, kPWaves, TM, TN>(cp, acc, lds_raw + stage_base, wm * WTM, wave_col0, lane);
  };

  if constexpr (kPWaves == 8) {
    // Two groups of four waves (one wave of each group per SIMD) alternate between
    // a memory phase (fragment reads of one k step + this wave's share of the
    // copies three steps ahead) and a compute phase (the step's 16 MFMAs), one
    // phase apart: while one group multiplies the other one loads, so the matrix
    // pipe only idles for the barrier hand-over between phases.
    const int group = wm;
    // Waits until at most the copies of the two newest steps are still in flight.
    auto copies_landed = [&]() {
      if (since_epilogue >= 2) pwait_vmcnt<WAIT_STEADY>();
      ++since_epilogue;
    };
    pwait_vmcnt<WAIT_STEADY>();
    phase_barrier();                      // everyone's copies of step 0 have landed
    while (true) {  // one tile per iteration
      if (group == 1) phase_barrier();
      // The ring position of a step is a compile-time constant: every tile has a
      // multiple of kPStages steps, so a tile always starts in slot 0.
      auto step = [&](auto slot_c) {
        constexpr int cslot = decltype(slot_c)::value;
        // ---- memory phase ----
        constexpr int lslot = (cslot + kPAhead) & (kPStages - 1);  // slot of the step before this one
        read_frags(slot_c, 0, 0);
        read_frags(slot_c, 1, 1);
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
          for (int j = 0; j < TN; ++j)
  #pragma unroll
            for (int i = 0; i < TM; ++i) {
              const int ii = (j & 1) ? TM - 1 - i : i;   // (one operand changes per product, see mfma_block below)
              acc[ii][j] = mfma_32x32x16(wf[kk][j], af[kk][ii], acc[ii][j]);
            }
        __builtin_amdgcn_s_setprio(DICE_PRIO_MEMORY);
        if (group == 0) copies_landed();
        phase_barrier();
      };
      for (int s = 0; s < cp.steps; s += kPStages) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{});
      }
      if (group == 0) phase_barrier();  // let the other group finish the tile's last step

      epilogue();
      // Every tile has more than AHEAD steps, so the copy side is exactly one
      // tile ahead here: the tile it is working on is the one to multiply next.
      cp = ld;
      if (!cp.valid) break;
      since_epilogue = 0;
      zero_acc();
    }
  }
  pwait_vmcnt<0>();
}

// ---------------------------------------------------------------------------
// 64-k pipeline, four waves, operands staged through registers.
//
// Two things bound the 32-k pipeline above.  The L2 serves whole 128-byte lines:
// a 32-k step asks for half a line per row and reaches about half the copy rate
// of a 64-k step.  And a copy takes 1 to 2 us from request to data while a 64-k
// step multiplies for 1.3 us, so more than one step has to be in flight - but a
// 64-k step of a 256x256 tile is 64 KB and only two fit the LDS next to the
// epilogue's staging area.
//
// Here a step is 64 k (rows of 128 bytes, two 64 KB LDS slots) and the data in
// flight lives in registers: four waves, one per SIMD with the whole register
// file, own 128x128 of the tile each (accumulators in the accumulation
// registers); every wave loads its share of a step (16 x 16 bytes per lane)
// into one of two register stages FOUR steps ahead and writes it to the LDS
// slot two steps later, as soon as that slot has been read for the last time.
// Loads and LDS writes are cut into quarters, one per 16-MFMA block, so every
// block carries the same small side load: 8 fragment reads, 4 LDS writes and 4
// global loads threaded between its MFMAs.  The one barrier of a step sits
// before its last block: by then every wave has read the last fragments of
// the step's slot (so the slot may be rewritten) and has finished writing the
// other slot (so the next step's first fragments may be read).
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

// BN is the number of weight rows of a tile: 256, or 192 for output widths that
// 192 divides and 256 does not (1152 = 6 x 192: no padded columns to multiply).
// GATHER: activation rows may be addressed through a row table (the dispatch
// permutation), which saves the separate gathered copy of the activations.
// W8: the weights are fp8 (e4m3) bytes with one fp32 scale per output channel
// (single-problem launches only).  A 16-byte load then holds 16 elements of a
// row; they are widened to bf16 (exactly) on their way into LDS, so the slots,
// the fragment reads and the MFMAs are those of the bf16 kernel; the scale
// multiplies the fp32 sums in the epilogue.
// REFILL: a workgroup may have more turns than the LDS tile table holds (very
// large batches); the table is then rewritten every kTableTurns tiles.  A
// separate instantiation, because even unused the rewrite costs the tile switch
// registers (1-2 % of fc1 at 8192 tokens).
template <int MODE, bool HAS_BIAS, int BN, bool GATHER, bool W8 = false, bool REFILL = false>
__device__ __forceinline__ void gemm_persist64_body(const PersistBatch &batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  static_assert(BN == 256 || (BN == 192 && !SWIGLU), "tile widths");
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTM = 128, WTN = BN / 2, TM = 4, TN = WTN / 32;
  // 16-byte-per-lane loads: 8 rows of 128 bytes each (fp8 weights: 16 rows of 64 bytes)
  constexpr int kRowsPerCopyB = W8 ? 16 : 8;
  constexpr int kCopiesA = kPBM / 8 / kQWaves, kCopiesB = BN / kRowsPerCopyB / kQWaves;
  constexpr int kQCopies = kCopiesA + kCopiesB;
  static_assert(kCopiesA % 2 == 0, "a step is four quarters: two of A, two of B");
  // (three scale buffers: the epilogue of a tile reads its scales while the first
  // wave, a little ahead, may already copy in those of the tile after the next)
  constexpr int kScaleBufFloats = 256, kScaleBytes = W8 ? 3 * kScaleBufFloats * 4 : 0;
  constexpr int kSlotUsed = (kPBM + BN) * 128;
  constexpr bool kScaleInSlot = W8 && kSlotUsed + kScaleBytes <= kQSlotBytes;  // 192-wide tiles leave a slot's tail free
  constexpr int kEpiReserve = kTableTurns * kTileWords * 4 + (W8 && !kScaleInSlot ? kScaleBytes + kPBM * 4 : 0);
  using Epi = EpiGeom<MODE, kQWaves, TM, TN, W8 ? kEpiReserve : 0>;
  const template_int<0> c0; const template_int<1> c1; const template_int<2> c2; const template_int<3> c3;

  // Three separate LDS objects, so that the compiler knows that fragment reads of
  // one slot and writes to the other never touch the same bytes and may pass
  // each other when the instructions of a block are interleaved.
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot0[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot1[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_stage[kPStageArea];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // This workgroup's tiles, described once and parked in LDS behind the epilogue's
  // staging rows; lane f of a table read gets word f of the description.
  constexpr int kTableBytes = kTableTurns * kTileWords * 4, kRowSlotBytes = kPBM * 4;
  // A 256-wide biased tile starts its accumulators from the bias (64 values per
  // lane that the epilogue then need not hold: it would spill); its epilogue
  // stages 16-row bands, which leaves room for two bias buffers of one tile's
  // columns each beside the tile table.  A 192-wide tile (48 values) adds the
  // bias in the epilogue.
  constexpr bool kBiasInAcc = HAS_BIAS && BN == 256;
  constexpr int kBiasBufFloats = 256, kBiasBytes = 2 * kBiasBufFloats * 4;
  static_assert(kQWaves * Epi::WAVE_BYTES + kTableBytes + (GATHER ? kRowSlotBytes : 0) +
                        (kBiasInAcc ? kRowSlotBytes + kBiasBytes : 0) +
                        (W8 && !kScaleInSlot ? kRowSlotBytes + kBiasBytes + kScaleBytes : 0) <= kPStageArea,
                "no room for the tile table");
  uint32_t *const tile_table = reinterpret_cast<uint32_t *>(lds_stage + kPStageArea - kTableBytes);
  // (gathered activations) the slots of the 256 rows of the tile the load side opens next
  int32_t *const lds_row_slots = reinterpret_cast<int32_t *>(lds_stage + kPStageArea - kTableBytes - kRowSlotBytes);
  // The first wave copies a tile's bias in (one global->LDS instruction) a whole
  // tile before the accumulators of that tile are initialised with it.
  float *const lds_bias =
      reinterpret_cast<float *>(lds_stage + kPStageArea - kTableBytes - kRowSlotBytes - kBiasBytes);
  // (fp8 weights) the scales of a tile's columns, copied in like the bias
  float *const lds_scale = reinterpret_cast<float *>(
      kScaleInSlot ? lds_slot1 + kSlotUsed
                   : lds_stage + kPStageArea - kTableBytes - kRowSlotBytes - kBiasBytes - 3 * kScaleBufFloats * 4);
  if (wave == 0) {
    TileWalker<BN_OUT> walk(batch, lane);
    walk.build_table(batch, lane, kQBK, tile_table, W8);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();
  // The table holds kTableTurns turns; a workgroup with more has its first wave
  // describe the next kTableTurns when the last entry has been fetched: every
  // wave arrives at that tile switch, so two barriers fence the rewrite.
  auto fetch_tile = [&](int turn) {
    if constexpr (REFILL) {
      if (turn != 0 && (turn & (kTableTurns - 1)) == 0) {
        phase_barrier();
        if (wave == 0) {
          TileWalker<BN_OUT> walk(batch, lane);
          walk.build_table(batch, lane, kQBK, tile_table, W8, turn);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        phase_barrier();
      }
    }
    return PackedTile{tile_table[(turn & (kTableTurns - 1)) * kTileWords + (lane < kTileWords ? lane : 0)]};
  };

  // ---- global loads: one instruction fetches 8 rows x 128 bytes (8 lanes per
  // row, i.e. whole lines); load l of a wave covers rows (wave + 4 (l % 8)) * 8
  // .. + 8 of the activation tile (l < 8) or of the weight tile. ----
  const int cp_row0 = wave * 8 + (lane >> 3);
  const int cp_chunk = lane & 7;
  // LDS address of this lane's chunk in slot 0 (row bits 1..3, which the swizzle
  // reads, are the same for every l)
  uint32_t wr_off = qring_off(cp_row0, cp_chunk);
  asm volatile("" : "+v"(wr_off));
  // fp8 weights: 4 lanes per 64-byte row, 16 rows per load; a lane's 16 bytes
  // become chunks 2c and 2c + 1 of the bf16 row in LDS.
  const int cpb_row0 = W8 ? wave * 16 + (lane >> 2) : cp_row0;
  const int cpb_chunk = W8 ? (lane & 3) : cp_chunk;
  uint32_t wr_off_b8 = W8 ? qring_off(cpb_row0, 2 * cpb_chunk) : 0;
  uint32_t wr_off_b8_hi = W8 ? qring_off(cpb_row0, 2 * cpb_chunk + 1) : 0;
  if constexpr (W8) asm volatile("" : "+v"(wr_off_b8), "+v"(wr_off_b8_hi));
  const uint32_t w8_magic = W8 ? (uint32_t)(0xffffffffull / (uint32_t)(batch.prob[0].a_div > 0 ? batch.prob[0].a_div : 1) + 1) : 0;
  // Per-lane byte offsets inside the tile being loaded.  Without a row table
  // load i of the activations is row cp_row0 + 32 i: one offset plus a scalar
  // stride.  With one, each of a lane's kCopiesA rows has its own offset, worked
  // out at the tile switch from the tile's 256 row numbers, which the first wave
  // copied into LDS (one global->LDS instruction) a tile earlier.
  uint32_t ld_voff_a = 0, ld_voff_b = 0;
  uint32_t ld_voff_rows[GATHER ? kCopiesA : 1];
  auto copy_row_slots = [&](const PackedTile &pk) {
    if constexpr (GATHER) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 21) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 20);
      const int rows = __builtin_amdgcn_readlane(pk.words, 23);
      if (wave == 0 && ptr != 0) {
        // rows past the group's end read as slot 0 (a legal row; their products are never stored)
        const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void *)ptr, 0, (uint32_t)rows * 4, kRsrcFlags);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)lds_row_slots, 16,
                                                 lane * 16, 0, 0, 0);
      }
    }
  };
  auto copy_bias = [&](const PackedTile &pk, int buf) {
    if constexpr (kBiasInAcc) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 9) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 8);
      const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
      if (wave == 0 && ptr != 0) {
        // columns past the matrix read as 0 (their products are never stored)
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(ptr + (uint64_t)n0 * 4), 0, (uint32_t)(n - n0) * 4, kRsrcFlags);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (__attribute__((address_space(3))) void *)(lds_bias + buf * kBiasBufFloats), 16, lane * 16, 0, 0, 0);
      }
    }
  };
  auto copy_scale = [&](const PackedTile &pk, int buf) {
    if constexpr (W8) {
      const uint32_t row = (uint32_t)__builtin_amdgcn_readlane(pk.words, 22);
      const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
      if (wave == 0) {
        const float *base = batch.prob[0].w_scale + row;
        // SwiGLU: 128 gate scales, then the 128 up scales up_offset rows further on;
        // otherwise the tile's columns, those past the matrix reading as 0
        const uint32_t bytes = SWIGLU ? (uint32_t)(batch.prob[0].up_offset + 128) * 4 : (uint32_t)(n - n0) * 4;
        const uint32_t voff = SWIGLU && lane >= 32 ? (uint32_t)batch.prob[0].up_offset * 4 + (lane - 32) * 16 : lane * 16;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, bytes, kRsrcFlags);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (__attribute__((address_space(3))) void *)(lds_scale + buf * kScaleBufFloats), 16, voff, 0, 0, 0);
      }
    }
  };
  auto set_copy_offsets = [&](const Tile &t) {
    ld_voff_a = (uint32_t)cp_row0 * t.a_pitch + cp_chunk * 16;
    ld_voff_b = (uint32_t)cpb_row0 * t.b_pitch + cpb_chunk * 16;
    asm volatile("" : "+v"(ld_voff_a), "+v"(ld_voff_b));
    if constexpr (GATHER) {
#pragma unroll
      for (int i = 0; i < kCopiesA; ++i) {
        const int r = cp_row0 + 32 * i;
        uint32_t off = ld_voff_a + (uint32_t)(32 * i) * t.a_pitch;
        if (t.a_rows) {
          const uint32_t slot = (uint32_t)lds_row_slots[r];
          // (one slot per source row: 2^32 / 1 does not fit the multiplier, which then reads 0)
          const uint32_t magic = W8 ? w8_magic : t.a_magic;
          const uint32_t src_row = magic ? __umulhi(slot, magic) : slot;
          off = r < t.rows ? src_row * t.a_pitch + cp_chunk * 16 : kOutOfRange;
        }
        ld_voff_rows[i] = off;
        asm volatile("" : "+v"(ld_voff_rows[i]));
      }
    }
  };
  u32x4_t stage_regs[2][kQCopies];

  // ---- fragment reads: lane part per 16-k block; 32-row blocks and the slot
  // add compile-time constants ----
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int b_row0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;
  uint32_t rd_a[4], rd_b[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    rd_a[kk] = qring_off(wm * WTM + frag_row, kk * 2 + frag_half);
    rd_b[kk] = kPBM * 128 + qring_off(b_row0 + frag_row, kk * 2 + frag_half);
    asm volatile("" : "+v"(rd_a[kk]), "+v"(rd_b[kk]));
  }
  h16x8_t wf[2][TN], af[2][TM];
  // Fragment R of 16-k block KK of slot SLOT into buffer BUF, in the order in which
  // the block's products first need them (mfma_at): weight block 0, the row
  // blocks, then the other weight blocks.
  auto read_frag = [&](auto slot_c, auto kk_c, auto buf_c, auto r_c) {
    constexpr int SLOT = decltype(slot_c)::value, KK = decltype(kk_c)::value, BUF = decltype(buf_c)::value;
    constexpr int R = decltype(r_c)::value;
    const unsigned char *base = SLOT == 0 ? lds_slot0 : lds_slot1;
    if constexpr (R == 0 || R > TM) {
      constexpr int J = R == 0 ? 0 : R - TM, HALF = TN / 2;
      constexpr int jrow = (SWIGLU && J >= HALF) ? BN / 2 + (J - HALF) * 32 : J * 32;
      wf[BUF][J] = *reinterpret_cast<const h16x8_t *>(base + rd_b[KK] + jrow * 128);
    } else {
      af[BUF][R - 1] = *reinterpret_cast<const h16x8_t *>(base + rd_a[KK] + (R - 1) * 32 * 128);
    }
  };
  auto read_frags = [&](auto slot_c, auto kk_c, auto buf_c) {
    static_for<TM + TN>([&](auto r_c) { read_frag(slot_c, kk_c, buf_c, r_c); });
  };

  const int wave_col0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;
  // The sums live in the accumulation registers by name: block (i, j) is
  // a[16 (kAccBlock0 + i TN + j) ..], the TM x TN blocks at the top of the
  // register file (see mfma_fixed, fixed_acc_clear).
  constexpr int kAccBlock0 = 16 - TM * TN;
  // (256-wide biased tiles) the accumulators start from the bias of their columns:
  // every 32-row block of a column block gets the same 16 values per lane.
  auto init_acc = [&](const Tile &t, int buf, int sbuf) {
    if constexpr (kBiasInAcc) {
      if (uni((int)(t.bias != nullptr))) {
        const float *src = lds_bias + buf * kBiasBufFloats + wave_col0 + frag_half * 4;
        static_for<TN>([&](auto j_c) {
          constexpr int j = decltype(j_c)::value;
          static_for<4>([&](auto q_c) {
            constexpr int q = decltype(q_c)::value;
            f32x4_t v = *reinterpret_cast<const f32x4_t *>(src + j * 32 + q * 8);
            if constexpr (W8) {  // the epilogue multiplies the sums by the scale
              const f32x4_t sc = *reinterpret_cast<const f32x4_t *>(
                  lds_scale + sbuf * kScaleBufFloats + wave_col0 + frag_half * 4 + j * 32 + q * 8);
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] = v[r] / sc[r];
            }
            static_for<4>([&](auto r_c) {
              constexpr int r = decltype(r_c)::value;
              static_for<TM>([&](auto i_c) {
                fixed_acc_set<(kAccBlock0 + decltype(i_c)::value * TN + j) * 16 + q * 4 + r>(v[r]);
              });
            });
          });
        });
        fixed_acc_settle();
        return;
      }
    }
    fixed_acc_clear<TM * TN * 16>();
    fixed_acc_settle();
  };
  // Product I of a 16-k block: weight block by weight block with the row blocks
  // up and down in turn, so that from one product to the next only one operand
  // changes, the left one (the weights) every TM-th time.
  auto mfma_at = [&](auto buf_c, auto i_c) {
    constexpr int BUF = decltype(buf_c)::value, I = decltype(i_c)::value;
    constexpr int j = I / TM, i = (j & 1) ? TM - 1 - I % TM : I % TM;
    mfma_fixed<kAccBlock0 + i * TN + j>(wf[BUF][j], af[BUF][i]);
  };

  // ---- pipeline state ----
  // The load side runs four steps ahead of the MFMAs, so it crosses into the
  // next tile once while a tile is multiplied.  That tile's description (`nxt`)
  // is worked out between tiles, where registers are free, not inside the k loop.
  int next_turn = 0;                              // this workgroup's next turn
  PackedTile nxt = fetch_tile(next_turn++);
  Tile ld = unpack_tile(nxt);                     // tile being loaded
  if (!ld.valid) return;                          // nothing to do for this workgroup
  int bias_buf = 0;                               // buffer that holds the bias of the tile being multiplied
  int scale_buf = 0;                              // ... and its scales (one of three)
  if constexpr (GATHER || kBiasInAcc || W8) {
    copy_row_slots(nxt);
    copy_bias(nxt, 0);
    copy_scale(nxt, 0);
    pwait_vmcnt<0>();
    phase_barrier();
  }
  Tile cp = ld;                                   // tile being multiplied
  int ld_kt = 0;
  set_copy_offsets(ld);
  nxt = fetch_tile(next_turn++);                  // the one the load side opens next
  if constexpr (GATHER) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // everyone has read the first tile's row slots
    phase_barrier();
    copy_row_slots(nxt);
  }
  copy_bias(nxt, 1);
  copy_scale(nxt, 1);
  auto advance_copy = [&]() {
    if (++ld_kt == ld.steps) {
      ld = unpack_tile(nxt);
      set_copy_offsets(ld);
      ld_kt = 0;
    }
  };
  // A step's loads in four quarters: the two halves of the activation rows, then
  // the two halves of the weight rows.  first(q) .. first(q + 1) are quarter q's
  // indices into the register stage.
  // Load l of the step the load side stands at, into register stage P.
  auto load_one = [&](auto stage_c, auto l_c) {
    constexpr int P = decltype(stage_c)::value, l = decltype(l_c)::value;
    if constexpr (l < kCopiesA) {
      // (uni() costs nothing while the description sits in scalar registers and
      // avoids a loop over lanes around the load if the compiler moved it out)
      const __amdgpu_buffer_rsrc_t rs =
          __builtin_amdgcn_make_buffer_rsrc((void *)uni(ld.a), 0, uni(ld.a_bytes), kRsrcFlags);
      uint32_t voff;
      if constexpr (GATHER) voff = ld_voff_rows[l];
      else voff = ld_voff_a + (uint32_t)(32 * l) * uni(ld.a_pitch);
      stage_regs[P][l] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, uni(ld_kt * 128), 0);
    } else {
      constexpr int i = l - kCopiesA;
      constexpr int kStride = kRowsPerCopyB * kQWaves;  // weight rows between a lane's consecutive loads
      constexpr bool up_half = SWIGLU && kStride * i >= BN / 2;  // a wave's rows of one load never cross the halves
      constexpr int row = up_half ? kStride * i - BN / 2 : kStride * i;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)uni(up_half ? ld.b1 : ld.b0), 0, uni(ld.b_bytes), kRsrcFlags);
      stage_regs[P][l] = __builtin_amdgcn_raw_buffer_load_b128(
          rs, ld_voff_b + (uint32_t)row * uni(ld.b_pitch), uni(ld_kt * (W8 ? 64 : 128)), 0);
    }
  };
  // Load l of register stage P into LDS slot P.
  auto write_one = [&](auto stage_c, auto l_c) {
    constexpr int P = decltype(stage_c)::value, l = decltype(l_c)::value;
    constexpr int i = l < kCopiesA ? l : l - kCopiesA;
    if constexpr (W8 && l >= kCopiesA) {
      unsigned char *row = (P == 0 ? lds_slot0 : lds_slot1) + kPBM * 128 + i * (kRowsPerCopyB * kQWaves) * 128;
      const u32x4_t src = stage_regs[P][l];
      u32x4_t lo, hi;
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        lo[2 * q] = widen_fp8_pair(src[q], false);
        lo[2 * q + 1] = widen_fp8_pair(src[q], true);
        hi[2 * q] = widen_fp8_pair(src[q + 2], false);
        hi[2 * q + 1] = widen_fp8_pair(src[q + 2], true);
      }
      *reinterpret_cast<u32x4_any_t *>(row + wr_off_b8) = lo;
      *reinterpret_cast<u32x4_any_t *>(row + wr_off_b8_hi) = hi;
    } else {
      unsigned char *dst = (P == 0 ? lds_slot0 : lds_slot1) + (l < kCopiesA ? 0 : kPBM * 128) + i * 32 * 128 + wr_off;
      *reinterpret_cast<u32x4_any_t *>(dst) = stage_regs[P][l];
    }
  };
  // Quarter Q of a step covers loads [quarter_first(Q), quarter_first(Q + 1)).
  auto load_quarter = [&](auto stage_c, auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    constexpr int F = quarter_first(kCopiesA, kCopiesB, Q), N = quarter_first(kCopiesA, kCopiesB, Q + 1) - F;
    static_for<N>([&](auto n_c) { load_one(stage_c, template_int<F + decltype(n_c)::value>{}); });
  };
  auto write_quarter = [&](auto stage_c, auto q_c) {
    constexpr int Q = decltype(q_c)::value;
    constexpr int F = quarter_first(kCopiesA, kCopiesB, Q), N = quarter_first(kCopiesA, kCopiesB, Q + 1) - F;
    static_for<N>([&](auto n_c) { write_one(stage_c, template_int<F + decltype(n_c)::value>{}); });
  };
  auto load_step = [&](auto stage_c) {
    load_quarter(stage_c, c0); load_quarter(stage_c, c1); load_quarter(stage_c, c2); load_quarter(stage_c, c3);
    advance_copy();
  };
  auto write_step = [&](auto stage_c) {
    write_quarter(stage_c, c0); write_quarter(stage_c, c1); write_quarter(stage_c, c2); write_quarter(stage_c, c3);
  };

  // Prologue: steps 0 and 1 through the stages into the slots (of step 1 only
  // the first quarter: the rest follows during step 0, as in the steady state),
  // steps 2 and 3 into the stages behind them.
  load_step(c0);           // step 0
  load_step(c1);           // step 1
  write_step(c0);
  load_step(c0);           // step 2
  write_quarter(c1, c0);
  load_quarter(c1, c0);    // first quarter of step 3; the stage keeps quarters 1..3 of step 1
  init_acc(cp, 0, 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();
  read_frags(c0, c0, c0);
  __builtin_amdgcn_sched_barrier(0);

  unsigned char *const stage_rows = lds_stage + wave * Epi::WAVE_BYTES;
  f32x16_t no_acc[TM][TN];  // (the epilogue takes the sums from the accumulation registers; never read)

  // One block of a step: the TM x TN products of fragment buffer MB and, threaded
  // between them (side_slot), the reads of the fragments of 16-k block RK of slot
  // RS into the other buffer, quarter Q of register stage WP into LDS slot WP, and
  // quarter Q of the step the load side stands at into that stage.  The products
  // are volatile asm statements, which no memory instruction is moved across: the
  // order below is the order of the instructions.
  auto block = [&](auto mb_c, auto rs_c, auto rk_c, auto wp_c, auto q_c) {
    constexpr int MB = decltype(mb_c)::value, Q = decltype(q_c)::value;
    constexpr int MF = TM * TN, RD = TM + TN;
    constexpr int F = quarter_first(kCopiesA, kCopiesB, Q), N = quarter_first(kCopiesA, kCopiesB, Q + 1) - F;
    const template_int<MB ^ 1> rb_c;
    static_assert(RD <= MF && N <= MF, "at most one item of a kind per product");
    static_for<MF>([&](auto i_c) {
      constexpr int I = decltype(i_c)::value;
      mfma_at(mb_c, i_c);
      constexpr int R = side_item(I, RD, MF, 0), W = side_item(I, N, MF, 1), L = side_item(I, N, MF, 3);
      // (where two share a gap the read goes first: a read queued behind a write
      // waits for the write's 16 cycles)
      if constexpr (R >= 0) read_frag(rs_c, rk_c, rb_c, template_int<R>{});
      if constexpr (R >= 0 && (W >= 0 || L >= 0)) __builtin_amdgcn_sched_barrier(0);
      if constexpr (W >= 0) write_one(wp_c, template_int<F + W>{});
      if constexpr (W >= 0 && L >= 0) __builtin_amdgcn_sched_barrier(0);
      if constexpr (L >= 0) load_one(wp_c, template_int<F + L>{});
    });
    __builtin_amdgcn_sched_barrier(0);
  };

  while (true) {  // one tile per iteration
    // Every tile has an even number of steps, so a tile always starts in slot 0.
    auto step = [&](auto slot_c) {
      constexpr int S = decltype(slot_c)::value;
      const template_int<S ^ 1> other_c;
      block(c0, slot_c, c1, other_c, c1);
      block(c1, slot_c, c2, other_c, c2);
      block(c0, slot_c, c3, other_c, c3);
      advance_copy();
      // This wave has read slot S for the last time and has finished writing the
      // other slot; after the barrier both hold for every wave.
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      phase_barrier();
      block(c1, other_c, c0, slot_c, c0);
    };
    for (int s = 0; s < cp.steps; s += 2) {
      step(c0);
      step(c1);
    }
    fixed_acc_settle();
    tile_epilogue<MODE, HAS_BIAS && !kBiasInAcc, kQWaves, TM, TN, W8, W8 ? kEpiReserve : 0, false, false, kAccBlock0, !kBiasInAcc>(
        cp, no_acc, stage_rows, wm * WTM, wave_col0, lane, lds_scale + scale_buf * kScaleBufFloats);
    // The load side is within the next tile here (every tile has at least
    // kQMinSteps steps).
    cp = ld;
    if (!cp.valid) break;
    nxt = fetch_tile(next_turn++);
    // The load side opened this tile's predecessor at least kQMinSteps - 4 steps
    // (each with a barrier) ago and read its row slots then: the buffer is free.
    // The copy below is older than every load of the coming steps, so the waits
    // for those (at most 32 newer loads are ever in flight) cover it long before
    // the load side opens `nxt`, at least two steps from here.
    copy_row_slots(nxt);
    // (the bias buffer written here was last read a whole tile ago, the one read
    // below was filled a whole tile ago: the same ordering as for the row slots)
    copy_bias(nxt, bias_buf);
    bias_buf ^= 1;
    scale_buf = scale_buf == 2 ? 0 : scale_buf + 1;       // the tile multiplied next
    copy_scale(nxt, scale_buf == 2 ? 0 : scale_buf + 1);  // the one after it
    // (without a bias the epilogue has cleared every block it read)
    if constexpr (kBiasInAcc) init_acc(cp, bias_buf, scale_buf);
    // The last block above already fetched these fragments; reading them again
    // here keeps 32 registers free during the epilogue.
    read_frags(c0, c0, c0);
  }
}

// ---------------------------------------------------------------------------
// The same 64-k pipeline with its k-loop in assembly (persist64_asm.inc, written by
// gen_persist64_asm.py: register plan, order of the pieces and wait counts are
// described there).  Every memory instruction of the loop, its registers and its
// waits are spelled out; the compiler's share between the statements is scalar
// bookkeeping (the load side's position, the tile switch) and the epilogue.
// What this buys over the loop the compiler schedules (gemm_persist64_body):
//   * a group's last tile multiplies only its live 64-row blocks (the two waves
//     that share a tile's columns take alternate 32-row blocks, so both have
//     work in every live block): one loop variant per number of live blocks;
//   * the first products of a tile start the sums (no clearing);
// neither of which the compiler-scheduled loop survives: a second copy of the
// loop or a branch inside it sends its register allocator through the
// accumulation registers and its wait-count pass to lgkmcnt(0) at every join
// (in-block branches: bit-identical results, 62 % longer layer call).
// Taken for 16-bit weights and bias-free tiles of the two shapes generated:
// KIND 0 = SwiGLU fc1 with gathered rows (256 weight rows), KIND 1 = fc2 with
// 192 weight rows.
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
typedef float f32x32_t __attribute__((ext_vector_type(32)));
#include "persist64_asm.inc"

template <int MODE, bool HAS_BIAS, int BN, bool GATHER, bool W8>
constexpr bool persist64_asm_applies() {
  return !W8 && !HAS_BIAS && ((MODE == kFc1Swiglu && BN == 256 && GATHER) || (MODE == kFc2 && BN == 192));
}

template <int MODE, int BN, bool GATHER, bool REFILL>
__device__ __forceinline__ void gemm_persist64_asm_body(const PersistBatch &batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int KIND = SWIGLU ? 0 : 1;
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTN = BN / 2, TM = 4, TN = WTN / 32;
  constexpr int kCopiesA = kPBM / 8 / kQWaves, kCopiesB = BN / 8 / kQWaves;
  constexpr int kAccBlock0 = 16 - TM * TN;
  using Epi = EpiGeom<MODE, kQWaves, TM, TN, 0>;
  typedef __attribute__((address_space(3))) unsigned char lds_byte_t;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot0[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot1[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_stage[kPStageArea];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  fixed_acc_declare();

  constexpr int kTableBytes = kTableTurns * kTileWords * 4, kRowSlotBytes = kPBM * 4;
  static_assert(kQWaves * Epi::WAVE_BYTES + kTableBytes + (GATHER ? kRowSlotBytes : 0) <= kPStageArea,
                "no room for the tile table");
  uint32_t *const tile_table = reinterpret_cast<uint32_t *>(lds_stage + kPStageArea - kTableBytes);
  int32_t *const lds_row_slots = reinterpret_cast<int32_t *>(lds_stage + kPStageArea - kTableBytes - kRowSlotBytes);
  if (wave == 0) {
    TileWalker<BN_OUT> walk(batch, lane);
    walk.build_table(batch, lane, kQBK, tile_table, false);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();
  auto fetch_tile = [&](int turn) {
    if constexpr (REFILL) {
      if (turn != 0 && (turn & (kTableTurns - 1)) == 0) {
        phase_barrier();
        if (wave == 0) {
          TileWalker<BN_OUT> walk(batch, lane);
          walk.build_table(batch, lane, kQBK, tile_table, false, turn);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        phase_barrier();
      }
    }
    int lane_c = lane;   // (opaque: worked out at the tile switch, not held through the k-loop)
    asm volatile("" : "+v"(lane_c));
    return PackedTile{tile_table[(turn & (kTableTurns - 1)) * kTileWords + (lane_c < kTileWords ? lane_c : 0)]};
  };

  // ---- addresses the assembly takes (see P64Addr) ----
  const int cp_row0 = wave * 8 + (lane >> 3), cp_chunk = lane & 7;
  const int b_row0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;
  const uint32_t slot_base[2] = {(uint32_t)(size_t)(lds_byte_t *)lds_slot0, (uint32_t)(size_t)(lds_byte_t *)lds_slot1};
  P64Addr ad;
  // Three of the LDS addresses are kept; the other fifteen follow from them at
  // the start of every tile (one integer instruction each: 16-k block kk of a
  // fragment row is the chunk index xor 2 kk, slot 1 lies a constant behind slot
  // 0), so that they do not hold registers through the epilogue.
  uint32_t wr0 = slot_base[0] + qring_off(cp_row0, cp_chunk);
  uint32_t ra0 = slot_base[0] + qring_off(wm * 32 + (lane & 31), lane >> 5);
  uint32_t rb0 = slot_base[0] + kPBM * 128 + qring_off(b_row0 + (lane & 31), lane >> 5);
  static_assert((kQSlotBytes & 1023) == 0, "the xor below must stay inside the chunk field");
  auto set_lds_addresses = [&]() {
    asm volatile("" : "+v"(wr0), "+v"(ra0), "+v"(rb0));
    const uint32_t slot1 = slot_base[1] - slot_base[0];
    ad.wr[0] = wr0;
    ad.wr[1] = wr0 + slot1;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      // (row block i of wave row wm = tile rows 64 i + 32 wm ..: the assembly adds i x 64 rows)
      ad.ra[0][kk] = ra0 ^ (uint32_t)(kk << 5);
      ad.rb[0][kk] = rb0 ^ (uint32_t)(kk << 5);
      ad.ra[1][kk] = ad.ra[0][kk] + slot1;
      ad.rb[1][kk] = ad.rb[0][kk] + slot1;
    }
  };
  set_lds_addresses();
#pragma unroll
  for (int i = 0; i < 8; ++i) ad.va[i] = 0;
  ad.vb = 0;
  uint32_t sb_row[8] = {}, sb[8] = {};   // scalar offsets of the weight loads: row part, and with the step's k offset
  auto copy_row_slots = [&](const PackedTile &pk) {
    if constexpr (GATHER) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 21) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 20);
      const int rows = __builtin_amdgcn_readlane(pk.words, 23);
      if (wave == 0 && ptr != 0) {
        // Global memory -> LDS without a register in between, as text: a load the
        // compiler knows of would have it wait for "its only load" with vmcnt(0)
        // before the next LDS access of its own - which drains the 32 operand
        // loads the assembly keeps in flight, once per tile.  Rows past the
        // group's end read as slot 0 (a legal row; their products are never
        // stored).  M0 holds the LDS address for the instruction and is put back.
        const u32x4_t rs = {uni((uint32_t)ptr), uni((uint32_t)(ptr >> 32) & 0xffffu), uni((uint32_t)rows * 4u),
                            kRsrcFlags};
        const uint32_t dst = uni((uint32_t)(size_t)(lds_byte_t *)lds_row_slots);
        int lane_c = lane;
        asm volatile("" : "+v"(lane_c));
        const uint32_t voff = (uint32_t)lane_c * 16u;
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
    }
  };
  // Descriptors of the tile being loaded, as plain register values (base, extent, flags).
  u32x4_t dA, dB0, dB1;
  auto set_copy_offsets = [&](const Tile &t) {
    auto desc = [](const unsigned char *base, uint32_t bytes) {
      const uint64_t p = (uint64_t)base;
      return u32x4_t{uni((uint32_t)p), uni((uint32_t)(p >> 32) & 0xffffu), uni(bytes), kRsrcFlags};
    };
    dA = desc(t.a, t.a_bytes);
    dB0 = desc(t.b0, t.b_bytes);
    dB1 = desc(t.b1, t.b_bytes);
    int row0 = cp_row0;   // (opaque, as the lane above)
    asm volatile("" : "+v"(row0));
    const uint32_t voff_a = (uint32_t)row0 * t.a_pitch + cp_chunk * 16;
    const uint32_t voff_b = (uint32_t)row0 * t.b_pitch + cp_chunk * 16;
#pragma unroll
    for (int i = 0; i < kCopiesA; ++i) {
      const int r = row0 + 32 * i;
      uint32_t off = voff_a + (uint32_t)(32 * i) * t.a_pitch;
      if constexpr (GATHER) {
        if (t.a_rows) {
          const uint32_t slot = (uint32_t)lds_row_slots[r];
          const uint32_t src_row = t.a_magic ? __umulhi(slot, t.a_magic) : slot;
          off = r < t.rows ? src_row * t.a_pitch + cp_chunk * 16 : kOutOfRange;
        }
      }
      ad.va[i] = off;
    }
    ad.vb = voff_b;
#pragma unroll
    for (int i = 0; i < kCopiesB; ++i) {
      const int row = (SWIGLU && 32 * i >= BN / 2) ? 32 * i - BN / 2 : 32 * i;   // (the up half has its own descriptor)
      sb_row[i] = uni((uint32_t)row * t.b_pitch);
    }
  };

  // ---- pipeline state (as gemm_persist64_body) ----
  int next_turn = 0;
  PackedTile nxt = fetch_tile(next_turn++);
  Tile ld = unpack_tile(nxt);
  if (!ld.valid) return;
  if constexpr (GATHER) {
    copy_row_slots(nxt);
    pwait_vmcnt<0>();
    phase_barrier();
  }
  Tile cp = ld;
  int ld_kt = 0;
  set_copy_offsets(ld);
  nxt = fetch_tile(next_turn++);
  if constexpr (GATHER) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    phase_barrier();
    copy_row_slots(nxt);
  }
  uint32_t koff = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) sb[i] = sb_row[i];
  auto advance_copy = [&]() {
    if (++ld_kt == ld.steps) {
      ld = unpack_tile(nxt);
      set_copy_offsets(ld);
      ld_kt = 0;
    }
    koff = uni((uint32_t)ld_kt * 128u);
#pragma unroll
    for (int i = 0; i < 8; ++i) sb[i] = uni(sb_row[i] + koff);
  };
  // The two register stages (v128..v255) carry loads in flight from one tile
  // into the next, across the epilogue: the assembly names them, and the kernel
  // is compiled with a budget of 128 vector registers (gemm_persist_kernel4a), so
  // the compiler's own values never sit there.
  {
    // (the prologue reads and writes no fragments; the buffers are values of a tile's
    // k-loop only, so that their registers are free for the epilogue)
    f32x32_t f0, f1;
    asm volatile("" : "={v[0:31]}"(f0), "={v[32:63]}"(f1));

  // Prologue: steps 0 and 1 through the stages into the slots (of step 1 only the
  // first quarter), steps 2 and 3 (first quarter) into the stages behind them.
  p64_load_step0<KIND, 4>(P64_ARGS);
  advance_copy();
  p64_load_step1<KIND, 4>(P64_ARGS);
  advance_copy();
  p64_write_step0<KIND, 4>(P64_ARGS);
  p64_load_step0<KIND, 4>(P64_ARGS);
  advance_copy();
  p64_write_q0_stage1<KIND, 4>(P64_ARGS);
  p64_load_q0_stage1<KIND, 4>(P64_ARGS);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();

  unsigned char *const stage_rows = lds_stage + wave * Epi::WAVE_BYTES;
  f32x16_t no_acc[TM][TN];
  const int wave_col0 = SWIGLU ? wn * (WTN / 2) : wn * WTN;

  // The steps of a tile whose rows fill its first LIVE 64-row blocks.
  auto run_tile = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    f32x32_t f0, f1;   // the fragment buffers: live inside the tile's k-loop only
    asm volatile("" : "={v[0:31]}"(f0), "={v[32:63]}"(f1));
    set_lds_addresses();
    p64_read_first<KIND, LIVE>(P64_ARGS);
    p64_abc_s0_v1<KIND, LIVE>(P64_ARGS);   // the first 16-k block's products start the sums
    advance_copy();
    p64_d_s0<KIND, LIVE>(P64_ARGS);
    p64_abc_s1_v0<KIND, LIVE>(P64_ARGS);
    advance_copy();
    p64_d_s1<KIND, LIVE>(P64_ARGS);
    for (int s = 2; s < cp.steps; s += 2) {
      p64_abc_s0_v0<KIND, LIVE>(P64_ARGS);
      advance_copy();
      p64_d_s0<KIND, LIVE>(P64_ARGS);
      p64_abc_s1_v0<KIND, LIVE>(P64_ARGS);
      advance_copy();
      p64_d_s1<KIND, LIVE>(P64_ARGS);
    }
  };

  while (true) {  // one tile per iteration
    const int live = uni((cp.rows + 63) >> 6);   // 64-row blocks of the tile that hold rows of its group
    if (live >= 4) run_tile(template_int<4>{});
    else if (live == 3) run_tile(template_int<3>{});
    else if (live == 2) run_tile(template_int<2>{});
    else run_tile(template_int<1>{});
    fixed_acc_settle();
    int lane_e = lane;   // (opaque: the epilogue's addresses are worked out here, not held through the k-loop)
    asm volatile("" : "+v"(lane_e));
    tile_epilogue<MODE, false, kQWaves, TM, TN, false, 0, false, false, kAccBlock0, false, 64>(
        cp, no_acc, stage_rows, wm * 32, wave_col0, lane_e, nullptr, nullptr, nullptr, live);
    cp = ld;
    if (!cp.valid) break;
    nxt = fetch_tile(next_turn++);
    copy_row_slots(nxt);
  }
}

#if DICE_PERSIST_F8
// ---------------------------------------------------------------------------
// fp8 x fp8 pipeline, four waves: e4m3 activations (one fp32 scale per row) times
// e4m3 weights (one fp32 scale per output channel) on v_mfma_f32_32x32x64_f8f6f4,
// which multiplies at twice the rate of the bf16 instruction.
//
// In bytes this is the 64-k pipeline above: rows of 128 bytes per step (now 128
// k), two 64 KB LDS slots, operands staged through register stages three
// steps ahead, the same 256x256 tile, wave tile, epilogue and tile table - so
// the bytes moved per matrix-pipe cycle are those of the bf16 kernel while every
// byte carries twice the arithmetic.  What differs:
//
//   * A fragment of the fp8 instruction is 32 bytes per lane (two 16-byte LDS
//     reads).  The hardware lets lanes 0-31 and 32-63 each hold 32 k of a row;
//     any assignment of k to (lane half, byte) works as long as both operands
//     use the same one, here: half h of k-block kb takes the row's 16-byte
//     chunks 4 kb + 2 h and 4 kb + 2 h + 1.
//   * Three register stages instead of four: two for the weight rows (loaded two
//     steps before they are written to LDS), one for the activation rows (one
//     step), see load_quarter.
//   * Fragments twice the size do not fit twice in the register file, so they
//     are not double-buffered.  A step is two halves of 16 MFMAs (one per 64-k
//     block), taken weight block by weight block (the row blocks up and down in
//     turn, so that only one operand changes from one product to the next);
//     during a half the next half's fragments are read into the registers of
//     operands as they die: weight block j behind the four MFMAs that use it,
//     the row blocks one by one during the last weight block, and what the
//     half's last MFMA still holds (the last weight block and one row block)
//     right behind it.  Eight fragments = 64 registers, as many as the bf16
//     kernel's double-buffered set.
//   * The workgroup barrier sits four MFMAs into the second half: by then
//     every wave has read the step's slot for the last time (the trailing reads
//     of the first half have had four MFMAs to land) and has finished writing
//     the other slot; behind it the second half starts to refill this slot and
//     to read the next step's fragments from the other one.  Each half writes
//     two quarters of a step into LDS and issues the loads that refill those
//     register stages.
//   * The epilogue multiplies the fp32 sums by the row's and the column's scale
//     and adds the bias (all three staged in LDS a tile ahead).
//
// Rows are contiguous (the quantiser writes the activations in grouped order),
// the reduction length is a multiple of 256 (an even number of steps), weight
// tiles are 256 rows (SwiGLU: 128 gate + 128 up), single-problem launches.
typedef int i32x8_t __attribute__((ext_vector_type(8)));
__device__ __forceinline__ f32x16_t mfma_f8_32x32x64(i32x8_t a, i32x8_t b, f32x16_t c) {
  // cbsz = blgp = 0: both operands e4m3; zero scale operands select the unscaled instruction
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// Instruction order of one half.  MFMA m (weight block m / 4) is followed by the
// fragment reads whose registers have just come free: weight block 0 behind MFMAs
// 4 and 5, weight block 1 behind 8 and 9, weight block 2 and three row blocks in
// pairs behind 12..15, the last row block and weight block 3 behind the half; and by
// the LDS writes of a register stage alternating with the global loads that
// refill it, from MFMA FIRST on (the second half of a step starts them behind its
// barrier: 16 of them over 12 MFMAs).
template <int M, int FIRST>
__device__ __forceinline__ void f8_sched_half() {
  if constexpr (M < 16) {
    if constexpr (M >= FIRST) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      constexpr int reads = (M == 4 || M == 5 || M == 8 || M == 9) ? 1 : (M >= 12 ? 2 : 0);
      if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);
      if constexpr (FIRST > 0 && M < 2 * FIRST) {
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      } else if constexpr (M % 2 == 0) {
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      } else {
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    f8_sched_half<M + 1, FIRST>();
  } else {
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
  }
}

template <int MODE, bool HAS_BIAS, bool REFILL>
__device__ __forceinline__ void gemm_persist_f8_body(const PersistBatch &batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  static_assert(!(SWIGLU && HAS_BIAS), "the SwiGLU expert has no bias");
  constexpr int BN_OUT = SWIGLU ? kPBN / 2 : kPBN;
  constexpr int WTM = 128, TM = 4, TN = 4;
  constexpr int kFBK = 128;                         // k per step (one byte per element)
  constexpr int kCopiesA = kPBM / 8 / kQWaves;      // 16-byte loads per lane and step: 8 + 8
  constexpr int kFCopies = 2 * kCopiesA;
  constexpr int kScaleBufFloats = 256, kBiasBufFloats = 256;
  constexpr int kTableBytes = kTableTurns * kTileWords * 4;
  // three buffers each for the column scales, the row scales and the bias: the
  // epilogue of a tile reads them while the first wave, a little ahead, may
  // already stage those of the tile after the next
  constexpr int kColScaleBytes = 3 * kScaleBufFloats * 4, kRowScaleBytes = 3 * kPBM * 4;
  constexpr int kBiasBytes = HAS_BIAS ? 3 * kBiasBufFloats * 4 : 0;
  constexpr int kEpiReserve = kTableBytes + kColScaleBytes + kRowScaleBytes + kBiasBytes;
  using Epi = EpiGeom<MODE, kQWaves, TM, TN, kEpiReserve>;
  static_assert(kQWaves * Epi::WAVE_BYTES + kEpiReserve <= kPStageArea, "no room beside the epilogue's staging rows");
  const template_int<0> c0; const template_int<1> c1; const template_int<2> c2; const template_int<3> c3;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot0[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot1[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_stage[kPStageArea];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  uint32_t *const tile_table = reinterpret_cast<uint32_t *>(lds_stage + kPStageArea - kTableBytes);
  float *const lds_colscale = reinterpret_cast<float *>(lds_stage + kPStageArea - kTableBytes - kColScaleBytes);
  float *const lds_rowscale =
      reinterpret_cast<float *>(lds_stage + kPStageArea - kTableBytes - kColScaleBytes - kRowScaleBytes);
  float *const lds_bias = reinterpret_cast<float *>(lds_stage + kPStageArea - kEpiReserve);
  if (wave == 0) {
    TileWalker<BN_OUT> walk(batch, lane);
    walk.build_table(batch, lane, kFBK, tile_table, true, 0, true);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();
  auto fetch_tile = [&](int turn) {
    if constexpr (REFILL) {
      if (turn != 0 && (turn & (kTableTurns - 1)) == 0) {
        phase_barrier();
        if (wave == 0) {
          TileWalker<BN_OUT> walk(batch, lane);
          walk.build_table(batch, lane, kFBK, tile_table, true, turn, true);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        phase_barrier();
      }
    }
    return PackedTile{tile_table[(turn & (kTableTurns - 1)) * kTileWords + (lane < kTileWords ? lane : 0)]};
  };

  // ---- what the first wave stages in LDS a tile ahead (one global->LDS
  // instruction each): column scales, row scales, bias ----
  auto copy_colscale = [&](const PackedTile &pk, int buf) {
    const uint32_t row = (uint32_t)__builtin_amdgcn_readlane(pk.words, 22);
    const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
    if (wave == 0) {
      const float *base = batch.prob[0].w_scale + row;
      // SwiGLU: 128 gate scales, then the 128 up scales up_offset rows further on;
      // otherwise the tile's columns, those past the matrix reading as 0
      const uint32_t bytes = SWIGLU ? (uint32_t)(batch.prob[0].up_offset + 128) * 4 : (uint32_t)(n - n0) * 4;
      const uint32_t voff = SWIGLU && lane >= 32 ? (uint32_t)batch.prob[0].up_offset * 4 + (lane - 32) * 16 : lane * 16;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, bytes, kRsrcFlags);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs, (__attribute__((address_space(3))) void *)(lds_colscale + buf * kScaleBufFloats), 16, voff, 0, 0, 0);
    }
  };
  auto copy_rowscale = [&](const PackedTile &pk, int buf) {
    const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 21) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane(pk.words, 20);
    const int rows = __builtin_amdgcn_readlane(pk.words, 23);
    if (wave == 0 && ptr != 0) {
      // rows past the group's end read as 0 (their products are never stored)
      const __amdgpu_buffer_rsrc_t rs =
          __builtin_amdgcn_make_buffer_rsrc((void *)ptr, 0, (uint32_t)rows * 4, kRsrcFlags);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs, (__attribute__((address_space(3))) void *)(lds_rowscale + buf * kPBM), 16, lane * 16, 0, 0, 0);
    }
  };
  auto copy_bias = [&](const PackedTile &pk, int buf) {
    if constexpr (HAS_BIAS) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 9) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 8);
      const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
      if (wave == 0) {
        // A tile without a bias (the later pieces of a tile that is cut along k)
        // gets zeros: a descriptor that covers no bytes.
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            ptr != 0 ? (void *)(ptr + (uint64_t)n0 * 4) : (void *)batch.prob[0].w_scale, 0,
            ptr != 0 ? (uint32_t)(n - n0) * 4 : 0u, kRsrcFlags);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (__attribute__((address_space(3))) void *)(lds_bias + buf * kBiasBufFloats), 16, lane * 16, 0, 0, 0);
      }
    }
  };

  // ---- global loads: one instruction fetches 8 rows x 128 bytes (8 lanes per
  // row, whole lines); load l of a wave covers rows wave * 8 + 32 (l % 8) .. + 8
  // of the activation tile (l < 8) or of the weight tile ----
  const int cp_row0 = wave * 8 + (lane >> 3);
  const int cp_chunk = lane & 7;
  uint32_t wr_off = qring_off(cp_row0, cp_chunk);
  asm volatile("" : "+v"(wr_off));
  uint32_t ld_voff_a = 0, ld_voff_b = 0;
  auto set_copy_offsets = [&](const Tile &t) {
    ld_voff_a = (uint32_t)cp_row0 * t.a_pitch + cp_chunk * 16;
    ld_voff_b = (uint32_t)cp_row0 * t.b_pitch + cp_chunk * 16;
    asm volatile("" : "+v"(ld_voff_a), "+v"(ld_voff_b));
  };
  u32x4_t stage_regs[2][kFCopies];

  // ---- fragment reads: lane part per (k-block, 16-byte half); 32-row blocks and
  // the slot add compile-time constants ----
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int b_row0 = SWIGLU ? wn * 64 : wn * 128;
  uint32_t rd_a[4], rd_b[4];   // [2 kb + t]: chunk 4 kb + 2 h + t of the lane's row
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      rd_a[kb * 2 + t] = qring_off(wm * WTM + frag_row, kb * 4 + frag_half * 2 + t);
      rd_b[kb * 2 + t] = kPBM * 128 + qring_off(b_row0 + frag_row, kb * 4 + frag_half * 2 + t);
      asm volatile("" : "+v"(rd_a[kb * 2 + t]), "+v"(rd_b[kb * 2 + t]));
    }
  auto read32 = [&](const unsigned char *slot, uint32_t off_lo, uint32_t off_hi) {
    const u32x4_t lo = *reinterpret_cast<const u32x4_any_t *>(slot + off_lo);
    const u32x4_t hi = *reinterpret_cast<const u32x4_any_t *>(slot + off_hi);
    i32x8_t f;
    f[0] = (int)lo[0]; f[1] = (int)lo[1]; f[2] = (int)lo[2]; f[3] = (int)lo[3];
    f[4] = (int)hi[0]; f[5] = (int)hi[1]; f[6] = (int)hi[2]; f[7] = (int)hi[3];
    return f;
  };
  // activation rows 32 i .. of the wave's 128, k-block KB of slot SLOT
  auto read_a = [&](auto slot_c, auto kb_c, int i) {
    constexpr int SLOT = decltype(slot_c)::value, KB = decltype(kb_c)::value;
    const unsigned char *base = (SLOT == 0 ? lds_slot0 : lds_slot1) + i * 32 * 128;
    return read32(base, rd_a[KB * 2], rd_a[KB * 2 + 1]);
  };
  // weight block j of the wave's four (SwiGLU: two of gate rows, two of up rows)
  auto read_w = [&](auto slot_c, auto kb_c, int j) {
    constexpr int SLOT = decltype(slot_c)::value, KB = decltype(kb_c)::value;
    const int jrow = (SWIGLU && j >= 2) ? kPBN / 2 + (j - 2) * 32 : j * 32;
    const unsigned char *base = (SLOT == 0 ? lds_slot0 : lds_slot1) + jrow * 128;
    return read32(base, rd_b[KB * 2], rd_b[KB * 2 + 1]);
  };

  const int wave_col0 = SWIGLU ? wn * 64 : wn * 128;
  f32x16_t acc[TM][TN];
  // (a bias is added in the epilogue, from LDS, behind the two scales)
  auto init_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
  };

  // ---- pipeline state (as in the 64-k pipeline) ----
  int next_turn = 0;
  PackedTile nxt = fetch_tile(next_turn++);
  Tile ld = unpack_tile(nxt);                     // tile being loaded
  if (!ld.valid) return;
  int scale_buf = 0;                              // buffer of the scales and the bias of the tile being multiplied
  copy_colscale(nxt, 0);
  copy_rowscale(nxt, 0);
  copy_bias(nxt, 0);
  pwait_vmcnt<0>();
  phase_barrier();
  Tile cp = ld;                                   // tile being multiplied
  int ld_kt = 0;
  set_copy_offsets(ld);
  nxt = fetch_tile(next_turn++);                  // the one the load side opens next
  copy_colscale(nxt, 1);
  copy_rowscale(nxt, 1);
  copy_bias(nxt, 1);
  auto advance_copy = [&]() {
    if (++ld_kt == ld.steps) {
      ld = unpack_tile(nxt);
      set_copy_offsets(ld);
      ld_kt = 0;
    }
  };
  // A step's loads in four quarters of four: the two halves of the activation
  // rows, then the two halves of the weight rows.  The weight rows of a step wait
  // in one of two register stages (by the parity of the step) for two steps, the
  // activation rows in a single stage for one: weight tiles stream from HBM and
  // need the longer flight; the activation tiles of an expert are re-read for
  // every n-tile and come from the L2.  A third stage of 32 registers more does
  // not fit: the register allocator then keeps one or two loads of every step
  // in scratch memory, and each such load drains the whole load queue twice.
  auto load_quarter = [&](auto stage_c, auto q_c) {
    constexpr int Q = decltype(q_c)::value, P = Q < 2 ? 0 : decltype(stage_c)::value;
#pragma unroll
    for (int l = 4 * Q; l < 4 * Q + 4; ++l) {
      // The row block of a load is folded into its descriptor (base moved on, extent
      // cut by as much: scalar arithmetic only), not into the scalar offset, which
      // the range check ignores: rows past the tile's end must read as zero, never
      // from beyond the matrix.
      if (l < kCopiesA) {
        const uint32_t skip = (uint32_t)(32 * l) * uni(ld.a_pitch);
        // (signed, both below 2^31: a scalar subtract and max; the unsigned form
        // becomes a saturating vector subtract and the descriptor a per-lane value)
        const int left = (int)uni(ld.a_bytes) - (int)skip;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(uni(ld.a) + skip), 0, uni((uint32_t)(left > 0 ? left : 0)), kRsrcFlags);
        stage_regs[P][l] = __builtin_amdgcn_raw_buffer_load_b128(rs, ld_voff_a, uni(ld_kt * kFBK), 0);
      } else {
        const int i = l - kCopiesA;
        const bool up_half = SWIGLU && 32 * i >= kPBN / 2;
        const int row = up_half ? 32 * i - kPBN / 2 : 32 * i;
        const uint32_t skip = (uint32_t)row * uni(ld.b_pitch);
        const int left = (int)uni(ld.b_bytes) - (int)skip;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(uni(up_half ? ld.b1 : ld.b0) + skip), 0, uni((uint32_t)(left > 0 ? left : 0)), kRsrcFlags);
        stage_regs[P][l] = __builtin_amdgcn_raw_buffer_load_b128(rs, ld_voff_b, uni(ld_kt * kFBK), 0);
      }
    }
  };
  // Quarter q of the register stage(s) into LDS slot SLOT.
  auto write_quarter = [&](auto slot_c, auto q_c) {
    constexpr int SLOT = decltype(slot_c)::value, Q = decltype(q_c)::value, P = Q < 2 ? 0 : SLOT;
#pragma unroll
    for (int l = 4 * Q; l < 4 * Q + 4; ++l) {
      const int i = l < kCopiesA ? l : l - kCopiesA;
      unsigned char *dst = (SLOT == 0 ? lds_slot0 : lds_slot1) + (l < kCopiesA ? 0 : kPBM * 128) + i * 32 * 128 + wr_off;
      *reinterpret_cast<u32x4_any_t *>(dst) = stage_regs[P][l];
    }
  };
  auto load_step = [&](auto stage_c) {
    load_quarter(stage_c, c0); load_quarter(stage_c, c1); load_quarter(stage_c, c2); load_quarter(stage_c, c3);
    advance_copy();
  };

  i32x8_t W[TN], A[TM];   // the 64-k block being multiplied: weight blocks, row blocks
  auto read_first_frags = [&]() {
#pragma unroll
    for (int j = 0; j < TN; ++j) W[j] = read_w(c0, c0, j);
#pragma unroll
    for (int i = 0; i < TM; ++i) A[i] = read_a(c0, c0, i);
  };

  // Prologue: step 0 through the stages into slot 0, the activation rows of step
  // 1 into slot 1 (its weight rows follow during the first half of step 0, as in
  // the steady state), the weight rows of steps 1 and 2 and the activation rows of
  // step 2 into the stages.  The load side then stands at step 3.
  load_step(c0);           // step 0
  write_quarter(c0, c0); write_quarter(c0, c1); write_quarter(c0, c2); write_quarter(c0, c3);
  load_step(c1);           // step 1
  write_quarter(c1, c0);
  write_quarter(c1, c1);
  load_step(c0);           // step 2
  init_acc();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();
  read_first_frags();
  __builtin_amdgcn_sched_barrier(0);

  unsigned char *const stage_rows = lds_stage + wave * Epi::WAVE_BYTES;

  // One half of a step: the 16 MFMAs of the 64-k block whose fragments sit in W
  // and A, while the fragments of block RKB of slot RSLOT replace them, quarters
  // WQ and WQ + 1 of their register stage go to LDS slot WSLOT and are loaded
  // again for the step the load side stands at.  BARRIER: the workgroup barrier of the step
  // sits behind the first weight block; everything but MFMAs follows it.
  auto half = [&](auto rslot_c, auto rkb_c, auto wslot_c, auto wq_c, auto barrier_c) {
    constexpr int WQ = decltype(wq_c)::value;
    constexpr bool BARRIER = decltype(barrier_c)::value != 0;
    static_assert(TM == TN, "the half below treats row blocks and weight blocks alike");
    // Weight block by weight block, the row blocks up and down in turn: from one
    // product to the next only one operand changes, the left one (the weights)
    // every fourth time.
    if constexpr (BARRIER) {
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[i][0] = mfma_f8_32x32x64(W[0], A[i], acc[i][0]);
      // This wave has read the step's slot for the last time and has finished
      // writing the other slot; after the barrier both hold for every wave.
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      phase_barrier();
    }
    // (program order = the order in which the registers come free)
    const i32x8_t nw0 = read_w(rslot_c, rkb_c, 0);
    const i32x8_t nw1 = read_w(rslot_c, rkb_c, 1);
    const i32x8_t nw2 = read_w(rslot_c, rkb_c, 2);
    i32x8_t na[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) na[i] = read_a(rslot_c, rkb_c, i);   // (the last column runs the row blocks 3..0)
    const i32x8_t nw3 = read_w(rslot_c, rkb_c, 3);
    write_quarter(wslot_c, template_int<WQ>{});
    load_quarter(wslot_c, template_int<WQ>{});
    write_quarter(wslot_c, template_int<WQ + 1>{});
    load_quarter(wslot_c, template_int<WQ + 1>{});
#pragma unroll
    for (int j = BARRIER ? 1 : 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int ii = (j & 1) ? TM - 1 - i : i;
        acc[ii][j] = mfma_f8_32x32x64(W[j], A[ii], acc[ii][j]);
      }
    f8_sched_half<0, BARRIER ? 4 : 0>();
    __builtin_amdgcn_sched_barrier(0);
    W[0] = nw0;
    W[1] = nw1;
    W[2] = nw2;
    W[3] = nw3;
#pragma unroll
    for (int i = 0; i < TM; ++i) A[i] = na[i];
  };

  while (true) {  // one tile per iteration
    // Every tile has an even number of steps, so a tile always starts in slot 0.
    auto step = [&](auto slot_c) {
      constexpr int S = decltype(slot_c)::value;
      const template_int<S ^ 1> other_c;
      // first k-block; the other slot receives the weight rows of the next step,
      // their stage the weight rows of the step the load side stands at
      half(slot_c, c1, other_c, c2, c0);
      // second k-block; behind its barrier this slot receives the activation rows
      // of the step after next, their stage those of the load side's step, and the
      // next step's first fragments are read
      half(other_c, c0, slot_c, c0, c1);
      advance_copy();
    };
    for (int s = 0; s < cp.steps; s += 2) {
      step(c0);
      step(c1);
    }
    // (the lane number is made opaque here: every address the epilogue derives from
    // it would otherwise be worked out once, ahead of the tile loop, and held in
    // registers through the k-loop, which has none to spare)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    tile_epilogue<MODE, false, kQWaves, TM, TN, true, kEpiReserve, true, HAS_BIAS>(
        cp, acc, stage_rows, wm * WTM, wave_col0, lane_e, lds_colscale + scale_buf * kScaleBufFloats,
        lds_rowscale + scale_buf * kPBM, lds_bias + scale_buf * kBiasBufFloats);
    // The load side is within the next tile here (every tile has at least
    // kQMinSteps steps).
    cp = ld;
    if (!cp.valid) break;
    nxt = fetch_tile(next_turn++);
    // (buffers written here were last read a whole tile ago; the copies are older
    // than every load of the coming steps, whose waits therefore cover them)
    scale_buf = scale_buf == 2 ? 0 : scale_buf + 1;          // the tile multiplied next
    copy_colscale(nxt, scale_buf == 2 ? 0 : scale_buf + 1);  // the one after it
    copy_rowscale(nxt, scale_buf == 2 ? 0 : scale_buf + 1);
    copy_bias(nxt, scale_buf == 2 ? 0 : scale_buf + 1);
    init_acc();
    // The last half above already fetched these fragments; reading them again
    // here keeps their registers free during the epilogue.
    read_first_frags();
  }
}

#endif  // DICE_PERSIST_F8

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

// The kernels are thin wrappers: builtins and inline assembly that only exist
// for the device must not appear in a __global__ template's own body, or the
// host pass silently drops its definition.
template <int MODE, bool HAS_BIAS>
__global__ __launch_bounds__(8 * kWave, 1) void gemm_persist_kernel8(PersistBatch batch) {
  gemm_persist_body<MODE, HAS_BIAS, 8>(batch);
}
// Four waves, one per SIMD, each with the whole 512-entry register file.
template <int MODE, bool HAS_BIAS, int BN, bool GATHER, bool W8 = false, bool REFILL = false>
__global__ __launch_bounds__(4 * kWave, 1) void gemm_persist_kernel4(PersistBatch batch) {
  gemm_persist64_body<MODE, HAS_BIAS, BN, GATHER, W8, REFILL>(batch);
}
// The same with the k-loop in assembly (gemm_persist64_asm_body).  The compiler
// allocates from v0..v127 only; v128..v255 and every accumulation register
// belong to the assembly text.
template <int MODE, int BN, bool GATHER, bool REFILL = false>
__global__ __launch_bounds__(4 * kWave, 1) __attribute__((amdgpu_num_vgpr(128)))
void gemm_persist_kernel4a(PersistBatch batch) {
  gemm_persist64_asm_body<MODE, BN, GATHER, REFILL>(batch);
}

#if DICE_PERSIST_F8
// fp8 activations and weights (see gemm_persist_f8_body).
template <int MODE, bool HAS_BIAS, bool REFILL>
__global__ __launch_bounds__(4 * kWave, 1) void gemm_persist_kernel_f8(PersistBatch batch) {
  gemm_persist_f8_body<MODE, HAS_BIAS, REFILL>(batch);
}
#endif

}  // namespace

#if DICE_PERSIST_F8
int persist_cu_count();
bool persist_fits_table(const PersistBatch &b, int mode);

// fp8 activations: single-problem launches of contiguous rows, an even number
// of 128-k steps, both scale tables, bf16 output.
bool persist_f8_supported(const PersistBatch &b, int mode) {
  if (b.n_problems != 1 || persist_cu_count() < kNumXcd) return false;
  const PersistProblem &p = b.prob[0];
  if (!p.a_scale || !p.w_scale || p.a_rows) return false;
  if (p.n_experts < 1 || p.n_experts > kWave) return false;
  if (p.k % 256 != 0 || p.k < 128 * kQMinSteps) return false;
  if (p.n % 8 != 0 || p.lda % 16 != 0 || p.ldc % 8 != 0) return false;  // 16-byte loads and stores
  if (mode == kFc1Swiglu && p.n % (kPBN / 2) != 0) return false;        // gate/up halves share one range check
  if ((size_t)kPBM * p.lda >= (1ull << 31) || (size_t)kPBN * p.k >= (1ull << 31)) return false;
  return true;
}

int launch_grouped_gemm_persist_f8(const PersistBatch &b, int mode, hipStream_t s) {
  if (!persist_f8_supported(b, mode))
    return fail(DICE_ERR_UNSUPPORTED, "fp8 expert GEMM: unsupported shape");
  const int grid = persist_cu_count() / kNumXcd * kNumXcd;
  const bool has_bias = mode != kFc1Swiglu && b.prob[0].bias != nullptr;
  const bool refill = !persist_fits_table(b, mode);
  void (*kern)(PersistBatch) = nullptr;
  if (mode == kFc1Swiglu)
    kern = refill ? gemm_persist_kernel_f8<kFc1Swiglu, false, true> : gemm_persist_kernel_f8<kFc1Swiglu, false, false>;
  else if (mode == kFc1Gelu && has_bias)
    kern = refill ? gemm_persist_kernel_f8<kFc1Gelu, true, true> : gemm_persist_kernel_f8<kFc1Gelu, true, false>;
  else if (mode == kFc1Gelu)
    kern = refill ? gemm_persist_kernel_f8<kFc1Gelu, false, true> : gemm_persist_kernel_f8<kFc1Gelu, false, false>;
  else if (has_bias)
    kern = refill ? gemm_persist_kernel_f8<kFc2, true, true> : gemm_persist_kernel_f8<kFc2, true, false>;
  else
    kern = refill ? gemm_persist_kernel_f8<kFc2, false, true> : gemm_persist_kernel_f8<kFc2, false, false>;
  PersistBatch launch = b;
  launch.band_tiles = persist_band_tiles(mode);
  launch.xcd_split = 1;   // (one problem: the two splits are the same)
  // (a last turn cut along k: only the plain epilogue is linear in k)
  if (mode != kFc2 || grid / kNumXcd < 2 || grid > kPersistSplitSlots || !split_may_apply(b, grid, kPBN))
    launch.split_ws = nullptr;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kQWaves * kWave), 0, s, launch);
  if (launch.split_ws) launch_split_sum<kPBN>(launch, grid, 128 /* k per step of the fp8 pipeline */, s);
  return launch_status("grouped_gemm_persist_f8");
}

}  // namespace dice
#else  // !DICE_PERSIST_F8
#if DICE_PERSIST_F16
extern int g_persist_waves;
int persist_variant(const PersistBatch &b, int mode);
bool persist_fits_table(const PersistBatch &b, int mode);
int persist_cu_count();
#define DICE_PERSIST_LAUNCH launch_grouped_gemm_persist_f16
namespace {
int cu_count() { return persist_cu_count(); }
}  // namespace
#else
#define DICE_PERSIST_LAUNCH launch_grouped_gemm_persist
int g_persist_waves = 4;  // tuning hook: 4 = 64-k register-staged pipeline first, 8 = 32-k ping-pong pipeline only

namespace {

int cu_count() {
  static thread_local int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess)
      cus = n;
  }
  return cus;
}

// Conditions both pipelines share.
bool persist_common_ok(const PersistBatch &b, int mode) {
  int groups = 0;
  for (int i = 0; i < b.n_problems; ++i) {
    const PersistProblem &p = b.prob[i];
    groups += p.n_experts;
    if (p.k % (kPBK * kPStages) != 0) return false;  // whole trips round the ring per tile
    if (p.n % 8 != 0 || p.lda % 8 != 0 || p.ldc % 8 != 0) return false;
    if (mode == kFc1Swiglu && p.n % (kPBN / 2) != 0) return false;  // gate/up halves share one range check
    if ((size_t)kPBM * p.lda * 2 >= (1ull << 31) || (size_t)kPBN * p.k * 2 >= (1ull << 31)) return false;
  }
  return groups >= 1 && groups <= kWave && cu_count() >= kNumXcd;
}

// Whether every workgroup's turns fit the LDS tile table of the 64-k kernel
// (the last entry stays an invalid tile), bounded from the host-side row
// bounds for either way of sharing the tiles out over the XCDs (the launcher
// picks one later): an eighth of every problem's tiles, or an eighth of the
// total cost - which, for an XCD that gets only the shortest tiles, is that
// cost divided by the shortest tile's.  Launches that do not fit take the
// table-rewriting kernels.
int64_t persist64_turn_bound(const PersistBatch &b, int mode, int wgs_per_xcd) {
  int64_t tiles_per_xcd = 0, total_cost = 0, min_k32 = 1 << 30;
  for (int i = 0; i < b.n_problems; ++i) {
    const PersistProblem &p = b.prob[i];
    const int bn_out = mode == kFc1Swiglu ? kPBN / 2 : (p.n % 192 == 0 && p.n % 256 != 0 ? 192 : kPBN);
    const int64_t m_tiles = ((int64_t)p.max_rows + kPBM - 1) / kPBM + p.n_experts;
    const int64_t n_tiles = (p.n + bn_out - 1) / bn_out;
    tiles_per_xcd += m_tiles * n_tiles / kNumXcd + 1;
    total_cost += m_tiles * n_tiles * (p.k / 32);
    min_k32 = std::min<int64_t>(min_k32, std::max(1, p.k / 32));
  }
  const int64_t by_cost = total_cost / kNumXcd / min_k32 + 2;
  const int64_t run = std::max(tiles_per_xcd, by_cost);
  return (run + wgs_per_xcd - 1) / wgs_per_xcd + 2;
}
bool persist64_fits_table(const PersistBatch &b, int mode) {
  return persist64_turn_bound(b, mode, cu_count() / kNumXcd) <= kTableTurns;
}

// 64-k kernel: long enough tiles.
bool persist64_ok(const PersistBatch &b, int mode) {
  for (int i = 0; i < b.n_problems; ++i) {
    const PersistProblem &p = b.prob[i];
    if (p.a_scale) return false;  // fp8 activations: the kernel of the fp8 compilation unit
    if (p.k < kQBK * kQMinSteps) return false;
    if (p.w_scale && b.n_problems != 1) return false;  // fp8 weights: single-problem launches
    if (p.a_rows) {  // gathered activation rows: SwiGLU instantiation only (the GELU one would
                     // spill, and measures no faster than a gathered copy plus the plain kernel)
      if (mode != kFc1Swiglu) return false;
      if (p.a_div < 1 || p.a_div > 16 || (int64_t)p.a_src_rows * p.a_div >= (1ll << 28)) return false;
      if ((size_t)p.a_src_rows * p.lda * 2 >= (1ull << 31)) return false;
    }
  }
  return true;
}

// 0: neither pipeline applies; 4: the 64-k four-wave kernel; 8: the 32-k eight-wave kernel.
}  // namespace
int persist_cu_count() { return cu_count(); }
bool persist_fits_table(const PersistBatch &b, int mode) { return persist64_fits_table(b, mode); }
// 0: neither pipeline takes the launch; 4 / 8: the waves of the one that does.
int persist_variant(const PersistBatch &b, int mode) {
  if (!persist_common_ok(b, mode)) return 0;
  if (g_persist_waves == 4 && persist64_ok(b, mode)) return 4;
  for (int i = 0; i < b.n_problems; ++i)
    if (b.prob[i].a_rows || b.prob[i].w_scale || b.prob[i].a_scale) return 0;  // the 32-k kernel wants contiguous rows and bf16 operands
  return 8;
}

bool persist_supported(const PersistBatch &b, int mode) { return persist_variant(b, mode) != 0; }
size_t persist_split_ws_bytes() { return (size_t)kPersistSplitSlots * kPBM * kPBN * 2; }
}  // namespace dice
extern "C" int dice_debug_persist_turns(int n_problems, const int64_t *max_rows, const int32_t *n_experts,
                                        const int32_t *n, const int32_t *k, int fc2, int wgs_per_xcd,
                                        int xcd_split, int64_t *bound_out, int64_t *turns_out) {
  using namespace dice;
  if (n_problems < 1 || n_problems > kMaxPersistProblems || !max_rows || !n_experts || !n || !k || !bound_out ||
      !turns_out || wgs_per_xcd < 1)
    return fail(DICE_ERR_BAD_ARG, "dice_debug_persist_turns: bad argument");
  PersistBatch b{};
  b.n_problems = n_problems;
  for (int i = 0; i < n_problems; ++i) {
    b.prob[i].max_rows = (int)max_rows[i];
    b.prob[i].n_experts = n_experts[i];
    b.prob[i].n = n[i];
    b.prob[i].k = k[i];
  }
  const int mode = fc2 ? kFc2 : kFc1Swiglu;
  *bound_out = persist64_turn_bound(b, mode, wgs_per_xcd);
  *turns_out = worst_case_turns(b.prob, n_problems, kPBN / 2, fc2 != 0, wgs_per_xcd, xcd_split);
  return DICE_OK;
}
namespace dice {
#endif  // !DICE_PERSIST_F16

namespace {
typedef void (*PersistKernel)(PersistBatch);
// The 64-k kernel for one tile shape: bf16/fp16 or fp8 weights, with or without
// the rewriting of the tile table.
template <int MODE, bool HAS_BIAS, int BN, bool GATHER>
PersistKernel pick64(bool w8, bool refill) {
  if (w8)
    return refill ? gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, true, true>
                  : gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, true, false>;
  if constexpr (persist64_asm_applies<MODE, HAS_BIAS, BN, GATHER, false>())
    return refill ? gemm_persist_kernel4a<MODE, BN, GATHER, true> : gemm_persist_kernel4a<MODE, BN, GATHER, false>;
  else
  return refill ? gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, false, true>
                : gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, false, false>;
}
}  // namespace

int DICE_PERSIST_LAUNCH(const PersistBatch &b, int mode, hipStream_t s) {
  const int waves = persist_variant(b, mode);
  if (waves == 0) return fail(DICE_ERR_UNSUPPORTED, "persistent expert GEMM: unsupported shape");
  const int grid = cu_count() / kNumXcd * kNumXcd;
  bool has_bias = false;
  for (int i = 0; i < b.n_problems; ++i) has_bias = has_bias || b.prob[i].bias != nullptr;
  if (mode == kFc1Swiglu) has_bias = false;
  void (*kern)(PersistBatch) = nullptr;
  bool gathered = false;
  for (int i = 0; i < b.n_problems; ++i) gathered = gathered || b.prob[i].a_rows != nullptr;
  // 192-row weight tiles where they avoid padded columns (n = 1152 = 6 x 192).
  bool narrow = mode != kFc1Swiglu;
  for (int i = 0; i < b.n_problems; ++i)
    narrow = narrow && b.prob[i].n % 192 == 0 && b.prob[i].n % 256 != 0;
  const bool w8 = b.prob[0].w_scale != nullptr;
  if (narrow && waves == 4) {
    // ... unless the 256-row tiles, padded columns and all, spare the launch a whole turn:
    // the model's longest workgroup with them at most 0.7 of that with the narrow
    // ones (a narrow tile's step takes about 0.8 of a wide one's).  DiT-XL width, 8
    // experts: 4096 and 4608 tokens, 347 -> 339 us per layer call at 4096; at 8192
    // the wide tiles cost +4.7 %.
    const int64_t m192 = persist_plan(b, 192, grid, mode == kFc2).makespan;
    const int64_t m256 = persist_plan(b, kPBN, grid, mode == kFc2).makespan;
    if (m256 * 10 <= m192 * 7) narrow = false;
  }
  if (waves == 4) {
    const bool refill = !persist_fits_table(b, mode);
    if (mode == kFc1Swiglu)
      kern = gathered ? pick64<kFc1Swiglu, false, 256, true>(w8, refill) : pick64<kFc1Swiglu, false, 256, false>(w8, refill);
    else if (mode == kFc1Gelu && narrow)
      kern = has_bias ? pick64<kFc1Gelu, true, 192, false>(w8, refill) : pick64<kFc1Gelu, false, 192, false>(w8, refill);
    else if (mode == kFc1Gelu)
      kern = has_bias ? pick64<kFc1Gelu, true, 256, false>(w8, refill) : pick64<kFc1Gelu, false, 256, false>(w8, refill);
    else if (narrow)
      kern = has_bias ? pick64<kFc2, true, 192, false>(w8, refill) : pick64<kFc2, false, 192, false>(w8, refill);
    else
      kern = has_bias ? pick64<kFc2, true, 256, false>(w8, refill) : pick64<kFc2, false, 256, false>(w8, refill);
  } else {
    switch (mode) {
      case kFc1Swiglu: kern = gemm_persist_kernel8<kFc1Swiglu, false>; break;
      case kFc1Gelu: kern = has_bias ? gemm_persist_kernel8<kFc1Gelu, true> : gemm_persist_kernel8<kFc1Gelu, false>; break;
      default: kern = has_bias ? gemm_persist_kernel8<kFc2, true> : gemm_persist_kernel8<kFc2, false>; break;
    }
  }
  const int slot = (mode * 2 + (has_bias ? 1 : 0)) * 2 + (waves == 4 ? 1 : 0);
  // The 32-k kernel takes its 160 KB of LDS as dynamic memory (which needs the
  // attribute once per kernel); the 64-k kernel declares its LDS statically.
  const size_t dyn_lds = waves == 4 ? 0 : kPLdsBytes;
  static thread_local bool configured[12] = {};
  if (dyn_lds != 0 && !configured[slot]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kPLdsBytes);
    if (e != hipSuccess)
      return fail(DICE_ERR_LAUNCH, "persistent expert GEMM: LDS attribute: %s", hipGetErrorString(e));
    configured[slot] = true;
  }
  PersistBatch launch = b;
  launch.band_tiles = persist_band_tiles(mode);
  const PersistPlan plan = persist_plan(b, mode == kFc1Swiglu ? kPBN / 2 : narrow ? 192 : kPBN, grid, mode == kFc2);
  if (plan.longest_first)
    std::stable_sort(launch.prob, launch.prob + launch.n_problems,
                     [](const PersistProblem &x, const PersistProblem &y) { return x.k > y.k; });
  launch.xcd_split = plan.xcd_split;
  // (a last turn cut along k: the plain epilogue is linear in k; the 32-k kernel
  // does not read its tiles from the table that describes the pieces)
  if (mode != kFc2 || waves != 4 || b.n_problems != 1 || grid / kNumXcd < 2 || grid > kPersistSplitSlots ||
      !split_may_apply(b, grid, narrow ? 192 : kPBN))
    launch.split_ws = nullptr;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * kWave), dyn_lds, s, launch);
  if (launch.split_ws) {
    if (narrow) launch_split_sum<192>(launch, grid, kQBK, s);
    else launch_split_sum<kPBN>(launch, grid, kQBK, s);
  }
  return launch_status("grouped_gemm_persist");
}

}  // namespace dice
#endif  // !DICE_PERSIST_F8
