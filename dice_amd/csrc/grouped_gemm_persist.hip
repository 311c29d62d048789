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
// What these kernels share with the one for fp8 activations
// (grouped_gemm_persist_f8.hip) - tile order, tile table, epilogue, the cut
// last turn - is in persist_core.h.
#include "persist_core.h"

namespace dice {
namespace {

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

template <int MODE, bool HAS_BIAS, int BN, bool GATHER, bool W8>
constexpr bool persist64_asm_applies() {
  return !W8 && ((!HAS_BIAS && MODE == kFc1Swiglu && (BN == 256 || BN == 128) && GATHER) || (!HAS_BIAS && MODE == kFc2 && BN == 192) ||
                 (MODE == kFc2 && BN == 128) || (MODE == kFc1Gelu && BN == 256));
}

// HAS_BIAS (fc2 on 128-row weight tiles and GELU fc1, whose staging rows leave room for it):
// the tile's bias is staged in LDS a tile ahead, as the fp8 kernel does, and added in the epilogue.
template <int MODE, int BN, bool GATHER, bool REFILL, bool HAS_BIAS = false>
__device__ __forceinline__ void gemm_persist64_asm_body(const PersistBatch &batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  constexpr int KIND = SWIGLU ? (BN == 256 ? 0 : 6) : MODE == kFc1Gelu ? 5 : BN == 192 ? 1 : 4;
  static_assert(SWIGLU ? (BN == 256 || BN == 128) : MODE == kFc1Gelu ? BN == 256 : (BN == 192 || BN == 128),
                "the shapes the generator writes");
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
  constexpr int WTN = BN / 2, TM = 4, TN = WTN / 32;
  constexpr int kCopiesA = kPBM / 8 / kQWaves, kCopiesB = BN / 8 / kQWaves;
  constexpr int kAccBlock0 = 16 - TM * TN;
  static_assert(!HAS_BIAS || (BN == 128 && !GATHER) || MODE == kFc1Gelu, "no LDS for a staged bias beside these staging rows");
  constexpr int kTableBytes = kTableTurns * kTileWords * 4, kRowSlotBytes = kPBM * 4;
  // (three bias buffers: the epilogue of a tile reads its bias while the first wave, a little ahead, may already
  // stage that of the tile after the next)
  constexpr int kBiasBufFloats = 256, kBiasBytes = HAS_BIAS ? 3 * kBiasBufFloats * 4 : 0;
  constexpr int kEpiReserve = kTableBytes + (GATHER ? kRowSlotBytes : 0) + kBiasBytes;
  // (what the epilogue's staging rows must leave free: passed on where it decides the height of a band)
  constexpr int kReserveArg = HAS_BIAS || MODE == kFc1Gelu ? kEpiReserve : 0;
  using Epi = EpiGeom<MODE, kQWaves, TM, TN, kReserveArg>;
  typedef __attribute__((address_space(3))) unsigned char lds_byte_t;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot0[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot1[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_stage[kPStageArea];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  fixed_acc_declare();

  static_assert(kQWaves * Epi::WAVE_BYTES + kEpiReserve <= kPStageArea, "no room for the tile table");
  uint32_t *const tile_table = reinterpret_cast<uint32_t *>(lds_stage + kPStageArea - kTableBytes);
  int32_t *const lds_row_slots = reinterpret_cast<int32_t *>(lds_stage + kPStageArea - kTableBytes - kRowSlotBytes);
  float *const lds_bias = reinterpret_cast<float *>(lds_stage + kPStageArea - kEpiReserve);
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
        // (as text, see lds_dma_x4_text; rows past the group's end read as slot 0, a
        // legal row: their products are never stored)
        const u32x4_t rs = {uni((uint32_t)ptr), uni((uint32_t)(ptr >> 32) & 0xffffu), uni((uint32_t)rows * 4u),
                            kRsrcFlags};
        int lane_c = lane;
        asm volatile("" : "+v"(lane_c));
        lds_dma_x4_text(rs, (uint32_t)(size_t)(lds_byte_t *)lds_row_slots, (uint32_t)lane_c * 16u);
      }
    }
  };
  auto copy_bias = [&](const PackedTile &pk, int buf) {
    if constexpr (HAS_BIAS) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 9) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 8);
      const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
      if (wave == 0) {
        // (a problem without a bias gets zeros: a descriptor that covers no bytes)
        const uint64_t src = ptr != 0 ? ptr + (uint64_t)n0 * 4 : (uint64_t)batch.prob[0].w;
        const u32x4_t rs = {uni((uint32_t)src), uni((uint32_t)(src >> 32) & 0xffffu),
                            uni(ptr != 0 ? (uint32_t)(n - n0) * 4u : 0u), kRsrcFlags};
        int lane_c = lane;
        asm volatile("" : "+v"(lane_c));
        lds_dma_x4_text(rs, (uint32_t)(size_t)(lds_byte_t *)(lds_bias + buf * kBiasBufFloats), (uint32_t)lane_c * 16u);
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
  int bias_buf = 0;   // buffer of the bias of the tile being multiplied
  if constexpr (GATHER || HAS_BIAS) {
    copy_row_slots(nxt);
    copy_bias(nxt, 0);
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
  copy_bias(nxt, 1);
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
    tile_epilogue<MODE, false, kQWaves, TM, TN, false, kReserveArg, false, HAS_BIAS, kAccBlock0, false, 64>(
        cp, no_acc, stage_rows, wm * 32, wave_col0, lane_e, nullptr, nullptr, lds_bias + bias_buf * kBiasBufFloats, live);
    cp = ld;
    if (!cp.valid) break;
    nxt = fetch_tile(next_turn++);
    copy_row_slots(nxt);
    // (the buffer written here was last read a whole tile ago; the copy is older than every load of the
    // coming steps, whose waits therefore cover it)
    bias_buf = bias_buf == 2 ? 0 : bias_buf + 1;          // the tile multiplied next
    copy_bias(nxt, bias_buf == 2 ? 0 : bias_buf + 1);     // the one after it
  }
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
template <int MODE, int BN, bool GATHER, bool REFILL = false, bool HAS_BIAS = false>
__global__ __launch_bounds__(4 * kWave, 1) __attribute__((amdgpu_num_vgpr(128)))
void gemm_persist_kernel4a(PersistBatch batch) {
  gemm_persist64_asm_body<MODE, BN, GATHER, REFILL, HAS_BIAS>(batch);
}

}  // namespace

#if DICE_PERSIST_F16
extern int g_persist_waves;
int persist_variant(const PersistBatch &b, int mode);
bool persist_fits_table(const PersistBatch &b, int mode);
bool persist_fits_table_slim(const PersistBatch &b, int mode);
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
    if (p.a_scale || p.a_block_scale || p.c_block_scale) return false;  // fp8 activations: the kernel of the fp8 compilation unit
    if (p.k < kQBK * kQMinSteps) return false;
    if (p.w_scale && b.n_problems != 1) return false;  // fp8 weights: single-problem launches
    if (p.a_rows) {  // gathered activation rows: the fc1 kernels with the generated k-loop (SwiGLU, and GELU on
                     // 256-row tiles of 16-bit weights; left to the compiler the GELU instantiation spilled)
      // (... and launches that fit the tile table: with the table's rewriting as well the instantiation runs out
      // of scalar registers, and the build check refuses where the compiler then parks them)
      if (mode == kFc2 || (mode == kFc1Gelu && (p.w_scale || (p.n % 192 == 0 && p.n % 256 != 0) ||
                                                 !persist64_fits_table(b, mode))))
        return false;
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
// ... with 128-row weight tiles (at most twice the tiles of the bound's widths)
bool persist_fits_table_slim(const PersistBatch &b, int mode) {
  return 2 * persist64_turn_bound(b, mode, cu_count() / kNumXcd) <= kTableTurns;
}
// 0: neither pipeline takes the launch; 4 / 8: the waves of the one that does.
int persist_variant(const PersistBatch &b, int mode) {
  if (!persist_common_ok(b, mode)) return 0;
  if (g_persist_waves == 4 && persist64_ok(b, mode)) return 4;
  for (int i = 0; i < b.n_problems; ++i)
    if (b.prob[i].a_rows || b.prob[i].w_scale || b.prob[i].a_scale || b.prob[i].a_block_scale || b.prob[i].c_block_scale)
      return 0;  // the 32-k kernel wants contiguous rows and bf16 operands
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
  if constexpr (!(MODE == kFc1Gelu && GATHER)) {   // (GELU fc1 gathers only with 16-bit weights: persist64_ok)
    if (w8)
      return refill ? gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, true, true>
                    : gemm_persist_kernel4<MODE, HAS_BIAS, BN, GATHER, true, false>;
  }
  if constexpr (MODE == kFc1Gelu && GATHER)   // (only launches that fit the tile table: persist64_ok)
    return gemm_persist_kernel4a<MODE, BN, GATHER, false, HAS_BIAS>;
  else if constexpr (persist64_asm_applies<MODE, HAS_BIAS, BN, GATHER, false>())
    return refill ? gemm_persist_kernel4a<MODE, BN, GATHER, true, HAS_BIAS> : gemm_persist_kernel4a<MODE, BN, GATHER, false, HAS_BIAS>;
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
  // 128-row weight tiles (fc2, 16-bit weights: the kernel with the generated k-loop).  A step of
  // such a tile takes about 0.75 of a 192-row tile's (two thirds of the products, 12 % more time per product:
  // the wave tile is 128 x 64 and reads 6 fragments for 8 products instead of 7 for 12), so they pay where
  // the finer grain shortens the longest workgroup by more than that: small batches, whose few long tiles
  // otherwise round up to a whole turn.  Tuning hook fc2 = 54 / 55: always / never.
  bool slim = mode == kFc2 && waves == 4 && !w8 && persist_slim_choice(kFc2) >= 0 &&
              persist_fits_table_slim(b, mode);
  for (int i = 0; i < b.n_problems; ++i) slim = slim && b.prob[i].n % 128 == 0;
  // (a single-problem launch with partial-tile slots cuts its last turn along k instead: the better remedy there)
  if (b.n_problems == 1 && b.split_ws != nullptr) slim = false;
  // (a biased 256-row tile starts its sums from the bias, a 128-row tile adds it behind them: the last bit could
  // differ, and with it the result between batch sizes that the model below sends different ways)
  if (has_bias && !narrow) slim = false;
  if (slim && persist_slim_choice(kFc2) == 0) {
    const int64_t m128 = persist_plan(b, 128, grid, true).makespan;
    const int64_t other = persist_plan(b, narrow ? 192 : kPBN, grid, true).makespan;
    // (time per step in units of a 192-row tile's: 128 rows 0.75, 256 rows 1.25)
    slim = m128 * 75 * 100 <= other * (narrow ? 100 : 125) * 93;
  }
  if (slim) narrow = false;
  // (time of a step of a 64-output fc1 tile in per cent of a 128-output tile's)
  constexpr int kSlimFc1StepCost = 60;
  // The same for SwiGLU fc1 with gathered rows: 128 weight rows (64 gate + 64 up: 64 outputs per tile).  Small
  // batches, where a tile is mostly the streaming of its weight rows and a launch two turns of which the second
  // is nearly empty.  Tuning hook fc1 = 54 / 55: always / never.
  bool slim1 = mode == kFc1Swiglu && waves == 4 && !w8 && gathered && persist_slim_choice(kFc1Swiglu) >= 0 &&
               persist_fits_table_slim(b, mode);
  for (int i = 0; i < b.n_problems; ++i) slim1 = slim1 && b.prob[i].n % 64 == 0;
  if (slim1 && persist_slim_choice(kFc1Swiglu) == 0) {
    const int64_t m64 = persist_plan(b, 64, grid, false).makespan;
    const int64_t m128 = persist_plan(b, kPBN / 2, grid, false).makespan;
    slim1 = m64 * kSlimFc1StepCost <= m128 * 93;
  }
  const int width = mode == kFc1Swiglu ? (slim1 ? 64 : kPBN / 2) : slim ? 128 : narrow ? 192 : kPBN;
  if (waves == 4) {
    const bool refill = !persist_fits_table(b, mode);
    if (mode == kFc1Swiglu && slim1)
      kern = gemm_persist_kernel4a<kFc1Swiglu, 128, true, false>;
    else if (mode == kFc1Swiglu)
      kern = gathered ? pick64<kFc1Swiglu, false, 256, true>(w8, refill) : pick64<kFc1Swiglu, false, 256, false>(w8, refill);
    else if (mode == kFc1Gelu && narrow)
      kern = has_bias ? pick64<kFc1Gelu, true, 192, false>(w8, refill) : pick64<kFc1Gelu, false, 192, false>(w8, refill);
    else if (mode == kFc1Gelu && gathered)
      kern = has_bias ? pick64<kFc1Gelu, true, 256, true>(w8, refill) : pick64<kFc1Gelu, false, 256, true>(w8, refill);
    else if (mode == kFc1Gelu)
      kern = has_bias ? pick64<kFc1Gelu, true, 256, false>(w8, refill) : pick64<kFc1Gelu, false, 256, false>(w8, refill);
    else if (slim)
      kern = has_bias ? gemm_persist_kernel4a<kFc2, 128, false, false, true> : gemm_persist_kernel4a<kFc2, 128, false, false>;
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
  const PersistPlan plan = persist_plan(b, width, grid, mode == kFc2);
  if (plan.longest_first)
    std::stable_sort(launch.prob, launch.prob + launch.n_problems,
                     [](const PersistProblem &x, const PersistProblem &y) { return x.k > y.k; });
  launch.xcd_split = plan.xcd_split;
  // (a last turn cut along k: the plain epilogue is linear in k; the 32-k kernel
  // does not read its tiles from the table that describes the pieces)
  if (mode != kFc2 || waves != 4 || slim || b.n_problems != 1 || grid / kNumXcd < 2 || grid > kPersistSplitSlots ||
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
