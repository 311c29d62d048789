// The persistent expert GEMM with fp8 (e4m3) activations AND weights (bf16
// output): its own kernel body on the fp8 MFMA; the tile order, the tile table,
// the epilogue and the cut last turn are those of the 16-bit kernels
// (persist_core.h).
#include "persist_core.h"

namespace dice {
namespace {

// ---------------------------------------------------------------------------
// fp8 x fp8 pipeline, four waves: e4m3 activations (one fp32 scale per row) times
// e4m3 weights (one fp32 scale per output channel) on v_mfma_f32_32x32x64_f8f6f4,
// which multiplies at twice the rate of the bf16 instruction.
//
// In bytes this is the 64-k pipeline of grouped_gemm_persist.hip: rows of 128
// bytes per step (now 128 k), two 64 KB LDS slots, operands staged through two
// register stages four steps ahead, the same 256x256 tile, wave tile, epilogue
// and tile table - so the bytes moved per matrix-pipe cycle are those of the bf16
// kernel while every byte carries twice the arithmetic.  What differs:
//
//   * A fragment of the fp8 instruction is 32 bytes per lane (two 16-byte LDS
//     reads).  The hardware lets lanes 0-31 and 32-63 each hold 32 k of a row;
//     any assignment of k to (lane half, byte) works as long as both operands
//     use the same one, here: half h of k-block kb takes the row's 16-byte
//     chunks 4 kb + 2 h and 4 kb + 2 h + 1.
//   * Fragments twice the size do not fit twice in the register file, so they
//     are not double-buffered.  A step is two k-blocks of 64, each taken weight
//     block by weight block with the row blocks up and down in turn (only one
//     operand changes from one product to the next); the next k-block's
//     fragments are read into the registers of operands as they die: weight
//     block j behind the last product that uses it, the row blocks one by one
//     during the last weight block.  The second k-block runs the rows the other
//     way round, so that the fragment read last is the one needed last.
//   * The workgroup barrier of a step sits one weight block into its second
//     k-block: by then every wave has read the step's slot for the last time and
//     has finished writing the other slot; behind it this slot receives the first
//     quarter of the step after next and the next step's first fragments are
//     read from the other slot.
//   * The epilogue multiplies the fp32 sums by the row's and the column's scale
//     and adds the bias (all three staged in LDS a tile ahead).
//
// The k-loop is generated assembly (persist64_asm.inc, kinds 2 and 3 of
// gen_persist64_asm.py), as for the two hot 16-bit shapes
// (gemm_persist64_asm_body in grouped_gemm_persist.hip): the sums on fixed
// accumulation registers, the eight fragments in v0..v63, the register stages
// in v128..v255 (named in the text only; the kernel is compiled with a budget of
// 128 vector registers).  A group's last tile multiplies only its live 64-row
// blocks (with 1024 +- 31 rows per expert every other group ends in an almost
// empty tile); the two waves that share a tile's columns take alternate 32-row
// blocks, so both have work in every live block.  Left to the compiler, a
// second copy of the loop spills 430-860 registers per instantiation, and even
// the single loop had to give up a register stage to fit.
//
// Rows are contiguous (the quantiser writes the activations in grouped order),
// the reduction length is a multiple of 256 (an even number of steps), weight
// tiles are 256 whole rows (SwiGLU: 128 gate + 128 up; the weight loads carry
// their row in the scalar offset, which the range check does not see),
// single-problem launches.
//
// BLK = 1 (fc1): the output goes out as e4m3 bytes with one power-of-two scale
// per row and 32 columns (tile_epilogue_blockq) - the quantiser of h fused into
// the epilogue.  BLK = 2 (fc2): the activations are such bytes; the products run
// on the scaled form of the instruction, which multiplies each lane's 32 k of the
// activation operand by a scale byte (generator kind 7: a step's scales travel
// through the register stage and 1 KB of LDS per slot like the operands
// themselves).  The hardware applies the byte of a lane in 0-31 to the first 16
// bytes of that row's operand in BOTH lane halves and the byte of the lane 32 on
// to the second 16 bytes, so here a lane half holds the 16-byte chunks
// 4 kb + h and 4 kb + 2 + h of a row and supplies the scale of the row's 32 k
// at 64 kb + 32 h.  There is no row scale then.
template <int MODE, bool HAS_BIAS, bool REFILL, int BLK = 0>
__device__ __forceinline__ void gemm_persist_f8_asm_body(const PersistBatch &batch) {
  constexpr bool SWIGLU = MODE == kFc1Swiglu;
  static_assert(!(SWIGLU && HAS_BIAS), "the SwiGLU expert has no bias");
  static_assert(BLK == 0 || (BLK == 1 && MODE != kFc2) || (BLK == 2 && MODE == kFc2), "block scales: h only");
  constexpr int KIND = BLK == 2 ? 7 : SWIGLU ? 2 : 3;
  constexpr int BN_OUT = SWIGLU ? kPBN / 2 : kPBN;
  constexpr int TM = 4, TN = 4;
  constexpr int kFBK = 128;
  constexpr int kScaleBufFloats = 256, kBiasBufFloats = 256;
  constexpr int kTableBytes = kTableTurns * kTileWords * 4;
  constexpr int kColScaleBytes = 3 * kScaleBufFloats * 4, kRowScaleBytes = 3 * kPBM * 4;
  constexpr int kBiasBytes = HAS_BIAS ? 3 * kBiasBufFloats * 4 : 0;
  constexpr int kEpiReserve = kTableBytes + kColScaleBytes + kRowScaleBytes + kBiasBytes;
  using Epi = EpiGeom<MODE, kQWaves, TM, TN, kEpiReserve>;
  static_assert(kQWaves * Epi::WAVE_BYTES + kEpiReserve <= kPStageArea, "no room beside the epilogue's staging rows");
  typedef __attribute__((address_space(3))) unsigned char lds_byte_t;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot0[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_slot1[kQSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_stage[kPStageArea];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  fixed_acc_declare();

  uint32_t *const tile_table = reinterpret_cast<uint32_t *>(lds_stage + kPStageArea - kTableBytes);
  float *const lds_colscale = reinterpret_cast<float *>(lds_stage + kPStageArea - kTableBytes - kColScaleBytes);
  float *const lds_rowscale =
      reinterpret_cast<float *>(lds_stage + kPStageArea - kTableBytes - kColScaleBytes - kRowScaleBytes);
  float *const lds_bias = reinterpret_cast<float *>(lds_stage + kPStageArea - kEpiReserve);
  // (BLK = 2: the row scales' area holds the two slots' block scales instead, 256 rows x 4 bytes each)
  static_assert(kRowScaleBytes >= 2 * 1024, "block scales of two slots");
  if constexpr (BLK == 2) asm volatile("v_mov_b32 v127, 0x7f7f7f7f");   // the weights' scale: 1.0 in every byte
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
    int lane_c = lane;   // (opaque: worked out at the tile switch, not held through the k-loop)
    asm volatile("" : "+v"(lane_c));
    return PackedTile{tile_table[(turn & (kTableTurns - 1)) * kTileWords + (lane_c < kTileWords ? lane_c : 0)]};
  };

  // ---- what the first wave stages in LDS a tile ahead (one global->LDS
  // instruction each, as text: see lds_dma_x4_text): column scales, row scales, bias ----
  auto desc = [](const void *base, uint32_t bytes) {
    const uint64_t p = (uint64_t)base;
    return u32x4_t{uni((uint32_t)p), uni((uint32_t)(p >> 32) & 0xffffu), uni(bytes), kRsrcFlags};
  };
  auto stage_copy = [&](u32x4_t rs, const float *dst, uint32_t voff) {
    lds_dma_x4_text(rs, (uint32_t)(size_t)(lds_byte_t *)dst, voff);
  };
  auto copy_colscale = [&](const PackedTile &pk, int buf) {
    const uint32_t row = (uint32_t)__builtin_amdgcn_readlane(pk.words, 22);
    const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
    if (wave == 0) {
      int lane_c = lane;
      asm volatile("" : "+v"(lane_c));
      // SwiGLU: 128 gate scales, then the 128 up scales up_offset rows further on;
      // otherwise the tile's columns, those past the matrix reading as 0
      const uint32_t bytes = SWIGLU ? (uint32_t)(batch.prob[0].up_offset + 128) * 4 : (uint32_t)(n - n0) * 4;
      const uint32_t voff =
          SWIGLU && lane_c >= 32 ? (uint32_t)batch.prob[0].up_offset * 4 + (lane_c - 32) * 16 : lane_c * 16;
      stage_copy(desc(batch.prob[0].w_scale + row, bytes), lds_colscale + buf * kScaleBufFloats, voff);
    }
  };
  auto copy_rowscale = [&](const PackedTile &pk, int buf) {
    const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 21) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane(pk.words, 20);
    const int rows = __builtin_amdgcn_readlane(pk.words, 23);
    if (BLK != 2 && wave == 0 && ptr != 0) {
      int lane_c = lane;
      asm volatile("" : "+v"(lane_c));
      // rows past the group's end read as 0 (their products are never stored)
      stage_copy(desc((const void *)ptr, (uint32_t)rows * 4), lds_rowscale + buf * kPBM, lane_c * 16);
    }
  };
  auto copy_bias = [&](const PackedTile &pk, int buf) {
    if constexpr (HAS_BIAS) {
      const uint64_t ptr = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(pk.words, 9) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(pk.words, 8);
      const int n0 = __builtin_amdgcn_readlane(pk.words, 16), n = __builtin_amdgcn_readlane(pk.words, 17);
      if (wave == 0) {
        int lane_c = lane;
        asm volatile("" : "+v"(lane_c));
        // A tile without a bias (the later pieces of a tile that is cut along k)
        // gets zeros: a descriptor that covers no bytes.
        stage_copy(desc(ptr != 0 ? (const void *)(ptr + (uint64_t)n0 * 4) : (const void *)batch.prob[0].w_scale,
                        ptr != 0 ? (uint32_t)(n - n0) * 4 : 0u),
                   lds_bias + buf * kBiasBufFloats, lane_c * 16);
      }
    }
  };

  // ---- addresses the assembly takes (see P64Addr; index kk = 2 kb + t: 16-byte
  // half t of the lane's 32 bytes of k-block kb) ----
  const int cp_row0 = wave * 8 + (lane >> 3), cp_chunk = lane & 7;
  const int b_row0 = SWIGLU ? wn * 64 : wn * 128;
  const uint32_t slot_base[2] = {(uint32_t)(size_t)(lds_byte_t *)lds_slot0, (uint32_t)(size_t)(lds_byte_t *)lds_slot1};
  P64Addr ad;
  // Three of the LDS addresses are kept; the others follow from them at the
  // start of every tile (chunk 4 kb + 2 h + t of a row is chunk 2 h with bits 2
  // and 0 flipped; slot 1 lies a constant behind slot 0).
  uint32_t wr0 = slot_base[0] + qring_off(cp_row0, cp_chunk);
  // (BLK = 2: the scaled instruction fixes the assignment - it multiplies the first 16 bytes of every lane by
  // the scale that lanes 0-31 supply and the second 16 by the one of lanes 32-63, so a scale's 32 k must be
  // the same 16-byte part of both lane halves: part t of half h is the row's chunk 4 kb + 2 t + h)
  const int half_chunk = BLK == 2 ? (lane >> 5) : (lane >> 5) * 2;
  uint32_t ra0 = slot_base[0] + qring_off(wm * 32 + (lane & 31), half_chunk);
  uint32_t rb0 = slot_base[0] + kPBM * 128 + qring_off(b_row0 + (lane & 31), half_chunk);
  static_assert((kQSlotBytes & 1023) == 0, "the xor below must stay inside the chunk field");
  auto set_lds_addresses = [&]() {
    asm volatile("" : "+v"(wr0), "+v"(ra0), "+v"(rb0));
    const uint32_t slot1 = slot_base[1] - slot_base[0];
    ad.wr[0] = wr0;
    ad.wr[1] = wr0 + slot1;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const uint32_t flip = (uint32_t)((kb * 4 + (BLK == 2 ? 2 * t : t)) << 4);
        ad.ra[0][kb * 2 + t] = ra0 ^ flip;
        ad.rb[0][kb * 2 + t] = rb0 ^ flip;
        ad.ra[1][kb * 2 + t] = (ra0 ^ flip) + slot1;
        ad.rb[1][kb * 2 + t] = (rb0 ^ flip) + slot1;
      }
  };
  set_lds_addresses();
#pragma unroll
  for (int i = 0; i < 8; ++i) ad.va[i] = 0;
  ad.vb = 0;
  uint32_t sb_row[8] = {}, sb[8] = {};   // scalar offsets of the weight loads: row part, and with the step's k offset
  u32x4_t dA, dB0, dB1;
  // (BLK = 2) block scales: a step's are one dword per row, the next step's max_rows dwords on; this lane loads
  // those of tile row 64 wave + lane
  const uint32_t scale_step = (uint32_t)batch.prob[0].max_rows * 4u;
  const uint32_t scale_lds = (uint32_t)(size_t)(lds_byte_t *)lds_rowscale;
  P64ScaleAddr sa;
  sa.vs = 0;
  sa.wrs = scale_lds + (uint32_t)(wave * 64 + lane) * 4;
  sa.rs = scale_lds + (uint32_t)(wm * 32 + (lane & 31)) * 4 + (uint32_t)(lane >> 5) * 2;
  u32x4_t dS = {};
  uint32_t kso = 0;
  auto set_copy_offsets = [&](const Tile &t) {
    dA = desc(t.a, t.a_bytes);
    if constexpr (BLK == 2) {
      // (a raw buffer's range check counts the scalar offset - the step - in: the extent covers every step, and
      // a row past the group's end gets an offset that no extent covers, so its scales read as 0 like its bytes)
      dS = desc(t.a_rows, (uint32_t)t.steps * scale_step);
      int srow = wave * 64 + lane;
      asm volatile("" : "+v"(srow));
      sa.vs = srow < t.rows ? (uint32_t)srow * 4u : kOutOfRange;
    }
    dB0 = desc(t.b0, t.b_bytes);
    dB1 = desc(t.b1, t.b_bytes);
    int row0 = cp_row0;   // (opaque, as the lane above)
    asm volatile("" : "+v"(row0));
    const uint32_t voff_a = (uint32_t)row0 * t.a_pitch + cp_chunk * 16;
    // (a row past the tile's end lies past the descriptor's extent and reads as zero)
#pragma unroll
    for (int i = 0; i < 8; ++i) ad.va[i] = voff_a + (uint32_t)(32 * i) * t.a_pitch;
    ad.vb = (uint32_t)row0 * t.b_pitch + cp_chunk * 16;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (SWIGLU && 32 * i >= kPBN / 2) ? 32 * i - kPBN / 2 : 32 * i;   // (the up half has its own descriptor)
      sb_row[i] = uni((uint32_t)row * t.b_pitch);
    }
  };

#define DICE_F8_STEP(name, live)                                     \
  do {                                                               \
    if constexpr (BLK == 2) p64s_##name<KIND, live>(P64S_ARGS);      \
    else p64_##name<KIND, live>(P64_ARGS);                           \
  } while (0)
  // ---- pipeline state ----
  int next_turn = 0;
  PackedTile nxt = fetch_tile(next_turn++);
  Tile ld = unpack_tile(nxt);
  if (!ld.valid) return;
  int scale_buf = 0;                              // buffer of the scales and the bias of the tile being multiplied
  copy_colscale(nxt, 0);
  copy_rowscale(nxt, 0);
  copy_bias(nxt, 0);
  pwait_vmcnt<0>();
  phase_barrier();
  Tile cp = ld;
  int ld_kt = 0;
  set_copy_offsets(ld);
  nxt = fetch_tile(next_turn++);
  copy_colscale(nxt, 1);
  copy_rowscale(nxt, 1);
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
    koff = uni((uint32_t)ld_kt * (uint32_t)kFBK);
    if constexpr (BLK == 2) kso = uni((uint32_t)ld_kt * scale_step);
#pragma unroll
    for (int i = 0; i < 8; ++i) sb[i] = uni(sb_row[i] + koff);
  };
  {
    // (the prologue reads and writes no fragments; they are values of a tile's
    // k-loop only, so that their registers are free for the epilogue)
    f32x32_t f0, f1;
    asm volatile("" : "={v[0:31]}"(f0), "={v[32:63]}"(f1));
    // Prologue: steps 0 and 1 through the stages into the slots (of step 1 only the
    // first quarter), steps 2 and 3 (first quarter) into the stages behind them.
    DICE_F8_STEP(load_step0, 4);
    advance_copy();
    DICE_F8_STEP(load_step1, 4);
    advance_copy();
    DICE_F8_STEP(write_step0, 4);
    DICE_F8_STEP(load_step0, 4);
    advance_copy();
    DICE_F8_STEP(write_q0_stage1, 4);
    DICE_F8_STEP(load_q0_stage1, 4);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  phase_barrier();

  unsigned char *const stage_rows = lds_stage + wave * Epi::WAVE_BYTES;
  f32x16_t no_acc[TM][TN];
  const int wave_col0 = SWIGLU ? wn * 64 : wn * 128;

  // The steps of a tile whose rows fill its first LIVE 64-row blocks.
  auto run_tile = [&](auto live_c) {
    constexpr int LIVE = decltype(live_c)::value;
    f32x32_t f0, f1;   // the fragments: live inside the tile's k-loop only
    asm volatile("" : "={v[0:31]}"(f0), "={v[32:63]}"(f1));
    set_lds_addresses();
    DICE_F8_STEP(read_first, LIVE);
    DICE_F8_STEP(abc_s0_v1, LIVE);   // the first k-block's products start the sums
    advance_copy();
    DICE_F8_STEP(d_s0, LIVE);
    DICE_F8_STEP(abc_s1_v0, LIVE);
    advance_copy();
    DICE_F8_STEP(d_s1, LIVE);
    for (int s = 2; s < cp.steps; s += 2) {
      DICE_F8_STEP(abc_s0_v0, LIVE);
      advance_copy();
      DICE_F8_STEP(d_s0, LIVE);
      DICE_F8_STEP(abc_s1_v0, LIVE);
      advance_copy();
      DICE_F8_STEP(d_s1, LIVE);
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
    if constexpr (BLK == 1) {
      // the tile's first row of block scales (its rows and the scales' are in the same, grouped order)
      const PersistProblem &pr = batch.prob[0];
      const uint32_t tile_row0 = uni((uint32_t)(cp.c - (const unsigned char *)pr.c) / cp.c_pitch);
      tile_epilogue_blockq<MODE, kQWaves, TM, TN, HAS_BIAS, 64, kEpiReserve>(
          cp, lds_stage + wave * BlockqGeom<MODE, kQWaves, TN, kEpiReserve>::WAVE_BYTES, wm * 32, wave_col0, lane_e, lds_colscale + scale_buf * kScaleBufFloats,
          lds_rowscale + scale_buf * kPBM, lds_bias + scale_buf * kBiasBufFloats, live,
          pr.c_block_scale + (size_t)tile_row0 * 4, (uint32_t)pr.max_rows);
    } else {
      tile_epilogue<MODE, false, kQWaves, TM, TN, true, kEpiReserve, BLK != 2, HAS_BIAS, 0, false, 64>(
          cp, no_acc, stage_rows, wm * 32, wave_col0, lane_e, lds_colscale + scale_buf * kScaleBufFloats,
          lds_rowscale + scale_buf * kPBM, lds_bias + scale_buf * kBiasBufFloats, live);
    }
    cp = ld;
    if (!cp.valid) break;
    nxt = fetch_tile(next_turn++);
    // (buffers written here were last read a whole tile ago; the copies are older
    // than every load of the coming steps, whose waits therefore cover them)
    scale_buf = scale_buf == 2 ? 0 : scale_buf + 1;          // the tile multiplied next
    copy_colscale(nxt, scale_buf == 2 ? 0 : scale_buf + 1);  // the one after it
    copy_rowscale(nxt, scale_buf == 2 ? 0 : scale_buf + 1);
    copy_bias(nxt, scale_buf == 2 ? 0 : scale_buf + 1);
  }
#undef DICE_F8_STEP
}

// fp8 activations and weights.  The compiler allocates from v0..v127 only;
// v128..v255 and every accumulation register belong to the assembly text.
template <int MODE, bool HAS_BIAS, bool REFILL, bool BLOCK_OUT = false>
__global__ __launch_bounds__(4 * kWave, 1) __attribute__((amdgpu_num_vgpr(128)))
void gemm_persist_kernel_f8a(PersistBatch batch) {
  gemm_persist_f8_asm_body<MODE, HAS_BIAS, REFILL, BLOCK_OUT ? 1 : 0>(batch);
}
// fc2 on block-scaled activations: v117..v127 too belong to the assembly text
// (the scales' register stage, the scales of the step's row blocks, the weights'
// scale).  The variant that rebuilds its tile table (more than 64 turns per
// workgroup) needs those registers for itself and is not built: the launcher
// refuses such launches.
template <bool HAS_BIAS>
__global__ __launch_bounds__(4 * kWave, 1) __attribute__((amdgpu_num_vgpr(128)))
void gemm_persist_kernel_f8s(PersistBatch batch) {
  gemm_persist_f8_asm_body<kFc2, HAS_BIAS, false, 2>(batch);
}
}  // namespace

int persist_cu_count();
bool persist_fits_table(const PersistBatch &b, int mode);

// fp8 activations: single-problem launches of contiguous rows, an even number
// of 128-k steps, whole weight tiles, both scale tables, bf16 output.
bool persist_f8_supported(const PersistBatch &b, int mode) {
  if (b.n_problems != 1 || persist_cu_count() < kNumXcd) return false;
  const PersistProblem &p = b.prob[0];
  // activations: one scale per row, or (fc2) block scales; block-scaled output: fc1 only
  if ((!p.a_scale == !p.a_block_scale) || !p.w_scale || p.a_rows) return false;
  if (p.a_block_scale && mode != kFc2) return false;
  if (p.c_block_scale && (mode == kFc2 || p.ldc % 16 != 0 || (uint64_t)p.max_rows * p.ldc >= (1ull << 32))) return false;
  if (p.n_experts < 1 || p.n_experts > kWave) return false;
  if (p.k % 256 != 0 || p.k < 128 * kQMinSteps) return false;
  if (p.lda % 16 != 0 || p.ldc % 8 != 0) return false;                  // 16-byte loads and stores
  // whole weight tiles (SwiGLU: its gate and its up half): the weight loads are not range-checked by row
  if (p.n % (mode == kFc1Swiglu ? kPBN / 2 : kPBN) != 0) return false;
  if ((size_t)kPBM * p.lda >= (1ull << 31) || (size_t)kPBN * p.k >= (1ull << 31)) return false;
  return true;
}

int launch_grouped_gemm_persist_f8(const PersistBatch &b, int mode, hipStream_t s) {
  if (!persist_f8_supported(b, mode))
    return fail(DICE_ERR_UNSUPPORTED, "fp8 expert GEMM: unsupported shape");
  const int grid = persist_cu_count() / kNumXcd * kNumXcd;
  const bool has_bias = mode != kFc1Swiglu && b.prob[0].bias != nullptr;
  const bool refill = !persist_fits_table(b, mode);
  if (refill && b.prob[0].a_block_scale)
    return fail(DICE_ERR_UNSUPPORTED, "fp8 expert GEMM on block-scaled activations: more than 64 tiles per workgroup");
  void (*kern)(PersistBatch) = nullptr;
#define DICE_F8_PICK(MODE, BIAS) \
  (refill ? gemm_persist_kernel_f8a<MODE, BIAS, true> : gemm_persist_kernel_f8a<MODE, BIAS, false>)
#define DICE_F8_PICK_OUT(MODE, BIAS) \
  (refill ? gemm_persist_kernel_f8a<MODE, BIAS, true, true> : gemm_persist_kernel_f8a<MODE, BIAS, false, true>)
  if (b.prob[0].a_block_scale)
    kern = has_bias ? gemm_persist_kernel_f8s<true> : gemm_persist_kernel_f8s<false>;
  else if (b.prob[0].c_block_scale)
    kern = mode == kFc1Swiglu ? DICE_F8_PICK_OUT(kFc1Swiglu, false)
           : has_bias         ? DICE_F8_PICK_OUT(kFc1Gelu, true)
                              : DICE_F8_PICK_OUT(kFc1Gelu, false);
  else if (mode == kFc1Swiglu)
    kern = DICE_F8_PICK(kFc1Swiglu, false);
  else if (mode == kFc1Gelu && has_bias)
    kern = DICE_F8_PICK(kFc1Gelu, true);
  else if (mode == kFc1Gelu)
    kern = DICE_F8_PICK(kFc1Gelu, false);
  else if (has_bias)
    kern = DICE_F8_PICK(kFc2, true);
  else
    kern = DICE_F8_PICK(kFc2, false);
#undef DICE_F8_PICK
#undef DICE_F8_PICK_OUT
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
