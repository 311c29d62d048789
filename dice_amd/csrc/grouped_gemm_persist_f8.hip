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

// fp8 activations and weights (see gemm_persist_f8_body).
template <int MODE, bool HAS_BIAS, bool REFILL>
__global__ __launch_bounds__(4 * kWave, 1) void gemm_persist_kernel_f8(PersistBatch batch) {
  gemm_persist_f8_body<MODE, HAS_BIAS, REFILL>(batch);
}
}  // namespace

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
