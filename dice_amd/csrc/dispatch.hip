// Dispatch tables: per-expert histogram, exclusive scan and the stable
// slot permutation, plus the optional row gather.
//
// Replaces argsort + bincount + cumsum of SparseMoeBlock.moe_infer (reference
// models.py:365-367) and of moe_infer_ep (expertpara/ep_fwd.py:70-76,100-106),
// including the slot drop of a skip step (ep_fwd.py:57-66).
//
// Slots are cut into contiguous spans, one per wavefront.  Inside a span a wave
// walks 64 slots per round; lanes that hold the same expert find each other
// with a handful of ballots, so a lane's rank among its peers is a popcount and
// only one lane per expert touches the LDS counter.  The order inside an expert
// group is therefore (span, round, lane) = ascending slot index: stable and
// independent of any atomic's timing.  Integer/byte work, HBM traffic is
// 4 B read + 8 B written per slot.  At the layer's sizes the kernels run for a
// few microseconds and are bound by latency, not by bytes: a wave requests all
// its slots (and its share of the count table) before it looks at any of them,
// nothing branches around a load, and the code is kept short - such a kernel
// spends a good part of its time fetching its own instructions.
#include <mutex>

#include "common.h"

namespace dice {
namespace {

constexpr int kMaxExperts = 256;
constexpr int kFusedWaves = 16;       // single-workgroup path: 1024 threads
constexpr int64_t kFusedMaxSlots = 2048;    // one workgroup, one launch: launch-latency bound sizes
constexpr int kMidRounds = 4;               // two-launch path: 256 slots per wave
constexpr int64_t kMidMaxWork = 1 << 22;    // ... while every wave summing the whole table (units^2 x experts reads) stays
                                            // cheaper than a third launch
constexpr int kTileWaves = 4;         // multi-workgroup path: 256 threads
constexpr int kTileRounds = 8;        // 512 slots per wave

// Bit mask of the lanes of this wave whose (valid) slot names the same expert.
__device__ __forceinline__ uint64_t peers_of(int e, bool valid, int nbits) {
  uint64_t mask = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1;
    const uint64_t bal = __ballot(bit);
    mask &= bit ? bal : ~bal;
  }
  return valid ? mask : 0ull;
}

struct SlotInfo {
  int64_t slot;
  int e;
  bool in_range;  // slot < n_slots
  bool valid;     // in range, not skipped, expert id legal
};

// A wave's span of ROUNDS x 64 slots, every round requested before the first is
// used: one memory round trip for the span instead of one per round.
template <int ROUNDS>
__device__ __forceinline__ void read_span(const int32_t *idx, const uint8_t *skip, int64_t n_slots,
                                          int n_experts, int64_t span_begin, int lane, SlotInfo (&s)[ROUNDS]) {
  // (without a mask a byte of the index array is read and ignored: no branch around a load)
  const uint8_t *mask = skip != nullptr ? skip : reinterpret_cast<const uint8_t *>(idx);
  int e[ROUNDS];
  uint8_t m[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int64_t slot = span_begin + (int64_t)r * kWave + lane;
    const int64_t at = slot < n_slots ? slot : 0;   // slots past the end re-read slot 0
    e[r] = idx[at];
    m[r] = mask[at];
  }
  // every load is on its way before the first value is looked at
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    s[r].slot = span_begin + (int64_t)r * kWave + lane;
    s[r].in_range = s[r].slot < n_slots;
    const bool dropped = (m[r] != 0) & (skip != nullptr);
    s[r].valid = s[r].in_range && !dropped && e[r] >= 0 && e[r] < n_experts;
    s[r].e = s[r].valid ? e[r] : 0;
  }
}

// Adds this wave's per-expert counts over its span into row[] (LDS).
template <int ROUNDS>
__device__ __forceinline__ void count_span(const SlotInfo (&s)[ROUNDS], int nbits, int32_t *row, int lane) {
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const uint64_t m = peers_of(s[r].e, s[r].valid, nbits);
    if (s[r].valid && (__ffsll((unsigned long long)m) - 1) == lane) row[s[r].e] += __popcll(m);
    wave_lds_sync();
  }
}

// Writes perm / inv_perm for this wave's span; row[] holds the next free
// grouped position per expert and is advanced as the span is walked.
template <int ROUNDS>
__device__ __forceinline__ void rank_span(const SlotInfo (&s)[ROUNDS], int nbits, int32_t *row, int lane,
                                          int32_t *perm, int32_t *inv_perm) {
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const uint64_t m = peers_of(s[r].e, s[r].valid, nbits);
    int pos = -1;
    if (s[r].valid) pos = row[s[r].e] + __popcll(m & below);
    wave_lds_sync();
    if (s[r].valid) {
      perm[pos] = (int32_t)s[r].slot;
      if ((__ffsll((unsigned long long)m) - 1) == lane) row[s[r].e] += __popcll(m);
    }
    if (s[r].in_range) inv_perm[s[r].slot] = pos;
    wave_lds_sync();
  }
}

// Single-workgroup path.  Each wave first pulls its whole span into registers
// (MAXR independent loads in flight: one memory latency instead of one per
// round), then counts, then ranks out of those registers.
// Slot codes: expert id >= 0 = live slot, -1 = dropped (skip mask / illegal id),
// -2 = past the end.
template <int MAXR>
__global__ __launch_bounds__(kFusedWaves *kWave) void dispatch_fused_kernel(
    const int32_t *__restrict__ idx, const uint8_t *__restrict__ skip, int64_t n_slots,
    int n_experts, int nbits, int rounds, int32_t *__restrict__ counts,
    int32_t *__restrict__ offsets, int32_t *__restrict__ perm, int32_t *__restrict__ inv_perm,
    int32_t *__restrict__ range_out, int32_t range_n) {
  __shared__ int32_t wrow[kFusedWaves][kMaxExperts];
  if (range_out && threadIdx.x == 0) {
    range_out[0] = 0;
    range_out[1] = range_n;
  }
  __shared__ int32_t eoff[kMaxExperts + 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t span = (int64_t)rounds * kWave;
  const int64_t begin = wave * span;

  int code[MAXR];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) code[r] = -2;
  if (n_slots > 0) {  // (an empty call may come without an index array)
    // No branch around a load (slots past the end re-read slot 0; without a mask a
    // byte of the index array is read and ignored), and every load issued before
    // the first value is looked at.
    const uint8_t *mask = skip != nullptr ? skip : reinterpret_cast<const uint8_t *>(idx);
    int e[MAXR];
    uint8_t m[MAXR];
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int64_t slot = begin + (int64_t)r * kWave + lane;
      const int64_t at = (r < rounds && slot < n_slots) ? slot : 0;
      e[r] = idx[at];
      m[r] = mask[at];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int64_t slot = begin + (int64_t)r * kWave + lane;
      const bool dropped = (m[r] != 0) & (skip != nullptr);
      if (r < rounds && slot < n_slots) code[r] = (!dropped && e[r] >= 0 && e[r] < n_experts) ? e[r] : -1;
    }
  }

  for (int e = lane; e < n_experts; e += kWave) wrow[wave][e] = 0;
  __syncthreads();
  int32_t *row = wrow[wave];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < rounds) {
      const bool valid = code[r] >= 0;
      const int e = valid ? code[r] : 0;
      const uint64_t m = peers_of(e, valid, nbits);
      if (valid && (__ffsll((unsigned long long)m) - 1) == lane) row[e] += __popcll(m);
      wave_lds_sync();
    }
  }
  __syncthreads();

  // Exclusive scan of the per-expert totals by the first wave.
  if (wave == 0) {
    int carry = 0;
    for (int c = 0; c < n_experts; c += kWave) {
      const int e = c + lane;
      int tot = 0;
      if (e < n_experts)
        for (int w = 0; w < kFusedWaves; ++w) tot += wrow[w][e];
      int inc = tot;
#pragma unroll
      for (int o = 1; o < kWave; o <<= 1) {
        int up = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += up;
      }
      if (e < n_experts) {
        eoff[e] = carry + inc - tot;
        counts[e] = tot;
        offsets[e] = carry + inc - tot;
      }
      carry += __shfl(inc, kWave - 1, kWave);
    }
    if (lane == 0) {
      eoff[n_experts] = carry;
      offsets[n_experts] = carry;
    }
  }
  __syncthreads();
  // Turn counts into start positions: expert-major, wave-minor.
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    int base = eoff[e];
    for (int w = 0; w < kFusedWaves; ++w) {
      const int t = wrow[w][e];
      wrow[w][e] = base;
      base += t;
    }
  }
  __syncthreads();
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < rounds) {
      const bool valid = code[r] >= 0;
      const int e = valid ? code[r] : 0;
      const int64_t slot = begin + (int64_t)r * kWave + lane;
      const uint64_t m = peers_of(e, valid, nbits);
      int pos = -1;
      if (valid) pos = row[e] + __popcll(m & below);
      wave_lds_sync();
      if (valid) {
        perm[pos] = (int32_t)slot;
        if ((__ffsll((unsigned long long)m) - 1) == lane) row[e] += __popcll(m);
      }
      if (code[r] != -2) inv_perm[slot] = pos;
      wave_lds_sync();
    }
  }
  const int total = eoff[n_experts];
  for (int64_t i = total + threadIdx.x; i < n_slots; i += blockDim.x) perm[i] = -1;
}

template <int ROUNDS>
__global__ __launch_bounds__(kTileWaves *kWave) void dispatch_count_kernel(
    const int32_t *__restrict__ idx, const uint8_t *__restrict__ skip, int64_t n_slots,
    int n_experts, int nbits, int units, int32_t *__restrict__ unit_cnt) {
  __shared__ int32_t wrow[kTileWaves][kMaxExperts];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int unit = blockIdx.x * kTileWaves + wave;
  SlotInfo span[ROUNDS];
  if (unit < units) read_span<ROUNDS>(idx, skip, n_slots, n_experts, (int64_t)unit * ROUNDS * kWave, lane, span);
  for (int e = lane; e < n_experts; e += kWave) wrow[wave][e] = 0;
  __syncthreads();
  if (unit < units) {
    count_span<ROUNDS>(span, nbits, wrow[wave], lane);
    for (int e = lane; e < n_experts; e += kWave) unit_cnt[(size_t)e * units + unit] = wrow[wave][e];
  }
}

// One workgroup: in-place exclusive scan of unit_cnt in expert-major order,
// plus counts[] and offsets[].
__global__ __launch_bounds__(1024) void dispatch_scan_kernel(int32_t *__restrict__ unit_cnt,
                                                             int n_experts, int units,
                                                             int32_t *__restrict__ counts,
                                                             int32_t *__restrict__ offsets,
                                                             int32_t *__restrict__ range_out,
                                                             int32_t range_n) {
  __shared__ int32_t wave_tot[16];
  if (range_out && threadIdx.x == 0) {
    range_out[0] = 0;
    range_out[1] = range_n;
  }
  __shared__ int32_t eoff[kMaxExperts + 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t total = (int64_t)n_experts * units;
  const int64_t per = (total + 1023) / 1024;
  const int64_t b = (int64_t)threadIdx.x * per;
  const int64_t e_ = b + per < total ? b + per : total;
  int local = 0;
  for (int64_t i = b; i < e_; ++i) local += unit_cnt[i];
  int inc = local;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  if (lane == kWave - 1) wave_tot[wave] = inc;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += wave_tot[w];
  int run = base + inc - local;
  for (int64_t i = b; i < e_; ++i) {
    const int c = unit_cnt[i];
    unit_cnt[i] = run;
    if (i % units == 0) eoff[i / units] = run;
    run += c;
  }
  if (threadIdx.x == 1023) eoff[n_experts] = run;
  __syncthreads();
  for (int e = threadIdx.x; e <= n_experts; e += blockDim.x) {
    offsets[e] = eoff[e];
    if (e < n_experts) counts[e] = eoff[e + 1] - eoff[e];
  }
}

__global__ __launch_bounds__(kTileWaves *kWave) void dispatch_rank_kernel(
    const int32_t *__restrict__ idx, const uint8_t *__restrict__ skip, int64_t n_slots,
    int n_experts, int nbits, int units, const int32_t *__restrict__ unit_base,
    const int32_t *__restrict__ offsets, int32_t *__restrict__ perm,
    int32_t *__restrict__ inv_perm) {
  __shared__ int32_t wrow[kTileWaves][kMaxExperts];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int unit = blockIdx.x * kTileWaves + wave;
  if (unit >= units) return;
  for (int e = lane; e < n_experts; e += kWave) wrow[wave][e] = unit_base[(size_t)e * units + unit];
  wave_lds_sync();
  const int64_t begin = (int64_t)unit * kTileRounds * kWave;
  SlotInfo span[kTileRounds];
  read_span<kTileRounds>(idx, skip, n_slots, n_experts, begin, lane, span);
  rank_span<kTileRounds>(span, nbits, wrow[wave], lane, perm, inv_perm);
  const int total = offsets[n_experts];
  for (int r = 0; r < kTileRounds; ++r) {
    const int64_t i = begin + (int64_t)r * kWave + lane;
    if (i >= total && i < n_slots) perm[i] = -1;
  }
}

// Second kernel of the two-launch path (mid-size inputs): every wave sums the
// unit table itself - totals per expert for the offsets, and the counts of the
// units before its own for its start positions - then ranks its unit.  The
// table is units x experts integers, a few KB, and comes out of the L2.
template <int ROUNDS>
__global__ __launch_bounds__(kTileWaves *kWave) void dispatch_scan_rank_kernel(
    const int32_t *__restrict__ idx, const uint8_t *__restrict__ skip, int64_t n_slots,
    int n_experts, int nbits, int units, const int32_t *__restrict__ unit_cnt,
    int32_t *__restrict__ counts, int32_t *__restrict__ offsets, int32_t *__restrict__ perm,
    int32_t *__restrict__ inv_perm, int32_t *__restrict__ range_out, int32_t range_n) {
  __shared__ int32_t wrow[kTileWaves][kMaxExperts];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int unit = blockIdx.x * kTileWaves + wave;
  if (range_out && blockIdx.x == 0 && threadIdx.x == 0) {
    range_out[0] = 0;
    range_out[1] = range_n;
  }
  if (unit >= units) return;
  // The wave's slots are requested first: they arrive while the table is summed.
  const int64_t begin = (int64_t)unit * ROUNDS * kWave;
  SlotInfo span[ROUNDS];
  read_span<ROUNDS>(idx, skip, n_slots, n_experts, begin, lane, span);
  // per expert: total over all units and total over the units before this one.
  // The lanes read an expert's unit counts side by side (one coalesced load per
  // 64 units), eight experts' rows requested together, and reduce across the
  // wave; lane e % 64 keeps expert e's sums.
  constexpr int kRows = 8;
  int carry = 0;  // running exclusive offset over experts
  for (int c = 0; c < n_experts; c += kWave) {
    const int e = c + lane;
    int tot = 0, before = 0;
    const int chunk_experts = n_experts - c < kWave ? n_experts - c : kWave;
    for (int ee0 = 0; ee0 < chunk_experts; ee0 += kRows) {
      int t[kRows], b[kRows];
#pragma unroll
      for (int k = 0; k < kRows; ++k) t[k] = b[k] = 0;
      for (int u0 = 0; u0 < units; u0 += kWave) {
        const int u = u0 + lane;
        int v[kRows];
#pragma unroll
        for (int k = 0; k < kRows; ++k) {
          const int ee = ee0 + k < chunk_experts ? ee0 + k : chunk_experts - 1;  // (past the chunk: the last row again, unused)
          v[k] = u < units ? unit_cnt[(size_t)(c + ee) * units + u] : 0;
        }
#pragma unroll
        for (int k = 0; k < kRows; ++k) {
          t[k] += v[k];
          b[k] += u < unit ? v[k] : 0;
        }
      }
#pragma unroll
      for (int k = 0; k < kRows; ++k) {
        const int ts = wave_sum_i32(t[k]), bs = wave_sum_i32(b[k]);
        if (lane == ee0 + k && ee0 + k < chunk_experts) {
          tot = ts;
          before = bs;
        }
      }
    }
    int inc = tot;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(inc, o, kWave);
      if (lane >= o) inc += up;
    }
    if (e < n_experts) {
      const int off = carry + inc - tot;
      wrow[wave][e] = off + before;
      if (unit == 0) {
        counts[e] = tot;
        offsets[e] = off;
      }
    }
    carry += __shfl(inc, kWave - 1, kWave);
  }
  if (unit == 0 && lane == 0) offsets[n_experts] = carry;
  wave_lds_sync();
  rank_span<ROUNDS>(span, nbits, wrow[wave], lane, perm, inv_perm);
  const int total = carry;
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int64_t i = begin + (int64_t)r * kWave + lane;
    if (i >= total && i < n_slots) perm[i] = -1;
  }
}

// dispatch_scan_rank_kernel for small tables (at most EMAX experts and 64 UMAX
// units): the wave's slots and its whole share of the table are requested in
// one go, in straight-line code, so the kernel costs one memory round trip
// before it ranks (around a loop the compiler waits for every load in flight).
template <int ROUNDS, int EMAX, int UMAX>
__global__ __launch_bounds__(kTileWaves *kWave) void dispatch_scan_rank_small_kernel(
    const int32_t *__restrict__ idx, const uint8_t *__restrict__ skip, int64_t n_slots,
    int n_experts, int nbits, int units, const int32_t *__restrict__ unit_cnt,
    int32_t *__restrict__ counts, int32_t *__restrict__ offsets, int32_t *__restrict__ perm,
    int32_t *__restrict__ inv_perm, int32_t *__restrict__ range_out, int32_t range_n) {
  static_assert(EMAX <= kWave, "expert e's sums live in lane e");
  __shared__ int32_t wrow[kTileWaves][kMaxExperts];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int unit = blockIdx.x * kTileWaves + wave;
  if (range_out && blockIdx.x == 0 && threadIdx.x == 0) {
    range_out[0] = 0;
    range_out[1] = range_n;
  }
  if (unit >= units) return;
  int v[EMAX][UMAX];
#pragma unroll
  for (int e = 0; e < EMAX; ++e)
#pragma unroll
    for (int j = 0; j < UMAX; ++j) {
      const int u = j * kWave + lane;
      const int row = e < n_experts ? e : n_experts - 1;   // (rows past the table: the last one again, unused)
      v[e][j] = unit_cnt[(size_t)row * units + (u < units ? u : 0)];
    }
  const int64_t begin = (int64_t)unit * ROUNDS * kWave;
  SlotInfo span[ROUNDS];
  read_span<ROUNDS>(idx, skip, n_slots, n_experts, begin, lane, span);
  int tot = 0, before = 0;
#pragma unroll
  for (int e = 0; e < EMAX; ++e) {
    int t = 0, b = 0;
#pragma unroll
    for (int j = 0; j < UMAX; ++j) {
      const int u = j * kWave + lane;
      t += u < units ? v[e][j] : 0;
      b += u < unit ? v[e][j] : 0;
    }
    t = wave_sum_i32(t);
    b = wave_sum_i32(b);
    if (lane == e) {
      tot = t;
      before = b;
    }
  }
  if (lane >= n_experts) tot = before = 0;
  int inc = tot;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int up = __shfl_up(inc, o, kWave);
    if (lane >= o) inc += up;
  }
  const int off = inc - tot;
  if (lane < n_experts) {
    wrow[wave][lane] = off + before;
    if (unit == 0) {
      counts[lane] = tot;
      offsets[lane] = off;
    }
  }
  const int total = __shfl(inc, kWave - 1, kWave);
  if (unit == 0 && lane == 0) offsets[n_experts] = total;
  wave_lds_sync();
  rank_span<ROUNDS>(span, nbits, wrow[wave], lane, perm, inv_perm);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int64_t i = begin + (int64_t)r * kWave + lane;
    if (i >= total && i < n_slots) perm[i] = -1;
  }
}

// `range_out` (optional) receives {0, range_n}: the one-group offset table of
// the shared expert, written here so the layer needs no extra launch for it.
template <typename V>
__global__ __launch_bounds__(256) void gather_rows_kernel(const V *__restrict__ x,
                                                          const int32_t *__restrict__ perm,
                                                          int slots_per_token, int64_t n_rows,
                                                          int vec_per_row, V *__restrict__ out,
                                                          int32_t *__restrict__ range_out,
                                                          int32_t range_n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (range_out && i == 0) {
    range_out[0] = 0;
    range_out[1] = range_n;
  }
  if (i >= n_rows * vec_per_row) return;
  const int64_t r = i / vec_per_row;
  const int c = (int)(i - r * vec_per_row);
  const int slot = perm[r];
  if (slot < 0) return;
  out[i] = x[(int64_t)(slot / slots_per_token) * vec_per_row + c];
}

int bits_for(int n_experts) {
  int nbits = 1;
  while ((1 << nbits) < n_experts) ++nbits;
  return nbits;
}

}  // namespace
}  // namespace dice

extern "C" size_t dice_dispatch_workspace_bytes(int64_t n_slots, int n_experts) {
  using namespace dice;
  if (n_slots <= kFusedMaxSlots || n_experts <= 0) return 256;
  const int64_t mid_units = (n_slots + kMidRounds * kWave - 1) / (kMidRounds * kWave);
  const int64_t units = mid_units * mid_units * n_experts <= kMidMaxWork
                            ? mid_units
                            : (n_slots + kTileRounds * kWave - 1) / (kTileRounds * kWave);
  return align_up((size_t)units * n_experts * sizeof(int32_t), 256);
}

namespace dice {
// `range_out` (optional) receives {0, range_n}: the one-group offset table of
// the shared expert, written here so that the layer needs no extra launch for it.
int dispatch_impl(const int32_t *flat_idx, const uint8_t *skip_mask, int64_t n_slots, int n_experts,
                  int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv_perm, void *workspace,
                  size_t workspace_bytes, int32_t *range_out, int32_t range_n, void *stream) {
  DICE_REQUIRE(counts && offsets && (n_slots == 0 || (flat_idx && perm && inv_perm)),
               DICE_ERR_BAD_ARG, "dice_dispatch: null pointer");
  DICE_REQUIRE(n_experts >= 1 && n_experts <= kMaxExperts, DICE_ERR_UNSUPPORTED,
               "dice_dispatch: n_experts %d outside [1, %d]", n_experts, kMaxExperts);
  DICE_REQUIRE(n_slots >= 0 && n_slots < (1ll << 31), DICE_ERR_BAD_ARG,
               "dice_dispatch: n_slots %lld outside [0, 2^31)", (long long)n_slots);
  hipStream_t s = (hipStream_t)stream;
  const int nbits = bits_for(n_experts);
  if (n_slots <= kFusedMaxSlots) {
    constexpr int kMaxRounds = (int)(kFusedMaxSlots / (kFusedWaves * kWave));
    const int rounds = (int)((n_slots + kFusedWaves * kWave - 1) / (kFusedWaves * kWave));
    hipLaunchKernelGGL(dispatch_fused_kernel<kMaxRounds>, dim3(1), dim3(kFusedWaves * kWave), 0, s, flat_idx,
                       skip_mask, n_slots, n_experts, nbits, rounds, counts, offsets, perm, inv_perm, range_out,
                       range_n);
    return launch_status("dice_dispatch");
  }
  const size_t need = dice_dispatch_workspace_bytes(n_slots, n_experts);
  DICE_REQUIRE(workspace && workspace_bytes >= need, DICE_ERR_WORKSPACE,
               "dice_dispatch: workspace %zu < %zu bytes", workspace_bytes, need);
  int32_t *unit_cnt = (int32_t *)workspace;
  const int64_t mid_units = (n_slots + kMidRounds * kWave - 1) / (kMidRounds * kWave);
  if (mid_units * mid_units * n_experts <= kMidMaxWork) {
    // Mid sizes: per-wave histograms, then one kernel that scans the (small)
    // table in every wave and ranks.
    const int units = (int)mid_units;
    const int blocks = (units + kTileWaves - 1) / kTileWaves;
    hipLaunchKernelGGL(dispatch_count_kernel<kMidRounds>, dim3(blocks), dim3(kTileWaves * kWave), 0, s, flat_idx,
                       skip_mask, n_slots, n_experts, nbits, units, unit_cnt);
    // (the instantiation that just covers the table: these kernels run for a few
    // microseconds, most of them spent fetching their own code)
#define DICE_SCAN_RANK_SMALL(EMAX, UMAX)                                                                      \
  hipLaunchKernelGGL((dispatch_scan_rank_small_kernel<kMidRounds, EMAX, UMAX>), dim3(blocks),                 \
                     dim3(kTileWaves * kWave), 0, s, flat_idx, skip_mask, n_slots, n_experts, nbits, units,   \
                     unit_cnt, counts, offsets, perm, inv_perm, range_out, range_n)
    if (n_experts <= 8 && units <= kWave)
      DICE_SCAN_RANK_SMALL(8, 1);
    else if (n_experts <= 8 && units <= 2 * kWave)
      DICE_SCAN_RANK_SMALL(8, 2);
    else if (n_experts <= 16 && units <= kWave)
      DICE_SCAN_RANK_SMALL(16, 1);
    else if (n_experts <= 16 && units <= 2 * kWave)
      DICE_SCAN_RANK_SMALL(16, 2);
#undef DICE_SCAN_RANK_SMALL
    else
      hipLaunchKernelGGL(dispatch_scan_rank_kernel<kMidRounds>, dim3(blocks), dim3(kTileWaves * kWave), 0, s,
                         flat_idx, skip_mask, n_slots, n_experts, nbits, units, unit_cnt, counts, offsets, perm,
                         inv_perm, range_out, range_n);
    return launch_status("dice_dispatch");
  }
  const int64_t units64 = (n_slots + kTileRounds * kWave - 1) / (kTileRounds * kWave);
  const int units = (int)units64;
  const int blocks = (units + kTileWaves - 1) / kTileWaves;
  hipLaunchKernelGGL(dispatch_count_kernel<kTileRounds>, dim3(blocks), dim3(kTileWaves * kWave), 0, s, flat_idx,
                     skip_mask, n_slots, n_experts, nbits, units, unit_cnt);
  hipLaunchKernelGGL(dispatch_scan_kernel, dim3(1), dim3(1024), 0, s, unit_cnt, n_experts, units,
                     counts, offsets, range_out, range_n);
  hipLaunchKernelGGL(dispatch_rank_kernel, dim3(blocks), dim3(kTileWaves * kWave), 0, s, flat_idx,
                     skip_mask, n_slots, n_experts, nbits, units, unit_cnt, offsets, perm, inv_perm);
  return launch_status("dice_dispatch");
}
}  // namespace dice

extern "C" int dice_dispatch(const int32_t *flat_idx, const uint8_t *skip_mask, int64_t n_slots,
                             int n_experts, int32_t *counts, int32_t *offsets, int32_t *perm,
                             int32_t *inv_perm, void *workspace, size_t workspace_bytes,
                             void *stream) {
  return dice::dispatch_impl(flat_idx, skip_mask, n_slots, n_experts, counts, offsets, perm, inv_perm,
                             workspace, workspace_bytes, nullptr, 0, stream);
}

// dice_dispatch for callers that cannot allocate: the per-span histogram table
// lives in a file-scope device array instead of a caller-provided workspace.
// Every GPU the library runs on holds its own copy of the array at its own
// address; the array's name is only a host-side handle, so the device address
// is looked up once per device and that pointer is what the kernels get.
namespace dice {
namespace {
constexpr size_t kStaticScratchBytes = DICE_DISPATCH_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (NULL + error text on failure).
void *static_scratch(int *rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *rc = fail(DICE_ERR_LAUNCH, "dice_dispatch_static: hipGetDevice: %s (device %d)",
               hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      *rc = fail(DICE_ERR_LAUNCH, "dice_dispatch_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *rc = DICE_OK;
  return g_scratch_ptr[dev];
}
}  // namespace
}  // namespace dice

extern "C" size_t dice_dispatch_static_scratch_bytes(void) { return dice::kStaticScratchBytes; }

extern "C" int dice_dispatch_static(const int32_t *flat_idx, const uint8_t *skip_mask, int64_t n_slots,
                                    int n_experts, int32_t *counts, int32_t *offsets, int32_t *perm,
                                    int32_t *inv_perm, void *stream) {
  using namespace dice;
  DICE_REQUIRE(n_experts >= 1 && n_experts <= kMaxExperts, DICE_ERR_UNSUPPORTED,
               "dice_dispatch_static: n_experts %d outside [1, %d]", n_experts, kMaxExperts);
  DICE_REQUIRE(n_slots >= 0 && n_slots < (1ll << 31), DICE_ERR_BAD_ARG,
               "dice_dispatch_static: n_slots %lld outside [0, 2^31)", (long long)n_slots);
  const size_t need = dice_dispatch_workspace_bytes(n_slots, n_experts);
  DICE_REQUIRE(need <= kStaticScratchBytes, DICE_ERR_WORKSPACE,
               "dice_dispatch_static: %lld slots x %d experts need %zu bytes of scratch, the static array "
               "holds %zu (use dice_dispatch with a workspace)",
               (long long)n_slots, n_experts, need, kStaticScratchBytes);
  int rc = DICE_OK;
  void *ptr = static_scratch(&rc);
  if (!ptr) return rc;
  // Every table entry a launch reads was written by the same call's count
  // kernel, so nothing has to be cleared between calls.
  return dispatch_impl(flat_idx, skip_mask, n_slots, n_experts, counts, offsets, perm, inv_perm, ptr,
                       kStaticScratchBytes, nullptr, 0, stream);
}

namespace dice {
int gather_rows_impl(const void *x, int dtype, const int32_t *perm, int slots_per_token,
                     int64_t n_rows, int hidden, void *out, int32_t *range_out, int32_t range_n,
                     void *stream) {
  DICE_REQUIRE(x && perm && out, DICE_ERR_BAD_ARG, "dice_gather_rows: null pointer");
  DICE_REQUIRE(slots_per_token >= 1, DICE_ERR_BAD_ARG, "dice_gather_rows: slots_per_token %d < 1",
               slots_per_token);
  const size_t es = dtype_size(dtype);
  DICE_REQUIRE(es == 2 || es == 4, DICE_ERR_UNSUPPORTED, "dice_gather_rows: dtype %d", dtype);
  const size_t row_bytes = (size_t)hidden * es;
  DICE_REQUIRE(hidden > 0 && row_bytes % 16 == 0, DICE_ERR_BAD_ARG,
               "dice_gather_rows: row of %zu bytes is not a multiple of 16", row_bytes);
  if (n_rows <= 0) return DICE_OK;
  const int vec_per_row = (int)(row_bytes / 16);
  const int64_t total = n_rows * vec_per_row;
  const int64_t blocks = (total + 255) / 256;
  hipLaunchKernelGGL(gather_rows_kernel<u32x4_t>, dim3((unsigned)blocks), dim3(256), 0,
                     (hipStream_t)stream, (const u32x4_t *)x, perm, slots_per_token, n_rows,
                     vec_per_row, (u32x4_t *)out, range_out, range_n);
  return launch_status("dice_gather_rows");
}
}  // namespace dice

extern "C" int dice_gather_rows(const void *x, int dtype, const int32_t *perm, int slots_per_token,
                                int64_t n_rows, int hidden, void *out, void *stream) {
  return dice::gather_rows_impl(x, dtype, perm, slots_per_token, n_rows, hidden, out, nullptr, 0, stream);
}
