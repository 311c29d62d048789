// C entry points of the expert MLP and of the whole layer.
#include "gemm_common.h"

namespace dice {
namespace {

int run_gemm(const GemmParams &p, int mode, int act_dtype, int w_dtype, int64_t max_rows,
             hipStream_t s) {
  if (act_dtype == DICE_F32) return launch_grouped_gemm_f32(p, mode, w_dtype, max_rows, s);
  if (act_dtype == DICE_F16) return launch_grouped_gemm_f16(p, mode, w_dtype, max_rows, s);
  return launch_grouped_gemm_bf16(p, mode, w_dtype, max_rows, s);
}

bool is_16bit(int dtype) { return dtype == DICE_BF16 || dtype == DICE_F16; }

int launch_persist(const PersistBatch &b, int mode, int act_dtype, hipStream_t s) {
  return act_dtype == DICE_F16 ? launch_grouped_gemm_persist_f16(b, mode, s)
                               : launch_grouped_gemm_persist(b, mode, s);
}

struct Carve {
  unsigned char *base;
  size_t used;
  template <typename T> T *take(size_t count) {
    T *ptr = reinterpret_cast<T *>(base ? base + used : nullptr);
    used += align_up(count * sizeof(T), 256);
    return ptr;
  }
  void *take_bytes(size_t bytes) { return take<unsigned char>(bytes); }
};

struct LayerWorkspace {
  int32_t *topk_idx;
  float *topk_weight;
  int32_t *counts, *offsets, *perm, *inv_perm;
  void *dispatch_ws;
  size_t dispatch_ws_bytes;
  void *h, *slot_out, *shared_h, *shared_out, *modulated;
  int32_t *shared_offsets;
  void *split_ws;    // partial-tile slots of fc2 launches whose last turn is cut along k (16-bit activations)
  uint8_t *q_rows;   // (act_quant) fp8 rows of the GEMM about to run: [slots, max(hidden, inter)]
  float *q_scale;    // ... and their scales [slots]
  size_t total;
};

// Widths the fp8 x fp8 expert path takes: whole 256-k pairs of steps, at least six
// steps per tile, rows the quantiser holds in registers.
bool act_quant_widths_ok(int hidden, int inter) {
  auto ok = [](int w) { return w % 256 == 0 && w >= 768 && w <= 8192; };
  return ok(hidden) && ok(inter);
}

// Whether a layer call can launch a single-problem fc2 (the only launches that
// cut a short last turn along k and need the partial-tile slots): routed experts
// with fp8 weights (their bf16 shared expert rides alone), no shared expert, or
// the small batches whose shared fc2 gets a launch of its own.
bool shared_fc2_alone(const dice_moe_layer_t *L, int64_t n_tokens, int64_t max_rows);
bool layer_may_split_fc2(const dice_moe_layer_t *L, int64_t n_tokens) {
  if (!is_16bit(L->act_dtype) || L->batch_invariant) return false;
  if (L->w_dtype == DICE_FP8_E4M3 || L->shared_inter == 0) return true;
  return shared_fc2_alone(L, n_tokens, 0);   // (fewer routed rows, as on a skip step, only make it likelier)
}

LayerWorkspace carve_layer(const dice_moe_layer_t *L, int64_t n_tokens, void *ws) {
  LayerWorkspace w;
  Carve c{(unsigned char *)ws, 0};
  const size_t es = dtype_size(L->act_dtype);
  const size_t slots = (size_t)n_tokens * L->top_k;
  w.topk_idx = c.take<int32_t>(slots);
  w.topk_weight = c.take<float>(slots);
  w.counts = c.take<int32_t>(L->n_experts);
  w.offsets = c.take<int32_t>(L->n_experts + 1);
  w.perm = c.take<int32_t>(slots);
  w.inv_perm = c.take<int32_t>(slots);
  w.dispatch_ws_bytes = dice_dispatch_workspace_bytes((int64_t)slots, L->n_experts);
  w.dispatch_ws = c.take_bytes(w.dispatch_ws_bytes);
  w.h = c.take_bytes(slots * L->inter * es);
  w.slot_out = c.take_bytes(slots * L->hidden * es);
  w.shared_offsets = c.take<int32_t>(2);
  if (L->shared_inter > 0) {
    w.shared_h = c.take_bytes((size_t)n_tokens * L->shared_inter * es);
    w.shared_out = c.take_bytes((size_t)n_tokens * L->hidden * es);
  } else {
    w.shared_h = w.shared_out = nullptr;
  }
  w.modulated = c.take_bytes((size_t)n_tokens * L->hidden * es);  // layer input when the caller's prologue runs here
  w.split_ws = layer_may_split_fc2(L, n_tokens) ? c.take_bytes(persist_split_ws_bytes()) : nullptr;
  w.q_rows = nullptr;
  w.q_scale = nullptr;
  if (L->act_quant) {
    w.q_rows = c.take<uint8_t>(slots * (size_t)(L->inter > L->hidden ? L->inter : L->hidden));
    w.q_scale = c.take<float>(slots);
  }
  w.total = c.used;
  return w;
}

// Stage timers of dice_moe_forward: HIP events recorded on the caller's stream
// between the launches, the counterpart of the reference's CudaProfiler scopes
// "moe.gate" / "moe.mlp" / "moe.mlp_shared" (models.py:305,356,375;
// cudaprof/prof.py:19-60).  Off by default; events are host objects created on
// first use.
// "moe.gather" is the gathered copy of the rows, or (fp8 activations) the
// quantiser of the fc1 input, which gathers; "moe.quant_h" the quantiser of the
// fc2 input.  The shared expert's stages are empty where its problems ride in
// the routed experts' launches.
constexpr int kStages = 9;
const char *const kStageNames[kStages] = {"moe.gate", "moe.dispatch", "moe.gather", "moe.mlp.fc1",
                                          "moe.mlp.shared_fc1", "moe.quant_h", "moe.mlp.fc2",
                                          "moe.mlp.shared_fc2", "moe.combine"};
// A ring of event sets, one per timed call, so that a run of back-to-back calls
// can be timed without a host synchronisation between them.
constexpr int kTimerRing = 64;
constexpr int kFc1Stage = 3;  // index of "moe.mlp.fc1"
struct StageTimers {
  int mode = 0;       // 0 off, 1 every stage, 2 only the brackets of moe.mlp.fc1
  bool have_events = false;
  int recorded = 0;   // calls recorded since the last read (saturates at kTimerRing)
  int next = 0;       // ring position of the call being recorded
  hipEvent_t ev[kTimerRing][kStages + 1];
};
StageTimers g_timers;

void stamp(int i, hipStream_t s) {
  if (g_timers.mode != 0 && g_timers.have_events) {
    if (g_timers.mode == 1 || i == kFc1Stage || i == kFc1Stage + 1)
      (void)hipEventRecord(g_timers.ev[g_timers.next][i], s);
    if (i == kStages) {
      g_timers.next = (g_timers.next + 1) % kTimerRing;
      if (g_timers.recorded < kTimerRing) ++g_timers.recorded;
    }
  }
}

int check_mlp_shape(const char *who, int act_dtype, int w_dtype, int act_variant, int hidden,
                    int inter, int n_experts) {
  DICE_REQUIRE(is_16bit(act_dtype) || act_dtype == DICE_F32, DICE_ERR_UNSUPPORTED,
               "%s: act_dtype %d (BF16, F16 or F32)", who, act_dtype);
  DICE_REQUIRE(w_dtype == act_dtype || (w_dtype == DICE_FP8_E4M3 && is_16bit(act_dtype)),
               DICE_ERR_UNSUPPORTED, "%s: w_dtype %d with act_dtype %d", who, w_dtype, act_dtype);
  DICE_REQUIRE(act_variant == DICE_ACT_SWIGLU || act_variant == DICE_ACT_GELU_TANH,
               DICE_ERR_BAD_ARG, "%s: act_variant %d", who, act_variant);
  DICE_REQUIRE(hidden > 0 && hidden % 64 == 0 && inter > 0 && inter % 64 == 0, DICE_ERR_UNSUPPORTED,
               "%s: hidden %d and inter %d must be positive multiples of 64", who, hidden, inter);
  DICE_REQUIRE(n_experts >= 1 && n_experts <= 256, DICE_ERR_UNSUPPORTED,
               "%s: n_experts %d outside [1, 256]", who, n_experts);
  return DICE_OK;
}

}  // namespace
}  // namespace dice

namespace dice {
namespace {
// The two fp8 x fp8 problems of an expert MLP whose activations are quantised
// per row on the way in: fc1 reads q_rows as [rows, hidden] bytes, fc2 as
// [rows, inter] bytes (the buffer is re-used between the stages).
// h_blocks: fc1 writes h as e4m3 bytes with one power-of-two scale per row and
// 32 columns into the buffer `h` itself ([rows, inter] bytes, then [rows,
// inter / 32] scale bytes: together just over half of the 16-bit h it replaces)
// and fc2 reads them there; no quantiser runs between the stages.
uint8_t *h_block_scales(void *h, int64_t max_rows, int inter) {
  return (uint8_t *)h + (((size_t)max_rows * inter + 255) & ~(size_t)255);
}
void a8_problems(const int32_t *offsets, int n_experts, int64_t max_rows, int hidden, int inter, const void *w1,
                 const float *b1, const void *w2, const float *b2, const float *w1_scale, const float *w2_scale,
                 bool swiglu, void *h, void *out, const uint8_t *q_rows, const float *q_scale, PersistBatch *f1,
                 PersistBatch *f2, bool h_blocks = false) {
  *f1 = PersistBatch{};
  *f2 = PersistBatch{};
  f1->n_problems = f2->n_problems = 1;
  f1->prob[0] = PersistProblem{q_rows, hidden, offsets, n_experts, w1, swiglu ? 2 * inter : inter, inter,
                               swiglu ? nullptr : b1, h, inter, inter, hidden, (int)max_rows};
  f2->prob[0] = PersistProblem{q_rows, inter, offsets, n_experts, w2, hidden, 0, swiglu ? nullptr : b2,
                               out, hidden, hidden, inter, (int)max_rows};
  f1->prob[0].w_scale = w1_scale;
  f2->prob[0].w_scale = w2_scale;
  f1->prob[0].a_scale = f2->prob[0].a_scale = q_scale;
  if (h_blocks) {
    f1->prob[0].c_block_scale = h_block_scales(h, max_rows, inter);
    f2->prob[0].a = h;
    f2->prob[0].a_scale = nullptr;
    f2->prob[0].a_block_scale = h_block_scales(h, max_rows, inter);
  }
}

// Stage 1: quantise the (gathered) input rows, fc1 + activation -> h (bf16).
// Stage 2: quantise h, fc2 -> out.  `mark(i)` is called in front of launch i
// (0 quantiser, 1 fc1, 2 what the caller runs between the stages, 3 quantiser,
// 4 fc2) and `between` runs between the stages: the layer call puts the shared
// expert's first launch and its timer stamps there.
template <typename Between, typename Mark>
int mlp_a8_run(int stages, const void *x, const int32_t *perm, int slots_per_token, const int32_t *offsets,
               int n_experts, int64_t max_rows, int hidden, int inter, const PersistBatch &f1, const PersistBatch &f2,
               bool swiglu, void *h, uint8_t *q_rows, float *q_scale, hipStream_t s, Between between, Mark mark) {
  const int m1 = swiglu ? kFc1Swiglu : kFc1Gelu;
  int rc = DICE_OK;
  if (stages & 1) {
    mark(0);
    rc = quantize_act_impl(x, DICE_BF16, perm, slots_per_token, offsets + n_experts, max_rows, hidden, q_rows,
                           q_scale, s);
    if (rc) return rc;
    mark(1);
    rc = launch_grouped_gemm_persist_f8(f1, m1, s);
    if (rc) return rc;
  }
  mark(2);
  rc = between();
  if (rc) return rc;
  if (stages & 2) {
    mark(3);
    if (!f2.prob[0].a_block_scale) {   // (else fc1's epilogue has quantised h)
      rc = quantize_act_impl(h, DICE_BF16, nullptr, 1, offsets + n_experts, max_rows, inter, q_rows, q_scale, s);
      if (rc) return rc;
    }
    mark(4);
    rc = launch_grouped_gemm_persist_f8(f2, kFc2, s);
  }
  return rc;
}
}  // namespace
}  // namespace dice

extern "C" int dice_grouped_mlp_a8(int stages, const void *x, int act_dtype, const int32_t *perm,
                                   int slots_per_token, const int32_t *offsets, int n_experts,
                                   int64_t max_rows, int hidden, int inter, const void *w1, const float *b1,
                                   const void *w2, const float *b2, const float *w1_scale,
                                   const float *w2_scale, int act_variant, int h_blocks, void *h, void *out,
                                   uint8_t *q_rows, float *q_scale, void *stream) {
  using namespace dice;
  DICE_REQUIRE(x && offsets && w1 && w2 && h && out && q_rows && q_scale && w1_scale && w2_scale, DICE_ERR_BAD_ARG,
               "dice_grouped_mlp_a8: null pointer");
  DICE_REQUIRE(stages >= 1 && stages <= 3, DICE_ERR_BAD_ARG, "dice_grouped_mlp_a8: stages %d (1 = fc1, 2 = fc2, 3 = both)",
               stages);
  DICE_REQUIRE(act_dtype == DICE_BF16, DICE_ERR_UNSUPPORTED, "dice_grouped_mlp_a8: act_dtype %d (BF16)", act_dtype);
  int rc = check_mlp_shape("dice_grouped_mlp_a8", act_dtype, DICE_FP8_E4M3, act_variant, hidden, inter, n_experts);
  if (rc) return rc;
  DICE_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31) &&
                   max_rows * (int64_t)(inter > hidden ? inter : hidden) < (1ll << 31),
               DICE_ERR_BAD_ARG, "dice_grouped_mlp_a8: max_rows %lld", (long long)max_rows);
  DICE_REQUIRE(!perm || slots_per_token >= 1, DICE_ERR_BAD_ARG, "dice_grouped_mlp_a8: slots_per_token %d",
               slots_per_token);
  if (max_rows == 0) return DICE_OK;
  const bool swiglu = act_variant == DICE_ACT_SWIGLU;
  PersistBatch f1, f2;
  DICE_REQUIRE(h_blocks == 0 || h_blocks == 1, DICE_ERR_BAD_ARG, "dice_grouped_mlp_a8: h_blocks %d (0 or 1)", h_blocks);
  a8_problems(offsets, n_experts, max_rows, hidden, inter, w1, b1, w2, b2, w1_scale, w2_scale, swiglu, h, out,
              q_rows, q_scale, &f1, &f2, h_blocks != 0);
  DICE_REQUIRE(persist_f8_supported(f1, swiglu ? kFc1Swiglu : kFc1Gelu) && persist_f8_supported(f2, kFc2),
               DICE_ERR_UNSUPPORTED,
               "dice_grouped_mlp_a8: hidden %d and inter %d must be multiples of 256 (at least 768), n_experts %d at most 64",
               hidden, inter, n_experts);
  return mlp_a8_run(stages, x, perm, slots_per_token, offsets, n_experts, max_rows, hidden, inter, f1, f2, swiglu, h,
                    q_rows, q_scale, (hipStream_t)stream, [] { return (int)DICE_OK; }, [](int) {});
}

namespace dice {
namespace {
int grouped_mlp_impl(int stages, const void *x, int act_dtype, const int32_t *perm,
                     int slots_per_token, const int32_t *offsets, int n_experts, int64_t max_rows,
                     int hidden, int inter, const void *w1, const float *b1, const void *w2,
                     const float *b2, const float *w1_scale, const float *w2_scale, int w_dtype,
                     int act_variant, void *h, void *out, int scatter_to_slots, void *stream) {
  DICE_REQUIRE(x && offsets && w1 && w2 && h && out, DICE_ERR_BAD_ARG, "dice_grouped_mlp: null pointer");
  int rc = check_mlp_shape("dice_grouped_mlp", act_dtype, w_dtype, act_variant, hidden, inter, n_experts);
  if (rc) return rc;
  DICE_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), DICE_ERR_BAD_ARG,
               "dice_grouped_mlp: max_rows %lld", (long long)max_rows);
  DICE_REQUIRE(!perm || slots_per_token >= 1, DICE_ERR_BAD_ARG,
               "dice_grouped_mlp: slots_per_token %d < 1", slots_per_token);
  DICE_REQUIRE(!scatter_to_slots || perm, DICE_ERR_BAD_ARG,
               "dice_grouped_mlp: scatter_to_slots needs perm");
  if (w_dtype == DICE_FP8_E4M3)
    DICE_REQUIRE(w1_scale && w2_scale, DICE_ERR_BAD_ARG, "dice_grouped_mlp: fp8 weights need scales");
  DICE_REQUIRE(max_rows * (int64_t)(inter > hidden ? inter : hidden) < (1ll << 31),
               DICE_ERR_UNSUPPORTED, "dice_grouped_mlp: max_rows * row length exceeds 2^31 elements");
  if (max_rows == 0) return DICE_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool swiglu = act_variant == DICE_ACT_SWIGLU;

  // 16-bit activations: each stage takes the persistent kernel where it applies
  // (fc1 addresses rows through the permutation itself in its SwiGLU form; fc2
  // writes grouped rows, so a scatter to slot order stays with the
  // permutation-addressed kernel), unless the tuning hook names a tiling.
  const int m1 = swiglu ? kFc1Swiglu : kFc1Gelu;
  PersistBatch pb1{}, pb2{};
  bool fc1_persist = false, fc2_persist = false;
  if (is_16bit(act_dtype)) {
    pb1.n_problems = pb2.n_problems = 1;
    pb1.prob[0] = PersistProblem{x, hidden, offsets, n_experts, w1, swiglu ? 2 * inter : inter, inter,
                                 swiglu ? nullptr : b1, h, inter, inter, hidden, (int)max_rows};
    if (perm) {
      // This entry point is not told how many rows x has: the row addresses get
      // the widest range the kernel can address (the permutation-addressed
      // kernel checks none either); slots beyond it fall back to that kernel.
      pb1.prob[0].a_rows = perm;
      pb1.prob[0].a_div = slots_per_token;
      const int64_t by_slots = ((1ll << 28) - 1) / slots_per_token;
      const int64_t by_bytes = ((1ll << 31) - 1) / ((int64_t)hidden * 2);
      pb1.prob[0].a_src_rows = (int)(by_slots < by_bytes ? by_slots : by_bytes);
    }
    pb2.prob[0] = PersistProblem{h, inter, offsets, n_experts, w2, hidden, 0, swiglu ? nullptr : b2,
                                 out, hidden, hidden, inter, (int)max_rows};
    if (w_dtype == DICE_FP8_E4M3) {
      pb1.prob[0].w_scale = w1_scale;
      pb2.prob[0].w_scale = w2_scale;
    }
    const bool few = few_rows_per_group(max_rows, n_experts);
    fc1_persist = gemm_config_allows_persistent(m1) && !(few && gemm_config_is_default(m1)) && persist_supported(pb1, m1);
    fc2_persist = !scatter_to_slots && gemm_config_allows_persistent(kFc2) &&
                  !(few && gemm_config_is_default(kFc2)) && persist_supported(pb2, kFc2);
  }

  if (stages & 1) {
    if (fc1_persist) {
      rc = launch_persist(pb1, m1, act_dtype, s);
    } else {
      GemmParams p1{};
      p1.a = x;
      p1.a_perm = perm;
      p1.a_div = perm ? slots_per_token : 1;
      p1.lda = hidden;
      p1.offsets = offsets;
      p1.n_experts = n_experts;
      p1.w = w1;
      p1.w_rows = swiglu ? 2 * inter : inter;
      p1.up_offset = inter;
      p1.bias = swiglu ? nullptr : b1;
      p1.w_scale = w_dtype == DICE_FP8_E4M3 ? w1_scale : nullptr;
      p1.c = h;
      p1.ldc = inter;
      p1.c_perm = nullptr;
      p1.n = inter;
      p1.k = hidden;
      rc = run_gemm(p1, m1, act_dtype, w_dtype, max_rows, s);
    }
    if (rc) return rc;
  }
  if (!(stages & 2)) return DICE_OK;
  if (fc2_persist) return launch_persist(pb2, kFc2, act_dtype, s);

  GemmParams p2{};
  p2.a = h;
  p2.a_perm = nullptr;
  p2.a_div = 1;
  p2.lda = inter;
  p2.offsets = offsets;
  p2.n_experts = n_experts;
  p2.w = w2;
  p2.w_rows = hidden;
  p2.up_offset = 0;
  p2.bias = swiglu ? nullptr : b2;
  p2.w_scale = w_dtype == DICE_FP8_E4M3 ? w2_scale : nullptr;
  p2.c = out;
  p2.ldc = hidden;
  p2.c_perm = scatter_to_slots ? perm : nullptr;
  p2.n = hidden;
  p2.k = inter;
  return run_gemm(p2, kFc2, act_dtype, w_dtype, max_rows, s);
}
}  // namespace
}  // namespace dice

extern "C" int dice_grouped_mlp(const void *x, int act_dtype, const int32_t *perm,
                                int slots_per_token, const int32_t *offsets, int n_experts,
                                int64_t max_rows, int hidden, int inter, const void *w1,
                                const float *b1, const void *w2, const float *b2,
                                const float *w1_scale, const float *w2_scale, int w_dtype,
                                int act_variant, void *h, void *out, int scatter_to_slots,
                                void *stream) {
  return dice::grouped_mlp_impl(3, x, act_dtype, perm, slots_per_token, offsets, n_experts, max_rows,
                                hidden, inter, w1, b1, w2, b2, w1_scale, w2_scale, w_dtype,
                                act_variant, h, out, scatter_to_slots, stream);
}

extern "C" int dice_grouped_mlp_stage(int stage, const void *x, int act_dtype, const int32_t *perm,
                                      int slots_per_token, const int32_t *offsets, int n_experts,
                                      int64_t max_rows, int hidden, int inter, const void *w1,
                                      const float *b1, const void *w2, const float *b2,
                                      const float *w1_scale, const float *w2_scale, int w_dtype,
                                      int act_variant, void *h, void *out, int scatter_to_slots,
                                      void *stream) {
  if (stage != 1 && stage != 2)
    return dice::fail(DICE_ERR_BAD_ARG, "dice_grouped_mlp_stage: stage %d (1 = fc1, 2 = fc2)", stage);
  return dice::grouped_mlp_impl(stage, x, act_dtype, perm, slots_per_token, offsets, n_experts,
                                max_rows, hidden, inter, w1, b1, w2, b2, w1_scale, w2_scale, w_dtype,
                                act_variant, h, out, scatter_to_slots, stream);
}

extern "C" size_t dice_moe_workspace_bytes(const dice_moe_layer_t *layer, int64_t n_tokens) {
  if (!layer || n_tokens < 0) return 0;
  return dice::carve_layer(layer, n_tokens, nullptr).total;
}

namespace dice {
namespace {
// Shared body of dice_moe_forward and dice_moe_forward_lagged.  `put` receives
// this call's routing (NULL: it lives in the workspace), `work` names the entry
// whose routed experts run now and `emit` the entry that is combined into y
// (NULL: the entry one stage earlier in put -> work -> emit).
// Small batches: all fc2 tiles of the routed and the shared expert together fill
// less than half of the compute units, the launch lasts as long as its longest
// tile, and a launch with two problems does not cut tiles along k.  The shared
// expert's fc2 then gets a launch of its own, so that both launches cut theirs
// (one piece per idle workgroup).  Measured at DiT-XL width, joint / separate, us
// per layer call: SwiGLU experts (shared k = 2304) 132 / 124 at 64 tokens, 146 /
// 142 at 512, 155 / 156 at 768, 164 / 167 at 1024; GELU experts with a shared
// expert of 2 x the routed width (k = 9216: twice the routed tiles' length) 166 /
// 116 at 64, 174 / 134 at 512, 216 / 190 at 1024, 241 / 242 at 1536.  The bound
// on the tile count is the host's (row counts live on the device).
bool shared_fc2_alone(const dice_moe_layer_t *L, int64_t n_tokens, int64_t max_rows) {
  const int choice = shared_fc2_launch_choice();
  if (choice != 0) return choice > 0;
  if (L->batch_invariant) return false;   // (the second launch only pays where both cut their tiles)
  // (tiles of fewer than 64 steps: a second launch costs what the cut saves - DiT-B width, 48 and 24
  // steps: 95 / 89 us at 64 tokens, but 114 / 119 at 1024 and 121 / 129 at 1536)
  if (!persist_split_allowed() || (L->inter < 4096 && L->shared_inter < 4096)) return false;
  const int64_t m_tiles = max_rows / 256 + L->n_experts + n_tokens / 256 + 1;
  const int64_t tiles = m_tiles * ((L->hidden + 255) / 256);
  return tiles * 16 <= (int64_t)persist_cu_count() * (L->shared_inter > L->inter ? 7 : 6);
}

int forward_impl(const char *who, const dice_moe_layer_t *L, const dice_moe_layer_t *LE, const void *x,
                 int64_t n_tokens, bool drop_skipped, const uint8_t *skip_mask,
                 dice_moe_lag_entry_t *put, const dice_moe_lag_entry_t *work_in,
                 const dice_moe_lag_entry_t *emit_in, int combine_mode, const void *cache_in,
                 void *cache_out, bool use_latest_weights, const dice_moe_caller_t *caller, void *y,
                 int32_t *topk_idx_out, float *topk_weight_out, void *workspace, size_t workspace_bytes,
                 void *stream) {
  DICE_REQUIRE(L && x && y, DICE_ERR_BAD_ARG, "%s: null pointer", who);
  if (caller)
    DICE_REQUIRE(caller->shift && caller->scale && caller->gate && caller->tokens_per_sample >= 1,
                 DICE_ERR_BAD_ARG, "%s: the caller's shift / scale / gate or tokens_per_sample", who);
  DICE_REQUIRE(combine_mode >= 0 && combine_mode <= 2, DICE_ERR_BAD_ARG, "%s: mode %d", who, combine_mode);
  DICE_REQUIRE(L->gate_w && LE->w1 && LE->w2, DICE_ERR_BAD_ARG, "%s: null weights", who);
  DICE_REQUIRE(L->top_k >= 1 && L->top_k <= 8 && L->top_k <= L->n_experts, DICE_ERR_BAD_ARG,
               "%s: top_k %d", who, L->top_k);
  int rc = check_mlp_shape(who, L->act_dtype, LE->w_dtype, LE->act_variant, L->hidden, LE->inter,
                           L->n_experts);
  if (rc) return rc;
  DICE_REQUIRE(L->n_experts <= 64, DICE_ERR_UNSUPPORTED, "%s: n_experts %d > 64", who, L->n_experts);
  DICE_REQUIRE(LE->hidden == L->hidden && LE->inter == L->inter && LE->n_experts == L->n_experts &&
                   LE->top_k == L->top_k && LE->act_dtype == L->act_dtype &&
                   LE->act_variant == L->act_variant,
               DICE_ERR_BAD_ARG, "%s: the layer whose experts run must have this layer's shape", who);
  if (L->shared_inter > 0) {
    DICE_REQUIRE(L->shared_w1 && L->shared_w2 && L->shared_inter % 64 == 0, DICE_ERR_BAD_ARG,
                 "%s: shared expert weights / shared_inter %d", who, L->shared_inter);
  }
  if (L->act_quant || LE->act_quant) {
    DICE_REQUIRE((L->act_quant == 1 || L->act_quant == 2) && LE->act_quant == L->act_quant &&
                     L->act_dtype == DICE_BF16 && LE->w_dtype == DICE_FP8_E4M3 && LE->w1_scale && LE->w2_scale,
                 DICE_ERR_UNSUPPORTED,
                 "%s: act_quant (0, 1 or 2) needs bf16 activations and fp8 expert weights with scales, in both layers",
                 who);
    // (what the fp8 kernels and the row quantiser take, checked before anything is launched)
    DICE_REQUIRE(act_quant_widths_ok(L->hidden, L->inter), DICE_ERR_UNSUPPORTED,
                 "%s: act_quant needs hidden %d and inter %d to be multiples of 256 between 768 and 8192", who,
                 L->hidden, L->inter);
    if (L->act_quant == 2) {
      // (fc2 on block-scaled rows has no variant that rebuilds its tile table: refused here, before the
      // router is launched, and not by the fc2 launch)
      PersistBatch probe{};
      probe.n_problems = 1;
      probe.prob[0].n_experts = L->n_experts;
      probe.prob[0].n = L->hidden;
      probe.prob[0].k = L->inter;
      probe.prob[0].max_rows = (int)(n_tokens * L->top_k);
      DICE_REQUIRE(persist_fits_table(probe, kFc2), DICE_ERR_UNSUPPORTED,
                   "%s: act_quant 2 takes at most 64 fc2 tiles of 256 x 256 per compute unit (%lld tokens make more); "
                   "use act_quant 1 or split the batch", who, (long long)n_tokens);
    }
  }
  if (combine_mode == 1)
    DICE_REQUIRE(skip_mask && cache_out, DICE_ERR_BAD_ARG, "%s: a put step needs skip_mask and cache_out", who);
  if (combine_mode == 2)
    DICE_REQUIRE(skip_mask && cache_in, DICE_ERR_BAD_ARG, "%s: a skip step needs skip_mask and cache_in", who);
  if (drop_skipped) DICE_REQUIRE(skip_mask, DICE_ERR_BAD_ARG, "%s: dropping slots needs skip_mask", who);
  if (drop_skipped || combine_mode == 2)
    DICE_REQUIRE(L->top_k == 2, DICE_ERR_UNSUPPORTED, "%s: skipping supports top_k == 2 only (got %d)",
                 who, L->top_k);
  DICE_REQUIRE(n_tokens >= 0 && n_tokens * L->top_k < (1ll << 31), DICE_ERR_BAD_ARG, "%s: n_tokens %lld",
               who, (long long)n_tokens);
  if (n_tokens == 0) return DICE_OK;
  // Entries are checked before anything is launched.
  if (work_in)
    DICE_REQUIRE(work_in->x && work_in->offsets && work_in->perm && work_in->rows && work_in->max_rows >= 0 &&
                     work_in->max_rows <= n_tokens * L->top_k,
                 DICE_ERR_BAD_ARG, "%s: the entry to run the experts on lacks a buffer or holds %lld rows (at most %lld)",
                 who, (long long)work_in->max_rows, (long long)(n_tokens * L->top_k));
  else if (put)
    DICE_REQUIRE(put->rows, DICE_ERR_BAD_ARG, "%s: the entry to fill lacks a buffer (its experts run in this call: rows)", who);
  if (emit_in)
    DICE_REQUIRE(emit_in->rows && emit_in->inv_perm && emit_in->topk_weight, DICE_ERR_BAD_ARG,
                 "%s: the entry to combine lacks a buffer", who);
  LayerWorkspace w = carve_layer(L, n_tokens, workspace);
  DICE_REQUIRE(workspace && workspace_bytes >= w.total, DICE_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes",
               who, workspace_bytes, w.total);
  hipStream_t s = (hipStream_t)stream;
  const int64_t slots = n_tokens * L->top_k;
  const size_t es = dtype_size(L->act_dtype);

  // This call's own routing entry: in the caller's buffers when it outlives
  // the call, else in the workspace.
  dice_moe_lag_entry_t own;
  if (put) {
    DICE_REQUIRE(put->x && put->offsets && put->perm && put->inv_perm && put->topk_weight,
                 DICE_ERR_BAD_ARG, "%s: the entry to fill lacks a buffer", who);
    own = *put;
  } else {
    own.x = nullptr;
    own.offsets = w.offsets;
    own.perm = w.perm;
    own.inv_perm = w.inv_perm;
    own.topk_weight = topk_weight_out ? topk_weight_out : w.topk_weight;
    own.rows = w.slot_out;
  }
  // A skip step recomputes one slot per token.
  own.max_rows = drop_skipped ? n_tokens * (L->top_k - 1) : slots;
  if (put) put->max_rows = own.max_rows;
  int32_t *idx = topk_idx_out ? topk_idx_out : w.topk_idx;
  float *wt = own.topk_weight;

  stamp(0, s);
  // With the caller's prologue the layer input is LN(x) modulated, written
  // straight into the entry that outlives the call when there is one; x itself
  // is then only the residual of the epilogue.
  const void *resid = nullptr;
  bool routed = false;
  if (caller) {
    void *hm = put ? put->x : w.modulated;
    DICE_REQUIRE(hm != x, DICE_ERR_BAD_ARG, "%s: the entry's input buffer aliases x", who);
    // The router runs inside the prologue kernel where that kernel takes the
    // shape: the modulated rows are then routed from LDS, not read back.
    routed = route_in_prologue_allowed() &&
             ln_modulate_route_applies(L->act_dtype, L->gate_w_dtype, n_tokens, L->hidden, L->n_experts);
    rc = routed ? ln_modulate_route_impl(x, caller->shift, caller->scale, hm, L->act_dtype, n_tokens, L->hidden,
                                         caller->tokens_per_sample, caller->ln_eps, L->gate_w, L->gate_bias,
                                         L->n_experts, L->top_k, L->norm_topk_prob, idx, wt, stream)
                : ln_modulate_impl(x, caller->shift, caller->scale, hm, L->act_dtype, n_tokens, L->hidden,
                                   caller->tokens_per_sample, caller->ln_eps, stream);
    if (rc) return rc;
    resid = x;
    x = hm;
  }
  if (!routed)
    rc = dice_gate_topk(x, L->act_dtype, L->gate_w, L->gate_w_dtype, L->gate_bias, n_tokens, L->hidden,
                        L->n_experts, L->top_k, L->norm_topk_prob, idx, nullptr, wt, nullptr, stream);
  if (rc) return rc;
  if (put && topk_weight_out)
    DICE_HIP(hipMemcpyAsync(topk_weight_out, wt, slots * sizeof(float), hipMemcpyDeviceToDevice, s));
  stamp(1, s);
  rc = dispatch_impl(idx, drop_skipped ? skip_mask : nullptr, slots, L->n_experts, w.counts, own.offsets,
                     own.perm, own.inv_perm, w.dispatch_ws, w.dispatch_ws_bytes,
                     L->shared_inter > 0 ? w.shared_offsets : nullptr, (int32_t)n_tokens, stream);
  if (rc) return rc;
  if (put && put->x != x)
    DICE_HIP(hipMemcpyAsync(put->x, x, (size_t)n_tokens * L->hidden * es, hipMemcpyDeviceToDevice, s));
  stamp(2, s);

  // The entry whose routed experts run in this call.
  dice_moe_lag_entry_t work = work_in ? *work_in : own;
  if (!work_in) work.x = const_cast<void *>(x);
  DICE_REQUIRE(work.x && work.offsets && work.perm && work.rows, DICE_ERR_BAD_ARG,
               "%s: the entry to run the experts on lacks a buffer", who);
  DICE_REQUIRE(work.max_rows >= 0 && work.max_rows <= slots, DICE_ERR_BAD_ARG,
               "%s: entry holds %lld rows, this call at most %lld", who, (long long)work.max_rows,
               (long long)slots);
  const dice_moe_lag_entry_t emit = emit_in ? *emit_in : work;
  DICE_REQUIRE(emit.rows && emit.inv_perm && emit.topk_weight, DICE_ERR_BAD_ARG,
               "%s: the entry to combine lacks a buffer", who);
  const int64_t max_rows = work.max_rows;
  const uint8_t *mask = combine_mode == 0 ? nullptr : skip_mask;
  const float *combine_wt = use_latest_weights ? wt : emit.topk_weight;

  // bf16 activations: two persistent launches, each covering the routed experts
  // and the shared expert together; with fp8 routed weights the shared expert
  // (bf16) gets launches of its own.
  bool done = false;
  const bool w8 = LE->w_dtype == DICE_FP8_E4M3;
  if (LE->act_quant) {
    // fp8 activations too: the routed experts run on the fp8 matrix pipe, each
    // GEMM behind a quantiser of its input rows; the shared expert (bf16)
    // keeps its own two launches.
    const bool swiglu = L->act_variant == DICE_ACT_SWIGLU;
    const int m1 = swiglu ? kFc1Swiglu : kFc1Gelu;
    PersistBatch f1, f2, s1{}, s2{};
    a8_problems(work.offsets, L->n_experts, max_rows, L->hidden, L->inter, LE->w1, LE->b1, LE->w2, LE->b2,
                LE->w1_scale, LE->w2_scale, swiglu, w.h, work.rows, w.q_rows, w.q_scale, &f1, &f2,
                LE->act_quant == 2);
    DICE_REQUIRE(persist_f8_supported(f1, m1) && persist_f8_supported(f2, kFc2), DICE_ERR_UNSUPPORTED,
                 "%s: act_quant needs hidden %d and inter %d to be multiples of 256 (at least 768)", who,
                 L->hidden, L->inter);
    if (L->shared_inter > 0) {
      const int si = L->shared_inter;
      s1.prob[0] = PersistProblem{x, L->hidden, w.shared_offsets, 1, L->shared_w1, swiglu ? 2 * si : si, si,
                                  swiglu ? nullptr : L->shared_b1, w.shared_h, si, si, L->hidden, (int)n_tokens};
      s2.prob[0] = PersistProblem{w.shared_h, si, w.shared_offsets, 1, L->shared_w2, L->hidden, 0,
                                  swiglu ? nullptr : L->shared_b2, w.shared_out, L->hidden, L->hidden, si, (int)n_tokens};
      s1.n_problems = s2.n_problems = 1;
    }
    f2.split_ws = s2.split_ws = persist_split_allowed() && !L->batch_invariant ? w.split_ws : nullptr;
    const bool shared_persist = s1.n_problems && persist_supported(s1, m1) && persist_supported(s2, kFc2);
    rc = mlp_a8_run(
        3, work.x, work.perm, L->top_k, work.offsets, L->n_experts, max_rows, L->hidden, L->inter, f1, f2, swiglu,
        w.h, w.q_rows, w.q_scale, s,
        [&]() -> int { return shared_persist ? launch_persist(s1, m1, L->act_dtype, s) : (int)DICE_OK; },
        [&](int i) { stamp(2 + i, s); });   // stages 2..6: quantiser, fc1, shared fc1, quantiser, fc2
    if (rc) return rc;
    stamp(7, s);
    if (shared_persist) {
      rc = launch_persist(s2, kFc2, L->act_dtype, s);
    } else if (L->shared_inter > 0) {
      rc = dice_grouped_mlp(x, L->act_dtype, nullptr, 1, w.shared_offsets, 1, n_tokens, L->hidden,
                            L->shared_inter, L->shared_w1, L->shared_b1, L->shared_w2, L->shared_b2, nullptr,
                            nullptr, L->act_dtype, L->act_variant, w.shared_h, w.shared_out, 0, stream);
    }
    if (rc) return rc;
    stamp(8, s);
    done = true;
  } else if (is_16bit(L->act_dtype) && (LE->w_dtype == L->act_dtype || (w8 && LE->w1_scale && LE->w2_scale))) {
    const bool swiglu = L->act_variant == DICE_ACT_SWIGLU;
    const int m1 = swiglu ? kFc1Swiglu : kFc1Gelu;
    PersistBatch f1{}, f2{};
    void *xg = w.slot_out;  // gathered rows, dead before fc2 could write its outputs there
    f1.prob[0] = PersistProblem{xg, L->hidden, work.offsets, L->n_experts, LE->w1,
                                swiglu ? 2 * L->inter : L->inter, L->inter, swiglu ? nullptr : LE->b1,
                                w.h, L->inter, L->inter, L->hidden, (int)max_rows};
    f2.prob[0] = PersistProblem{w.h, L->inter, work.offsets, L->n_experts, LE->w2, L->hidden, 0,
                                swiglu ? nullptr : LE->b2, work.rows, L->hidden, L->hidden, L->inter,
                                (int)max_rows};
    f1.n_problems = f2.n_problems = 1;
    if (w8) {
      f1.prob[0].w_scale = LE->w1_scale;
      f2.prob[0].w_scale = LE->w2_scale;
    }
    PersistBatch s1{}, s2{};  // the shared expert on its own (fp8 routed weights only)
    if (L->shared_inter > 0) {
      const int si = L->shared_inter;
      const PersistProblem p1{x, L->hidden, w.shared_offsets, 1, L->shared_w1, swiglu ? 2 * si : si, si,
                              swiglu ? nullptr : L->shared_b1, w.shared_h, si, si, L->hidden, (int)n_tokens};
      const PersistProblem p2{w.shared_h, si, w.shared_offsets, 1, L->shared_w2, L->hidden, 0,
                              swiglu ? nullptr : L->shared_b2, w.shared_out, L->hidden, L->hidden, si, (int)n_tokens};
      if (w8) {
        s1.prob[0] = p1;
        s2.prob[0] = p2;
        s1.n_problems = s2.n_problems = 1;
      } else if (shared_fc2_alone(L, n_tokens, max_rows)) {
        f1.prob[1] = p1;
        f1.n_problems = 2;
        s2.prob[0] = p2;
        s2.n_problems = 1;
      } else {
        f1.prob[1] = p1;
        f2.prob[1] = p2;
        f1.n_problems = f2.n_problems = 2;
      }
    }
    f2.split_ws = s2.split_ws = persist_split_allowed() && !L->batch_invariant ? w.split_ws : nullptr;
    const bool shared_ok = (s1.n_problems == 0 || persist_supported(s1, m1)) &&
                           (s2.n_problems == 0 || persist_supported(s2, kFc2));
    // Where the kernel can address the activation rows through the permutation
    // itself, the gathered copy is skipped.
    PersistBatch f1g = f1;
    f1g.prob[0].a = work.x;
    f1g.prob[0].a_rows = work.perm;
    f1g.prob[0].a_div = L->top_k;
    f1g.prob[0].a_src_rows = (int)n_tokens;
    const bool fused_gather = shared_ok && persist_supported(f1g, m1) && persist_supported(f2, kFc2);
    if (fused_gather || (shared_ok && persist_supported(f1, m1) && persist_supported(f2, kFc2))) {
      if (fused_gather) {
        f1 = f1g;
      } else {
        rc = gather_rows_impl(work.x, L->act_dtype, work.perm, L->top_k, max_rows, L->hidden, xg, nullptr, 0,
                              stream);
        if (rc) return rc;
      }
      stamp(3, s);
      rc = launch_persist(f1, m1, L->act_dtype, s);
      if (rc) return rc;
      stamp(4, s);
      if (s1.n_problems) {
        rc = launch_persist(s1, m1, L->act_dtype, s);
        if (rc) return rc;
      }
      stamp(5, s);
      stamp(6, s);
      rc = launch_persist(f2, kFc2, L->act_dtype, s);
      if (rc) return rc;
      stamp(7, s);
      if (s2.n_problems) {
        rc = launch_persist(s2, kFc2, L->act_dtype, s);
        if (rc) return rc;
      }
      stamp(8, s);
      done = true;
    }
  }
  if (!done) {
    // Every other case (fp32, shapes the persistent kernels do not take): the
    // per-stage kernels, one launch per stage and expert set, each in its own
    // timer stage.
    const bool shared = L->shared_inter > 0;
    for (int stage = 1; stage <= 2; ++stage) {
      stamp(stage == 1 ? 3 : 6, s);
      rc = grouped_mlp_impl(stage, work.x, L->act_dtype, work.perm, L->top_k, work.offsets, L->n_experts, max_rows,
                            L->hidden, L->inter, LE->w1, LE->b1, LE->w2, LE->b2, LE->w1_scale, LE->w2_scale,
                            LE->w_dtype, L->act_variant, w.h, work.rows, 0, stream);
      if (rc) return rc;
      stamp(stage == 1 ? 4 : 7, s);
      if (shared) {
        rc = grouped_mlp_impl(stage, x, L->act_dtype, nullptr, 1, w.shared_offsets, 1, n_tokens, L->hidden,
                              L->shared_inter, L->shared_w1, L->shared_b1, L->shared_w2, L->shared_b2, nullptr,
                              nullptr, L->act_dtype, L->act_variant, w.shared_h, w.shared_out, 0, stream);
        if (rc) return rc;
      }
      stamp(stage == 1 ? 5 : 8, s);
    }
  }
  rc = combine_impl(emit.rows, emit.inv_perm, combine_wt, w.shared_out, mask,
                    combine_mode == 2 ? cache_in : nullptr, combine_mode == 1 ? cache_out : nullptr, y,
                    L->act_dtype, n_tokens, L->top_k, L->hidden, resid, caller ? caller->gate : nullptr,
                    caller ? caller->tokens_per_sample : 1, stream);
  stamp(kStages, s);
  return rc;
}
}  // namespace
}  // namespace dice

extern "C" int dice_moe_forward(const dice_moe_layer_t *L, const void *x, int64_t n_tokens,
                                int mode, const uint8_t *skip_mask, const void *cache_in,
                                void *cache_out, void *y, int32_t *topk_idx_out,
                                float *topk_weight_out, void *workspace, size_t workspace_bytes,
                                void *stream) {
  DICE_REQUIRE(mode >= 0 && mode <= 2, DICE_ERR_BAD_ARG, "dice_moe_forward: mode %d", mode);
  return dice::forward_impl("dice_moe_forward", L, L, x, n_tokens, mode == 2, skip_mask, nullptr, nullptr,
                            nullptr, mode, cache_in, cache_out, false, nullptr, y, topk_idx_out,
                            topk_weight_out, workspace, workspace_bytes, stream);
}

extern "C" int dice_moe_forward_modulated(const dice_moe_layer_t *L, const dice_moe_caller_t *caller,
                                          const void *x, int64_t n_tokens, int mode,
                                          const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                                          void *out, int32_t *topk_idx_out, float *topk_weight_out,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  DICE_REQUIRE(caller, DICE_ERR_BAD_ARG, "dice_moe_forward_modulated: null pointer");
  DICE_REQUIRE(mode >= 0 && mode <= 2, DICE_ERR_BAD_ARG, "dice_moe_forward_modulated: mode %d", mode);
  return dice::forward_impl("dice_moe_forward_modulated", L, L, x, n_tokens, mode == 2, skip_mask, nullptr,
                            nullptr, nullptr, mode, cache_in, cache_out, false, caller, out, topk_idx_out,
                            topk_weight_out, workspace, workspace_bytes, stream);
}

extern "C" int dice_moe_forward_lagged(const dice_moe_layer_t *L, const dice_moe_layer_t *experts_of,
                                       const void *x, int64_t n_tokens, int drop_skipped,
                                       const uint8_t *skip_mask, dice_moe_lag_entry_t *put,
                                       const dice_moe_lag_entry_t *work, const dice_moe_lag_entry_t *emit,
                                       int combine_mode, const void *cache_in, void *cache_out,
                                       int use_latest_weights, const dice_moe_caller_t *caller, void *y,
                                       int32_t *topk_idx_out, float *topk_weight_out, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  DICE_REQUIRE(L, DICE_ERR_BAD_ARG, "dice_moe_forward_lagged: null pointer");
  return dice::forward_impl("dice_moe_forward_lagged", L, experts_of ? experts_of : L, x, n_tokens,
                            drop_skipped != 0, skip_mask, put, work, emit, combine_mode, cache_in, cache_out,
                            use_latest_weights != 0, caller, y, topk_idx_out, topk_weight_out, workspace,
                            workspace_bytes, stream);
}

extern "C" int dice_profile_enable(int on) {
  using namespace dice;
  if (on && !g_timers.have_events) {
    for (int r = 0; r < kTimerRing; ++r)
      for (int i = 0; i <= kStages; ++i) {
        hipError_t e = hipEventCreate(&g_timers.ev[r][i]);
        if (e != hipSuccess) return fail(DICE_ERR_LAUNCH, "dice_profile_enable: %s", hipGetErrorString(e));
      }
    g_timers.have_events = true;
  }
  g_timers.mode = on == 2 ? 2 : (on != 0 ? 1 : 0);
  g_timers.recorded = 0;
  return DICE_OK;
}

extern "C" int dice_profile_stage_count(void) { return dice::kStages; }

extern "C" const char *dice_profile_stage_name(int i) {
  return i >= 0 && i < dice::kStages ? dice::kStageNames[i] : "";
}

extern "C" int dice_profile_read(float *ms_out, int n) {
  using namespace dice;
  DICE_REQUIRE(ms_out && n >= kStages, DICE_ERR_BAD_ARG, "dice_profile_read: need room for %d stages", kStages);
  DICE_REQUIRE(g_timers.mode != 0 && g_timers.recorded > 0, DICE_ERR_BAD_ARG,
               "dice_profile_read: no timed dice_moe_forward call since dice_profile_enable or the last read");
  const int calls = g_timers.recorded;
  const int last = (g_timers.next + kTimerRing - 1) % kTimerRing;
  hipError_t e = hipEventSynchronize(g_timers.ev[last][g_timers.mode == 1 ? kStages : kFc1Stage + 1]);
  if (e != hipSuccess) return fail(DICE_ERR_LAUNCH, "dice_profile_read: %s", hipGetErrorString(e));
  for (int i = 0; i < kStages; ++i) ms_out[i] = 0.f;
  for (int c = 0; c < calls; ++c) {
    const int r = (last + kTimerRing - c) % kTimerRing;
    for (int i = 0; i < kStages; ++i) {
      if (g_timers.mode == 2 && i != kFc1Stage) continue;
      float ms = 0.f;
      e = hipEventElapsedTime(&ms, g_timers.ev[r][i], g_timers.ev[r][i + 1]);
      if (e != hipSuccess) return fail(DICE_ERR_LAUNCH, "dice_profile_read: %s", hipGetErrorString(e));
      ms_out[i] += ms / calls;
    }
  }
  g_timers.recorded = 0;
  return DICE_OK;
}
