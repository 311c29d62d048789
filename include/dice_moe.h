/*
 * dice_moe.h - C ABI of the MI355X (gfx950) DiT-MoE sparse expert layer.
 *
 * The reference (Cobalt-27/DICE) is pure Python on torch and has no FFI of its
 * own; every entry point below names the reference function whose work it
 * replaces.  Paths are relative to the reference tree.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - the caller owns every buffer; the library never allocates, frees or
 *     synchronises; all work is enqueued on `stream` (a hipStream_t passed as
 *     void*; NULL = the default stream);
 *   - return value 0 = ok, negative = error (see DICE_ERR_*); the text of the
 *     last error on the calling thread is available from dice_last_error();
 *   - matrices are row-major and contiguous; "slot" s = k*token + j is entry j
 *     of token's top-k list (token-major, as models.py:311-312 flattens it).
 */
#ifndef DICE_MOE_H
#define DICE_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DICE_MOE_ABI_VERSION 2

/* element types */
#define DICE_F32 0
#define DICE_BF16 1
#define DICE_F16 2
#define DICE_FP8_E4M3 3 /* OCP e4m3fn, weights only */

/* expert MLP variants */
#define DICE_ACT_SWIGLU 0    /* down(silu(gate(x)) * up(x)), models.py:271 */
#define DICE_ACT_GELU_TANH 1 /* fc2(gelu_tanh(fc1(x)+b1))+b2, models.py:496 */

/* errors */
#define DICE_OK 0
#define DICE_ERR_BAD_ARG (-1)
#define DICE_ERR_UNSUPPORTED (-2)
#define DICE_ERR_WORKSPACE (-3)
#define DICE_ERR_LAUNCH (-4)

int dice_abi_version(void);
const char *dice_last_error(void);

/*
 * Router.  Replaces MoEGate.forward, inference branch (models.py:179-196):
 * logits = x W^T (+ bias, an extension; NULL = reference), fp32 softmax over
 * experts, top-k in descending score order (slot 0 = arg-max; ties -> lower
 * expert id), optional renormalisation by (sum + 1e-20) (models.py:194-196).
 *   x        [n_tokens, hidden]   x_dtype in {F32, BF16, F16}
 *   w        [n_experts, hidden]  w_dtype in {F32, BF16, F16}
 *   bias     [n_experts] fp32 or NULL
 *   topk_idx   [n_tokens, top_k] int32   (required)
 *   topk_idx64 [n_tokens, top_k] int64   (optional, the reference's dtype)
 *   topk_weight[n_tokens, top_k] fp32
 *   logits     [n_tokens, n_experts] fp32 (optional, for tie audits)
 * Limits: n_experts <= 64, top_k <= 8, hidden % 8 == 0.
 */
int dice_gate_topk(const void *x, int x_dtype, const void *w, int w_dtype,
                   const float *bias, int64_t n_tokens, int hidden,
                   int n_experts, int top_k, int norm_topk_prob,
                   int32_t *topk_idx, int64_t *topk_idx64, float *topk_weight,
                   float *logits, void *stream);

/*
 * Dispatch tables.  Replaces argsort + bincount + cumsum of
 * SparseMoeBlock.moe_infer (models.py:365-367) and of moe_infer_ep
 * (expertpara/ep_fwd.py:70-76,100-106), including the slot drop of a skip
 * step (ep_fwd.py:57-66): slots whose skip_mask byte is non-zero are left out.
 *   flat_idx  [n_slots] int32 expert id per slot
 *   skip_mask [n_slots] uint8 or NULL
 *   counts    [n_experts] int32      rows per expert
 *   offsets   [n_experts+1] int32    exclusive scan of counts
 *   perm      [n_slots] int32        grouped row -> slot (stable: ascending
 *                                    slot inside each expert); entries past
 *                                    offsets[n_experts] are set to -1
 *   inv_perm  [n_slots] int32        slot -> grouped row, -1 for dropped slots
 *   workspace: dice_dispatch_workspace_bytes(n_slots, n_experts) bytes
 */
size_t dice_dispatch_workspace_bytes(int64_t n_slots, int n_experts);
int dice_dispatch(const int32_t *flat_idx, const uint8_t *skip_mask,
                  int64_t n_slots, int n_experts, int32_t *counts,
                  int32_t *offsets, int32_t *perm, int32_t *inv_perm,
                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * dice_dispatch without a workspace argument and without any allocation.  It
 * has no counterpart in the reference; it is for callers that cannot allocate
 * device memory around the call: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The per-span histogram table that
 * dice_dispatch keeps in `workspace` lives in a file-scope device array of
 * DICE_DISPATCH_STATIC_SCRATCH_BYTES instead (one copy per GPU, held until the
 * process ends; its device address is looked up once per device on the first
 * call there).  Same outputs as dice_dispatch, bit for bit.  Sizes whose table
 * exceeds the array (dice_dispatch_workspace_bytes(n_slots, n_experts) >
 * DICE_DISPATCH_STATIC_SCRATCH_BYTES) are refused with DICE_ERR_WORKSPACE.
 * All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (different streams) race; calls on one stream are ordered.
 */
#define DICE_DISPATCH_STATIC_SCRATCH_BYTES (1u << 20)
size_t dice_dispatch_static_scratch_bytes(void);
int dice_dispatch_static(const int32_t *flat_idx, const uint8_t *skip_mask,
                         int64_t n_slots, int n_experts, int32_t *counts,
                         int32_t *offsets, int32_t *perm, int32_t *inv_perm,
                         void *stream);

/*
 * Row gather.  Replaces _local_dispatch (expertpara/ep_fwd.py:345-347) and
 * x[exp_token_idx] (models.py:373): out[r] = x[perm[r] / slots_per_token] for
 * r < n_rows with perm[r] >= 0.  The fused expert path below reads x through
 * perm directly and does not need this copy; it exists for callers that want
 * the grouped activations themselves.
 */
int dice_gather_rows(const void *x, int dtype, const int32_t *perm,
                     int slots_per_token, int64_t n_rows, int hidden,
                     void *out, void *stream);

/*
 * Grouped expert MLP.  Replaces the per-expert loop of moe_infer
 * (models.py:368-377) / proc_experts (expertpara/ep_fwd.py:200-211) with
 * MoeMLP.forward (models.py:252-273) as the expert, in two grouped GEMMs:
 *   fc1: h[r] = act(A[r] W1[e]^T)     fc2: out[dst(r)] = h[r] W2[e]^T
 * for grouped rows r in [offsets[e], offsets[e+1]).
 *   x        [n_tokens, hidden] activations (act_dtype in {BF16, F16, F32}; weights
 *            in the same type, or FP8_E4M3 with 16-bit activations)
 *   perm     [>= max_rows] int32 grouped row -> slot, or NULL (row r = token r)
 *   slots_per_token  divisor turning a slot into its token row of x
 *   offsets  [n_experts+1] int32 (device)
 *   max_rows host upper bound of offsets[n_experts] (sizes the launch)
 *   w1       SWIGLU: [n_experts, 2, inter, hidden] = row-concatenated
 *            [gate_proj; up_proj]; GELU_TANH: [n_experts, inter, hidden]
 *   b1       GELU_TANH: [n_experts, inter] fp32 or NULL
 *   w2       [n_experts, hidden, inter]
 *   b2       GELU_TANH: [n_experts, hidden] fp32 or NULL
 *   w1_scale [n_experts, (2*)inter], w2_scale [n_experts, hidden] fp32 per
 *            output channel, required iff w_dtype == FP8_E4M3
 *   h        [max_rows, inter] workspace in act_dtype
 *   out      act_dtype; scatter_to_slots != 0: row perm[r] of [n_slots, hidden]
 *            (this is _local_combine, ep_fwd.py:350-354, fused into the fc2
 *            epilogue); else row r of [max_rows, hidden]
 * Expert outputs are NOT scaled by the routing weight here (the skip cache
 * stores them unscaled, ep_fwd.py:188); dice_combine applies the weights.
 * Limits: hidden % 64 == 0, inter % 64 == 0, n_experts <= 256.
 */
int dice_grouped_mlp(const void *x, int act_dtype, const int32_t *perm,
                     int slots_per_token, const int32_t *offsets,
                     int n_experts, int64_t max_rows, int hidden, int inter,
                     const void *w1, const float *b1, const void *w2,
                     const float *b2, const float *w1_scale,
                     const float *w2_scale, int w_dtype, int act_variant,
                     void *h, void *out, int scatter_to_slots, void *stream);

/*
 * One stage of dice_grouped_mlp on its own, same arguments: stage 1 = fc1 with
 * its activation (writes h), stage 2 = fc2 (reads h, writes out).  For callers
 * that schedule the two GEMMs themselves (other streams, per-kernel timing as
 * the reference's CudaProfiler scopes do around "moe.mlp", models.py:375).
 */
int dice_grouped_mlp_stage(int stage, const void *x, int act_dtype,
                           const int32_t *perm, int slots_per_token,
                           const int32_t *offsets, int n_experts,
                           int64_t max_rows, int hidden, int inter,
                           const void *w1, const float *b1, const void *w2,
                           const float *b2, const float *w1_scale,
                           const float *w2_scale, int w_dtype, int act_variant,
                           void *h, void *out, int scatter_to_slots,
                           void *stream);

/*
 * Combine.  Replaces mul_ by the routing weight + scatter_reduce_ of moe_infer
 * (models.py:377-381), i.e. final.mul_(w).view(N,k,h).sum(1) of moe_infer_ep
 * (expertpara/ep_fwd.py:190-195), the shared-expert add (models.py:355-357)
 * and the skip-cache blend / put (ep_fwd.py:176-188):
 *   y[t] = sum_j w[t,j] * row(t,j) (+ shared[t])
 *   row(t,j) = cache_in[t]               if skip_mask[k*t+j] and cache_in
 *            = slot_out[src(k*t+j)]      otherwise
 *   src(s) = inv_perm[s] if inv_perm else s
 *   cache_out[t] = slot_out[src(s)] for the slot s of token t with
 *                  skip_mask[s] != 0     (if cache_out; the "put" of a full step)
 * skip_mask must mark exactly one slot per token when a cache pointer is given.
 * Deterministic: fp32 accumulation in slot order, one rounding to `dtype`.
 */
int dice_combine(const void *slot_out, const int32_t *inv_perm,
                 const float *topk_weight, const void *shared_out,
                 const uint8_t *skip_mask, const void *cache_in,
                 void *cache_out, void *y, int dtype, int64_t n_tokens,
                 int top_k, int hidden, void *stream);

/*
 * Per-output-channel fp8 quantiser for expert weights (build-defined, the
 * reference has no fp8 path): scale[r] = amax(|w[r,:]|)/448 (1 if the row is
 * all zero), q[r,c] = e4m3fn(rne(w[r,c]/scale[r])).
 *   w [rows, cols] in_dtype in {BF16, F16, F32};  q [rows, cols] uint8;  scale [rows]
 */
int dice_quantize_fp8_rowwise(const void *w, int in_dtype, int64_t rows,
                              int64_t cols, uint8_t *q, float *scale,
                              void *stream);

/*
 * Per-row fp8 quantiser for activations (build-defined, the reference has no
 * fp8 path), with the dispatch gather fused in: for output row r < max_rows
 *   src = perm ? perm[r] / slots_per_token : r     (rows with perm[r] < 0 and
 *         rows >= *n_rows_dev, when that device pointer is given, are skipped)
 *   amax = max |x[src,:]|;  scale[r] = amax/448 (1 if the row is all zero)
 *   q[r,c] = e4m3fn(rne(x[src,c] * (448/amax)))
 *   x [*, cols] in_dtype in {BF16, F16};  q [max_rows, cols] uint8;  scale [max_rows]
 * cols % 8 == 0, cols <= 8192.
 */
int dice_quantize_fp8_act(const void *x, int in_dtype, const int32_t *perm,
                          int slots_per_token, const int32_t *n_rows_dev,
                          int64_t max_rows, int cols, uint8_t *q, float *scale,
                          void *stream);

/*
 * dice_grouped_mlp with fp8 weights AND fp8 activations, on the fp8 matrix
 * pipe (v_mfma_f32_32x32x64_f8f6f4): each GEMM is preceded by
 * dice_quantize_fp8_act of its input rows (fc1: rows of x gathered through
 * perm; fc2: rows of h), the fp32 sums are multiplied by the row's and the
 * output channel's scale in the epilogue; h and out are BF16.  Same reference
 * lines as dice_grouped_mlp (models.py:252-273, 368-377); the quantisation is
 * build-defined.
 *   stages   1 = fc1 (writes h), 2 = fc2 (reads h), 3 = both
 *   h_blocks 0: h is BF16 and a quantiser launch (one scale per row) runs in
 *            front of fc2.  1: fc1's epilogue quantises h itself, from the
 *            value rounded to BF16, with one power-of-two scale per row and
 *            32 columns:  t = amax * fp32(1/448);  e = exponent field of t,
 *            plus one unless t is a power of two;  byte = e4m3(rne(h *
 *            2^(127 - e)))  (a block with a NaN or an infinity: NaN bytes,
 *            e = 127).  fc2 multiplies with v_mfma_scale_f32_32x32x64_f8f6f4,
 *            which applies 2^(e - 127) to the block.  The buffer h then holds
 *            [max_rows, inter] bytes and, from the next multiple of 256
 *            bytes, [inter / 128, max_rows, 4] bytes e (the four of a row's
 *            128 columns in the order 0, 2, 1, 3); no more than 64 tiles of
 *            256 x 256 per compute unit in fc2.
 *   q_rows   [max_rows, max(hidden, inter)] bytes of scratch (the fp8 rows)
 *   q_scale  [max_rows] floats of scratch (their scales)
 * Output rows are in grouped order.  Limits: act_dtype BF16, hidden and inter
 * multiples of 256 and at least 768, n_experts <= 64.
 */
int dice_grouped_mlp_a8(int stages, const void *x, int act_dtype,
                        const int32_t *perm, int slots_per_token,
                        const int32_t *offsets, int n_experts, int64_t max_rows,
                        int hidden, int inter, const void *w1, const float *b1,
                        const void *w2, const float *b2, const float *w1_scale,
                        const float *w2_scale, int act_variant, int h_blocks,
                        void *h, void *out, uint8_t *q_rows, float *q_scale,
                        void *stream);

/*
 * Whole layer.  Replaces SparseMoeBlock.forward, inference branch
 * (models.py:302-312,321-358) with moe_infer / moe_infer_ep as above:
 * gate -> dispatch -> grouped MLP (+ shared expert MLP) -> combine, enqueued
 * back to back on `stream` with no host synchronisation (the reference's
 * .cpu() at models.py:366 disappears: offsets stay on the device).
 */
typedef struct dice_moe_layer {
  int32_t hidden, inter, n_experts, top_k;
  int32_t act_dtype;      /* DICE_BF16, DICE_F16 or DICE_F32 */
  int32_t w_dtype;        /* act_dtype, or DICE_FP8_E4M3 for routed experts */
  int32_t act_variant;    /* DICE_ACT_* */
  int32_t norm_topk_prob; /* models.py:170: 0 in the reference */
  int32_t gate_w_dtype;
  int32_t shared_inter;   /* 0 = no shared expert */
  const void *gate_w;     /* [n_experts, hidden] */
  const float *gate_bias; /* NULL in the reference */
  const void *w1, *w2;    /* routed experts, layout of dice_grouped_mlp */
  const float *b1, *b2, *w1_scale, *w2_scale;
  const void *shared_w1, *shared_w2; /* one expert, act_dtype */
  const float *shared_b1, *shared_b2;
  int32_t act_quant;      /* 2: as 1, with h quantised inside fc1's epilogue
                           * (h_blocks of dice_grouped_mlp_a8) instead of by a
                           * launch of its own.
                           * 0: 16-bit activations (fp8 weights are widened and
                           * multiplied on the 16-bit matrix pipe); 1: the routed
                           * experts' activations are quantised per row to e4m3
                           * on the way into each GEMM (dice_quantize_fp8_act)
                           * and multiplied on the fp8 matrix pipe: needs
                           * act_dtype BF16, w_dtype FP8_E4M3, hidden and inter
                           * multiples of 256 between 768 and 8192 */
  int32_t batch_invariant; /* 1: a token's result does not depend on what else is in
                           * the call.  By default an fc2 launch that carries one
                           * problem (fp8 routed weights, no shared expert, or a
                           * small batch whose shared expert gets its own launch)
                           * and whose tiles leave most workgroups idle in their
                           * last turn cuts that turn's tiles along k and adds the
                           * 16-bit pieces in fp32 in a fixed order: deterministic,
                           * but a token's last bit can then depend on the number
                           * of tokens (or dropped slots) in the call, and a skip
                           * step fed its own cache need not reproduce the full
                           * step bit for bit.  1 multiplies every tile whole. */
} dice_moe_layer_t;

/* mode: 0 = plain step; 1 = full step that also writes cache_out ("put");
 *       2 = skip step: slots with skip_mask != 0 are not recomputed and take
 *           cache_in instead. */
size_t dice_moe_workspace_bytes(const dice_moe_layer_t *layer, int64_t n_tokens);
int dice_moe_forward(const dice_moe_layer_t *layer, const void *x,
                     int64_t n_tokens, int mode, const uint8_t *skip_mask,
                     const void *cache_in, void *cache_out, void *y,
                     int32_t *topk_idx_out, float *topk_weight_out,
                     void *workspace, size_t workspace_bytes, void *stream);

/*
 * The layer's caller, fused.  Replaces the MoE line of DiTBlock.forward
 * (models.py:519)
 *   x = x + gate_mlp.unsqueeze(1) * self.moe(modulate(self.norm2(x), shift_mlp, scale_mlp))
 * with norm2 = LayerNorm(hidden, elementwise_affine=False, eps=1e-6)
 * (models.py:497) and modulate(x, shift, scale) = x*(1+scale)+shift per sample
 * (models.py:75-76).
 *
 * dice_ln_modulate is the prologue alone: out[t] = LN(x[t]) * (1 + scale[b]) +
 * shift[b], b = t / tokens_per_sample; statistics and arithmetic in fp32
 * (biased variance around the mean, eps inside the square root), one rounding
 * to `dtype`.   x, out [n_tokens, hidden]; shift, scale [n_samples, hidden].
 *
 * dice_combine_residual is dice_combine followed by the epilogue
 * out[t] = resid[t] + gate[b] * y[t], applied to the fp32 sum before the one
 * rounding; `out` may alias `resid`.
 *
 * dice_moe_forward_modulated is dice_moe_forward between the two: x is the
 * residual stream, the layer runs on the modulated rows (kept in the
 * workspace) and `out` (which may alias x) receives the updated stream.
 */
typedef struct dice_moe_caller {
  const void *shift, *scale, *gate; /* [n_samples, hidden], activation dtype */
  int64_t tokens_per_sample;        /* T of x [B, T, hidden] */
  float ln_eps;                     /* 1e-6 in the reference */
} dice_moe_caller_t;

int dice_ln_modulate(const void *x, const void *shift, const void *scale, void *out,
                     int dtype, int64_t n_tokens, int hidden, int64_t tokens_per_sample,
                     float eps, void *stream);
int dice_combine_residual(const void *slot_out, const int32_t *inv_perm,
                          const float *topk_weight, const void *shared_out,
                          const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                          const void *resid, const void *gate, int64_t tokens_per_sample,
                          void *out, int dtype, int64_t n_tokens, int top_k, int hidden,
                          void *stream);
int dice_moe_forward_modulated(const dice_moe_layer_t *layer, const dice_moe_caller_t *caller,
                               const void *x, int64_t n_tokens, int mode,
                               const uint8_t *skip_mask, const void *cache_in, void *cache_out,
                               void *out, int32_t *topk_idx_out, float *topk_weight_out,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * Step-lagged layer call.  Replaces moe_infer_ep with async_op=True
 * (expertpara/ep_fwd.py:133-172) and the dispatch / combine caches behind
 * global_dispatch_async / global_combine_async (expertpara/diep.py:17-28,
 * 196-289) on one GPU, where every all-to-all is a copy and what is left of the
 * asynchrony is its step lag: the routed experts run on an entry an earlier
 * call left behind, and the call returns the entry before that one.
 *
 * A dice_moe_lag_entry_t is one call's routing and what it refers to; it moves
 * through three roles, each in a different call unless the caller forces a
 * synchronous step by leaving `work` and `emit` NULL:
 *   put  - filled by this call: x (copy of the layer input; may alias x, then
 *          no copy is made and the caller keeps x unchanged while the entry
 *          lives), offsets, perm, inv_perm (dice_dispatch tables), topk_weight
 *          and, on the host, max_rows = n_tokens*top_k, or n_tokens when
 *          drop_skipped
 *   work - its routed experts run now: reads x, offsets, perm, max_rows (host
 *          bound on offsets[n_experts]); writes rows [max_rows, hidden],
 *          grouped and unweighted
 *   emit - combined into y: reads rows, inv_perm and, unless
 *          use_latest_weights, topk_weight (ep_fwd.py:190-193)
 * NULL roles default to the entry one stage earlier (work = put or the
 * workspace, emit = work), so all-NULL is dice_moe_forward.
 *   experts_of    layer whose routed expert weights the `work` entry needs (the
 *                 interweaved mode runs the previous lagged layer's experts,
 *                 diep.py:184-194,221-226); NULL = `layer`.  Gate and shared
 *                 expert always come from `layer` and run on x.
 *   drop_skipped  this call's dispatch leaves out slots with skip_mask != 0
 *                 (skip_now of ep_fwd.py:57-66)
 *   combine_mode  0 plain; 1 also write cache_out from the emitted entry; 2 the
 *                 emitted entry was produced with drop_skipped: masked slots
 *                 take cache_in (ep_fwd.py:176-188)
 *   caller        NULL, or the fused caller above: x is then the residual
 *                 stream, the entry's x receives the modulated rows directly
 *                 (no copy) and y the updated stream
 */
typedef struct dice_moe_lag_entry {
  void *x;
  int32_t *offsets, *perm, *inv_perm;
  float *topk_weight;
  void *rows;
  int64_t max_rows;
} dice_moe_lag_entry_t;

int dice_moe_forward_lagged(const dice_moe_layer_t *layer, const dice_moe_layer_t *experts_of,
                            const void *x, int64_t n_tokens, int drop_skipped,
                            const uint8_t *skip_mask, dice_moe_lag_entry_t *put,
                            const dice_moe_lag_entry_t *work, const dice_moe_lag_entry_t *emit,
                            int combine_mode, const void *cache_in, void *cache_out,
                            int use_latest_weights, const dice_moe_caller_t *caller,
                            void *y, int32_t *topk_idx_out,
                            float *topk_weight_out, void *workspace, size_t workspace_bytes,
                            void *stream);

/*
 * Stage timers.  Replace the reference's CudaProfiler scopes around the MoE
 * layer ("moe.gate", "moe.mlp", "moe.mlp_shared": models.py:305,356,375;
 * cudaprof/prof.py:19-60, expertpara/prof_analyse.py:3-17).  When enabled,
 * dice_moe_forward records HIP events on the caller's stream
 * between its launches (a ring of 64 event sets, so that back-to-back calls
 * need no host synchronisation in between); dice_profile_read waits for the
 * last one and returns, per stage, the mean elapsed milliseconds over the calls
 * made since the previous read (the most recent 64 at most).  Stages, one per
 * launch: "moe.gate", "moe.dispatch", "moe.gather" (the gathered copy of the
 * rows where one is made; with act_quant the quantiser of the fc1 input),
 * "moe.mlp.fc1" (routed experts, and the shared expert where it rides in the
 * same launch), "moe.mlp.shared_fc1" (its own launch: fp8 routed weights),
 * "moe.quant_h" (act_quant: quantiser of the fc2 input), "moe.mlp.fc2",
 * "moe.mlp.shared_fc2", "moe.combine"; a stage without a launch reads as the
 * gap between two events.  on = 1 times every stage; on = 2 only brackets
 * "moe.mlp.fc1" (two events per call, for timing the dominant launch inside a
 * throughput measurement; the other stages read as 0).
 */
int dice_profile_enable(int on);
int dice_profile_stage_count(void);
const char *dice_profile_stage_name(int i);
int dice_profile_read(float *ms_out, int n);

/*
 * Tuning hook, no counterpart in the reference: one code per GEMM stage of the
 * bf16/fp8 expert MLPs (0 = library default).  Process-wide; meant for benchmarks
 * and tests that compare kernels, not for the drop-in path (a caller who needs
 * results that do not depend on the batch sets dice_moe_layer_t.batch_invariant).
 * Any code from DICE_GEMM_CFG_PIPE32 on also keeps a dice_grouped_mlp stage whose
 * groups average at most 128 rows on the persistent kernels, which by default
 * leave it to the 64-row tiles of the permutation-addressed ones.
 */
#define DICE_GEMM_CFG_DEFAULT 0
/* 1..4: force a tiling of the permutation-addressed kernels (either stage) */
#define DICE_GEMM_CFG_PIPE32 20          /* persistent launches on the 32-k pipeline only */
#define DICE_GEMM_CFG_PERSISTENT 21      /* nothing but the small-group rule above */
#define DICE_GEMM_CFG_BANDS(b) (30 + (b)) /* b = 1..16: tiles of the persistent launches in bands of b m-tiles */
#define DICE_GEMM_CFG_FC1_ROUTER_OWN_LAUNCH 50 /* fc1: dice_moe_forward_modulated launches the router behind the prologue
                                                * kernel instead of inside it (same results) */
#define DICE_GEMM_CFG_FC2_WHOLE_TILES 50 /* fc2: no last turn is cut along k (as batch_invariant, for every layer) */
#define DICE_GEMM_CFG_FC2_SHARED_ALONE 51 /* fc2: the shared expert's fc2 always in a launch of its own */
#define DICE_GEMM_CFG_FC2_SHARED_JOINT 52 /* fc2: ... never (by default: small batches only) */
#define DICE_GEMM_CFG_SLIM_TILES 54      /* either stage: 128-row weight tiles wherever a launch can take them (fc2;
                                            SwiGLU fc1 with gathered rows) */
#define DICE_GEMM_CFG_NO_SLIM_TILES 55   /* ... never (by default: where the host's model of the workgroups' loads
                                            says they shorten the launch: fc1 below about 1000 tokens at DiT-XL width,
                                            fc2 between about 1000 and 2000) */
int dice_set_gemm_config(int fc1_cfg, int fc2_cfg);

/*
 * Test hook, no counterpart in the reference: the host-side bound on the turns
 * a workgroup of a persistent expert-GEMM launch may walk (which decides whether
 * the launch takes the kernel that rewrites its tile table) and, for the same
 * shapes with every group as tall as the bound allows, the most turns any
 * workgroup gets when the tiles are shared out over the XCDs by cost
 * (xcd_split 0) or per problem (1).  Arrays of n_problems entries.
 */
int dice_debug_persist_turns(int n_problems, const int64_t *max_rows, const int32_t *n_experts,
                             const int32_t *n, const int32_t *k, int fc2, int wgs_per_xcd,
                             int xcd_split, int64_t *bound_out, int64_t *turns_out);

#ifdef __cplusplus
}
#endif
#endif /* DICE_MOE_H */
