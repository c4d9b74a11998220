/*
 * C ABI of libmoe_hip.so: the FP8 fused-MoE inference path for AMD MI355X (gfx950).
 *
 * Plain C, no torch types.  Every pointer is a DEVICE pointer unless the comment says
 * otherwise; every entry point enqueues its kernels on `stream` (a hipStream_t passed as
 * void*) and returns without synchronising.  Nothing here allocates: outputs, scratch and
 * the workspace are the caller's (the reference's ops follow the same rule: the caller of
 * torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:117-236 allocates output and all scratch).
 *
 * Return value: 0 = enqueued; < 0 = invalid argument (MOE_E_*); > 0 = a hipError_t raised
 * by a launch.  Never throws.  This mirrors the reference's inner launcher convention
 * (`int moe_multi_core_bf16_fp8e4m3(stream, addrs..., ints...)` returning 0 or an error
 * code, torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:27-37) and its status enum
 * (third_party/tpuDNN/include/tpuDNN.h:8-12).
 *
 * Data formats
 *   fp8      OCP e4m3fn bytes (gfx950's native FP8), saturating encode at +-448.
 *   W13      [E, 2*I, H] fp8, rows 0..I-1 = gate projection, rows I..2I-1 = up projection,
 *            fp32 scales [E, 2*I/128, H/128]  (one per 128x128 block).
 *   W2       [E, H, I] fp8, fp32 scales [E, H/128, I/128].
 *   Every weight matrix handed to a GEMM entry point (w13, w2, shared_*, the dense layers' w, the bf16
 *   variants' weights) is TILE-BLOCKED, not row-major: moe_pack_weights() below re-orders a row-major
 *   matrix once, when the checkpoint is loaded (the reference's layout is re-packed at that point anyway:
 *   separate gate / up, pre-transposed down, python/regression/test_llm/test_moe.py:285-288).  Scales keep
 *   their plain [.., rows/128, cols/128] order.
 *   acts     bf16 [T, H]; quantised per token per 128 columns: scale = max(amax,1e-10)/448.
 *   ids      int32 [T, K], the K experts of a token are distinct.
 *   H and I must be multiples of 128.
 */
#ifndef MOE_HIP_H
#define MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Pointers to per-token data (activations, ids, routing weights, outputs) may be NULL when the
 * token count is 0: an empty batch is a valid call that does nothing (moe_permute still writes
 * its all-zero expert_offsets). */
#define MOE_OK                0
#define MOE_E_NULL           -1   /* a required pointer is NULL                          */
#define MOE_E_SHAPE          -2   /* a dimension is out of the supported range           */
#define MOE_E_ALIGN          -3   /* H or I not a multiple of 128, or pointer misaligned */
#define MOE_E_WORKSPACE      -4   /* workspace smaller than moe_workspace_bytes()        */
#define MOE_E_MODE           -5   /* unknown mode / dtype selector                       */
#define MOE_E_STATIC_SCRATCH -6   /* needs more scratch than MOE_STATIC_SCRATCH_BYTES    */

#define MOE_DTYPE_F32   0
#define MOE_DTYPE_BF16  1

#define MOE_ROUTE_SOFTMAX 0   /* select on logits; weights = softmax over all experts      */
#define MOE_ROUTE_SIGMOID 1   /* scores = sigmoid(logit); select on scores + bias          */
#define MOE_ROUTE_SCORES  2   /* the input already holds scores; select on scores + bias   */
#define MOE_ROUTE_SOFTMAX_LOGIT_BIAS 3  /* MOE_ROUTE_SOFTMAX on logits + bias: the bias is part of the logits
                                           (selection AND weights see it), as a softmax router's own bias term */

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOPK    32

/*
 * Library version and the gfx target it was built for.  The version changes whenever a caller built against an
 * older header would get wrong results without an error:
 *   100  weights row-major;
 *   200  every GEMM entry point (moe_fused_experts_*, moe_gemm1_swiglu, moe_gemm2, moe_mm_*, moe_mlp_fp8,
 *        moe_layer_fp8*) reads its weight bytes TILE-BLOCKED: pass them through moe_pack_weights once.
 * Callers check moe_hip_version() >= MOE_HIP_VERSION at load time.
 */
#define MOE_HIP_VERSION 200
int moe_hip_version(void);
const char *moe_hip_arch(void);
/* Text for a code returned by any entry point (static storage). */
const char *moe_hip_strerror(int code);

/*
 * Group-limited top-k.  Replaces at::noaux_tc_topk -> tpudnnNoauxTcTopkAsync
 * (torch_tpu/csrc/ops/my_ops/NoauxTcTopk.cpp:9-67, third_party/tpuDNN/include/tpuDNNTensor.h:728-737).
 * scores [T, E] viewed [T, n_groups, E/n_groups]; group score = sum of the group's two best
 * scores, rounded to the scores' dtype; the `topk_groups` best groups stay, the others
 * count as -inf; `top_k` best of the row follow, descending.  Equal values: lower index wins.
 * values_out [T, top_k] in the scores' dtype, indices_out [T, top_k] int32.
 */
int moe_noaux_tc_topk(void *stream, const void *scores, int scores_dtype, int T, int E,
                      int n_groups, int topk_groups, int top_k,
                      void *values_out, int32_t *indices_out);

/*
 * Router selection + weights from logits (or scores).  Replaces the aten recipe the
 * reference's callers run (python/regression/test_llm/test_torch_ops.py:441-456:
 * sigmoid -> topk -> sum -> div -> mul) and the softmax/top-k variant
 * (torch_tpu/csrc/ops/native_ops/Topk.cpp:91-205).
 * logits [T, E] (dtype selector), bias [E] fp32 or NULL (added for selection only; with
 * MOE_ROUTE_SOFTMAX_LOGIT_BIAS added to the logits themselves, so that selection and weights both see it).
 * n_groups <= 1 disables group limiting.  renorm != 0 divides by the sum of the selected
 * weights; the result is multiplied by `scale`.
 * weights_out [T, K] fp32, ids_out [T, K] int32 (descending selection order),
 * scores_out [T, E] fp32 or NULL (the scores selection ran on, before the bias).
 */
int moe_route_topk(void *stream, const void *logits, int logits_dtype, const float *bias,
                   int T, int E, int K, int mode, int n_groups, int topk_groups,
                   int renorm, float scale,
                   float *weights_out, int32_t *ids_out, float *scores_out);

/*
 * Token permutation = stable counting sort of the flattened ids.  Replaces the index
 * building phases of the reference kernel (torch_tpu/csrc/ops/my_ops/fusedMoE.pl:624-756:
 * per expert, ascending token ids / ascending flat slot ids).
 * sorted_slot [T*K]: flat slot ids t*K+k grouped by expert, ascending inside an expert.
 * expert_offsets [E+1]: rows of expert e are sorted_slot[expert_offsets[e] .. expert_offsets[e+1]).
 * slot_to_row [T*K]: inverse permutation.
 * Ids outside [0, E) are dropped: they get no row, slot_to_row = -1.
 * workspace: moe_permute_workspace_bytes(T, K, E) bytes.
 */
size_t moe_permute_workspace_bytes(int T, int K, int E);
/* Rows of one expert that a grouped-GEMM workgroup owns for this problem shape (16..192); the
 * permutation leaves the matching tile list in its workspace.  The reference's launcher picks
 * its token slice per core the same way, on the host (fusedMoE.cpp:60-78). */
int moe_tile_rows(int T, int K, int E);
int moe_permute(void *stream, const int32_t *ids, int T, int K, int E,
                int32_t *sorted_slot, int32_t *expert_offsets, int32_t *slot_to_row,
                void *workspace, size_t workspace_bytes);

/*
 * Weight layout.  The matrix [rows, row_bytes] (rows = all experts' rows stacked, a multiple of 16; row_bytes a
 * multiple of 128: the reduction dimension in bytes, K for fp8, 2*K for bf16) is cut into tiles of 16 rows and
 * steps of 128 bytes.  Tile-blocked order: tiles in row order, a tile's steps one after the other, 2 KB per
 * (tile, step) pair, and inside the 2 KB: half h = 0, 1, then lane l = 0..63, 16 bytes each = row l % 16 of the
 * tile, bytes 16 * (l / 16 + 4 h) .. + 15 of the step.  That is a wavefront's operand of
 * v_mfma_f32_16x16x128_f8f6f4: each load instruction of the GEMMs reads 1 KB of consecutive memory and a tile's
 * steps stream from one contiguous region.  Replaces the weight re-layout the reference's kernel does per call
 * on its way into local memory (torch_tpu/csrc/ops/my_ops/fusedMoE.pl:298-347, weight prefetch per expert).
 * Out of place (MOE_E_MODE when source and destination are the same buffer); pointers 16-byte aligned.
 */
int moe_pack_weights(void *stream, const void *w_rowmajor, int64_t rows, int row_bytes, void *w_blocked);
int moe_unpack_weights(void *stream, const void *w_blocked, int64_t rows, int row_bytes, void *w_rowmajor);

/*
 * Activation-scale tensors (the s of moe_act_quant, xs / hs of the stage entry points) hold one
 * fp32 per row and 128-column group, rows padded to moe_scale_pitch(groups) floats - whole
 * 64-byte pieces, which the grouped GEMMs fetch with single aligned reads.  The padding is never
 * interpreted.  Base addresses must be 64-byte aligned.
 */
int moe_scale_pitch(int n_groups);

/*
 * Per-token, per-128-column dynamic quantisation of bf16 activations.
 * x [R, C] bf16 -> q [R, C] fp8, s [R, moe_scale_pitch(C/128)] fp32.  No counterpart in the open
 * part of the reference (its W8A8 sibling is closed: torch_tpu/csrc/ops/my_ops/MlpW8A8Quant.cpp:34-46).
 */
int moe_act_quant(void *stream, const void *x_bf16, int R, int C, uint8_t *q, float *s);

/*
 * The expert computation.  Replaces at::fused_moe_fused_experts ->
 * tpudnnFusedMoEFusedExpertsMultiCoreAsync (torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:117-236,
 * third_party/tpuDNN/include/tpuDNNTensor.h:1585-1610) and its _v2 twin (fusedMoE.cpp:237-318):
 *   permute -> quantise x -> grouped FP8 GEMM with W13 + SwiGLU + re-quantise
 *           -> grouped FP8 GEMM with W2 -> un-permute.
 * out_mode 0: out is bf16 [T, K, H], un-weighted per-slot results (the reference's form;
 *             routing_weights may be NULL).
 * out_mode 1: out is bf16 [T, H] = sum_k routing_weights[t,k] * slot result (fp32 sum).
 *             If the shared_* pointers are non-NULL a shared expert (W13 [1,2*I_sh,H],
 *             W2 [1,H,I_sh]) is applied to every token and added with weight 1.
 * A slot whose id lies outside [0, E) has no expert (how a rank of an expert-parallel group marks the
 * experts it does not hold): its row in the [T, K, H] form is zero and it adds nothing to the sum.
 * workspace: moe_fused_experts_workspace_bytes(...) bytes, 256-byte aligned.
 */
size_t moe_fused_experts_workspace_bytes(int T, int H, int I, int E, int K, int I_shared);
int moe_fused_experts_fp8(void *stream,
                          const void *x_bf16, int T, int H,
                          const uint8_t *w13, const float *w13_scale,
                          const uint8_t *w2, const float *w2_scale, int I, int E,
                          const int32_t *ids, const float *routing_weights, int K,
                          const uint8_t *shared_w13, const float *shared_w13_scale,
                          const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                          void *out_bf16, int out_mode,
                          void *workspace, size_t workspace_bytes);
/*
 * The same with the routing weights in the dtype the caller holds them in: routing_weights_dtype MOE_DTYPE_F32 or
 * MOE_DTYPE_BF16 (the reference's callers hand the op bf16 routing weights,
 * python/regression/test_llm/test_moe.py:263; torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:117-131 takes the tensor as it is).  bf16 weights are widened inside the weighted sum (exact), so no
 * conversion kernel runs in front of the call, and the result equals that of moe_fused_experts_fp8 on the widened
 * weights bit for bit.
 */
int moe_fused_experts_fp8_rw(void *stream,
                             const void *x_bf16, int T, int H,
                             const uint8_t *w13, const float *w13_scale,
                             const uint8_t *w2, const float *w2_scale, int I, int E,
                             const int32_t *ids, const void *routing_weights, int routing_weights_dtype, int K,
                             const uint8_t *shared_w13, const float *shared_w13_scale,
                             const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                             void *out_bf16, int out_mode,
                             void *workspace, size_t workspace_bytes);

/*
 * Stages of the above, exposed for tests and for timing one kernel at a time.  All take
 * the permutation produced by moe_permute() and the tile list it leaves in its workspace.
 *
 * moe_gemm1_swiglu:  hq [T*K, I] fp8 / hs [T*K, moe_scale_pitch(I/128)] fp32 (rows in permuted order)
 *                    = requant(silu(x W_gate^T) * (x W_up^T)) with xq/xs from moe_act_quant.
 * moe_gemm2:         y [T*K, H] bf16, row of slot s at y[s] (slot order, i.e. [T, K, H]).
 * moe_weighted_reduce: out [T, H] bf16 = sum_k w[t,k] * y[t,k,:] (+ shared_y[t,:] if given).
 */
int moe_gemm1_swiglu(void *stream, const uint8_t *xq, const float *xs, int T, int H,
                     const uint8_t *w13, const float *w13_scale, int I, int E, int K,
                     const int32_t *sorted_slot, const int32_t *expert_offsets,
                     const void *permute_workspace,
                     uint8_t *hq, float *hs);
int moe_gemm2(void *stream, const uint8_t *hq, const float *hs, int T, int H,
              const uint8_t *w2, const float *w2_scale, int I, int E, int K,
              const int32_t *sorted_slot, const int32_t *expert_offsets,
              const void *permute_workspace,
              void *y_bf16);
int moe_weighted_reduce(void *stream, const void *y_bf16, const float *routing_weights,
                        const void *shared_y_bf16, int T, int K, int H, void *out_bf16);

/*
 * The same expert computation on un-quantised weights: the reference's op with its scale arguments
 * absent (fusedMoE.cpp:117-236 with gate/up/down_scales undefined; python/test/fused_moe_bf16.py:113-122).
 * x [T,H] bf16, w13 [E,2I,H] bf16 (gate rows, then up rows), w2 [E,H,I] bf16; products in bf16 matrix
 * instructions with fp32 accumulation, bf16 intermediate.  H and I multiples of 128, no shared expert.
 */
size_t moe_fused_experts_bf16_workspace_bytes(int T, int H, int I, int E, int K);
int moe_fused_experts_bf16(void *stream, const void *x_bf16, int T, int H, const void *w13_bf16,
                           const void *w2_bf16, int I, int E, const int32_t *ids,
                           const float *routing_weights, int K, void *out_bf16, int out_mode,
                           void *workspace, size_t workspace_bytes);

/*
 * The reference's own arithmetic on the packed FP8 weights: bf16 activations against weights that are
 * de-quantised on the way into the matrix instruction, w = bf16(float(code) * block scale) - what
 * weight_dequant_bc does in front of the reference kernel's bf16 products (fusedMoE.pl:11-34, 217-269) and what
 * its tests compute on the CPU (python/regression/test_llm/test_moe.py:10-50, 63-98).  No activation
 * quantisation, bf16 intermediate, fp32 accumulation; the weights are read once, at one byte per element.
 * Same tensors as moe_fused_experts_fp8 (tile-blocked w13 / w2, fp32 block scales), same workspace as
 * moe_fused_experts_bf16; the results are those of moe_fused_experts_bf16 on weights de-quantised beforehand, up to
 * the order of the matrix instructions' internal sums (a few results land on the neighbouring bf16).
 * H and I multiples of 128 and at most 16384, no shared expert.
 */
int moe_fused_experts_w8a16(void *stream, const void *x_bf16, int T, int H, const uint8_t *w13,
                            const float *w13_scale, const uint8_t *w2, const float *w2_scale, int I, int E,
                            const int32_t *ids, const float *routing_weights, int K, void *out_bf16,
                            int out_mode, void *workspace, size_t workspace_bytes);

/*
 * Dense block-scaled FP8 layers: the same kernels with a single "expert" that owns every row.
 *
 * moe_mm_fp8 replaces at::mm_w8a16_dq_forward -> tpudnnMmW8A16DqAsync
 * (torch_tpu/csrc/ops/my_ops/MmW8A16Dq.cpp:185-228): out [M, N] bf16 = x [M, K] bf16 times the
 * transpose of w [N, K] fp8 with fp32 scales [ceil(N/128), K/128].  K a multiple of 128, N a
 * multiple of 16.  Up to 128 rows a per-wavefront kernel slices the reduction over the chip and a
 * second kernel adds the slices in a fixed order (for the MLP the SwiGLU and re-quantisation ride in that
 * reduction) - for a single product only where that pays (K > 2048 and N < 12288; narrow layers keep it
 * further: N <= 2048 up to 384 rows, N <= 1024 up to 512); otherwise the grouped kernel runs with one expert.  Which of the two ran changes the order of the sums, not
 * the arithmetic: a result is reproducible for a given (M, K, N).
 * moe_mlp_fp8 replaces at::mlp_w8a16_dq_forward -> tpudnnMlpW8A16DqAsync
 * (torch_tpu/csrc/ops/my_ops/MlpW8A16Dq.cpp:189-241): out [M, H] bf16 =
 * (silu(x Wg^T) * (x Wu^T)) Wd^T with w13 [2I, H] = gate rows then up rows, w2 [H, I].
 * Unlike the reference (bf16 activations against de-quantised weights) both quantise the
 * activations per row and 128 columns, as the expert path does; the matrix products run in FP8.
 */
size_t moe_mm_fp8_workspace_bytes(int M, int K, int N);
int moe_mm_fp8(void *stream, const void *x_bf16, int M, int K, const uint8_t *w, const float *w_scale, int N,
               void *out_bf16, void *workspace, size_t workspace_bytes);
/*
 * The reference's own arithmetic for the same dense layer (MmW8A16Dq.cpp:185-228 multiplies bf16
 * activations with weights de-quantised to bf16): out [M, N] bf16 = x [M, K] bf16 times the transpose of
 * w [N, K] bf16, bf16 matrix instructions with fp32 accumulation.  The caller de-quantises once; this is
 * also the route for block sizes that do not divide into 128-blocks (the reference's tests use 64:
 * python/regression/test_llm/test_deepseek_mm.py:225).  K a multiple of 64 and at most 16384, N a multiple
 * of 16.  No workspace.
 */
int moe_mm_bf16(void *stream, const void *x_bf16, int M, int K, const void *w_bf16, int N, void *out_bf16);
/*
 * The same arithmetic without a de-quantised copy: w [N, K] fp8 (tile-blocked) with fp32 scales
 * [ceil(N/128), K/128] is de-quantised to bf16(float(code) * scale) in registers on the way into the bf16 matrix
 * instructions (MmW8A16Dq.cpp:185-228; python/regression/test_llm/test_mm_w8a16_dq.py:10-60).  K a multiple of 128
 * and at most 16384, N a multiple of 16.  No workspace.
 */
int moe_mm_w8a16(void *stream, const void *x_bf16, int M, int K, const uint8_t *w, const float *w_scale, int N,
                 void *out_bf16);
size_t moe_mlp_fp8_workspace_bytes(int M, int H, int I);
int moe_mlp_fp8(void *stream, const void *x_bf16, int M, int H, const uint8_t *w13, const float *w13_scale,
                const uint8_t *w2, const float *w2_scale, int I, void *out_bf16, void *workspace,
                size_t workspace_bytes);

/*
 * Router and experts of one layer in a single call, E <= MOE_MAX_EXPERTS experts.  Replaces, in one go, what the reference's callers chain on the host for every
 * token batch (python/regression/test_llm/test_torch_ops.py:440-456: logits = x Wr^T in bf16 -> sigmoid ->
 * top-k -> renormalise -> scale) and the expert op behind it
 * (torch_tpu/csrc/ops/my_ops/fusedMoE.cpp:117-236).
 * Decode-size batches (T * K <= 256 slots, E <= 256): two launches stand in front of the grouped GEMMs - the router
 * logits together with the activation quantisation, then routing and permutation.  Larger batches: the
 * router product runs on the matrix cores with its reduction cut into slices, the routing kernel adds
 * the slices, and the activations are quantised by extra workgroups of the permutation's scan launch.  Either way the logits
 * are fp32 sums rounded once to bf16.
 * router_w_bf16 [E, H] bf16; router_bias [E] fp32 or NULL (selection only, or part of the logits with
 * MOE_ROUTE_SOFTMAX_LOGIT_BIAS, as in moe_route_topk);
 * mode MOE_ROUTE_SOFTMAX or MOE_ROUTE_SIGMOID; the other routing arguments as in moe_route_topk.
 * out bf16 [T, H] (the weighted sum, shared expert added when its pointers are non-NULL).
 * logits_out_bf16 [T, E], weights_out [T, K], ids_out [T, K]: optional copies of what the router
 * produced (NULL to skip).  Given the same logits, ids and weights equal moe_route_topk's, and given the
 * same ids and weights the output equals moe_fused_experts_fp8's, bit for bit.
 * workspace: moe_layer_fp8_workspace_bytes(...) bytes, 256-byte aligned.
 */
size_t moe_layer_fp8_workspace_bytes(int T, int H, int I, int E, int K, int I_shared);
int moe_layer_fp8(void *stream, const void *x_bf16, int T, int H,
                         const void *router_w_bf16, const float *router_bias, int E, int K, int mode,
                         int n_groups, int topk_groups, int renorm, float scale,
                         const uint8_t *w13, const float *w13_scale,
                         const uint8_t *w2, const float *w2_scale, int I,
                         const uint8_t *shared_w13, const float *shared_w13_scale,
                         const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                         void *out_bf16, void *logits_out_bf16, float *weights_out, int32_t *ids_out,
                         void *workspace, size_t workspace_bytes);

/*
 * Batches of 512 tokens and more with a shared expert of the routed experts' width: moe_layer_fp8 runs the shared
 * expert's first GEMM, which needs nothing of the routing, on a stream of the library's own beside the router
 * product, routing and permutation launches (short chains that leave most of the chip idle), fenced by events on
 * both sides, so that to the caller the call is still work on its one stream; the results are the same bit for bit.
 * The side stream and its two events are created per (device, caller's stream) at the first call that uses them.
 * Not used while the caller's stream is being captured into a graph.  No counterpart in the reference (its device
 * runtime schedules the whole op).  moe_set_shared_overlap(0) switches it off, (1) on (the default); returns the
 * previous setting.
 */
int moe_set_shared_overlap(int enabled);

/*
 * moe_layer_fp8 for callers that cannot allocate device memory or hand over a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its ops take
 * every scratch tensor from the caller, fusedMoE.cpp:237-318).  Same arguments, same kernels and the same
 * result bits as moe_layer_fp8, minus the workspace: the scratch is an array of MOE_STATIC_SCRATCH_BYTES that
 * lives inside the library, one copy per GPU, held until the process ends.  It calls no hipMalloc / hipFree.
 * A problem whose moe_layer_fp8_workspace_bytes() exceeds MOE_STATIC_SCRATCH_BYTES is refused with
 * MOE_E_STATIC_SCRATCH before anything is launched (the DeepSeek-V3 layer fits up to T = 100 tokens).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe.
 * moe_hip_init() looks the array's device address up for the current device (once per device; the entry
 * point does the same on its first call there) - call it before capturing a graph on that device.
 * moe_static_scratch_address() reports that device address (for the current device): what the kernels of
 * moe_layer_fp8_static are handed as their workspace, so that a test can watch the array itself.
 */
#define MOE_STATIC_SCRATCH_BYTES (16u << 20)
int moe_hip_init(void);
int moe_static_scratch_address(void **address);
int moe_layer_fp8_static(void *stream, const void *x_bf16, int T, int H,
                         const void *router_w_bf16, const float *router_bias, int E, int K, int mode,
                         int n_groups, int topk_groups, int renorm, float scale,
                         const uint8_t *w13, const float *w13_scale,
                         const uint8_t *w2, const float *w2_scale, int I,
                         const uint8_t *shared_w13, const float *shared_w13_scale,
                         const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                         void *out_bf16, void *logits_out_bf16, float *weights_out, int32_t *ids_out);

/*
 * The router product on its own (any T, E <= MOE_MAX_EXPERTS): logits [T, E] bf16 = x [T, H] . router_w [E, H]^T, the
 * first step of the routing recipe (test_torch_ops.py:440).  The kernel moe_layer_fp8 uses for batches
 * beyond the decode size, followed by the sum over its slices.
 * workspace: moe_router_logits_workspace_bytes(T, H, E) bytes, 256-byte aligned.
 */
size_t moe_router_logits_workspace_bytes(int T, int H, int E);
int moe_router_logits(void *stream, const void *x_bf16, int T, int H, const void *router_w_bf16, int E,
                      void *logits_bf16, void *workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* MOE_HIP_H */
