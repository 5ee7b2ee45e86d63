/*
 * planmoe_hip.h -- C ABI of libplanmoe_hip.so: the per-GPU MoE data path of PlanMoE
 * (top-k gating with capacity slots, dispatch / combine kernels with their backward
 * passes, the "int8" and zfp fixed-rate codecs) as hand-written HIP kernels for gfx950.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the parameter name ends in _host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); every call only
 *     enqueues work on that stream and returns without synchronising;
 *   - the library never allocates device memory: callers pass outputs and, where a call
 *     needs scratch, a workspace sized by the matching *_workspace_bytes() query;
 *   - return value 0 = success; anything else is an error whose text is available from
 *     planmoe_last_error() (thread local).  Nothing is enqueued when an error is returned;
 *   - choice planes: per-token routing data of the k choices are k planes of `samples`
 *     elements, plane j starting at base + j * plane_stride (elements, >= samples).  This is
 *     the list-of-k-tensors of the reference (fast_dispatch.py:99-101) laid out in one buffer.
 *   - a (token, choice) pair is LIVE iff location < capacity and index >= 0
 *     (jit_kernels/sparse.py:29,50,78; custom_kernel.cpp:73,84,101).
 *
 * File:line citations name the interface of the reference (PlanMoE/...) each entry
 * point replaces.
 */
#ifndef PLANMOE_HIP_H
#define PLANMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PLANMOE_ABI_VERSION 1

typedef enum planmoe_dtype {
    PLANMOE_F32 = 0,
    PLANMOE_BF16 = 1,
    PLANMOE_F16 = 2
} planmoe_dtype;

/* ---------------------------------------------------------------- housekeeping */

int planmoe_abi_version(void);

/* Text of the last error raised on the calling thread ("" if none). Host pointer. */
const char *planmoe_last_error(void);

/* ---------------------------------------------------------------- capacity cumsum
 * Replaces torch.ops.tutel_ops.cumsum / warp_cumsum (custom/custom_kernel.cpp:331-385),
 * reached through fast_cumsum_sub_one (jit_kernels/gating.py:17-22).
 * out[t][c] = (sum of in[0..t][c]) - 1 for an int32 row-major [samples, columns] matrix.
 * Workspace: planmoe_cumsum_workspace_bytes(samples, columns). */
size_t planmoe_cumsum_workspace_bytes(int samples, int columns);
int planmoe_cumsum_sub_one(const int32_t *in, int32_t *out, int samples, int columns,
                           void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- routing
 * Replaces extract_critical (impls/fast_dispatch.py:140-195) for the capacity_factor > 0,
 * non-batch-prioritised case, together with the softmax of the layer's routing closure
 * (impls/moe_layer.py:239) and the GShard auxiliary loss (impls/losses.py:12-19).
 */

/* capacity = k * int(cf * ceil(T / E)) rounded up to `alignment`  (fast_dispatch.py:179-190).
 * Host-only arithmetic; capacity_factor must be > 0. */
int planmoe_capacity(int samples, int experts, int top_k, double capacity_factor,
                     int alignment, int *capacity_host);

size_t planmoe_route_workspace_bytes(int samples, int experts, int top_k);

/* input        [samples, experts] row-major in `dtype` (F32 or BF16): softmax scores, or
 *              gate logits when input_is_logits != 0 (softmax over experts is then applied
 *              first, in fp32, rounded to `dtype`).
 * logit_bias   optional fp32 [experts] added to the logits before the softmax (NULL = none;
 *              only with input_is_logits).
 * indices      out int32 k planes   expert id of the j-th largest score (ties: lower id)
 * locations    out int32 k planes   slot inside that expert; all first choices of an expert
 *              come first in token order, then all second choices, ...
 * gates        out `dtype` k planes score of the chosen expert, divided by
 *              clamp(sum over the k choices, eps(dtype)) when normalize_gate and k > 1
 * scores_out   optional out [samples, experts] `dtype`: the scores routing was done on
 * l_aux        optional out fp32 scalar: sum_e(me[e] * ce[e]) / samples with me = column sums
 *              of the scores and ce = (experts / samples) * number of first choices of e
 * expert_counts optional out int32 [top_k, experts]: tokens whose j-th choice is e
 * top_k is clamped to `experts` (fast_dispatch.py:142); planes beyond the clamp are untouched.
 */
int planmoe_route_topk(const void *input, int dtype, int input_is_logits, const float *logit_bias,
                       int samples, int experts, int top_k, int normalize_gate,
                       int32_t *indices, int32_t *locations, void *gates, int64_t plane_stride,
                       void *scores_out, float *l_aux, int32_t *expert_counts,
                       void *workspace, size_t workspace_bytes, void *stream);

/* Slot locations for routing decisions that already exist, with the tokens taking their slots in
 * a given order: compute_sorted_location of batch-prioritised routing (fast_dispatch.py:135-138,
 * 152-154), and with order == NULL the plain fast_cumsum_sub_one path (:156-168).
 *   indices       int32 top_k planes (base + j*plane_stride); an index outside [0, experts)
 *                 takes no slot and gets location -1
 *   order         optional int32 [samples]: order[p] = token that is p-th to be served (a
 *                 permutation, e.g. the stable argsort of -max score); NULL = 0, 1, 2, ...
 *   locations     out int32 planes: all first choices of an expert before all its second
 *                 choices, inside a plane the served order
 *   expert_counts optional out int32 [top_k, experts]
 *   workspace     planmoe_route_workspace_bytes(samples, experts, top_k) bytes
 * top_k is NOT clamped here: it is the number of planes present. */
int planmoe_route_locations(const int32_t *indices, int64_t plane_stride, int samples, int experts,
                            int top_k, const int32_t *order, int32_t *locations,
                            int32_t *expert_counts, void *workspace, size_t workspace_bytes,
                            void *stream);

/* Backward of planmoe_route_topk with respect to its input: what autograd derives from the
 * tensor algebra of extract_critical (fast_dispatch.py:148, 170-172: gates are score entries,
 * divided by their clamped sum) and of gshard_loss (losses.py:12-19: me depends on the scores,
 * ce does not).
 *   scores        [samples, experts] `dtype`, the scores routing ran on (scores_out)
 *   grad_gates    `dtype` k planes: gradient arriving at the gates
 *   grad_l_aux    optional fp32 scalar: gradient arriving at l_aux (needs first_choice_counts =
 *                 row 0 of expert_counts)
 *   through_softmax != 0: grad_scores receives the gradient of the logits instead
 *                 (softmax backward applied; for input_is_logits callers)
 *   grad_scores   out [samples, experts] `dtype` */
int planmoe_route_bwd(const void *scores, int dtype, const int32_t *indices, const void *grad_gates,
                      int64_t plane_stride, int samples, int experts, int top_k, int normalize_gate,
                      const float *grad_l_aux, const int32_t *first_choice_counts,
                      int through_softmax, void *grad_scores, void *stream);

/* Gate logits  logits[samples, experts] = x[samples, model_dim] . wg[experts, model_dim]^T
 * (gates/top.py:20-26).  x and wg are in `dtype` (BF16: MFMA with fp32 accumulation; F32:
 * fp32 FMA); logits are written in `out_dtype` (F32 = the fp32_gate flow, or `dtype`). */
int planmoe_gate_logits(const void *x, const void *wg, int dtype, void *logits, int out_dtype,
                        int samples, int model_dim, int experts, void *stream);

/* The gate's share of the gradient of x, added in place: dx[t, :] += sum_e grad_logits[t, e] *
 * wg[e, :] -- the backward of LinearTopKGate.forward (gates/top.py:20-26, which autograd runs as
 * a GEMM and an accumulation into x.grad) as one streaming read-modify-write of dx.  dx and wg in
 * `dtype`, grad_logits fp32 [samples, experts] (rounded to `dtype` first, as the cast in front of
 * the GEMM would); up to 8 experts (above that a GEMM is the better tool); model_dim a multiple
 * of 16 bytes' worth of elements. */
int planmoe_gate_dx_accumulate(void *dx, int dtype, const float *grad_logits, const void *wg, int samples,
                               int model_dim, int experts, void *stream);

/* ---------------------------------------------------------------- dispatch / combine
 * Replace the JIT kernels of jit_kernels/sparse.py (create_forward :17-35,
 * create_backward_data :38-64, create_backward_gate :67-134), their CPU twins
 * invoke_cpu_fp32 (custom/custom_kernel.cpp:57-112) and the per-choice launch loops of
 * GatingEncoder / GatingDecoder (impls/fast_dispatch.py:16-79).
 * Tensors are in `dtype` (F32, BF16 or F16); arithmetic is fp32 with one rounding per
 * operation, as the reference's dispatcher computes (fast_dispatch.py:91-93,121-131).
 * `gates` are fp32 planes or NULL for the all-ones helper (fast_dispatch.py:24,57).
 */

size_t planmoe_dispatch_workspace_bytes(int experts, int capacity);

/* GatingEncoder.forward (fast_dispatch.py:18-29) == GatingDecoder.backward's scatter (:66-71):
 *   dispatched[(idx*capacity + loc), :] = 0 + gate * x[t, :]   for every live pair,
 *   every other row of dispatched[experts*capacity, model_dim] = 0.
 * Live pairs must address distinct slots (true for planmoe_route_topk's output); when two
 * pairs collide the later write wins instead of the reference's sum. */
int planmoe_dispatch_fwd(const void *x, int dtype, const float *gates, const int32_t *indices,
                         const int32_t *locations, int64_t plane_stride, int top_k,
                         int samples, int model_dim, int experts, int capacity,
                         void *dispatched, void *workspace, size_t workspace_bytes, void *stream);

/* GatingDecoder.forward (fast_dispatch.py:51-64) == GatingEncoder.backward's data path (:33-38):
 *   out[t, :] = sum over j (left to right) of (live_j ? gate_j * dispatched[slot_j, :] : 0). */
int planmoe_combine_fwd(const void *dispatched, int dtype, const float *gates,
                        const int32_t *indices, const int32_t *locations, int64_t plane_stride,
                        int top_k, int samples, int model_dim, int capacity, void *out,
                        void *stream);

/* create_backward_gate for all k planes at once (fast_dispatch.py:40-45, 73-78):
 *   grad_gates[j][t] = live ? <dispatched[slot_j, :], x[t, :]> : 0    (fp32 planes) */
int planmoe_bwd_gate(const void *x, const void *dispatched, int dtype, const int32_t *indices,
                     const int32_t *locations, int64_t plane_stride, int top_k, int samples,
                     int model_dim, int capacity, float *grad_gates, void *stream);

/* ---------------------------------------------------------------- "int8" codec
 * Replaces Int8Compressor::compress / ::decompress (custom/compressor/int8.cpp:7-60).
 * Per row of row_len elements: bias = min, scale = max - min,
 *   code = uint8(((x - bias) / scale) * 255)      three roundings in `dtype`, truncation;
 *   rows with scale == 0 (e.g. empty capacity slots) encode to 0.
 * bias and scale are written in `dtype` (one element per row).
 *   out  = ((code / 255) * scale) + bias          three roundings in `dtype`. */
int planmoe_int8_compress(const void *x, int dtype, int64_t rows, int row_len, uint8_t *codes,
                          void *bias, void *scale, void *stream);
int planmoe_int8_decompress(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                            int64_t rows, int row_len, void *out, void *stream);

/* Dispatch and compress in one pass (fast_encode followed by Compress.apply with "int8":
 * impls/moe_layer.py:265 then impls/overlap.py:12-16): the codes/bias/scale that
 * planmoe_int8_compress would produce from planmoe_dispatch_fwd's output, without the
 * intermediate [experts*capacity, model_dim] tensor ever reaching memory. */
int planmoe_dispatch_int8(const void *x, int dtype, const float *gates, const int32_t *indices,
                          const int32_t *locations, int64_t plane_stride, int top_k,
                          int samples, int model_dim, int experts, int capacity,
                          uint8_t *codes, void *bias, void *scale,
                          void *workspace, size_t workspace_bytes, void *stream);

/* GatingDecoder.backward followed by the int8 compressor of the backward all-to-all
 * (fast_dispatch.py:66-79, then Decompress.backward = compress_operation, overlap.py:33-34):
 *   grad_expert[slot_j, :] = 0 + gate_j * grad_out[t, :]   -> codes / bias / scale as above,
 *   grad_gates[j][t] = <grad_out[t, :], expert_out[slot_j, :]>  (0 for a dropped pair; fp32 planes
 *   with the same plane_stride).
 * gates must not be NULL (the reference computes gate gradients only for real gates). */
int planmoe_combine_bwd_int8(const void *grad_out, const void *expert_out, int dtype,
                             const float *gates, const int32_t *indices, const int32_t *locations,
                             int64_t plane_stride, int top_k, int samples, int model_dim,
                             int experts, int capacity, uint8_t *codes, void *bias, void *scale,
                             float *grad_gates, void *workspace, size_t workspace_bytes, void *stream);
/* The same with the expert output given as the int8 codes the receive side holds anyway
 * (expert_codes [experts * capacity, model_dim], expert_bias / expert_scale per row, as
 * planmoe_int8_compress wrote them): the rows are decoded on the fly to the values
 * planmoe_int8_decompress would give, so grad_gates and the outputs are bit-identical, and the
 * decompressed copy of the expert output need not exist in the backward pass. */
int planmoe_combine_bwd_int8_coded(const void *grad_out, const uint8_t *expert_codes,
                                   const void *expert_bias, const void *expert_scale, int dtype,
                                   const float *gates, const int32_t *indices,
                                   const int32_t *locations, int64_t plane_stride, int top_k,
                                   int samples, int model_dim, int experts, int capacity,
                                   uint8_t *codes, void *bias, void *scale, float *grad_gates,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* Decompress and combine in one pass (Decompress.apply with "int8" followed by fast_decode:
 * impls/overlap.py:22-29, int8.cpp:46-60, fast_dispatch.py:203-207): what planmoe_combine_fwd
 * produces from planmoe_int8_decompress's output, without the intermediate
 * [experts*capacity, model_dim] tensor.  codes / bias / scale as planmoe_int8_compress writes
 * them; gates fp32 planes or NULL; out [samples, model_dim] in `dtype`.  Needs model_dim a
 * multiple of 8 (bf16/fp16) or 4 (fp32). */
int planmoe_combine_int8(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                         const float *gates, const int32_t *indices, const int32_t *locations,
                         int64_t plane_stride, int top_k, int samples, int model_dim, int capacity,
                         void *out, void *stream);

/* ---------------------------------------------------------------- fused forward chain
 * The layer's forward path up to the all-to-all send buffer in two launches (three when
 * top_k > 4): gate GEMM + routing (gates/top.py:20-26, moe_layer.py:230-256,
 * fast_dispatch.py:140-195), then fast_encode + Int8Compressor::compress
 * (fast_dispatch.py:197-201, int8.cpp:7-44) with the prefix over the routing groups folded in.
 * Limits: experts <= 64, model_dim a multiple of 8 (bf16/fp16) or 4 (fp32), the all-ones gate
 * helper at encode (is_postscore), capacity_factor > 0 routing.
 *
 * x [samples, model_dim] and wg [experts, model_dim] in `dtype`.  fp32_gate != 0: logits,
 * scores and gates are fp32 (top.py:21-23); otherwise they are rounded to `dtype`.
 * gates, logits_out, scores_out are in that score dtype; logits_out / scores_out / l_aux /
 * expert_counts / logit_bias may be NULL.  Other arguments as in planmoe_route_topk.
 * Calls sharing a workspace must not overlap. */
size_t planmoe_forward_workspace_bytes(int samples, int experts, int top_k);

/* gate GEMM + routing only (the outputs of planmoe_gate_logits + planmoe_route_topk) */
int planmoe_gate_route(const void *x, const void *wg, int dtype, int fp32_gate,
                       const float *logit_bias, int samples, int model_dim, int experts, int top_k,
                       int normalize_gate, int32_t *indices, int32_t *locations, void *gates,
                       int64_t plane_stride, void *logits_out, void *scores_out, float *l_aux,
                       int32_t *expert_counts, void *workspace, size_t workspace_bytes, void *stream);

/* gate GEMM + routing + dispatch without a codec (LinearTopKGate + extract_critical + fast_encode with
 * no gates, moe_layer.py:230-266 when no compressor is set): additionally `dispatched`
 * [experts*capacity, model_dim] in `dtype`, equal to what planmoe_dispatch_fwd produces from the same
 * routing (kept rows as 0 + x, empty slots zero).  Two launches; the second works out the slots from
 * the first one's group histograms, so planmoe_gate_route's launch that finishes them is not needed. */
int planmoe_forward_plain(const void *x, const void *wg, int dtype, int fp32_gate,
                          const float *logit_bias, int samples, int model_dim, int experts, int top_k,
                          int normalize_gate, int capacity, int32_t *indices, int32_t *locations,
                          void *gates, int64_t plane_stride, void *logits_out, void *scores_out,
                          float *l_aux, int32_t *expert_counts, void *dispatched,
                          void *workspace, size_t workspace_bytes, void *stream);
/* gate GEMM + routing + dispatch + int8 compress: additionally codes [experts*capacity,
 * model_dim] uint8 and bias / scale [experts*capacity] in `dtype`, equal to what
 * planmoe_dispatch_int8 produces from the same routing. */
int planmoe_forward_int8(const void *x, const void *wg, int dtype, int fp32_gate,
                         const float *logit_bias, int samples, int model_dim, int experts, int top_k,
                         int normalize_gate, int capacity, int32_t *indices, int32_t *locations,
                         void *gates, int64_t plane_stride, void *logits_out, void *scores_out,
                         float *l_aux, int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                         void *workspace, size_t workspace_bytes, void *stream);

/* The same chain in ONE launch that reads x once (the two launches above read it twice: the slot
 * of a second choice needs the first-choice counts of the whole batch).  Work-groups of up to 64
 * tokens, all resident at once, hold the codes of their tokens on chip (LDS and registers) until
 * every work-group has published its expert histogram, then write them to their slots.  Served shapes: bf16, model_dim
 * a multiple of 256 up to 4096, experts <= 16, top_k <= 4, samples <= 64 x the number of work-groups
 * that are resident at once (one per compute unit, two for rows of up to 1792 values:
 * planmoe_forward_int8_single_serves tells); any other shape is an error here, and nothing is enqueued (planmoe_forward_int8
 * takes every shape; the Python layer asks the query and picks).  Outputs as
 * planmoe_forward_int8 (logits may differ from it in the last bit: another summation order).
 * The wait between the work-groups is bounded: spin_limit polls (0 = the default, about a second);
 * a work-group that gives up writes none of its rows, marks its tokens dropped (locations =
 * capacity), makes *l_aux NaN and sets *gave_up to 1 (device word, cleared by the caller): the
 * caller reads that word before it uses any output and, if it is set, runs planmoe_forward_int8.
 * Two such launches that run at the same time on one GPU could keep each other's work-groups from
 * becoming resident, so the library puts them in a row: a launch on another stream than the one
 * before it on the same device first waits (on the device) for an event recorded at the tail of
 * that earlier stream.  Launches recorded into a HIP graph are outside that order: keep replays
 * of such graphs apart.
 * The first FWD region of the workspace (its launch counter and published words) is written by
 * this entry point alone; the other entry points that take a forward workspace keep their tables
 * behind it, so one workspace may serve all of them in turn, whatever the shapes.
 * It has no counterpart in the reference. */
int planmoe_forward_int8_single(const void *x, const void *wg, int dtype, int fp32_gate,
                                const float *logit_bias, int samples, int model_dim, int experts,
                                int top_k, int normalize_gate, int capacity, int32_t *indices,
                                int32_t *locations, void *gates, int64_t plane_stride,
                                void *logits_out, void *scores_out, float *l_aux,
                                int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                                void *workspace, size_t workspace_bytes, int spin_limit,
                                int32_t *gave_up, void *stream);

/* 1 if planmoe_forward_int8_single takes the shape on the current device, else 0: the limits above,
 * and every work-group of the launch resident at once (work-groups of at most 64 tokens; rows of up
 * to 1792 values leave room for two of them per compute unit, so twice the tokens).  Asks the
 * runtime once per kernel and device; launches nothing.  No counterpart in the reference: for
 * callers that pick between the two forward entry points (the Python layer does). */
int planmoe_forward_int8_single_serves(int dtype, int fp32_gate, int samples, int model_dim, int experts, int top_k);

/* A measuring stick for planmoe_forward_int8_single, not a product path: one launch with that
 * kernel's grid, its loads of x, one exchange of tagged words between all work-groups and its
 * streaming stores (every row of codes [experts*capacity, 4096], bias, scale, and planes =
 * 3 x [2][samples] int32 standing for indices / locations / gates), and none of its arithmetic.
 * What it writes means nothing; what it takes is the floor under that way of moving the bytes on
 * the GPU at hand.  mode 0: read everything, exchange, store everything (the structure of
 * planmoe_forward_int8_single); mode 1: the same with nobody waiting at the exchange, i.e. what the
 * loads and stores alone cost when no slot depends on another work-group (the floor under any
 * arrangement of them); mode 2: tokens dealt in two halves, the first-choice rows of the first
 * half stored while the second half is read, one more exchange.  Serves model_dim 4096 bf16,
 * 8 experts, top-2, samples a multiple of 128, capacity >= samples / 4.  Workspace, spin_limit,
 * gave_up and the ordering of launches as for planmoe_forward_int8_single (it uses the same
 * region of the workspace).  It has no counterpart in the reference. */
int planmoe_forward_int8_single_ceiling(const void *x, int samples, int model_dim, int experts, int top_k,
                                        int capacity, uint8_t *codes, void *bias, void *scale,
                                        int32_t *planes, void *workspace, size_t workspace_bytes,
                                        int mode, int spin_limit, int32_t *gave_up, void *stream);

/* planmoe_forward_int8 for callers that cannot allocate device memory or carry a workspace
 * around (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * the same launches with the workspace taken from a 4 MiB buffer built into the library's device
 * image (a static __device__ array; every GPU the library runs on holds its own copy until the
 * process ends).  It has no counterpart in the reference.  Calls no allocator.  Shapes whose
 * planmoe_forward_workspace_bytes exceed 4 MiB are refused with an error (the five benchmark
 * configurations need 0.4 - 1.7 MiB).  All calls on one GPU share that GPU's buffer, which keeps
 * the previous call's contents: calls that overlap on one GPU (two streams, two threads) race;
 * calls on one stream do not.  The first call on a device looks the buffer's address up
 * (hipGetSymbolAddress): make that call outside a graph capture.  Outputs as planmoe_forward_int8. */
int planmoe_forward_int8_static(const void *x, const void *wg, int dtype, int fp32_gate,
                                const float *logit_bias, int samples, int model_dim, int experts,
                                int top_k, int normalize_gate, int capacity, int32_t *indices,
                                int32_t *locations, void *gates, int64_t plane_stride,
                                void *logits_out, void *scores_out, float *l_aux,
                                int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                                void *stream);

/* Runs only the last launch of planmoe_forward_int8 (slot finalisation + dispatch + int8
 * compress) again, from the state a preceding planmoe_forward_int8 call with the same shapes
 * left in `workspace`.  Same outputs; meant for profiling that launch on its own.  It has no
 * counterpart in the reference. */
int planmoe_forward_int8_redispatch(const void *x, int dtype, int samples, int model_dim,
                                    int experts, int top_k, int capacity, const int32_t *indices,
                                    int32_t *locations, int64_t plane_stride, uint8_t *codes,
                                    void *bias, void *scale, void *workspace, size_t workspace_bytes,
                                    void *stream);

/* ---------------------------------------------------------------- expert FFN on int8 codes
 * The first batched GEMM of FusedExpertsNetwork.forward (experts/ffn.py:77) with the receive
 * side's Int8Compressor::decompress (int8.cpp:46-60, reached from overlap.py:66) as its prologue:
 *   out[e][r][n] = bf16( bf16( sum_k dec(e, r, k) * w[e][n][k] ) + fc_bias[e][n] )
 * where dec(e, r, k) is the bf16 value planmoe_int8_decompress would have stored for code
 * codes[e][r][k] with bias[e][r], scale[e][r].  The decoded [experts, rows, model_dim] tensor
 * never exists in memory.  weight_k_major is the layer's batched_fc1_w [experts, model_dim,
 * hidden] transposed to [experts, hidden, model_dim] (k fastest: what both MFMA operands want);
 * fc_bias [experts, hidden] may be NULL.  bf16 only; model_dim a multiple of 64, hidden of 128.
 * Results equal torch.matmul on the decompressed tensor up to the order of the fp32 sums. */
int planmoe_ffn_fc1_int8(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                         const void *weight_k_major, const void *fc_bias, int experts, int rows,
                         int model_dim, int hidden, void *out, void *stream);

/* The same step (int8.cpp:46-60 + experts/ffn.py:77) with the row's affine map taken out of the
 * sum: the matrix cores multiply the codes themselves and the epilogue applies
 *   out[e][r][n] = bf16( bf16( scale[e][r] / 255 * sum_k code[e][r][k] w[e][n][k]
 *                              + bias[e][r] * weight_colsum[e][n] ) + fc_bias[e][n] )
 * weight_colsum [experts, hidden] fp32 = sum over model_dim of weight_k_major, computed by the
 * caller once per weight.  Skips the three bf16 roundings Int8Compressor::decompress applies to
 * every element (and their arithmetic: fifteen instructions per two codes against three), so it
 * agrees with decompress + GEMM to about one ulp of the bf16 result (tolerance-level parity) and is
 * the faster of the two.  Same shape limits as planmoe_ffn_fc1_int8. */
int planmoe_ffn_fc1_int8_affine(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                                const void *weight_k_major, const float *weight_colsum,
                                const void *fc_bias, int experts, int rows, int model_dim, int hidden,
                                void *out, void *stream);

/* ---------------------------------------------------------------- expert FFN: batched bf16 GEMM
 * The batched matrix products of FusedExpertsNetwork (experts/ffn.py:63-82: x @ batched_fc1_w,
 * activation, @ batched_fc2_w, each followed by torch.add of the bias) and of their backward pass,
 * on the matrix cores, in the one form a matrix-core operand wants: both operands with the
 * reduction index running fastest,
 *   c[e][i][j] = act( bf16( bf16( sum_k a[e][i][k] * b[e][j][k] ) + bias[e][j] ) )
 * a [batches, m, k] with rows lda elements apart, b [batches, n, k] (ldb), c [batches, m, n] (ldc),
 * all bf16, batches batch_stride_* elements apart; bias [batches, n] bf16 or NULL (then the sum is
 * rounded once); activation 0 = none, 1 = relu (the reference's default activation_fn).  The sum is
 * kept in fp32.  k, n and the pitches must be multiples of 8, one batch of an operand under 4 GiB.
 *   forward   y  = x @ W (+ bias):  a = x,  b = W transposed to [out, in] (planmoe_transpose_bf16)
 *   backward  dx = dy @ W^T:        a = dy, b = W as stored [in, out]
 *             dW = x^T @ dy:        a = x^T [in, rows], b = dy^T [out, rows] (transposed copies whose
 *                                   k dimension planmoe_transpose_bf16 pads with zeros) */
int planmoe_gemm_nt_bf16(const void *a, const void *b, const void *bias, int activation, int batches,
                         int m, int n, int k, int lda, int ldb, int ldc, int64_t batch_stride_a,
                         int64_t batch_stride_b, int64_t batch_stride_c, void *c, void *stream);

/* c[e] = act(bf16(bf16(a[e] b[e]) + bias[e])) for bf16 a [batches, m, k] and b [batches, k, n] with n the
 * fast index -- a weight as experts/ffn.py:33-56 stores it, [E, in, out]: the matmul + add of
 * ffn.py:77-79 with no transposed copy of the weight.  k a multiple of 64; n and the pitches multiples
 * of 8; bias, activation, roundings and the order of the sums as planmoe_gemm_nt_bf16. */
int planmoe_gemm_nn_bf16(const void *a, const void *b, const void *bias, int activation, int batches,
                         int m, int n, int k, int lda, int ldb, int ldc, int64_t batch_stride_a,
                         int64_t batch_stride_b, int64_t batch_stride_c, void *c, void *stream);

/* c[e] = a[e]^T b[e] for bf16 a [batches, k, m], b [batches, k, n] (row pitches lda >= m, ldb >= n,
 * the reduction index the slow one) -> c [batches, m, n] bf16, fp32 sums, one rounding: the weight
 * gradient matmul(x.transpose(1, 2), dy) of the autograd of experts/ffn.py:77-79 with both operands
 * as they lie in memory (no transposed copies; the fragments are transposed on their way out of
 * LDS).  k a multiple of 64; m, n and the pitches multiples of 8; sums in the order of
 * planmoe_gemm_nt_bf16 on transposed copies. */
int planmoe_gemm_tn_bf16(const void *a, const void *b, int batches, int m, int n, int k, int lda, int ldb,
                         int ldc, int64_t batch_stride_a, int64_t batch_stride_b, int64_t batch_stride_c,
                         void *c, void *stream);

/* out[e][j][i] = in[e][i][j] for bf16 matrices [batches, rows, cols] -> [batches, cols, rows_out];
 * rows_out >= rows, the columns rows .. rows_out - 1 of out are zero (padding of a reduction index).
 * cols and rows_out multiples of 8.  Stands for the .transpose(...).contiguous() the GEMM form
 * above needs for the weights of experts/ffn.py:33-56 and for the operands of their gradients. */
int planmoe_transpose_bf16(const void *in, int batches, int rows, int cols, int rows_out, void *out,
                           void *stream);

/* ---------------------------------------------------------------- zfp fixed-rate codec
 * Replaces ZfpCompressor::compress / ::decompress (custom/compressor/zfpc.cpp:23-86), i.e.
 * zfp_compress / zfp_decompress of the third-party zfp library in fixed-rate mode on fp32.
 * The stream is bit-identical to stock zfp 0.5.5 (64-bit words, no header).
 *   dims = 2: the reference's call, field nx = fastest axis, ny rows, 4x4 blocks;
 *   dims = 1: the nx*ny values as one array, blocks of 4.
 * nx and ny must be multiples of 4 (zfpc.cpp:26-28); maxbits = floor(4^dims * rate + 0.5)
 * must be a multiple of 32 (rate 8, the reference's default zfpc.h:17, qualifies in both). */

/* zfp_stream_maximum_size for the field: what the reference sizes its buffer with (zfpc.cpp:39) */
size_t planmoe_zfp_max_bytes(int dims, int64_t nx, int64_t ny, double rate);
/* bytes zfp_compress returns (`length`, zfpc.cpp:48) */
size_t planmoe_zfp_stream_bytes(int dims, int64_t nx, int64_t ny, double rate);

int planmoe_zfp_compress(const float *field, int dims, int64_t nx, int64_t ny, double rate,
                         void *stream_out, size_t stream_capacity, void *stream);
int planmoe_zfp_decompress(const void *stream_in, int dims, int64_t nx, int64_t ny, double rate,
                           float *field, void *stream);

/* fast_encode followed by ZfpCompressor::compress in one pass (GatingEncoder.forward,
 * fast_dispatch.py:26-29, then zfpc.cpp:23-51; with `gates` also GatingDecoder.backward's scatter,
 * fast_dispatch.py:69-71, followed by Decompress.backward's compress, overlap.py:32-34): the
 * stream is that of planmoe_zfp_compress(dims = 2, nx = model_dim, ny = experts * capacity) on
 * the buffer planmoe_dispatch_fwd would have written, and that buffer never exists.  fp32 only (the
 * codec reads its field as fp32, zfpc.cpp:31); model_dim and experts * capacity multiples of 4;
 * gates may be NULL (gate = 1). */
size_t planmoe_dispatch_zfp_workspace_bytes(int experts, int capacity);
int planmoe_dispatch_zfp(const float *x, const float *gates, const int32_t *indices,
                         const int32_t *locations, int64_t plane_stride, int top_k, int samples,
                         int model_dim, int experts, int capacity, double rate, void *stream_out,
                         size_t stream_capacity, void *workspace, size_t workspace_bytes, void *stream);

/* ZfpCompressor::decompress followed by fast_decode in one pass (zfpc.cpp:66-86, then
 * GatingDecoder.forward, fast_dispatch.py:59-64; without gates GatingEncoder.backward's gather,
 * fast_dispatch.py:33-38): out[t] = sum over the choices of token t, left to right, of
 * gate * (decoded slot row), bit for bit what planmoe_zfp_decompress + planmoe_combine_fwd give,
 * and the decoded buffer never exists (empty slots are not even decoded).  fp32, 2-D stream with
 * nx = model_dim, ny = experts * capacity; gates may be NULL (gate = 1).  2 + 2 * top_k launches. */
size_t planmoe_combine_zfp_workspace_bytes(int experts, int capacity);
int planmoe_combine_zfp(const void *stream_in, double rate, const float *gates, const int32_t *indices,
                        const int32_t *locations, int64_t plane_stride, int top_k, int samples,
                        int model_dim, int experts, int capacity, float *out, void *workspace,
                        size_t workspace_bytes, void *stream);

/* The gate gradients of GatingDecoder.backward (create_backward_gate, fast_dispatch.py:73-78)
 * straight from the stream of the expert output that the decode consumed (what
 * ZfpCompressor::decompress would have produced, zfpc.cpp:66-86):
 * grad_gates[j][t] = <grad_out[t], decoded slot row of choice j>, 0 for a choice without a slot;
 * what planmoe_zfp_decompress + planmoe_bwd_gate give to rounding (the sum runs in another
 * order), without the decoded buffer.  fp32, 2-D stream with nx = model_dim, ny = experts *
 * capacity; workspace as for planmoe_combine_zfp.  4 launches. */
int planmoe_bwd_gate_zfp(const void *stream_in, double rate, const float *grad_out, const int32_t *indices,
                         const int32_t *locations, int64_t plane_stride, int top_k, int samples,
                         int model_dim, int experts, int capacity, float *grad_gates, void *workspace,
                         size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- GPULZ ("lz") lossless codec
 * Replaces lz_compress / lz_decompress (custom/compressor/gpulz.cu:408-535), the codec behind
 * LzCompressor (custom/compressor/lz.cpp:3-60).  The input is taken as 32-bit symbols in blocks
 * of 2048 bytes (512 symbols); a block holds one flag bit per token (least significant bit
 * first, 1 = match) and the token bytes: 4 for a literal symbol, 2 (length, offset) for a match
 * into the 32 symbols before it.  Symbols are compared as floats (gpulz.cu:62): +0 equals -0, a
 * NaN equals nothing.  Streams are byte-identical to the reference's four tensors:
 *   flag_offsets, data_offsets   int32 [blocks + 1]   exclusive prefix sums of the per-block sizes
 *   flags                        uint8 [blocks * 64]  zero beyond flag_offsets[blocks]
 *   data                         uint8 [blocks * 2048] zero beyond data_offsets[blocks]
 * with blocks = planmoe_lz_blocks(nbytes).  nbytes must be a multiple of 4 and below 2^31; a
 * last partial block is coded as if padded with zero symbols (the reference reads past the end
 * of its input there, gpulz.cu:36-39), and decoding writes only the first nbytes.
 * Compression sizes every block, scans the sizes in place in the offset tables and then packs
 * every block at its final offset; there is no full-size staging buffer (gpulz.cu:148-211,
 * 220-258 have two).  All five pointers must be 16-byte aligned. */
int64_t planmoe_lz_blocks(int64_t nbytes);
size_t planmoe_lz_workspace_bytes(int64_t nbytes);
int planmoe_lz_compress(const void *input, int64_t nbytes, int32_t *flag_offsets, int32_t *data_offsets,
                        uint8_t *flags, uint8_t *data, void *workspace, size_t workspace_bytes,
                        void *stream);
/* Streams that this coder cannot have written (offsets out of order, a match that reaches
 * before its block) never make the kernel read or write out of bounds; the symbols they cover
 * decode as zero. */
int planmoe_lz_decompress(void *output, int64_t nbytes, const int32_t *flag_offsets,
                          const int32_t *data_offsets, const uint8_t *flags, const uint8_t *data,
                          void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PLANMOE_HIP_H */
