/* C ABI of libtgo_hip.so: MI355X (gfx950) kernels for matmul against packed GGUF weights.
 *
 * Every pointer is a device pointer unless stated otherwise, every size is in elements of
 * the named unit, `stream` is a hipStream_t passed as void*.  A function returns 0 on
 * success; on failure it launches nothing, returns a TGO_ERR_* code and leaves a message in
 * tgo_last_error() (thread local).  Nothing here allocates, synchronises or copies to the
 * host: the caller owns outputs and workspaces and sizes them with the *_bytes() helpers.
 *
 * Data formats
 *   activations, cotangents, outputs : bf16, row-major, 16-byte aligned
 *   packed weights                   : raw GGUF super-blocks, uint8 [rows, (K/256)*block_bytes]
 *                                      (grouped: [experts, rows, ...]), 16-byte aligned
 *   quant_type                       : ggml ids  Q3_K=11 Q4_K=12 Q5_K=13 Q6_K=14 IQ2_S=22
 *   expert_indices / expert_offsets  : int64 [G] expert of each group / int32 [G] inclusive
 *                                      cumulative row ends of expert-sorted rows
 *
 * The entry points replace the launcher seam of the reference extension; each comment names
 * the reference host function it stands in for (paths relative to the reference checkout).
 */
#ifndef TGO_H
#define TGO_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TGO_OK 0
#define TGO_ERR_INVALID 1   /* argument rejected before launch             */
#define TGO_ERR_HIP 2       /* a HIP runtime call or kernel launch failed  */

#define TGO_TYPE_Q3_K 11
#define TGO_TYPE_Q4_K 12
#define TGO_TYPE_Q5_K 13
#define TGO_TYPE_Q6_K 14
#define TGO_TYPE_IQ2_S 22

/* Library version (major*10000 + minor*100 + patch). */
int tgo_version(void);

/* Message of the last failure on the calling thread ("" if none). Host pointer. */
const char * tgo_last_error(void);

/* Bytes of one 256-weight super-block, 0 for an unsupported type.
 * Replaces packed_block_bytes(), csrc/mmq_hip.cu:38-48. */
int tgo_block_bytes(int quant_type);

/* Bytes of the activation workspace the forward entry points need for `rows` rows of
 * `in_features` values: q8_1 blocks (two bytes per value, one fp32 scale and one fp32 sum per 32
 * values, for the scaled operands also a power of two and 16 bytes of block sums per 256 values and a power of
 * two per row), rows padded to 32.  The arrangement inside is the library's business (32-row tiles in MFMA
 * fragment order holding the quants as int8, as fp16 numbers or as scaled fp16 values, see
 * tgo_set_forward_operand, or plain int8 rows for decode-sized calls); tgo_q8_workspace_unpack reads any of them.
 * Replaces the workspace sizing in csrc/mmq_hip.cu:643-652 and :529-537. */
int64_t tgo_q8_workspace_bytes(int64_t rows, int64_t in_features);

/* Bytes of the tile-task list the grouped entry points build on the device
 * (2 counters + 3 int32 per task, at most ceil(rows/tile)+groups tasks, sized for the smallest tile).
 * Replaces new_grouped_row_task_workspace(), csrc/mmq_hip.cu:548-558. */
int64_t tgo_task_workspace_bytes(int64_t rows, int64_t num_groups);

/* Dequantize packed rows to bf16 [rows, in_features]; bit-exact with the reference's scalar
 * decoder decode_gguf_value<type>, csrc/ck/gguf_decode.cuh:54-149, followed by
 * __float2bfloat16. */
int tgo_dequant_bf16(const void * packed, void * out_bf16, int64_t rows, int64_t in_features,
                     int quant_type, void * stream);

/* Quantize bf16 [rows, in_features] to q8_1 blocks in `workspace`
 * (tgo_q8_workspace_bytes).  Same arithmetic as quantize_bf16_mmq_q8_1,
 * csrc/mmq_core.cuh:151-209, with scale and sum kept in fp32. */
int tgo_quantize_q8_1(const void * input_bf16, void * workspace, int64_t rows,
                      int64_t in_features, void * stream);

/* Copies the q8_1 workspace into plain row-major arrays for inspection:
 * q int8 [rows, K], d fp32 [rows, K/32], sum fp32 [rows, K/32]. */
int tgo_q8_workspace_unpack(const void * workspace, void * q_int8, void * d_f32, void * sum_f32,
                            int64_t rows, int64_t in_features, void * stream);

/* output[rows, out_features] = bf16( input[rows, in_features] x W^T ), activations quantized
 * to q8_1, int8 MFMA dot products per block, fp32 scales and accumulation.
 * Decode-sized calls of Q3_K / Q6_K / IQ2_S (dense: at most 8 rows; grouped: at most 64 rows that
 * average at most 4 per listed group, over at most 1024 listed groups) are a single launch whose workgroups quantize their own rows
 * (same q8_1 arithmetic) and, in the grouped entry points, find their task in the group list; such a
 * call leaves `workspace` untouched.
 * Replaces launch_dense_mmq<type>, csrc/mmq_hip.cu:117-147 (called by mmq_cuda, :587-678). */
int tgo_mmq_forward(const void * input_bf16, const void * packed, void * output_bf16,
                    void * workspace, int64_t rows, int64_t in_features, int64_t out_features,
                    int quant_type, void * stream);

/* tgo_mmq_forward without a workspace argument and without any allocation: the q8_1 activation
 * workspace is a fixed array inside the library's code object (one copy per GPU, held until the
 * process ends), TGO_STATIC_WORKSPACE_BYTES large.  Calls whose
 * tgo_q8_workspace_bytes(rows, in_features) exceeds that are rejected with TGO_ERR_INVALID and a
 * message; nothing is launched then.  Results are bit-identical to tgo_mmq_forward.  All calls on
 * one GPU share the array: calls that overlap in time on one GPU (different streams or threads)
 * race on it and must be serialised by the caller.  The array's address is looked up on the first
 * call on each device (hipGetSymbolAddress, no allocation), so make that first call outside any
 * stream capture.  No counterpart in the reference (its dense operator allocates its workspace
 * through torch, csrc/mmq_hip.cu:646-652); this is for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc. */
#define TGO_STATIC_WORKSPACE_BYTES (4 * 1024 * 1024)
int tgo_mmq_forward_static(const void * input_bf16, const void * packed, void * output_bf16,
                           int64_t rows, int64_t in_features, int64_t out_features, int quant_type,
                           void * stream);

/* The second half of tgo_mmq_forward alone: `workspace` already holds the q8_1 form of the
 * activations (written by tgo_quantize_q8_1 for the same rows and in_features) and is only read.
 * Several projections of one input (q/k/v, shared gate/up) quantize once and call this once per
 * weight; results are bit-identical to tgo_mmq_forward.  No counterpart in the reference, which
 * quantizes inside every dense call (csrc/mmq_hip.cu:643-665) and names the reuse as its next
 * step (docs/mmq_fwd_optimization.md:299-307). */
int tgo_mmq_forward_prepared(const void * workspace, const void * packed, void * output_bf16,
                             int64_t rows, int64_t in_features, int64_t out_features,
                             int quant_type, void * stream);

/* tgo_quantize_q8_1 and tgo_mmq_forward_prepared for a caller that names the operand kind itself
 * (TGO_OPERAND_INT8, TGO_OPERAND_HALF or TGO_OPERAND_SCALED, see tgo_set_forward_operand) instead of
 * leaving it to the setting: a caller that knows every projection it will run on the workspace
 * asks tgo_forward_operand_for with their summed out_features and passes the answer to both, which
 * gives several large projections of one input the scaled kernels that a single large call gets.
 * Both calls must name the same kind; outputs turn into NaN when they do not.  No counterpart in
 * the reference. */
int tgo_quantize_q8_1_as(const void * input_bf16, void * workspace, int64_t rows, int64_t in_features,
                         int operand, void * stream);
int tgo_mmq_forward_prepared_as(const void * workspace, const void * packed, void * output_bf16,
                                int64_t rows, int64_t in_features, int64_t out_features,
                                int quant_type, int operand, void * stream);

/* Bytes of the workspace of the grad-input entry points: the cotangent(s) copied into MFMA
 * fragment order (rows padded to 32, columns to 16), preceded by the task list when
 * num_groups > 0.  `sources` is 1, or 2 for the fused pair; num_groups is 0 for the dense call.
 * No counterpart in the reference, whose kernels read the cotangent row-major
 * (csrc/ck/mmq_backward.cuh:855-874). */
int64_t tgo_grad_workspace_bytes(int64_t rows, int64_t out_features, int64_t num_groups, int sources);

/* Bytes of `workspace` for tgo_mmq_grad_input: the packed cotangent as above, plus, for calls of so
 * few rows that whole reductions per workgroup would leave most of the chip idle, room for the
 * fp32 partial results of a reduction split over several workgroups (added up in a fixed order);
 * which calls split depends on the format, hence `quant_type`.
 * No counterpart in the reference.  -1 on invalid sizes. */
int64_t tgo_dense_grad_workspace_bytes(int64_t rows, int64_t out_features, int64_t in_features,
                                       int quant_type);

/* grad_input[rows, in_features] = bf16( grad_output[rows, out_features] x bf16(W) ), weights
 * dequantized to bf16 in LDS, bf16 MFMA, fp32 accumulation, one rounding.
 * `workspace` holds tgo_dense_grad_workspace_bytes(rows, out_features, in_features, quant_type) bytes.
 * Replaces launch_dense_mmq_grad_input<type>, csrc/ck/mmq_backward.cuh:1066-1241. */
int tgo_mmq_grad_input(const void * grad_output_bf16, const void * packed, void * grad_input_bf16,
                       void * workspace, int64_t rows, int64_t out_features, int64_t in_features,
                       int quant_type, void * stream);

/* Grouped forward over expert-sorted rows: group g covers rows [offsets[g-1], offsets[g]) and
 * uses the weights of expert indices[g]; invalid or empty groups are skipped, rows outside
 * every group are left untouched.  `packed_second`/`output_second` may both be NULL (single
 * projection) or both set (gate+up pair sharing one q8_1 workspace).
 * `workspace` holds tgo_q8_workspace_bytes() + tgo_task_workspace_bytes() bytes.
 * Replaces launch_grouped_quantize / launch_grouped_row_task_setup /
 * launch_grouped_row_task_projection / launch_grouped_projection, csrc/mmq_hip.cu:149-314
 * (called by grouped_mmq_cuda :954-1052 and grouped_mmq_pair_cuda :1054-1193). */
int tgo_grouped_mmq_forward(const void * input_bf16, const void * packed_first,
                            const void * packed_second, void * output_first, void * output_second,
                            const int64_t * expert_indices, const int32_t * expert_offsets,
                            void * workspace, int64_t rows, int64_t in_features,
                            int64_t out_features, int64_t num_experts, int64_t num_groups,
                            int quant_type, void * stream);

/* tgo_grouped_mmq_forward with the token -> expert-sorted-row gather folded into the quantizer:
 * row r of the operator is row row_index[r] of input_bf16[input_rows, in_features] (an index outside
 * [0, input_rows) gives a row of zeros).  The sorted copy of the activations that a caller would
 * otherwise build (read and write of rows x in_features bf16) is never materialised.
 * No counterpart in the reference, whose grouped operators take pre-sorted rows
 * (torch_ggml_ops/grouped_mmq.py:216); for callers that hold unsorted token activations. */
int tgo_grouped_mmq_forward_gathered(const void * input_bf16, const int64_t * row_index,
                                     int64_t input_rows, const void * packed_first,
                                     const void * packed_second, void * output_first,
                                     void * output_second, const int64_t * expert_indices,
                                     const int32_t * expert_offsets, void * workspace, int64_t rows,
                                     int64_t in_features, int64_t out_features, int64_t num_experts,
                                     int64_t num_groups, int quant_type, void * stream);

/* Gate/up pair with the SwiGLU activation fused into the epilogue: output_gate[rows, out_features] is the
 * first projection as tgo_grouped_mmq_forward writes it, output_activated[rows, out_features] is
 * bf16( silu(gate) * up ) with gate and up rounded to bf16 first, i.e. what the caller-side
 * silu(gate) * up computes from the pair's outputs, up to one rounding less.  With int8 or exact fp16
 * operands the up projection is never written and no activation kernel re-reads the pair; with the scaled
 * operands of large calls the up projection passes through output_activated and an elementwise launch
 * replaces it (same values; still faster than the other kinds at that size).  `row_index` may be NULL (rows are input rows) or the
 * gather index of tgo_grouped_mmq_forward_gathered.  Same workspace as tgo_grouped_mmq_forward.  Calls of
 * decode size run the pair in the decode-regime kernels and the same elementwise launch.  No counterpart in the reference, whose pair operator returns both projections
 * (grouped_mmq_pair_cuda, csrc/mmq_hip.cu:1054-1193) and leaves the activation to the caller. */
int tgo_grouped_mmq_swiglu(const void * input_bf16, const int64_t * row_index, int64_t input_rows,
                           const void * packed_gate, const void * packed_up, void * output_gate,
                           void * output_activated, const int64_t * expert_indices,
                           const int32_t * expert_offsets, void * workspace, int64_t rows,
                           int64_t in_features, int64_t out_features, int64_t num_experts,
                           int64_t num_groups, int quant_type, void * stream);

/* activated[i] = bf16( silu(gate[i]) * up[i] ) over `count` bf16 values, fp32 arithmetic: the elementwise pass that
 * tgo_grouped_mmq_swiglu runs itself after a scaled-operand pair, for a caller that ran the pair (tgo_grouped_mmq_forward)
 * and wants to keep the up projection, e.g. for the backward pass.  `activated_bf16` may be `up_bf16`.  No counterpart in
 * the reference (the activation is the caller's tensor operation there, csrc/mmq_hip.cu:1054-1193). */
int tgo_swiglu_rows(const void * gate_bf16, const void * up_bf16, void * activated_bf16, int64_t count, void * stream);

/* The cotangent of tgo_grouped_mmq_swiglu's activated output taken back to the two projections, elementwise over
 * `count` bf16 values: with s = sigmoid(gate),
 *   d_up = bf16(grad_activated * gate * s),   d_gate = bf16(grad_activated * up * s * (1 + gate * (1 - s)) + grad_gate),
 * every factor read as bf16, the arithmetic in fp32.  `grad_gate_bf16` (a cotangent of the gate output itself) may be
 * NULL.  d_gate and d_up are what tgo_grouped_mmq_grad_input takes as its two cotangents.  No counterpart in the
 * reference, whose pair operator leaves the activation and its derivative to the caller's tensor operations
 * (csrc/mmq_hip.cu:1054-1193). */
int tgo_swiglu_backward(const void * gate_bf16, const void * up_bf16, const void * grad_activated_bf16,
                        const void * grad_gate_bf16, void * d_gate_bf16, void * d_up_bf16, int64_t count, void * stream);

/* Routing of a small batch in one launch: the [tokens, top_k] expert choices sorted by expert (stable), as the
 * metadata the grouped entry points take, with one group per expert:
 *   slot_rows int64 [tokens * top_k]       sorted row of each (token, choice) slot; -1 for an expert outside [0, num_experts)
 *   row_index int64 [tokens * top_k]       token of each sorted row (the gather index of the gathered entry points);
 *                                          -1 behind the last row
 *   expert_indices int64 [num_experts]     0, 1, 2, ...
 *   expert_offsets int32 [num_experts]     rows of experts 0..e
 * At most TGO_ROUTE_SMALL_LIMIT slots and experts (one workgroup sorts them); larger batches are sorted by the caller.
 * No counterpart in the reference, whose callers sort with tensor operations (torch_ggml_ops/grouped_mmq.py:216 takes
 * the sorted metadata); at decode sizes those operations are a dozen launches, more than the layer's own. */
#define TGO_ROUTE_SMALL_LIMIT 4096
int tgo_route_small(const int64_t * slot_experts, int64_t tokens, int64_t top_k, int64_t num_experts, int64_t * row_index,
                    int64_t * slot_rows, int64_t * expert_indices, int32_t * expert_offsets, void * stream);

/* The row gather of the gathered entry points run backwards: the gradients of the sorted rows summed per token,
 *   output[t, :] = bf16( sum of rows[order[i], :] for starts[t] <= i < starts[t + 1] )      (t < tokens)
 * rows bf16 [num_rows, features]; order int64 [num_rows] lists the sorted rows token by token (a stable sort of the
 * gather index: rows of one token stay in row order); starts int64 [tokens + 1] is where each token's run begins.  The
 * rows of a run are added in list order in fp32 and rounded once: no atomics, the same bits on every run.  Entries of
 * `order` outside [0, num_rows) and the parts of a run outside the list contribute nothing, so rows whose gather index
 * named no token are left out by ending the last run before them.  `features` is a multiple of 8.  No counterpart in
 * the reference, whose operators take expert-sorted rows and leave gather and scatter to the caller
 * (torch_ggml_ops/grouped_mmq.py:216). */
int tgo_rows_to_tokens(const void * rows_bf16, const int64_t * order, const int64_t * starts, void * output_bf16,
                       int64_t tokens, int64_t num_rows, int64_t features, void * stream);

/* Routing-weighted return from expert-sorted rows to tokens:
 *   output[t, :] = sum_j slot_weights[t, j] * rows[slot_rows[t, j], :]      (t < tokens, j < top_k)
 * rows bf16 [num_rows, features], slot_rows int64 [tokens, top_k] (the sorted row of each choice; a value
 * outside [0, num_rows) contributes nothing), slot_weights fp32 [tokens, top_k], output bf16
 * [tokens, features].  Choices are accumulated in index order in fp32 and rounded once, so the result is
 * deterministic (no atomics).  `features` is a multiple of 8.  One pass over the rows replaces the caller-side
 * scale and index_add of a MoE layer.  No counterpart in the reference, which leaves this to the caller
 * (its grouped operators end at expert-sorted rows, torch_ggml_ops/grouped_mmq.py:216). */
int tgo_moe_combine(const void * rows_bf16, const int64_t * slot_rows, const float * slot_weights,
                    void * output_bf16, int64_t tokens, int64_t top_k, int64_t num_rows, int64_t features,
                    void * stream);

/* Grouped grad-input.  With `grad_output_second`/`packed_second` set, both Jacobian products
 * are summed in one fp32 accumulator and rounded once.  `workspace` holds
 * tgo_grad_workspace_bytes(rows, out_features, num_groups, 1 or 2) bytes.
 * Replaces launch_grouped_mmq_grad_input<type>, csrc/ck/grouped_mmq_backward.cuh:154-306, and
 * launch_grouped_mmq_pair_grad_input<type>, :460-568. */
int tgo_grouped_mmq_grad_input(const void * grad_output_first, const void * grad_output_second,
                               const void * packed_first, const void * packed_second,
                               void * grad_input_bf16, const int64_t * expert_indices,
                               const int32_t * expert_offsets, void * workspace, int64_t rows,
                               int64_t out_features, int64_t in_features, int64_t num_experts,
                               int64_t num_groups, int quant_type, void * stream);

/* tgo_grouped_mmq_grad_input (single projection) with the routing-weighted return of a mixture-of-experts
 * layer, run backwards, folded into the cotangent's packing: cotangent row r of the operator is
 *   bf16( row_weight[r] * grad_tokens[row_token[r], :] )        (fp32 product, one rounding)
 * with grad_tokens bf16 [tokens, out_features] the gradient of the layer's per-token output, row_token int64
 * [rows] the token of each expert-sorted row and row_weight fp32 [rows] its routing weight; a row whose token
 * lies outside [0, tokens) has a zero cotangent.  (One token and weight per row: this is the backward of
 * tgo_moe_combine only for slot_rows that name every row at most once.)  The expert-sorted cotangent that the caller would otherwise
 * build from the gradient of tgo_moe_combine (rows x out_features bf16, written and read again) is never
 * materialised.  Same workspace as tgo_grouped_mmq_grad_input with one source.  No counterpart in the reference,
 * which leaves the combine and its gradient to the caller (torch_ggml_ops/grouped_mmq.py:216). */
int tgo_grouped_mmq_grad_input_weighted(const void * grad_tokens_bf16, const int64_t * row_token,
                                        const float * row_weight, int64_t tokens, const void * packed,
                                        void * grad_input_bf16, const int64_t * expert_indices,
                                        const int32_t * expert_offsets, void * workspace, int64_t rows,
                                        int64_t out_features, int64_t in_features, int64_t num_experts,
                                        int64_t num_groups, int quant_type, void * stream);

/* Name of the kernel family the forward entry points pick for a shape ("mfma" or "gemv");
 * host pointer to a static string.  Lets callers and benchmarks label what they measure. */
const char * tgo_forward_kernel_family(int64_t rows, int64_t num_groups);

/* ---- optional per-kernel timing (benchmarks only) ---------------------------------------
 * While enabled, every kernel launch of the library is bracketed by a pair of HIP events
 * recorded on the launch's own stream.  This is the one place where the library creates
 * runtime objects (the events) and, in tgo_profile_read, waits for the device.  Not thread
 * safe; leave it disabled in production.  No counterpart in the reference. */
#define TGO_KERNEL_QUANTIZE 0
#define TGO_KERNEL_BUILD_TASKS 1   /* never recorded: the task list is built inside the quantize / pack launches */
#define TGO_KERNEL_FORWARD 2
#define TGO_KERNEL_GRAD_INPUT 3
#define TGO_KERNEL_DEQUANT 4
#define TGO_KERNEL_FORWARD_GEMV 5
#define TGO_KERNEL_PACK_COTANGENT 6
#define TGO_KERNEL_COMBINE 7
#define TGO_KERNEL_COUNT 8

/* Switches timing on (1) or off (0); either way the recorded launches are dropped. */
int tgo_profile_enable(int enabled);

/* Waits for the recorded launches of `kernel` and returns their summed duration and count. */
int tgo_profile_read(int kernel, double * total_ms, int64_t * launches);

/* Matrix operands of the forward kernels that run on the matrix cores (not the decode-sized GEMV family), a
 * process-wide setting.
 *   TGO_OPERAND_INT8    int8 quants on the int8 matrix instruction, scales applied per 32-value block in fp32 (the
 *                       arithmetic of the reference's kernel, csrc/vendor/llama_cpp/mmq-vec-dot.cuh).
 *   TGO_OPERAND_HALF    fp16 numbers that hold the quantized activations and the integer weight operands exactly:
 *                       the same integer dot products per block as with int8 operands.
 *   TGO_OPERAND_SCALED  both operands carry their scales into the matrix instruction: the dequantized q8_1
 *                       activation and the dequantized weight, each normalised by a power of two per row and rounded
 *                       to fp16 once (relative 2^-11; same quants, block scales and sums as the other kinds).  Results
 *                       differ from the other kinds by up to 5e-4 of the largest output; the fastest kind for calls
 *                       that fill the chip.  Its kernel has no SwiGLU epilogue: tgo_grouped_mmq_swiglu then stores both
 *                       projections and finishes with an elementwise pass (same results as the pair followed by
 *                       silu(gate) * up on the bf16 values).
 *   TGO_OPERAND_AUTO    (default) scaled for calls of at least 128 tiles of 256 rows x 128 outputs (total rows of
 *                       a grouped call; both projections of a pair count), otherwise fp16 for IQ2_S (whose integer
 *                       operand needs two int8 planes but one fp16 number) and int8 for the other formats.
 * Workspaces that are quantized before their format is known (tgo_quantize_q8_1 / tgo_mmq_forward_prepared) take int8
 * unless TGO_OPERAND_HALF is forced (their _as variants take the kind as an argument).  The activation workspace is laid out for one kind and says which in its last
 * KiB: tgo_q8_workspace_unpack follows that tag, and tgo_mmq_forward_prepared turns its outputs into NaN when the
 * setting was changed between quantizing a workspace and using it.  A call reads the setting once.
 * tgo_forward_operand() returns the current setting; tgo_forward_operand_for() the kind (never AUTO) that a forward
 * call of this format and shape would use under it (`projections`: 2 for a pair).  No counterpart in the reference. */
#define TGO_OPERAND_INT8 0
#define TGO_OPERAND_HALF 1
#define TGO_OPERAND_AUTO 2
#define TGO_OPERAND_SCALED 3
int tgo_set_forward_operand(int operand);
int tgo_forward_operand(void);
int tgo_forward_operand_for(int quant_type, int64_t rows, int64_t out_features, int projections);

#ifdef __cplusplus
}
#endif

#endif /* TGO_H */
