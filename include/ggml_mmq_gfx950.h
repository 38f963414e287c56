/* C ABI of libggml_mmq_gfx950.so: packed GGUF-weight matmul kernels for LoRA training on gfx950.
 *
 * The library replaces, behind plain pointers and sizes, the native operators the reference reaches
 * through torch.ops.torch_ggml_ops (un-vendored wheel), AITER gmm/ptgmm, its Triton routing kernels and
 * Liger's cross-entropy kernel.  Each declaration names the reference call site it stands in for
 * (file:line in the reference repository).
 *
 * Conventions
 *   - every pointer is a device pointer unless it is a `stream` (a hipStream_t passed as void*);
 *   - matrices are row-major and contiguous; activations and LoRA factors are bf16 (uint16 storage);
 *   - packed weights are the raw GGUF blocks of a [N, K] tensor, row after row, read-only, never
 *     copied or repacked; supported GGML type ids: 8 (Q8_0), 10 (Q2_K), 11 (Q3_K), 12 (Q4_K), 13 (Q5_K),
 *     14 (Q6_K), 16 (IQ2_XXS);
 *     K must be a multiple of 64 and of the type's block size;
 *   - nothing is allocated inside: the caller passes outputs and, where stated, a workspace whose size
 *     comes from the matching *_workspace_bytes function (256-byte aligned carving inside);
 *   - work is enqueued on `stream` and the call returns without synchronising;
 *   - return value 0 = success; negative = error (-1 type id, -2 shape, -3 alignment, -4 null pointer,
 *     -5 HIP runtime, -6 workspace too small) with text available from ggq_last_error() (thread-local).
 *     Errors are detected before any launch; nothing is repaired silently (no hidden operand copies).
 *   - expert groups: `expert_ids[g]` (int64) is the expert of group g and `end_offsets[g]` (int32) the
 *     cumulative END row of group g in the expert-sorted row order (test_fast_moe_lora.py:136-137:
 *     experts [0,2,5], offsets [2,5,6]).  groups == 0 means one dense group that uses expert 0.
 */
#ifndef GGML_MMQ_GFX950_H
#define GGML_MMQ_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ggq_last_error(void);

/* Kernel timing aid (the reference profiles with Kineto module ranges, deepseek_v4_profiler.py:39-74):
 * between begin and end every launch of a packed-weight matmul kernel is bracketed by HIP events on
 * its stream.  ggq_profile_end synchronises on them and fills host arrays (milliseconds, GGML type id,
 * mode 0 = forward / 1 = grad-input, epilogue id 0 = store / 1 = fp32 accumulate, and - unless `shape` is NULL - the kernel
 * family: 0 = tall tiles, 1 = wide tiles, 3 = the Q4_K kernels whose MFMA waves decode the weights, 4 = one launch of wide and
 * tall tiles, 5 = the IQ2_XXS forward of small groups) for up to `capacity` launches; returns the number written or a negative error.  Not thread safe; at most
 * 8192 launches are recorded. */
int ggq_profile_begin(void);
int ggq_profile_end(float* ms, int* qt, int* mode, int* epilogue, int* shape, int capacity);

/* Measurement aid with no counterpart in the reference: the bf16 MFMA rate (TFLOP/s, into the HOST float tflops_out) a
 * register-only loop of 32x32x16 MFMAs sustains on this device when its operands are drawn from the two device sample
 * buffers (`elems` bf16 values each, at least 4096, 16-byte aligned).  The device is power limited and its clock depends on
 * the operand values, so this - measured with a workload's own activations and decoded weights - is that workload's
 * MFMA-bound ceiling.  `sink` is a device buffer of at least 256 bytes that the kernel may write (nothing is allocated
 * here).  Synchronous: times `iters` loop trips with HIP events on `stream` and waits. */
int ggq_measure_mfma_ceiling(const void* a_samples, const void* b_samples, int64_t elems, int iters, void* sink, float* tflops_out, void* stream);

/* Tuning switch with no counterpart in the reference.  A grouped backward call that returns factor gradients enqueues
 * its grad-input launch on the caller's stream and the dA / dB launches on a stream of the library's own (one per device,
 * default priority, created on the first such call outside a stream capture), forked behind the rank-sized product they
 * read and joined back before the call returns: to the caller the call stays one ordered piece of work on `stream`, under
 * stream capture the fork and join become graph edges, and the results are bit-identical either way.  0 keeps every launch
 * on the caller's stream; 1 (the default) forks.  Process-wide. */
int ggq_set_factor_gradient_overlap(int enabled);

/* Test aid with no counterpart in the reference: force the kernel family of the grouped launches that follow (0 = tall
 * tiles, 1 = the wide / tall tile mix and nothing else, 3 = the Q4_K kernels whose MFMA waves decode the weights themselves,
 * 5 = the wide / tall mix with the IQ2_XXS forward of groups of up to 128 rows on its decoding-wave kernel, which is also what
 * IQ2_XXS calls get by default, each wherever its operand conditions hold; -1 = the library's own choice, the default).
 * FOR TESTS ONLY: a process-wide setting that stays until it is set back to -1 and changes the kernel choice of every later
 * caller in the process; not thread safe (no launch may run in another thread while it changes); results are the same to
 * the stated tolerances whatever is chosen. */
int ggq_debug_force_grouped_shape(int shape);

/* fast_lora.py:24-31 (_NATIVE_MMQ_QUANT_TYPES / supports_native_mmq): 1 if this library has kernels
 * for the GGML type id. */
int ggq_supports_quant_type(int qt);

/* Bytes of one packed row of K elements (gguf GGML_QUANT_SIZES, test_deepseek_v4_moe_lora.py:58);
 * -1 if K is not a whole number of blocks or the type is unknown. */
int64_t ggq_row_bytes(int qt, int64_t k);

/* dequantize_gguf_tensor (transformers gguf fork; used at fast_moe_lora.py:163-165, 235-240 and as the
 * oracle of test_fast_lora.py:110-115): packed [rows, K] -> bf16 (out_is_f32 = 0) or fp32 values,
 * bit-exact with ggml's dequantize_row_* followed by round-to-nearest-even to bf16. */
int ggq_dequantize(int qt, const void* packed, int64_t rows, int64_t k, void* out, int out_is_f32, void* stream);

/* torch.ops.torch_ggml_ops.mmq (fast_lora.py:155-160, gguf_liger_loss.py:109-114): y[M,N] = x[M,K] . W^T. */
int ggq_mmq(const void* x, const void* packed, int qt, int64_t m, int64_t n, int64_t k, void* y, void* stream);

/* torch.ops.torch_ggml_ops.mmq_grad_input (gguf_liger_loss.py:172-177; autograd of mmq,
 * test_fast_lora.py:104-105): dx[M,K] = dy[M,N] . W with W decoded to bf16, fp32 accumulation. */
int ggq_mmq_grad_input(const void* dy, const void* packed, int qt, int64_t m, int64_t n, int64_t k, void* dx, void* stream);

/* Workspace bound for the four LoRA entry points below (n_total = N, or 2N for a pair).  groups = 0 (the dense calls)
 * includes the fp32 partial sums of the factor gradients, whose rows are then dealt over the whole chip. */
int64_t ggq_lora_workspace_bytes(int64_t rows, int64_t groups, int64_t experts, int64_t n_total, int64_t k, int r);

/* FastGGUFLoraLinear._base_layer_forward + _fused_lora_add (fast_lora.py:34-65, 134-163) in one call:
 *   xa_out[M, r16] = bf16(x . A^T)  (r16 = r rounded up to 16, zero padded),
 *   y[M,N] = x . W^T + scale * xa . B^T.      A [r,K], B [N,r].  A = B = NULL gives plain mmq. */
int ggq_lora_mmq_forward(const void* x, const void* packed, int qt, int64_t m, int64_t n, int64_t k, const void* lora_a,
                         const void* lora_b, int r, float scale, void* xa_out, void* y, void* ws, int64_t ws_bytes,
                         void* stream);

/* Autograd of the above (test_fast_lora.py:101-134): dx = dy . W + scale * (dy . B) . A,
 * dB[N,r] = scale * dy^T . xa, dA[r,K] = scale * (dy . B)^T . x; dA / dB may be NULL. */
int ggq_lora_mmq_backward(const void* dy, const void* packed, int qt, int64_t m, int64_t n, int64_t k, const void* x,
                          const void* xa, const void* lora_a, const void* lora_b, int r, float scale, void* dx,
                          void* d_lora_a, void* d_lora_b, void* ws, int64_t ws_bytes, void* stream);

/* torch.ops.torch_ggml_ops.grouped_mmq / grouped_mmq_pair (fast_moe_lora.py:221-228, 339-347) fused with
 * the per-expert LoRA delta that the reference computes with AITER gmm (_lora_grouped_linear,
 * fast_moe_lora.py:675-682, added at :743-745 / :763).  packed1/packed2 [E,N,bytes]; packed2 != NULL
 * selects the pair form (two outputs y1, y2 from one x; LoRA B is [E,2N,r], first N rows for y1).
 * A [E,r,K].  A = B = NULL gives the plain grouped ops. */
int ggq_grouped_lora_mmq_forward(const void* x, const void* packed1, const void* packed2, const int64_t* expert_ids,
                                 const int32_t* end_offsets, int64_t groups, int64_t experts, int qt, int64_t rows, int64_t n,
                                 int64_t k, const void* lora_a, const void* lora_b, int r, float scale, void* xa_out, void* y1,
                                 void* y2, const void* group_tables, void* ws, int64_t ws_bytes, void* stream);

/* torch.ops.torch_ggml_ops.grouped_mmq_grad_input / grouped_mmq_pair_grad_input
 * (fast_moe_lora.py:255-262, 364-375: both cotangents of a pair land in one fp32 accumulator and are
 * rounded once) plus the LoRA input gradient (gmm with transposed rhs, fast_moe_lora.py:56-73) and the
 * factor gradients (ptgmm, fast_moe_lora.py:76-87; all E planes written, inactive experts exactly zero,
 * test_fast_moe_lora.py:331-333).  dA [E,r,K], dB [E,N or 2N,r]; may be NULL. */
int ggq_grouped_lora_mmq_backward(const void* dy1, const void* dy2, const void* packed1, const void* packed2,
                                  const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts, int qt,
                                  int64_t rows, int64_t n, int64_t k, const void* x, const void* xa, const void* lora_a,
                                  const void* lora_b, int r, float scale, void* dx, void* d_lora_a, void* d_lora_b,
                                  const void* group_tables, void* ws, int64_t ws_bytes, void* stream);

/* Row-tile tables of one grouping, built once for the launches that share it (no counterpart in the reference: its ops take
 * expert ids and offsets only, docs/plan_qwen3.5.md:32).  Every grouped call turns (expert_ids, end_offsets) into tables of
 * row tiles on the device before its kernels run; the four packed-weight calls of an expert layer's step see the same
 * grouping, so a caller may build the tables once (ggq_group_tables_build, into ggq_group_tables_bytes(rows, groups,
 * experts) bytes of device memory, 16-byte aligned) and pass them as `group_tables` to the grouped calls made with the same
 * expert_ids / end_offsets / groups / experts / rows while the offsets are unchanged.  group_tables = NULL: the call builds
 * its own, as before.  The tables serve the Q4_K decoding-wave kernels; a call that runs another kernel shape ignores them
 * and builds its own.  Results are bit-identical either way. */
int64_t ggq_group_tables_bytes(int64_t rows, int64_t groups, int64_t experts);
int ggq_group_tables_build(const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts, int64_t rows,
                           void* tables, int64_t tables_bytes, void* stream);

/* The two calls above over rows that are never materialised: the reference gathers the routed rows first
 * (prepare_expert_routing, fast_moe_routing.py:379-420: _RouteGather.apply(hidden_states, permutation, ...)) and hands the
 * copy to the grouped ops; here row i of the expert-sorted layout is read in place as row row_index[i] / index_div of
 * x [x_rows, k] (row_index = the sorted-position -> route permutation, index_div = top_k).  Results are bit-identical to
 * the plain calls on the gathered copy.  x must stay under 4 GiB (the kernels address its rows with 32-bit offsets): ask
 * ggq_grouped_forward_reads_indexed_rows (host-only, 1 = yes) with the same qt / rows / groups / x_rows / k first; the
 * indexed forward returns the shape error otherwise.  dx is still per expert-sorted row, [rows, k]. */
int ggq_grouped_forward_reads_indexed_rows(int qt, int64_t rows, int64_t groups, int64_t x_rows, int64_t k);
int ggq_grouped_lora_mmq_forward_indexed(const void* x, int64_t x_rows, const int64_t* row_index, int index_div, const void* packed1,
                                         const void* packed2, const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups,
                                         int64_t experts, int qt, int64_t rows, int64_t n, int64_t k, const void* lora_a,
                                         const void* lora_b, int r, float scale, void* xa_out, void* y1, void* y2,
                                         const void* group_tables, void* ws, int64_t ws_bytes, void* stream);
int ggq_grouped_lora_mmq_backward_indexed(const void* dy1, const void* dy2, const void* packed1, const void* packed2,
                                          const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts,
                                          int qt, int64_t rows, int64_t n, int64_t k, const void* x, int64_t x_rows,
                                          const int64_t* row_index, int index_div, const void* xa, const void* lora_a,
                                          const void* lora_b, int r, float scale, void* dx, void* d_lora_a, void* d_lora_b,
                                          const void* group_tables, void* ws, int64_t ws_bytes, void* stream);

/* torch_ggml_ops.fixed_grouped_mmq (deepseek_v4_lora.py:91-124: DeepSeek's frozen eight-group output projection) and
 * its input gradient: x [rows, groups, k] bf16, packed_groups [groups, n_group, row bytes], y [rows, groups, n_group];
 * y[:, g, :] = x[:, g, :] . W_g^T.  Each group runs as the dense launch over its strided rows, so the results are
 * bit-identical to ggq_mmq / ggq_mmq_grad_input on contiguous per-group copies (the relation the reference pins,
 * test_deepseek_v4_lora.py:131-151). */
int ggq_fixed_grouped_mmq(const void* x, const void* packed_groups, int qt, int64_t rows, int groups, int64_t n_group, int64_t k, void* y,
                          void* stream);
int ggq_fixed_grouped_mmq_grad_input(const void* dy, const void* packed_groups, int qt, int64_t rows, int groups, int64_t n_group, int64_t k,
                                     void* dx, void* stream);

/* prepare_expert_routing (fast_moe_routing.py:379-428: torch.sort of the flat top-k ids + inverse
 * permutation kernel :88-98) and the grouped-execution offsets of the expert module
 * (fast_moe_lora.py:709-719, 652-672).  Stable order: ties keep ascending route index.
 *   sorted_ids, permutation, inverse: int64 [tokens*top_k];  counts, end_offsets: int32 [num_experts];
 *   active_ids int64 / active_end_offsets int32 [num_experts]: compact list of experts with rows (tail
 *   entries repeat the total);  status int32[2] = {number of active experts, 1 if an id was outside
 *   [0,num_experts) (such ids are clamped)}. */
int64_t ggq_route_plan_workspace_bytes(int64_t tokens, int top_k, int num_experts);
int ggq_route_plan(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts, int64_t* sorted_ids,
                   int64_t* permutation, int64_t* inverse, int32_t* counts, int32_t* end_offsets, int64_t* active_ids,
                   int32_t* active_end_offsets, int32_t* status, void* ws, int64_t ws_bytes, void* stream);

/* ggq_route_plan without a workspace and without any allocation.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory around the call (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  The sort's scratch (per-route ranks, per-chunk histograms) lives in a 2.1 MB device array
 * inside the library, one copy per GPU, held until the process ends; its address is looked up on the first call on
 * each device.  Limits: tokens * top_k <= 262144 routes and num_experts <= 256, otherwise the shape error (-2) is
 * returned and nothing is launched.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and need no clearing in between.  Outputs and results
 * are those of ggq_route_plan, bit for bit. */
int ggq_route_plan_static(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts, int64_t* sorted_ids,
                          int64_t* permutation, int64_t* inverse, int32_t* counts, int32_t* end_offsets, int64_t* active_ids,
                          int32_t* active_end_offsets, int32_t* status, void* stream);

/* _route_gather_forward_kernel (fast_moe_routing.py:101-123): selected[s] = hidden[permutation[s] / k]. */
int ggq_route_gather_forward(const void* hidden, const int64_t* permutation, void* selected, int64_t tokens, int top_k, int hidden_dim, void* stream);

/* _route_gather_backward_kernel (fast_moe_routing.py:126-159): per token, routes added in ascending
 * sorted position with a bf16 rounding after every add. */
int ggq_route_gather_backward(const void* grad_selected, const int64_t* inverse, void* grad_hidden, int64_t tokens, int top_k, int hidden_dim, void* stream);

/* _route_combine_forward_kernel (fast_moe_routing.py:162-194); weights [tokens, top_k] fp32 or bf16. */
int ggq_route_combine_forward(const void* expert_out, const void* weights, int weights_are_bf16, const int64_t* inverse, void* out, int64_t tokens, int top_k, int hidden_dim, void* stream);

/* _route_combine_backward_kernel (fast_moe_routing.py:197-226); either gradient may be NULL. */
int ggq_route_combine_backward(const void* expert_out, const void* weights, int weights_are_bf16, const int64_t* permutation, const void* grad_out, void* grad_expert_out, void* grad_weights, int64_t tokens, int top_k, int hidden_dim, void* stream);

/* The combine's backward folded into the down projection's (what _RouteCombine.backward, fast_moe_routing.py:197-226 /
 * :276-300, followed by grouped_mmq_grad_input and the grouped LoRA GEMMs, fast_moe_lora.py:255-262 and :42-151, compute in
 * several passes): grad_out is the [tokens, n] cotangent of the COMBINED output, and expert-sorted row i stands for
 * weights[permutation[i]] * grad_out[permutation[i] / top_k] without that [rows, n] matrix ever being written.
 * dx_unscaled [rows, k] = grad_out[token] . W[expert] + LoRA term, WITHOUT the routing weight (ggq_swiglu_backward_routed
 * applies it); d_lora_a / d_lora_b (may be NULL) include it.  x [rows, k] and xa are the projection's forward input and its
 * x . A^T.  Workspace as for ggq_grouped_lora_mmq_backward. */
int ggq_grouped_lora_mmq_backward_routed_output(const void* grad_out, int64_t tokens, const int64_t* permutation, int top_k,
                                                const void* weights, int weights_are_bf16, const void* packed,
                                                const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts,
                                                int qt, int64_t rows, int64_t n, int64_t k, const void* x, const void* xa,
                                                const void* lora_a, const void* lora_b, int r, float scale, void* dx_unscaled,
                                                void* d_lora_a, void* d_lora_b, const void* group_tables, void* ws, int64_t ws_bytes,
                                                void* stream);

/* The second half of that backward: dh_unweighted [rows, inter] is dx_unscaled above, the cotangent of
 * h = silu(gate) * up (limit > 0: the clamped form) before the routing weight.  Writes dgate, dup for the cotangent
 * weights[permutation[i]] * dh_unweighted[i], and grad_weights[permutation[i]] = <dh_unweighted[i], h[i]> (fp32 sum; equal
 * to the <grad_out[token], expert_out[i]> of fast_moe_routing.py:217-224 up to rounding; NULL: not wanted), in the
 * weights' type. */
int ggq_swiglu_backward_routed(const void* gate, const void* up, const void* dh_unweighted, const void* weights, int weights_are_bf16,
                               const int64_t* permutation, void* dgate, void* dup, void* grad_weights, int64_t rows, int inter, float limit,
                               void* stream);

/* AITER's grouped products as the reference calls them (gmm / ptgmm, fast_moe_lora.py:22, 42-87; _AiterGroupedMM :90-151),
 * for bf16 or fp16 matrices (is_f16; both operands and the output share the type) with no packed weight: the LoRA factors of an expert layer (:674-682) and expert weights without a
 * packed kernel (:230-247).  group_sizes [experts] int32 on the device: consecutive row groups of lhs, group e owning
 * rhs[e].  Sizes are clipped to m, negative ones count as zero; rows no group covers give zero output rows.
 *   ggq_gmm:   out [m, n]: out[i] = lhs[i] . rhs[e], lhs [m, k] row-major, rhs[e] stored [n][k] (rhs_k_contiguous = 1:
 *              the reference's `factor.transpose(1, 2)` of an [E, n, k] factor) or [k][n] (0: its grad-input call, :53-68).
 *   ggq_ptgmm: out [experts, k, n]: out[e] = lhs[rows of e]^T . grad_out[rows of e] (:71-87); experts without rows
 *              get zeros, every plane is written.
 * fp32 accumulation, one rounding to the 16-bit type.  Any k and n (16-byte loads when k resp. n is a multiple of 8 and the base
 * addresses are 16-byte aligned).  ws: ggq_gmm_workspace_bytes(experts) bytes of device memory, 4-byte aligned. */
int64_t ggq_gmm_workspace_bytes(int64_t experts);
int ggq_gmm(const void* lhs, const void* rhs, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts,
            int rhs_k_contiguous, int is_f16, void* ws, int64_t ws_bytes, void* stream);
int ggq_ptgmm(const void* lhs, const void* grad_out, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts,
              int is_f16, void* ws, int64_t ws_bytes, void* stream);

/* GGUFExperts._apply_split_gate (fork; called at fast_moe_lora.py:747): h = silu(gate) * up, and its
 * autograd.  elems = rows * intermediate. */
int ggq_swiglu_forward(const void* gate, const void* up, void* h, int64_t elems, void* stream);
int ggq_swiglu_backward(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, void* stream);

/* The DeepSeek form of the same step (config.swiglu_limit; pinned by test_deepseek_v4_moe_lora.py:184-199):
 * h = silu(min(gate, limit)) * clamp(up, -limit, limit), and its autograd (no gradient into a clamped input). */
int ggq_swiglu_clamped_forward(const void* gate, const void* up, void* h, int64_t elems, float limit, void* stream);
int ggq_swiglu_clamped_backward(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, float limit, void* stream);

/* router_topk_indices (fast_moe_ranking.py:197-271; Triton kernel :163-194, key order :71-80 and :119-160): per
 * token the top_k experts of up to 256 router scores, best first, equal scores in ascending expert index.
 *   score_function 0: the logit itself (bf16 or fp32); 1: sqrt(softplus(logit)) in fp32 plus the optional
 *   correction_bias float[num_experts] (:88-102).  indices int64 [tokens, top_k].
 * Optional routing weights of the selected experts (weights may be NULL / weights_mode 0):
 *   1: softmax over the selected logits in fp32, stored in the logits' type (_qwen_router_forward, :273-284);
 *   2: sqrt(softplus(logit)) / (sum + 1e-20) * routed_scaling as fp32 (_deepseek_topk_router_forward, :287-303).
 * num_experts a multiple of 4, at most 256; top_k at most 8. */
int ggq_router_topk(const void* logits, int logits_are_bf16, int64_t tokens, int num_experts, int top_k, const float* correction_bias,
                    int score_function, int64_t* indices, void* weights, int weights_mode, float routed_scaling, void* stream);

/* _packed_q8_linear_cross_entropy_forward (gguf_liger_loss.py:38-186): chunked mmq -> Liger
 * cross-entropy -> mmq_grad_input in one call.  labels int64 [rows];
 * loss_per_row fp32 [rows] (already divided by the number of non-ignored rows when reduction_mean);
 * grad_hidden bf16 [rows, hidden]; lse_out fp32 [rows] or NULL;
 * status_out int32[2] or NULL: {number of rows that count, number of labels outside [0, vocab) other than ignore_index}.
 *   Such labels are treated as ignored (no loss, no gradient) and only reported here: nothing on the host waits for them.
 * predicted_tokens int64 [rows] or NULL: the row's argmax over the bf16 logits (the first maximum), -1 for rows that do not
 *   count; token_correct fp32 [rows] or NULL: 1 where the argmax is the label, else 0 (Liger's RETURN_PREDICTED_TOKENS /
 *   RETURN_TOKEN_ACCURACY outputs, gguf_liger_loss.py:92-100, 117-185; the accuracy is sum(token_correct) / status_out[0]).
 * Memory: `chunk` stands for the reference's [chunk, vocab] logits tensor.  From 4096 rows per chunk on, or when one chunk
 * covers all rows, the chunk's bf16 logits are kept in the workspace and rewritten as their gradient.  Below that nothing wider
 * than 8192 vocabulary columns is held (one sweep over the vocabulary with a running max, sum and argmax per row), but the
 * sweep takes min(rows, 4096) rows at a time whatever the chunk: the workspace then holds a [min(rows, 4096), 8192] bf16 slab,
 * an fp32 [min(rows, 4096), hidden] accumulator and two bf16-sized [.., hidden] label-row buffers (about 128 MiB at hidden 2048),
 * for chunk 64 as for chunk 1024.  Two vocabulary-sized GEMMs either way. */
int64_t ggq_lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden_dim, int64_t chunk);
int ggq_lmhead_cross_entropy(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
                             int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_per_row,
                             void* grad_hidden, float* lse_out, int32_t* status_out, int64_t* predicted_tokens, float* token_correct, void* ws,
                             int64_t ws_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif
