/*
 * moe_i8.h — C-ABI of the gfx950 INT8 W8A8 fused-MoE library (libmoe_i8.so).
 *
 * Every entry point takes raw device pointers, plain sizes and a HIP stream
 * (passed as void*).  The library never allocates or frees device memory,
 * never synchronises and never touches any stream but the one it is given, so
 * every call can be recorded into a HIP graph.  The caller owns all buffers,
 * including the workspace.
 *
 * Return value: 0 on success, a negative MOE_I8_E* code otherwise; the text of
 * the last error of the calling thread is available from moe_i8_last_error().
 *
 * The reference (prime-rl) holds no FFI for this path: its rollout engine
 * reaches these operations through vLLM 0.28.0 (reference pyproject.toml:58),
 * selected by the `quantization` pass-through
 * (packages/prime-rl-configs/src/prime_rl/configs/inference.py:108-109).  Each
 * declaration below names the vLLM operation it replaces and the closest
 * statement of the same semantics that is in the reference tree.
 */
#ifndef MOE_I8_H_
#define MOE_I8_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_I8_OK 0
#define MOE_I8_EINVAL (-1)     /* bad argument (null pointer, size, alignment, limit) */
#define MOE_I8_EWORKSPACE (-2) /* workspace or output capacity too small */
#define MOE_I8_ELAUNCH (-3)    /* HIP reported an error at launch */
#define MOE_I8_EUNSUPPORTED (-4)

#define MOE_I8_MAX_EXPERTS 1024

/* Activation element types accepted by the quantiser / produced by the GEMMs. */
#define MOE_I8_DTYPE_BF16 0

/* GEMM kernel families; MOE_I8_GEMM_AUTO picks by rows-per-expert. */
#define MOE_I8_GEMM_AUTO 0
#define MOE_I8_GEMM_STREAM 1 /* weights streamed global->registers, 16-row MFMA sub-tiles (decode) */
#define MOE_I8_GEMM_TILE 2   /* LDS-staged tiles, 32x32x32 MFMA (prefill); geometry by rows per expert */
#define MOE_I8_GEMM_NARROW 3 /* 64-row tiles, three LDS stages kept in flight (tens of rows per expert) */
#define MOE_I8_GEMM_TILE_WIDE 4 /* the LDS-tiled family with 256-row tiles and two stages (many rows per expert) */
#define MOE_I8_GEMM_TILE_DEEP 5 /* the LDS-tiled family with 128-row tiles and three stages (around 100 rows per expert) */
#define MOE_I8_GEMM_TILE_RING 6 /* 256-row tiles through a ring of four 32 KB stages: a measured alternative to _TILE_WIDE, \
                                   same results, 7-10 % slower; MOE_I8_GEMM_AUTO never picks it */

/* Router score functions (reference TokenChoiceTopKRouter.score_func). */
#define MOE_I8_SCORE_SOFTMAX 0      /* softmax over all experts */
#define MOE_I8_SCORE_SIGMOID 1      /* sigmoid per expert */
#define MOE_I8_SCORE_TOPK_SOFTMAX 2 /* select on the logits, softmax over the selected k */

int moe_i8_version(void);
const char* moe_i8_last_error(void);

/* Capacity rules shared with the Python host: sorted_token_ids needs
 * min(P + E*(B-1), P*B) entries (P = number of (token, expert) pairs) and
 * expert_ids needs ceil(that / B). */
int64_t moe_i8_sorted_capacity(int64_t num_pairs, int num_experts, int block_size);
int64_t moe_i8_align_workspace_bytes(int64_t num_pairs, int num_experts, int block_size);

/*
 * Replaces vLLM `fused_topk(hidden_states, gating_output, topk, renormalize)` (topk_softmax op,
 * csrc/moe/topk_softmax_kernels.cu) and `grouped_topk(..., num_expert_group, topk_group,
 * scoring_func, routed_scaling_factor, e_score_correction_bias)`
 * (model_executor/layers/fused_moe/fused_moe.py); in-tree semantics: TokenChoiceTopKRouter.forward,
 * src/prime_rl/trainer/models/layers/moe.py:261-307 (fp32 scores :262-269, selection-only bias
 * :281-283, top-k :284-289, gather of unbiased scores :290, top-k softmax :292-293, route_norm with
 * +1e-20 :302-304, route_scale :305).
 * logits fp32 [m, num_experts] -> topk_weights fp32 [m, top_k], topk_ids int32 [m, top_k] in
 * descending order of the selection value, equal values by ascending expert index.
 * num_groups > 1: experts form num_groups equal contiguous groups, a group scores the sum of its two
 * largest selection values (group_score_top2 != 0) or its largest, only the topk_groups best groups
 * stay eligible.
 * capture_dtype != 0 additionally writes the ids as uint8 (1) or uint16 (2) to
 * capture[token * capture_token_stride + capture_offset + j] — the [seq_len, layers, topk] record of
 * src/prime_rl/inference/vllm/routed_experts.py:11-33 (stride = layers * topk, offset = layer * topk).
 */
int moe_i8_route_topk(const float* logits, int64_t m, int num_experts, int top_k, int score_func,
                      const float* selection_bias, int num_groups, int topk_groups, int group_score_top2,
                      int renormalize, float route_scale, float* topk_weights, int32_t* topk_ids,
                      void* capture, int capture_dtype, int64_t capture_token_stride,
                      int64_t capture_offset, void* stream);

/*
 * Replaces vLLM `moe_align_block_size(topk_ids, block_size, num_experts)`
 * (csrc/moe/moe_align_sum_kernels.cu).  In-tree semantics: stable expert sort
 * trainer/distributed/token_dispatcher.py:139-145, per-expert padding :107-121.
 * topk_ids int32 [num_pairs] -> sorted_token_ids int32 [sorted_cap] (flat pair
 * index, ascending inside each expert segment, unused slots = num_pairs),
 * expert_ids int32 [expert_cap] (unused blocks = -1), num_tokens_post_padded
 * int32 [1].  Ids outside [0, num_experts) are ignored.
 */
int moe_i8_align_block_size(const int32_t* topk_ids, int64_t num_pairs, int num_experts,
                            int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                            int32_t* expert_ids, int64_t expert_cap,
                            int32_t* num_tokens_post_padded, void* workspace,
                            int64_t workspace_bytes, void* stream);

/*
 * Replaces vLLM `per_token_quant_int8(x)` (quantization/utils/int8_utils.py);
 * in-tree analogue trainer/models/kernels/fp8_utils.py:186-201.
 * x [*, cols] (dtype code, row stride in elements) -> q int8 [rows, cols] and
 * scale fp32 [rows].  With gather != NULL output row r quantises input row
 * gather[r] / gather_div; a source row >= src_rows yields a zero row.
 */
int moe_i8_quant_rows(const void* x, int dtype, int64_t src_rows, int64_t cols, int64_t row_stride,
                      const int32_t* gather, int gather_div, int64_t rows, int8_t* q, float* scale,
                      void* stream);

/*
 * Per-output-channel symmetric int8 quantisation of bf16 expert weights into the kernel layout,
 * for in-place updates of a quantised engine after a policy step: the int8 analogue of the
 * reference's `quantize_to_vllm_kernel_format` (src/prime_rl/trainer/models/fp8.py:5-64: scale =
 * absmax / qmax clamped from below, q = w / scale) + `torch.cat([gate, up], dim=1)`
 * (src/prime_rl/trainer/models/glm_moe_dsa/converting_glm_moe_dsa.py:97-104) feeding the in-place
 * `param.copy_` of src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134.
 * w bf16 [rows, cols] -> q int8 and scale fp32 at output row
 * (r / rows_per_group) * out_rows_per_group + out_row_offset + r % rows_per_group
 * (rows_per_group == 0: output row == r); scale = max(absmax / 127, 1e-12),
 * q = clamp(rint(w / scale), -127, 127) with ties to even.
 */
int moe_i8_quant_weights(const void* w, int dtype, int64_t rows, int64_t cols, int64_t rows_per_group,
                         int64_t out_rows_per_group, int64_t out_row_offset, int8_t* q, float* scale,
                         void* stream);

/*
 * Replaces vLLM `fused_moe_kernel` (gate_up GEMM, use_int8_w8a8, per-channel) +
 * `silu_and_mul` (csrc/activation_kernels.cu).  In-tree semantics: grouped GEMM
 * contract tests/unit/train/models/test_moe.py:60-66; gate-then-up stacking
 * trainer/models/layers/moe.py:146-148; activation trainer/models/layers/activations.py:29-34.
 * x_q int8 [M, H], a_scale fp32 [M], w1 int8 [E, 2I, H], w1_scale fp32 [E, 2I]
 * -> act bf16 [num_pairs, I], row t = pair t (token t / top_k).
 * The routing may come from anywhere, with one requirement every router meets: the top_k experts
 * of one token are distinct, so an expert holds at most num_pairs / top_k rows (the streaming
 * family sizes its launch on that; rows beyond it would not be computed).
 */
int moe_i8_gemm_gate_up_silu(const int8_t* x_q, const float* a_scale, const int8_t* w1,
                             const float* w1_scale, const int32_t* sorted_token_ids,
                             const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                             int64_t num_pairs, int top_k, int num_experts, int hidden, int inter,
                             int block_size, int64_t sorted_cap, void* act_out, int variant,
                             void* stream);

/*
 * Replaces vLLM `fused_moe_kernel` (down GEMM, top_k=1, MUL_ROUTED_WEIGHT).
 * In-tree semantics: weight applied after the experts in fp32 then cast,
 * trainer/distributed/token_dispatcher.py:159-160.
 * h_q int8 [num_pairs, I], a_scale fp32 [num_pairs], w2 int8 [E, H, I],
 * w2_scale fp32 [E, H], topk_weights fp32 [num_pairs] (NULL = all ones) -> out bf16 [num_pairs, H].
 */
int moe_i8_gemm_down(const int8_t* h_q, const float* a_scale, const int8_t* w2,
                     const float* w2_scale, const float* topk_weights,
                     const int32_t* sorted_token_ids, const int32_t* expert_ids,
                     const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts,
                     int hidden, int inter, int block_size, int64_t sorted_cap, void* out,
                     int variant, void* stream);

/*
 * The down GEMM with the second `per_token_quant_int8` folded in (streaming family only, inter <= 1024):
 * act bf16 [num_pairs, I] is quantised row by row inside the kernel with the arithmetic of
 * moe_i8_quant_rows, so the result equals moe_i8_quant_rows followed by moe_i8_gemm_down bit for bit.
 * moe_i8_fused_experts uses it when it picks the streaming family for the down GEMM and experts hold
 * at most three rows on average (num_pairs <= 3 * num_experts); with more rows the separate
 * quantisation launch is the cheaper one, because every workgroup of a block repeats the quantisation.
 */
int moe_i8_gemm_down_bf16(const void* act, const int8_t* w2, const float* w2_scale, const float* topk_weights,
                          const int32_t* sorted_token_ids, const int32_t* expert_ids,
                          const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts, int hidden,
                          int inter, int block_size, int64_t sorted_cap, void* out, void* stream);

/*
 * Raw int32 accumulators of either grouped GEMM (inspection / parity only):
 * acc[t, n] = sum_K a_q[t / row_div, K] * w[e_t, n, K] for every routed pair t.
 * a_q int8 [*, K], w int8 [E, N, K] -> acc int32 [num_pairs, N].
 */
int moe_i8_gemm_acc_i32(const int8_t* a_q, const int8_t* w, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                        int64_t num_pairs, int row_div, int num_experts, int n, int k,
                        int block_size, int64_t sorted_cap, int32_t* acc_out, int variant,
                        void* stream);

/*
 * Replaces vLLM `ops.moe_sum(input, output)` (csrc/moe/moe_align_sum_kernels.cu);
 * in-tree analogue: scatter_add combine, trainer/distributed/token_dispatcher.py:162-165.
 * in bf16 [M, top_k, H] -> out bf16 [M, H].
 */
int moe_i8_sum(const void* in, void* out, int64_t m, int top_k, int hidden, void* stream);

/* Bytes of caller-owned workspace moe_i8_fused_experts needs. */
int64_t moe_i8_workspace_bytes(int64_t m, int top_k, int num_experts, int hidden, int inter,
                               int block_size);

/*
 * Replaces vLLM `fused_experts(hidden_states, w1, w2, topk_weights, topk_ids,
 * use_int8_w8a8=True, per_channel_quant=True, w1_scale, w2_scale,
 * a1_scale=None, a2_scale=None)` -> `fused_experts_impl`
 * (model_executor/layers/fused_moe/fused_moe.py): quant, align, gate_up GEMM +
 * SiLU*mul, quant, down GEMM * routed weight, sum — all on `stream`, no host
 * synchronisation.  hidden bf16 [M, H]; out bf16 [M, H] (may alias hidden).
 * Every topk_id must lie in [0, num_experts): a pair with another id is skipped by the alignment and
 * the GEMMs, so its row of the intermediate buffer is never written and the combine would add
 * whatever the workspace holds there (expert-parallel maps are not part of this path).  The top_k
 * ids of one token must be distinct (see moe_i8_gemm_gate_up_silu).
 */
int moe_i8_fused_experts(const void* hidden, const int8_t* w1, const int8_t* w2,
                         const float* topk_weights, const int32_t* topk_ids,
                         const float* w1_scale, const float* w2_scale, void* out, int64_t m,
                         int top_k, int num_experts, int hidden_size, int inter, int block_size,
                         void* workspace, int64_t workspace_bytes, int variant, void* stream);

/*
 * What moe_i8_fused_experts would launch for a layer shape, decided on the host from the sizes alone (no GPU
 * call): the GEMM kernel of each projection (MOE_I8_GEMM_STREAM, _NARROW, _TILE_WIDE or _TILE_DEEP) and the
 * number of kernel launches of one call.  A diagnostic with no counterpart in the reference (upstream picks its
 * kernel configuration from tuned tables per shape): it lets a test pin which measured kernel each benchmark
 * point runs on, so that a retune of the hand-over points cannot silently move one.  Any output pointer may be
 * null.  Returns MOE_I8_EUNSUPPORTED when `variant` demands a family that does not handle the shape.
 */
int moe_i8_layer_plan(int64_t m, int top_k, int num_experts, int hidden_size, int inter, int block_size,
                      int variant, int* gate_up_kernel, int* down_kernel, int* launches);

/*
 * moe_i8_fused_experts for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and result as moe_i8_fused_experts without the workspace: the intermediate buffers
 * live in a device array of MOE_I8_STATIC_SCRATCH_BYTES that is part of the library's code object
 * (every GPU the library runs on holds its own copy until the process ends).  The call allocates and
 * frees nothing.  A shape whose moe_i8_workspace_bytes() exceeds the array is rejected with
 * MOE_I8_EWORKSPACE.  All calls on one GPU share the array: calls that overlap on one GPU (different
 * streams or threads) race; calls ordered on one stream do not.  Nothing has to be cleared between
 * calls: every region is written before it is read.
 */
#define MOE_I8_STATIC_SCRATCH_BYTES (32 << 20)
int moe_i8_fused_experts_static(const void* hidden, const int8_t* w1, const int8_t* w2,
                                const float* topk_weights, const int32_t* topk_ids,
                                const float* w1_scale, const float* w2_scale, void* out, int64_t m,
                                int top_k, int num_experts, int hidden_size, int inter, int block_size,
                                int variant, void* stream);

/*
 * Dense W8A8 layers (shared experts, dense first-k MLPs) on the same kernels with one group.
 *
 * moe_i8_scaled_int8_quant replaces vLLM `ops.scaled_int8_quant(x, scale=None)` (dynamic per-token
 * symmetric, csrc/quantization/compressed_tensors/int8_quant_kernels.cu): q = rint(x * (127 / absmax)),
 * ties to even — the rounding that separates it from per_token_quant_int8 above; scale = absmax / 127.
 *
 * moe_i8_w8a8_linear replaces `ops.cutlass_scaled_mm(x_q, w.t(), scale_a, scale_b, out_dtype=bf16)` after
 * that quantisation: x bf16 [m, k], w int8 [n, k], w_scale fp32 [n] -> out bf16 [m, n] =
 * bf16((acc * a_scale) * w_scale).
 *
 * moe_i8_w8a8_mlp is the shared-expert MLP down(silu(gate(x)) * up(x))
 * (FeedForward.forward, src/prime_rl/trainer/models/layers/mlp.py:29-32; added to the routed output at
 * src/prime_rl/trainer/models/layers/moe.py:453-462): w13 int8 [2*inter, hidden] gate rows first,
 * w2 int8 [hidden, inter]; x bf16 [m, hidden] -> out bf16 [m, hidden].
 */
int moe_i8_scaled_int8_quant(const void* x, int dtype, int64_t rows, int64_t cols, int64_t row_stride,
                             int8_t* q, float* scale, void* stream);
int64_t moe_i8_dense_workspace_bytes(int64_t m, int k, int inter /* 0 for the plain linear */);
int moe_i8_w8a8_linear(const void* x, const int8_t* w, const float* w_scale, void* out, int64_t m, int n,
                       int k, void* workspace, int64_t workspace_bytes, int variant, void* stream);
int moe_i8_w8a8_mlp(const void* x, const int8_t* w13, const float* w13_scale, const int8_t* w2,
                    const float* w2_scale, void* out, int64_t m, int hidden, int inter, void* workspace,
                    int64_t workspace_bytes, int variant, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_I8_H_ */
