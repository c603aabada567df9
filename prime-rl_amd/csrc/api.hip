// C-ABI of libmoe_i8.so: argument validation, workspace carving and kernel launches.
// Nothing here allocates device memory or synchronises; every launch goes to the caller's stream.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "../../include/moe_i8.h"
#include "common.hpp"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(hipError_t err, const char* what) {
  if (err == hipSuccess) return MOE_I8_OK;
  return fail(MOE_I8_ELAUNCH, "%s: %s", what, hipGetErrorString(err));
}

bool valid_block_size(int b) { return b == 16 || b == 32 || b == 64 || b == 128; }

int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_gemm_common(const void* a_q, const void* w, const int32_t* sorted, const int32_t* eids,
                      const int32_t* npp, const void* out, int64_t num_pairs, int num_experts,
                      int n, int k, int block_size, int64_t sorted_cap, int variant) {
  if (!a_q || !w || !sorted || !eids || !npp || !out) return fail(MOE_I8_EINVAL, "null pointer");
  if (!aligned16(a_q) || !aligned16(w) || !aligned16(out))
    return fail(MOE_I8_EINVAL, "activation, weight and output pointers must be 16-byte aligned");
  if (num_pairs < 0 || num_pairs > INT32_MAX - 1) return fail(MOE_I8_EINVAL, "num_pairs out of range");
  if (num_experts < 1 || num_experts > MOE_I8_MAX_EXPERTS)
    return fail(MOE_I8_EINVAL, "num_experts must be in [1, %d]", MOE_I8_MAX_EXPERTS);
  if (!valid_block_size(block_size)) return fail(MOE_I8_EINVAL, "block_size must be 16, 32, 64 or 128");
  if (n < 16 || n % 16) return fail(MOE_I8_EINVAL, "output channels (%d) must be a positive multiple of 16", n);
  if (k < 64 || k % 64) return fail(MOE_I8_EINVAL, "reduction length (%d) must be a positive multiple of 64", k);
  if (sorted_cap < moe_i8_sorted_capacity(num_pairs, num_experts, block_size))
    return fail(MOE_I8_EWORKSPACE, "sorted_token_ids capacity %lld too small", (long long)sorted_cap);
  if (variant < MOE_I8_GEMM_AUTO || variant > MOE_I8_GEMM_TILE_RING)
    return fail(MOE_I8_EINVAL, "unknown GEMM variant %d", variant);
  return MOE_I8_OK;
}

// The streaming family reads an expert's weights once per 16 of its rows: it is the fastest kernel
// while every block fits one such pass, and loses badly as soon as a few experts hold more (a
// shared expert that every token visits, skewed routing), which the host cannot see.  It is
// therefore picked where no expert can hold more than 16 rows (it holds at most one per token),
// or where there is at most one routed row per expert on average.
constexpr int kStreamMaxRows = 16;
constexpr int kStreamRowsPerExpert = 1;

int tile_geometry_of(int variant) {
  return variant == MOE_I8_GEMM_TILE_WIDE ? moe_i8::kTileWide
         : variant == MOE_I8_GEMM_TILE_DEEP ? moe_i8::kTileDeep
         : variant == MOE_I8_GEMM_TILE_RING ? moe_i8::kTileRing
                                            : moe_i8::kTileAuto;
}

// Routed rows per expert up to which the narrow tiles beat the deep geometry of the LDS-tiled family.
// The narrow tiles (two small workgroups per compute unit, 64 x 128 tasks) start up faster and
// balance better; the deep tiles stream an expert's weights once for up to 128 rows, which counts
// the more the longer a launch runs and the more the routing is skewed.  Measured crossovers, with
// the weight bytes of the launch: 0.2-0.4 GB (Qwen3-30B-A3B, even routing) 40 rows, 0.7-1.5 GB
// (GLM-4.5-Air, Zipf routing and a shared expert) 24-32, 3.8-7.5 GB (DeepSeek-V3) about 8.
int narrow_rows_per_expert(const moe_i8::GemmArgs& g) {
  const int64_t weight_bytes = (int64_t)g.num_experts * g.n * g.k;
  return weight_bytes < (512ll << 20) ? 40 : weight_bytes < (2048ll << 20) ? 28 : 8;
}

// Which family a launch goes to (MOE_I8_GEMM_STREAM, _TILE or _NARROW); -1 with the error set if a
// family was demanded for a shape it does not handle.
int picks_family(const moe_i8::GemmArgs& g0, int variant) {
  moe_i8::GemmArgs g = g0;
  g.tile_geometry = tile_geometry_of(variant);
  if (variant == MOE_I8_GEMM_TILE || variant == MOE_I8_GEMM_TILE_WIDE || variant == MOE_I8_GEMM_TILE_DEEP ||
      variant == MOE_I8_GEMM_TILE_RING) {
    if (!moe_i8::gemm_tile_supports(g))
      return fail(MOE_I8_EUNSUPPORTED, "tile GEMM does not support this shape"), -1;
    return MOE_I8_GEMM_TILE;
  }
  if (variant == MOE_I8_GEMM_NARROW) {
    if (!moe_i8::gemm_narrow_supports(g))
      return fail(MOE_I8_EUNSUPPORTED, "narrow-tile GEMM does not support this shape"), -1;
    return MOE_I8_GEMM_NARROW;
  }
  if (variant == MOE_I8_GEMM_STREAM) return MOE_I8_GEMM_STREAM;
  // Measured crossovers, in routed rows per expert.  With evenly spread routing the streaming family
  // would win up to about 4 (by 1-2 % over the narrow tiles); with one expert that every token visits,
  // or Zipf-skewed routing, the narrow tiles win by 18-34 % from 24 tokens on.  Then the narrow tiles
  // while most experts hold a single 64-row block, then the LDS-tiled family (which picks its own
  // geometry).
  const int64_t rows_x_experts = g.num_pairs;
  const int64_t most_rows = g.max_rows_per_expert > 0 && g.max_rows_per_expert < g.num_pairs ? g.max_rows_per_expert
                                                                                             : g.num_pairs;
  if (most_rows <= kStreamMaxRows || rows_x_experts <= (int64_t)kStreamRowsPerExpert * g.num_experts)
    return MOE_I8_GEMM_STREAM;
  if (rows_x_experts <= (int64_t)narrow_rows_per_expert(g) * g.num_experts && moe_i8::gemm_narrow_supports(g))
    return MOE_I8_GEMM_NARROW;
  if (moe_i8::gemm_tile_supports(g)) return MOE_I8_GEMM_TILE;
  return moe_i8::gemm_narrow_supports(g) ? MOE_I8_GEMM_NARROW : MOE_I8_GEMM_STREAM;
}

int run_gemm(const moe_i8::GemmArgs& g0, int variant, hipStream_t stream) {
  if (g0.num_pairs == 0) return MOE_I8_OK;
  moe_i8::GemmArgs g = g0;
  g.tile_geometry = tile_geometry_of(variant);
  switch (picks_family(g, variant)) {
    case MOE_I8_GEMM_TILE: return check_launch(moe_i8::launch_gemm_tile(g, stream), "gemm_tile");
    case MOE_I8_GEMM_NARROW: return check_launch(moe_i8::launch_gemm_narrow(g, stream), "gemm_narrow");
    case MOE_I8_GEMM_STREAM: return check_launch(moe_i8::launch_gemm_stream(g, stream), "gemm_stream");
    default: return MOE_I8_EUNSUPPORTED;
  }
}

moe_i8::GemmArgs gate_up_args(const int8_t* x_q, const float* a_scale, const int8_t* w1, const float* w1_scale,
                              const int32_t* sorted_token_ids, const int32_t* expert_ids,
                              const int32_t* num_tokens_post_padded, int64_t num_pairs, int top_k, int num_experts,
                              int hidden, int inter, int block_size, int64_t sorted_cap, void* act_out) {
  moe_i8::GemmArgs g{};
  g.mode = moe_i8::kGateUpSilu;
  g.a_q = x_q;
  g.a_scale = a_scale;
  g.w = w1;
  g.w_scale = w1_scale;
  g.row_weight = nullptr;
  g.sorted_token_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_tokens_post_padded = num_tokens_post_padded;
  g.num_pairs = num_pairs;
  g.row_div = top_k;
  g.num_experts = num_experts;
  g.n = 2 * inter;
  g.k = hidden;
  g.block_size = block_size;
  g.sorted_cap = sorted_cap;
  g.out = act_out;
  g.max_rows_per_expert = (num_pairs + top_k - 1) / top_k;  // an expert sees a token at most once
  return g;
}

// The family of `picks_family` with the geometry of the LDS-tiled family spelled out
// (MOE_I8_GEMM_STREAM, _NARROW, _TILE_WIDE or _TILE_DEEP; _TILE_RING only when demanded); -1 as there.
int picks_kernel(const moe_i8::GemmArgs& g0, int variant) {
  const int family = picks_family(g0, variant);
  if (family != MOE_I8_GEMM_TILE) return family;
  moe_i8::GemmArgs g = g0;
  g.tile_geometry = tile_geometry_of(variant);
  switch (moe_i8::gemm_tile_geometry(g)) {
    case moe_i8::kTileDeep: return MOE_I8_GEMM_TILE_DEEP;
    case moe_i8::kTileRing: return MOE_I8_GEMM_TILE_RING;
    default: return MOE_I8_GEMM_TILE_WIDE;
  }
}

moe_i8::GemmArgs down_args(const int8_t* h_q, const float* a_scale, const int8_t* w2, const float* w2_scale,
                           const float* topk_weights, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                           const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts, int hidden,
                           int inter, int block_size, int64_t sorted_cap, void* out) {
  moe_i8::GemmArgs g{};
  g.mode = moe_i8::kDown;
  g.a_q = h_q;
  g.a_scale = a_scale;
  g.w = w2;
  g.w_scale = w2_scale;
  g.row_weight = topk_weights;
  g.sorted_token_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_tokens_post_padded = num_tokens_post_padded;
  g.num_pairs = num_pairs;
  g.row_div = 1;
  g.num_experts = num_experts;
  g.n = hidden;
  g.k = inter;
  g.block_size = block_size;
  g.sorted_cap = sorted_cap;
  g.out = out;
  return g;
}

}  // namespace

extern "C" {

int moe_i8_version(void) { return 1; }

const char* moe_i8_last_error(void) { return g_error; }

int64_t moe_i8_sorted_capacity(int64_t num_pairs, int num_experts, int block_size) {
  if (num_pairs < 0 || num_experts < 1 || block_size < 1) return -1;
  const int64_t full = num_pairs + (int64_t)num_experts * (block_size - 1);
  const int64_t tight = num_pairs * block_size;
  return full < tight ? full : tight;
}

int64_t moe_i8_align_workspace_bytes(int64_t num_pairs, int num_experts, int block_size) {
  (void)block_size;
  if (num_pairs < 0 || num_experts < 1) return -1;
  return moe_i8::align_workspace_ints(num_pairs, num_experts) * (int64_t)sizeof(int32_t);
}

int moe_i8_align_block_size(const int32_t* topk_ids, int64_t num_pairs, int num_experts,
                            int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                            int32_t* expert_ids, int64_t expert_cap,
                            int32_t* num_tokens_post_padded, void* workspace,
                            int64_t workspace_bytes, void* stream) {
  if (num_pairs < 0 || num_pairs > INT32_MAX - 1) return fail(MOE_I8_EINVAL, "num_pairs out of range");
  if (num_experts < 1 || num_experts > MOE_I8_MAX_EXPERTS)
    return fail(MOE_I8_EINVAL, "num_experts must be in [1, %d]", MOE_I8_MAX_EXPERTS);
  if (!valid_block_size(block_size)) return fail(MOE_I8_EINVAL, "block_size must be 16, 32, 64 or 128");
  if (!num_tokens_post_padded || (num_pairs > 0 && !topk_ids))
    return fail(MOE_I8_EINVAL, "null pointer");
  const int64_t need = moe_i8_sorted_capacity(num_pairs, num_experts, block_size);
  if (sorted_cap < need)
    return fail(MOE_I8_EWORKSPACE, "sorted_token_ids capacity %lld < %lld", (long long)sorted_cap,
                (long long)need);
  if (expert_cap < (sorted_cap + block_size - 1) / block_size)
    return fail(MOE_I8_EWORKSPACE, "expert_ids capacity %lld too small", (long long)expert_cap);
  if ((sorted_cap > 0 && !sorted_token_ids) || (expert_cap > 0 && !expert_ids))
    return fail(MOE_I8_EINVAL, "null pointer");
  const int64_t ws_need = moe_i8_align_workspace_bytes(num_pairs, num_experts, block_size);
  if (ws_need > 0 && (!workspace || workspace_bytes < ws_need))
    return fail(MOE_I8_EWORKSPACE, "align workspace %lld < %lld bytes", (long long)workspace_bytes,
                (long long)ws_need);
  moe_i8::AlignArgs a;
  a.topk_ids = topk_ids;
  a.num_pairs = num_pairs;
  a.num_experts = num_experts;
  a.block_size = block_size;
  a.sorted_token_ids = sorted_token_ids;
  a.sorted_cap = sorted_cap;
  a.expert_ids = expert_ids;
  a.expert_cap = expert_cap;
  a.num_tokens_post_padded = num_tokens_post_padded;
  a.workspace = static_cast<int32_t*>(workspace);
  return check_launch(moe_i8::launch_align(a, static_cast<hipStream_t>(stream)), "moe_align");
}

static int quant_rows_impl(const void* x, int dtype, int64_t src_rows, int64_t cols, int64_t row_stride,
                           const int32_t* gather, int gather_div, int64_t rows, int8_t* q, float* scale,
                           int round_even, void* stream) {
  if (dtype != MOE_I8_DTYPE_BF16) return fail(MOE_I8_EUNSUPPORTED, "only bf16 activations are supported");
  if (rows < 0 || src_rows < 0) return fail(MOE_I8_EINVAL, "negative row count");
  if (rows == 0) return MOE_I8_OK;
  if (!x || !q || !scale) return fail(MOE_I8_EINVAL, "null pointer");
  if (cols < 8 || cols % 8 || cols > INT32_MAX) return fail(MOE_I8_EINVAL, "cols (%lld) must be a positive multiple of 8", (long long)cols);
  if (row_stride < cols || row_stride % 8) return fail(MOE_I8_EINVAL, "row stride must be >= cols and a multiple of 8");
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u))
    return fail(MOE_I8_EINVAL, "x must be 16-byte and q 8-byte aligned");
  if (gather && gather_div < 1) return fail(MOE_I8_EINVAL, "gather_div must be >= 1");
  if (!gather && rows > src_rows) return fail(MOE_I8_EINVAL, "rows exceeds src_rows");
  moe_i8::QuantArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.src_rows = src_rows;
  a.cols = (int)cols;
  a.row_stride = row_stride;
  a.gather = gather;
  a.gather_div = gather ? gather_div : 1;
  a.rows = rows;
  a.q = q;
  a.scale = scale;
  a.round_even = round_even;
  return check_launch(moe_i8::launch_quant_rows(a, static_cast<hipStream_t>(stream)), "quant_rows");
}

int moe_i8_quant_rows(const void* x, int dtype, int64_t src_rows, int64_t cols, int64_t row_stride,
                      const int32_t* gather, int gather_div, int64_t rows, int8_t* q, float* scale,
                      void* stream) {
  return quant_rows_impl(x, dtype, src_rows, cols, row_stride, gather, gather_div, rows, q, scale, 0, stream);
}

int moe_i8_scaled_int8_quant(const void* x, int dtype, int64_t rows, int64_t cols, int64_t row_stride,
                             int8_t* q, float* scale, void* stream) {
  return quant_rows_impl(x, dtype, rows, cols, row_stride, nullptr, 1, rows, q, scale, 1, stream);
}

int moe_i8_route_topk(const float* logits, int64_t m, int num_experts, int top_k, int score_func,
                      const float* selection_bias, int num_groups, int topk_groups, int group_score_top2,
                      int renormalize, float route_scale, float* topk_weights, int32_t* topk_ids,
                      void* capture, int capture_dtype, int64_t capture_token_stride,
                      int64_t capture_offset, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative token count");
  if (num_experts < 1 || num_experts > MOE_I8_MAX_EXPERTS)
    return fail(MOE_I8_EINVAL, "num_experts (%d) must be in [1, %d]", num_experts, MOE_I8_MAX_EXPERTS);
  if (top_k < 1 || top_k > num_experts || top_k > 64)
    return fail(MOE_I8_EINVAL, "top_k (%d) must be in [1, min(num_experts, 64)]", top_k);
  if (score_func != MOE_I8_SCORE_SOFTMAX && score_func != MOE_I8_SCORE_SIGMOID &&
      score_func != MOE_I8_SCORE_TOPK_SOFTMAX)
    return fail(MOE_I8_EINVAL, "unknown score function %d", score_func);
  if (num_groups < 1 || num_experts % num_groups) return fail(MOE_I8_EINVAL, "num_groups must divide num_experts");
  if (num_groups > 1) {
    const int per_lane = moe_i8::route_experts_per_lane(num_experts);
    const int group_size = num_experts / num_groups;
    const int lanes = group_size / per_lane;
    if (group_size % per_lane || lanes < 1 || (lanes & (lanes - 1)))
      return fail(MOE_I8_EUNSUPPORTED, "group size %d must be a power-of-two multiple of %d experts", group_size,
                  per_lane);
    if (topk_groups < 1 || topk_groups > num_groups) return fail(MOE_I8_EINVAL, "topk_groups out of range");
    if (group_score_top2 && group_size < 2) return fail(MOE_I8_EINVAL, "top-2 group score needs groups of >= 2");
    if (top_k > topk_groups * group_size) return fail(MOE_I8_EINVAL, "top_k exceeds the experts of the kept groups");
  }
  if (capture_dtype < 0 || capture_dtype > 2) return fail(MOE_I8_EINVAL, "capture dtype must be 0, 1 (u8) or 2 (u16)");
  if (capture_dtype == 1 && num_experts > 256) return fail(MOE_I8_EINVAL, "uint8 capture holds at most 256 experts");
  if (capture_dtype && (!capture || capture_token_stride < top_k || capture_offset < 0 ||
                        capture_offset + top_k > capture_token_stride))
    return fail(MOE_I8_EINVAL, "capture needs a buffer and offset + top_k <= token stride");
  if (m == 0) return MOE_I8_OK;
  if (!logits || !topk_weights || !topk_ids) return fail(MOE_I8_EINVAL, "null pointer");
  moe_i8::RouteArgs a;
  a.logits = logits;
  a.m = m;
  a.num_experts = num_experts;
  a.top_k = top_k;
  a.score_func = score_func;
  a.bias = selection_bias;
  a.num_groups = num_groups;
  a.topk_groups = topk_groups;
  a.group_top2 = group_score_top2;
  a.renormalize = renormalize;
  a.route_scale = route_scale;
  a.weights = topk_weights;
  a.ids = topk_ids;
  a.capture = capture_dtype ? capture : nullptr;
  a.capture_bytes = capture_dtype;
  a.capture_stride = capture_token_stride;
  a.capture_offset = capture_offset;
  return check_launch(moe_i8::launch_route_topk(a, static_cast<hipStream_t>(stream)), "route_topk");
}

int moe_i8_quant_weights(const void* w, int dtype, int64_t rows, int64_t cols, int64_t rows_per_group,
                         int64_t out_rows_per_group, int64_t out_row_offset, int8_t* q, float* scale,
                         void* stream) {
  if (dtype != MOE_I8_DTYPE_BF16) return fail(MOE_I8_EUNSUPPORTED, "only bf16 weights are supported");
  if (rows < 0) return fail(MOE_I8_EINVAL, "negative row count");
  if (rows == 0) return MOE_I8_OK;
  if (!w || !q || !scale) return fail(MOE_I8_EINVAL, "null pointer");
  if (cols < 8 || cols % 8 || cols > INT32_MAX)
    return fail(MOE_I8_EINVAL, "cols (%lld) must be a positive multiple of 8", (long long)cols);
  if (!aligned16(w) || (reinterpret_cast<uintptr_t>(q) & 7u))
    return fail(MOE_I8_EINVAL, "w must be 16-byte and q 8-byte aligned");
  if (rows_per_group < 0 || (rows_per_group > 0 && (rows % rows_per_group || out_row_offset < 0 ||
                                                     out_row_offset + rows_per_group > out_rows_per_group)))
    return fail(MOE_I8_EINVAL, "row groups must tile the input and fit inside the output groups");
  moe_i8::QuantArgs a;
  a.x = static_cast<const uint16_t*>(w);
  a.src_rows = rows;
  a.cols = (int)cols;
  a.row_stride = cols;
  a.gather = nullptr;
  a.gather_div = 1;
  a.rows = rows;
  a.q = q;
  a.scale = scale;
  a.rows_per_group = rows_per_group;
  a.out_rows_per_group = out_rows_per_group;
  a.out_row_offset = out_row_offset;
  return check_launch(moe_i8::launch_quant_weights(a, static_cast<hipStream_t>(stream)), "quant_weights");
}

// The gate_up GEMM behind the entry point; `from_align`: the routing arrays are moe_align's own
// output (the caller of the entry point may pass anything).
static int gemm_gate_up_impl(const int8_t* x_q, const float* a_scale, const int8_t* w1, const float* w1_scale,
                             const int32_t* sorted_token_ids, const int32_t* expert_ids,
                             const int32_t* num_tokens_post_padded, int64_t num_pairs, int top_k, int num_experts,
                             int hidden, int inter, int block_size, int64_t sorted_cap, void* act_out, int variant,
                             bool from_align, void* stream) {
  if (num_pairs == 0) return MOE_I8_OK;
  if (inter < 16 || inter % 16 || inter > (1 << 29)) return fail(MOE_I8_EINVAL, "inter (%d) must be a positive multiple of 16", inter);
  if (int rc = check_gemm_common(x_q, w1, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                 act_out, num_pairs, num_experts, 2 * inter, hidden, block_size,
                                 sorted_cap, variant))
    return rc;
  if (!a_scale || !w1_scale) return fail(MOE_I8_EINVAL, "null scale pointer");
  if (!aligned16(w1_scale)) return fail(MOE_I8_EINVAL, "w1_scale must be 16-byte aligned");
  if (top_k < 1) return fail(MOE_I8_EINVAL, "top_k must be >= 1");
  moe_i8::GemmArgs g = gate_up_args(x_q, a_scale, w1, w1_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                    num_pairs, top_k, num_experts, hidden, inter, block_size, sorted_cap, act_out);
  g.expert_ids_ascend = from_align;
  return run_gemm(g, variant, static_cast<hipStream_t>(stream));
}

int moe_i8_gemm_gate_up_silu(const int8_t* x_q, const float* a_scale, const int8_t* w1,
                             const float* w1_scale, const int32_t* sorted_token_ids,
                             const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                             int64_t num_pairs, int top_k, int num_experts, int hidden, int inter,
                             int block_size, int64_t sorted_cap, void* act_out, int variant,
                             void* stream) {
  return gemm_gate_up_impl(x_q, a_scale, w1, w1_scale, sorted_token_ids, expert_ids, num_tokens_post_padded, num_pairs,
                           top_k, num_experts, hidden, inter, block_size, sorted_cap, act_out, variant, false, stream);
}

// The down GEMM behind the entry point; `max_rows` bounds the rows any one expert can hold (0: unknown),
// `from_align` as above.
static int gemm_down_impl(const int8_t* h_q, const float* a_scale, const int8_t* w2, const float* w2_scale,
                          const float* topk_weights, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                          const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts, int hidden,
                          int inter, int block_size, int64_t sorted_cap, void* out, int variant, int64_t max_rows,
                          bool from_align, void* stream) {
  if (num_pairs == 0) return MOE_I8_OK;
  if (int rc = check_gemm_common(h_q, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, out,
                                 num_pairs, num_experts, hidden, inter, block_size, sorted_cap,
                                 variant))
    return rc;
  if (!a_scale || !w2_scale) return fail(MOE_I8_EINVAL, "null scale pointer");
  if (!aligned16(w2_scale)) return fail(MOE_I8_EINVAL, "w2_scale must be 16-byte aligned");
  moe_i8::GemmArgs g = down_args(h_q, a_scale, w2, w2_scale, topk_weights, sorted_token_ids, expert_ids,
                                 num_tokens_post_padded, num_pairs, num_experts, hidden, inter, block_size,
                                 sorted_cap, out);
  g.max_rows_per_expert = max_rows;
  g.expert_ids_ascend = from_align;
  return run_gemm(g, variant, static_cast<hipStream_t>(stream));
}

int moe_i8_gemm_down(const int8_t* h_q, const float* a_scale, const int8_t* w2,
                     const float* w2_scale, const float* topk_weights,
                     const int32_t* sorted_token_ids, const int32_t* expert_ids,
                     const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts,
                     int hidden, int inter, int block_size, int64_t sorted_cap, void* out,
                     int variant, void* stream) {
  return gemm_down_impl(h_q, a_scale, w2, w2_scale, topk_weights, sorted_token_ids, expert_ids,
                        num_tokens_post_padded, num_pairs, num_experts, hidden, inter, block_size, sorted_cap, out,
                        variant, 0, false, stream);
}

int moe_i8_gemm_down_bf16(const void* act, const int8_t* w2, const float* w2_scale, const float* topk_weights,
                          const int32_t* sorted_token_ids, const int32_t* expert_ids,
                          const int32_t* num_tokens_post_padded, int64_t num_pairs, int num_experts, int hidden,
                          int inter, int block_size, int64_t sorted_cap, void* out, void* stream) {
  if (num_pairs == 0) return MOE_I8_OK;
  if (int rc = check_gemm_common(act, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, out, num_pairs,
                                 num_experts, hidden, inter, block_size, sorted_cap, MOE_I8_GEMM_STREAM))
    return rc;
  if (!w2_scale) return fail(MOE_I8_EINVAL, "null scale pointer");
  if (!aligned16(w2_scale)) return fail(MOE_I8_EINVAL, "w2_scale must be 16-byte aligned");
  if (!moe_i8::gemm_stream_fuses_quant(inter))
    return fail(MOE_I8_EUNSUPPORTED, "inter (%d) is too long for the GEMM that quantises its own activations", inter);
  moe_i8::GemmArgs g = down_args(nullptr, nullptr, w2, w2_scale, topk_weights, sorted_token_ids, expert_ids,
                                 num_tokens_post_padded, num_pairs, num_experts, hidden, inter, block_size,
                                 sorted_cap, out);
  g.a_bf16 = static_cast<const uint16_t*>(act);
  return check_launch(moe_i8::launch_gemm_stream(g, static_cast<hipStream_t>(stream)), "gemm_stream");
}

int moe_i8_gemm_acc_i32(const int8_t* a_q, const int8_t* w, const int32_t* sorted_token_ids,
                        const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                        int64_t num_pairs, int row_div, int num_experts, int n, int k,
                        int block_size, int64_t sorted_cap, int32_t* acc_out, int variant,
                        void* stream) {
  if (num_pairs == 0) return MOE_I8_OK;
  if (int rc = check_gemm_common(a_q, w, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                 acc_out, num_pairs, num_experts, n, k, block_size, sorted_cap,
                                 variant))
    return rc;
  if (row_div < 1) return fail(MOE_I8_EINVAL, "row_div must be >= 1");
  moe_i8::GemmArgs g{};
  g.mode = moe_i8::kAccI32;
  g.a_q = a_q;
  g.w = w;
  g.sorted_token_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_tokens_post_padded = num_tokens_post_padded;
  g.num_pairs = num_pairs;
  g.row_div = row_div;
  g.num_experts = num_experts;
  g.n = n;
  g.k = k;
  g.block_size = block_size;
  g.sorted_cap = sorted_cap;
  g.out = acc_out;
  return run_gemm(g, variant, static_cast<hipStream_t>(stream));
}

int moe_i8_sum(const void* in, void* out, int64_t m, int top_k, int hidden, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative m");
  if (m == 0) return MOE_I8_OK;
  if (!in || !out) return fail(MOE_I8_EINVAL, "null pointer");
  if (top_k < 1) return fail(MOE_I8_EINVAL, "top_k must be >= 1");
  if (hidden < 8 || hidden % 8) return fail(MOE_I8_EINVAL, "hidden (%d) must be a positive multiple of 8", hidden);
  if (!aligned16(in) || !aligned16(out)) return fail(MOE_I8_EINVAL, "pointers must be 16-byte aligned");
  return check_launch(moe_i8::launch_moe_sum(static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out),
                                             m, top_k, hidden, static_cast<hipStream_t>(stream)),
                      "moe_sum");
}

// Workspace layout of moe_i8_fused_experts (every region 256-byte aligned):
//   x_q i8[M*H] | a1_scale f32[M] | sorted i32[cap] | expert_ids i32[cap/B] | npp i32[1] |
//   align scratch | act bf16[P*I] | act_q i8[P*I] | a2_scale f32[P] | down_out bf16[P*H]
namespace {
struct Carve {
  int64_t x_q, a1, sorted, eids, npp, align_ws, act, act_q, a2, down, total;
  int64_t cap, ecap, align_bytes;
};
Carve carve(int64_t m, int top_k, int num_experts, int hidden, int inter, int block_size) {
  Carve c{};
  const int64_t p = m * top_k;
  c.cap = moe_i8_sorted_capacity(p, num_experts, block_size);
  c.ecap = (c.cap + block_size - 1) / block_size;
  c.align_bytes = moe_i8_align_workspace_bytes(p, num_experts, block_size);
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    const int64_t at = off;
    off = align_up(off + bytes, 256);
    return at;
  };
  c.x_q = take(m * hidden);
  c.a1 = take(m * 4);
  c.sorted = take(c.cap * 4);
  c.eids = take(c.ecap * 4);
  c.npp = take(4);
  c.align_ws = take(c.align_bytes);
  c.act = take(p * inter * 2);
  c.act_q = take(p * inter);
  c.a2 = take(p * 4);
  c.down = take(p * hidden * 2);
  c.total = off;
  return c;
}

// What moe_i8_fused_experts launches for a layer shape: decided on the host from the sizes alone.
struct LayerPlan {
  int gate_up_kernel;   // MOE_I8_GEMM_STREAM, _NARROW, _TILE_WIDE or _TILE_DEEP; -1 = shape not supported by the demanded family
  int down_kernel;
  bool fuse_align_quant;  // moe_align and the quantisation of the layer input in one launch
  bool down_quantises;    // the streaming down GEMM quantises its own bf16 activations (one launch less)
  int launches;
};

LayerPlan plan_layer(int64_t m, int top_k, int num_experts, int hidden, int inter, int block_size, int variant) {
  const Carve c = carve(m, top_k, num_experts, hidden, inter, block_size);
  const int64_t p = m * top_k;
  LayerPlan plan{};
  moe_i8::GemmArgs gu = gate_up_args(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, p, top_k, num_experts,
                                     hidden, inter, block_size, c.cap, nullptr);
  gu.expert_ids_ascend = true;
  plan.gate_up_kernel = picks_kernel(gu, variant);
  moe_i8::GemmArgs dg = down_args(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, p, num_experts,
                                  hidden, inter, block_size, c.cap, nullptr);
  dg.expert_ids_ascend = true;
  dg.max_rows_per_expert = m;
  plan.down_kernel = picks_kernel(dg, variant);
  // Very few rows per expert (decode): the streaming down GEMM quantises its activations itself, one
  // launch less.  Every workgroup of a block repeats that quantisation, so from about four rows
  // per expert on (measured) the separate launch is the cheaper one again.
  plan.down_quantises = plan.down_kernel == MOE_I8_GEMM_STREAM && moe_i8::gemm_stream_fuses_quant(inter) &&
                        p <= (int64_t)3 * num_experts;
  moe_i8::AlignArgs aa{};
  aa.num_pairs = p;
  aa.num_experts = num_experts;
  aa.block_size = block_size;
  aa.sorted_cap = c.cap;
  aa.expert_cap = c.ecap;
  moe_i8::QuantArgs qa{};
  qa.src_rows = m;
  qa.cols = hidden;
  qa.row_stride = hidden;
  qa.gather_div = 1;
  qa.rows = m;
  plan.fuse_align_quant = moe_i8::align_quant_fusable(aa, qa);
  plan.launches = moe_i8::align_launches(aa) + (plan.fuse_align_quant ? 0 : 1) + 1 + (plan.down_quantises ? 1 : 2) + 1;
  return plan;
}
}  // namespace

int64_t moe_i8_workspace_bytes(int64_t m, int top_k, int num_experts, int hidden, int inter,
                               int block_size) {
  if (m < 0 || top_k < 1 || num_experts < 1 || hidden < 1 || inter < 1 || !valid_block_size(block_size))
    return -1;
  return carve(m, top_k, num_experts, hidden, inter, block_size).total;
}

int moe_i8_fused_experts(const void* hidden, const int8_t* w1, const int8_t* w2,
                         const float* topk_weights, const int32_t* topk_ids,
                         const float* w1_scale, const float* w2_scale, void* out, int64_t m,
                         int top_k, int num_experts, int hidden_size, int inter, int block_size,
                         void* workspace, int64_t workspace_bytes, int variant, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative m");
  if (m == 0) return MOE_I8_OK;
  if (!hidden || !w1 || !w2 || !topk_weights || !topk_ids || !w1_scale || !w2_scale || !out || !workspace)
    return fail(MOE_I8_EINVAL, "null pointer");
  if (top_k < 1 || m * top_k > INT32_MAX - 1) return fail(MOE_I8_EINVAL, "top_k / num_pairs out of range");
  if (!valid_block_size(block_size)) return fail(MOE_I8_EINVAL, "block_size must be 16, 32, 64 or 128");
  if (hidden_size < 64 || hidden_size % 64 || inter < 64 || inter % 64)
    return fail(MOE_I8_EINVAL, "hidden (%d) and inter (%d) must be positive multiples of 64", hidden_size, inter);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(MOE_I8_EINVAL, "workspace must be 256-byte aligned");
  const Carve c = carve(m, top_k, num_experts, hidden_size, inter, block_size);
  if (workspace_bytes < c.total)
    return fail(MOE_I8_EWORKSPACE, "workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)c.total);
  char* ws = static_cast<char*>(workspace);
  int8_t* x_q = reinterpret_cast<int8_t*>(ws + c.x_q);
  float* a1 = reinterpret_cast<float*>(ws + c.a1);
  int32_t* sorted = reinterpret_cast<int32_t*>(ws + c.sorted);
  int32_t* eids = reinterpret_cast<int32_t*>(ws + c.eids);
  int32_t* npp = reinterpret_cast<int32_t*>(ws + c.npp);
  void* act = ws + c.act;
  int8_t* act_q = reinterpret_cast<int8_t*>(ws + c.act_q);
  float* a2 = reinterpret_cast<float*>(ws + c.a2);
  void* down = ws + c.down;
  const int64_t p = m * top_k;

  const LayerPlan plan = plan_layer(m, top_k, num_experts, hidden_size, inter, block_size, variant);
  if (plan.gate_up_kernel < 0 || plan.down_kernel < 0) return MOE_I8_EUNSUPPORTED;

  // Small batches: moe_align (one workgroup) and the quantisation of the input share one launch.
  moe_i8::AlignArgs aa;
  aa.topk_ids = topk_ids;
  aa.num_pairs = p;
  aa.num_experts = num_experts;
  aa.block_size = block_size;
  aa.sorted_token_ids = sorted;
  aa.sorted_cap = c.cap;
  aa.expert_ids = eids;
  aa.expert_cap = c.ecap;
  aa.num_tokens_post_padded = npp;
  aa.workspace = reinterpret_cast<int32_t*>(ws + c.align_ws);
  moe_i8::QuantArgs qa;
  qa.x = static_cast<const uint16_t*>(hidden);
  qa.src_rows = m;
  qa.cols = hidden_size;
  qa.row_stride = hidden_size;
  qa.gather = nullptr;
  qa.gather_div = 1;
  qa.rows = m;
  qa.q = x_q;
  qa.scale = a1;
  if (num_experts >= 1 && num_experts <= MOE_I8_MAX_EXPERTS && aligned16(hidden) &&
      moe_i8::align_quant_fusable(aa, qa)) {
    if (int rc = check_launch(moe_i8::launch_align_quant(aa, qa, static_cast<hipStream_t>(stream)),
                              "align_quant"))
      return rc;
  } else {
    if (int rc = moe_i8_quant_rows(hidden, MOE_I8_DTYPE_BF16, m, hidden_size, hidden_size, nullptr, 1, m,
                                   x_q, a1, stream))
      return rc;
    if (int rc = moe_i8_align_block_size(topk_ids, p, num_experts, block_size, sorted, c.cap, eids, c.ecap,
                                         npp, ws + c.align_ws, c.align_bytes, stream))
      return rc;
  }
  if (int rc = gemm_gate_up_impl(x_q, a1, w1, w1_scale, sorted, eids, npp, p, top_k, num_experts, hidden_size, inter,
                                 block_size, c.cap, act, variant, true, stream))
    return rc;
  if (plan.down_quantises) {
    if (int rc = moe_i8_gemm_down_bf16(act, w2, w2_scale, topk_weights, sorted, eids, npp, p, num_experts,
                                       hidden_size, inter, block_size, c.cap, down, stream))
      return rc;
  } else {
    if (int rc = moe_i8_quant_rows(act, MOE_I8_DTYPE_BF16, p, inter, inter, nullptr, 1, p, act_q, a2, stream))
      return rc;
    if (int rc = gemm_down_impl(act_q, a2, w2, w2_scale, topk_weights, sorted, eids, npp, p, num_experts,
                                hidden_size, inter, block_size, c.cap, down, variant, m, true, stream))
      return rc;
  }
  return moe_i8_sum(down, out, m, top_k, hidden_size, stream);
}

int moe_i8_layer_plan(int64_t m, int top_k, int num_experts, int hidden_size, int inter, int block_size,
                      int variant, int* gate_up_kernel, int* down_kernel, int* launches) {
  if (m < 1 || top_k < 1 || m * top_k > INT32_MAX - 1) return fail(MOE_I8_EINVAL, "m / top_k out of range");
  if (num_experts < 1 || num_experts > MOE_I8_MAX_EXPERTS)
    return fail(MOE_I8_EINVAL, "num_experts must be in [1, %d]", MOE_I8_MAX_EXPERTS);
  if (!valid_block_size(block_size)) return fail(MOE_I8_EINVAL, "block_size must be 16, 32, 64 or 128");
  if (hidden_size < 64 || hidden_size % 64 || inter < 64 || inter % 64)
    return fail(MOE_I8_EINVAL, "hidden (%d) and inter (%d) must be positive multiples of 64", hidden_size, inter);
  if (variant < MOE_I8_GEMM_AUTO || variant > MOE_I8_GEMM_TILE_RING)
    return fail(MOE_I8_EINVAL, "unknown GEMM variant %d", variant);
  const LayerPlan plan = plan_layer(m, top_k, num_experts, hidden_size, inter, block_size, variant);
  if (plan.gate_up_kernel < 0 || plan.down_kernel < 0) return MOE_I8_EUNSUPPORTED;
  if (gate_up_kernel) *gate_up_kernel = plan.gate_up_kernel;
  if (down_kernel) *down_kernel = plan.down_kernel;
  if (launches) *launches = plan.launches;
  return MOE_I8_OK;
}

// ---- the entry point that allocates nothing ----
// The workspace of the layer lives in a file-scope device array instead of caller memory.  The
// array's name is only a host-side handle: the device address is asked from the runtime once per
// device (each device holds its own copy at its own address) and that pointer is what the launches get.
namespace {
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[MOE_I8_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out) {
  int dev = -1;
  const hipError_t derr = hipGetDevice(&dev);
  if (derr != hipSuccess) return fail(MOE_I8_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(derr));
  if (dev < 0 || dev >= kMaxDevices) return fail(MOE_I8_EUNSUPPORTED, "device index %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !p)
      return fail(MOE_I8_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(err));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MOE_I8_OK;
}
}  // namespace

int moe_i8_fused_experts_static(const void* hidden, const int8_t* w1, const int8_t* w2,
                                const float* topk_weights, const int32_t* topk_ids,
                                const float* w1_scale, const float* w2_scale, void* out, int64_t m,
                                int top_k, int num_experts, int hidden_size, int inter, int block_size,
                                int variant, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative m");
  if (m == 0) return MOE_I8_OK;
  const int64_t need = moe_i8_workspace_bytes(m, top_k, num_experts, hidden_size, inter, block_size);
  if (need < 0) return fail(MOE_I8_EINVAL, "bad layer shape");
  if (need > (int64_t)MOE_I8_STATIC_SCRATCH_BYTES)
    return fail(MOE_I8_EWORKSPACE,
                "this call needs %lld bytes of scratch, the static array holds %lld: use moe_i8_fused_experts "
                "with a caller-owned workspace",
                (long long)need, (long long)MOE_I8_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // every region of the workspace is written by the call before it is read: nothing to clear
  return moe_i8_fused_experts(hidden, w1, w2, topk_weights, topk_ids, w1_scale, w2_scale, out, m, top_k,
                              num_experts, hidden_size, inter, block_size, ws, MOE_I8_STATIC_SCRATCH_BYTES, variant,
                              stream);
}

// Workspace of the dense entry points (every region 256-byte aligned):
//   x_q i8[M*K] | a1 f32[M] | sorted i32[cap] | expert_ids i32[cap/64] | npp i32[1] |
//   (mlp only) act bf16[M*I] | act_q i8[M*I] | a2 f32[M]
namespace {
constexpr int kDenseBlock = 64;
constexpr int kDenseSelfQuantRows = 16;  // up to this many rows the down GEMM of the MLP quantises its own input
struct DenseCarve {
  int64_t x_q, a1, sorted, eids, npp, act, act_q, a2, total, cap;
};
DenseCarve dense_carve(int64_t m, int k, int inter) {
  DenseCarve c{};
  c.cap = moe_i8_sorted_capacity(m, 1, kDenseBlock);
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    const int64_t at = off;
    off = align_up(off + bytes, 256);
    return at;
  };
  c.x_q = take(m * k);
  c.a1 = take(m * 4);
  c.sorted = take(c.cap * 4);
  c.eids = take((c.cap + kDenseBlock - 1) / kDenseBlock * 4);
  c.npp = take(4);
  if (inter > 0) {
    c.act = take(m * inter * 2);
    c.act_q = take(m * inter);
    c.a2 = take(m * 4);
  }
  c.total = off;
  return c;
}

int dense_prologue(const void* x, int64_t m, int k, void* workspace, int64_t workspace_bytes,
                   const DenseCarve& c, void* stream) {
  if (m > INT32_MAX - kDenseBlock) return fail(MOE_I8_EINVAL, "too many rows");
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(MOE_I8_EINVAL, "workspace must be 256-byte aligned");
  if (workspace_bytes < c.total)
    return fail(MOE_I8_EWORKSPACE, "workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)c.total);
  char* ws = static_cast<char*>(workspace);
  // one launch: the ties-to-even row quantiser, whose threads also write the identity routing
  if (k < 8 || k % 8) return fail(MOE_I8_EINVAL, "k (%d) must be a positive multiple of 8", k);
  if (!aligned16(x)) return fail(MOE_I8_EINVAL, "x must be 16-byte aligned");
  moe_i8::QuantArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.src_rows = m;
  a.cols = k;
  a.row_stride = k;
  a.gather = nullptr;
  a.gather_div = 1;
  a.rows = m;
  a.q = reinterpret_cast<int8_t*>(ws + c.x_q);
  a.scale = reinterpret_cast<float*>(ws + c.a1);
  a.round_even = 1;
  a.route_sorted = reinterpret_cast<int32_t*>(ws + c.sorted);
  a.route_expert_ids = reinterpret_cast<int32_t*>(ws + c.eids);
  a.route_npp = reinterpret_cast<int32_t*>(ws + c.npp);
  a.route_block = kDenseBlock;
  a.route_cap = c.cap;
  return check_launch(moe_i8::launch_quant_rows(a, static_cast<hipStream_t>(stream)), "quant_rows");
}
}  // namespace

int64_t moe_i8_dense_workspace_bytes(int64_t m, int k, int inter) {
  if (m < 0 || k < 1 || inter < 0) return -1;
  return dense_carve(m, k, inter).total;
}

int moe_i8_w8a8_linear(const void* x, const int8_t* w, const float* w_scale, void* out, int64_t m, int n,
                       int k, void* workspace, int64_t workspace_bytes, int variant, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative m");
  if (m == 0) return MOE_I8_OK;
  if (!x || !w || !w_scale || !out || !workspace) return fail(MOE_I8_EINVAL, "null pointer");
  const DenseCarve c = dense_carve(m, k, 0);
  if (int rc = dense_prologue(x, m, k, workspace, workspace_bytes, c, stream)) return rc;
  char* ws = static_cast<char*>(workspace);
  return moe_i8_gemm_down(reinterpret_cast<int8_t*>(ws + c.x_q), reinterpret_cast<float*>(ws + c.a1), w, w_scale,
                          nullptr, reinterpret_cast<int32_t*>(ws + c.sorted), reinterpret_cast<int32_t*>(ws + c.eids),
                          reinterpret_cast<int32_t*>(ws + c.npp), m, 1, n, k, kDenseBlock, c.cap, out, variant,
                          stream);
}

int moe_i8_w8a8_mlp(const void* x, const int8_t* w13, const float* w13_scale, const int8_t* w2,
                    const float* w2_scale, void* out, int64_t m, int hidden, int inter, void* workspace,
                    int64_t workspace_bytes, int variant, void* stream) {
  if (m < 0) return fail(MOE_I8_EINVAL, "negative m");
  if (m == 0) return MOE_I8_OK;
  if (!x || !w13 || !w13_scale || !w2 || !w2_scale || !out || !workspace) return fail(MOE_I8_EINVAL, "null pointer");
  if (inter < 64 || inter % 64) return fail(MOE_I8_EINVAL, "inter (%d) must be a positive multiple of 64", inter);
  const DenseCarve c = dense_carve(m, hidden, inter);
  if (int rc = dense_prologue(x, m, hidden, workspace, workspace_bytes, c, stream)) return rc;
  char* ws = static_cast<char*>(workspace);
  int8_t* x_q = reinterpret_cast<int8_t*>(ws + c.x_q);
  float* a1 = reinterpret_cast<float*>(ws + c.a1);
  int32_t* sorted = reinterpret_cast<int32_t*>(ws + c.sorted);
  int32_t* eids = reinterpret_cast<int32_t*>(ws + c.eids);
  int32_t* npp = reinterpret_cast<int32_t*>(ws + c.npp);
  int8_t* act_q = reinterpret_cast<int8_t*>(ws + c.act_q);
  float* a2 = reinterpret_cast<float*>(ws + c.a2);
  if (int rc = moe_i8_gemm_gate_up_silu(x_q, a1, w13, w13_scale, sorted, eids, npp, m, 1, 1, hidden, inter,
                                        kDenseBlock, c.cap, ws + c.act, variant, stream))
    return rc;
  // A few rows (decode): the streaming down GEMM quantises them itself (ties to even here), one
  // launch less.
  moe_i8::GemmArgs dg = down_args(act_q, a2, w2, w2_scale, nullptr, sorted, eids, npp, m, 1, hidden, inter,
                                  kDenseBlock, c.cap, out);
  dg.expert_ids_ascend = true;
  const int family = picks_family(dg, variant);
  if (family < 0) return MOE_I8_EUNSUPPORTED;
  if (family == MOE_I8_GEMM_STREAM && m <= kDenseSelfQuantRows && moe_i8::gemm_stream_fuses_quant(inter)) {
    if (int rc = check_gemm_common(ws + c.act, w2, sorted, eids, npp, out, m, 1, hidden, inter, kDenseBlock, c.cap,
                                   MOE_I8_GEMM_STREAM))
      return rc;
    if (!aligned16(w2_scale)) return fail(MOE_I8_EINVAL, "w2_scale must be 16-byte aligned");
    dg.a_q = nullptr;
    dg.a_scale = nullptr;
    dg.a_bf16 = reinterpret_cast<const uint16_t*>(ws + c.act);
    dg.a_round_even = true;
    return check_launch(moe_i8::launch_gemm_stream(dg, static_cast<hipStream_t>(stream)), "gemm_stream");
  }
  if (int rc = moe_i8_scaled_int8_quant(ws + c.act, MOE_I8_DTYPE_BF16, m, inter, inter, act_q, a2, stream)) return rc;
  return moe_i8_gemm_down(act_q, a2, w2, w2_scale, nullptr, sorted, eids, npp, m, 1, hidden, inter, kDenseBlock,
                          c.cap, out, variant, stream);
}

}  // extern "C"
