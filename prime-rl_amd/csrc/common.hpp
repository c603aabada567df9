// Shared device helpers and launcher declarations for the gfx950 INT8 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moe_i8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;
constexpr int kMaxExperts = 1024;  // == MOE_I8_MAX_EXPERTS

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Compute units of the current device (asked once per process; 256 if the runtime will not say).
inline int device_cu_count() {
  static const int count = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) return 256;
    return n;
  }();
  return count;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float round_to_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}

// Wave-wide reductions on the VALU's data-parallel-primitive lane permutes (no LDS traffic, a few
// cycles per step): quads, half rows and rows of 16 by mirror permutes, then row 15 -> next row and
// row 31 -> upper half broadcasts leave the total in lane 63, which is read back as a scalar.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), kCtrl, kRowMask, 0xf, false));
}
__device__ __forceinline__ float wave_reduce_max(float v) {
  v = fmaxf(v, dpp_move<0xb1, 0xf>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_move<0x4e, 0xf>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_move<0x141, 0xf>(v));  // row_half_mirror
  v = fmaxf(v, dpp_move<0x140, 0xf>(v));  // row_mirror
  v = fmaxf(v, dpp_move<0x142, 0xa>(v));  // row_bcast:15 into rows 1 and 3
  v = fmaxf(v, dpp_move<0x143, 0xc>(v));  // row_bcast:31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_reduce_sum(float v) {
  v += dpp_move<0xb1, 0xf>(v);
  v += dpp_move<0x4e, 0xf>(v);
  v += dpp_move<0x141, 0xf>(v);
  v += dpp_move<0x140, 0xf>(v);
  // the broadcasts must add only into the rows they target: elsewhere the permute returns the
  // lane's own value and would double it
  const float b15 = dpp_move<0x142, 0xa>(v);
  v += (lane_id() & 16) ? b15 : 0.0f;
  const float b31 = dpp_move<0x143, 0xc>(v);
  v += (lane_id() & 32) ? b31 : 0.0f;
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Inclusive add-scan over the 64 lanes on the same lane permutes: shifts by 1, 2, 4 and 8 inside rows
// of 16 (a lane without a source adds 0), then the total of row 0 / 2 into every lane of row 1 / 3 and
// the total of the lower half into the upper half.
__device__ __forceinline__ int wave_inclusive_scan_add(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

typedef float f2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf2 __attribute__((ext_vector_type(2)));

// Two fp32 -> packed bf16 (v_cvt_pk_bf16_f32, round to nearest even); lo in bits 15:0.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const bf2 b = __builtin_convertvector(f2{lo, hi}, bf2);
  return *reinterpret_cast<const uint32_t*>(&b);
}

// SiLU with the hardware exp2 / reciprocal approximations (a few fp32 ulp); every GEMM family uses
// this one definition so that the result does not depend on which kernel ran.
__device__ __forceinline__ float fast_silu(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
}

// Four (gate, up) accumulator pairs -> four bf16 outputs with the rounding points of an unfused
// pipeline: gate and up rounded to bf16, silu(gate) rounded to bf16, product rounded to bf16.
__device__ __forceinline__ uint2 silu_mul_epilogue4(const int (&g)[4], const int (&u)[4], float a_scale,
                                                    const float4& wg, const float4& wu) {
  const float wgv[4] = {wg.x, wg.y, wg.z, wg.w};
  const float wuv[4] = {wu.x, wu.y, wu.z, wu.w};
  float h[4];
#pragma unroll
  for (int r = 0; r < 4; r += 2) {
    const uint32_t g2 = pack_bf16((float)g[r] * a_scale * wgv[r], (float)g[r + 1] * a_scale * wgv[r + 1]);
    const uint32_t u2 = pack_bf16((float)u[r] * a_scale * wuv[r], (float)u[r + 1] * a_scale * wuv[r + 1]);
    const uint32_t s2 =
        pack_bf16(fast_silu(__uint_as_float(g2 << 16)), fast_silu(__uint_as_float(g2 & 0xffff0000u)));
    h[r] = __uint_as_float(s2 << 16) * __uint_as_float(u2 << 16);
    h[r + 1] = __uint_as_float(s2 & 0xffff0000u) * __uint_as_float(u2 & 0xffff0000u);
  }
  return make_uint2(pack_bf16(h[0], h[1]), pack_bf16(h[2], h[3]));
}

// Four down-projection accumulators -> four bf16 outputs: acc * a_scale * w_scale * routed weight.
__device__ __forceinline__ uint2 down_epilogue4(const int (&acc)[4], float a_scale, const float4& ws, float rw) {
  return make_uint2(pack_bf16((float)acc[0] * a_scale * ws.x * rw, (float)acc[1] * a_scale * ws.y * rw),
                    pack_bf16((float)acc[2] * a_scale * ws.z * rw, (float)acc[3] * a_scale * ws.w * rw));
}

// ---- launchers (defined one per .hip file; all asynchronous on `stream`) ----

struct AlignArgs {
  const int32_t* topk_ids;
  int64_t num_pairs;
  int num_experts;
  int block_size;
  int32_t* sorted_token_ids;
  int64_t sorted_cap;
  int32_t* expert_ids;
  int64_t expert_cap;
  int32_t* num_tokens_post_padded;
  int32_t* workspace;
};
int64_t align_workspace_ints(int64_t num_pairs, int num_experts);
hipError_t launch_align(const AlignArgs& a, hipStream_t stream);
int align_launches(const AlignArgs& a);  // 1, 2 or 3 by the number of pairs

struct QuantArgs {
  const uint16_t* x;  // bf16 bits
  int64_t src_rows;
  int cols;
  int64_t row_stride;
  const int32_t* gather;
  int gather_div;
  int64_t rows;
  int8_t* q;
  float* scale;
  // Output row of input row r is (r / rows_per_group) * out_rows_per_group + out_row_offset +
  // r % rows_per_group; rows_per_group == 0 means out row == r.  Lets one call drop the gate or
  // the up projection of every expert into its half of a stacked [E, 2I, H] tensor.
  int64_t rows_per_group = 0;
  int64_t out_rows_per_group = 0;
  int64_t out_row_offset = 0;
  int round_even = 0;  // activations: ties to even instead of away from zero
  // Row quantiser only: also write the routing of a dense layer seen as one expert that every row
  // visits (rows in order, padded to whole blocks with the sentinel, used blocks owned by expert
  // 0, the rest of both arrays marked unused) — one launch less in front of a dense GEMM.
  int32_t* route_sorted = nullptr;  // null: no routing
  int32_t* route_expert_ids = nullptr;
  int32_t* route_npp = nullptr;
  int route_block = 0;
  int64_t route_cap = 0;
};
hipError_t launch_quant_rows(const QuantArgs& a, hipStream_t stream);
// Router: scores -> (grouped) top-k -> weights, one wavefront per token.
enum ScoreFunc { kScoreSoftmax = 0, kScoreSigmoid = 1, kScoreTopkSoftmax = 2 };
struct RouteArgs {
  const float* logits;  // [m, num_experts]
  int64_t m;
  int num_experts;
  int top_k;
  int score_func;
  const float* bias;  // [num_experts] or null; added for selection only
  int num_groups;     // 1 = no group pre-selection
  int topk_groups;
  int group_top2;  // group score: 1 = sum of the two largest selection values, 0 = the largest
  int renormalize;
  float route_scale;
  float* weights;  // [m, top_k]
  int32_t* ids;    // [m, top_k]
  void* capture;   // compact copy of ids at capture[tok * capture_stride + capture_offset + j]
  int capture_bytes;  // 0 = none, 1 = uint8, 2 = uint16
  int64_t capture_stride;
  int64_t capture_offset;
};
int route_experts_per_lane(int num_experts);
hipError_t launch_route_topk(const RouteArgs& a, hipStream_t stream);

// Per-output-channel weight quantisation (round to nearest even of w / scale, scale = absmax / 127).
hipError_t launch_quant_weights(const QuantArgs& a, hipStream_t stream);
// moe_align and the quantisation of `q` in one launch; only when align_quant_fusable() says so.
bool align_quant_fusable(const AlignArgs& a, const QuantArgs& q);
hipError_t launch_align_quant(const AlignArgs& a, const QuantArgs& q, hipStream_t stream);

enum GemmMode { kGateUpSilu = 0, kDown = 1, kAccI32 = 2 };

struct GemmArgs {
  int mode;
  const uint16_t* a_bf16 = nullptr;  // down, streaming family only: bf16 activations [P, K] quantised in the kernel
  bool a_round_even = false;         // ... rounding ties to even (dense path) instead of away from zero (MoE path)
  const int8_t* a_q;      // [*, K] activations (int8)
  const float* a_scale;   // per activation row
  const int8_t* w;        // [E, N, K]
  const float* w_scale;   // [E, N]
  const float* row_weight;  // [P] routed weights (down); null = 1
  const int32_t* sorted_token_ids;
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_padded;
  int64_t num_pairs;
  int row_div;  // activation row of pair t is t / row_div
  int num_experts;
  int n;  // weight rows per expert (2I for gate_up, H for down)
  int k;  // reduction length
  int block_size;
  int64_t sorted_cap;
  void* out;  // bf16 [P, I] | bf16 [P, H] | int32 [P, N]
  int64_t max_rows_per_expert = 0;  // upper bound if the caller knows one (the token count), else 0
  bool expert_ids_ascend = false;   // expert_ids is known to come from moe_align (non-decreasing over the used blocks)
  int tile_geometry = 0;            // LDS-tiled family: kTileAuto, kTileWide (256-row tiles), kTileDeep (128-row tiles) or kTileRing (256-row tiles, four-stage ring; on demand only)
};
constexpr int kTileAuto = 0, kTileWide = 1, kTileDeep = 2, kTileRing = 3;
constexpr int kTileDeepRowsPerExpert = 96;  // the LDS-tiled family picks its deep geometry up to this many routed rows per expert
hipError_t launch_gemm_stream(const GemmArgs& a, hipStream_t stream);
// register-only int8 MFMA loop (measurement aid): sink holds mfma_probe_sink_bytes(workgroups)
int64_t mfma_probe_sink_bytes(int workgroups);
double mfma_probe_ops(int workgroups, int iters);
hipError_t launch_mfma_probe(bool random_operands, int workgroups, int iters, int32_t* sink, hipStream_t stream);
bool gemm_stream_fuses_quant(int k);  // the down GEMM can quantise bf16 activations of this length itself
hipError_t launch_gemm_tile(const GemmArgs& a, hipStream_t stream);
bool gemm_tile_supports(const GemmArgs& a);
bool gemm_tile_prefers_deep(const GemmArgs& a);
int gemm_tile_geometry(const GemmArgs& a);  // kTileWide or kTileDeep (kTileRing on demand): what a launch of the family would use
hipError_t launch_gemm_narrow(const GemmArgs& a, hipStream_t stream);
bool gemm_narrow_supports(const GemmArgs& a);

hipError_t launch_moe_sum(const uint16_t* in, uint16_t* out, int64_t m, int top_k, int hidden,
                          hipStream_t stream);

}  // namespace moe_i8
