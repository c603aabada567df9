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
};
hipError_t launch_quant_rows(const QuantArgs& a, hipStream_t stream);
// Per-output-channel weight quantisation (round to nearest even of w / scale, scale = absmax / 127).
hipError_t launch_quant_weights(const QuantArgs& a, hipStream_t stream);
// moe_align and the quantisation of `q` in one launch; only when align_quant_fusable() says so.
bool align_quant_fusable(const AlignArgs& a, const QuantArgs& q);
hipError_t launch_align_quant(const AlignArgs& a, const QuantArgs& q, hipStream_t stream);

enum GemmMode { kGateUpSilu = 0, kDown = 1, kAccI32 = 2 };

struct GemmArgs {
  int mode;
  const int8_t* a_q;      // [*, K] activations (int8)
  const float* a_scale;   // per activation row
  const int8_t* w;        // [E, N, K]
  const float* w_scale;   // [E, N]
  const float* row_weight;  // [P] routed weights (down) or null
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
};
hipError_t launch_gemm_stream(const GemmArgs& a, hipStream_t stream);
hipError_t launch_gemm_tile(const GemmArgs& a, hipStream_t stream);
bool gemm_tile_supports(const GemmArgs& a);

hipError_t launch_moe_sum(const uint16_t* in, uint16_t* out, int64_t m, int top_k, int hidden,
                          hipStream_t stream);

}  // namespace moe_i8
