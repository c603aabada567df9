// Per-token int8 quantisation of one row by one wavefront (shared by the stand-alone quantiser and
// by the launch that fuses it with moe_align for small batches).
#pragma once

#include "common.hpp"

namespace moe_i8 {

constexpr int kQuantVec = 8;  // bf16 elements per 16-byte load

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = kWave / 2; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
  return v;
}

__device__ __forceinline__ float absmax8(const uint4& v) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m = fmaxf(m, fabsf(__uint_as_float(w[i] << 16)));
    m = fmaxf(m, fabsf(__uint_as_float(w[i] & 0xffff0000u)));
  }
  return m;
}

__device__ __forceinline__ uint2 quant8(const uint4& v, float inv) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t out[2] = {0u, 0u};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lo = (int)roundf(__uint_as_float(w[i] << 16) * inv);
    const int hi = (int)roundf(__uint_as_float(w[i] & 0xffff0000u) * inv);
    const uint32_t pair = ((uint32_t)lo & 0xffu) | (((uint32_t)hi & 0xffu) << 8);
    out[i >> 1] |= pair << ((i & 1) * 16);
  }
  return make_uint2(out[0], out[1]);
}

// VPL = 16-byte vectors per lane held in registers (covers cols <= VPL * 512).
// VPL == 0: rows of any length, read twice (second read served by the caches).
template <int VPL>
__device__ __forceinline__ void quant_one_row(const QuantArgs& a, int64_t row) {
  const int lane = lane_id();
  const int64_t src = a.gather ? (int64_t)(a.gather[row] / a.gather_div) : row;
  const bool have = src >= 0 && src < a.src_rows;
  const uint4* in = reinterpret_cast<const uint4*>(a.x + (have ? src : 0) * a.row_stride);
  uint2* out = reinterpret_cast<uint2*>(a.q + row * (int64_t)a.cols);
  const int nvec = a.cols / kQuantVec;

  if constexpr (VPL > 0) {
    uint4 v[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = lane + i * kWave;
      v[i] = (have && c < nvec) ? in[c] : make_uint4(0u, 0u, 0u, 0u);
    }
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) m = fmaxf(m, absmax8(v[i]));
    const float absmax = fmaxf(wave_max(m), 1e-10f);
    const float inv = 127.0f / absmax;
    if (lane == 0) a.scale[row] = absmax / 127.0f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = lane + i * kWave;
      if (c < nvec) out[c] = quant8(v[i], inv);
    }
  } else {
    float m = 0.0f;
    if (have)
      for (int c = lane; c < nvec; c += kWave) m = fmaxf(m, absmax8(in[c]));
    const float absmax = fmaxf(wave_max(m), 1e-10f);
    const float inv = 127.0f / absmax;
    if (lane == 0) a.scale[row] = absmax / 127.0f;
    for (int c = lane; c < nvec; c += kWave)
      out[c] = have ? quant8(in[c], inv) : make_uint2(0u, 0u);
  }
}

// Smallest register-resident variant that covers a row of `cols` elements (0 = streaming variant).
inline int quant_vectors_per_lane(int cols) {
  const int nvec = cols / kQuantVec;
  for (int v = 1; v <= 16; v *= 2)
    if (nvec <= v * kWave) return v;
  return 0;
}

}  // namespace moe_i8
