// Per-token dynamic symmetric int8 quantisation for gfx950, optionally fused with a row gather.
//
// One 64-lane wavefront owns one output row.  The row is read once with 16-byte loads (8 bf16 per
// lane per load, all loads issued before the first use), the absolute maximum is reduced across
// the wavefront with lane shuffles, and 8 int8 per lane are written with 8-byte stores.  HBM
// traffic is the minimum 2 + 1 bytes per element plus 4 bytes per row.
//
// Arithmetic (fp32): absmax = max(max|x|, 1e-10); scale = absmax / 127;
// q = roundf(x * (127 / absmax))  (ties away from zero).
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / kWave;
constexpr int kVec = 8;  // bf16 elements per 16-byte load

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
__global__ __launch_bounds__(kThreads) void quant_rows_kernel(
    const uint16_t* __restrict__ x, int64_t src_rows, int cols, int64_t row_stride,
    const int32_t* __restrict__ gather, int gather_div, int64_t rows, int8_t* __restrict__ q,
    float* __restrict__ scale) {
  const int lane = lane_id();
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row >= rows) return;
  const int64_t src = gather ? (int64_t)(gather[row] / gather_div) : row;
  const bool have = src >= 0 && src < src_rows;
  const uint4* in = reinterpret_cast<const uint4*>(x + (have ? src : 0) * row_stride);
  uint2* out = reinterpret_cast<uint2*>(q + row * (int64_t)cols);
  const int nvec = cols / kVec;

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
    if (lane == 0) scale[row] = absmax / 127.0f;
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
    if (lane == 0) scale[row] = absmax / 127.0f;
    for (int c = lane; c < nvec; c += kWave)
      out[c] = have ? quant8(in[c], inv) : make_uint2(0u, 0u);
  }
}

}  // namespace

hipError_t launch_quant_rows(const QuantArgs& a, hipStream_t stream) {
  if (a.rows == 0) return hipSuccess;
  const dim3 grid((unsigned)((a.rows + kRowsPerBlock - 1) / kRowsPerBlock));
  const dim3 block(kThreads);
  const int nvec = a.cols / kVec;
#define MOE_I8_QUANT_LAUNCH(V)                                                                  \
  hipLaunchKernelGGL(quant_rows_kernel<V>, grid, block, 0, stream, a.x, a.src_rows, a.cols,     \
                     a.row_stride, a.gather, a.gather_div, a.rows, a.q, a.scale)
  if (nvec <= 1 * kWave) MOE_I8_QUANT_LAUNCH(1);
  else if (nvec <= 2 * kWave) MOE_I8_QUANT_LAUNCH(2);
  else if (nvec <= 4 * kWave) MOE_I8_QUANT_LAUNCH(4);
  else if (nvec <= 8 * kWave) MOE_I8_QUANT_LAUNCH(8);
  else if (nvec <= 16 * kWave) MOE_I8_QUANT_LAUNCH(16);
  else MOE_I8_QUANT_LAUNCH(0);
#undef MOE_I8_QUANT_LAUNCH
  return hipGetLastError();
}

}  // namespace moe_i8
