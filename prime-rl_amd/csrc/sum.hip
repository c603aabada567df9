// Top-k combine for gfx950: out[m, :] = sum_j in[m, j, :] over bf16 rows.
//
// One lane owns 8 consecutive columns (one 16-byte load per routed row, one 16-byte store).
// For k in {2, 3, 4} the adds round to bf16 after every step; any other k accumulates in fp32
// in ascending j and rounds once.  Traffic is the minimum (k + 1) * M * H * 2 bytes.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;

template <bool kRoundEachAdd>
__global__ __launch_bounds__(kThreads) void moe_sum_kernel(const uint4* __restrict__ in,
                                                           uint4* __restrict__ out, int64_t total,
                                                           int top_k, int vec_per_row) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t m = i / vec_per_row;
  const int c = (int)(i - m * vec_per_row);
  const uint4* src = in + m * (int64_t)top_k * vec_per_row + c;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
  for (int j = 0; j < top_k; ++j) {
    const uint4 v = src[(int64_t)j * vec_per_row];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = __uint_as_float(w[e] << 16);
      const float hi = __uint_as_float(w[e] & 0xffff0000u);
      if (kRoundEachAdd && j > 0) {
        acc[2 * e] = round_to_bf16(acc[2 * e] + lo);
        acc[2 * e + 1] = round_to_bf16(acc[2 * e + 1] + hi);
      } else {
        acc[2 * e] += lo;
        acc[2 * e + 1] += hi;
      }
    }
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    o[e] = f32_to_bf16_bits(acc[2 * e]) | (f32_to_bf16_bits(acc[2 * e + 1]) << 16);
  out[i] = make_uint4(o[0], o[1], o[2], o[3]);
}

}  // namespace

hipError_t launch_moe_sum(const uint16_t* in, uint16_t* out, int64_t m, int top_k, int hidden,
                          hipStream_t stream) {
  const int vec_per_row = hidden / 8;
  const int64_t total = m * vec_per_row;
  if (total == 0) return hipSuccess;
  const dim3 grid((unsigned)((total + kThreads - 1) / kThreads));
  if (top_k >= 2 && top_k <= 4)
    hipLaunchKernelGGL(moe_sum_kernel<true>, grid, dim3(kThreads), 0, stream,
                       reinterpret_cast<const uint4*>(in), reinterpret_cast<uint4*>(out), total,
                       top_k, vec_per_row);
  else
    hipLaunchKernelGGL(moe_sum_kernel<false>, grid, dim3(kThreads), 0, stream,
                       reinterpret_cast<const uint4*>(in), reinterpret_cast<uint4*>(out), total,
                       top_k, vec_per_row);
  return hipGetLastError();
}

}  // namespace moe_i8
