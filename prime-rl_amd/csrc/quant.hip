// Per-token dynamic symmetric int8 quantisation for gfx950, optionally fused with a row gather.
//
// One 64-lane wavefront owns one output row.  The row is read once with 16-byte loads (8 bf16 per
// lane per load, all loads issued before the first use), the absolute maximum is reduced across
// the wavefront with lane shuffles, and 8 int8 per lane are written with 8-byte stores.  HBM
// traffic is the minimum 2 + 1 bytes per element plus 4 bytes per row.
//
// Arithmetic (fp32): absmax = max(max|x|, 1e-10); scale = absmax / 127;
// q = roundf(x * (127 / absmax))  (ties away from zero).
#include "quant_body.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / kWave;

template <int VPL>
__global__ __launch_bounds__(kThreads) void quant_rows_kernel(QuantArgs a) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row < a.rows) quant_one_row<VPL>(a, row);
}

}  // namespace

hipError_t launch_quant_rows(const QuantArgs& a, hipStream_t stream) {
  if (a.rows == 0) return hipSuccess;
  const dim3 grid((unsigned)((a.rows + kRowsPerBlock - 1) / kRowsPerBlock));
  const dim3 block(kThreads);
  switch (quant_vectors_per_lane(a.cols)) {
    case 1: hipLaunchKernelGGL(quant_rows_kernel<1>, grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL(quant_rows_kernel<2>, grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL(quant_rows_kernel<4>, grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL(quant_rows_kernel<8>, grid, block, 0, stream, a); break;
    case 16: hipLaunchKernelGGL(quant_rows_kernel<16>, grid, block, 0, stream, a); break;
    default: hipLaunchKernelGGL(quant_rows_kernel<0>, grid, block, 0, stream, a); break;
  }
  return hipGetLastError();
}

}  // namespace moe_i8
