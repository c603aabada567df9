// Symmetric int8 quantisation for gfx950, one scale per row: activations (per token, optionally
// fused with a row gather) and weights (per output channel).
//
// Activations: one 64-lane wavefront owns one output row.  The row is read once with 16-byte loads
// (8 bf16 per lane per load, all loads issued before the first use), the absolute maximum is
// reduced across the wavefront with lane permutes, and 8 int8 per lane are written with 8-byte
// stores.  HBM traffic is the minimum 2 + 1 bytes per element plus 4 bytes per row.
// Arithmetic (fp32): absmax = max(max|x|, 1e-10); scale = absmax / 127;
// q = round(x * (127 / absmax)), ties away from zero (MoE path) or to even (dense path).
//
// Weights: scale = max(absmax / 127, 1e-12); q = rint(x / scale); a wavefront walks several
// consecutive rows with the next rows' loads in flight (see quant_weights_kernel).
#include "quant_body.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / kWave;

template <int VPL, int kMode>
__global__ __launch_bounds__(kThreads) void quant_rows_kernel(QuantArgs a) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row < a.rows) quant_one_row<VPL, kMode>(a, row);
  if (a.route_sorted != nullptr) {
    // identity routing of a.rows rows, written by all threads of the launch in strides
    const int rows = (int)a.rows;
    const int padded = (rows + a.route_block - 1) / a.route_block * a.route_block;
    const int64_t blocks_cap = (a.route_cap + a.route_block - 1) / a.route_block;
    const int64_t step = (int64_t)gridDim.x * kThreads;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < a.route_cap; i += step) {
      a.route_sorted[i] = i < rows ? (int32_t)i : rows;
      if (i < blocks_cap) a.route_expert_ids[i] = i < padded / a.route_block ? 0 : -1;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) *a.route_npp = padded;
  }
}

template <int kMode>
void launch_quant_rows_mode(const QuantArgs& a, dim3 grid, dim3 block, hipStream_t stream) {
  switch (quant_vectors_per_lane(a.cols)) {
    case 1: hipLaunchKernelGGL((quant_rows_kernel<1, kMode>), grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL((quant_rows_kernel<2, kMode>), grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL((quant_rows_kernel<4, kMode>), grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL((quant_rows_kernel<8, kMode>), grid, block, 0, stream, a); break;
    case 16: hipLaunchKernelGGL((quant_rows_kernel<16, kMode>), grid, block, 0, stream, a); break;
    default: hipLaunchKernelGGL((quant_rows_kernel<0, kMode>), grid, block, 0, stream, a); break;
  }
}

// Weights: rows are contiguous and there are many of them, so a wavefront walks kWeightRowsPerWave
// consecutive rows through a ring of kDepth row buffers in registers: the loads of the next
// kDepth - 1 rows stay in flight while the current row is reduced, quantised and stored (a
// wavefront that lives for a single row spends much of its life with nothing outstanding, and
// short rows need several in flight to cover the HBM latency).  kDepth * VPL = 8 vectors of 16
// bytes per lane, 8 KB per wavefront.  Loads and stores are nontemporal: every byte is touched once.
constexpr int kWeightRowsPerWave = 16;
constexpr int kWeightVectorsInFlight = 8;  // 16-byte loads per lane kept in flight

// No branch around the loads (the compiler would wait for everything outstanding at the join):
// lanes past the end of the row, and rows past the end of the wavefront's share, read the first
// vector of the share instead, one cached line for the whole wavefront.
template <int VPL>
__device__ __forceinline__ void load_weight_row(const v4i* first, const v4i* in, bool row_valid, int nvec,
                                                int lane, v4i (&v)[VPL]) {
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = lane + i * kWave;
    v[i] = __builtin_nontemporal_load(row_valid && c < nvec ? in + c : first);
  }
}

__device__ __forceinline__ uint4 as_uint4(const v4i& v) {
  return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}

template <int VPL>
__global__ __launch_bounds__(kThreads) void quant_weights_kernel(QuantArgs a) {
  constexpr int kDepth = kWeightVectorsInFlight / VPL > 1 ? kWeightVectorsInFlight / VPL : 1;
  static_assert(kWeightRowsPerWave % kDepth == 0, "ring depth must divide the rows of a wavefront");
  const int lane = lane_id();
  const int64_t wave = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  const int64_t row0 = wave * kWeightRowsPerWave;
  if (row0 >= a.rows) return;
  const int n = (int)(a.rows - row0 < kWeightRowsPerWave ? a.rows - row0 : kWeightRowsPerWave);
  const int nvec = a.cols / kQuantVec;
  const int64_t vec_stride = a.row_stride / kQuantVec;
  const v4i* first = reinterpret_cast<const v4i*>(a.x + row0 * a.row_stride);
  // output row of the share's first row; later rows step by one and jump at a group boundary
  int64_t orow = row0, left_in_group = a.rows;
  if (a.rows_per_group > 0) {
    const int64_t g = row0 / a.rows_per_group, w = row0 - g * a.rows_per_group;
    orow = g * a.out_rows_per_group + a.out_row_offset + w;
    left_in_group = a.rows_per_group - w;
  }
  v4i ring[kDepth][VPL];
#pragma unroll
  for (int s = 0; s < kDepth; ++s) load_weight_row<VPL>(first, first + s * vec_stride, s < n, nvec, lane, ring[s]);
  for (int r0 = 0; r0 < n; r0 += kDepth) {
#pragma unroll
    for (int s = 0; s < kDepth; ++s) {
      const int r = r0 + s;
      float m = 0.0f;
#pragma unroll
      for (int i = 0; i < VPL; ++i)
        m = fmaxf(m, lane + i * kWave < nvec ? absmax8_packed(as_uint4(ring[s][i])) : 0.0f);
      const WeightRcp ws = weight_rcp(fmaxf(wave_max(m) / 127.0f, 1e-12f));
      if (r < n) {
        if (lane == 0) a.scale[orow] = ws.scale;
        uint2* out = reinterpret_cast<uint2*>(a.q + orow * (int64_t)a.cols);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
          const int c = lane + i * kWave;
          if (c < nvec) {
            const uint2 q = quant8_weights(as_uint4(ring[s][i]), ws);
            uint32_t* p = reinterpret_cast<uint32_t*>(out + c);
            __builtin_nontemporal_store(q.x, p);
            __builtin_nontemporal_store(q.y, p + 1);
          }
        }
      }
      load_weight_row<VPL>(first, first + (r + kDepth) * vec_stride, r + kDepth < n, nvec, lane, ring[s]);
      ++orow;
      if (--left_in_group == 0) {
        orow += a.out_rows_per_group - a.rows_per_group;
        left_in_group = a.rows_per_group;
      }
    }
  }
}

// Rows too long to hold in registers: one wavefront per row, read twice.
__global__ __launch_bounds__(kThreads) void quant_weights_long_rows_kernel(QuantArgs a) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row < a.rows) quant_one_row<0, kQuantWeights>(a, row);
}

}  // namespace

hipError_t launch_quant_rows(const QuantArgs& a, hipStream_t stream) {
  if (a.rows == 0) return hipSuccess;
  const dim3 grid((unsigned)((a.rows + kRowsPerBlock - 1) / kRowsPerBlock));
  const dim3 block(kThreads);
  if (a.round_even)
    launch_quant_rows_mode<kQuantEven>(a, grid, block, stream);
  else
    launch_quant_rows_mode<kQuantAway>(a, grid, block, stream);
  return hipGetLastError();
}

hipError_t launch_quant_weights(const QuantArgs& a, hipStream_t stream) {
  if (a.rows == 0) return hipSuccess;
  const int64_t waves = (a.rows + kWeightRowsPerWave - 1) / kWeightRowsPerWave;
  const dim3 grid((unsigned)((waves + kRowsPerBlock - 1) / kRowsPerBlock));
  const dim3 block(kThreads);
  switch (quant_vectors_per_lane(a.cols)) {
    case 1: hipLaunchKernelGGL(quant_weights_kernel<1>, grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL(quant_weights_kernel<2>, grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL(quant_weights_kernel<4>, grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL(quant_weights_kernel<8>, grid, block, 0, stream, a); break;
    case 16: hipLaunchKernelGGL(quant_weights_kernel<16>, grid, block, 0, stream, a); break;
    default:
      hipLaunchKernelGGL(quant_weights_long_rows_kernel,
                         dim3((unsigned)((a.rows + kRowsPerBlock - 1) / kRowsPerBlock)), block, 0, stream, a);
      break;
  }
  return hipGetLastError();
}

}  // namespace moe_i8
