// Measurement aid, built into its own library (libmoe_i8_probe.so) that only the benchmark loads:
// a register-only v_mfma_i32_32x32x32_i8 loop on every compute unit.
//
// The published int8 peak assumes the full shader clock.  Under the board's power limit the clock the
// matrix pipes sustain depends on how much the operand bits toggle, so the rate reached with
// constant operands and with pseudo-random ones brackets what any int8 GEMM on real data can reach
// on the device at hand.  The benchmark prints both next to its roofline.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kProbeThreads = 512;
constexpr int kProbeTiles = 8;  // independent accumulator tiles per wavefront

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

template <bool kRandom>
__global__ __launch_bounds__(kProbeThreads) void mfma_rate_kernel(int32_t* sink, int iters) {
  v4i a[4], b[2];
  const uint32_t id = (blockIdx.x * kProbeThreads + threadIdx.x) * 32u;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) a[i][r] = kRandom ? (int)mix32(id + i * 4 + r) : 0x01010101;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) b[i][r] = kRandom ? (int)mix32(id + 16 + i * 4 + r) : 0x02020202;
  v16i acc[kProbeTiles];
#pragma unroll
  for (int i = 0; i < kProbeTiles; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kProbeTiles; ++i)
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i / 2], b[i % 2], acc[i], 0, 0, 0);
  }
  int32_t s = 0;
#pragma unroll
  for (int i = 0; i < kProbeTiles; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  sink[(int64_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
}

}  // namespace

int64_t mfma_probe_sink_bytes(int workgroups) { return (int64_t)workgroups * kProbeThreads * sizeof(int32_t); }

double mfma_probe_ops(int workgroups, int iters) {
  return (double)workgroups * (kProbeThreads / kWave) * iters * kProbeTiles * (2.0 * 32 * 32 * 32);
}

hipError_t launch_mfma_probe(bool random_operands, int workgroups, int iters, int32_t* sink, hipStream_t stream) {
  if (random_operands)
    hipLaunchKernelGGL(mfma_rate_kernel<true>, dim3((unsigned)workgroups), dim3(kProbeThreads), 0, stream, sink, iters);
  else
    hipLaunchKernelGGL(mfma_rate_kernel<false>, dim3((unsigned)workgroups), dim3(kProbeThreads), 0, stream, sink, iters);
  return hipGetLastError();
}

}  // namespace moe_i8

// C entry points of the probe library.  sink: device buffer of moe_i8_probe_sink_bytes(workgroups)
// bytes (written, never read); returns 0 or a HIP error code.
extern "C" {
long long moe_i8_probe_sink_bytes(int workgroups) { return moe_i8::mfma_probe_sink_bytes(workgroups); }
double moe_i8_probe_mfma_ops(int workgroups, int iters) {
  return workgroups > 0 && iters > 0 ? moe_i8::mfma_probe_ops(workgroups, iters) : 0.0;
}
int moe_i8_probe_mfma(int random_operands, int workgroups, int iters, void* sink, long long sink_bytes, void* stream) {
  if (workgroups < 1 || workgroups > 65535 || iters < 1 || !sink || sink_bytes < moe_i8::mfma_probe_sink_bytes(workgroups))
    return (int)hipErrorInvalidValue;
  return (int)moe_i8::launch_mfma_probe(random_operands != 0, workgroups, iters, static_cast<int32_t*>(sink),
                                        static_cast<hipStream_t>(stream));
}
}
