// Grouped int8 GEMM for gfx950, weight-streaming family (few rows per expert: decode).
//
// In this regime every weight byte is used by one 64-row block only, so the kernel is a pure
// HBM stream: weights go global -> registers in the MFMA operand layout with 16-byte loads, never
// through LDS, and the activation rows (a few KB per block) are re-read from the vector cache.
//
// v_mfma_i32_16x16x64_i8 is used "transposed": the A operand carries 16 weight rows (output
// channels), the B operand 16 token rows, so each lane ends up with 4 consecutive channels of one
// token and the epilogue stores 8 (bf16) or 16 (int32) contiguous bytes per lane.  Lane l feeds
// row/column l % 16 and the 16 reduction bytes [16 * (l / 16), +16) of each 64-byte step; both
// operands use the same split, so the reduction order inside the instruction is immaterial.
//
// A 64-row block is handled as up to four 16-row sub-tiles; sub-tiles that hold only padding are
// skipped (valid rows are a prefix of the block), so a block with 1..16 routed rows costs one
// MFMA per 64 weight bytes per lane group.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kSub = 16;    // token rows per sub-tile (MFMA N)
constexpr int kGroup = 4;   // sub-tiles processed per pass over the weights
constexpr int kStepK = 64;  // reduction bytes per MFMA
#ifndef MOE_I8_STREAM_UNROLL
#define MOE_I8_STREAM_UNROLL 4
#endif
#ifndef MOE_I8_STREAM_TPW
#define MOE_I8_STREAM_TPW 2
#endif
#ifndef MOE_I8_STREAM_NT
#define MOE_I8_STREAM_NT 1
#endif
constexpr int kUnroll = MOE_I8_STREAM_UNROLL;  // MFMA steps whose loads are issued together

struct StreamParams {
  const int8_t* a_q;
  const float* a_scale;
  const int8_t* w;
  const float* w_scale;
  const float* row_weight;
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* npp;
  int64_t P;
  int row_div;
  int E;
  int N;
  int K;
  int B;
  void* out;
};

__device__ __forceinline__ v4i load_weights(const int8_t* p) {
#if MOE_I8_STREAM_NT
  return __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
#else
  return *reinterpret_cast<const v4i*>(p);
#endif
}

template <int MODE, int TPW, int NS>
__device__ __forceinline__ void stream_pass(const StreamParams& p, int blk, int e, int sub0,
                                            const int (&wrow)[TPW], const bool (&wok)[TPW]) {
  const int lane = lane_id();
  const int col = lane & 15;  // token slot inside a sub-tile / weight row inside a tile
  const int grp = lane >> 4;  // which 16 reduction bytes of each step; which 4 output channels
  const int K = p.K;

  int32_t tok[NS];
  bool tok_ok[NS];
  const int8_t* ap[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    tok[s] = p.sorted_ids[(int64_t)blk * p.B + (sub0 + s) * kSub + col];
    tok_ok[s] = tok[s] >= 0 && tok[s] < p.P;
    const int64_t arow = tok_ok[s] ? tok[s] / p.row_div : 0;
    ap[s] = p.a_q + arow * K + grp * 16;
  }
  const int8_t* wp[TPW];
#pragma unroll
  for (int t = 0; t < TPW; ++t)
    wp[t] = p.w + ((int64_t)e * p.N + wrow[t] + col) * K + grp * 16;

  v4i acc[TPW][NS];
#pragma unroll
  for (int t = 0; t < TPW; ++t)
#pragma unroll
    for (int s = 0; s < NS; ++s) acc[t][s] = v4i{0, 0, 0, 0};

  int k0 = 0;
  for (; k0 + kStepK * kUnroll <= K; k0 += kStepK * kUnroll) {
    v4i wv[kUnroll][TPW];
    v4i av[kUnroll][NS];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int t = 0; t < TPW; ++t)
        wv[u][t] = load_weights(wp[t] + k0 + u * kStepK);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int s = 0; s < NS; ++s)
        av[u][s] = *reinterpret_cast<const v4i*>(ap[s] + k0 + u * kStepK);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s)
          acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[u][t], av[u][s], acc[t][s], 0, 0, 0);
  }
  for (; k0 < K; k0 += kStepK) {
    v4i wv[TPW];
    v4i av[NS];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
      wv[t] = load_weights(wp[t] + k0);
#pragma unroll
    for (int s = 0; s < NS; ++s) av[s] = *reinterpret_cast<const v4i*>(ap[s] + k0);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int s = 0; s < NS; ++s)
        acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[t], av[s], acc[t][s], 0, 0, 0);
  }

  // Epilogue: lane holds channels wrow[t] + 4 * grp + {0..3} of token tok[s].
  if constexpr (MODE == kAccI32) {
    int32_t* out = static_cast<int32_t*>(p.out);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (wok[t] && tok_ok[s])
          *reinterpret_cast<v4i*>(out + (int64_t)tok[s] * p.N + wrow[t] + 4 * grp) = acc[t][s];
  } else if constexpr (MODE == kDown) {
    uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (!tok_ok[s]) continue;
      const float as = p.a_scale[tok[s] / p.row_div];
      const float rw = p.row_weight[tok[s]];
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        if (!wok[t]) continue;
        const int n = wrow[t] + 4 * grp;
        const float4 ws = *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + n);
        const int v[4] = {acc[t][s][0], acc[t][s][1], acc[t][s][2], acc[t][s][3]};
        *reinterpret_cast<uint2*>(out + (int64_t)tok[s] * p.N + n) = down_epilogue4(v, as, ws, rw);
      }
    }
  } else {  // kGateUpSilu: tiles come in (gate, up) pairs; out is [P, N / 2]
    uint16_t* out = static_cast<uint16_t*>(p.out);
    const int inter = p.N / 2;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (!tok_ok[s]) continue;
      const float as = p.a_scale[tok[s] / p.row_div];
#pragma unroll
      for (int t = 0; t < TPW; t += 2) {
        if (!wok[t]) continue;
        const int n = wrow[t] + 4 * grp;  // gate channel; up channel is n + inter
        const float4 wg = *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + n);
        const float4 wu =
            *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + inter + n);
        const int g[4] = {acc[t][s][0], acc[t][s][1], acc[t][s][2], acc[t][s][3]};
        const int u[4] = {acc[t + 1][s][0], acc[t + 1][s][1], acc[t + 1][s][2], acc[t + 1][s][3]};
        *reinterpret_cast<uint2*>(out + (int64_t)tok[s] * inter + n) = silu_mul_epilogue4(g, u, as, wg, wu);
      }
    }
  }
}

// grid.x: groups of kWaves wave-tiles along the weight rows; grid.y: 64-row (B-row) blocks.
template <int MODE, int TPW>
__global__ __launch_bounds__(kThreads) void gemm_stream_kernel(StreamParams p) {
  const int blk = blockIdx.y;
  const int npp = *p.npp;
  if ((int64_t)blk * p.B >= npp) return;
  const int e = p.expert_ids[blk];
  if (e < 0 || e >= p.E) return;
  const int lane = lane_id();
  const int wt = blockIdx.x * kWaves + threadIdx.x / kWave;

  int wrow[TPW];
  bool wok[TPW];
  if constexpr (MODE == kGateUpSilu) {
    const int inter = p.N / 2;
#pragma unroll
    for (int t = 0; t < TPW; t += 2) {
      const int ch = (wt * (TPW / 2) + t / 2) * 16;
      wok[t] = wok[t + 1] = ch < inter;
      wrow[t] = wok[t] ? ch : 0;
      wrow[t + 1] = wok[t] ? inter + ch : 0;
    }
  } else {
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int ch = (wt * TPW + t) * 16;
      wok[t] = ch < p.N;
      wrow[t] = wok[t] ? ch : 0;
    }
  }
  if (!wok[0]) return;

  // Valid rows are a prefix of the block: count them to know how many sub-tiles to run.
  int nvalid = 0;
  for (int base = 0; base < p.B; base += kWave) {
    const int slot = base + lane;
    const int32_t t = slot < p.B ? p.sorted_ids[(int64_t)blk * p.B + slot] : -1;
    nvalid += __popcll(__ballot(t >= 0 && t < p.P));
  }
  const int nsub = (nvalid + kSub - 1) / kSub;
  for (int sub0 = 0; sub0 < nsub; sub0 += kGroup) {
    const int ns = nsub - sub0 < kGroup ? nsub - sub0 : kGroup;
    switch (ns) {
      case 1: stream_pass<MODE, TPW, 1>(p, blk, e, sub0, wrow, wok); break;
      case 2: stream_pass<MODE, TPW, 2>(p, blk, e, sub0, wrow, wok); break;
      case 3: stream_pass<MODE, TPW, 3>(p, blk, e, sub0, wrow, wok); break;
      default: stream_pass<MODE, TPW, 4>(p, blk, e, sub0, wrow, wok); break;
    }
  }
}

template <int MODE, int TPW>
hipError_t launch_mode(const GemmArgs& a, hipStream_t stream) {
  StreamParams p;
  p.a_q = a.a_q;
  p.a_scale = a.a_scale;
  p.w = a.w;
  p.w_scale = a.w_scale;
  p.row_weight = a.row_weight;
  p.sorted_ids = a.sorted_token_ids;
  p.expert_ids = a.expert_ids;
  p.npp = a.num_tokens_post_padded;
  p.P = a.num_pairs;
  p.row_div = a.row_div;
  p.E = a.num_experts;
  p.N = a.n;
  p.K = a.k;
  p.B = a.block_size;
  p.out = a.out;
  const int row_tiles = MODE == kGateUpSilu ? a.n / 2 / 16 : a.n / 16;
  const int tiles_per_wave = MODE == kGateUpSilu ? TPW / 2 : TPW;
  const int wave_tiles = (row_tiles + tiles_per_wave - 1) / tiles_per_wave;
  const int64_t blocks = (a.sorted_cap + a.block_size - 1) / a.block_size;
  if (blocks == 0 || wave_tiles == 0) return hipSuccess;
  if (blocks > 65535) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((wave_tiles + kWaves - 1) / kWaves), (unsigned)blocks);
  hipLaunchKernelGGL((gemm_stream_kernel<MODE, TPW>), grid, dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_stream(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case kGateUpSilu: return launch_mode<kGateUpSilu, MOE_I8_STREAM_TPW>(a, stream);
    case kDown: return launch_mode<kDown, MOE_I8_STREAM_TPW>(a, stream);
    case kAccI32: return launch_mode<kAccI32, MOE_I8_STREAM_TPW>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe_i8
