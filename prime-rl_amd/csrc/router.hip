// Token-choice top-k routing for gfx950: scores, optional grouped pre-selection, top-k, weight
// normalisation and the compact routed-experts record, one launch.
//
// One 64-lane wavefront owns one token.  Lane l holds experts [l*C, (l+1)*C) in registers
// (C = 1, 2, 4, 8 or 16, so up to 1024 experts), which makes every expert group a run of whole
// lanes: group reductions are xor-butterflies over that run.  Selection is k rounds of a wave-wide
// arg-max: the maximum by lane permutes on the VALU, then a ballot of the lanes that hold it; the
// lowest such lane wins, and inside a lane the lowest slot, so equal values resolve to the lowest
// expert index and the result comes out in descending order.  HBM traffic is the minimum: the
// logits once in, k weights and k indices out.
//
// Arithmetic is fp32 throughout.  score: softmax over all experts, sigmoid, or the raw logit
// (softmax over the selected k afterwards).  A selection bias is added for choosing only; the
// returned weights come from the unbiased scores, optionally divided by (their sum + 1e-20) and
// multiplied by a scale.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kTokensPerBlock = kThreads / kWave;
constexpr float kNegInf = -__builtin_huge_valf();

// Lowest lane whose value equals the wave-wide maximum of `v` (lanes with `live` false never win
// unless no lane is live, which the callers exclude).
__device__ __forceinline__ int wave_argmax_lane(float v, bool live) {
  const float top = wave_reduce_max(live ? v : kNegInf);
  const uint64_t holders = __ballot(live && v == top);
  return __ffsll((unsigned long long)holders) - 1;
}

template <int C>
__global__ __launch_bounds__(kThreads) void route_topk_kernel(RouteArgs a) {
  const int lane = lane_id();
  const int64_t tok = (int64_t)blockIdx.x * kTokensPerBlock + threadIdx.x / kWave;
  if (tok >= a.m) return;
  const int E = a.num_experts;
  const int k = a.top_k;
  const int e0 = lane * C;
  const float* row = a.logits + tok * (int64_t)E;

  float s[C];  // unbiased score (the source of the returned weights)
  float v[C];  // selection value
#pragma unroll
  for (int j = 0; j < C; ++j) s[j] = e0 + j < E ? row[e0 + j] : kNegInf;

  if (a.score_func == kScoreSoftmax) {
    float mx = kNegInf;
#pragma unroll
    for (int j = 0; j < C; ++j) mx = fmaxf(mx, s[j]);
    mx = wave_reduce_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < C; ++j) {
      s[j] = e0 + j < E ? expf(s[j] - mx) : 0.0f;
      sum += s[j];
    }
    sum = wave_reduce_sum(sum);
#pragma unroll
    for (int j = 0; j < C; ++j) s[j] = s[j] / sum;
  } else if (a.score_func == kScoreSigmoid) {
#pragma unroll
    for (int j = 0; j < C; ++j) s[j] = 1.0f / (1.0f + expf(-s[j]));
  }
#pragma unroll
  for (int j = 0; j < C; ++j) {
    v[j] = kNegInf;
    if (e0 + j < E) v[j] = a.bias ? s[j] + a.bias[e0 + j] : s[j];
  }

  if (a.num_groups > 1) {
    // group score = largest (or sum of the two largest) selection values of the group
    const int lanes_per_group = E / a.num_groups / C;
    float t1 = kNegInf, t2 = kNegInf;
#pragma unroll
    for (int j = 0; j < C; ++j) {
      t2 = fmaxf(t2, fminf(t1, v[j]));
      t1 = fmaxf(t1, v[j]);
    }
    for (int d = 1; d < lanes_per_group; d <<= 1) {
      const float o1 = __shfl_xor(t1, d), o2 = __shfl_xor(t2, d);
      t2 = fmaxf(fminf(t1, o1), fmaxf(t2, o2));
      t1 = fmaxf(t1, o1);
    }
    const float group_score = a.group_top2 ? t1 + t2 : t1;
    const int group = lane / lanes_per_group;
    bool chosen = false;
    for (int it = 0; it < a.topk_groups; ++it) {
      const int win = wave_argmax_lane(group_score, !chosen && group < a.num_groups) / lanes_per_group;
      if (group == win) chosen = true;
    }
#pragma unroll
    for (int j = 0; j < C; ++j) v[j] = chosen ? v[j] : kNegInf;
  }

  uint32_t taken = 0u;
  float my_w = 0.0f;
  int my_id = 0;
  for (int it = 0; it < k; ++it) {
    float best_v = kNegInf, best_s = 0.0f;
    int best_j = -1;
#pragma unroll
    for (int j = 0; j < C; ++j) {
      const bool open = e0 + j < E && !((taken >> j) & 1u);
      if (open && (best_j < 0 || v[j] > best_v)) {
        best_v = v[j];
        best_s = s[j];
        best_j = j;
      }
    }
    const int owner = wave_argmax_lane(best_v, best_j >= 0);
    const int e = __builtin_amdgcn_readlane(e0 + best_j, owner);
    const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(best_s), owner));
    if (lane == owner) taken |= 1u << best_j;
    if (lane == it) {
      my_w = w;
      my_id = e;
    }
  }

  const bool mine = lane < k;
  if (a.score_func == kScoreTopkSoftmax) {
    const float mx = wave_reduce_max(mine ? my_w : kNegInf);
    const float ex = mine ? expf(my_w - mx) : 0.0f;
    my_w = ex / wave_reduce_sum(ex);
  }
  if (a.renormalize) my_w = my_w / (wave_reduce_sum(mine ? my_w : 0.0f) + 1e-20f);
  my_w *= a.route_scale;
  if (mine) {
    a.weights[tok * k + lane] = my_w;
    a.ids[tok * k + lane] = my_id;
    const int64_t at = tok * a.capture_stride + a.capture_offset + lane;
    if (a.capture_bytes == 1) static_cast<uint8_t*>(a.capture)[at] = (uint8_t)my_id;
    if (a.capture_bytes == 2) static_cast<uint16_t*>(a.capture)[at] = (uint16_t)my_id;
  }
}

}  // namespace

int route_experts_per_lane(int num_experts) {
  int c = 1;
  while (c * kWave < num_experts) c <<= 1;
  return c;
}

hipError_t launch_route_topk(const RouteArgs& a, hipStream_t stream) {
  if (a.m == 0) return hipSuccess;
  const dim3 grid((unsigned)((a.m + kTokensPerBlock - 1) / kTokensPerBlock));
  const dim3 block(kThreads);
  switch (route_experts_per_lane(a.num_experts)) {
    case 1: hipLaunchKernelGGL(route_topk_kernel<1>, grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL(route_topk_kernel<2>, grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL(route_topk_kernel<4>, grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL(route_topk_kernel<8>, grid, block, 0, stream, a); break;
    case 16: hipLaunchKernelGGL(route_topk_kernel<16>, grid, block, 0, stream, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace moe_i8
