// Per-token int8 quantisation of one row by one wavefront (shared by the stand-alone quantiser and
// by the launch that fuses it with moe_align for small batches).
#pragma once

#include "common.hpp"

namespace moe_i8 {

constexpr int kQuantVec = 8;  // bf16 elements per 16-byte load

__device__ __forceinline__ float wave_max(float v) { return wave_reduce_max(v); }

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

// kEven: ties to even (rintf) instead of away from zero (roundf).
template <bool kEven = false>
__device__ __forceinline__ uint2 quant8(const uint4& v, float inv) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t out[2] = {0u, 0u};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float flo = __uint_as_float(w[i] << 16) * inv, fhi = __uint_as_float(w[i] & 0xffff0000u) * inv;
    const int lo = (int)(kEven ? rintf(flo) : roundf(flo));
    const int hi = (int)(kEven ? rintf(fhi) : roundf(fhi));
    const uint32_t pair = ((uint32_t)lo & 0xffu) | (((uint32_t)hi & 0xffu) << 8);
    out[i >> 1] |= pair << ((i & 1) * 16);
  }
  return make_uint2(out[0], out[1]);
}

// Largest |x| of 8 packed bf16 as a float.  Without the sign bit, bf16 patterns order like unsigned
// integers, so the maximum is taken on packed 16-bit lanes (two elements per operation).
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float absmax8_packed(const uint4& v) {
  const uint32_t w[4] = {v.x & 0x7fff7fffu, v.y & 0x7fff7fffu, v.z & 0x7fff7fffu, v.w & 0x7fff7fffu};
  u16x2 m = __builtin_elementwise_max(
      __builtin_elementwise_max(__builtin_bit_cast(u16x2, w[0]), __builtin_bit_cast(u16x2, w[1])),
      __builtin_elementwise_max(__builtin_bit_cast(u16x2, w[2]), __builtin_bit_cast(u16x2, w[3])));
  const uint32_t top = m[0] > m[1] ? m[0] : m[1];
  return __uint_as_float(top << 16);
}

// Weight flavour of quant8: q = rint(x / scale) (ties to even, the correctly rounded fp32 quotient),
// |q| <= 127 by construction of scale for finite weights.
//
// A correctly rounded division costs ~11 VALU operations per element.  Instead
// fma(x, r, 1.5 * 2^23) rounds the exact product x * r to the nearest-even integer in ONE operation
// (at that magnitude one ulp is 1) and leaves it as a two's complement byte in the low mantissa
// bits.  It is evaluated for r = rcp(scale) * (1 -+ 2^-21): v_rcp_f32 is within 1 ulp, so the true
// quotient and its fp32 rounding both lie between the two products, and rounding to an integer is
// monotonic — when both give the same integer, that integer is the answer.  Only when they differ
// (the quotient is within ~1e-4 of k + 0.5) is the vector redone with the true division.
struct WeightRcp {
  float scale, lo, hi;
};
__device__ __forceinline__ WeightRcp weight_rcp(float scale) {
  const float r = __builtin_amdgcn_rcpf(scale);
  return {scale, r * (1.0f - 0x1p-21f), r * (1.0f + 0x1p-21f)};
}

__device__ __forceinline__ uint2 quant8_weights(const uint4& v, const WeightRcp& s) {
  constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  float x[8];
  uint32_t y[8];
  uint32_t differ = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = __uint_as_float(w[i] << 16);
    x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    y[i] = __float_as_uint(fmaf(x[i], s.lo, kMagic));
    differ |= y[i] ^ __float_as_uint(fmaf(x[i], s.hi, kMagic));
    asm("" : "+v"(differ));  // keeps this one xor-or per element (else it becomes 8 compares + a bit mask)
  }
  if (differ) {
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = __float_as_uint(rintf(x[i] / s.scale) + kMagic);
  }
  uint32_t out[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    // low bytes of four results -> one dword (selector: 0-3 = bytes of the 2nd operand, 4-7 = of the 1st)
    const uint32_t p01 = __builtin_amdgcn_perm(y[4 * h + 1], y[4 * h], 0x0c0c0400u);
    const uint32_t p23 = __builtin_amdgcn_perm(y[4 * h + 3], y[4 * h + 2], 0x04000c0cu);
    out[h] = p01 | p23;
  }
  return make_uint2(out[0], out[1]);
}

// VPL = 16-byte vectors per lane held in registers (covers cols <= VPL * 512).
// VPL == 0: rows of any length, read twice (second read served by the caches).
// kMode: kQuantAway = activations, q = roundf(x * (127 / absmax)) (ties away from zero);
// kQuantEven = the same with ties to even; kQuantWeights = per-output-channel weights,
// scale = max(absmax / 127, 1e-12), q = rint(x / scale).
enum QuantMode { kQuantAway = 0, kQuantWeights = 1, kQuantEven = 2 };
template <int VPL, int kMode = kQuantAway>
__device__ __forceinline__ void quant_one_row(const QuantArgs& a, int64_t row) {
  const int lane = lane_id();
  const int64_t src = a.gather ? (int64_t)(a.gather[row] / a.gather_div) : row;
  const bool have = src >= 0 && src < a.src_rows;
  const uint4* in = reinterpret_cast<const uint4*>(a.x + (have ? src : 0) * a.row_stride);
  const int64_t orow = a.rows_per_group > 0
                           ? (row / a.rows_per_group) * a.out_rows_per_group + a.out_row_offset + row % a.rows_per_group
                           : row;
  uint2* out = reinterpret_cast<uint2*>(a.q + orow * (int64_t)a.cols);
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
    if constexpr (kMode == kQuantWeights) {
      const WeightRcp s = weight_rcp(fmaxf(wave_max(m) / 127.0f, 1e-12f));
      if (lane == 0) a.scale[orow] = s.scale;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int c = lane + i * kWave;
        if (c < nvec) out[c] = quant8_weights(v[i], s);
      }
    } else {
      const float absmax = fmaxf(wave_max(m), 1e-10f);
      const float inv = 127.0f / absmax;
      if (lane == 0) a.scale[orow] = absmax / 127.0f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int c = lane + i * kWave;
        if (c < nvec) out[c] = quant8<kMode == kQuantEven>(v[i], inv);
      }
    }
  } else {
    // four independent 16-byte loads per lane and trip, so that a long row is not one load latency per
    // 1 KB of it
    constexpr int kUnroll = 4;
    float m = 0.0f;
    if (have) {
      for (int c0 = lane; c0 < nvec; c0 += kUnroll * kWave) {
        uint4 t[kUnroll];
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
          const int c = c0 + i * kWave;
          t[i] = c < nvec ? in[c] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) m = fmaxf(m, absmax8(t[i]));
      }
    }
    auto second_pass = [&](auto quantise) {
      for (int c0 = lane; c0 < nvec; c0 += kUnroll * kWave) {
        uint4 t[kUnroll];
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
          const int c = c0 + i * kWave;
          t[i] = (have && c < nvec) ? in[c] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
          const int c = c0 + i * kWave;
          if (c < nvec) out[c] = have ? quantise(t[i]) : make_uint2(0u, 0u);
        }
      }
    };
    if constexpr (kMode == kQuantWeights) {
      const WeightRcp s = weight_rcp(fmaxf(wave_max(m) / 127.0f, 1e-12f));
      if (lane == 0) a.scale[orow] = s.scale;
      second_pass([&](const uint4& v) { return quant8_weights(v, s); });
    } else {
      const float absmax = fmaxf(wave_max(m), 1e-10f);
      const float inv = 127.0f / absmax;
      if (lane == 0) a.scale[orow] = absmax / 127.0f;
      second_pass([&](const uint4& v) { return quant8<kMode == kQuantEven>(v, inv); });
    }
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
