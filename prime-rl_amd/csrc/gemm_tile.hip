// Grouped int8 GEMM for gfx950, LDS-tiled family (many rows per expert: prefill).
//
// Workgroup tile: 128 token rows x 256 weight rows (output channels), reduction in steps of 64
// bytes, 256 threads = 4 wavefronts arranged 2 (token halves) x 2 (channel halves); each wavefront
// owns 64 tokens x 128 channels as 2 x 4 v_mfma_i32_32x32x32_i8 tiles (128 accumulator VGPRs).
// The MFMA is used "transposed" (A operand = weight rows, B operand = token rows) so a lane ends
// up with runs of 4 consecutive channels of one token.
//
// moe_align blocks are 64 rows; two consecutive blocks of the same expert form one 128-row tile.
// A pair that straddles two experts is processed as two passes of one 64-row half each.
//
// Both operands go global -> LDS directly (global_load_lds_dwordx4: no staging registers, no
// ds_write) into a ring of three stages: while step s is multiplied the loads of steps s+1 and s+2
// are in flight, with one s_barrier per step and explicit vmcnt waits (the loads complete in
// order).  LDS rows are 64 bytes; a wavefront's load fills 16 rows contiguously, so the XOR swizzle
// of the 16-byte chunk index (which makes the MFMA-layout reads - 32 consecutive rows, same chunk -
// spread over all banks) is applied to the global source address of each lane instead.
//
// Workgroup ids are remapped so that each of the 8 XCDs (id % 8) works on a contiguous range of
// tiles, channel tile fastest: tiles resident on one XCD share token rows and expert weights in
// that XCD's L2.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kBM = 128;  // token rows per tile
constexpr int kBN = 256;  // weight rows per tile
constexpr int kBK = 64;   // reduction bytes per stage
constexpr int kStageBytes = (kBM + kBN) * kBK;
constexpr int kXcds = 8;

struct TileParams {
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
  int ntiles;  // channel tiles
  void* out;
};

__device__ __forceinline__ int swizzle_of_row(int r) {
  return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1);
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = bits 3:0 and
// 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maximum).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// 16 bytes per lane from global memory straight into LDS: lane i lands at lds_base + 16 * i
// (lds_base is wave-uniform and goes through M0).  Issued as inline assembly so that the waits are
// the explicit vmcnt waits of the ring below and not a conservative vmcnt(0) before every LDS read.
__device__ __forceinline__ void load_to_lds_16(const int8_t* src, char* lds_base) {
  const uint32_t dst = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) char*)lds_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(dst)), "v"(src)
               : "memory", "m0");
}

struct TileLoads {
  const int8_t* wsrc[4];
  const int8_t* xsrc[2];
  int wave;
};

// One reduction step of both operands into `stage`: wavefront w fills rows 16 * (w + 4 * i) .. +15.
__device__ __forceinline__ void issue_stage_loads(const TileLoads& ld, char* stage, int koff) {
#pragma unroll
  for (int i = 0; i < 4; ++i) load_to_lds_16(ld.wsrc[i] + koff, stage + (ld.wave + 4 * i) * 1024);
#pragma unroll
  for (int i = 0; i < 2; ++i)
    load_to_lds_16(ld.xsrc[i] + koff, stage + kBN * kBK + (ld.wave + 4 * i) * 1024);
}

struct TileReads {
  int w_ld[4];
  int x_ld[2];
  int chunk[4];  // swizzled byte offset of logical chunk 2 * kk + (lane >> 5), kk = 0..1 -> [kk]
};

__device__ __forceinline__ void multiply_stage(const TileReads& rd, const char* stage, v16i (&acc)[4][2]) {
  v4i a[2][4], b[2][2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) a[kk][ci] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[ci] + rd.chunk[kk]);
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) b[kk][tj] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[tj] + rd.chunk[kk]);
  }
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
        acc[ci][tj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[kk][ci], b[kk][tj], acc[ci][tj], 0, 0, 0);
  // all 12 operand reads first, then the 16 MFMAs (the waits in between become progressive)
  __builtin_amdgcn_sched_group_barrier(0x100, 12, 0);
  __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);
}

// Step s of the ring: wait for this wavefront's loads of step s (the 6 of step s+1 may stay in
// flight), barrier so that everybody's have landed and everybody is done reading the stage that is
// refilled next, issue step s+2, multiply step s.
__device__ __forceinline__ void ring_step(const TileLoads& ld, const TileReads& rd, char* cur, char* refill,
                                          int s, int nk, bool compute, v16i (&acc)[4][2]) {
  if (s + 1 < nk) wait_vmcnt<6>(); else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  if (s + 2 < nk) issue_stage_loads(ld, refill, (s + 2) * kBK);
  if (compute) multiply_stage(rd, cur, acc);
}

template <int MODE>
__device__ __forceinline__ void tile_pass(const TileParams& p, char* st0, char* st1, char* st2, int e, int nt,
                                          int64_t slot0, bool second_half) {
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int th = wave >> 1;   // token half of this wavefront
  const int chh = wave & 1;   // channel half
  const int K = p.K;
  const int inter = p.N / 2;  // gate_up only

  // ---- loads: lane fills LDS slot (lane & 3) of row 16 * (wave + 4 * i) + (lane >> 2), i.e. it
  //      fetches the logical chunk (lane & 3) ^ swizzle(row) of that row ----
  TileLoads ld;
  ld.wave = wave;
  const int lr = t >> 2;
  const int src_chunk = ((lane & 3) ^ swizzle_of_row(lane >> 2)) * 16;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = lr + 64 * i;
    int n;
    if constexpr (MODE == kGateUpSilu) {
      const int ch = nt * 128 + (row & 127);
      n = (ch < inter ? ch : inter - 1) + (row >= 128 ? inter : 0);
    } else {
      const int ch = nt * kBN + row;
      n = ch < p.N ? ch : p.N - 1;
    }
    ld.wsrc[i] = p.w + ((int64_t)e * p.N + n) * K + src_chunk;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = lr + 64 * i;
    int64_t arow = 0;
    if (i == 0 || second_half) {
      const int32_t tok = p.sorted_ids[slot0 + row];
      if (tok >= 0 && tok < p.P) arow = tok / p.row_div;
    }
    ld.xsrc[i] = p.a_q + arow * K + src_chunk;
  }

  // ---- MFMA operand reads: lane feeds row (lane & 31), 16-byte chunk 2 * kk + (lane >> 5) ----
  const int lrow = lane & 31;
  const int lsw = swizzle_of_row(lrow);
  const int lhalf = lane >> 5;
  TileReads rd;
#pragma unroll
  for (int ci = 0; ci < 4; ++ci) {
    int row0;
    if constexpr (MODE == kGateUpSilu)
      row0 = (ci < 2 ? 0 : 128) + chh * 64 + (ci & 1) * 32;
    else
      row0 = chh * 128 + ci * 32;
    rd.w_ld[ci] = (row0 + lrow) * kBK;
  }
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) rd.x_ld[tj] = kBN * kBK + (th * 64 + tj * 32 + lrow) * kBK;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) rd.chunk[kk] = ((2 * kk + lhalf) ^ lsw) * 16;
  const bool compute = th == 0 || second_half;

  v16i acc[4][2];
#pragma unroll
  for (int ci = 0; ci < 4; ++ci)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ci][tj][r] = 0;

  const int nk = K / kBK;
  // Everybody must be done with the stages (a previous pass) and this wavefront's earlier vector
  // memory operations must have drained before the counted waits below start.
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  issue_stage_loads(ld, st0, 0);
  if (nk > 1) issue_stage_loads(ld, st1, kBK);
  for (int s = 0; s < nk; s += 3) {
    ring_step(ld, rd, st0, st2, s, nk, compute, acc);
    if (s + 1 < nk) ring_step(ld, rd, st1, st0, s + 1, nk, compute, acc);
    if (s + 2 < nk) ring_step(ld, rd, st2, st1, s + 2, nk, compute, acc);
  }
  if (!compute) return;

  // ---- epilogue: acc[ci][tj][4q + r] is channel base(ci) + 8q + 4 * lhalf + r of token row
  //      th * 64 + tj * 32 + lrow ----
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    const int32_t tok = p.sorted_ids[slot0 + th * 64 + tj * 32 + lrow];
    if (tok < 0 || tok >= p.P) continue;
    if constexpr (MODE == kAccI32) {
      int32_t* out = static_cast<int32_t*>(p.out) + (int64_t)tok * p.N;
#pragma unroll
      for (int ci = 0; ci < 4; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = nt * kBN + chh * 128 + ci * 32 + 8 * q + 4 * lhalf;
          if (n < p.N)
            *reinterpret_cast<v4i*>(out + n) =
                v4i{acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
        }
    } else if constexpr (MODE == kDown) {
      uint16_t* out = static_cast<uint16_t*>(p.out) + (int64_t)tok * p.N;
      const float as = p.a_scale[tok / p.row_div];
      const float rw = p.row_weight[tok];
      const float* wsc = p.w_scale + (int64_t)e * p.N;
#pragma unroll
      for (int ci = 0; ci < 4; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = nt * kBN + chh * 128 + ci * 32 + 8 * q + 4 * lhalf;
          if (n >= p.N) continue;
          const float4 ws = *reinterpret_cast<const float4*>(wsc + n);
          const float wsv[4] = {ws.x, ws.y, ws.z, ws.w};
          uint32_t b[4];
#pragma unroll
          for (int r = 0; r < 4; ++r)
            b[r] = f32_to_bf16_bits((float)acc[ci][tj][4 * q + r] * as * wsv[r] * rw);
          *reinterpret_cast<uint2*>(out + n) = make_uint2(b[0] | (b[1] << 16), b[2] | (b[3] << 16));
        }
    } else {
      uint16_t* out = static_cast<uint16_t*>(p.out) + (int64_t)tok * inter;
      const float as = p.a_scale[tok / p.row_div];
      const float* wsc = p.w_scale + (int64_t)e * p.N;
#pragma unroll
      for (int ci = 0; ci < 2; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = nt * 128 + chh * 64 + ci * 32 + 8 * q + 4 * lhalf;  // gate channel
          if (n >= inter) continue;
          const float4 wg = *reinterpret_cast<const float4*>(wsc + n);
          const float4 wu = *reinterpret_cast<const float4*>(wsc + inter + n);
          const float wgv[4] = {wg.x, wg.y, wg.z, wg.w};
          const float wuv[4] = {wu.x, wu.y, wu.z, wu.w};
          uint32_t b[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = round_to_bf16((float)acc[ci][tj][4 * q + r] * as * wgv[r]);
            const float u = round_to_bf16((float)acc[ci + 2][tj][4 * q + r] * as * wuv[r]);
            b[r] = silu_mul_bf16_bits(g, u);
          }
          *reinterpret_cast<uint2*>(out + n) = make_uint2(b[0] | (b[1] << 16), b[2] | (b[3] << 16));
        }
    }
  }
}

template <int MODE>
__global__ __launch_bounds__(kThreads, 2) void gemm_tile_kernel(TileParams p) {
  __shared__ __align__(16) char st0[kStageBytes];
  __shared__ __align__(16) char st1[kStageBytes];
  __shared__ __align__(16) char st2[kStageBytes];
  const int npp = *p.npp;
  const int mtiles = (npp + kBM - 1) / kBM;
  const int total = mtiles * p.ntiles;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int local = blockIdx.x / kXcds;
  const int tile = (blockIdx.x % kXcds) * per_xcd + local;
  if (local >= per_xcd || tile >= total) return;
  const int nt = tile % p.ntiles;
  const int mt = tile / p.ntiles;
  const int64_t slot0 = (int64_t)mt * kBM;

  if (p.B == kBM) {
    const int e = p.expert_ids[mt];
    if (e >= 0 && e < p.E) tile_pass<MODE>(p, st0, st1, st2, e, nt, slot0, true);
    return;
  }
  // 64-row blocks: this tile covers blocks 2 * mt and 2 * mt + 1
  const int e0 = p.expert_ids[2 * mt];
  const bool have1 = slot0 + 64 < npp;
  const int e1 = have1 ? p.expert_ids[2 * mt + 1] : -1;
  if (e0 == e1) {
    if (e0 >= 0 && e0 < p.E) tile_pass<MODE>(p, st0, st1, st2, e0, nt, slot0, true);
    return;
  }
  if (e0 >= 0 && e0 < p.E) tile_pass<MODE>(p, st0, st1, st2, e0, nt, slot0, false);
  if (e1 >= 0 && e1 < p.E) tile_pass<MODE>(p, st0, st1, st2, e1, nt, slot0 + 64, false);
}

template <int MODE>
hipError_t launch_mode(const GemmArgs& a, hipStream_t stream) {
  TileParams p;
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
  p.ntiles = MODE == kGateUpSilu ? (a.n / 2 + 127) / 128 : (a.n + kBN - 1) / kBN;
  p.out = a.out;
  const int64_t mtiles = (a.sorted_cap + kBM - 1) / kBM;
  const int64_t total = mtiles * p.ntiles;
  if (total == 0) return hipSuccess;
  const int64_t per_xcd = (total + kXcds - 1) / kXcds;
  const int64_t grid = per_xcd * kXcds;
  if (grid > INT32_MAX) return hipErrorInvalidValue;
  hipLaunchKernelGGL(gemm_tile_kernel<MODE>, dim3((unsigned)grid), dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

bool gemm_tile_supports(const GemmArgs& a) {
  return (a.block_size == 64 || a.block_size == 128) && a.k % kBK == 0 && a.n % 16 == 0;
}

hipError_t launch_gemm_tile(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case kGateUpSilu: return launch_mode<kGateUpSilu>(a, stream);
    case kDown: return launch_mode<kDown>(a, stream);
    case kAccI32: return launch_mode<kAccI32>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe_i8
