// Grouped int8 GEMM for gfx950, LDS-tiled family (many rows per expert: prefill).
//
// Persistent workgroups (one per CU, 512 threads = 8 wavefronts) walk a list of tiles.  A tile is
// up to 256 token rows of ONE expert (up to four 64-row moe_align blocks, aligned to the start of
// the expert's segment) x 256 weight rows (output channels); the reduction runs in steps of 128
// bytes.  Wavefront w owns token sub-block w / 2 (64 rows) x channel half w % 2 (128 channels) as
// 2 x 4 v_mfma_i32_32x32x32_i8 tiles (128 accumulator VGPRs).  The MFMA is used "transposed"
// (A operand = weight rows, B operand = token rows), so a lane ends up with runs of 4 consecutive
// channels of one token.
//
// Both operands go global -> LDS directly (global_load_lds_dwordx4: no staging registers, no
// ds_write) into two 64 KB stages: while step s is multiplied the loads of step s+1 are in flight,
// with one s_barrier per step and explicit vmcnt waits.  Every wavefront-level load covers 8 rows
// x 128 contiguous bytes, i.e. whole cache lines.  LDS rows are 128 bytes; the 16-byte chunk index
// is XOR-swizzled with row bits so that the MFMA-layout reads (32 consecutive rows, same chunk)
// spread over all banks; because a load fills LDS linearly the swizzle is applied to the global
// source address of each lane.
//
// The tile list is derived inside the kernel from expert_ids (block -> expert, ascending): every
// workgroup scans it once into LDS.  Tasks (tile, channel tile) are numbered channel tile fastest
// and split into 8 contiguous ranges, one per XCD (workgroup id % 8), so that the workgroups
// running on one XCD at a time share token rows and expert weights in that XCD's L2.  The first
// loads of the next task are issued before the epilogue of the current one.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kTileTok = 256;  // token rows per tile
constexpr int kBN = 256;       // weight rows per tile
constexpr int kBK = 128;       // reduction bytes per step
constexpr int kTokOffset = kBN * kBK;
constexpr int kStageBytes = (kBN + kTileTok) * kBK;  // 64 KB
constexpr int kMaxTiles = 6144;                      // capacity of the in-LDS tile list
constexpr int kXcds = 8;
constexpr int kGroupTiles = 8;  // token tiles of one expert whose tasks are interleaved per channel tile

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

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = bits 3:0 and
// 15:14; expcnt 6:4 and lgkmcnt 11:8 left at their maximum).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// 16 bytes per lane from global memory straight into LDS: lane i lands at lds_addr + 16 * i
// (lds_addr is wave-uniform and goes through M0).  Issued as inline assembly so that the waits are
// the explicit vmcnt waits of the ring below and not a conservative vmcnt(0) before every LDS read.
// The source is a wave-uniform base (SGPR pair) plus an unsigned 32-bit byte offset per lane.
__device__ __forceinline__ void load_to_lds_16(const int8_t* base, uint32_t offset, uint32_t lds_addr) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  // readfirstlane yields a signed int: go through uint32_t so that the low half is not sign-extended
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  const uint64_t ub = (uint64_t)lo | ((uint64_t)hi << 32);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"((uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(offset), "s"(ub)
               : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) char*)p);
}

__device__ __forceinline__ int swizzle_of_row(int r) { return (r & 7) ^ ((r >> 3) & 1); }

// ---- block-wide scans over kThreads threads (used once per workgroup, for the tile list) ----
template <bool kMax>
__device__ __forceinline__ int scan_op(int a, int b) {
  return kMax ? (a > b ? a : b) : a + b;
}

template <bool kMax>
__device__ __forceinline__ void block_scan(int v, int* wave_part, int& incl, int& excl) {
  const int ident = kMax ? -1 : 0;
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  int x = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int n = __shfl_up(x, d);
    if (lane >= d) x = scan_op<kMax>(n, x);
  }
  int prev = __shfl_up(x, 1);
  if (lane == 0) prev = ident;
  if (lane == kWave - 1) wave_part[wave] = x;
  __syncthreads();
  int carry = ident;
  for (int i = 0; i < wave; ++i) carry = scan_op<kMax>(carry, wave_part[i]);
  __syncthreads();
  incl = scan_op<kMax>(carry, x);
  excl = scan_op<kMax>(carry, prev);
}

// tile_desc[t] = first block | number of blocks << 16 | rank in group << 20 | group size << 24.
// Tiles start at multiples of `per_tile` blocks inside each run of equal expert ids and never cross
// a run; up to kGroupTiles consecutive tiles of a run form a group.  scratch holds nblocks ints.
__device__ int build_tile_list(const int32_t* __restrict__ expert_ids, int nblocks, int per_tile, int* scratch,
                               int* wave_part, uint32_t* tile_desc, int* total_out) {
  const int tid = threadIdx.x;
  for (int j = tid; j < nblocks; j += kThreads) scratch[j] = expert_ids[j];
  __syncthreads();
  const int chunk = (nblocks + kThreads - 1) / kThreads;
  const int j0 = tid * chunk < nblocks ? tid * chunk : nblocks;
  const int j1 = j0 + chunk < nblocks ? j0 + chunk : nblocks;
  // start of the run that contains block j = prefix max of (j if a run starts at j else -1)
  int local_start = -1;
  for (int j = j0; j < j1; ++j)
    if (j == 0 || scratch[j] != scratch[j - 1]) local_start = j;
  int incl, carry_start;
  block_scan<true>(local_start, wave_part, incl, carry_start);
  int leaders = 0;
  int cur = carry_start;
  for (int j = j0; j < j1; ++j) {
    if (j == 0 || scratch[j] != scratch[j - 1]) cur = j;
    if ((j - cur) % per_tile == 0) ++leaders;
  }
  int incl_leaders, t;
  block_scan<false>(leaders, wave_part, incl_leaders, t);
  cur = carry_start;
  for (int j = j0; j < j1; ++j) {
    if (j == 0 || scratch[j] != scratch[j - 1]) cur = j;
    if ((j - cur) % per_tile == 0) {
      int nb = 1;
      while (nb < per_tile && j + nb < nblocks && scratch[j + nb] == scratch[j]) ++nb;
      // bits 0-15 first block, 16-19 blocks, 20-22 rank of the tile inside its group, 24-27 group size
      if (t < kMaxTiles)
        tile_desc[t] = (uint32_t)j | ((uint32_t)nb << 16) | ((uint32_t)(((j - cur) / per_tile) % kGroupTiles) << 20);
      ++t;
    }
  }
  if (tid == kThreads - 1) *total_out = incl_leaders < kMaxTiles ? incl_leaders : kMaxTiles;
  __syncthreads();
  // Groups: up to kGroupTiles consecutive tiles of one expert.  The leader of a group counts its
  // members and writes the size into all of them.
  const int total = *total_out;
  for (int g = tid; g < total; g += kThreads) {
    if (((tile_desc[g] >> 20) & 7u) != 0) continue;
    int count = 1;
    while (count < kGroupTiles && g + count < total && ((tile_desc[g + count] >> 20) & 7u) == (uint32_t)count) ++count;
    for (int i = 0; i < count; ++i) tile_desc[g + i] |= (uint32_t)count << 24;
  }
  __syncthreads();
  return total;
}

struct Task {
  int e;          // expert; -1 = no more work, -2 = tile of ignored expert ids
  int nt;         // channel tile
  int64_t slot0;  // first slot of the tile in sorted_ids
  int nsub;       // active 64-row sub-blocks (1..4)
};

struct TaskLoads {
  const int8_t* wbase;  // weights of the task's expert (wave-uniform)
  uint32_t woff[4];     // per lane: byte offset of its chunk of weight row i from wbase
  uint32_t xoff[4];     // per lane: byte offset of its chunk of token row i from a_q
};

// Lane fills LDS slot (lane & 7) of row 32 * wave + 8 * i + (lane >> 3): it fetches the logical
// chunk (lane & 7) ^ swizzle(row) of that row, and swizzle(row) = (lane >> 3) ^ (i & 1).
template <int MODE>
__device__ __forceinline__ void setup_loads(const TileParams& p, const Task& tk, int wave, int lane, TaskLoads& ld) {
  const int K = p.K;
  const int inter = p.N / 2;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 32 * wave + 8 * i + (lane >> 3);
    const int chunk = ((lane & 7) ^ (lane >> 3) ^ (i & 1)) * 16;
    int n;
    if constexpr (MODE == kGateUpSilu) {
      const int ch = tk.nt * 128 + (row & 127);
      n = (ch < inter ? ch : inter - 1) + (row >= 128 ? inter : 0);
    } else {
      const int ch = tk.nt * kBN + row;
      n = ch < p.N ? ch : p.N - 1;
    }
    ld.woff[i] = (uint32_t)n * (uint32_t)K + chunk;
    uint32_t arow = 0;
    if ((wave >> 1) < tk.nsub) {
      const int32_t tok = p.sorted_ids[tk.slot0 + row];
      if (tok >= 0 && tok < p.P) arow = (uint32_t)(tok / p.row_div);
    }
    ld.xoff[i] = arow * (uint32_t)K + chunk;
  }
  ld.wbase = p.w + (int64_t)tk.e * p.N * K;
}

__device__ __forceinline__ void issue_stage_loads(const TaskLoads& ld, const int8_t* a_q, uint32_t stage_addr,
                                                  int wave, int koff, bool tokens) {
#pragma unroll
  for (int i = 0; i < 4; ++i) load_to_lds_16(ld.wbase + koff, ld.woff[i], stage_addr + (wave * 4 + i) * 1024);
  if (tokens) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      load_to_lds_16(a_q + koff, ld.xoff[i], stage_addr + kTokOffset + (wave * 4 + i) * 1024);
  }
}

struct TileReads {
  int w_ld[4];
  int x_ld[2];
  int chunk[4];  // swizzled byte offset of logical chunk 2 * kk + (lane >> 5)
};

__device__ __forceinline__ void multiply_stage(const TileReads& rd, const char* stage, v16i (&acc)[4][2]) {
  v4i a[4][4], b[4][2];
  // reads in the order the MFMAs consume them: b0 a0 | b1 | a1 | a2 | a3 per 32-byte sub-step
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    b[kk][0] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[0] + rd.chunk[kk]);
    a[kk][0] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[0] + rd.chunk[kk]);
    b[kk][1] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[1] + rd.chunk[kk]);
#pragma unroll
    for (int ci = 1; ci < 4; ++ci) a[kk][ci] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[ci] + rd.chunk[kk]);
  }
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
        acc[ci][tj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[kk][ci], b[kk][tj], acc[ci][tj], 0, 0, 0);
  // Fine interleave, one group ahead: the first MFMA issues as soon as three operands are in and
  // every later read is issued at least one MFMA group before its first use, so it is hidden
  // behind MFMAs already queued (8 wavefronts share the LDS: a long burst of reads in front of the
  // first MFMA would leave the matrix pipe idle at the start of every step).
  __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);  // b0 a0 b1 of sub-step 0
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // a0 b0
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a1
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // a0 b1
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a2
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // a1
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a3
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // a2
    if (kk < 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // next b0 a0
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // a3
    if (kk < 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // next b1
  }
}

// acc[ci][tj][4q + r] is channel base(ci) + 8q + 4 * (lane >> 5) + r of token row
// tb * 64 + tj * 32 + (lane & 31) of the tile.  The bf16 results are transposed through an 8 KB
// LDS region private to the wavefront so that the global stores are 16 bytes per lane and cover
// whole cache lines of an output row (rows of 16-byte chunks, chunk index XOR-swizzled with the row
// so that neither the 8-byte writes nor the 16-byte reads pile up on a bank).
template <int MODE>
__device__ __forceinline__ void epilogue(const TileParams& p, const Task& tk, int chh, int tb, int lane,
                                         v16i (&acc)[4][2], char* wave_lds, float* wave_scales) {
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  const int inter = p.N / 2;
  int32_t tok[2];
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    tok[tj] = p.sorted_ids[tk.slot0 + tb * 64 + tj * 32 + lrow];
    if (tok[tj] < 0 || tok[tj] >= p.P) tok[tj] = -1;
  }
  if constexpr (MODE == kAccI32) {
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      if (tok[tj] < 0) continue;
      int32_t* out = static_cast<int32_t*>(p.out) + (int64_t)tok[tj] * p.N;
#pragma unroll
      for (int ci = 0; ci < 4; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = tk.nt * kBN + chh * 128 + ci * 32 + 8 * q + 4 * lhalf;
          if (n < p.N)
            *reinterpret_cast<v4i*>(out + n) =
                v4i{acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
        }
    }
  } else if constexpr (MODE == kDown) {
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * kBN + chh * 128;  // first channel of this wavefront
    // The 128 channel scales of this wavefront go through LDS: read from there they do not count
    // as vector-memory loads, so the second half's arithmetic does not have to wait for the first
    // half's stores (the vector-memory counter retires in order).
    {
      const int n = n0 + 2 * lane;
      *reinterpret_cast<float2*>(wave_scales + 2 * lane) =
          n < p.N ? *reinterpret_cast<const float2*>(wsc + n) : make_float2(0.0f, 0.0f);
    }
    float as[2], rw[2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      as[tj] = tok[tj] >= 0 ? p.a_scale[tok[tj] / p.row_div] : 0.0f;
      rw[tj] = tok[tj] >= 0 ? (p.row_weight ? p.row_weight[tok[tj]] : 1.0f) : 0.0f;
    }
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      // 32 token rows x 128 channels: rows of 256 bytes = 16 chunks
#pragma unroll
      for (int ci = 0; ci < 4; ++ci) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 ws = *reinterpret_cast<const float4*>(wave_scales + ci * 32 + 8 * q + 4 * lhalf);
          const int v[4] = {acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
          *reinterpret_cast<uint2*>(wave_lds + lrow * 256 + (((ci * 4 + q) ^ (lrow & 15)) * 16) + lhalf * 8) =
              down_epilogue4(v, as[tj], ws, rw[tj]);
        }
      }
      // Before the first stores everything this wavefront has in flight is complete (its share of
      // the next tile's first stage, issued during the last step, and the loads above), so the
      // stores are the only vector-memory work still pending when the next tile starts.
      if (tj == 0) wait_vmcnt<0>();
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int row = r * 4 + (lane >> 4);
        const int chunk = lane & 15;
        const uint4 v = *reinterpret_cast<const uint4*>(wave_lds + row * 256 + ((chunk ^ (row & 15)) * 16));
        const int32_t t = __shfl(tok[tj], row);
        const int n = n0 + chunk * 8;
        if (t >= 0 && n < p.N)
          __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * p.N + n));
      }
    }
  } else {
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * 128 + chh * 64;  // first gate channel of this wavefront
    // 64 token rows x 64 channels: rows of 128 bytes = 8 chunks
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const float as = tok[tj] >= 0 ? p.a_scale[tok[tj] / p.row_div] : 0.0f;
      const int row = tj * 32 + lrow;
#pragma unroll
      for (int ci = 0; ci < 2; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + ci * 32 + 8 * q + 4 * lhalf;
          const int ns = n < inter ? n : 0;
          const float4 wg = *reinterpret_cast<const float4*>(wsc + ns);
          const float4 wu = *reinterpret_cast<const float4*>(wsc + inter + ns);
          const int g[4] = {acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
          const int u[4] = {acc[ci + 2][tj][4 * q], acc[ci + 2][tj][4 * q + 1], acc[ci + 2][tj][4 * q + 2],
                            acc[ci + 2][tj][4 * q + 3]};
          *reinterpret_cast<uint2*>(wave_lds + row * 128 + (((ci * 4 + q) ^ (row & 7)) * 16) + lhalf * 8) =
              silu_mul_epilogue4(g, u, as, wg, wu);
        }
    }
    wait_vmcnt<0>();  // as in the down epilogue: only the stores below stay pending
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int row = r * 8 + (lane >> 3);
      const int chunk = lane & 7;
      const uint4 v = *reinterpret_cast<const uint4*>(wave_lds + row * 128 + ((chunk ^ (row & 7)) * 16));
      const int32_t t = __shfl(tok[r >> 2], row & 31);
      const int n = n0 + chunk * 8;
      if (t >= 0 && n < inter)
        __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * inter + n));
    }
  }
}

template <int MODE>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_kernel(TileParams p) {
  __shared__ __align__(16) char stages[2 * kStageBytes];
  __shared__ uint32_t tile_desc[kMaxTiles];
  __shared__ int wave_part[kWaves];
  __shared__ __align__(16) float channel_scales[kWaves * 128];
  __shared__ int total_tiles;

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int tb = wave >> 1;  // token sub-block of this wavefront
  const int chh = wave & 1;  // channel half
  const int nk = p.K / kBK;

  const int npp = *p.npp;
  const int nblocks = npp / p.B;
  const int sub_per_block = p.B / 64;
  const int ntile = build_tile_list(p.expert_ids, nblocks, kTileTok / p.B, reinterpret_cast<int*>(stages), wave_part,
                                    tile_desc, &total_tiles);
  const int total = ntile * p.ntiles;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int stride = gridDim.x / kXcds;

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
  for (int tj = 0; tj < 2; ++tj) rd.x_ld[tj] = kTokOffset + (tb * 64 + tj * 32 + lrow) * kBK;
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd.chunk[kk] = ((2 * kk + lhalf) ^ lsw) * 16;

  const uint32_t stage0 = lds_address(stages);

  auto decode = [&](int it) {
    Task tk;
    tk.e = -1;
    tk.nt = 0;
    tk.slot0 = 0;
    tk.nsub = 0;
    if (it < per_xcd && xcd * per_xcd + it < total) {
      const int task = xcd * per_xcd + it;
      // The tasks of a group of T token tiles of one expert run channel tile by channel tile: T
      // consecutive tasks (on neighbouring compute units) stream the same weight tile.
      const int tile0 = task / p.ntiles;
      const uint32_t d0 = tile_desc[tile0];
      const int first = tile0 - (int)((d0 >> 20) & 7u);
      const int T = (int)((d0 >> 24) & 15u);
      const int pos = task - first * p.ntiles;
      const uint32_t d = tile_desc[first + pos % T];
      tk.nt = pos / T;
      const int blk = (int)(d & 0xffffu);
      const int e = p.expert_ids[blk];
      tk.slot0 = (int64_t)blk * p.B;
      tk.nsub = (int)((d >> 16) & 15u) * sub_per_block;
      tk.e = (e >= 0 && e < p.E) ? e : -2;
    }
    return tk;
  };

  int it = blockIdx.x / kXcds;
  Task tk = decode(it);
  while (tk.e == -2) tk = decode(it += stride);
  if (tk.e < 0) return;
  TaskLoads ld;
  setup_loads<MODE>(p, tk, wave, lane, ld);
  bool my_tokens = tb < tk.nsub;
  int parity = 0;
  // The scratch of the tile list lived in the stage memory; everybody is past it (the builder ends
  // with a barrier), so the first stage can be filled now.
  issue_stage_loads(ld, p.a_q, stage0, wave, 0, my_tokens);

  bool stores_pending = false;
  while (true) {
    v16i acc[4][2];
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ci][tj][r] = 0;

    // look ahead: the first loads of the next task are issued during the last step of this one
    int nit = it + stride;
    Task nx = decode(nit);
    while (nx.e == -2) nx = decode(nit += stride);
    TaskLoads nld = ld;
    if (nx.e >= 0) setup_loads<MODE>(p, nx, wave, lane, nld);
    const bool nx_tokens = tb < nx.nsub;

    for (int s = 0; s < nk; ++s) {
      // this wavefront's loads of step s have landed (nothing newer is in flight) ...  A wavefront
      // that has just run an epilogue waited for its loads there and only has the epilogue's
      // stores pending: it lets them drain behind the first step instead of stalling on them.
      if (s > 0 || !stores_pending) wait_vmcnt<0>();
      // ... and so have everybody's; everybody is also done reading the other stage
      __builtin_amdgcn_s_barrier();
      const uint32_t other = stage0 + (parity ^ 1) * kStageBytes;
      if (s + 1 < nk)
        issue_stage_loads(ld, p.a_q, other, wave, (s + 1) * kBK, my_tokens);
      else if (nx.e >= 0)
        issue_stage_loads(nld, p.a_q, other, wave, 0, nx_tokens);
      if (my_tokens) multiply_stage(rd, stages + parity * kStageBytes, acc);
      parity ^= 1;
    }
    // everybody is done reading the stage of the last step: it becomes the epilogue's staging area
    // (the next task's first loads went to the other stage)
    __builtin_amdgcn_s_barrier();
    if (my_tokens)
      epilogue<MODE>(p, tk, chh, tb, lane, acc, stages + (parity ^ 1) * kStageBytes + wave * 8192,
                     channel_scales + wave * 128);
    stores_pending = my_tokens && MODE != kAccI32;
    if (nx.e < 0) break;
    tk = nx;
    ld = nld;
    my_tokens = nx_tokens;
    it = nit;
  }
  wait_vmcnt<0>();
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
  const int grid = device_cu_count() / kXcds * kXcds;
  hipLaunchKernelGGL(gemm_tile_kernel<MODE>, dim3((unsigned)grid), dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

bool gemm_tile_supports(const GemmArgs& a) {
  // per-lane source offsets are 32-bit: one expert's weights and the activation matrix must each
  // span less than 4 GiB
  const int64_t act_rows = (a.num_pairs + a.row_div - 1) / a.row_div;
  if (!((a.block_size == 64 || a.block_size == 128) && a.k % kBK == 0 && a.k >= 2 * kBK && a.n % 16 == 0 &&
        (int64_t)a.n * a.k < (1ll << 32) && act_rows * a.k < (1ll << 32)))
    return false;
  // The tile list lives in LDS.  A run of equal expert ids of L blocks makes ceil(L / blocks per
  // tile) tiles; moe_align's ids ascend, so there is one run per expert.  Ids of unknown order could
  // make every block a tile of its own.  While the list is built the block ids sit in the stages.
  const int64_t blocks = (a.sorted_cap + a.block_size - 1) / a.block_size;
  const int per_tile = kTileTok / a.block_size;
  const int64_t tiles = a.expert_ids_ascend ? (blocks + per_tile - 1) / per_tile + a.num_experts : blocks;
  return tiles <= kMaxTiles && blocks <= (int64_t)(2 * kStageBytes / sizeof(int)) && blocks <= 65535;
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
