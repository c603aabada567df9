// Grouped int8 GEMM for gfx950, LDS-tiled family (prefill: from a few dozen routed rows per expert up).
//
// Persistent workgroups (one per CU, 512 threads = 8 wavefronts) walk a list of tiles.  A tile is
// a run of 64-row moe_align sub-blocks of ONE expert (aligned to the start of the expert's segment)
// x 256 weight rows (output channels); the reduction runs in steps of 128 bytes.  The MFMA
// (v_mfma_i32_32x32x32_i8) is used "transposed" (A operand = weight rows, B operand = token rows),
// so a lane ends up with runs of 4 consecutive channels of one token.
//
// Two geometries (template parameter DEEP):
//  * wide: up to 256 token rows per tile, two 64 KB LDS stages, loads one step ahead.  Wavefront w
//    owns token sub-block w / 2 x channel half w % 2 as 4 x 2 MFMA tiles (128 accumulator VGPRs).
//    Bound by the matrix pipe; a weight tile is reused by up to four sub-blocks.
//  * deep: up to 128 token rows per tile, a ring of three 48 KB stages, loads two steps ahead.  With
//    few rows per expert a step holds little arithmetic and the kernel is bound by the weight stream
//    from HBM, i.e. by the bytes a compute unit keeps in flight.  All eight wavefronts multiply in
//    every task: with two active sub-blocks wavefront w owns sub-block w / 4 and a quarter of the
//    channels, with one an eighth of the channels.
//
// Both operands go global -> LDS directly (global_load_lds_dwordx4: no staging registers, no
// ds_write), with one s_barrier per step and explicit vmcnt waits.  Every wavefront-level load
// covers 8 rows x 128 contiguous bytes, i.e. whole cache lines.  LDS rows are 128 bytes; the 16-byte
// chunk index is XOR-swizzled with row bits so that the MFMA-layout reads (32 consecutive rows, same
// chunk) spread over all banks; because a load fills LDS linearly the swizzle is applied to the
// global source address of each lane.
//
// The tile list is derived inside the kernel from expert_ids (block -> expert, ascending): every
// workgroup scans it once into LDS.  Tasks (tile, channel tile) are numbered channel tile fastest
// and split into 8 contiguous ranges, one per XCD (workgroup id % 8), so that the workgroups
// running on one XCD at a time share token rows and expert weights in that XCD's L2.  The first
// loads of the next task are issued before the epilogue of the current one.
#include <type_traits>

#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kBN = 256;       // weight rows per tile
constexpr int kBK = 128;       // reduction bytes per step
constexpr int kTokOffset = kBN * kBK;

// Two geometries.  Wide: tiles of up to 256 token rows, two 64 KB stages (loads one step ahead).
// Deep: tiles of up to 128 token rows, a ring of three 48 KB stages (loads two steps ahead): with
// few rows per expert a step holds little arithmetic, and what bounds the kernel is how many bytes
// of the weight stream a compute unit keeps in flight.
template <bool DEEP>
struct Geometry {
  static constexpr int kTileTok = DEEP ? 128 : 256;               // token rows per tile
  static constexpr int kSlots = DEEP ? 3 : 2;                     // LDS stages
  static constexpr int kStageBytes = (kBN + kTileTok) * kBK;      // 48 KB | 64 KB
  static constexpr int kMaxTiles = DEEP ? 2048 : 6144;            // capacity of the in-LDS tile list
  static constexpr int kTokLoads = kTileTok / 64;                 // wave-level loads of 8 token rows per wavefront and step
};
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
  int ascend;  // expert_ids is known to ascend over the used blocks (it comes from moe_align)
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

// The same with the non-temporal hint: for launches in which no expert holds more rows than one
// tile, so that every weight row is read by exactly one workgroup.  Streamed that way the weights
// do not displace the token rows from L2 (measured: 5-8 % on launches bound by the weight stream;
// a loss as soon as a second tile of an expert would have found the rows in L2).
__device__ __forceinline__ void load_to_lds_16_stream(const int8_t* base, uint32_t offset, uint32_t lds_addr) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  const uint64_t ub = (uint64_t)lo | ((uint64_t)hi << 32);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
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
                               int* wave_part, uint32_t* tile_desc, int* total_out, int max_tiles) {
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
      if (t < max_tiles)
        tile_desc[t] = (uint32_t)j | ((uint32_t)nb << 16) | ((uint32_t)(((j - cur) / per_tile) % kGroupTiles) << 20);
      ++t;
    }
  }
  if (tid == kThreads - 1) *total_out = incl_leaders < max_tiles ? incl_leaders : max_tiles;
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

// The same list when the expert ids are known to ascend over the used blocks (what moe_align writes):
// every expert then owns at most one run of blocks, found by comparing a block with its neighbours, and
// the number of tiles in front of an expert is one scan over the experts instead of two over the blocks
// (a third of the time on a long list).  Runs of ids outside [0, E) get no tiles.  scratch holds
// 2 * num_experts ints; per_tile is 1 << per_tile_log2.
__device__ int build_tile_list_ascending(const int32_t* __restrict__ expert_ids, int nblocks, int num_experts,
                                         int per_tile_log2, int* scratch, int* wave_part, uint32_t* tile_desc,
                                         int* total_out, int max_tiles) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  int* first = scratch;               // first block of the expert's run
  int* end = scratch + num_experts;   // one past its last block
  for (int e = tid; e < 2 * num_experts; e += kThreads) scratch[e] = 0;
  __syncthreads();
  for (int j = tid; j < nblocks; j += kThreads) {
    const int e = expert_ids[j];
    const int prev = j > 0 ? expert_ids[j - 1] : -1;
    const int next = j + 1 < nblocks ? expert_ids[j + 1] : -1;
    if (e >= 0 && e < num_experts) {
      if (j == 0 || e != prev) first[e] = j;
      if (j + 1 == nblocks || e != next) end[e] = j + 1;
    }
  }
  __syncthreads();
  // thread t owns experts 2t and 2t + 1 (num_experts <= 2 * kThreads)
  const int per_tile = 1 << per_tile_log2;
  int f[2], nb[2], tiles[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = 2 * tid + i;
    f[i] = e < num_experts ? first[e] : 0;
    nb[i] = e < num_experts ? end[e] - f[i] : 0;
    tiles[i] = (nb[i] + per_tile - 1) >> per_tile_log2;
  }
  const int mine = tiles[0] + tiles[1];
  const int incl = wave_inclusive_scan_add(mine);
  if (lane == kWave - 1) wave_part[wave] = incl;
  __syncthreads();
  int carry = 0, total = 0;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) {
    const int w = wave_part[i];
    if (i < wave) carry += w;
    total += w;
  }
  int t = carry + incl - mine;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    for (int r = 0; r < tiles[i]; ++r, ++t) {
      if (t >= max_tiles) break;
      const int left = nb[i] - (r << per_tile_log2);
      const int in_group = tiles[i] - (r & ~(kGroupTiles - 1));
      tile_desc[t] = (uint32_t)(f[i] + (r << per_tile_log2)) | ((uint32_t)(left < per_tile ? left : per_tile) << 16) |
                     ((uint32_t)(r & (kGroupTiles - 1)) << 20) |
                     ((uint32_t)(in_group < kGroupTiles ? in_group : kGroupTiles) << 24);
    }
  }
  if (tid == 0) *total_out = total < max_tiles ? total : max_tiles;
  __syncthreads();
  return total < max_tiles ? total : max_tiles;
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

// Weights: lane fills LDS slot (lane & 7) of row 32 * wave + 8 * i + (lane >> 3): it fetches the logical
// chunk (lane & 7) ^ swizzle(row) of that row, and swizzle(row) = (lane >> 3) ^ (i & 1).  Token rows
// likewise, of row (8 * kTokLoads) * wave + 8 * i + (lane >> 3).
template <int MODE, bool DEEP>
__device__ __forceinline__ void setup_loads(const TileParams& p, const Task& tk, int wave, int lane, TaskLoads& ld) {
  constexpr int kTokLoads = Geometry<DEEP>::kTokLoads;
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
    if (i < kTokLoads) {
      const int trow = 8 * kTokLoads * wave + 8 * i + (lane >> 3);
      uint32_t arow = 0;
      if ((trow >> 6) < tk.nsub) {
        const int32_t tok = p.sorted_ids[tk.slot0 + trow];
        if (tok >= 0 && tok < p.P) arow = (uint32_t)(tok / p.row_div);
      }
      ld.xoff[i] = arow * (uint32_t)K + chunk;
    }
  }
  ld.wbase = p.w + (int64_t)tk.e * p.N * K;
}

// `tokens`: this wavefront's token rows belong to an active sub-block.  The deep geometry issues the
// token loads regardless (rows of inactive sub-blocks fetch row 0), so that every wavefront has the
// same number of loads in flight per step and the counted waits of the ring hold for all of them.
template <bool DEEP, bool NT>
__device__ __forceinline__ void issue_stage_loads(const TaskLoads& ld, const int8_t* a_q, uint32_t stage_addr,
                                                  int wave, int koff, bool tokens) {
  constexpr int kTokLoads = Geometry<DEEP>::kTokLoads;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (NT)
      load_to_lds_16_stream(ld.wbase + koff, ld.woff[i], stage_addr + (wave * 4 + i) * 1024);
    else
      load_to_lds_16(ld.wbase + koff, ld.woff[i], stage_addr + (wave * 4 + i) * 1024);
  }
  if (DEEP || tokens) {
#pragma unroll
    for (int i = 0; i < kTokLoads; ++i)
      load_to_lds_16(a_q + koff, ld.xoff[i], stage_addr + kTokOffset + (wave * kTokLoads + i) * 1024);
  }
}

struct TileReads {
  int w_ld[4];
  int x_ld[2];
  int chunk[4];  // swizzled byte offset of logical chunk 2 * kk + (lane >> 5)
};

// How the eight wavefronts share a task.  A task with NCI = 4 has three or four active 64-row
// sub-blocks: wavefront w owns sub-block w / 2 and half of the channels (4 MFMA tiles of 32 weight
// rows, twice 32 token rows).  With two active sub-blocks (NCI = 2) it owns sub-block w / 4 and a
// quarter of the channels, with one (NCI = 1) an eighth of the channels: every wavefront multiplies
// in every task, so a tile with few rows costs its loads and not the serial MFMA chain of the one
// or two wavefronts its rows would otherwise belong to.
template <int MODE, int NCI>
__device__ __forceinline__ void make_reads(int wave, int lane, TileReads& rd) {
  constexpr int kParts = 8 / NCI;
  const int tg = wave / kParts;
  const int cpart = wave % kParts;
  const int lrow = lane & 31;
#pragma unroll
  for (int ci = 0; ci < NCI; ++ci) {
    int row;
    if constexpr (MODE == kGateUpSilu) {
      // LDS rows 0..127 hold gate channels, 128..255 the matching up channels
      if constexpr (NCI == 4)
        row = (ci < 2 ? 0 : 128) + cpart * 64 + (ci & 1) * 32 + lrow;
      else if constexpr (NCI == 2)
        row = ci * 128 + cpart * 32 + lrow;
      else
        row = (lrow < 16 ? 0 : 128 - 16) + cpart * 16 + lrow;  // 16 gate rows, then their 16 up rows
    } else {
      row = cpart * (NCI * 32) + ci * 32 + lrow;
    }
    rd.w_ld[ci] = row * kBK;
  }
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) rd.x_ld[tj] = kTokOffset + (tg * 64 + tj * 32 + lrow) * kBK;
}

template <int NCI>
__device__ __forceinline__ void multiply_stage(const TileReads& rd, const char* stage, v16i (&acc)[NCI][2]) {
  v4i a[4][NCI], b[4][2];
  // reads in the order the MFMAs consume them: b0 a0 | b1 | a1 | a2 | a3 per 32-byte sub-step
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    b[kk][0] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[0] + rd.chunk[kk]);
    a[kk][0] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[0] + rd.chunk[kk]);
    b[kk][1] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[1] + rd.chunk[kk]);
#pragma unroll
    for (int ci = 1; ci < NCI; ++ci) a[kk][ci] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[ci] + rd.chunk[kk]);
  }
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
#pragma unroll
    for (int ci = 0; ci < NCI; ++ci)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
        acc[ci][tj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[kk][ci], b[kk][tj], acc[ci][tj], 0, 0, 0);
  if constexpr (NCI == 4) {
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
}

// acc[ci][tj][4q + r] is weight row 32 * ci + 8q + 4 * (lane >> 5) + r of the wavefront's MFMA tiles
// and token row tg * 64 + tj * 32 + (lane & 31) of the tile.  The bf16 results are transposed through
// an LDS region private to the wavefront (at most 8 KB) so that the global stores are 16 bytes per
// lane and cover whole runs of an output row (rows of 16-byte chunks, chunk index XOR-swizzled with
// the row so that neither the 8-byte writes nor the 16-byte reads pile up on a bank).
template <int CPR>
__device__ __forceinline__ int staging_swizzle(int row) {
  // rows of CPR chunks: 16 / CPR rows span all banks, rows that far apart must differ in the swizzle
  if constexpr (CPR >= 8)
    return row & (CPR - 1);
  else if constexpr (CPR == 4)
    return (row >> 2) & 3;
  else
    return (row >> 3) & 1;
}

template <int MODE, int NCI>
__device__ __forceinline__ void epilogue(const TileParams& p, const Task& tk, int wave, int lane, v16i (&acc)[NCI][2],
                                         char* wave_lds, float* wave_scales) {
  constexpr int kParts = 8 / NCI;
  const int tg = wave / kParts;
  const int cpart = wave % kParts;
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  const int inter = p.N / 2;
  int32_t tok[2];
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    tok[tj] = p.sorted_ids[tk.slot0 + tg * 64 + tj * 32 + lrow];
    if (tok[tj] < 0 || tok[tj] >= p.P) tok[tj] = -1;
  }
  if constexpr (MODE == kAccI32) {
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      if (tok[tj] < 0) continue;
      int32_t* out = static_cast<int32_t*>(p.out) + (int64_t)tok[tj] * p.N;
#pragma unroll
      for (int ci = 0; ci < NCI; ++ci)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = tk.nt * kBN + cpart * (NCI * 32) + ci * 32 + 8 * q + 4 * lhalf;
          if (n < p.N)
            *reinterpret_cast<v4i*>(out + n) =
                v4i{acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
        }
    }
  } else if constexpr (MODE == kDown) {
    constexpr int kChannels = NCI * 32;  // of this wavefront
    constexpr int CPR = NCI * 4;         // 16-byte chunks per staged row
    constexpr int kRowBytes = CPR * 16;
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * kBN + cpart * kChannels;  // first channel of this wavefront
    // The channel scales of this wavefront go through LDS: read from there they do not count
    // as vector-memory loads, so the second half's arithmetic does not have to wait for the first
    // half's stores (the vector-memory counter retires in order).
    if (2 * lane < kChannels) {
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
      // 32 token rows x kChannels channels
#pragma unroll
      for (int ci = 0; ci < NCI; ++ci) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 ws = *reinterpret_cast<const float4*>(wave_scales + ci * 32 + 8 * q + 4 * lhalf);
          const int v[4] = {acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
          *reinterpret_cast<uint2*>(wave_lds + lrow * kRowBytes + (((ci * 4 + q) ^ staging_swizzle<CPR>(lrow)) * 16) +
                                    lhalf * 8) = down_epilogue4(v, as[tj], ws, rw[tj]);
        }
      }
      // Before the first stores everything this wavefront has in flight is complete (its share of
      // the next tile's first stage, issued during the last step, and the loads above), so the
      // stores are the only vector-memory work still pending when the next tile starts.
      if (tj == 0) wait_vmcnt<0>();
#pragma unroll
      for (int r = 0; r < CPR / 2; ++r) {
        const int row = r * (64 / CPR) + lane / CPR;
        const int chunk = lane % CPR;
        const uint4 v =
            *reinterpret_cast<const uint4*>(wave_lds + row * kRowBytes + ((chunk ^ staging_swizzle<CPR>(row)) * 16));
        const int32_t t = __shfl(tok[tj], row);
        const int n = n0 + chunk * 8;
        if (t >= 0 && n < p.N)
          __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * p.N + n));
      }
    }
  } else {
    constexpr int kChannels = NCI * 16;  // activation channels of this wavefront
    constexpr int CPR = NCI * 2;
    constexpr int kRowBytes = CPR * 16;
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * 128 + cpart * kChannels;  // first gate channel of this wavefront
    // 64 token rows x kChannels channels
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const float as = tok[tj] >= 0 ? p.a_scale[tok[tj] / p.row_div] : 0.0f;
      const int row = tj * 32 + lrow;
#pragma unroll
      for (int c = 0; c < CPR; ++c) {
        // gate rows sit in MFMA tile gi at 8 * gq, the matching up rows in tile ui at 8 * uq
        constexpr int kHalfTiles = NCI >= 2 ? NCI / 2 : 1;
        const int gi = NCI >= 2 ? c / 4 : 0;
        const int gq = NCI >= 2 ? c % 4 : c;
        const int ui = NCI >= 2 ? gi + kHalfTiles : 0;
        const int uq = NCI >= 2 ? gq : c + 2;
        const int n = n0 + c * 8 + 4 * lhalf;
        const int ns = n < inter ? n : 0;
        const float4 wg = *reinterpret_cast<const float4*>(wsc + ns);
        const float4 wu = *reinterpret_cast<const float4*>(wsc + inter + ns);
        const int g[4] = {acc[gi][tj][4 * gq], acc[gi][tj][4 * gq + 1], acc[gi][tj][4 * gq + 2], acc[gi][tj][4 * gq + 3]};
        const int u[4] = {acc[ui][tj][4 * uq], acc[ui][tj][4 * uq + 1], acc[ui][tj][4 * uq + 2], acc[ui][tj][4 * uq + 3]};
        *reinterpret_cast<uint2*>(wave_lds + row * kRowBytes + ((c ^ staging_swizzle<CPR>(row)) * 16) + lhalf * 8) =
            silu_mul_epilogue4(g, u, as, wg, wu);
      }
    }
    wait_vmcnt<0>();  // as in the down epilogue: only the stores below stay pending
#pragma unroll
    for (int r = 0; r < CPR; ++r) {
      const int row = r * (64 / CPR) + lane / CPR;
      const int chunk = lane % CPR;
      const uint4 v =
          *reinterpret_cast<const uint4*>(wave_lds + row * kRowBytes + ((chunk ^ staging_swizzle<CPR>(row)) * 16));
      const int32_t t = __shfl(tok[(r * (64 / CPR)) >> 5], row & 31);
      const int n = n0 + chunk * 8;
      if (t >= 0 && n < inter)
        __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * inter + n));
    }
  }
}

template <int MODE, bool DEEP>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_kernel(TileParams p) {
  using G = Geometry<DEEP>;
  constexpr int kStageBytes = G::kStageBytes;
  __shared__ __align__(16) char stages[G::kSlots * kStageBytes];
  __shared__ uint32_t tile_desc[G::kMaxTiles];
  __shared__ int wave_part[kWaves];
  __shared__ __align__(16) float channel_scales[kWaves * 128];
  __shared__ int total_tiles;

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int load_sub = wave * G::kTokLoads / 8;  // token sub-block whose rows this wavefront loads
  const int nk = p.K / kBK;

  const int npp = *p.npp;
  const int nblocks = npp / p.B;
  const int sub_per_block = p.B / 64;
  const int per_tile = G::kTileTok / p.B;  // 1, 2 or 4 blocks
  const int ntile =
      p.ascend ? build_tile_list_ascending(p.expert_ids, nblocks, p.E, per_tile == 4 ? 2 : per_tile == 2 ? 1 : 0,
                                           reinterpret_cast<int*>(stages), wave_part, tile_desc, &total_tiles,
                                           G::kMaxTiles)
               : build_tile_list(p.expert_ids, nblocks, per_tile, reinterpret_cast<int*>(stages), wave_part, tile_desc,
                                 &total_tiles, G::kMaxTiles);
  const int total = ntile * p.ntiles;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int stride = gridDim.x / kXcds;

  // ---- MFMA operand reads: lane feeds row (lane & 31), 16-byte chunk 2 * kk + (lane >> 5) ----
  const int lsw = swizzle_of_row(lane & 31);
  const int lhalf = lane >> 5;
  TileReads rd;
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

  // Does any run of blocks make more than one tile?  (A tile that is not the first of its group, or a
  // group of more than one.)  If none does, every weight row is read by one workgroup only and is
  // fetched with the non-temporal hint; the choice is made once per launch so that the step loop
  // carries no test.
  bool shared_local = false;
  for (int g = t; g < ntile; g += kThreads) shared_local |= (tile_desc[g] >> 20) != (1u << 4);  // rank 0, group size 1
  const bool weights_shared = __syncthreads_or(shared_local ? 1 : 0) != 0;

  auto run = [&](auto nt_tag) {
  constexpr bool NT = decltype(nt_tag)::value;
  int it = blockIdx.x / kXcds;
  Task tk = decode(it);
  while (tk.e == -2) tk = decode(it += stride);
  if (tk.e < 0) return;
  TaskLoads ld;
  setup_loads<MODE, DEEP>(p, tk, wave, lane, ld);
  bool my_tokens = load_sub < tk.nsub;
  int slot = 0;  // stage of the step being multiplied
  // The scratch of the tile list lived in the stage memory; everybody is past it (the builder ends
  // with a barrier), so the first stage(s) can be filled now.
  issue_stage_loads<DEEP, NT>(ld, p.a_q, stage0, wave, 0, my_tokens);
  if constexpr (DEEP) issue_stage_loads<DEEP, NT>(ld, p.a_q, stage0 + kStageBytes, wave, kBK, my_tokens);
  constexpr int kLoadsPerStep = 4 + G::kTokLoads;  // per wavefront (deep geometry: always that many)

  bool stores_pending = false;
  while (true) {
    // look ahead: the first loads of the next task are issued during the last step(s) of this one
    int nit = it + stride;
    Task nx = decode(nit);
    while (nx.e == -2) nx = decode(nit += stride);
    TaskLoads nld = ld;
    if (nx.e >= 0) setup_loads<MODE, DEEP>(p, nx, wave, lane, nld);
    const bool nx_tokens = load_sub < nx.nsub;

    // NCI = MFMA tiles of 32 weight rows per wavefront; `active`: the wavefront multiplies in this task
    auto run_task = [&](auto nci_tag, bool active) {
      constexpr int NCI = decltype(nci_tag)::value;
      v16i acc[NCI][2];
#pragma unroll
      for (int ci = 0; ci < NCI; ++ci)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[ci][tj][r] = 0;
      make_reads<MODE, NCI>(wave, lane, rd);
      for (int s = 0; s < nk; ++s) {
        // This wavefront's loads of step s have landed ...  A wavefront that has just run an
        // epilogue waited for all its loads there and only has the epilogue's stores pending: it
        // lets them drain behind the first step instead of stalling on them.
        if constexpr (DEEP) {
          // in flight behind step s: the loads of step s + 1 (issued one step ago), if there is one
          if (s > 0 || !stores_pending) {
            if (s + 1 < nk || nx.e >= 0)
              wait_vmcnt<kLoadsPerStep>();
            else
              wait_vmcnt<0>();
          }
        } else {
          if (s > 0 || !stores_pending) wait_vmcnt<0>();
        }
        // ... and so have everybody's; everybody is also done reading the stage of the step before,
        // which is the one to fill next
        __builtin_amdgcn_s_barrier();
        constexpr int kAhead = G::kSlots - 1;
        int fill = slot + kAhead;
        if (fill >= G::kSlots) fill -= G::kSlots;
        const uint32_t fill_addr = stage0 + fill * kStageBytes;
        if (s + kAhead < nk)
          issue_stage_loads<DEEP, NT>(ld, p.a_q, fill_addr, wave, (s + kAhead) * kBK, my_tokens);
        else if (nx.e >= 0)
          issue_stage_loads<DEEP, NT>(nld, p.a_q, fill_addr, wave, (s + kAhead - nk) * kBK, nx_tokens);
        if (active) multiply_stage<NCI>(rd, stages + slot * kStageBytes, acc);
        slot = slot + 1 == G::kSlots ? 0 : slot + 1;
      }
      // everybody is done reading the stage of the last step: it becomes the epilogue's staging area
      // (the next task's first loads went to the other stages)
      __builtin_amdgcn_s_barrier();
      const int last = slot == 0 ? G::kSlots - 1 : slot - 1;
      if (active)
        epilogue<MODE, NCI>(p, tk, wave, lane, acc, stages + last * kStageBytes + wave * 8192 / (4 / NCI),
                            channel_scales + wave * 128);
      stores_pending = active && MODE != kAccI32;
    };
    if constexpr (DEEP) {
      if (tk.nsub >= 2)
        run_task(std::integral_constant<int, 2>{}, true);
      else
        run_task(std::integral_constant<int, 1>{}, true);
    } else {
      run_task(std::integral_constant<int, 4>{}, load_sub < tk.nsub);
    }
    if (nx.e < 0) break;
    tk = nx;
    ld = nld;
    my_tokens = nx_tokens;
    it = nit;
  }
  wait_vmcnt<0>();
  };
  if (weights_shared)
    run(std::false_type{});
  else
    run(std::true_type{});
}

// ---------------------------------------------------------------------------------------------
// Ring pipeline for the 256 x 256 tile (the geometry kTileRing; never chosen by itself, kept as a
// measured alternative to the two-stage pipeline above): reduction steps of 64 bytes through a ring
// of four 32 KB stages (16 KB of weight rows, then 16 KB of token rows), every stage filled three
// steps before it is multiplied, so that up to 96 KB of loads are in flight per compute unit
// against the 64 KB of the two-stage pipeline.  LDS rows are 64 bytes (four 16-byte chunks); a
// wave-level load covers 16 rows.
//
// One barrier per step, placed in the MIDDLE of the step: the operands of the step's second
// 32-byte half are read while the first half multiplies; once they are in registers the whole
// stage has been consumed, so the barrier both frees it for the loads four steps ahead and
// publishes the next stage, whose first-half operands are then read while the second half
// multiplies.  The matrix pipe therefore always has eight MFMAs with their operands in registers
// on either side of the barrier.
//
// Measured against the two-stage pipeline on 65536 routed rows x 128 experts (gate_up 4096 x 2048,
// down 2048 x 2048): same results bit for bit, 7-10 % slower.  A lane's 16-byte load takes a
// quarter of a 64-byte row, so every 128-byte line is requested from L2 twice (the request count
// per launch doubles, the bytes fetched from HBM stay), and the path from L2 into LDS, not the
// depth of the pipeline, is what bounds the loads of this tile.
constexpr int kRingBK = 64;
constexpr int kRingSlots = 4;
constexpr int kRingHalf = kBN * kRingBK;    // 16 KB
constexpr int kRingStage = 2 * kRingHalf;   // 32 KB
constexpr int kRingLoads = 4;               // wave-level loads per wavefront and step

// chunk swizzle of a 64-byte LDS row: 16 consecutive rows reading one logical chunk, and 8 rows
// reading two neighbouring chunks, both spread over all banks
__device__ __forceinline__ int swizzle_of_row64(int r) { return (((r >> 2) & 1) << 1) | ((r >> 3) & 1); }

struct RingLoads {
  const int8_t* wbase;
  uint32_t woff[2];
  uint32_t xoff[2];
};

// lane fills slot (lane & 3) of row 32 * wave + 16 * i + (lane >> 2) of the weight half and of the token half
template <int MODE>
__device__ __forceinline__ void ring_setup_loads(const TileParams& p, const Task& tk, int wave, int lane, RingLoads& ld) {
  const int K = p.K;
  const int inter = p.N / 2;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = 32 * wave + 16 * i + (lane >> 2);
    const int chunk = ((lane & 3) ^ swizzle_of_row64(row)) * 16;
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
    if ((row >> 6) < tk.nsub) {
      const int32_t tok = p.sorted_ids[tk.slot0 + row];
      if (tok >= 0 && tok < p.P) arow = (uint32_t)(tok / p.row_div);
    }
    ld.xoff[i] = arow * (uint32_t)K + chunk;
  }
  ld.wbase = p.w + (int64_t)tk.e * p.N * K;
}

__device__ __forceinline__ void ring_issue_loads(const RingLoads& ld, const int8_t* a_q, uint32_t stage_addr, int wave,
                                                 int koff) {
#pragma unroll
  for (int i = 0; i < 2; ++i) load_to_lds_16(a_q + koff, ld.xoff[i], stage_addr + kRingHalf + (wave * 2 + i) * 1024);
#pragma unroll
  for (int i = 0; i < 2; ++i) load_to_lds_16(ld.wbase + koff, ld.woff[i], stage_addr + (wave * 2 + i) * 1024);
}

struct RingReads {
  int w_ld[4];
  int x_ld[2];
  int chunk[2];
};

struct RingOperands {
  v4i a[4], b[2];
};

__device__ __forceinline__ void ring_read(const RingReads& rd, const char* stage, int kk, RingOperands& o) {
  o.b[0] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[0] + rd.chunk[kk]);
  o.a[0] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[0] + rd.chunk[kk]);
  o.b[1] = *reinterpret_cast<const v4i*>(stage + rd.x_ld[1] + rd.chunk[kk]);
#pragma unroll
  for (int ci = 1; ci < 4; ++ci) o.a[ci] = *reinterpret_cast<const v4i*>(stage + rd.w_ld[ci] + rd.chunk[kk]);
}

__device__ __forceinline__ void ring_multiply(const RingOperands& o, v16i (&acc)[4][2]) {
#pragma unroll
  for (int ci = 0; ci < 4; ++ci)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) acc[ci][tj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a[ci], o.b[tj], acc[ci][tj], 0, 0, 0);
}

__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }  // lgkmcnt(0), others free

// The epilogue of the ring pipeline: the same arithmetic as `epilogue` with four MFMA tiles per
// wavefront, staged through 4 KB per wavefront (32 token rows x 64 channels of bf16 at a time).
template <int MODE>
__device__ __forceinline__ void ring_epilogue(const TileParams& p, const Task& tk, int wave, int lane, v16i (&acc)[4][2],
                                              char* wave_lds, float* wave_scales) {
  const int tg = wave / 2;
  const int cpart = wave % 2;
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  const int inter = p.N / 2;
  int32_t tok[2];
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    tok[tj] = p.sorted_ids[tk.slot0 + tg * 64 + tj * 32 + lrow];
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
          const int n = tk.nt * kBN + cpart * 128 + ci * 32 + 8 * q + 4 * lhalf;
          if (n < p.N)
            *reinterpret_cast<v4i*>(out + n) =
                v4i{acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
        }
    }
  } else if constexpr (MODE == kDown) {
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * kBN + cpart * 128;  // first channel of this wavefront
    // channel scales through LDS (see `epilogue`)
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
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // 32 token rows x 64 channels (MFMA tiles 2h and 2h + 1)
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int ci = 2 * h + c / 4;
          const int q = c % 4;
          const float4 ws = *reinterpret_cast<const float4*>(wave_scales + ci * 32 + 8 * q + 4 * lhalf);
          const int v[4] = {acc[ci][tj][4 * q], acc[ci][tj][4 * q + 1], acc[ci][tj][4 * q + 2], acc[ci][tj][4 * q + 3]};
          *reinterpret_cast<uint2*>(wave_lds + lrow * 128 + ((c ^ staging_swizzle<8>(lrow)) * 16) + lhalf * 8) =
              down_epilogue4(v, as[tj], ws, rw[tj]);
        }
        // everything this wavefront has in flight is complete before its first stores, which
        // are then the only vector-memory work still pending when the next tile starts
        if (tj == 0 && h == 0) wait_vmcnt<0>();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = r * 8 + lane / 8;
          const int chunk = lane % 8;
          const uint4 v = *reinterpret_cast<const uint4*>(wave_lds + row * 128 + ((chunk ^ staging_swizzle<8>(row)) * 16));
          const int32_t t = __shfl(tok[tj], row);
          const int n = n0 + h * 64 + chunk * 8;
          if (t >= 0 && n < p.N)
            __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w},
                                        reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * p.N + n));
        }
      }
    }
  } else {
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    const int n0 = tk.nt * 128 + cpart * 64;  // first gate channel of this wavefront
    float as[2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) as[tj] = tok[tj] >= 0 ? p.a_scale[tok[tj] / p.row_div] : 0.0f;
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      // 32 token rows x 64 activation channels
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        // gate rows sit in MFMA tile gi at 8 * gq, the matching up rows in tile gi + 2
        const int gi = c / 4;
        const int gq = c % 4;
        const int ui = gi + 2;
        const int n = n0 + c * 8 + 4 * lhalf;
        const int ns = n < inter ? n : 0;
        const float4 wg = *reinterpret_cast<const float4*>(wsc + ns);
        const float4 wu = *reinterpret_cast<const float4*>(wsc + inter + ns);
        const int g[4] = {acc[gi][tj][4 * gq], acc[gi][tj][4 * gq + 1], acc[gi][tj][4 * gq + 2], acc[gi][tj][4 * gq + 3]};
        const int u[4] = {acc[ui][tj][4 * gq], acc[ui][tj][4 * gq + 1], acc[ui][tj][4 * gq + 2], acc[ui][tj][4 * gq + 3]};
        *reinterpret_cast<uint2*>(wave_lds + lrow * 128 + ((c ^ staging_swizzle<8>(lrow)) * 16) + lhalf * 8) =
            silu_mul_epilogue4(g, u, as[tj], wg, wu);
      }
      if (tj == 0) wait_vmcnt<0>();  // as in the down epilogue: only the stores below stay pending
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = r * 8 + lane / 8;
        const int chunk = lane % 8;
        const uint4 v = *reinterpret_cast<const uint4*>(wave_lds + row * 128 + ((chunk ^ staging_swizzle<8>(row)) * 16));
        const int32_t t = __shfl(tok[tj], row);
        const int n = n0 + chunk * 8;
        if (t >= 0 && n < inter)
          __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w},
                                      reinterpret_cast<v4i*>(static_cast<uint16_t*>(p.out) + (int64_t)t * inter + n));
      }
    }
  }
}

template <int MODE>
__global__ __launch_bounds__(kThreads, 1) void gemm_ring_kernel(TileParams p) {
  constexpr int kMaxTiles = 6144;
  __shared__ __align__(16) char stages[kRingSlots * kRingStage];
  __shared__ uint32_t tile_desc[kMaxTiles];
  __shared__ int wave_part[kWaves];
  __shared__ __align__(16) float channel_scales[kWaves * 128];
  __shared__ int total_tiles;

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int my_sub = wave / 2;  // token sub-block this wavefront multiplies
  const int nk = p.K / kRingBK;

  const int npp = *p.npp;
  const int nblocks = npp / p.B;
  const int sub_per_block = p.B / 64;
  const int per_tile = 256 / p.B;  // 2 or 4 blocks
  const int ntile =
      p.ascend ? build_tile_list_ascending(p.expert_ids, nblocks, p.E, per_tile == 4 ? 2 : 1, reinterpret_cast<int*>(stages),
                                           wave_part, tile_desc, &total_tiles, kMaxTiles)
               : build_tile_list(p.expert_ids, nblocks, per_tile, reinterpret_cast<int*>(stages), wave_part, tile_desc,
                                 &total_tiles, kMaxTiles);
  const int total = ntile * p.ntiles;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int stride = gridDim.x / kXcds;

  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  RingReads rd;
  {
    const int cpart = wave % 2;
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) {
      int row;
      if constexpr (MODE == kGateUpSilu)
        row = (ci < 2 ? 0 : 128) + cpart * 64 + (ci & 1) * 32 + lrow;  // LDS rows 0..127 gate, 128..255 up
      else
        row = cpart * 128 + ci * 32 + lrow;
      rd.w_ld[ci] = row * kRingBK;
    }
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) rd.x_ld[tj] = kRingHalf + (my_sub * 64 + tj * 32 + lrow) * kRingBK;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) rd.chunk[kk] = ((2 * kk + lhalf) ^ swizzle_of_row64(lrow)) * 16;
  }
  const uint32_t stage0 = lds_address(stages);

  auto decode = [&](int it) {
    Task tk;
    tk.e = -1;
    tk.nt = 0;
    tk.slot0 = 0;
    tk.nsub = 0;
    if (it < per_xcd && xcd * per_xcd + it < total) {
      const int task = xcd * per_xcd + it;
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
  RingLoads ld;
  ring_setup_loads<MODE>(p, tk, wave, lane, ld);
  int slot = 0;  // stage of the step being multiplied
  // the scratch of the tile list lived in the stage memory; the builder ends with a barrier
#pragma unroll
  for (int s = 0; s < kRingSlots - 1; ++s) ring_issue_loads(ld, p.a_q, stage0 + s * kRingStage, wave, s * kRingBK);

  bool stores_pending = false;
  bool first_task = true;
  while (true) {
    int nit = it + stride;
    Task nx = decode(nit);
    while (nx.e == -2) nx = decode(nit += stride);
    RingLoads nld = ld;
    if (nx.e >= 0) ring_setup_loads<MODE>(p, nx, wave, lane, nld);
    const bool has_next = nx.e >= 0;
    const bool active = my_sub < tk.nsub;

    // Task start.  The loads of steps 0..2 were issued during the previous task (or above), and every
    // wavefront has waited for its share of step 0 (at the previous task's last barrier; here for the
    // first task).  The barrier also ends the epilogue's use of the stage that step 3 goes to.
    if (first_task) wait_vmcnt<2 * kRingLoads>();
    first_task = false;
    __builtin_amdgcn_s_barrier();
    {
      int fill = slot + kRingSlots - 1;
      if (fill >= kRingSlots) fill -= kRingSlots;
      ring_issue_loads(ld, p.a_q, stage0 + fill * kRingStage, wave, (kRingSlots - 1) * kRingBK);
    }
    v16i acc[4][2];
#pragma unroll
    for (int ci = 0; ci < 4; ++ci)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ci][tj][r] = 0;
    RingOperands o0, o1;
    if (active) ring_read(rd, stages + slot * kRingStage, 0, o0);
    for (int s = 0; s < nk; ++s) {
      const char* stage = stages + slot * kRingStage;
      if (active) {
        ring_read(rd, stage, 1, o1);
        ring_multiply(o0, acc);
      }
      // The loads of the following step (this task's, or the next task's step 0) have landed for this
      // wavefront.  Behind them in the queue: the loads of the two steps after it, where they exist.  A
      // wavefront that has just run an epilogue waited for everything there and has only stores pending
      // in front of the loads it issued since: it lets them drain for two steps.
      const bool follows = s + 1 < nk || has_next;
      if (follows && !(stores_pending && s < 2)) {
        const int later = has_next ? 2 : nk - 2 - s;
        if (later >= 2)
          wait_vmcnt<2 * kRingLoads>();
        else if (later == 1)
          wait_vmcnt<kRingLoads>();
        else
          wait_vmcnt<0>();
      }
      wait_lds_reads();  // this wavefront is done with the stage
      __builtin_amdgcn_s_barrier();
      int nslot = slot + 1 == kRingSlots ? 0 : slot + 1;
      if (s + 1 < nk) {
        // refill the stage just consumed with the step four ahead (the last step's stage is left to
        // the epilogue; its loads are issued at the start of the next task)
        const int ahead = s + kRingSlots;
        if (ahead < nk)
          ring_issue_loads(ld, p.a_q, stage0 + slot * kRingStage, wave, ahead * kRingBK);
        else if (has_next)
          ring_issue_loads(nld, p.a_q, stage0 + slot * kRingStage, wave, (ahead - nk) * kRingBK);
        if (active) ring_read(rd, stages + nslot * kRingStage, 0, o0);
      }
      if (active) ring_multiply(o1, acc);
      slot = nslot;
    }
    const int last = slot == 0 ? kRingSlots - 1 : slot - 1;
    if (active)
      ring_epilogue<MODE>(p, tk, wave, lane, acc, stages + last * kRingStage + wave * 4096, channel_scales + wave * 128);
    stores_pending = active && MODE != kAccI32;
    if (!has_next) break;
    tk = nx;
    ld = nld;
    it = nit;
  }
  wait_vmcnt<0>();
}

bool ring_supports(const GemmArgs& a) {
  const int64_t act_rows = (a.num_pairs + a.row_div - 1) / a.row_div;
  if (!((a.block_size == 64 || a.block_size == 128) && a.k % kRingBK == 0 && a.k >= kRingSlots * kRingBK && a.n % 16 == 0 &&
        (int64_t)a.n * a.k < (1ll << 32) && act_rows * a.k < (1ll << 32)))
    return false;
  const int64_t blocks = (a.sorted_cap + a.block_size - 1) / a.block_size;
  const int per_tile = 256 / a.block_size;
  const int64_t tiles = a.expert_ids_ascend ? (blocks + per_tile - 1) / per_tile + a.num_experts : blocks;
  return tiles <= 6144 && blocks <= (int64_t)(kRingSlots * kRingStage / sizeof(int)) && blocks <= 65535;
}

template <int MODE, bool DEEP, bool RING = false>
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
  p.ascend = a.expert_ids_ascend && a.num_experts <= 2 * kThreads ? 1 : 0;
  p.out = a.out;
  const int grid = device_cu_count() / kXcds * kXcds;
  if constexpr (RING)
    hipLaunchKernelGGL((gemm_ring_kernel<MODE>), dim3((unsigned)grid), dim3(kThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_tile_kernel<MODE, DEEP>), dim3((unsigned)grid), dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

template <bool DEEP>
bool geometry_supports(const GemmArgs& a) {
  using G = Geometry<DEEP>;
  // per-lane source offsets are 32-bit: one expert's weights and the activation matrix must each
  // span less than 4 GiB
  const int64_t act_rows = (a.num_pairs + a.row_div - 1) / a.row_div;
  if (!((a.block_size == 64 || a.block_size == 128) && a.k % kBK == 0 && a.k >= G::kSlots * kBK && a.n % 16 == 0 &&
        (int64_t)a.n * a.k < (1ll << 32) && act_rows * a.k < (1ll << 32)))
    return false;
  // The tile list lives in LDS.  A run of equal expert ids of L blocks makes ceil(L / blocks per
  // tile) tiles; moe_align's ids ascend, so there is one run per expert.  Ids of unknown order could
  // make every block a tile of its own.  While the list is built the block ids sit in the stages.
  const int64_t blocks = (a.sorted_cap + a.block_size - 1) / a.block_size;
  const int per_tile = G::kTileTok / a.block_size;
  const int64_t tiles = a.expert_ids_ascend ? (blocks + per_tile - 1) / per_tile + a.num_experts : blocks;
  return tiles <= G::kMaxTiles && blocks <= (int64_t)(G::kSlots * G::kStageBytes / sizeof(int)) && blocks <= 65535;
}

}  // namespace

bool gemm_tile_supports(const GemmArgs& a) {
  switch (a.tile_geometry) {
    case kTileWide: return geometry_supports<false>(a);
    case kTileDeep: return geometry_supports<true>(a);
    case kTileRing: return ring_supports(a);
    default: return geometry_supports<false>(a) || geometry_supports<true>(a);
  }
}

// Measured on three layer shapes (Qwen3-30B-A3B, GLM-4.5-Air, DeepSeek-V3): the deep geometry wins up
// to about a hundred routed rows per expert, where a 256-row tile would be mostly padding and the
// kernel is bound by the weight stream; beyond that the wide tile's reuse of a weight tile by up to
// four sub-blocks wins.
bool gemm_tile_prefers_deep(const GemmArgs& a) {
  return a.num_pairs <= (int64_t)kTileDeepRowsPerExpert * a.num_experts;
}

// The geometry a launch of this family uses for `a` (kTileWide or kTileDeep; kTileRing only on demand).
int gemm_tile_geometry(const GemmArgs& a) {
  if (a.tile_geometry == kTileWide) return kTileWide;
  if (a.tile_geometry == kTileDeep) return kTileDeep;
  if (a.tile_geometry == kTileRing) return kTileRing;
  return geometry_supports<true>(a) && (gemm_tile_prefers_deep(a) || !geometry_supports<false>(a)) ? kTileDeep : kTileWide;
}

hipError_t launch_gemm_tile(const GemmArgs& a, hipStream_t stream) {
  const int geometry = gemm_tile_geometry(a);
  if (geometry == kTileRing) {
    switch (a.mode) {
      case kGateUpSilu: return launch_mode<kGateUpSilu, false, true>(a, stream);
      case kDown: return launch_mode<kDown, false, true>(a, stream);
      case kAccI32: return launch_mode<kAccI32, false, true>(a, stream);
      default: return hipErrorInvalidValue;
    }
  }
  if (geometry == kTileDeep) {
    switch (a.mode) {
      case kGateUpSilu: return launch_mode<kGateUpSilu, true>(a, stream);
      case kDown: return launch_mode<kDown, true>(a, stream);
      case kAccI32: return launch_mode<kAccI32, true>(a, stream);
      default: return hipErrorInvalidValue;
    }
  }
  switch (a.mode) {
    case kGateUpSilu: return launch_mode<kGateUpSilu, false>(a, stream);
    case kDown: return launch_mode<kDown, false>(a, stream);
    case kAccI32: return launch_mode<kAccI32, false>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe_i8
