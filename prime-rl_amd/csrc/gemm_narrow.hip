// Grouped int8 GEMM for gfx950, narrow-tile family (tens of rows per expert: small prefill chunks,
// large decode batches).
//
// In this regime every expert is active, a block of 64 rows is all the reuse a weight byte gets,
// and the layer is bound by streaming the weights from HBM once.  What matters is that the stream
// never stops: a workgroup keeps two reduction steps of loads in flight at all times, also across
// the end of a tile and through its epilogue.
//
// A workgroup is 4 wavefronts and two of them share a compute unit.  A tile is 64 token rows (one
// 64-row sub-block of a moe_align block) x 128 weight rows; the reduction runs in steps of 128
// bytes through a ring of three 24 KB LDS stages that both operands reach by global -> LDS loads
// (global_load_lds_dwordx4, no staging registers).  Wavefront w multiplies weight rows
// [32w, 32w + 32) of the tile with all 64 token rows as two v_mfma_i32_32x32x32_i8 tiles, used
// "transposed" (A operand = weight rows), so a lane ends up with runs of 4 consecutive channels of
// one token and stores its results straight from registers, 8 bytes at a time.  For the gate_up
// GEMM the 32 weight rows of a wavefront are 16 gate rows and the 16 matching up rows, which puts a
// gate value and its up value into the same lane.
//
// Nothing in the steady state is a compiler-visible vector load: token ids, activation scales,
// routed weights and channel scales of the NEXT tile also travel global -> LDS (4 bytes per lane)
// while the current tile is reduced, into a small double-buffered area.  The only waits on vector
// memory are therefore the explicit ones of the ring, which leave the most recent group of loads
// in flight.  (The vector-memory counter retires loads and stores in order, so the ring waits
// before it issues a tile's stores and never has to count them.)
//
// LDS rows are 128 bytes; the 16-byte chunk index is XOR-swizzled with row bits so that the MFMA
// operand reads (32 consecutive rows, same chunk) spread over all banks; because a load fills LDS
// linearly the swizzle is applied to the global source address of each lane.
#include "common.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kTok = 64;    // token rows per tile
constexpr int kCh = 128;    // weight rows per tile
constexpr int kBK = 128;    // reduction bytes per step
constexpr int kStages = 3;
constexpr int kTokOffset = kCh * kBK;
constexpr int kStageBytes = (kCh + kTok) * kBK;  // 24 KB
constexpr int kStageLoads = 6;                   // 1 KB loads per wavefront and step: 4 weight + 2 token
constexpr int kXcds = 8;
constexpr int kFirstGroup = 2;                   // the last loads of the start-up: token rows of step 1
constexpr int kMinSteps = 4;  // the look-ahead of the next tile's inputs needs this many steps per tile

// Inputs of one tile's epilogue (and of the loads of its token rows), filled by 4-byte global -> LDS
// loads while the previous tile is reduced.
struct TileAux {
  int32_t ids[kTok];    // sorted_token_ids of the tile's rows
  float a_scale[kTok];  // activation scale of each row (0 index for padding rows)
  float row_w[kTok];    // routed weight of each row (down GEMM)
  float w_scale[kCh];   // down: scales of the tile's 128 channels; gate_up: 64 gate scales, 64 up scales
};

struct NarrowParams {
  const int8_t* a_q;
  const float* a_scale;
  const int8_t* w;
  const float* w_scale;
  const float* row_weight;  // null = 1
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

__device__ __forceinline__ uint64_t uniform_address(const void* base) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  // readfirstlane yields a signed int: go through uint32_t so that the low half is not sign-extended
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  return (uint64_t)lo | ((uint64_t)hi << 32);
}

// 16 (or 4) bytes per lane from global memory straight into LDS: lane i lands at lds_addr + 16 * i
// (+ 4 * i).  lds_addr is wave-uniform and goes through M0; the source is a wave-uniform base plus
// an unsigned 32-bit byte offset per lane.  Inline assembly, so that the compiler neither counts
// these loads nor waits for them: the ring's explicit waits do.
__device__ __forceinline__ void load_to_lds_16(const void* base, uint32_t offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"((uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(offset), "s"(uniform_address(base))
               : "memory", "m0");
}
// The same with the non-temporal hint: for weight rows that no other tile of this launch reads (the
// expert's rows fit in one tile).  Streamed that way they do not displace the token rows and the
// other tiles' shared weights from L2: measured 8-13 % on launches bound by the weight stream, and
// a loss wherever a second tile of the expert would have found the rows in L2, hence per task.
__device__ __forceinline__ void load_to_lds_16_stream(const void* base, uint32_t offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"((uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(offset), "s"(uniform_address(base))
               : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_4(const void* base, uint32_t offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"((uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(offset), "s"(uniform_address(base))
               : "memory", "m0");
}

// Two ints from wave-uniform addresses through the scalar (read-only) path, one wait for both.
// After the inline assembly above the compiler no longer proves that global memory is unchanged and
// would fetch such values with vector loads, whose wait would drain the ring; this only waits for
// itself.  Only for data written before the launch (the scalar cache does not see this kernel's
// stores).
__device__ __forceinline__ void scalar_load2(const int32_t* pa, const int32_t* pb, int32_t& a, int32_t& b) {
  asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(a), "=&s"(b)
               : "s"(uniform_address(pa)), "s"(uniform_address(pb))
               : "memory");
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) char*)p);
}

__device__ __forceinline__ int swizzle_of_row(int r) { return (r & 7) ^ ((r >> 3) & 1); }

struct Task {
  int e;          // expert; -1 = no more work
  int ct;         // channel tile
  int64_t slot0;  // first slot of the tile in sorted_ids
  bool single;    // the expert's rows fit in this one tile: nothing else reads its weight rows
};

struct TaskLoads {
  const int8_t* wbase;  // weights of the task's expert (wave-uniform)
  bool stream;          // fetch the weight rows with the non-temporal hint
  uint32_t woff[4];     // per lane: byte offset of its chunk of weight row i from wbase
  uint32_t xoff[2];     // per lane: byte offset of its chunk of token row i from a_q
};

// Extra 4-byte loads per wavefront in the step that fetches the next tile's scales.
template <int MODE>
constexpr int aux_loads() {
  return MODE == kDown ? 4 : MODE == kGateUpSilu ? 3 : 0;
}

// Waits until at most the `n` most recent vector-memory operations of this wavefront are pending;
// n is the size of the group issued last, one of four values.
template <int MODE>
__device__ __forceinline__ void wait_all_but(int n) {
  if (n == kStageLoads)
    wait_vmcnt<kStageLoads>();
  else if (n == kFirstGroup)
    wait_vmcnt<kFirstGroup>();
  else if (n == kStageLoads + 1)
    wait_vmcnt<kStageLoads + 1>();
  else
    wait_vmcnt<kStageLoads + aux_loads<MODE>()>();
}

template <int MODE>
__global__ __launch_bounds__(kThreads, 2) void gemm_narrow_kernel(NarrowParams p) {
  __shared__ __align__(16) char stages[kStages * kStageBytes];
  __shared__ __align__(16) TileAux aux[2];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  const int K = p.K;
  const int nk = K / kBK;
  const int inter = p.N / 2;

  // ---- this workgroup's tasks: (tile, channel tile), channel tile fastest, split into 8 contiguous
  // ranges, one per XCD (workgroup id % 8), so that workgroups that run side by side share token
  // rows and expert weights in that XCD's L2 ----
  const int npp = *p.npp;
  const int sub_per_block = p.B / kTok;
  const int total = (npp / kTok) * p.ntiles;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds;
  const int stride = gridDim.x / kXcds;
  const int range_end = (xcd + 1) * per_xcd < total ? (xcd + 1) * per_xcd : total;

  // The first task at or after candidate `it` (in steps of `stride`) whose expert id is valid and
  // whose rows are not all padding (valid rows are a prefix of a block).
  auto find_task = [&](int& it) {
    Task tk;
    tk.e = -1;
    tk.ct = 0;
    tk.slot0 = 0;
    tk.single = false;
    for (; xcd * per_xcd + it < range_end; it += stride) {
      const int task = xcd * per_xcd + it;
      const int tile = task / p.ntiles;
      const int blk = tile / sub_per_block;
      const int64_t slot0 = (int64_t)blk * p.B + (int64_t)(tile % sub_per_block) * kTok;
      int32_t e, first;
      scalar_load2(p.expert_ids + blk, p.sorted_ids + slot0, e, first);
      if (e >= 0 && e < p.E && first >= 0 && first < p.P) {
        tk.e = e;
        tk.ct = task - tile * p.ntiles;
        tk.slot0 = slot0;
        // Does the expert hold other tiles?  Its neighbours in the block list, and the other
        // 64-row half of a 128-row block (valid rows are a prefix: a second half means the first is
        // full, and the second half's first slot says whether it is in use).
        const int nblocks = npp / p.B;
        int32_t before, after;
        scalar_load2(p.expert_ids + (blk > 0 ? blk - 1 : blk), p.expert_ids + (blk + 1 < nblocks ? blk + 1 : blk), before,
                     after);
        bool single = (blk == 0 || before != e) && (blk + 1 >= nblocks || after != e);
        if (single && sub_per_block > 1) {
          if (tile % sub_per_block != 0) {
            single = false;
          } else {
            int32_t other, unused;
            scalar_load2(p.sorted_ids + slot0 + kTok, p.sorted_ids + slot0, other, unused);
            single = !(other >= 0 && other < p.P);
          }
        }
        tk.single = single;
        break;
      }
    }
    return tk;
  };

  const uint32_t stage0 = lds_address(stages);

  // ---- global -> LDS loads ----
  // Lane fills LDS slot (lane & 7) of row base + 8 * i + (lane >> 3): it fetches the logical chunk
  // (lane & 7) ^ swizzle(row) of that row, and swizzle(row) = (lane >> 3) ^ (i & 1).
  auto setup_weight_loads = [&](const Task& tk, TaskLoads& ld) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 32 * wave + 8 * i + (lane >> 3);  // LDS weight row; wavefront row / 32 multiplies it
      const int chunk = ((lane & 7) ^ (lane >> 3) ^ (i & 1)) * 16;
      int n;
      if constexpr (MODE == kGateUpSilu) {
        const int j = row & 31;
        const int ch = tk.ct * 64 + (row >> 5) * 16 + (j & 15);
        n = (ch < inter ? ch : inter - 1) + (j >= 16 ? inter : 0);
      } else {
        const int ch = tk.ct * kCh + row;
        n = ch < p.N ? ch : p.N - 1;
      }
      ld.woff[i] = (uint32_t)n * (uint32_t)K + chunk;
    }
    ld.wbase = p.w + (int64_t)tk.e * p.N * K;
    ld.stream = tk.single;
  };
  auto setup_token_loads = [&](const TileAux& ax, TaskLoads& ld) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 16 * wave + 8 * i + (lane >> 3);
      const int chunk = ((lane & 7) ^ (lane >> 3) ^ (i & 1)) * 16;
      const int32_t tok = ax.ids[row];
      const uint32_t arow = (tok >= 0 && tok < p.P) ? (uint32_t)(tok / p.row_div) : 0u;
      ld.xoff[i] = arow * (uint32_t)K + chunk;
    }
  };
  auto issue_weights = [&](const TaskLoads& ld, int stage, int koff) {
    const uint32_t base = stage0 + stage * kStageBytes;
    if (ld.stream) {
#pragma unroll
      for (int i = 0; i < 4; ++i) load_to_lds_16_stream(ld.wbase + koff, ld.woff[i], base + (wave * 4 + i) * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) load_to_lds_16(ld.wbase + koff, ld.woff[i], base + (wave * 4 + i) * 1024);
    }
  };
  auto issue_tokens = [&](const TaskLoads& ld, int stage, int koff) {
    const uint32_t base = stage0 + stage * kStageBytes + kTokOffset;
#pragma unroll
    for (int i = 0; i < 2; ++i) load_to_lds_16(p.a_q + koff, ld.xoff[i], base + (wave * 2 + i) * 1024);
  };
  auto issue_stage = [&](const TaskLoads& ld, int stage, int koff) {
    issue_weights(ld, stage, koff);
    issue_tokens(ld, stage, koff);
  };
  // Every wavefront fetches the whole (tiny) set: identical values to identical places, and each
  // wavefront's own wait covers what it reads.
  auto issue_ids = [&](const Task& tk, TileAux& ax) {
    load_to_lds_4(p.sorted_ids + tk.slot0, (uint32_t)lane * 4u, lds_address(ax.ids));
  };
  auto issue_scales = [&](const Task& tk, TileAux& ax) {
    if constexpr (MODE == kAccI32) return;
    const int32_t tok = ax.ids[lane];
    const uint32_t t = (tok >= 0 && tok < p.P) ? (uint32_t)tok : 0u;
    load_to_lds_4(p.a_scale, (t / (uint32_t)p.row_div) * 4u, lds_address(ax.a_scale));
    const float* wsc = p.w_scale + (int64_t)tk.e * p.N;
    if constexpr (MODE == kDown) {
      // without routed weights the slot is filled with something readable and never used
      if (p.row_weight)
        load_to_lds_4(p.row_weight, t * 4u, lds_address(ax.row_w));
      else
        load_to_lds_4(p.a_scale, 0u, lds_address(ax.row_w));
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = tk.ct * kCh + 64 * j + lane;
        load_to_lds_4(wsc, (uint32_t)(n < p.N ? n : p.N - 1) * 4u, lds_address(ax.w_scale + 64 * j));
      }
    } else {
      const int ch = tk.ct * 64 + lane;
      const uint32_t c = (uint32_t)(ch < inter ? ch : inter - 1);
      load_to_lds_4(wsc, c * 4u, lds_address(ax.w_scale));
      load_to_lds_4(wsc, (c + (uint32_t)inter) * 4u, lds_address(ax.w_scale + 64));
    }
  };

  // ---- MFMA operand reads: lane feeds row (lane & 31), 16-byte chunk 2 * kk + (lane >> 5) ----
  const int w_ld = (32 * wave + lrow) * kBK;
  int x_ld[2], chunk[4];
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) x_ld[tj] = kTokOffset + (tj * 32 + lrow) * kBK;
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) chunk[kk] = ((2 * kk + lhalf) ^ swizzle_of_row(lrow)) * 16;

  // acc[tj][4q + r] is weight row 8q + 4 * (lane >> 5) + r of this wavefront's 32, token row
  // tj * 32 + (lane & 31) of the tile.
  auto epilogue = [&](const Task& tk, const TileAux& ax, v16i (&acc)[2]) {
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const int row = tj * 32 + lrow;
      const int32_t tok = ax.ids[row];
      if (tok < 0 || tok >= p.P) continue;
      if constexpr (MODE == kAccI32) {
        int32_t* out = static_cast<int32_t*>(p.out) + (int64_t)tok * p.N;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = tk.ct * kCh + 32 * wave + 8 * q + 4 * lhalf;
          if (n < p.N)
            *reinterpret_cast<v4i*>(out + n) =
                v4i{acc[tj][4 * q], acc[tj][4 * q + 1], acc[tj][4 * q + 2], acc[tj][4 * q + 3]};
        }
      } else if constexpr (MODE == kDown) {
        uint16_t* out = static_cast<uint16_t*>(p.out) + (int64_t)tok * p.N;
        const float as = ax.a_scale[row];
        const float rw = p.row_weight ? ax.row_w[row] : 1.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int c = 32 * wave + 8 * q + 4 * lhalf;
          const int n = tk.ct * kCh + c;
          const float4 ws = *reinterpret_cast<const float4*>(ax.w_scale + c);
          const int v[4] = {acc[tj][4 * q], acc[tj][4 * q + 1], acc[tj][4 * q + 2], acc[tj][4 * q + 3]};
          if (n < p.N) *reinterpret_cast<uint2*>(out + n) = down_epilogue4(v, as, ws, rw);
        }
      } else {
        // weight rows 0..15 of the wavefront are gate channels, 16..31 the matching up channels
        uint16_t* out = static_cast<uint16_t*>(p.out) + (int64_t)tok * inter;
        const float as = ax.a_scale[row];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int c = 16 * wave + 8 * q + 4 * lhalf;
          const int n = tk.ct * 64 + c;
          const float4 wg = *reinterpret_cast<const float4*>(ax.w_scale + c);
          const float4 wu = *reinterpret_cast<const float4*>(ax.w_scale + 64 + c);
          const int g[4] = {acc[tj][4 * q], acc[tj][4 * q + 1], acc[tj][4 * q + 2], acc[tj][4 * q + 3]};
          const int u[4] = {acc[tj][4 * q + 8], acc[tj][4 * q + 9], acc[tj][4 * q + 10], acc[tj][4 * q + 11]};
          if (n < inter) *reinterpret_cast<uint2*>(out + n) = silu_mul_epilogue4(g, u, as, wg, wu);
        }
      }
    }
  };

  // ---- start-up: the first task's token ids, its weights (which need no ids) behind them, then
  // what depends on the ids: token rows and scales ----
  int it = blockIdx.x / kXcds;
  Task tk = find_task(it);
  if (tk.e < 0) return;
  int par = 0;
  TaskLoads ld;
  issue_ids(tk, aux[0]);
  setup_weight_loads(tk, ld);
  issue_weights(ld, 0, 0);
  issue_weights(ld, 1, kBK);
  wait_vmcnt<8>();  // the ids are in; every wavefront fetched its own copy, so no barrier is needed
  setup_token_loads(aux[0], ld);
  issue_scales(tk, aux[0]);
  issue_tokens(ld, 0, 0);
  issue_tokens(ld, 1, kBK);
  int last_group = kFirstGroup;  // size of the most recent group of loads: the token rows of step 1
  int nit = it + stride;
  Task nx = find_task(nit);
  int nnit = nit;
  Task nnx = nx;
  TaskLoads nld = ld;

  bool landed = false;  // the loads of the coming step are known to have landed (waited for before the stores)
  int stage = 0;        // ring position of the step being multiplied
  while (true) {
    v16i acc[2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[tj][r] = 0;

    for (int s = 0; s < nk; ++s) {
      // this wavefront's loads of step s have landed (only the group issued last is still in flight) ...
      if (!landed) wait_all_but<MODE>(last_group);
      landed = false;
      // ... and so have everybody's; everybody is also done reading the stage that is filled next
      __builtin_amdgcn_s_barrier();
      const int fill = stage >= 1 ? stage - 1 : kStages - 1;  // (stage + 2) % 3
      last_group = kStageLoads;
      if (s == 0) {
        // ids of the next tile (of this one again if it is the last: harmless)
        issue_ids(nx.e >= 0 ? nx : tk, aux[par ^ 1]);
        last_group = kStageLoads + 1;
      } else if (s == 2) {
        // they are in (issued two steps ago): the next tile's row addresses and scales
        const Task& t2 = nx.e >= 0 ? nx : tk;
        setup_weight_loads(t2, nld);
        setup_token_loads(aux[par ^ 1], nld);
        issue_scales(t2, aux[par ^ 1]);
        last_group = kStageLoads + aux_loads<MODE>();
      }
      if (s + 2 < nk)
        issue_stage(ld, fill, (s + 2) * kBK);
      else if (nx.e >= 0)
        issue_stage(nld, fill, (s + 2 - nk) * kBK);
      else
        issue_stage(ld, fill, (nk - 1) * kBK);  // nothing left to fetch: keeps the group sizes uniform
      if (s == 3 && nx.e >= 0) {
        // The task after the next is looked up here, where the wait for the two scalar loads hides
        // behind the loads just issued, and not between two tiles.
        nnit = nit + stride;
        nnx = find_task(nnit);
      }
      const char* st = stages + stage * kStageBytes;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const v4i a = *reinterpret_cast<const v4i*>(st + w_ld + chunk[kk]);
        const v4i b0 = *reinterpret_cast<const v4i*>(st + x_ld[0] + chunk[kk]);
        const v4i b1 = *reinterpret_cast<const v4i*>(st + x_ld[1] + chunk[kk]);
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b0, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b1, acc[1], 0, 0, 0);
      }
      stage = stage + 1 < kStages ? stage + 1 : 0;
    }
    // Before the stores, everything but the group issued in the last step is complete: the coming
    // step's loads have landed, and the stores need not be counted by the next wait.
    wait_all_but<MODE>(last_group);
    landed = true;
    epilogue(tk, aux[par], acc);
    if (nx.e < 0) break;
    tk = nx;
    ld = nld;
    par ^= 1;
    it = nit;
    nit = nnit;
    nx = nnx;
  }
  wait_vmcnt<0>();
}

template <int MODE>
hipError_t launch_mode(const GemmArgs& a, hipStream_t stream) {
  NarrowParams p;
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
  p.ntiles = MODE == kGateUpSilu ? (a.n / 2 + 63) / 64 : (a.n + kCh - 1) / kCh;
  p.out = a.out;
  const int grid = 2 * (device_cu_count() / kXcds * kXcds);  // two workgroups per compute unit
  hipLaunchKernelGGL(gemm_narrow_kernel<MODE>, dim3((unsigned)grid), dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

bool gemm_narrow_supports(const GemmArgs& a) {
  // per-lane source offsets are 32-bit: one expert's weights, the activation matrix and the per-pair
  // arrays must each span less than 4 GiB
  const int64_t act_rows = (a.num_pairs + a.row_div - 1) / a.row_div;
  return (a.block_size == 64 || a.block_size == 128) && a.k % kBK == 0 && a.k >= kMinSteps * kBK && a.n % 16 == 0 &&
         (int64_t)a.n * a.k < (1ll << 32) && act_rows * a.k < (1ll << 32) && a.num_pairs < (1ll << 30) &&
         a.sorted_cap / kTok * ((a.n + 63) / 64) < (1ll << 31);
}

hipError_t launch_gemm_narrow(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case kGateUpSilu: return launch_mode<kGateUpSilu>(a, stream);
    case kDown: return launch_mode<kDown>(a, stream);
    case kAccI32: return launch_mode<kAccI32>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe_i8
