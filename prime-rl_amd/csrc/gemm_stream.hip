// Grouped int8 GEMM for gfx950, weight-streaming family (few rows per expert: decode).
//
// In this regime every weight byte is used by one 64-row block only, so the kernel is a pure HBM
// stream and what matters is that DRAM sees long contiguous reads with many of them in flight.
// Each wavefront owns 32 weight rows (two 16-row MFMA tiles; for the gate_up GEMM 16 gate rows and
// the 16 matching up rows) and walks the reduction dimension in windows of 256 bytes per row.  A
// window is fetched with eight 16-byte-per-lane loads, each covering 4 rows x 256 contiguous bytes,
// and the loads of the next window are issued before the current one is consumed.  The registers
// are then transposed into the MFMA operand layout through an 8 KB LDS area private to the
// wavefront (16-byte chunks XOR-swizzled with the row, so that neither the row-linear writes nor
// the 16-rows-same-chunk reads collide on a bank); no barrier is ever needed.  The few activation
// rows of the block are read from global memory (vector cache) directly in the operand layout.
//
// v_mfma_i32_16x16x64_i8 is used "transposed": the A operand carries 16 weight rows (output
// channels), the B operand 16 token rows, so each lane ends up with 4 consecutive channels of one
// token and the epilogue stores 8 (bf16) or 16 (int32) contiguous bytes per lane.  Lane l feeds
// row/column l % 16 and the 16 reduction bytes [16 * (l / 16), +16) of each 64-byte step; both
// operands use the same split, so the reduction order inside the instruction is immaterial.
//
// A 64-row block is handled as 16-row sub-tiles, one pass over the weights each (a second pass
// finds them in L2); sub-tiles that hold only padding are skipped (valid rows are a prefix of the
// block).  Blocks with many rows belong to the LDS-tiled family.
#include "common.hpp"
#include "quant_body.hpp"

namespace moe_i8 {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kSub = 16;      // token rows per sub-tile (MFMA N)
// Sub-tiles processed per pass over the weights: one while blocks rarely hold more than 16 rows (12
// wavefronts fit a CU), two beyond (the second sub-tile reuses the weights in registers instead of
// a second pass; the larger register set leaves 8 wavefronts per CU).  Measured crossover on the
// Qwen3-30B-A3B shape: about 10 routed rows per expert.
constexpr int kPairRowsPerExpert = 10;
constexpr int kStepK = 64;    // reduction bytes per MFMA
constexpr int kTiles = 2;     // 16-row weight tiles per wavefront
constexpr int kWinBytes = 256;                              // bytes of every weight row per window
constexpr int kWinSteps = kWinBytes / kStepK;               // MFMA steps per window
constexpr int kWinLoads = kTiles * 16 * kWinBytes / 1024;   // 1 KB wave-level loads per window
constexpr int kWaveLds = kTiles * 16 * kWinBytes;           // LDS bytes per wavefront
// Down GEMM that quantises its own activations: the 16 rows of a sub-tile are quantised from bf16
// into this LDS area by the workgroup (rows padded by 16 bytes so that the 16 rows of one operand
// read fall on different banks), reduction length limited accordingly.
constexpr int kFusedMaxK = 1024;
constexpr int kFusedRowPad = 16;

struct StreamParams {
  const uint16_t* a_bf16;  // fused-quantisation variant: bf16 activations [P, K] instead of a_q / a_scale
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
  int64_t cap;        // entries of sorted_ids
  int wave_capacity;  // wavefronts of this kernel the device holds at a time
  int round_even;     // in-kernel quantisation: ties to even instead of away from zero
  void* out;
};

template <int NS>
struct Window {
  v4i w[kWinLoads];
  v4i a[NS][kWinSteps];
};

// Rows of the q-th tile pair of the weight matrix: (gate tile, matching up tile) for gate_up,
// two consecutive tiles otherwise.  An invalid tile points at row 0 and is never stored.
template <int MODE>
__device__ __forceinline__ void pair_rows(const StreamParams& p, int q, int (&wrow)[kTiles], bool (&wok)[kTiles]) {
  if constexpr (MODE == kGateUpSilu) {
    const int inter = p.N / 2;
    const int ch = q * 16;
    wok[0] = wok[1] = ch < inter;
    wrow[0] = wok[0] ? ch : 0;
    wrow[1] = wok[0] ? inter + ch : 0;
  } else {
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
      const int ch = (q * kTiles + t) * 16;
      wok[t] = ch < p.N;
      wrow[t] = wok[t] ? ch : 0;
    }
  }
}

// `count_valid`: first pass over a block; the number of valid rows of the block is counted here,
// after the first weight window has been requested, and returned.
//
// kFused: the activations arrive as bf16; the workgroup quantises the 16 rows of the sub-tile into
// `a_lds` (int8) and `s_lds` (row scales) with the arithmetic of the stand-alone quantiser and the
// operand reads come from there.  Every wavefront of the workgroup must call this, also those with
// no weight rows left (`npairs` == 0): they take part in the quantisation and its two barriers.
template <int MODE, int NS, bool kFused>
__device__ __forceinline__ int stream_pass(const StreamParams& p, int blk, int e, int sub0, int first_pair,
                                           int npairs, char* wave_lds, bool count_valid, char* a_lds,
                                           float* s_lds, int32_t top_id) {
  const int lane = lane_id();
  const int col = lane & 15;  // token slot inside a sub-tile / weight row inside a tile
  const int grp = lane >> 4;  // which 16 reduction bytes of each step; which 4 output channels
  const int K = p.K;

  // Load j of a window covers rows 4 * (j % 4) + (lane >> 4) of tile j / 4, chunk lane & 15.
  const int ld_row = lane >> 4;
  const int ld_chunk = lane & 15;
  const int8_t* wbase = p.w + ((int64_t)e * p.N + ld_row) * K + ld_chunk * 16;
  // LDS: [32 rows][256 B]; chunk c of row r sits at position c ^ (r & 15)
  const int st_base = ld_row * kWinBytes + ((ld_chunk ^ ld_row) * 16);  // ^ (j % 4) * 64, + j * 1024
  const int rd_base = col * kWinBytes + ((grp ^ col) * 16);             // ^ u * 64, + t * 4096

  // The wavefront walks windows (pair 0, k 0), (pair 0, k 256), ..., (pair 1, k 0), ... ; `fq`/`fk`
  // track the window whose weights are being fetched (`fk` also the one whose activation rows are),
  // `cq`/`ck` the one being consumed.
  int fq = 0, wk = 0, fk = 0;
  auto fetch_weights = [&](Window<NS>& win) {
    int wrow[kTiles];
    bool wok[kTiles];
    pair_rows<MODE>(p, first_pair + fq, wrow, wok);
    const bool chunk_in = wk + ld_chunk * 16 < K;  // only the last window of a ragged K is partial
#pragma unroll
    for (int j = 0; j < kWinLoads; ++j) {
      const int8_t* src = wbase + (int64_t)(wrow[j / 4] + 4 * (j % 4)) * K + wk;
      win.w[j] = chunk_in ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src)) : v4i{0, 0, 0, 0};
    }
    wk += kWinBytes;
    if (wk >= K) {
      wk = 0;
      ++fq;
    }
  };

  // The weights of the first two windows depend on nothing but the expert of the block: they are
  // requested from HBM before the chain of dependent reads (row list -> token -> activation row,
  // or the quantisation of the rows) that the rest of the set-up is.
  const int nwin = (K + kWinBytes - 1) / kWinBytes;
  const int total = npairs * nwin;
  Window<NS> w0, w1;
  if (total > 0) fetch_weights(w0);
  if (total > 1) fetch_weights(w1);

  int nvalid = 0;
  if (count_valid) {
    for (int base = 0; base < p.B; base += kWave) {
      const int slot = base + lane;
      int32_t t;
      if (!kFused && base == 0)
        t = top_id;  // fetched at kernel entry
      else
        t = slot < p.B ? p.sorted_ids[(int64_t)blk * p.B + slot] : -1;
      nvalid += __popcll(__ballot(t >= 0 && t < p.P));
    }
  }

  if constexpr (kFused) {
    static_assert(NS == 1, "one sub-tile per pass");
    const int wave = threadIdx.x / kWave;
    const int row_bytes = K + kFusedRowPad;
    __syncthreads();  // the previous pass is done reading a_lds
    // valid rows are a prefix of the sub-tile: dealt round-robin, the wavefronts share them evenly
#pragma unroll
    for (int i = 0; i < kSub / kWaves; ++i) {
      const int r = i * kWaves + wave;
      const int32_t t = p.sorted_ids[(int64_t)blk * p.B + sub0 * kSub + r];  // wave-uniform
      if (t < 0 || t >= p.P) continue;
      const uint4* in = reinterpret_cast<const uint4*>(p.a_bf16 + (int64_t)t * K);
      const int nvec = K / kQuantVec;
      uint4 v[kFusedMaxK / kQuantVec / kWave];
      float m = 0.0f;
#pragma unroll
      for (int c = 0; c < kFusedMaxK / kQuantVec / kWave; ++c) {
        const int idx = lane + c * kWave;
        v[c] = idx < nvec ? in[idx] : make_uint4(0u, 0u, 0u, 0u);
        m = fmaxf(m, absmax8(v[c]));
      }
      const float absmax = fmaxf(wave_max(m), 1e-10f);
      const float inv = 127.0f / absmax;
      if (lane == 0) s_lds[r] = absmax / 127.0f;
#pragma unroll
      for (int c = 0; c < kFusedMaxK / kQuantVec / kWave; ++c) {
        const int idx = lane + c * kWave;
        if (idx < nvec)
          *reinterpret_cast<uint2*>(a_lds + r * row_bytes + idx * 8) =
              p.round_even ? quant8<true>(v[c], inv) : quant8<false>(v[c], inv);
      }
    }
    __syncthreads();
    if (npairs == 0) return nvalid;
  }

  int32_t tok[NS];
  bool tok_ok[NS];
  const int8_t* ap[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int slot = (sub0 + s) * kSub + col;  // a second sub-tile may lie past the end of a small block
    if (!kFused && (sub0 + s) * kSub < kWave) {
      const int32_t early = __shfl(top_id, slot & (kWave - 1));  // one of the first 64 slots: fetched at kernel entry
      tok[s] = slot < p.B ? early : -1;
    } else
      tok[s] = slot < p.B ? p.sorted_ids[(int64_t)blk * p.B + slot] : -1;
    tok_ok[s] = tok[s] >= 0 && tok[s] < p.P;
    const int64_t arow = tok_ok[s] ? tok[s] / p.row_div : 0;
    ap[s] = kFused ? nullptr : p.a_q + arow * K + grp * 16;
  }
  const char* a_row = a_lds + col * (K + kFusedRowPad) + grp * 16;  // fused: this lane's operand row

  v4i acc[kTiles][NS];
#pragma unroll
  for (int t = 0; t < kTiles; ++t)
#pragma unroll
    for (int s = 0; s < NS; ++s) acc[t][s] = v4i{0, 0, 0, 0};

  auto fetch_rows = [&](Window<NS>& win) {
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int u = 0; u < kWinSteps; ++u) {
        if constexpr (kFused)
          win.a[s][u] = fk + u * kStepK < K ? *reinterpret_cast<const v4i*>(a_row + fk + u * kStepK)
                                             : v4i{0, 0, 0, 0};
        else
          win.a[s][u] = fk + u * kStepK < K ? *reinterpret_cast<const v4i*>(ap[s] + fk + u * kStepK)
                                             : v4i{0, 0, 0, 0};
      }
    fk += kWinBytes;
    if (fk >= K) fk = 0;
  };
  auto fetch = [&](Window<NS>& win) {
    fetch_weights(win);
    fetch_rows(win);
  };

  // Epilogue of one tile pair: lane holds channels wrow[t] + 4 * grp + {0..3} of token tok[s].
  auto finish_pair = [&](int q) {
    int wrow[kTiles];
    bool wok[kTiles];
    pair_rows<MODE>(p, first_pair + q, wrow, wok);
    if constexpr (MODE == kAccI32) {
      int32_t* out = static_cast<int32_t*>(p.out);
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s)
          if (wok[t] && tok_ok[s])
            *reinterpret_cast<v4i*>(out + (int64_t)tok[s] * p.N + wrow[t] + 4 * grp) = acc[t][s];
    } else if constexpr (MODE == kDown) {
      uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (!tok_ok[s]) continue;
        const float as = kFused ? s_lds[col] : p.a_scale[tok[s] / p.row_div];
        const float rw = p.row_weight ? p.row_weight[tok[s]] : 1.0f;
#pragma unroll
        for (int t = 0; t < kTiles; ++t) {
          if (!wok[t]) continue;
          const int n = wrow[t] + 4 * grp;
          const float4 ws = *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + n);
          const int v[4] = {acc[t][s][0], acc[t][s][1], acc[t][s][2], acc[t][s][3]};
          *reinterpret_cast<uint2*>(out + (int64_t)tok[s] * p.N + n) = down_epilogue4(v, as, ws, rw);
        }
      }
    } else {  // kGateUpSilu: tile 0 is gate, tile 1 the matching up rows; out is [P, N / 2]
      uint16_t* out = static_cast<uint16_t*>(p.out);
      const int inter = p.N / 2;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (!tok_ok[s] || !wok[0]) continue;
        const float as = p.a_scale[tok[s] / p.row_div];
        const int n = wrow[0] + 4 * grp;  // gate channel; up channel is n + inter
        const float4 wg = *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + n);
        const float4 wu = *reinterpret_cast<const float4*>(p.w_scale + (int64_t)e * p.N + inter + n);
        const int g[4] = {acc[0][s][0], acc[0][s][1], acc[0][s][2], acc[0][s][3]};
        const int u[4] = {acc[1][s][0], acc[1][s][1], acc[1][s][2], acc[1][s][3]};
        *reinterpret_cast<uint2*>(out + (int64_t)tok[s] * inter + n) = silu_mul_epilogue4(g, u, as, wg, wu);
      }
    }
#pragma unroll
    for (int t = 0; t < kTiles; ++t)
#pragma unroll
      for (int s = 0; s < NS; ++s) acc[t][s] = v4i{0, 0, 0, 0};
  };

  int cq = 0, ck = 0;
  auto consume = [&](const Window<NS>& win) {
#pragma unroll
    for (int j = 0; j < kWinLoads; ++j)
      *reinterpret_cast<v4i*>(wave_lds + j * 1024 + (st_base ^ ((j % 4) * 64))) = win.w[j];
#pragma unroll
    for (int u = 0; u < kWinSteps; ++u) {
      v4i frag[kTiles];
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
        frag[t] = *reinterpret_cast<const v4i*>(wave_lds + t * 4096 + (rd_base ^ (u * 64)));
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s)
          acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(frag[t], win.a[s][u], acc[t][s], 0, 0, 0);
    }
    ck += kWinBytes;
    if (ck >= K) {
      finish_pair(cq);
      ck = 0;
      ++cq;
    }
  };

  fetch_rows(w0);
  for (int i = 0; i < total; i += 2) {
    if (i + 1 < total) {
      if (i > 0) fetch_weights(w1);  // the weights of window 1 were requested up front
      fetch_rows(w1);
    }
    consume(w0);
    if (i + 1 >= total) break;
    if (i + 2 < total) fetch(w0);
    consume(w1);
  }
  return nvalid;
}

// grid.x * grid.y: one workgroup of kWaves wavefronts per kWaves tile pairs and per block of the
// row list's capacity (grid.z: see below).  NS = sub-tiles per pass.
template <int MODE, bool kFused, int NS>
__global__ __launch_bounds__(kThreads, NS == 1 ? 3 : 2) void gemm_stream_kernel(StreamParams p) {
  __shared__ __align__(16) char lds[kWaves * kWaveLds];
  __shared__ __align__(16) char a_lds[kFused ? kSub * (kFusedMaxK + kFusedRowPad) : 16];
  __shared__ float s_lds[kSub];
  // Everything that depends only on the position in the grid is requested together with the number of
  // padded rows, not after it: at kernel entry every such read is a full trip to memory.  (grid.y is the
  // capacity of the row list in blocks, so these reads are inside the arrays whatever is in use.)
  const int npp = *p.npp;
  int e_entry = -1;
  int32_t top_id = -1;
  if constexpr (!kFused) {
    e_entry = p.expert_ids[blockIdx.y];
    const int lane0 = threadIdx.x & (kWave - 1);
    const int64_t slot0 = (int64_t)blockIdx.y * p.B + lane0;
    top_id = lane0 < p.B && slot0 < p.cap ? p.sorted_ids[slot0] : -1;
  }
  const int nblocks = npp / p.B;  // blocks in use: the first ones of the grid's capacity
  const int total_pairs = MODE == kGateUpSilu ? p.N / 2 / 16 : (p.N / 16 + kTiles - 1) / kTiles;
  // Consecutive tile pairs a wavefront streams back to back: one (more wavefronts in flight beat
  // longer streams per wavefront), except where the workgroup quantises the block's rows itself.
  // Every workgroup of a block repeats that quantisation, so there a wavefront takes 2 or 4 pairs
  // once the blocks in use need more wavefronts than the device holds at a time anyway.  Known
  // only here: the number of blocks in use.
  int ppw = 1;
  if constexpr (kFused) {
    const int64_t wanted = (int64_t)nblocks * total_pairs;
    ppw = wanted > 2 * (int64_t)p.wave_capacity ? 4 : wanted > p.wave_capacity ? 2 : 1;
  }
  // With more than one pair per wavefront a block needs fewer workgroups than the grid has for it.
  // The work is then dealt to the workgroups in the order the device dispatches them (x fastest,
  // then y), so that the ones with nothing to do are the last ones and the others spread evenly
  // over the chip's dies and compute units (leaving every block's surplus workgroups idle in place
  // would starve the dies those land on).
  int blk = blockIdx.y, group = blockIdx.x;
  if constexpr (kFused) {
    const int groups = (total_pairs + kWaves * ppw - 1) / (kWaves * ppw);  // workgroups per block
    const uint32_t order = blockIdx.x + gridDim.x * blockIdx.y;  // the launcher keeps grid.x * grid.y below 2^31
    if (order >= (uint32_t)nblocks * (uint32_t)groups) return;
    blk = (int)(order / (uint32_t)groups);
    group = (int)(order - (uint32_t)blk * (uint32_t)groups);
  } else {
    if (blk >= nblocks) return;
  }
  const int e = kFused ? p.expert_ids[blk] : e_entry;
  if (e < 0 || e >= p.E) return;
  const int first_pair = (group * kWaves + threadIdx.x / kWave) * ppw;
  // a wavefront past the last weight rows leaves, unless the workgroup needs it for the quantisation
  if (!kFused && first_pair >= total_pairs) return;
  const int left = total_pairs - first_pair;
  const int npairs = left < 0 ? 0 : left < ppw ? left : ppw;

  char* wave_lds = lds + (threadIdx.x / kWave) * kWaveLds;
  if (gridDim.z > 1) {
    // The passes of a block are spread over grid.z workgroups (they run side by side instead of one
    // after the other, which matters when a few experts hold most rows).  Valid rows are a prefix
    // of the block: a pass whose first row is padding has nothing to do.
    const int sub0 = blockIdx.z * NS;
    if (sub0 * kSub >= p.B) return;
    const int32_t t = p.sorted_ids[(int64_t)blk * p.B + sub0 * kSub];
    if (t < 0 || t >= p.P) return;
    stream_pass<MODE, NS, kFused>(p, blk, e, sub0, first_pair, npairs, wave_lds, false, a_lds, s_lds, top_id);
    return;
  }
  // One workgroup walks all passes; the first one counts the valid rows (a prefix of the block, at
  // least one: the block is in use) to know how many sub-tiles there are.
  const int nvalid = stream_pass<MODE, NS, kFused>(p, blk, e, 0, first_pair, npairs, wave_lds, true, a_lds, s_lds, top_id);
  const int nsub = (nvalid + kSub - 1) / kSub;
  for (int sub0 = NS; sub0 < nsub; sub0 += NS)
    stream_pass<MODE, NS, kFused>(p, blk, e, sub0, first_pair, npairs, wave_lds, false, a_lds, s_lds, top_id);
}

template <int MODE, bool kFused = false>
hipError_t launch_mode(const GemmArgs& a, hipStream_t stream) {
  StreamParams p;
  p.a_bf16 = a.a_bf16;
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
  p.cap = a.sorted_cap;
  const int total_pairs = MODE == kGateUpSilu ? a.n / 2 / 16 : (a.n / 16 + kTiles - 1) / kTiles;
  const int waves = total_pairs;  // the kernel groups pairs per wavefront once it knows the blocks in use
  const int64_t blocks = (a.sorted_cap + a.block_size - 1) / a.block_size;
  if (blocks == 0 || waves == 0) return hipSuccess;
  if (blocks > 65535 || blocks * ((waves + kWaves - 1) / kWaves) >= (1ll << 31)) return hipErrorInvalidValue;
  const bool two = !kFused && a.num_pairs > (int64_t)kPairRowsPerExpert * a.num_experts;
  // Passes per block that can be needed: no expert holds more rows than there are tokens (or pairs,
  // when the caller did not say).  One workgroup per pass once there can be more than one.
  const int ns = two ? 2 : 1;
  const int64_t most_rows = a.max_rows_per_expert > 0 && a.max_rows_per_expert < a.num_pairs ? a.max_rows_per_expert
                                                                                             : a.num_pairs;
  const int64_t rows = most_rows < a.block_size ? most_rows : a.block_size;
  const int passes = kFused ? 1 : (int)((rows + kSub * ns - 1) / (kSub * ns));
  const dim3 grid((unsigned)((waves + kWaves - 1) / kWaves), (unsigned)blocks, (unsigned)(passes > 1 ? passes : 1));
  p.wave_capacity = device_cu_count() * kWaves * (two ? 2 : 3);
  p.round_even = a.a_round_even ? 1 : 0;
  if (two)
    hipLaunchKernelGGL((gemm_stream_kernel<MODE, kFused, kFused ? 1 : 2>), grid, dim3(kThreads), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_stream_kernel<MODE, kFused, 1>), grid, dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

bool gemm_stream_fuses_quant(int k) { return k <= kFusedMaxK; }

hipError_t launch_gemm_stream(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case kGateUpSilu: return launch_mode<kGateUpSilu>(a, stream);
    case kDown:
      if (a.a_bf16) {
        if (a.k > kFusedMaxK || a.row_div != 1) return hipErrorInvalidValue;
        return launch_mode<kDown, true>(a, stream);
      }
      return launch_mode<kDown>(a, stream);
    case kAccI32: return launch_mode<kAccI32>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace moe_i8
