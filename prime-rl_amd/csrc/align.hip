// moe_align_block_size for gfx950: stable counting sort of (token, expert) pairs by expert,
// each expert segment padded to a multiple of the block size.
//
// The unit of work is one 64-lane wavefront walking a contiguous chunk of pairs.  Counting uses
// LDS atomics on counters private to the wavefront (a count has no order).  In the scatter the
// rank of a pair among the lanes that hold the same expert comes from ballots (one per bit of the
// expert id) and a population count below the lane, so the order inside an expert segment is the
// ascending flat pair index whatever order the hardware resolves conflicts in.
//
// Small inputs run in one 1024-thread workgroup (histogram, scans and scatter fused).  Medium
// inputs use two launches: one workgroup counts everything (sixteen chunks, one per wavefront) and
// scans, sixteen workgroups scatter a chunk each.  Large inputs use three launches: per-wave
// histograms, one scan workgroup, scatter.
#include "common.hpp"
#include "quant_body.hpp"

namespace moe_i8 {
namespace {

constexpr int kSingleThreads = 1024;
constexpr int kSingleWaves = kSingleThreads / kWave;
constexpr int kMultiThreads = 256;
constexpr int kMultiWaves = kMultiThreads / kWave;
constexpr int kMultiChunk = 1024;         // pairs per workgroup in the multi-launch path
constexpr int64_t kSingleMaxPairs = 8192;  // above this the multi-launch path is used
constexpr int kSingleIters = (int)(kSingleMaxPairs / kSingleWaves / kWave);  // 64-pair steps per wavefront
// Two-launch path: kSingleWaves chunks, each scattered by one workgroup the way the single workgroup
// handles a whole small input.  Its one counting workgroup is what the first launch waits for; next to
// the quantisation of many rows that costs more than the launch it saves (measured per layer against
// the three-launch path: -2.7 us at 12k pairs, -2.5 at 16k, -1.2 at 24k, -0.3 at 32k, +0.9 at 64k).
constexpr int64_t kChunkedMaxPairs = 4 * kSingleMaxPairs;
constexpr int kMultiIters = kMultiChunk / kMultiWaves / kWave;

// Lanes of this wavefront that are active and hold the same expert id as the caller.
__device__ __forceinline__ uint64_t peers_of(int e, bool active, int nbits) {
  uint64_t m = __ballot(active);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1;
    const uint64_t bm = __ballot(active && bit);
    m &= bit ? bm : ~bm;
  }
  return m;
}

// Expert ids of the pairs [begin, end) this wavefront walks, 64 per iteration, all loads issued
// before the first use (-1 past the end).
template <int kIters>
__device__ __forceinline__ void wave_load_ids(const int32_t* __restrict__ ids, int64_t begin, int64_t end,
                                              int (&e)[kIters]) {
  const int lane = lane_id();
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    const int64_t idx = begin + i * kWave + lane;
    e[i] = idx < end ? ids[idx] : -1;
  }
}

// counts[x] += number of loaded pairs routed to x; counts is private to the wavefront (LDS).  Counting
// needs no order, so it is one LDS atomic per pair (lanes that hit the same counter are serialised by
// the LDS); only the scatter below needs the rank of a pair among its peers.
template <int kIters>
__device__ __forceinline__ void wave_histogram(const int (&ids)[kIters], int64_t count, int E, int* counts) {
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    if ((int64_t)i * kWave >= count) break;  // wave-uniform: nothing left in this wavefront's range
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(counts + e, 1);
  }
}

// The same placement with the peer masks taken from LDS instead of ballots, for a wavefront that shares its
// compute unit with fifteen others: there the ~60 vector instructions per 64 pairs that the ballots and the
// 64-bit per-lane mask arithmetic cost are what bounds the scatter (measured at 8192 pairs in one 1024-thread
// workgroup: 5.3 of 12.8 us).  Every lane ORs its own bit into a 64-bit word of its expert (`masks`, E words
// private to the wavefront, zero on entry and on exit); OR does not depend on the order in which the LDS
// resolves lanes that hit the same word, so the word read back is exactly the ballot-built peer mask.  The
// lowest lane of a group clears the word and advances the expert's cursor with one LDS atomic whose old value
// the group picks up by lane permute.  A wavefront's LDS instructions are carried out in program order, which
// is what makes the read see every lane's OR and keeps the steps of the loop in ascending pair order.
template <int kIters>
__device__ __forceinline__ void wave_scatter_masks(const int (&ids)[kIters], int64_t begin, int64_t count, int E,
                                                   int* cursor, unsigned long long* masks,
                                                   int32_t* __restrict__ sorted, int64_t sorted_cap) {
  const int lane = lane_id();
  const unsigned long long my_bit = 1ull << lane;
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    if ((int64_t)i * kWave >= count) break;
    const int e = ids[i];
    const bool active = e >= 0 && e < E;
    if (active) atomicOr(masks + e, my_bit);
    __builtin_amdgcn_wave_barrier();
    const unsigned long long peers = active ? masks[e] : my_bit;
    __builtin_amdgcn_wave_barrier();
    const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
    int first = 0;
    if (active && rank == 0) {
      masks[e] = 0ull;
      first = atomicAdd(cursor + e, __popcll(peers));
    }
    const int pos = __shfl(first, __ffsll(peers) - 1) + rank;
    if (active && pos < sorted_cap) sorted[pos] = (int32_t)(begin + i * kWave + lane);
  }
}

// sorted[cursor[x]++] = pair index, in ascending pair index per expert.
template <int kIters>
__device__ __forceinline__ void wave_scatter(const int (&ids)[kIters], int64_t begin, int64_t count, int E,
                                             int nbits, int* cursor, int32_t* __restrict__ sorted,
                                             int64_t sorted_cap) {
  const int lane = lane_id();
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    if ((int64_t)i * kWave >= count) break;
    const int e = ids[i];
    const bool active = e >= 0 && e < E;
    const uint64_t peers = peers_of(e, active, nbits);
    const int rank = __popcll(peers & ((1ull << lane) - 1ull));
    int pos = 0;
    if (active) pos = cursor[e] + rank;
    __builtin_amdgcn_wave_barrier();
    if (active && rank == 0) cursor[e] += __popcll(peers);
    __builtin_amdgcn_wave_barrier();
    if (active && pos < sorted_cap) sorted[pos] = (int32_t)(begin + i * kWave + lane);
  }
}

__device__ __forceinline__ int wave_inclusive_scan(int v) { return wave_inclusive_scan_add(v); }

// Exclusive scan over the 1024 threads of the block; returns the exclusive prefix, *total = sum.
__device__ __forceinline__ int block_exclusive_scan_1024(int v, int* wave_sums, int* total) {
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const int incl = wave_inclusive_scan(v);
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  if (wave == 0) {
    const int s = lane < kSingleWaves ? wave_sums[lane] : 0;
    const int si = wave_inclusive_scan(s);
    if (lane < kSingleWaves) wave_sums[lane] = si - s;
    if (lane == kSingleWaves - 1) wave_sums[kSingleWaves] = si;
  }
  __syncthreads();
  *total = wave_sums[kSingleWaves];
  return wave_sums[wave] + incl - v;
}

// From per-expert padded segment starts (seg[0..E], seg[E] = total) write expert_ids.
__device__ __forceinline__ void write_expert_ids(const int* seg, int E, int B, int npp,
                                                 int32_t* __restrict__ expert_ids,
                                                 int64_t expert_cap) {
  for (int64_t j = threadIdx.x; j < expert_cap; j += blockDim.x) {
    const int64_t pos = j * B;
    int e = -1;
    if (pos < npp) {
      // largest e with seg[e] <= pos (an empty expert shares its start with its successor)
      int lo = 0, hi = E - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (seg[mid] <= pos) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    expert_ids[j] = e;
  }
}

// Ints of LDS in front of the peer-mask words, a multiple of two so that those are 8-byte aligned.
__host__ __device__ constexpr size_t single_lds_ints(int E) {
  return ((size_t)kSingleWaves * E + E + 1 + kSingleWaves + 1 + 1) / 2 * 2;
}

// LDS layout: hist[kSingleWaves][E] | seg[E + 1] | wave_sums[kSingleWaves + 1] | with `use_masks`:
// peer masks[kSingleWaves][E] (64-bit)
__device__ __forceinline__ void align_single_body(
    const int32_t* __restrict__ ids, int P, int E, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_cap, int32_t* __restrict__ expert_ids,
    int64_t expert_cap, int32_t* __restrict__ npp_out, int* smem, bool use_masks) {
  int* hist = smem;
  int* seg = hist + kSingleWaves * E;
  int* wave_sums = seg + E + 1;
  unsigned long long* masks = reinterpret_cast<unsigned long long*>(smem + single_lds_ints(E));
  const int tid = threadIdx.x;
  const int wave = tid / kWave;

  for (int i = tid; i < kSingleWaves * E; i += kSingleThreads) hist[i] = 0;
  if (use_masks)
    for (int i = tid; i < kSingleWaves * E; i += kSingleThreads) masks[i] = 0ull;
  for (int64_t i = tid; i < sorted_cap; i += kSingleThreads) sorted[i] = P;
  __syncthreads();

  const int per_wave = ((P + kSingleWaves - 1) / kSingleWaves + kWave - 1) / kWave * kWave;
  const int64_t begin = (int64_t)wave * per_wave < P ? (int64_t)wave * per_wave : P;
  const int64_t end = begin + per_wave < P ? begin + per_wave : P;
  int mine[kSingleIters];
  wave_load_ids(ids, begin, end, mine);
  wave_histogram(mine, end - begin, E, hist + wave * E);
  __syncthreads();

  int padded = 0;
  if (tid < E) {
    int run = 0;
    for (int w = 0; w < kSingleWaves; ++w) {
      const int c = hist[w * E + tid];
      hist[w * E + tid] = run;
      run += c;
    }
    padded = (run + B - 1) / B * B;
  }
  int npp;
  const int start = block_exclusive_scan_1024(padded, wave_sums, &npp);
  if (tid < E) seg[tid] = start;
  if (tid == 0) {
    seg[E] = npp;
    *npp_out = npp;
  }
  __syncthreads();
  if (tid < E)
    for (int w = 0; w < kSingleWaves; ++w) hist[w * E + tid] += start;
  write_expert_ids(seg, E, B, npp, expert_ids, expert_cap);
  __syncthreads();
  if (use_masks)
    wave_scatter_masks(mine, begin, end - begin, E, hist + wave * E, masks + wave * E, sorted, sorted_cap);
  else
    wave_scatter(mine, begin, end - begin, E, nbits, hist + wave * E, sorted, sorted_cap);
}

__global__ __launch_bounds__(kSingleThreads) void align_single_kernel(
    const int32_t* __restrict__ ids, int P, int E, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_cap, int32_t* __restrict__ expert_ids,
    int64_t expert_cap, int32_t* __restrict__ npp_out, int use_masks) {
  extern __shared__ int smem[];
  align_single_body(ids, P, E, B, nbits, sorted, sorted_cap, expert_ids, expert_cap, npp_out, smem, use_masks != 0);
}

// One launch for small batches: workgroup 0 runs moe_align, every other workgroup quantises 16
// activation rows (one per wavefront).  The two halves are independent.
template <int VPL>
__global__ __launch_bounds__(kSingleThreads) void align_quant_kernel(
    const int32_t* __restrict__ ids, int P, int E, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_cap, int32_t* __restrict__ expert_ids,
    int64_t expert_cap, int32_t* __restrict__ npp_out, int use_masks, QuantArgs q) {
  extern __shared__ int smem[];
  if (blockIdx.x == 0) {
    align_single_body(ids, P, E, B, nbits, sorted, sorted_cap, expert_ids, expert_cap, npp_out, smem, use_masks != 0);
    return;
  }
  const int64_t row = (int64_t)(blockIdx.x - 1) * kSingleWaves + threadIdx.x / kWave;
  if (row < q.rows) quant_one_row<VPL>(q, row);
}

// ---- multi-launch path -------------------------------------------------------------------
// One 256-thread workgroup per unit of kMultiChunk pairs; wavefront w of a unit walks the w-th
// quarter.  workspace: unit_hist[units][E] | unit_base[units][E] | seg[E + 1]

// smem[w][e] = number of pairs of wavefront w's quarter routed to e
__device__ __forceinline__ void unit_wave_histograms(const int (&mine)[kMultiIters], int64_t count, int E,
                                                     int* smem) {
  const int tid = threadIdx.x;
  for (int i = tid; i < kMultiWaves * E; i += kMultiThreads) smem[i] = 0;
  __syncthreads();
  wave_histogram(mine, count, E, smem + (tid / kWave) * E);
  __syncthreads();
}

__global__ __launch_bounds__(kMultiThreads) void align_hist_kernel(
    const int32_t* __restrict__ ids, int64_t P, int E, int32_t* __restrict__ unit_hist,
    int32_t* __restrict__ sorted, int64_t sorted_cap) {
  extern __shared__ int smem[];
  const int tid = threadIdx.x;
  const int64_t begin = (int64_t)blockIdx.x * kMultiChunk + (tid / kWave) * (kMultiChunk / kMultiWaves);
  const int64_t end = begin + kMultiChunk / kMultiWaves < P ? begin + kMultiChunk / kMultiWaves : P;
  int mine[kMultiIters];
  wave_load_ids(ids, begin, end, mine);
  for (int64_t i = (int64_t)blockIdx.x * kMultiThreads + tid; i < sorted_cap;
       i += (int64_t)gridDim.x * kMultiThreads)
    sorted[i] = (int32_t)P;
  unit_wave_histograms(mine, end - begin, E, smem);
  for (int e = tid; e < E; e += kMultiThreads) {
    int sum = 0;
#pragma unroll
    for (int w = 0; w < kMultiWaves; ++w) sum += smem[w * E + e];
    unit_hist[(int64_t)blockIdx.x * E + e] = sum;
  }
}

__device__ __forceinline__ void align_scan_body(
    int E, int B, int units, const int32_t* __restrict__ unit_hist, int32_t* __restrict__ unit_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ expert_ids, int64_t expert_cap,
    int32_t* __restrict__ npp_out) {
  __shared__ int seg[kMaxExperts + 1];
  __shared__ int wave_sums[kSingleWaves + 1];
  const int tid = threadIdx.x;
  int padded = 0;
  if (tid < E) {
    int run = 0;
#pragma unroll 8
    for (int u = 0; u < units; ++u) {
      const int c = unit_hist[(int64_t)u * E + tid];
      unit_base[(int64_t)u * E + tid] = run;
      run += c;
    }
    padded = (run + B - 1) / B * B;
  }
  int npp;
  const int start = block_exclusive_scan_1024(padded, wave_sums, &npp);
  if (tid < E) {
    seg[tid] = start;
    seg_out[tid] = start;
  }
  if (tid == 0) {
    seg[E] = npp;
    seg_out[E] = npp;
    *npp_out = npp;
  }
  __syncthreads();
  write_expert_ids(seg, E, B, npp, expert_ids, expert_cap);
}

__global__ __launch_bounds__(kSingleThreads) void align_scan_kernel(
    int E, int B, int units, const int32_t* __restrict__ unit_hist, int32_t* __restrict__ unit_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ expert_ids, int64_t expert_cap,
    int32_t* __restrict__ npp_out) {
  align_scan_body(E, B, units, unit_hist, unit_base, seg_out, expert_ids, expert_cap, npp_out);
}

// The scan is one workgroup; the quantisation of the layer input, which does not depend on the
// routing, fills the rest of the machine in the same launch (workgroups >= 1, 16 rows each).
template <int VPL>
__global__ __launch_bounds__(kSingleThreads) void align_scan_quant_kernel(
    int E, int B, int units, const int32_t* __restrict__ unit_hist, int32_t* __restrict__ unit_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ expert_ids, int64_t expert_cap,
    int32_t* __restrict__ npp_out, QuantArgs q) {
  if (blockIdx.x == 0) {
    align_scan_body(E, B, units, unit_hist, unit_base, seg_out, expert_ids, expert_cap, npp_out);
    return;
  }
  const int64_t row = (int64_t)(blockIdx.x - 1) * kSingleWaves + threadIdx.x / kWave;
  if (row < q.rows) quant_one_row<VPL>(q, row);
}

__global__ __launch_bounds__(kMultiThreads) void align_scatter_kernel(
    const int32_t* __restrict__ ids, int64_t P, int E, int nbits, const int32_t* __restrict__ unit_base,
    const int32_t* __restrict__ seg, int32_t* __restrict__ sorted, int64_t sorted_cap) {
  extern __shared__ int smem[];
  const int tid = threadIdx.x;
  const int64_t begin = (int64_t)blockIdx.x * kMultiChunk + (tid / kWave) * (kMultiChunk / kMultiWaves);
  const int64_t end = begin + kMultiChunk / kMultiWaves < P ? begin + kMultiChunk / kMultiWaves : P;
  int mine[kMultiIters];
  wave_load_ids(ids, begin, end, mine);
  unit_wave_histograms(mine, end - begin, E, smem);
  // counts -> write cursors: segment start + pairs of earlier units + pairs of earlier wavefronts
  for (int e = tid; e < E; e += kMultiThreads) {
    int run = seg[e] + unit_base[(int64_t)blockIdx.x * E + e];
#pragma unroll
    for (int w = 0; w < kMultiWaves; ++w) {
      const int c = smem[w * E + e];
      smem[w * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
  wave_scatter(mine, begin, end - begin, E, nbits, smem + (tid / kWave) * E, sorted, sorted_cap);
}

// ---- two-launch path ---------------------------------------------------------------------
// Pairs per chunk: a sixteenth of the input, rounded up to whole 64-pair steps.
__device__ __host__ __forceinline__ int64_t chunk_pairs(int64_t P) {
  return ((P + kSingleWaves - 1) / kSingleWaves + kWave - 1) / kWave * kWave;
}

// sorted[i] = P (the padding sentinel) for this workgroup's share of the array.
__device__ __forceinline__ void fill_sentinel(int32_t* __restrict__ sorted, int64_t sorted_cap, int64_t P, int part,
                                              int parts) {
  const int64_t per = (sorted_cap + parts - 1) / parts;
  const int64_t lo = (int64_t)part * per;
  const int64_t hi = lo + per < sorted_cap ? lo + per : sorted_cap;
  for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) sorted[i] = (int32_t)P;
}

// One workgroup: wavefront w counts chunk w, then the scans.  chunk_base[w][e] = pairs of expert e in
// chunks before w.  LDS layout as the single-workgroup kernel.
__device__ __forceinline__ void align_count_body(
    const int32_t* __restrict__ ids, int64_t P, int E, int B, int32_t* __restrict__ chunk_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ expert_ids, int64_t expert_cap,
    int32_t* __restrict__ npp_out, int* smem) {
  int* hist = smem;
  int* seg = hist + kSingleWaves * E;
  int* wave_sums = seg + E + 1;
  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = lane_id();
  for (int i = tid; i < kSingleWaves * E; i += kSingleThreads) hist[i] = 0;
  __syncthreads();
  const int64_t chunk = chunk_pairs(P);
  const int64_t begin = wave * chunk < P ? wave * chunk : P;
  const int64_t end = begin + chunk < P ? begin + chunk : P;
  int* counts = hist + wave * E;
  // sixteen loads in flight per wavefront: next to the quantisation in the other workgroups a load
  // takes microseconds, and this workgroup is the one the launch waits for
  constexpr int kBatch = 16;
  for (int64_t base = begin; base < end; base += kBatch * kWave) {
    int e[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const int64_t idx = base + i * kWave + lane;
      e[i] = idx < end ? ids[idx] : -1;
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i)
      if (e[i] >= 0 && e[i] < E) atomicAdd(counts + e[i], 1);
  }
  __syncthreads();
  int padded = 0;
  if (tid < E) {
    int run = 0;
    for (int w = 0; w < kSingleWaves; ++w) {
      chunk_base[w * E + tid] = run;
      run += hist[w * E + tid];
    }
    padded = (run + B - 1) / B * B;
  }
  int npp;
  const int start = block_exclusive_scan_1024(padded, wave_sums, &npp);
  if (tid < E) {
    seg[tid] = start;
    seg_out[tid] = start;
  }
  if (tid == 0) {
    seg[E] = npp;
    seg_out[E] = npp;
    *npp_out = npp;
  }
  __syncthreads();
  write_expert_ids(seg, E, B, npp, expert_ids, expert_cap);
}

// Workgroup 0 counts and scans; the others write the padding sentinel.
__global__ __launch_bounds__(kSingleThreads) void align_count_kernel(
    const int32_t* __restrict__ ids, int64_t P, int E, int B, int32_t* __restrict__ chunk_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ sorted, int64_t sorted_cap,
    int32_t* __restrict__ expert_ids, int64_t expert_cap, int32_t* __restrict__ npp_out) {
  extern __shared__ int smem[];
  if (blockIdx.x == 0)
    align_count_body(ids, P, E, B, chunk_base, seg_out, expert_ids, expert_cap, npp_out, smem);
  else
    fill_sentinel(sorted, sorted_cap, P, (int)blockIdx.x - 1, (int)gridDim.x - 1);
}

// The same with the quantisation of the layer input, which does not depend on the routing, in the
// other workgroups (16 rows each, then their share of the sentinel).
template <int VPL>
__global__ __launch_bounds__(kSingleThreads) void align_count_quant_kernel(
    const int32_t* __restrict__ ids, int64_t P, int E, int B, int32_t* __restrict__ chunk_base,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ sorted, int64_t sorted_cap,
    int32_t* __restrict__ expert_ids, int64_t expert_cap, int32_t* __restrict__ npp_out, QuantArgs q) {
  extern __shared__ int smem[];
  if (blockIdx.x == 0) {
    align_count_body(ids, P, E, B, chunk_base, seg_out, expert_ids, expert_cap, npp_out, smem);
    return;
  }
  const int64_t row = (int64_t)(blockIdx.x - 1) * kSingleWaves + threadIdx.x / kWave;
  if (row < q.rows) quant_one_row<VPL>(q, row);
  fill_sentinel(sorted, sorted_cap, P, (int)blockIdx.x - 1, (int)gridDim.x - 1);
}

// Workgroup c scatters chunk c: its sixteen wavefronts walk a sixteenth of the chunk each.
__global__ __launch_bounds__(kSingleThreads) void align_scatter_chunk_kernel(
    const int32_t* __restrict__ ids, int64_t P, int E, int nbits, const int32_t* __restrict__ chunk_base,
    const int32_t* __restrict__ seg, int32_t* __restrict__ sorted, int64_t sorted_cap) {
  extern __shared__ int smem[];
  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int64_t chunk = chunk_pairs(P);
  const int64_t cb = (int64_t)blockIdx.x * chunk < P ? (int64_t)blockIdx.x * chunk : P;
  const int64_t ce = cb + chunk < P ? cb + chunk : P;
  const int64_t per_wave = (chunk / kSingleWaves + kWave - 1) / kWave * kWave;  // at most kSingleIters steps
  const int64_t begin = cb + wave * per_wave < ce ? cb + wave * per_wave : ce;
  const int64_t end = begin + per_wave < ce ? begin + per_wave : ce;
  int mine[kSingleIters];
  wave_load_ids(ids, begin, end, mine);
  for (int i = tid; i < kSingleWaves * E; i += kSingleThreads) smem[i] = 0;
  __syncthreads();
  wave_histogram(mine, end - begin, E, smem + wave * E);
  __syncthreads();
  // counts -> write cursors: segment start + pairs of earlier chunks + pairs of earlier wavefronts
  if (tid < E) {
    int run = seg[tid] + chunk_base[(int64_t)blockIdx.x * E + tid];
    for (int w = 0; w < kSingleWaves; ++w) {
      const int c = smem[w * E + tid];
      smem[w * E + tid] = run;
      run += c;
    }
  }
  __syncthreads();
  wave_scatter(mine, begin, end - begin, E, nbits, smem + wave * E, sorted, sorted_cap);
}

int bits_for(int E) {
  int b = 0;
  while ((1 << b) < E) ++b;
  return b;
}

}  // namespace

int64_t align_workspace_ints(int64_t num_pairs, int num_experts) {
  if (num_pairs <= kSingleMaxPairs) return 0;
  const int64_t units = (num_pairs + kMultiChunk - 1) / kMultiChunk;
  return 2 * units * num_experts + num_experts + 1;
}

// Launches launch_align (and launch_align_quant) make for this many pairs.
int align_launches(const AlignArgs& a) {
  return a.num_pairs <= kSingleMaxPairs ? 1 : a.num_pairs <= kChunkedMaxPairs ? 2 : 3;
}

bool align_quant_fusable(const AlignArgs& a, const QuantArgs& q) {
  if (q.rows <= 0 || q.rows > (int64_t)kSingleWaves * 0x7ffffff0) return false;
  return a.num_pairs > kSingleMaxPairs || q.rows <= kSingleMaxPairs;
}

namespace {
size_t single_lds_bytes(int E) { return sizeof(int) * ((size_t)kSingleWaves * E + E + 1 + kSingleWaves + 1); }
// The single-workgroup kernel with its peer masks in LDS: used while they fit beside the histograms and while
// there is more than one 64-pair step per wavefront to rank (otherwise there is nothing to gain).
constexpr int kMaskMaxExperts = 256;
bool single_uses_masks(int E, int64_t num_pairs) { return E <= kMaskMaxExperts && num_pairs > kSingleWaves * kWave; }
size_t single_masks_lds_bytes(int E) { return sizeof(int) * single_lds_ints(E) + sizeof(unsigned long long) * kSingleWaves * (size_t)E; }
constexpr int kSingleMasksLdsMax = (int)(sizeof(int) * single_lds_ints(kMaskMaxExperts) + sizeof(unsigned long long) * kSingleWaves * (size_t)kMaskMaxExperts);
constexpr int kSingleLdsMax = (int)(sizeof(int) * ((size_t)kSingleWaves * kMaxExperts + kMaxExperts + kSingleWaves + 2));

// The kernels of the two-launch path may need more dynamic LDS than the default limit (1024 experts).
hipError_t set_chunked_lds_limits() {
  hipError_t err = hipFuncSetAttribute((const void*)align_count_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       kSingleLdsMax);
  if (err != hipSuccess) return err;
#define MOE_I8_LIMIT(V)                                                                              \
  err = hipFuncSetAttribute((const void*)align_count_quant_kernel<V>,                                \
                            hipFuncAttributeMaxDynamicSharedMemorySize, kSingleLdsMax);              \
  if (err != hipSuccess) return err
  MOE_I8_LIMIT(0);
  MOE_I8_LIMIT(1);
  MOE_I8_LIMIT(2);
  MOE_I8_LIMIT(4);
  MOE_I8_LIMIT(8);
#undef MOE_I8_LIMIT
  return hipFuncSetAttribute((const void*)align_scatter_chunk_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                             kSingleLdsMax);
}

hipError_t launch_scatter_chunks(const AlignArgs& a, const int32_t* chunk_base, const int32_t* seg,
                                 hipStream_t stream) {
  const int E = a.num_experts;
  hipLaunchKernelGGL(align_scatter_chunk_kernel, dim3(kSingleWaves), dim3(kSingleThreads),
                     sizeof(int) * (size_t)kSingleWaves * E, stream, a.topk_ids, a.num_pairs, E, bits_for(E),
                     chunk_base, seg, a.sorted_token_ids, a.sorted_cap);
  return hipGetLastError();
}
}  // namespace

// The fused kernels are 1024-thread workgroups (the aligning one needs them), which caps a thread at
// 128 registers: a row held in 16 vectors per lane would spill (measured: 33 us instead of 6 us for 64
// rows of 7168), so rows that long take the variant that reads the row twice, the second time from
// the cache (the `default` of the switches below).
hipError_t launch_align_quant(const AlignArgs& a, const QuantArgs& q, hipStream_t stream) {
  const int E = a.num_experts;
  const dim3 grid(1 + (unsigned)((q.rows + kSingleWaves - 1) / kSingleWaves));
  if (a.num_pairs > kSingleMaxPairs && a.num_pairs <= kChunkedMaxPairs) {
    // two launches as launch_align, the first one (a single counting workgroup) also quantises
    static const hipError_t attr = set_chunked_lds_limits();
    if (attr != hipSuccess) return attr;
    int32_t* chunk_base = a.workspace;
    int32_t* seg = chunk_base + (int64_t)kSingleWaves * E;
#define MOE_I8_COUNT_QUANT(V)                                                                               \
  hipLaunchKernelGGL(align_count_quant_kernel<V>, grid, dim3(kSingleThreads), single_lds_bytes(E), stream,  \
                     a.topk_ids, a.num_pairs, E, a.block_size, chunk_base, seg, a.sorted_token_ids,         \
                     a.sorted_cap, a.expert_ids, a.expert_cap, a.num_tokens_post_padded, q)
    switch (quant_vectors_per_lane(q.cols)) {
      case 1: MOE_I8_COUNT_QUANT(1); break;
      case 2: MOE_I8_COUNT_QUANT(2); break;
      case 4: MOE_I8_COUNT_QUANT(4); break;
      case 8: MOE_I8_COUNT_QUANT(8); break;
      default: MOE_I8_COUNT_QUANT(0); break;
    }
#undef MOE_I8_COUNT_QUANT
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    return launch_scatter_chunks(a, chunk_base, seg, stream);
  }
  if (a.num_pairs > kSingleMaxPairs) {
    // three launches as launch_align, the middle one (a single scanning workgroup) also quantises
    const int nbits = bits_for(E);
    const int units = (int)((a.num_pairs + kMultiChunk - 1) / kMultiChunk);
    int32_t* unit_hist = a.workspace;
    int32_t* unit_base = unit_hist + (int64_t)units * E;
    int32_t* seg = unit_base + (int64_t)units * E;
    const size_t lds = sizeof(int) * (size_t)kMultiWaves * E;
    hipLaunchKernelGGL(align_hist_kernel, dim3(units), dim3(kMultiThreads), lds, stream, a.topk_ids,
                       a.num_pairs, E, unit_hist, a.sorted_token_ids, a.sorted_cap);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
#define MOE_I8_SCAN_QUANT(V)                                                                           \
  hipLaunchKernelGGL(align_scan_quant_kernel<V>, grid, dim3(kSingleThreads), 0, stream, E, a.block_size, \
                     units, unit_hist, unit_base, seg, a.expert_ids, a.expert_cap, a.num_tokens_post_padded, q)
    switch (quant_vectors_per_lane(q.cols)) {
      case 1: MOE_I8_SCAN_QUANT(1); break;
      case 2: MOE_I8_SCAN_QUANT(2); break;
      case 4: MOE_I8_SCAN_QUANT(4); break;
      case 8: MOE_I8_SCAN_QUANT(8); break;
      default: MOE_I8_SCAN_QUANT(0); break;
    }
#undef MOE_I8_SCAN_QUANT
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(align_scatter_kernel, dim3(units), dim3(kMultiThreads), lds, stream,
                       a.topk_ids, a.num_pairs, E, nbits, unit_base, seg, a.sorted_token_ids,
                       a.sorted_cap);
    return hipGetLastError();
  }
  const bool use_masks = single_uses_masks(E, a.num_pairs);
  const size_t lds_bytes = use_masks ? single_masks_lds_bytes(E) : single_lds_bytes(E);
#define MOE_I8_FUSED_LAUNCH(V)                                                                      \
  do {                                                                                              \
    static const hipError_t attr = hipFuncSetAttribute(                                             \
        (const void*)align_quant_kernel<V>, hipFuncAttributeMaxDynamicSharedMemorySize,             \
        kSingleLdsMax > kSingleMasksLdsMax ? kSingleLdsMax : kSingleMasksLdsMax);                   \
    if (attr != hipSuccess) return attr;                                                            \
    hipLaunchKernelGGL(align_quant_kernel<V>, grid, dim3(kSingleThreads), lds_bytes,                \
                       stream, a.topk_ids, (int)a.num_pairs, E, a.block_size, bits_for(E),          \
                       a.sorted_token_ids, a.sorted_cap, a.expert_ids, a.expert_cap,                \
                       a.num_tokens_post_padded, use_masks ? 1 : 0, q);                             \
  } while (0)
  switch (quant_vectors_per_lane(q.cols)) {
    case 1: MOE_I8_FUSED_LAUNCH(1); break;
    case 2: MOE_I8_FUSED_LAUNCH(2); break;
    case 4: MOE_I8_FUSED_LAUNCH(4); break;
    case 8: MOE_I8_FUSED_LAUNCH(8); break;
    default: MOE_I8_FUSED_LAUNCH(0); break;
  }
#undef MOE_I8_FUSED_LAUNCH
  return hipGetLastError();
}

hipError_t launch_align(const AlignArgs& a, hipStream_t stream) {
  const int E = a.num_experts;
  const int nbits = bits_for(E);
  if (a.num_pairs <= kSingleMaxPairs) {
    const bool use_masks = single_uses_masks(E, a.num_pairs);
    const size_t lds = use_masks ? single_masks_lds_bytes(E) : single_lds_bytes(E);
    static const hipError_t attr = hipFuncSetAttribute(
        (const void*)align_single_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
        kSingleLdsMax > kSingleMasksLdsMax ? kSingleLdsMax : kSingleMasksLdsMax);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(align_single_kernel, dim3(1), dim3(kSingleThreads), lds, stream, a.topk_ids,
                       (int)a.num_pairs, E, a.block_size, nbits, a.sorted_token_ids, a.sorted_cap,
                       a.expert_ids, a.expert_cap, a.num_tokens_post_padded, use_masks ? 1 : 0);
    return hipGetLastError();
  }
  if (a.num_pairs <= kChunkedMaxPairs) {
    static const hipError_t attr = set_chunked_lds_limits();
    if (attr != hipSuccess) return attr;
    int32_t* chunk_base = a.workspace;
    int32_t* seg = chunk_base + (int64_t)kSingleWaves * E;
    // one counting workgroup and enough others to write the sentinel in about the same time
    const int fillers = (int)((a.sorted_cap + 16383) / 16384);
    hipLaunchKernelGGL(align_count_kernel, dim3(1 + fillers), dim3(kSingleThreads), single_lds_bytes(E), stream,
                       a.topk_ids, a.num_pairs, E, a.block_size, chunk_base, seg, a.sorted_token_ids, a.sorted_cap,
                       a.expert_ids, a.expert_cap, a.num_tokens_post_padded);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    return launch_scatter_chunks(a, chunk_base, seg, stream);
  }
  const int units = (int)((a.num_pairs + kMultiChunk - 1) / kMultiChunk);
  int32_t* unit_hist = a.workspace;
  int32_t* unit_base = unit_hist + (int64_t)units * E;
  int32_t* seg = unit_base + (int64_t)units * E;
  const size_t lds = sizeof(int) * (size_t)kMultiWaves * E;
  hipLaunchKernelGGL(align_hist_kernel, dim3(units), dim3(kMultiThreads), lds, stream, a.topk_ids,
                     a.num_pairs, E, unit_hist, a.sorted_token_ids, a.sorted_cap);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(kSingleThreads), 0, stream, E, a.block_size,
                     units, unit_hist, unit_base, seg, a.expert_ids, a.expert_cap,
                     a.num_tokens_post_padded);
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(align_scatter_kernel, dim3(units), dim3(kMultiThreads), lds, stream,
                     a.topk_ids, a.num_pairs, E, nbits, unit_base, seg, a.sorted_token_ids,
                     a.sorted_cap);
  return hipGetLastError();
}

}  // namespace moe_i8
