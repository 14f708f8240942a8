// moe_align: stable counting sort of routed pairs by expert id, built from LDS
// histograms, a per-expert scan and wavefront ballot ranks.
//
// Decomposition: the P pairs are cut into chunks of kChunk consecutive pairs,
// one workgroup each; inside a chunk wave w owns the next kWave*steps pairs.
// The sorted row of pair j with expert e is
//   lod[e] + (#pairs of e in earlier chunks) + (#pairs of e in earlier waves /
//   steps of this chunk) + (#lower lanes of this step with expert e),
// which is exactly the stable order (ties by ascending j).
#include "kmoe_common.h"

namespace kmoe {
namespace {

constexpr int kThreads = 1024;            // workgroup size of the multi-workgroup kernels
constexpr int kWaves = kThreads / kWave;  // 16
constexpr int kMaxE = 1024;
constexpr int kSingleMaxP = 4096;         // one workgroup handles up to this many pairs
constexpr int kChunk = 2048;              // pairs per workgroup in the multi-workgroup path

__device__ inline int key_bits(int E) { return 32 - __builtin_clz(max(E - 1, 1)); }

// Rank of this lane among the lower lanes holding the same key, and the number
// of lanes holding it. Lanes with key < 0 are idle. One ballot per key bit: the
// lanes whose key agrees with mine on every bit are the lanes with my key.
__device__ inline void wave_match_rank(int key, int bits, int& rank, int& count) {
  const bool live = key >= 0;
  uint64_t same = __ballot(live);
  for (int b = 0; b < bits; ++b) {
    const bool bit = (key >> b) & 1;
    const uint64_t set = __ballot(live && bit);
    same &= bit ? set : ~set;
  }
  rank = live ? __builtin_popcountll(same & lanemask_lt()) : 0;
  count = live ? __builtin_popcountll(same) : 0;
}

// The expert ids of the routed pairs as the routing kernel wrote them, seen by a launch that owns the experts
// [first, first + E) of them (an expert-parallel share; first = 0: all of them): ids outside come out outside [0, E).
struct IdView {
  const int32_t* ids;
  int first;
  __device__ int operator[](int j) const { return ids[j] - first; }
};

__device__ inline int load_key(const IdView ids, int j, int end, int E) {
  if (j >= end) return -1;
  const int e = ids[j];
  return static_cast<unsigned>(e) < static_cast<unsigned>(E) ? e : -1;  // ids outside [0,E): no sorted row
}

// Counting phase for one chunk: wave w owns pairs [begin + w*64*steps, +64*steps).
// Leaves in wcnt[w][e] the number of expert-e pairs of this chunk in waves < w and
// returns to thread e < E the chunk's total for expert e (0 to the other threads).
// `wcnt` is LDS scratch [waves][E].
__device__ inline int count_chunk(const IdView ids, int begin, int end, int E, int steps,
                                  int* wcnt) {
  const int waves = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int bits = key_bits(E);
  const int wbegin = begin + wave * kWave * steps;
  for (int i = threadIdx.x; i < waves * E; i += blockDim.x) wcnt[i] = 0;
  __syncthreads();
  int* mine = wcnt + wave * E;
  for (int s = 0; s < steps; ++s) {
    const int key = load_key(ids, wbegin + s * kWave + lane, end, E);
    int rank, count;
    wave_match_rank(key, bits, rank, count);
    if (key >= 0 && rank == 0) mine[key] += count;  // one lane per distinct expert; a wave's LDS ops stay in order
  }
  __syncthreads();
  int total = 0;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {  // at most one trip: blockDim.x >= E
    for (int w = 0; w < waves; ++w) {
      const int c = wcnt[w * E + e];
      wcnt[w * E + e] = total;
      total += c;
    }
  }
  return total;
}

// Scatter phase: pair j of expert e lands at base[e] + wcnt[wave][e] + (rank among the
// wave's earlier pairs of e). Call after count_chunk and a barrier that publishes base.
__device__ inline void scatter_chunk(const IdView ids, int begin, int end, int E, int steps,
                                     const int* base, int* wcnt, int32_t* __restrict__ moe_index,
                                     int32_t* __restrict__ sorted_src) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int bits = key_bits(E);
  const int wbegin = begin + wave * kWave * steps;
  int* mine = wcnt + wave * E;
  for (int s = 0; s < steps; ++s) {
    const int j = wbegin + s * kWave + lane;
    const int key = load_key(ids, j, end, E);
    int rank, count;
    wave_match_rank(key, bits, rank, count);
    if (j < end && key < 0) moe_index[j] = -1;
    if (key >= 0) {
      const int pos = base[key] + mine[key] + rank;
      moe_index[j] = pos;
      if (sorted_src) sorted_src[pos] = j;
    }
    __builtin_amdgcn_wave_barrier();
    if (key >= 0 && rank == 0) mine[key] += count;
    __builtin_amdgcn_wave_barrier();
  }
}

// Exclusive scan of cnt[0..E) by one workgroup (blockDim.x >= E): a shuffle scan
// inside each wave, then the wave totals through LDS. Writes lod[0..E] and
// expert_m, and leaves lod[e] also in out_base[e]. `wtot` is LDS scratch of 16 ints.
__device__ inline void scan_experts(int my_count /* thread e < E */, int E, int* wtot, int* out_base,
                                    int32_t* __restrict__ lod, int32_t* __restrict__ expert_m) {
  const int t = threadIdx.x;
  const int lane = lane_id();
  int incl = t < E ? my_count : 0;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int o = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += o;
  }
  if (lane == kWave - 1) wtot[t >> 6] = incl;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < (t >> 6); ++w) before += wtot[w];
  if (t < E) {
    const int excl = before + incl - my_count;
    out_base[t] = excl;
    lod[t] = excl;
    if (expert_m) expert_m[t] = my_count;
    if (t == E - 1) lod[E] = before + incl;
  }
  __syncthreads();
}

// Single-workgroup path (P <= kSingleMaxP); blockDim.x is 256 or 1024, >= E.
__global__ __launch_bounds__(kThreads) void align_single_kernel(
    const IdView ids, int P, int E, int steps, int32_t* __restrict__ moe_index,
    int32_t* __restrict__ sorted_src, int32_t* __restrict__ expert_m, int32_t* __restrict__ lod) {
  extern __shared__ int lds[];
  int* wtot = lds;          // [16]
  int* base = wtot + 16;    // [E]
  int* wcnt = base + E;     // [waves][E]
  const int mine = count_chunk(ids, 0, P, E, steps, wcnt);
  scan_experts(mine, E, wtot, base, lod, expert_m);
  scatter_chunk(ids, 0, P, E, steps, base, wcnt, moe_index, sorted_src);
}

// Multi-workgroup path, kernel 1: chunk histograms -> hist[chunk][E].
__global__ __launch_bounds__(kThreads) void align_hist_kernel(const IdView ids, int P, int E,
                                                             int32_t* __restrict__ hist) {
  extern __shared__ int lds[];
  for (int e = threadIdx.x; e < E; e += kThreads) lds[e] = 0;
  __syncthreads();
  const int begin = blockIdx.x * kChunk;
  const int end = min(P, begin + kChunk);
  for (int j = begin + threadIdx.x; j < end; j += kThreads) {
    const int e = ids[j];
    if (static_cast<unsigned>(e) < static_cast<unsigned>(E)) atomicAdd(&lds[e], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kThreads) hist[static_cast<size_t>(blockIdx.x) * E + e] = lds[e];
}

// Kernel 2 (one workgroup): per-expert prefix over chunks, then lod; hist is
// rewritten in place to the sorted row where each chunk's expert-e pairs begin.
__global__ __launch_bounds__(kThreads) void align_scan_kernel(int E, int n_chunks, int32_t* __restrict__ hist,
                                                             int32_t* __restrict__ expert_m,
                                                             int32_t* __restrict__ lod) {
  __shared__ int scan[16];
  __shared__ int base[kMaxE];
  const int e = threadIdx.x;
  int total = 0;
  constexpr int kBatch = 8;  // loads of a batch are independent: one memory round trip per 8 chunks, not per chunk
  if (e < E) {
    for (int c0 = 0; c0 < n_chunks; c0 += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = c0 + i < n_chunks ? hist[static_cast<size_t>(c0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        if (c0 + i < n_chunks) hist[static_cast<size_t>(c0 + i) * E + e] = total;
        total += v[i];
      }
    }
  }
  scan_experts(total, E, scan, base, lod, expert_m);
  if (e < E) {
    const int b = base[e];
    for (int c0 = 0; c0 < n_chunks; c0 += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = c0 + i < n_chunks ? hist[static_cast<size_t>(c0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i)
        if (c0 + i < n_chunks) hist[static_cast<size_t>(c0 + i) * E + e] = v[i] + b;
    }
  }
}

// Kernel 3: stable scatter of each chunk.
__global__ __launch_bounds__(kThreads) void align_scatter_kernel(const IdView ids, int P, int E,
                                                                const int32_t* __restrict__ hist,
                                                                int32_t* __restrict__ moe_index,
                                                                int32_t* __restrict__ sorted_src) {
  extern __shared__ int lds[];
  int* base = lds;       // [E]
  int* wcnt = base + E;  // [kWaves][E]
  for (int e = threadIdx.x; e < E; e += kThreads) base[e] = hist[static_cast<size_t>(blockIdx.x) * E + e];
  const int begin = blockIdx.x * kChunk;
  const int end = min(P, begin + kChunk);
  count_chunk(ids, begin, end, E, kChunk / kThreads, wcnt);
  __syncthreads();
  scatter_chunk(ids, begin, end, E, kChunk / kThreads, base, wcnt, moe_index, sorted_src);
}

__global__ void block_statistic_kernel(const int32_t* __restrict__ ids, int P, int E, int per_block,
                                       int32_t* __restrict__ out) {
  extern __shared__ int lds[];
  for (int e = threadIdx.x; e < E; e += blockDim.x) lds[e] = 0;
  __syncthreads();
  const int begin = blockIdx.x * per_block;
  const int end = min(P, begin + per_block);
  for (int j = begin + threadIdx.x; j < end; j += blockDim.x) {
    const int e = ids[j];
    if (e >= 0 && e < E) atomicAdd(&lds[e], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) out[static_cast<size_t>(blockIdx.x) * E + e] = lds[e];
}

__global__ void gather_rows_kernel(const uint16_t* __restrict__ src, int64_t ld_src,
                                   const int32_t* __restrict__ sorted_src, int K, int H,
                                   uint16_t* __restrict__ dst, int64_t ld_dst) {
  const int r = blockIdx.x;
  const int tok = sorted_src[r] / K;
  const uint4* s = reinterpret_cast<const uint4*>(src + static_cast<size_t>(tok) * ld_src);
  uint4* d = reinterpret_cast<uint4*>(dst + static_cast<size_t>(r) * ld_dst);
  for (int i = threadIdx.x; i < H / 8; i += blockDim.x) d[i] = s[i];
}

}  // namespace
}  // namespace kmoe

using namespace kmoe;

extern "C" size_t kmoe_align_workspace_bytes(int P, int E) {
  if (P <= kSingleMaxP || E <= 0) return 256;  // unused, but never report zero
  return align_up(static_cast<size_t>(ceil_div(P, kChunk)) * E * sizeof(int32_t), 256);
}

extern "C" int kmoe_align(const int32_t* topk_ids, int P, int E, int32_t* moe_index, int32_t* sorted_src,
                          int32_t* expert_m, int32_t* lod, void* workspace, size_t workspace_bytes,
                          kmoe_stream_t stream) {
  return kmoe_align_local(topk_ids, P, E, 0, moe_index, sorted_src, expert_m, lod, workspace, workspace_bytes, stream);
}

extern "C" int kmoe_align_local(const int32_t* ids_global, int P, int E, int first_expert, int32_t* moe_index,
                                int32_t* sorted_src, int32_t* expert_m, int32_t* lod, void* workspace,
                                size_t workspace_bytes, kmoe_stream_t stream) {
  const IdView topk_ids{ids_global, first_expert};
  KMOE_REQUIRE(first_expert >= 0, KMOE_ERR_SHAPE, "align: first_expert=%d", first_expert);
  KMOE_REQUIRE(lod && (P == 0 || (ids_global && moe_index)), KMOE_ERR_NULL, "align: NULL pointer");
  KMOE_REQUIRE(E >= 1 && E <= kMaxE, KMOE_ERR_SHAPE, "align: E=%d outside [1,%d]", E, kMaxE);
  KMOE_REQUIRE(P >= 0 && P <= (1 << 24), KMOE_ERR_SHAPE, "align: P=%d outside [0,2^24]", P);
  hipStream_t s = as_stream(stream);
  if (P <= kSingleMaxP) {
    const int threads = (E <= 256 && P <= 512) ? 256 : kThreads;  // few waves: cheap barriers for decode sizes
    const int steps = max(1, ceil_div(P, threads));
    const size_t lds = sizeof(int) * (16 + E + static_cast<size_t>(threads / kWave) * E);
    hipLaunchKernelGGL(align_single_kernel, dim3(1), dim3(threads), lds, s, topk_ids, P, E, steps, moe_index,
                       sorted_src, expert_m, lod);
    return check_launch("kmoe_align");
  }
  const int n_chunks = ceil_div(P, kChunk);
  const size_t need = static_cast<size_t>(n_chunks) * E * sizeof(int32_t);
  KMOE_REQUIRE(workspace, KMOE_ERR_WORKSPACE, "align: workspace is NULL (need %zu bytes)", need);
  KMOE_REQUIRE(workspace_bytes >= need, KMOE_ERR_WORKSPACE, "align: workspace %zu < %zu bytes", workspace_bytes,
               need);
  int32_t* hist = static_cast<int32_t*>(workspace);
  hipLaunchKernelGGL(align_hist_kernel, dim3(n_chunks), dim3(kThreads), sizeof(int) * E, s, topk_ids, P, E, hist);
  hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(kThreads), 0, s, E, n_chunks, hist, expert_m, lod);
  hipLaunchKernelGGL(align_scatter_kernel, dim3(n_chunks), dim3(kThreads),
                     sizeof(int) * (E + static_cast<size_t>(kWaves) * E), s, topk_ids, P, E, hist, moe_index,
                     sorted_src);
  return check_launch("kmoe_align");
}

extern "C" int kmoe_block_statistic(const int32_t* topk_ids, int P, int E, int n_blocks,
                                    int32_t* block_statistic, kmoe_stream_t stream) {
  KMOE_REQUIRE(topk_ids && block_statistic, KMOE_ERR_NULL, "block_statistic: NULL pointer");
  KMOE_REQUIRE(E >= 1 && E <= 8192, KMOE_ERR_SHAPE, "block_statistic: E=%d outside [1,8192]", E);
  KMOE_REQUIRE(P >= 0 && n_blocks >= 1, KMOE_ERR_SHAPE, "block_statistic: P=%d n_blocks=%d", P, n_blocks);
  const int per_block = max(1, ceil_div(P, n_blocks));
  hipLaunchKernelGGL(block_statistic_kernel, dim3(n_blocks), dim3(256), sizeof(int) * E, as_stream(stream),
                     topk_ids, P, E, per_block, block_statistic);
  return check_launch("kmoe_block_statistic");
}

extern "C" int kmoe_gather_rows(const uint16_t* src, int64_t ld_src, const int32_t* sorted_src, int P, int K,
                                int H, uint16_t* dst, int64_t ld_dst, kmoe_stream_t stream) {
  KMOE_REQUIRE(src && sorted_src && dst, KMOE_ERR_NULL, "gather_rows: NULL pointer");
  KMOE_REQUIRE(P >= 0 && K >= 1 && H >= 8 && H % 8 == 0, KMOE_ERR_SHAPE, "gather_rows: P=%d K=%d H=%d", P, K, H);
  KMOE_REQUIRE(ld_src % 8 == 0 && ld_dst % 8 == 0 && ld_src >= H && ld_dst >= H, KMOE_ERR_SHAPE,
               "gather_rows: row strides %lld/%lld must be multiples of 8 and >= H", (long long)ld_src,
               (long long)ld_dst);
  if (P == 0) return KMOE_OK;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(P), dim3(256), 0, as_stream(stream), src, ld_src, sorted_src, K, H,
                     dst, ld_dst);
  return check_launch("kmoe_gather_rows");
}
