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

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / kWave;  // 16
constexpr int kMaxE = 1024;
constexpr int kSingleMaxP = 8192;         // one workgroup handles up to this many pairs
constexpr int kChunk = 2048;              // pairs per workgroup in the multi-workgroup path

// Rank of this lane among the lower lanes holding the same key, and the number
// of lanes holding it. Lanes with key < 0 are idle.
__device__ inline void wave_match_rank(int key, int& rank, int& count) {
  rank = 0;
  count = 0;
  bool done = key < 0;
  uint64_t pending = __ballot(!done);
  while (pending) {
    const int leader = __builtin_ctzll(pending);
    const int lk = __shfl(key, leader, kWave);
    const uint64_t same = __ballot(!done && key == lk);
    if (!done && key == lk) {
      rank = __builtin_popcountll(same & lanemask_lt());
      count = __builtin_popcountll(same);
      done = true;
    }
    pending &= ~same;
  }
}

// Scatter phase for one chunk. `base[e]` (LDS) holds the sorted row at which
// this chunk's first pair of expert e lands. `wcnt` is LDS scratch [kWaves][E].
__device__ inline void scatter_chunk(const int32_t* __restrict__ ids, int begin, int end, int E,
                                     int steps, int* base, int* wcnt, int32_t* __restrict__ moe_index,
                                     int32_t* __restrict__ sorted_src) {
  const int wave = threadIdx.x >> 6;
  const int lane = lane_id();
  const int wbegin = begin + wave * kWave * steps;
  for (int i = threadIdx.x; i < kWaves * E; i += kThreads) wcnt[i] = 0;
  __syncthreads();
  // per-wave histogram of the wave's slice
  for (int s = 0; s < steps; ++s) {
    const int j = wbegin + s * kWave + lane;
    if (j < end) {
      const int e = ids[j];
      if (static_cast<unsigned>(e) < static_cast<unsigned>(E)) atomicAdd(&wcnt[wave * E + e], 1);
    }
  }
  __syncthreads();
  // exclusive prefix over waves for each expert, offset by the chunk base
  for (int e = threadIdx.x; e < E; e += kThreads) {
    int run = base[e];
    for (int w = 0; w < kWaves; ++w) {
      const int c = wcnt[w * E + e];
      wcnt[w * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
  int* mine = wcnt + wave * E;
  for (int s = 0; s < steps; ++s) {
    const int j = wbegin + s * kWave + lane;
    int key = j < end ? ids[j] : -1;
    if (key >= E) key = -1;  // ids outside [0,E) are skipped: no sorted row
    int rank, count;
    wave_match_rank(key, rank, count);
    if (j < end && key < 0) moe_index[j] = -1;
    if (key >= 0) {
      const int pos = mine[key] + rank;
      moe_index[j] = pos;
      if (sorted_src) sorted_src[pos] = j;
    }
    __builtin_amdgcn_wave_barrier();
    if (key >= 0 && rank == 0) mine[key] += count;  // one lane per distinct expert
    __builtin_amdgcn_wave_barrier();
  }
}

// Exclusive scan of cnt[0..E) by one workgroup; writes lod[0..E] and expert_m.
// `scan` is LDS scratch of kThreads ints. Leaves lod values also in out_base[e].
__device__ inline void scan_experts(int my_count /* thread e < E */, int E, int* scan, int* out_base,
                                    int32_t* __restrict__ lod, int32_t* __restrict__ expert_m) {
  const int t = threadIdx.x;
  scan[t] = t < E ? my_count : 0;
  __syncthreads();
  for (int off = 1; off < kThreads; off <<= 1) {  // Hillis-Steele inclusive scan
    const int v = t >= off ? scan[t - off] : 0;
    __syncthreads();
    scan[t] += v;
    __syncthreads();
  }
  if (t < E) {
    const int excl = scan[t] - my_count;
    out_base[t] = excl;
    lod[t] = excl;
    if (expert_m) expert_m[t] = my_count;
    if (t == E - 1) lod[E] = scan[t];
  }
  __syncthreads();
}

__global__ __launch_bounds__(kThreads) void align_single_kernel(
    const int32_t* __restrict__ ids, int P, int E, int steps, int32_t* __restrict__ moe_index,
    int32_t* __restrict__ sorted_src, int32_t* __restrict__ expert_m, int32_t* __restrict__ lod) {
  extern __shared__ int lds[];
  int* scan = lds;               // [kThreads]
  int* base = scan + kThreads;   // [E]
  int* wcnt = base + E;          // [kWaves][E]
  for (int e = threadIdx.x; e < E; e += kThreads) base[e] = 0;
  __syncthreads();
  for (int j = threadIdx.x; j < P; j += kThreads) {
    const int e = ids[j];
    if (static_cast<unsigned>(e) < static_cast<unsigned>(E)) atomicAdd(&base[e], 1);
  }
  __syncthreads();
  const int mine = threadIdx.x < E ? base[threadIdx.x] : 0;
  __syncthreads();
  scan_experts(mine, E, scan, base, lod, expert_m);
  scatter_chunk(ids, 0, P, E, steps, base, wcnt, moe_index, sorted_src);
}

// Multi-workgroup path, kernel 1: chunk histograms -> hist[chunk][E].
__global__ __launch_bounds__(kThreads) void align_hist_kernel(const int32_t* __restrict__ ids, int P, int E,
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
  __shared__ int scan[kThreads];
  __shared__ int base[kMaxE];
  const int e = threadIdx.x;
  int total = 0;
  if (e < E) {
    for (int c = 0; c < n_chunks; ++c) {
      const int v = hist[static_cast<size_t>(c) * E + e];
      hist[static_cast<size_t>(c) * E + e] = total;
      total += v;
    }
  }
  scan_experts(total, E, scan, base, lod, expert_m);
  if (e < E) {
    const int b = base[e];
    for (int c = 0; c < n_chunks; ++c) hist[static_cast<size_t>(c) * E + e] += b;
  }
}

// Kernel 3: stable scatter of each chunk.
__global__ __launch_bounds__(kThreads) void align_scatter_kernel(const int32_t* __restrict__ ids, int P, int E,
                                                                const int32_t* __restrict__ hist,
                                                                int32_t* __restrict__ moe_index,
                                                                int32_t* __restrict__ sorted_src) {
  extern __shared__ int lds[];
  int* base = lds;       // [E]
  int* wcnt = base + E;  // [kWaves][E]
  for (int e = threadIdx.x; e < E; e += kThreads) base[e] = hist[static_cast<size_t>(blockIdx.x) * E + e];
  __syncthreads();
  const int begin = blockIdx.x * kChunk;
  const int end = min(P, begin + kChunk);
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
  KMOE_REQUIRE(lod && (P == 0 || (topk_ids && moe_index)), KMOE_ERR_NULL, "align: NULL pointer");
  KMOE_REQUIRE(E >= 1 && E <= kMaxE, KMOE_ERR_SHAPE, "align: E=%d outside [1,%d]", E, kMaxE);
  KMOE_REQUIRE(P >= 0 && P <= (1 << 24), KMOE_ERR_SHAPE, "align: P=%d outside [0,2^24]", P);
  hipStream_t s = as_stream(stream);
  if (P <= kSingleMaxP) {
    const int steps = max(1, ceil_div(P, kThreads));
    const size_t lds = sizeof(int) * (kThreads + E + static_cast<size_t>(kWaves) * E);
    hipLaunchKernelGGL(align_single_kernel, dim3(1), dim3(kThreads), lds, s, topk_ids, P, E, steps, moe_index,
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
