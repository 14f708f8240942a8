// MFMA-bound W8A8 grouped GEMM for the prefill regime (hundreds of rows per
// expert), v_mfma_i32_16x16x64_i8, tiled int8 weights.
//
// Workgroup = 4 waves on a 128-row x 256-channel tile; each wave owns 64 channels
// of all 128 rows: 8 x 4 accumulator fragments = 128 registers. Two workgroups
// share a CU (2 waves per SIMD): one workgroup's LDS/L2 waits, barriers and its
// VALU-heavy epilogue (dequant, exp, divide) run under the other's MFMAs.
//   activations: global (rows gathered through the sort) -> registers -> LDS,
//                128 bytes of K per row and chunk, double-buffered, pitch 160 B
//                (measured: fragment reads at full LDS rate; pitch 144 costs 60% more);
//                every A fragment read from LDS feeds 4 MFMAs.
//   weights:     straight from L2 into registers, 1 KB of consecutive bytes per
//                fragment and MFMA step (tiled layout), through a ring of 4 step
//                buffers loaded 3 MFMA steps (~1 us) ahead of use; every B fragment
//                feeds 8 MFMAs. No weight byte goes through LDS.
// Per CU and clock that is 64 B of LDS reads and 32 B of L2 reads against 8192
// int8 operations.
// Tiles are found from lod by a wave scan (no host-side work list, so routing skew
// is balanced inside one launch), and workgroup ids are re-mapped so that the
// tiles sharing an expert's weights run on the same XCD (one L2).
#include "kmoe_common.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over [base, base + 4 GiB): loads take a 32-bit per-lane offset
// plus a scalar offset, so no 64-bit address arithmetic sits in the MFMA loop.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
__device__ inline v4i buffer_load16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t wave_off) {
  return (v4i)__builtin_amdgcn_raw_buffer_load_b128(r, lane_off, wave_off, 0);
}

constexpr int kMF = 8, kNF = 4, kWavesT = 4;
constexpr int kTM = 16 * kMF;              // 128 rows
constexpr int kThreads = kWavesT * kWave;  // 256
constexpr int kChunk = 128;                // bytes of K per row and chunk (2 MFMA steps)
constexpr int kSteps = kChunk / 64;
constexpr int kPitchT = kChunk + 32;       // 160 B: measured conflict-free for the b128 fragment reads (144 is not)
constexpr int kGroupTiles = 4;              // consecutive m-tiles kept on one XCD
constexpr int kNA = kTM * (kChunk / 16) / kThreads;  // 16-byte activation vectors per thread and chunk (= 4)

struct TiledParams {
  const int8_t* a;
  int64_t lda;
  const float* a_max;
  const int32_t* row_src;
  int32_t src_div;
  const int8_t* w;  // tiled
  const float* w_max;
  const int32_t* lod;
  int32_t E, n, k;
  uint16_t* y;
  int64_t ldy;
  int32_t* acc_out;
  const int8_t* w_tail;
  const float* w_max_tail;
  int32_t tail_row0, tail_rows, tail_src0;
  int32_t n_blocks;   // channel blocks per tile
  int32_t max_tiles;  // upper bound of m-tiles (grid = n_blocks * max_tiles, rounded up to 8)
};

__device__ inline int t_rows_begin(const TiledParams& p, int e) { return e < p.E ? p.lod[e] : p.tail_row0; }
__device__ inline int t_rows_end(const TiledParams& p, int e) {
  return e < p.E ? p.lod[e + 1] : p.tail_row0 + p.tail_rows;
}

__device__ inline int t_incl_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int o = __shfl_up(v, off, kWave);
    if (lane >= off) v += o;
  }
  return v;
}

__device__ inline bool t_locate(const TiledParams& p, int t, int& e_out, int& row0_out) {
  const int lane = lane_id();
  const int E = p.E + (p.w_tail ? 1 : 0);
  const int epl = (E + kWave - 1) / kWave;
  const int e_begin = lane * epl;
  int local = 0;
  for (int i = 0; i < epl; ++i) {
    const int e = e_begin + i;
    if (e < E) local += (t_rows_end(p, e) - t_rows_begin(p, e) + kTM - 1) / kTM;
  }
  const int incl = t_incl_scan(local);
  const int total = __shfl(incl, kWave - 1, kWave);
  if (t >= total) return false;
  int excl = incl - local;
  int found_e = -1, found_row = 0;
  if (t >= excl && t < incl) {
    for (int i = 0; i < epl; ++i) {
      const int e = e_begin + i;
      if (e >= E) break;
      const int lo = t_rows_begin(p, e);
      const int tiles = (t_rows_end(p, e) - lo + kTM - 1) / kTM;
      if (t < excl + tiles) {
        found_e = e;
        found_row = lo + (t - excl) * kTM;
        break;
      }
      excl += tiles;
    }
  }
  const uint64_t who = __ballot(found_e >= 0);
  const int src_lane = __builtin_ctzll(who);
  e_out = __shfl(found_e, src_lane, kWave);
  row0_out = __shfl(found_row, src_lane, kWave);
  return true;
}

template <bool SWIGLU>
__global__ __launch_bounds__(kThreads, 2) void tiled_gemm_i8_kernel(const TiledParams p) {
  constexpr int NFH = SWIGLU ? kNF / 2 : kNF;
  __shared__ __attribute__((aligned(16))) int8_t lds_a[2][kTM * kPitchT];

  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;

  // Workgroups are dealt round-robin to the 8 XCDs. Re-map ids so that a run of
  // kGroupTiles consecutive tiles (about one expert: same weights) lands on ONE XCD
  // and its L2, while successive runs still rotate over the XCDs (the empty tiles at
  // the end of the list are then spread over all of them).
  const int run = p.n_blocks * kGroupTiles;  // workgroups per run; gridDim.x is a multiple of 8 * run
  const int xcd = blockIdx.x & 7;
  const int j = blockIdx.x >> 3;             // index among this XCD's workgroups
  const int lid = ((j / run) * 8 + xcd) * run + j % run;
  const int tile = lid / p.n_blocks;
  const int nb = lid - tile * p.n_blocks;
  if (tile >= p.max_tiles) return;

  int e, row0;
  if (!t_locate(p, tile, e, row0)) return;
  e = __builtin_amdgcn_readfirstlane(e);  // wave-uniform by construction; tell the compiler
  row0 = __builtin_amdgcn_readfirstlane(row0);
  const bool tail = e >= p.E;
  const int row_end = min(t_rows_end(p, e), row0 + kTM);
  const int8_t* w_base = tail ? p.w_tail : p.w + static_cast<size_t>(e) * p.n * p.k;
  const float* w_max = tail ? p.w_max_tail : p.w_max + static_cast<size_t>(e) * p.n;

  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int ksteps = p.k / 64;
  const int nchunks = ksteps / kSteps;  // the host only sends k % 128 == 0 here
  const int col_base = (nb * kWavesT + wave) * NFH * 16;

  // Weight fragment offsets (bytes from w_base) of this lane. Fragments past the last
  // channel read fragment 0 instead (valid memory): their results are never stored.
  bool wok[kNF];
  int col[kNF];
  uint32_t woff[kNF];
#pragma unroll
  for (int f = 0; f < kNF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    woff[f] = static_cast<uint32_t>(wok[f] ? col[f] / 16 : 0) * ksteps * 1024u + lane * 16u;
  }

  // Activation slots of this thread in the LDS tile. Rows past the tile's end read
  // the tile's first row (valid memory); their results are never stored.
  uint32_t aoff[kNA];
  int a_lds[kNA];
#pragma unroll
  for (int i = 0; i < kNA; ++i) {
    const int v = threadIdx.x + i * kThreads;
    const int r = v >> 3;  // 8 vectors of 16 B per row and chunk
    const int kv = v & 7;
    a_lds[i] = r * kPitchT + kv * 16;
    const int rr = row0 + r < row_end ? row0 + r : row0;
    const int sr = tail ? p.tail_src0 + rr - p.tail_row0 : (p.row_src ? p.row_src[rr] / p.src_div : rr);
    aoff[i] = static_cast<uint32_t>(sr) * static_cast<uint32_t>(p.lda) + kv * 16;  // < 4 GiB: host-checked
  }
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(w_base), a_rsrc = make_rsrc(p.a);

  v4i acc[kMF][kNF];
#pragma unroll
  for (int mf = 0; mf < kMF; ++mf)
#pragma unroll
    for (int f = 0; f < kNF; ++f) acc[mf][f] = (v4i){0, 0, 0, 0};

  v4i wring[4][kNF];  // weight fragments of MFMA step s live in slot s % 4
  v4i areg[kNA];

  // Every load below is unconditional (indices clamped to the last valid step / chunk),
  // so the loop body is one basic block the scheduler can interleave freely.
  const int last_step = ksteps - 1, last_chunk = nchunks - 1;
  auto load_w = [&](v4i(&dst)[kNF], int kb) {
    const uint32_t off = static_cast<uint32_t>(min(kb, last_step)) * 1024u;
#pragma unroll
    for (int f = 0; f < kNF; ++f) dst[f] = buffer_load16(w_rsrc, woff[f], off);
  };
  auto load_a = [&](int chunk) {
    const uint32_t kc = static_cast<uint32_t>(min(chunk, last_chunk)) * kChunk;
#pragma unroll
    for (int i = 0; i < kNA; ++i) areg[i] = buffer_load16(a_rsrc, aoff[i], kc);
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kNA; ++i) *reinterpret_cast<v4i*>(&lds_a[buf][a_lds[i]]) = areg[i];
  };
  // one MFMA step: 8 A fragments from LDS, each against the 4 weight fragments of the slot
  auto compute = [&](const v4i(&wcur)[kNF], int buf, int j) {
#pragma unroll
    for (int mf = 0; mf < kMF; ++mf) {
      const v4i af = *reinterpret_cast<const v4i*>(&lds_a[buf][(mf * 16 + li) * kPitchT + j * 64 + lg * 16]);
#pragma unroll
      for (int f = 0; f < kNF; ++f)
        acc[mf][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wcur[f], af, acc[mf][f], 0, 0, 0);
    }
  };

  load_a(0);
  load_w(wring[0], 0);
  load_w(wring[1], 1);
  load_w(wring[2], 2);
  store_a(0);
  __syncthreads();
  int c = 0;
  for (; c + 1 < nchunks; c += 2) {  // two chunks = four MFMA steps per iteration; k % 128 == 0
    // The fences pin the issue order: loads leave at the START of the MFMA run that
    // hides them, and each wait sits just before the first use (the counters retire in
    // issue order, so a wait lets the later loads stay in flight).
    const int s0 = c * kSteps;
    load_a(c + 1);
    load_w(wring[3], s0 + 3);
    __builtin_amdgcn_sched_barrier(0);
    compute(wring[0], 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(wring[0], s0 + 4);
    __builtin_amdgcn_sched_barrier(0);
    compute(wring[1], 0, 1);
    __builtin_amdgcn_sched_barrier(0);
    store_a(1);
    __syncthreads();
    load_a(c + 2);
    load_w(wring[1], s0 + 5);
    __builtin_amdgcn_sched_barrier(0);
    compute(wring[2], 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(wring[2], s0 + 6);
    __builtin_amdgcn_sched_barrier(0);
    compute(wring[3], 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    store_a(0);
    __syncthreads();
  }
  if (c < nchunks) {  // odd number of chunks: the last one sits in buffer 0, slots 0 and 1
    compute(wring[0], 0, 0);
    compute(wring[1], 0, 1);
  }

  // ---- epilogue: dequantise, optional SiLU-mul, store ----
  // per-channel scales once per fragment (not per row fragment): the 4 channels of this lane
  float sw[kNF][4];
#pragma unroll
  for (int f = 0; f < kNF; ++f) {
    const float4 wm = wok[f] ? *reinterpret_cast<const float4*>(w_max + col[f] + lg * 4) : make_float4(0, 0, 0, 0);
    sw[f][0] = wm.x / 127.0f;
    sw[f][1] = wm.y / 127.0f;
    sw[f][2] = wm.z / 127.0f;
    sw[f][3] = wm.w / 127.0f;
  }
#pragma unroll
  for (int mf = 0; mf < kMF; ++mf) {
    const int r = row0 + mf * 16 + li;
    if (r >= row_end) continue;
    const int sr = tail ? p.tail_src0 + r - p.tail_row0 : (p.row_src ? p.row_src[r] / p.src_div : r);
    const float sa = p.a_max[sr] / 127.0f;
#pragma unroll
    for (int f = 0; f < NFH; ++f) {
      if (!wok[f]) continue;
      const int c0 = col[f] + lg * 4;
      float yv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) yv[q] = (static_cast<float>(acc[mf][f][q]) * sa) * sw[f][q];
      if (p.acc_out) *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + c0) = acc[mf][f];
      if (SWIGLU) {
        const int fu = f + NFH;
        if (p.acc_out)
          *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + col[fu] + lg * 4) = acc[mf][fu];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float g = bf16_to_f32(f32_to_bf16_hw(yv[q]));  // gate and up are bf16 values first
          const float u = bf16_to_f32(f32_to_bf16_hw((static_cast<float>(acc[mf][fu][q]) * sa) * sw[fu][q]));
          yv[q] = silu_fixed(g) * u;
        }
      }
      *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) =
          make_uint2(pack2_bf16(yv[0], yv[1]), pack2_bf16(yv[2], yv[3]));
    }
  }
}

}  // namespace

int tiled_gemm_i8(const kmoe_gemm_i8_args* a, hipStream_t s) {
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  const int n_half = swiglu ? a->n / 2 : a->n;
  const int nfh = swiglu ? kNF / 2 : kNF;
  const int tail_rows = a->w_tail ? a->tail_rows : 0;
  const int n_exp = a->E + (a->w_tail ? 1 : 0);
  // 32-bit buffer offsets: one expert's weights and every source row of the activations
  KMOE_REQUIRE(static_cast<int64_t>(a->n) * a->k < (1ll << 32), KMOE_ERR_SHAPE,
               "grouped_gemm_i8 (tiled): n*k = %lld needs 32-bit offsets", static_cast<long long>(a->n) * a->k);
  KMOE_REQUIRE((static_cast<int64_t>(a->rows) + a->tail_src0 + tail_rows + 1) * a->lda < (1ll << 32), KMOE_ERR_SHAPE,
               "grouped_gemm_i8 (tiled): activations span more than 4 GiB");
  TiledParams p{a->a,      a->lda,        a->a_max,      a->row_src, a->src_div,   a->w,         a->w_max, a->lod,
                a->E,      a->n,          a->k,          a->y,       a->ldy,       a->acc_out,   a->w_tail,
                a->w_max_tail, a->tail_row0, tail_rows,  a->tail_src0,
                ceil_div(n_half, kWavesT * nfh * 16),
                (a->rows + tail_rows) / kTM + min(n_exp, a->rows + tail_rows)};
  const int grid = ceil_div(p.n_blocks * p.max_tiles, 8 * p.n_blocks * kGroupTiles) * 8 * p.n_blocks * kGroupTiles;
  if (swiglu) {
    hipLaunchKernelGGL((tiled_gemm_i8_kernel<true>), dim3(grid), dim3(kThreads), 0, s, p);
  } else {
    hipLaunchKernelGGL((tiled_gemm_i8_kernel<false>), dim3(grid), dim3(kThreads), 0, s, p);
  }
  return check_launch("kmoe_grouped_gemm_i8 (tiled)");
}

}  // namespace kmoe
