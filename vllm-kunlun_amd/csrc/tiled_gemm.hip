// Grouped GEMM for the prefill regime (hundreds of rows per expert) on MFMA, tiled weights;
// int8 (v_mfma_i32_16x16x64_i8), fp8 block-scaled and bf16 operands.
//
// Two workgroup shapes. Four waves on a 128-row x 256-channel tile (64-, 96-row forms for few rows per
// expert), each wave owning 64 channels of all the rows (8 x 4 accumulator fragments = 128 registers), two
// workgroups per CU: one workgroup's waits, barriers and VALU-heavy epilogue run under the other's MFMAs.
// And, int8 with more than 72 rows per expert: EIGHT waves side by side along the channels (WN = 8) on a
// 128-, 192- or 256-row x 256-channel tile, each wave owning 32 channels of all the rows, one workgroup
// per CU, a deeper weight ring, and row fragments past an expert's last row skipped (see tiled_gemm_i8).
//   activations: int8 / bf16: asynchronous copies global -> LDS (rows gathered through the
//                sort), 128 bytes of K per row and chunk, three chunks ahead into a ring of
//                four chunk buffers, swizzled so that fragment reads are conflict-free without
//                padding; no register holds them. fp8: through registers into two padded
//                buffers (pitch 160 B), one chunk ahead, with the row scales of the chunk.
//                Every A fragment read from LDS feeds 4 MFMAs.
//   weights:     straight from L2 into registers, 1 KB of consecutive bytes per
//                fragment and MFMA step (tiled layout), through a ring of 4 step
//                buffers loaded 3 MFMA steps ahead of use; every B fragment
//                feeds 8 MFMAs. No weight byte goes through LDS.
// Workgroups are persistent: each walks a strided list of tiles. The tile after
// the current one is located (from an LDS copy of lod) and its gather indices are
// fetched while the current tile computes; its first activation chunks and weight
// steps are requested BEFORE the current tile's epilogue, which hides their
// latency. Per-row and per-channel scales of a tile wait in LDS, so the epilogue
// touches global memory only to store. Output tiles are transposed through a
// per-wave LDS patch so every store instruction writes whole 64/128-byte row
// segments. The tiles that read the same weight bytes run side by side on one XCD
// (one L2), so an expert's weights leave HBM about once.
//
// The compiler drains every asynchronous copy in flight before any LDS access it can see.
// Inside the pipeline the LDS accesses are therefore inline assembly with their own waits, and
// the waits on the copies are explicit s_waitcnt vmcnt(N): a wave's loads complete in issue
// order, so "at most N in flight" means "everything older than the N youngest has landed". Each
// N below is the number of loads the wave is known to have issued after the copies it needs.
#include <cstdlib>
#include <type_traits>

#include "buffer_ops.h"
#include "kmoe_common.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// LDS reads issued from assembly statements, each with its own wait on the LDS counter: an LDS read that the compiler
// sees makes it wait first for every global load, store and asynchronous copy of the wave (it cannot tell a copy's
// destination from the address read), which in the tile loop means thousands of clocks.
__device__ __forceinline__ void lds_read1_b32(float& a, uint32_t addr) {
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(a) : "v"(addr) : "memory");
}
template <int STRIDE>
__device__ __forceinline__ void lds_read4_b32(float& a, float& b, float& c, float& d, uint32_t addr) {
  asm volatile(
      "ds_read_b32 %0, %4\n\t"
      "ds_read_b32 %1, %4 offset:%5\n\t"
      "ds_read_b32 %2, %4 offset:%6\n\t"
      "ds_read_b32 %3, %4 offset:%7\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d)
      : "v"(addr), "n"(STRIDE), "n"(2 * STRIDE), "n"(3 * STRIDE)
      : "memory");
}
// fp8 on the asynchronous path: the two K halves of an activation fragment and its row scale, requested without a
// wait (IMM: byte offset of the fragment in the chunk buffer, SOFF: of its scale), and the wait that makes them
// (and the chunk's two weight scales) usable while at most N younger LDS operations stay in flight.
template <int IMM, int SOFF>
__device__ __forceinline__ void f8_request(v4i& lo, v4i& hi, float& sa, uint32_t a_lo, uint32_t a_hi, uint32_t sc_addr) {
  asm volatile(
      "ds_read_b128 %0, %3 offset:%6\n\t"
      "ds_read_b128 %1, %4 offset:%6\n\t"
      "ds_read_b32 %2, %5 offset:%7"
      : "=&v"(lo), "=&v"(hi), "=&v"(sa)
      : "v"(a_lo), "v"(a_hi), "v"(sc_addr), "n"(IMM), "n"(SOFF)
      : "memory");
}
template <int N>
__device__ __forceinline__ void f8_wait(v4i& lo, v4i& hi, float& sa, float& s0, float& s1) {
  asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(lo), "+v"(hi), "+v"(sa), "+v"(s0), "+v"(s1) : "n"(N));
}
template <int OFF>
__device__ __forceinline__ void lds_request_b32(float& v, uint32_t addr) {
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
}
// lds_wait<n> for an n that is a constant only after unrolling (at most 7 younger LDS operations stay in flight)
template <typename V>
__device__ __forceinline__ void lds_wait_upto(int n, V& v) {
  switch (n) {
    case 0: lds_wait<0>(v); break;
    case 1: lds_wait<1>(v); break;
    case 2: lds_wait<2>(v); break;
    case 3: lds_wait<3>(v); break;
    case 4: lds_wait<4>(v); break;
    case 5: lds_wait<5>(v); break;
    case 6: lds_wait<6>(v); break;
    default: lds_wait<7>(v); break;
  }
}
__device__ __forceinline__ void lds_read1_b128(v4f& a, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(a) : "v"(addr) : "memory");
}
template <int STRIDE>
__device__ __forceinline__ void lds_read2_b128(v4f& a, v4f& b, uint32_t addr) {
  asm volatile(
      "ds_read_b128 %0, %2\n\t"
      "ds_read_b128 %1, %2 offset:%3\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(a), "=&v"(b)
      : "v"(addr), "n"(STRIDE)
      : "memory");
}
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

// Operand format. F8: e4m3fn codes with block scales (one f32 per 128x128 weight block and
// per activation row and 128 of K); one v_mfma_scale_f32_16x16x128_f8f6f4 covers a whole
// 128-byte chunk (the two 1 KB weight blocks of a chunk are its two K halves, and the
// activation fragment takes the same two halves), its partial sum is scaled and added in f32.
// BF16: unscaled bf16 operands on v_mfma_f32_16x16x32_bf16; sizes along K are in BYTES here (a
// 1 KB weight block holds 16 channels x 32 values, a 128-byte chunk two MFMA steps).
enum class TKind { I8, F8, BF16 };
constexpr int kMaxKBlocks = 64;  // F8: K <= 8192

constexpr int kWavesT = 4;                 // 4 waves side by side along the channels
constexpr int kChunk = 128;                // bytes of K per row and chunk (2 MFMA steps)
constexpr int kSteps = kChunk / 64;
constexpr int kPitchT = kChunk + 32;       // 160 B: measured conflict-free for the b128 fragment reads (144 is not)
constexpr int kStagesA = 4;                // chunk buffers of the asynchronous activation path
constexpr int kMaxExperts = 1024 + 1;      // routed experts + the tail expert

struct TiledParams {
  const int8_t* a;
  int64_t lda;
  const float* a_max;   // I8: [a_rows] absmax. F8: [a_rows, k/128] scales
  const int32_t* row_src;
  int32_t src_div;
  const int8_t* w;  // tiled
  const float* w_max;   // I8: [E, n] absmax. F8: [E, n/128, k/128] scales
  const int32_t* lod;
  int32_t E, n, k;
  uint16_t* y;
  int64_t ldy;
  int32_t* acc_out;
  const int8_t* w_tail;
  const float* w_max_tail;
  int32_t tail_row0, tail_rows, tail_src0;
  int32_t n_blocks;  // channel blocks per tile
  int32_t max_items; // upper bound of work items (n_blocks * bound of m-tiles): caps the grid
  // BF16 only (the expert-bias branch of the reference, ops/_kunlun_ops.py:433-468):
  const uint16_t* bias;        // NULL, or [E, n] bf16: y = bf16(bf16(gemm) + bias)
  float oai_alpha, oai_limit;  // OAI kernels: out[r, i] = swigluoai(y[r, 2i], y[r, 2i + 1])
  // One of two launches of the same GEMM on different tiles, of which the routing decides on the device which
  // one works (the other finds out in its prologue and leaves): the tall tiles of pick_rows rows pay while few
  // routed experts overflow them (at most one in 16). pick = 1: this launch runs if they do, pick = 2: if not;
  // 0: it always runs.
  int32_t pick, pick_rows;
  // Order of an expert's items. 0: channel block by channel block, the m-tiles of one block next to each other (they
  // read the same weight bytes at the same time; the paced kernels need it). 1: m-tile by m-tile, the channel blocks
  // of one m-tile next to each other (they read the same rows at the same time) - for experts whose weights stay in an
  // XCD's L2 anyway, where an expert with many m-tiles would otherwise fetch its rows once per channel block.
  int32_t m_major;
};

// Progress board of the persistent workgroups: slot b (64 bytes apart) holds where workgroup b is,
// ((position in its item list + 1) << 16) | chunk of K, 0xffffffff once it has no work left, 0 before
// its first launch. The m-tiles of one (expert, channel block) stream the same weight bytes; they are
// neighbouring items of the work list and therefore run on neighbouring workgroups of one XCD at the
// same position of their lists. A workgroup that gets ahead of such a sibling by more than kSyncSlack
// chunks waits for it (bounded), so the siblings' requests for a weight line meet in the XCD's L2
// while the line is still there, and the weights of an expert leave HBM once instead of once per
// m-tile. The board only paces the workgroups: no result depends on it, every wait has an upper bound,
// and two launches that overlap on one GPU merely pace each other badly.
constexpr int kBoardSlots = 2048;
constexpr int kBoardStride = 16;  // 32-bit words: one slot per 64-byte line
constexpr uint32_t kSyncSlack = 2;
constexpr int kSyncPatience = 96;  // polls a workgroup spends waiting per tile at most (about 1 us each)
static __device__ uint32_t g_board[kBoardSlots * kBoardStride];  // word 0 of a slot: the progress; word 1: never written

struct Tile {
  int it;    // position in this workgroup's list
  int sib;   // bit 0: the item before is an m-tile of the same (expert, channel block); bit 1: the item after
  int e;     // expert (E = the tail expert)
  int row0;  // first sorted row
  int nb;    // channel block
  int end;   // the tile's rows end here (its share of the expert's rows)
  bool valid;
};

// NF: 16-channel fragments per wave (4: 256-channel tiles, 2: 128-channel tiles);
// R: weight ring slots (R - 1 MFMA steps of weights in flight per wave), 4 or 8;
// WGS: workgroups per CU the register budget is cut for.
// <4,4,2> is the shape in use; <2,8,2> trades operand reuse for narrower tiles and more bytes
// in flight (a tuning variant).
// WM: rows of waves. 1: 128-row tiles, 4 waves; 2: 256-row tiles, 8 waves, where the two waves
// that share channels read the same weight bytes within one barrier interval (an expert with
// up to 256 rows then streams its weights from HBM once).
// M32: 32x32 MFMA shapes (v_mfma_i32_32x32x32_i8, v_mfma_f32_32x32x16_bf16) on the same tiles and
// the same bytes: a wave's 128 x 64 patch is 4 x 2 accumulator fragments of 16 registers. One
// wave alone on a SIMD issues these at 89 % of the peak rate (measured), the 16x16 shapes at
// 58 %; with two waves on the SIMD both reach 91 %. A 32-channel weight fragment of one MFMA
// (32 bytes of K) is two 16-lane quarters of two neighbouring 1 KB blocks, lanes 32-63 taking
// the next 16 bytes of K; the activation fragment takes the same bytes of its rows, so the
// order of K inside a step differs from the 16x16 path while the sums (exact in int32) do not.
// MF: 16-row fragments of a wave along the rows. 8: 128-row tiles; 4: 64-row tiles for launches whose
// experts hold a few dozen rows each (half the MFMAs, fragment reads and epilogue per weight byte,
// and registers for a third workgroup per CU).
// OAI (bf16, no SiLU-mul): gate and up columns interleaved, the gpt-oss activation on each (gate, up) pair of
// a lane's four consecutive channels - n / 2 outputs per row (ops/_custom_ops.py:728-742).
// PACE: the m-tiles of one (expert, channel block) keep in step through the progress board (g_board), which
// brings the bytes fetched by L2 down to little more than once per weight byte where experts have two or three
// m-tiles (int8: a few percent of time, the re-reads were mostly served by the memory-side cache; fp8: 14 %).
// F16: the outputs, and the rounding of gate and up before SiLU-mul, are IEEE half instead of bf16 (int8 and
// fp8 operands); with KIND = BF16 the operands are half as well (v_mfma_f32_16x16x32_f16).
template <TKind KIND, bool SWIGLU, int NF, int R, int WGS, int WM, bool M32 = false, int MF = 8, bool OAI = false,
          bool PACE = false, bool F16 = false, int WN = kWavesT>
__global__ __launch_bounds__(WM * WN * kWave, WGS) void tiled_gemm_kernel(const TiledParams p) {
  constexpr int kWN = WN;  // waves side by side along the channels
  static_assert(!F16 || KIND != TKind::BF16 || !OAI, "the interleaved activation is a bf16 epilogue");
  static_assert(!OAI || (KIND == TKind::BF16 && !SWIGLU && !M32), "the interleaved activation is a bf16 epilogue");
  constexpr int kMF = MF;
  // 16-byte activation vectors per thread and chunk; an odd MF rounds up: the copies then cover up to 8 rows per
  // wave past the tile's last row (rows of the next tile, or the tile's first row again), which land in buffer
  // rows that no fragment reads
  constexpr int kNA = (16 * kMF * (kChunk / 16) + kWN * kWave - 1) / (kWN * kWave);
  static_assert(kNA >= 1 && (M32 ? MF % 2 == 0 : true), "tile height");
  static_assert(MF % 2 == 0 || KIND != TKind::F8, "an odd tile height needs the asynchronous activation path");
  constexpr bool F8 = KIND == TKind::F8;
  constexpr bool I8 = KIND == TKind::I8;
  constexpr bool BF = KIND == TKind::BF16;
  static_assert(!(M32 && F8), "the 32x32 shapes are wired for int8 and bf16");
  using acc_t = std::conditional_t<M32, std::conditional_t<I8, v16i, v16f>, std::conditional_t<I8, v4i, v4f>>;
  constexpr int kFragRows = M32 ? 32 : 16;       // rows (and channels) of an accumulator fragment
  constexpr int AM = 16 * kMF / kFragRows;       // accumulator fragments of a wave along the rows
  constexpr int AN = 16 * NF / kFragRows;        // ... and along the channels
  constexpr int kAccRegs = M32 ? 16 : 4;
  constexpr int kTM = WM * 16 * kMF;             // rows of a tile
  constexpr int kThreads = WM * kWN * kWave;
  static_assert(R == 4 || R == 8, "the chunk buffer parity is static only for R/2 even");
  constexpr int kNF = NF;
  constexpr int NFH = SWIGLU ? kNF / 2 : kNF;
  constexpr int kOutBytes = NFH * 16 * 2 / (OAI ? 2 : 1);  // bytes of one output row owned by a wave: 32 .. 128
  constexpr int kPatchPitch = kOutBytes + 16;  // bytes per row of a wave's output patch (16 rows)
  // ADMA: activations go global -> LDS asynchronously, three chunks ahead, into a ring of four
  // unpadded chunk buffers (row r, 16-byte vector c of a chunk at r * 128 + 16 (c ^ r % 8): eight
  // consecutive rows of one fragment column fall on eight different bank groups). F8 keeps the
  // register path (its row scales travel with the data): two padded buffers.
  constexpr bool ADMA = !F8 || WN == 8;  // (fp8: the wide tiles; its 4-wave tiles keep the register path)
  constexpr int kStageBytes = ADMA ? WM * kWN * kNA * 8 * kChunk : kTM * kPitchT;  // (ADMA: kTM rows, or the copies' 8 kNA per wave)
  __shared__ __attribute__((aligned(1024))) int8_t lds_a[ADMA ? kStagesA : 2][kStageBytes];
  // (wide tiles with two output fragments a wave: patches for kPatchGroup row fragments, transposed in one LDS round trip)
  constexpr int kPatchGroup = (!OAI && !M32 && NFH == 2 && WN == 8) ? (MF % 4 == 0 && MF < 16 ? 4 : 2) : 1;
  static_assert((16 * kMF / kFragRows) % kPatchGroup == 0, "row fragments per patch group");
  __shared__ __attribute__((aligned(16)))
  int8_t patch[WM * kWN][(!OAI && !M32 && NFH == 1) ? 16 : kPatchGroup * kFragRows * kPatchPitch];
  // I8, per tile parity: channel scales (w_max / 127) and row scales (a_max / 127)
  __shared__ __attribute__((aligned(16))) float sw_lds[I8 ? 2 : 1][I8 ? kWN * NF * 16 : 4];
  // (a wave's copy of row maxes always writes 64 slots: tiles of fewer rows still get 64)
  __shared__ float sa_lds[I8 ? 2 : 1][I8 ? (kTM + kWave - 1) / kWave * kWave : 4];
  // F8: weight block scales of the tile [parity][wave][fragment][k block], and the row scales
  // of the chunk in each activation buffer
  __shared__ float wsc_lds[F8 ? 2 : 1][F8 ? kWN * NF * kMaxKBlocks : 4];
  // (register path: every thread stores, rows repeat - no branch in the loop; asynchronous path: a ring like the
  // chunks', each wave copying 64 row scales per chunk, waves past the tile's rows repeating earlier ones)
  static_assert(!(F8 && ADMA) || kTM % kWave == 0, "row scales are copied 64 at a time");
  __shared__ float asc_lds[F8 ? (ADMA ? kStagesA : 2) : 1][F8 ? (ADMA ? kTM : kThreads) : 4];
  extern __shared__ int dyn_lds[];
  const int n_exp = p.E + (p.w_tail ? 1 : 0);
  int* row_lo = dyn_lds;               // [E + 1]: lod
  int* tile_lo = dyn_lds + p.E + 1;    // [n_exp + 1]: first m-tile of each expert, then the total

  const int lane = lane_id();
  const int wave_id = threadIdx.x >> 6;
  const int wave = WM == 1 ? wave_id : wave_id % kWN;  // position along the channels
  const int wave_m = WM == 1 ? 0 : wave_id / kWN;      // position along the rows
  const int li = lane & (kFragRows - 1);  // row (or channel) of a fragment held by this lane
  const int lg = lane / kFragRows;        // 16-byte group of K (16x16: 0..3; 32x32: 0..1)
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int ksteps = p.k / 64;
  // Chunks of two MFMA steps. An odd number of steps (int8: k % 128 == 64, bf16: k % 64 == 32; the host sends
  // those only with at least one whole chunk) ends in a half chunk: its copy starts 64 bytes early, so that it
  // stays inside the row, which puts the last step's bytes into the chunk's second half; the first half (the
  // step before, once more) is read from LDS and set to zero before it meets the MFMA (zero activations
  // against finite weights add nothing; zero weights would turn an infinite activation into NaN).
  const int nfull = ksteps / kSteps;
  const bool half_chunk = ADMA && (ksteps & 1);
  const int nchunks = nfull + (half_chunk ? 1 : 0);
  const int last_step = ksteps - 1, last_chunk = nchunks - 1;
  const uint32_t last_chunk_byte = static_cast<uint32_t>(ksteps * 64 - kChunk);
  auto rows_begin = [&](int e) { return e < p.E ? row_lo[e] : p.tail_row0; };
  auto rows_end = [&](int e) { return e < p.E ? row_lo[e + 1] : p.tail_row0 + p.tail_rows; };

  // ---- once per workgroup: rows and m-tiles of every expert into LDS ----
  for (int e = threadIdx.x; e <= p.E; e += kThreads) row_lo[e] = p.lod[e];
  __syncthreads();
  if (wave_id == 0) {
    int carry = 0, over = 0;
    for (int base = 0; base < n_exp; base += kWave) {
      const int e = base + lane;
      const int mine = e < n_exp ? (rows_end(e) - rows_begin(e) + kTM - 1) / kTM : 0;
      int incl = mine;
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) {
        const int o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
      }
      if (e < n_exp) tile_lo[e] = carry + incl - mine;
      carry += __shfl(incl, kWave - 1, kWave);
      over += __popcll(__ballot(e < p.E && row_lo[e + 1] - row_lo[e] > p.pick_rows));
    }
    if (lane == 0) {
      tile_lo[n_exp] = carry;
      tile_lo[n_exp + 1] = over;  // routed experts with more rows than a tall tile holds
    }
  }
  __syncthreads();
  const int total_tiles = tile_lo[n_exp];
  const bool tall_pays = tile_lo[n_exp + 1] * 16 <= p.E;
  const bool not_my_launch = (p.pick == 1 && !tall_pays) || (p.pick == 2 && tall_pays);

  // Work items = (m-tile, channel block) pairs, n_items of them, all non-empty, numbered expert
  // by expert; inside an expert the m-tiles of one channel block are consecutive. The list is
  // cut into 8 equal segments, one per XCD (workgroup b runs on XCD b % 8), and the workgroups
  // of an XCD walk their segment side by side: the m-tiles that read the same weight bytes (and
  // the channel blocks that read the same rows) run at the same time behind ONE L2, so an
  // expert's weights leave HBM once - except for the experts a segment or a round cuts in two.
  const int n_items = total_tiles * p.n_blocks;
  const int seg = (n_items + 7) >> 3;
  const int xcd = blockIdx.x & 7;
  const int seg_end = min((xcd + 1) * seg, n_items);
  // The items of this workgroup are resolved 64 at a time: lane l of wave 0 finds item it0 + l (a binary
  // search over tile_lo and two divisions, all lanes at once) and leaves (expert, first row, channel
  // block) in LDS; the tile loop then reads three words per tile instead of searching.
  __shared__ int items[5][kWave];  // per resolved item: expert, first row, channel block, sibling flag, the tile's row end
  int* const item_e = items[0];
  int* const item_row0 = items[1];
  int* const item_nb = items[2];
  int* const item_sib = items[3];
  int* const item_end = items[4];
  const int per_xcd = gridDim.x >> 3;  // gridDim.x is a multiple of 8
  // item lid of the list (lid < seg_end) -> expert, first row, channel block, sibling flags
  auto resolve_item = [&](int lid, int& e, int& row0, int& nb, int& sib, int& end) {
    const int m_tile = lid / p.n_blocks;
    // the last e with tile_lo[e] <= m_tile: of a run of equal entries (empty experts) the one that owns the tile
    int lo = 0, hi = n_exp - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (tile_lo[mid] <= m_tile) lo = mid;
      else hi = mid - 1;
    }
    e = lo;
    const int first = tile_lo[e], mt = tile_lo[e + 1] - first;
    const int u = lid - first * p.n_blocks;
    int m;
    if (p.m_major) {
      m = u / p.n_blocks;
      nb = u - m * p.n_blocks;
    } else {
      nb = u / mt;
      m = u - nb * mt;
    }
    // An expert's rows are split EVENLY over its m-tiles (whole 16-row fragments): kernels that skip the row
    // fragments past a tile's end then spend about the same time on each of them, so the m-tiles of one channel
    // block, which start together on neighbouring workgroups, stay in step and share the weight bytes in L2 - a
    // full tile next to a nearly empty one would fetch them twice. (Experts with more m-tiles than a tile has
    // fragments keep full tiles: the rounding could leave a trailing tile without rows.)
    const int rows_e = rows_end(e) - rows_begin(e);
    const int stride = mt <= kTM / 16 ? (((rows_e + mt - 1) / mt + 15) & ~15) : kTM;
    row0 = rows_begin(e) + m * stride;
    end = min(rows_end(e), row0 + stride);
    // siblings run on the workgroups before / after this one in the XCD, at the same list position
    const int j = blockIdx.x >> 3;
    if (m > 0 && j > 0) sib |= 1;
    if (m + 1 < mt && j + 1 < per_xcd && lid + 1 < seg_end) sib |= 2;
  };
  auto resolve_items = [&](int it0) {
    if (wave_id == 0) {
      const int lid = xcd * seg + (blockIdx.x >> 3) + (it0 + lane) * per_xcd;
      int e = -1, row0 = 0, nb = 0, sib = 0, end = 0;
      if (lid < seg_end) resolve_item(lid, e, row0, nb, sib, end);
      item_end[lane] = end;
      item_sib[lane] = sib;
      item_e[lane] = e;
      item_row0[lane] = row0;
      item_nb[lane] = nb;
    }
    __syncthreads();
  };
  resolve_items(0);
  // (called by every wave at the same point of the tile loop: the refill every 64 tiles has a barrier inside)
  auto find_tile = [&](int it) -> Tile {
    if (it > 0 && (it & (kWave - 1)) == 0) resolve_items(it);
    // The five words of the item come out of LDS through an assembly statement: an LDS read that the compiler sees
    // makes it wait for every load, store and asynchronous copy of the wave first (it cannot tell the copies'
    // destinations from this address) - at the loop top that is the epilogue's stores, thousands of clocks.
    Tile t{it, 0, 0, 0, 0, 0, false};
    const int slot = it & (kWave - 1);
    const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&items[0][0])) + 4u * slot;
    int e, sib, row0, nb, end;
    asm volatile(
        "ds_read_b32 %0, %5 offset:%6\n\t"
        "ds_read_b32 %1, %5 offset:%7\n\t"
        "ds_read_b32 %2, %5 offset:%8\n\t"
        "ds_read_b32 %3, %5 offset:%9\n\t"
        "ds_read_b32 %4, %5 offset:%10\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(e), "=&v"(sib), "=&v"(row0), "=&v"(nb), "=&v"(end)
        : "v"(base), "n"(0), "n"(4 * kWave * 3), "n"(4 * kWave * 1), "n"(4 * kWave * 2), "n"(4 * kWave * 4)
        : "memory");
    t.e = __builtin_amdgcn_readfirstlane(e);
    if (t.e < 0) return t;
    t.sib = __builtin_amdgcn_readfirstlane(sib);
    t.row0 = __builtin_amdgcn_readfirstlane(row0);
    t.nb = __builtin_amdgcn_readfirstlane(nb);
    t.end = __builtin_amdgcn_readfirstlane(end);
    t.valid = true;
    return t;
  };

  // ---- per-tile state of the loads ----
  __amdgpu_buffer_rsrc_t w_rsrc;
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(p.a);
  uint32_t woff[kNF];
  uint32_t aoff[kNA];
  int a_lds[kNA];
#pragma unroll
  for (int i = 0; i < kNA; ++i) {
    const int v = threadIdx.x + i * kThreads;
    a_lds[i] = (v >> 3) * kPitchT + (v & 7) * 16;  // row v/8, 16-byte vector v%8 of the chunk
  }
  v4i wring[R][kNF];  // weight fragments of MFMA step s live in slot s % R
  v4i areg[ADMA ? 1 : kNA];
  // ADMA: copy i of this wave fills rows 8 (kNA wave_id + i) + lane / 8 of a chunk buffer; the lane
  // fetches vector (lane % 8) ^ (lane / 8 % 8) of its row, which lands at position lane % 8.
  const int dma_row = wave_id * 8 * kNA + (lane >> 3);
  const uint32_t dma_vec = static_cast<uint32_t>((lane & 7) ^ ((lane >> 3) & 7));
  const uint32_t lds_a_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&lds_a[0][0]));
  // fragment reads: row li (+ 16 or 32 per fragment: same row % 8), vector v of the chunk at (v ^ li % 8)
  auto frag_addr = [&](int v) -> uint32_t {
    return lds_a_base + static_cast<uint32_t>((wave_m * 16 * kMF + li) * kChunk + ((v ^ (li & 7)) << 4));
  };
  // 16x16: vector 4 j + lg of step j; 32x32: vector 4 j + 2 t + lg of step j, K part t
  uint32_t fa[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) fa[q] = M32 ? frag_addr(2 * q + lg) : frag_addr(4 * (q & 1) + lg);
  acc_t acc[AM][AN];
  const int kblocks = p.k / 128;  // F8: scale blocks along K (= chunks)
  int my_srow = 0;                // F8: source row of tile row threadIdx.x % kTM
  float asc_reg = 0.0f;           // F8: that row's scale of the chunk in flight

  // Every load is unconditional (indices clamped to the last valid step / chunk, rows past a
  // tile's end read its first row, fragments past the last channel read fragment 0): the
  // results of those are never stored, and the loop body stays one basic block.
  auto load_w = [&](v4i(&dst)[kNF], int kb) {
    const uint32_t off = static_cast<uint32_t>(min(kb, last_step)) * 1024u;
    if constexpr (M32) {
#pragma unroll
      for (int f = 0; f < kNF; ++f) dst[f] = buffer_load16(w_rsrc, woff[f >> 1], off + (f & 1) * 512u);
    } else {
#pragma unroll
      for (int f = 0; f < kNF; ++f) dst[f] = buffer_load16(w_rsrc, woff[f], off);
    }
  };
  auto load_a = [&](int chunk) {
    if constexpr (!ADMA) {
      const uint32_t kc = static_cast<uint32_t>(min(chunk, last_chunk)) * kChunk;
#pragma unroll
      for (int i = 0; i < kNA; ++i) areg[i] = buffer_load16(a_rsrc, aoff[i], kc);
      if constexpr (F8) asc_reg = p.a_max[static_cast<size_t>(my_srow) * kblocks + min(chunk, last_chunk)];
    }
  };
  auto store_a = [&](int buf) {
    if constexpr (!ADMA) {
#pragma unroll
      for (int i = 0; i < kNA; ++i) *reinterpret_cast<v4i*>(&lds_a[buf][a_lds[i]]) = areg[i];
      if constexpr (F8) asc_lds[buf][threadIdx.x] = asc_reg;
    }
  };
  // ADMA: requests chunk `chunk` of the tile into ring buffer `stage` (4 copies per wave)
  auto dma_a = [&](int chunk, int stage) {
    if constexpr (ADMA) {
      const uint32_t kc = min(static_cast<uint32_t>(chunk) * kChunk, last_chunk_byte);
#pragma unroll
      for (int i = 0; i < kNA; ++i)
        buffer_load16_to_lds(a_rsrc, (lds_ptr_t)&lds_a[stage][(wave_id * kNA + i) * 1024], aoff[i], kc);
      if constexpr (F8) {
        // the chunk's row scales travel the same way: lane l of wave w brings the scale of tile row (64 w + l) % kTM
        const uint32_t kb = static_cast<uint32_t>(min(chunk, last_chunk));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(p.a_max), (lds_ptr_t)&asc_lds[stage][(wave_id * kWave) % kTM], 4,
                                                 (static_cast<uint32_t>(my_srow) * static_cast<uint32_t>(kblocks) + kb) * 4u,
                                                 0, 0, 0);
      }
    }
  };
  constexpr int kND = kNA + ((F8 && ADMA) ? 1 : 0);  // copies per chunk and wave
  // one MFMA step: 8 A fragments from LDS, each against the 4 weight fragments of the slot
  auto mfma_row = [&](const v4i(&wcur)[kNF], const v4i& af, int mf, int t) {
    if constexpr (M32) {
      // slot entry 2 g + t: 32-channel fragment g, K bytes [32 t, 32 t + 32) of the step
#pragma unroll
      for (int g = 0; g < AN; ++g) {
        if constexpr (BF && F16)
          acc[mf][g] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, wcur[2 * g + t]),
                                                              __builtin_bit_cast(v8h, af), acc[mf][g], 0, 0, 0);
        else if constexpr (BF)
          acc[mf][g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, wcur[2 * g + t]),
                                                               __builtin_bit_cast(v8bf, af), acc[mf][g], 0, 0, 0);
        else if constexpr (I8)
          acc[mf][g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wcur[2 * g + t], af, acc[mf][g], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        if constexpr (BF && F16)  // the unquantized path on half operands
          acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wcur[f]),
                                                              __builtin_bit_cast(v8h, af), acc[mf][f], 0, 0, 0);
        else if constexpr (BF)
          acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wcur[f]),
                                                               __builtin_bit_cast(v8bf, af), acc[mf][f], 0, 0, 0);
        else if constexpr (I8)
          acc[mf][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wcur[f], af, acc[mf][f], 0, 0, 0);
      }
    }
  };
  // fragment n of a step: (row fragment, K part); 16x16: 8 row fragments; 32x32: 2 K parts x 4
  constexpr int kFragReads = M32 ? 2 * AM : kMF;
  // Row fragments of this wave that hold rows of the current tile (wave-uniform, set per tile): the K loop of the
  // int8 path neither reads nor multiplies the others (the padding of an expert's last tile).
  int live_frags = kMF;
  // One row fragment of one MFMA step, int8: LDS read of the NEXT live fragment, wait for this one's, NF MFMAs -
  // all inside one assembly statement, because the skip is a branch: a branch the compiler can see splits the
  // loop body into basic blocks, after which its register allocator spills hundreds of registers. `live` is
  // wave-uniform (an SGPR); a live fragment falls through its test, a dead one costs a compare and a taken branch.
  // LDS operations of a wave complete in order, so "at most one in flight" means this fragment's read has landed.
  auto frag_i8 = [&](const v4i(&w)[kNF], v4i& af_cur, v4i& af_next, uint32_t addr, auto n_tag, auto off_own, auto off_next,
                     int mf) {
    constexpr int n = decltype(n_tag)::value;
    constexpr bool kFirst = n == 0, kLast = n + 1 == kMF;
    static_assert(kNF == 4 || kNF == 2, "fragment step written for 2 or 4 channel fragments per wave");
// dead fragment: leave
#define KMOE_FRAG_HEAD "s_cmp_lt_i32 %[live], %[n1]\n\ts_cbranch_scc1 3f\n\t"
// the first fragment of a step requests its own bytes
#define KMOE_FRAG_OWN "ds_read_b128 %[cur], %[addr] offset:%[own]\n\t"
// request the next fragment's bytes, then wait for this one's. The request is unconditional: a taken branch costs a
// wave some twenty cycles, and a test for "the next one is dead" would put one on the path of every live fragment.
// If the next fragment is dead its bytes arrive unused, and the wait at the end of the step retires the request.
#define KMOE_FRAG_NEXT "ds_read_b128 %[nxt], %[addr] offset:%[onext]\n\ts_waitcnt lgkmcnt(1)\n\t"
#define KMOE_FRAG_WAIT "s_waitcnt lgkmcnt(0)\n\t"
#define KMOE_FRAG_MFMA2                                          \
  "v_mfma_i32_16x16x64_i8 %[c0], %[w0], %[cur], %[c0]\n\t"       \
  "v_mfma_i32_16x16x64_i8 %[c1], %[w1], %[cur], %[c1]\n\t"
#define KMOE_FRAG_MFMA4                                          \
  KMOE_FRAG_MFMA2                                                \
  "v_mfma_i32_16x16x64_i8 %[c2], %[w2], %[cur], %[c2]\n\t"       \
  "v_mfma_i32_16x16x64_i8 %[c3], %[w3], %[cur], %[c3]\n\t"
#define KMOE_FRAG_IMMS                                                                                       \
  [addr] "v"(addr), [live] "s"(live_frags), [n1] "n"(n + 1), [own] "n"(decltype(off_own)::value), \
      [onext] "n"(decltype(off_next)::value)
    if constexpr (kNF == 4) {
#define KMOE_FRAG_ACC [c0] "+v"(acc[mf][0]), [c1] "+v"(acc[mf][1]), [c2] "+v"(acc[mf][2]), [c3] "+v"(acc[mf][3])
#define KMOE_FRAG_W [w0] "v"(w[0]), [w1] "v"(w[1]), [w2] "v"(w[2]), [w3] "v"(w[3])
      if constexpr (kFirst && kLast)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_OWN KMOE_FRAG_WAIT KMOE_FRAG_MFMA4 "3:\n\t"
                     : KMOE_FRAG_ACC, [cur] "=&v"(af_cur) : KMOE_FRAG_W, KMOE_FRAG_IMMS : "scc", "memory");
      else if constexpr (kFirst)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_OWN KMOE_FRAG_NEXT KMOE_FRAG_MFMA4 "3:\n\t"
                     : KMOE_FRAG_ACC, [cur] "=&v"(af_cur), [nxt] "=&v"(af_next) : KMOE_FRAG_W, KMOE_FRAG_IMMS
                     : "scc", "memory");
      else if constexpr (kLast)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_WAIT KMOE_FRAG_MFMA4 "3:\n\t"
                     : KMOE_FRAG_ACC : KMOE_FRAG_W, [cur] "v"(af_cur), KMOE_FRAG_IMMS : "scc", "memory");
      else
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_NEXT KMOE_FRAG_MFMA4 "3:\n\t"
                     : KMOE_FRAG_ACC, [nxt] "=&v"(af_next) : KMOE_FRAG_W, [cur] "v"(af_cur), KMOE_FRAG_IMMS
                     : "scc", "memory");
#undef KMOE_FRAG_ACC
#undef KMOE_FRAG_W
    } else {
#define KMOE_FRAG_ACC [c0] "+v"(acc[mf][0]), [c1] "+v"(acc[mf][1])
#define KMOE_FRAG_W [w0] "v"(w[0]), [w1] "v"(w[1])
      if constexpr (kFirst && kLast)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_OWN KMOE_FRAG_WAIT KMOE_FRAG_MFMA2 "3:\n\t"
                     : KMOE_FRAG_ACC, [cur] "=&v"(af_cur) : KMOE_FRAG_W, KMOE_FRAG_IMMS : "scc", "memory");
      else if constexpr (kFirst)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_OWN KMOE_FRAG_NEXT KMOE_FRAG_MFMA2 "3:\n\t"
                     : KMOE_FRAG_ACC, [cur] "=&v"(af_cur), [nxt] "=&v"(af_next) : KMOE_FRAG_W, KMOE_FRAG_IMMS
                     : "scc", "memory");
      else if constexpr (kLast)
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_WAIT KMOE_FRAG_MFMA2 "3:\n\t"
                     : KMOE_FRAG_ACC : KMOE_FRAG_W, [cur] "v"(af_cur), KMOE_FRAG_IMMS : "scc", "memory");
      else
        asm volatile(KMOE_FRAG_HEAD KMOE_FRAG_NEXT KMOE_FRAG_MFMA2 "3:\n\t"
                     : KMOE_FRAG_ACC, [nxt] "=&v"(af_next) : KMOE_FRAG_W, [cur] "v"(af_cur), KMOE_FRAG_IMMS
                     : "scc", "memory");
#undef KMOE_FRAG_ACC
#undef KMOE_FRAG_W
    }
#undef KMOE_FRAG_HEAD
#undef KMOE_FRAG_OWN
#undef KMOE_FRAG_NEXT
#undef KMOE_FRAG_WAIT
#undef KMOE_FRAG_MFMA2
#undef KMOE_FRAG_MFMA4
#undef KMOE_FRAG_IMMS
  };
  // The same for tiles whose waves own TWO channel fragments (eight waves along the channels): a statement handles
  // a pair of row fragments - four MFMAs again, so that the reads of the next pair have as many clocks to arrive -
  // and the skip works on pairs (a pair with one live fragment is computed whole).
  auto frag_pair_i8 = [&](const v4i(&w)[kNF], v4i& c0, v4i& c1, v4i& n0, v4i& n1, uint32_t addr, auto p_tag, auto off_own,
                          int mf) {
    constexpr int pr = decltype(p_tag)::value;
    constexpr bool kFirst = pr == 0, kLast = 2 * pr + 2 == kMF;
    constexpr int kOwn = decltype(off_own)::value, kStep = 16 * kChunk;
#define KMOE_PAIR_HEAD "s_cmp_lt_i32 %[live], %[n1]\n\ts_cbranch_scc1 3f\n\t"
#define KMOE_PAIR_OWN "ds_read_b128 %[a0], %[addr] offset:%[o0]\n\tds_read_b128 %[a1], %[addr] offset:%[o1]\n\t"
#define KMOE_PAIR_NEXT \
  "ds_read_b128 %[b0], %[addr] offset:%[o2]\n\tds_read_b128 %[b1], %[addr] offset:%[o3]\n\ts_waitcnt lgkmcnt(2)\n\t"
#define KMOE_PAIR_WAIT "s_waitcnt lgkmcnt(0)\n\t"
#define KMOE_PAIR_MFMA                                          \
  "v_mfma_i32_16x16x64_i8 %[c00], %[w0], %[a0], %[c00]\n\t"     \
  "v_mfma_i32_16x16x64_i8 %[c01], %[w1], %[a0], %[c01]\n\t"     \
  "v_mfma_i32_16x16x64_i8 %[c10], %[w0], %[a1], %[c10]\n\t"     \
  "v_mfma_i32_16x16x64_i8 %[c11], %[w1], %[a1], %[c11]\n\t"
#define KMOE_PAIR_ACC \
  [c00] "+v"(acc[mf][0]), [c01] "+v"(acc[mf][1]), [c10] "+v"(acc[mf + 1][0]), [c11] "+v"(acc[mf + 1][1])
#define KMOE_PAIR_INS                                                                                              \
  [w0] "v"(w[0]), [w1] "v"(w[1]), [addr] "v"(addr), [live] "s"(live_frags), [n1] "n"(2 * pr + 1), [o0] "n"(kOwn),    \
      [o1] "n"(kOwn + kStep), [o2] "n"(kOwn + 2 * kStep), [o3] "n"(kOwn + 3 * kStep)
    if constexpr (kFirst && kLast)
      asm volatile(KMOE_PAIR_HEAD KMOE_PAIR_OWN KMOE_PAIR_WAIT KMOE_PAIR_MFMA "3:\n\t"
                   : KMOE_PAIR_ACC, [a0] "=&v"(c0), [a1] "=&v"(c1) : KMOE_PAIR_INS : "scc", "memory");
    else if constexpr (kFirst)
      asm volatile(KMOE_PAIR_HEAD KMOE_PAIR_OWN KMOE_PAIR_NEXT KMOE_PAIR_MFMA "3:\n\t"
                   : KMOE_PAIR_ACC, [a0] "=&v"(c0), [a1] "=&v"(c1), [b0] "=&v"(n0), [b1] "=&v"(n1) : KMOE_PAIR_INS
                   : "scc", "memory");
    else if constexpr (kLast)
      asm volatile(KMOE_PAIR_HEAD KMOE_PAIR_WAIT KMOE_PAIR_MFMA "3:\n\t"
                   : KMOE_PAIR_ACC : [a0] "v"(c0), [a1] "v"(c1), KMOE_PAIR_INS : "scc", "memory");
    else
      asm volatile(KMOE_PAIR_HEAD KMOE_PAIR_NEXT KMOE_PAIR_MFMA "3:\n\t"
                   : KMOE_PAIR_ACC, [b0] "=&v"(n0), [b1] "=&v"(n1) : [a0] "v"(c0), [a1] "v"(c1), KMOE_PAIR_INS
                   : "scc", "memory");
#undef KMOE_PAIR_HEAD
#undef KMOE_PAIR_OWN
#undef KMOE_PAIR_NEXT
#undef KMOE_PAIR_WAIT
#undef KMOE_PAIR_MFMA
#undef KMOE_PAIR_ACC
#undef KMOE_PAIR_INS
  };
  // keep: std::false_type (every fragment as read), or an int mask (0: the fragments count as zeros)
  auto compute = [&](const v4i(&wcur)[kNF], auto buf_tag, auto j_tag, auto keep) {
    constexpr int buf = decltype(buf_tag)::value, j = decltype(j_tag)::value;
    if constexpr (ADMA && I8 && !M32 && kNF == 2 && kMF % 2 == 0 && kWN == 8) {
      constexpr bool kFarStages = kStagesA * kStageBytes > 65536;
      constexpr int kImm = kFarStages ? 0 : buf * kStageBytes;
      const uint32_t addr = fa[j] + (kFarStages ? buf * kStageBytes : 0);
      v4i wm[kNF];
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        if constexpr (std::is_same_v<decltype(keep), int>) wm[f] = wcur[f] & (v4i){keep, keep, keep, keep};
        else wm[f] = wcur[f];
      }
      v4i af[4];
      auto run = [&](auto self, auto p_tag) {
        constexpr int pr = decltype(p_tag)::value;
        if constexpr (2 * pr < kMF) {
          frag_pair_i8(wm, af[(2 * pr) & 3], af[(2 * pr + 1) & 3], af[(2 * pr + 2) & 3], af[(2 * pr + 3) & 3], addr, p_tag,
                       std::integral_constant<int, kImm + 2 * pr * 16 * kChunk>{}, 2 * pr);
          self(self, std::integral_constant<int, pr + 1>{});
        }
      };
      run(run, std::integral_constant<int, 0>{});
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]), "+v"(af[2]), "+v"(af[3]));
    } else if constexpr (ADMA && I8 && !M32) {
      constexpr bool kFarStages = kStagesA * kStageBytes > 65536;
      constexpr int kImm = kFarStages ? 0 : buf * kStageBytes;
      const uint32_t addr = fa[j] + (kFarStages ? buf * kStageBytes : 0);
      // (a masked step zeroes the WEIGHTS: integers have no infinity that a zero could turn into NaN)
      v4i wm[kNF];
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        if constexpr (std::is_same_v<decltype(keep), int>) wm[f] = wcur[f] & (v4i){keep, keep, keep, keep};
        else wm[f] = wcur[f];
      }
      v4i af[2];
      auto run = [&](auto self, auto n_tag) {
        constexpr int n = decltype(n_tag)::value;
        if constexpr (n < kMF) {
          frag_i8(wm, af[n & 1], af[(n + 1) & 1], addr, n_tag, std::integral_constant<int, kImm + n * 16 * kChunk>{},
                  std::integral_constant<int, kImm + (n + 1 < kMF ? n + 1 : n) * 16 * kChunk>{}, n);
          self(self, std::integral_constant<int, n + 1>{});
        }
      };
      run(run, std::integral_constant<int, 0>{});
      // (retires the request a live fragment made for a dead one; the two registers count as in use until here)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]));
    } else if constexpr (ADMA) {
      // two fragments in flight: the read of fragment n + 1 leaves before the MFMAs of fragment n
      v4i af[2];
      // (the instruction's offset field has 16 bits: with 32 KB buffers the buffer's offset goes into the address)
      constexpr bool kFarStages = kStagesA * kStageBytes > 65536;
      constexpr int kImm = kFarStages ? 0 : buf * kStageBytes;
      uint32_t fa_s[2];
      fa_s[0] = fa[M32 ? 2 * j : j] + (kFarStages ? buf * kStageBytes : 0);
      fa_s[1] = M32 ? fa[2 * j + 1] + (kFarStages ? buf * kStageBytes : 0) : fa_s[0];
      af[0] = lds_read16_raw<kImm>(fa_s[0]);
#pragma unroll
      for (int n = 0; n < kFragReads; ++n) {
        const int mf = M32 ? n % AM : n, t = M32 ? n / AM : 0;
        if (n + 1 < kFragReads) {
          const int mf1 = M32 ? (n + 1) % AM : n + 1, t1 = M32 ? (n + 1) / AM : 0;
          asm volatile("ds_read_b128 %0, %1 offset:%2"
                       : "=v"(af[(n + 1) & 1])
                       : "v"(fa_s[t1]), "i"(kImm + mf1 * kFragRows * kChunk)
                       : "memory");
          lds_wait<1>(af[n & 1]);
        } else {
          lds_wait<0>(af[n & 1]);
        }
        if constexpr (std::is_same_v<decltype(keep), int>) af[n & 1] &= (v4i){keep, keep, keep, keep};
        mfma_row(wcur, af[n & 1], mf, t);
      }
    }
  };
  // F8 on the asynchronous path, one whole chunk (the two ring slots are the K halves of one MFMA): every LDS
  // access is an assembly statement (an LDS read the compiler sees waits for the copies in flight). The bytes and
  // the row scale of fragment n + 1 are requested before fragment n is waited for; fragments past the tile's rows
  // are read (whatever the buffer holds) and not multiplied.
  auto compute_f8_dma = [&](const v4i(&w_lo)[kNF], const v4i(&w_hi)[kNF], auto buf_tag, int chunk, int parity) {
    if constexpr (F8 && ADMA) {
      constexpr int buf = decltype(buf_tag)::value;
      constexpr bool kFarStages = kStagesA * kStageBytes > 65536;
      constexpr int kImm = kFarStages ? 0 : buf * kStageBytes;
      const uint32_t a_lo = fa[0] + (kFarStages ? buf * kStageBytes : 0);
      const uint32_t a_hi = fa[1] + (kFarStages ? buf * kStageBytes : 0);
      const uint32_t sc_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
          (lds_ptr_t)&asc_lds[buf][wave_m * 16 * kMF + li]));
      const uint32_t wsc_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
          (lds_ptr_t)&wsc_lds[parity][wave * kNF * kMaxKBlocks + chunk]));
      static_assert(kNF == 2, "the asynchronous fp8 path is written for two channel fragments a wave");
      float swc[kNF];
      lds_request_b32<0>(swc[0], wsc_addr);
      lds_request_b32<kMaxKBlocks * 4>(swc[1], wsc_addr);
      v4i lo[2], hi[2];
      float sar[2];
      f8_request<kImm, 0>(lo[0], hi[0], sar[0], a_lo, a_hi, sc_addr);
      v4f blk[2][kNF];     // partial sums of the fragment whose MFMAs were issued last, and of the one before
      float scp[2][kNF];   // ... and their scales
      auto run = [&](auto self, auto n_tag) {
        constexpr int n = decltype(n_tag)::value;
        if constexpr (n < kMF) {
          if constexpr (n + 1 < kMF) {
            f8_request<kImm + (n + 1) * 16 * kChunk, (n + 1) * 64>(lo[(n + 1) & 1], hi[(n + 1) & 1], sar[(n + 1) & 1], a_lo, a_hi,
                                                                  sc_addr);
            f8_wait<3>(lo[n & 1], hi[n & 1], sar[n & 1], swc[0], swc[1]);
          } else {
            f8_wait<0>(lo[n & 1], hi[n & 1], sar[n & 1], swc[0], swc[1]);
          }
          // the scaling of fragment n - 1 follows the MFMAs of fragment n: the wave does not wait for the matrix pipe
          if (n < live_frags) {  // (wave-uniform)
            v8i av;
            av.lo = lo[n & 1];
            av.hi = hi[n & 1];
#pragma unroll
            for (int f = 0; f < kNF; ++f) {
              v8i wv;
              wv.lo = w_lo[f];
              wv.hi = w_hi[f];
              blk[n & 1][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, av, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0,
                                                                              0x7f7f7f7f, 0, 0x7f7f7f7f);
              scp[n & 1][f] = sar[n & 1] * swc[f];
            }
          }
          if constexpr (n > 0) {
            if (n - 1 < live_frags) {
#pragma unroll
              for (int f = 0; f < kNF; ++f)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                  acc[n - 1][f][q] = __builtin_fmaf(blk[(n - 1) & 1][f][q], scp[(n - 1) & 1][f], acc[n - 1][f][q]);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          self(self, std::integral_constant<int, n + 1>{});
        }
      };
      run(run, std::integral_constant<int, 0>{});
      if (kMF - 1 < live_frags) {
#pragma unroll
        for (int f = 0; f < kNF; ++f)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            acc[kMF - 1][f][q] = __builtin_fmaf(blk[(kMF - 1) & 1][f][q], scp[(kMF - 1) & 1][f], acc[kMF - 1][f][q]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // F8, one whole chunk: the two ring slots of the chunk are the K halves of one MFMA
  auto compute_f8 = [&](const v4i(&w_lo)[kNF], const v4i(&w_hi)[kNF], int buf, int chunk, int parity) {
    if constexpr (!M32) {
    float swc[kNF];
#pragma unroll
    for (int f = 0; f < kNF; ++f) swc[f] = wsc_lds[parity][(wave * kNF + f) * kMaxKBlocks + chunk];
#pragma unroll
    for (int mf = 0; mf < kMF; ++mf) {
      const int row = wave_m * 16 * kMF + mf * 16 + li;
      v8i av;
      av.lo = *reinterpret_cast<const v4i*>(&lds_a[buf][row * kPitchT + lg * 16]);
      av.hi = *reinterpret_cast<const v4i*>(&lds_a[buf][row * kPitchT + 64 + lg * 16]);
      const float sa = asc_lds[buf][row];
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        v8i wv;
        wv.lo = w_lo[f];
        wv.hi = w_hi[f];
        const v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, av, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0,
                                                                         0x7f7f7f7f, 0, 0x7f7f7f7f);
        const float sc = sa * swc[f];
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[mf][f][q] = __builtin_fmaf(blk[q], sc, acc[mf][f][q]);
      }
      // keep the partial sums of one row fragment at a time in registers: without the fence the
      // scheduler issues all 32 MFMAs first and spills their 128 results
      __builtin_amdgcn_sched_barrier(0);
    }
    }
  };
  // Gather index of sorted row r of tile t (rows past the expert's end: the tile's first row),
  // and the source row (row of p.a / p.a_max) it names. With a gather the value fetched is returned as loaded,
  // untouched: any arithmetic on it here would make the wave wait for the load - and with it for every older
  // load and store - at the loop top instead of after the MFMA loop.
  auto fetch_src = [&](const Tile& t, int r) -> int {
    const int rr = r < t.end ? r : t.row0;
    if (!p.row_src) return rr;
    return p.row_src[t.e < p.E ? rr : 0];  // always one load (the tail expert's rows are not gathered: value unused)
  };
  // gather entries are flat (source row, slot) ids: source row = entry / src_div (a shift for the usual powers of two)
  const int src_shift = (p.src_div & (p.src_div - 1)) == 0 ? __builtin_ctz(p.src_div) : -1;
  auto src_row = [&](const Tile& t, int r, int fetched) -> int {
    if (t.e >= p.E) return p.tail_src0 + (r < t.end ? r : t.row0) - p.tail_row0;
    if (!p.row_src) return fetched;
    return src_shift >= 0 ? fetched >> src_shift : fetched / p.src_div;
  };
  auto col_of = [&](const Tile& t, int f, bool& ok) -> int {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = (t.nb * kWN + wave) * NFH * 16 + fh * 16;
    ok = c < n_half;
    return (SWIGLU && f >= NFH) ? n_half + c : c;
  };

  // tile row and byte column (within a chunk) of this thread's i-th activation vector
  auto a_row = [&](int i) -> int { return ADMA ? dma_row + 8 * i : (threadIdx.x + i * kThreads) >> 3; };
  const uint32_t a_col = ADMA ? dma_vec * 16u : (threadIdx.x & 7) * 16u;  // kThreads % 8 == 0
  // ---- pacing against sibling tiles (see g_board) ----
  uint32_t* const my_slot = &g_board[blockIdx.x * kBoardStride];
  const uint32_t* const no_slot = my_slot + 1;  // second word of the own line, never written: 0 = "nobody to wait for"
  const uint32_t* prev_slot = no_slot;
  const uint32_t* next_slot = no_slot;
  uint32_t seen_prev = 0, seen_next = 0;  // the neighbours' progress as polled one chunk ago (wave-uniform)
  int patience = 0;
  if constexpr (PACE) __hip_atomic_store(my_slot, 1u << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // Waits (bounded by `patience`) while the workgroup behind `slot` is more than the allowed slack behind `prog`.
  // One opaque instruction to the compiler: a visible branch here would split the MFMA loop's basic block.
  auto wait_for = [&](uint32_t& seen, const uint32_t* slot, uint32_t prog) {
    uint32_t tmp;
    const uint32_t lim = prog - kSyncSlack;
    asm volatile(
        "s_cmp_eq_u32 %[seen], 0\n\t"
        "s_cbranch_scc1 2f\n"
        "1:\n\t"
        "s_cmp_ge_u32 %[seen], %[lim]\n\t"
        "s_cbranch_scc1 2f\n\t"
        "s_cmp_lt_i32 %[pat], 1\n\t"
        "s_cbranch_scc1 2f\n\t"
        "s_sub_u32 %[pat], %[pat], 1\n\t"
        "s_sleep 4\n\t"
        "global_load_dword %[tmp], %[zero], %[slot] sc1\n\t"
        "s_waitcnt vmcnt(0)\n\t"
        "v_readfirstlane_b32 %[seen], %[tmp]\n\t"
        "s_branch 1b\n"
        "2:\n\t"
        : [seen] "+s"(seen), [pat] "+s"(patience), [tmp] "=&v"(tmp)
        : [lim] "s"(lim), [slot] "s"(slot), [zero] "v"(0)
        : "scc", "memory");
  };
  // The siblings' progress is polled with loads that go past this CU's L1; such a load takes longer than a
  // chunk, and a wave's loads return in order, so the polls are issued AFTER the chunk's own loads and the
  // chunk's wait leaves them in flight: they have a whole further chunk to arrive (polled[parity of the chunk]).
  uint32_t polled[2][2] = {{0, 0}, {0, 0}};
  constexpr int kPolls = PACE ? 2 : 0;  // loads per chunk on top of the chunk's own
  // start of chunk `chunk` of item `it`: publish it, wait for siblings that have fallen behind
  auto pace = [&](int it, int chunk) {
    if constexpr (!PACE) return;
    const uint32_t prog = (static_cast<uint32_t>(it + 1) << 16) | static_cast<uint32_t>(chunk);
    // one lane stores (64 lanes writing one address through to memory cost a third of the kernel's time)
    uint64_t saved_exec;
    asm volatile(
        "s_mov_b64 %[ex], exec\n\t"
        "s_mov_b64 exec, 1\n\t"
        "global_store_dword %[zero], %[val], %[slot] \n\t"
        "s_mov_b64 exec, %[ex]\n\t"
        : [ex] "=&s"(saved_exec)
        : [zero] "v"(0), [val] "v"(prog), [slot] "s"(my_slot)
        : "memory");
    wait_for(seen_prev, prev_slot, prog);
    wait_for(seen_next, next_slot, prog);
  };
  auto pace_poll = [&](auto parity_tag) {  // after the chunk's loads have been issued
    if constexpr (!PACE) return;
    constexpr int q = decltype(parity_tag)::value;
    polled[q][0] = __hip_atomic_load(prev_slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    polled[q][1] = __hip_atomic_load(next_slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  auto pace_collect = [&](auto parity_tag, int chunk) {  // after the chunk's wait: the PREVIOUS chunk's polls are in
    if constexpr (!PACE) return;
    constexpr int q = decltype(parity_tag)::value ^ 1;
    const uint32_t a = __builtin_amdgcn_readfirstlane(polled[q][0]);
    const uint32_t b = __builtin_amdgcn_readfirstlane(polled[q][1]);
    seen_prev = chunk > 0 ? a : 0u;  // (a tile's first chunk would collect the polls of the tile before)
    seen_next = chunk > 0 ? b : 0u;
  };
  Tile cur = find_tile(0);
  if (!cur.valid || not_my_launch) {  // the whole workgroup leaves together
    if constexpr (PACE) __hip_atomic_store(my_slot, 0xffffffffu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  int rs[kNA];             // gather indices of this thread's activation rows
#pragma unroll
  for (int i = 0; i < kNA; ++i) rs[i] = fetch_src(cur, cur.row0 + a_row(i));
  // gather index of the tile row whose scale this thread fetches (I8: row threadIdx.x; F8: threadIdx.x % kTM)
  const int scale_row = F8 ? threadIdx.x % kTM : min(static_cast<int>(threadIdx.x), kTM - 1);
  int rs_scale = fetch_src(cur, cur.row0 + scale_row);
  float wsc_reg[kMaxKBlocks / 16];     // F8: weight block scales k = c, c + 16, ... of fragment lane / 16

  // Points the loaders at tile t and requests its first chunk, first three weight steps and scales.
  auto start_tile = [&](const Tile& t, int t_parity) {
    const int8_t* w_base = t.e >= p.E ? p.w_tail : p.w + static_cast<size_t>(t.e) * p.n * p.k;
    [[maybe_unused]] const float* w_max = t.e >= p.E ? p.w_max_tail : p.w_max + static_cast<size_t>(t.e) * p.n;
    w_rsrc = make_rsrc(w_base);
    if constexpr (M32) {
      // lane: channel lane % 32 of the fragment = row lane % 16 of block (lane / 16) % 2; K quarter lane / 32 (+ 2 t)
#pragma unroll
      for (int g = 0; g < AN; ++g) {
        bool ok;
        const int c = col_of(t, 2 * g + ((lane >> 4) & 1), ok);
        woff[g] = static_cast<uint32_t>(ok ? c / 16 : 0) * ksteps * 1024u + (lane >> 5) * 256u + (lane & 15) * 16u;
      }
    } else {
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        bool ok;
        const int c = col_of(t, f, ok);
        woff[f] = static_cast<uint32_t>(ok ? c / 16 : 0) * ksteps * 1024u + lane * 16u;
      }
    }
#pragma unroll
    for (int i = 0; i < kNA; ++i)
      aoff[i] = static_cast<uint32_t>(src_row(t, t.row0 + a_row(i), rs[i])) * static_cast<uint32_t>(p.lda) + a_col;  // < 4 GiB: host-checked
    if constexpr (F8) my_srow = src_row(t, t.row0 + scale_row, rs_scale);
    load_a(0);
    dma_a(0, 0);
    dma_a(1, 1);
    dma_a(2, 2);
    if constexpr (I8) {
      // the tile's absmax values travel the same way, 4 bytes per lane, straight into the slots
      // their scales will occupy (the loop top divides them by 127 in place)
      if (wave_m == 0 && (lane >> 4) < kNF) {  // lane = 16 f + c: channel c of fragment f of this wave
        bool ok;
        const int c = col_of(t, lane >> 4, ok);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(w_max), (lds_ptr_t)&sw_lds[t_parity][wave * kNF * 16], 4,
                                                 static_cast<uint32_t>(ok ? c + (lane & 15) : 0) * 4u, 0, 0, 0);
      }
      if (wave_id * kWave < kTM)  // thread r: tile row r
        __builtin_amdgcn_raw_ptr_buffer_load_lds(make_rsrc(p.a_max), (lds_ptr_t)&sa_lds[t_parity][wave_id * kWave], 4,
                                                 static_cast<uint32_t>(src_row(t, t.row0 + scale_row, rs_scale)) * 4u, 0, 0,
                                                 0);
    }
    __builtin_amdgcn_sched_barrier(0);  // the weight loads below stay younger than the copies above (see the wait at the loop top)
#pragma unroll
    for (int i = 0; i < R - 1; ++i) load_w(wring[i], i);
    if constexpr (F8) {
      if (wave_m == 0 && (lane >> 4) < kNF) {  // thread (wave, f = lane / 16, c = lane % 16): block scales c, c + 16, ...
        bool ok;
        const int c = col_of(t, lane >> 4, ok);
        const float* ws = (t.e >= p.E ? p.w_max_tail : p.w_max + static_cast<size_t>(t.e) * (p.n / 128) * kblocks) +
                          static_cast<size_t>(ok ? c / 128 : 0) * kblocks;
#pragma unroll
        for (int i = 0; i < kMaxKBlocks / 16; ++i) {
          const int kb = (lane & 15) + 16 * i;
          wsc_reg[i] = kb < kblocks ? ws[kb] : 0.0f;
        }
      }
    }
  };
  start_tile(cur, 0);

  for (int parity = 0;; parity ^= 1) {
    // the tile after this one: found now, its gather indices travel during the MFMA loop
    const Tile nxt = find_tile(cur.it + 1);
    // (after the last tile the loads repeat the current one's: always kNA + 1 loads, which the
    // wait below counts on)
    const Tile look = nxt.valid ? nxt : cur;
    if constexpr (PACE) {
      prev_slot = (cur.sib & 1) ? &g_board[(blockIdx.x - 8) * kBoardStride] : no_slot;
      next_slot = (cur.sib & 2) ? &g_board[(blockIdx.x + 8) * kBoardStride] : no_slot;
      seen_prev = seen_next = 0;  // nothing polled for this tile yet: its first chunk starts without waiting
      patience = kSyncPatience;
    }
    if constexpr ((ADMA && I8 && !M32) || (F8 && ADMA)) {
      const int rows_here = min(cur.end, cur.row0 + kTM) - cur.row0 - wave_m * 16 * kMF;
      live_frags = __builtin_amdgcn_readfirstlane(max(0, min(kMF, (rows_here + 15) >> 4)));
    }
    int rs_next[kNA];
#pragma unroll
    for (int i = 0; i < kNA; ++i) rs_next[i] = fetch_src(look, look.row0 + a_row(i));
    const int rs_scale_next = fetch_src(look, look.row0 + scale_row);
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (F8) {
      if (wave_m == 0 && (lane >> 4) < kNF) {
#pragma unroll
        for (int i = 0; i < kMaxKBlocks / 16; ++i) {
          float* slot = &wsc_lds[parity][(wave * kNF + (lane >> 4)) * kMaxKBlocks + (lane & 15) + 16 * i];
          if constexpr (ADMA) {  // (an LDS store the compiler sees would wait for the copies in flight)
            const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)slot));
            asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(wsc_reg[i]) : "memory");
          } else {
            *slot = wsc_reg[i];
          }
        }
      }
    }
    store_a(0);
    // ADMA: the copies of chunks 0-2 have landed - after them start_tile issued its (R - 1) kNF
    // weight loads and the lines above kNA + 1 index loads (with a gather), so that many younger
    // operations may stay in flight (the epilogue's stores among them); the barrier below then
    // publishes the chunks
    if constexpr (ADMA) {
      if (p.row_src) vmem_wait<(R - 1) * kNF + kNA + 1>();
      else vmem_wait<(R - 1) * kNF>();
    }
    if constexpr (I8) {
      // absmax -> scale in place, each slot by the thread that requested it (LDS instructions
      // the compiler does not see: no wait for the gather-index loads just issued)
      auto scale_in_place = [&](const float* slot) {
        const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)slot));
        float raw;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(raw) : "v"(addr) : "memory");
        const float scaled = raw / 127.0f;
        asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(scaled) : "memory");
      };
      if (wave_m == 0 && (lane >> 4) < kNF) scale_in_place(&sw_lds[parity][wave * kNF * 16 + lane]);
      if (threadIdx.x < kTM) scale_in_place(&sa_lds[parity][threadIdx.x]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
#pragma unroll
    for (int mf = 0; mf < AM; ++mf)
#pragma unroll
      for (int f = 0; f < AN; ++f)
#pragma unroll
        for (int q = 0; q < kAccRegs; ++q) acc[mf][f][q] = 0;
    // ADMA: everything this wave must publish has been waited for above (the copies by count, the scale writes
    // by the LDS counter), so a bare barrier is enough; the fence of __syncthreads would also wait for the
    // weight loads and the epilogue's stores still in flight
    if constexpr (ADMA) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    } else {
      __syncthreads();
    }

    // One chunk (two MFMA steps) of the pipeline; h = position of the chunk in the ring
    // period, c0 = first chunk of the period. The fences pin the issue order: loads leave at
    // the START of the MFMA run that hides them, and each wait sits just before the first use
    // (the counters retire in issue order, so a wait lets the later loads stay in flight).
    // keep_j0: all ones, or zero for the half chunk at the end of an odd number of steps (the leftover
    // chunks below pass it; in the main loop it is a constant).
    auto chunk_step = [&](int c0, auto h_tag, auto keep_j0) {
      constexpr int h = decltype(h_tag)::value;
      constexpr int buf = ADMA ? h % kStagesA : h & 1;
      using buf_t = std::integral_constant<int, buf>;
      using j0_t = std::integral_constant<int, 0>;
      using j1_t = std::integral_constant<int, 1>;
      const int s0 = (c0 + h) * kSteps;
      pace(cur.it, c0 + h);
      __builtin_amdgcn_sched_barrier(0);
      load_a(c0 + h + 1);
      load_w(wring[(2 * h + R - 1) % R], s0 + R - 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (F8 && ADMA) {
        compute_f8_dma(wring[(2 * h) % R], wring[(2 * h + 1) % R], buf_t{}, c0 + h, parity);
        __builtin_amdgcn_sched_barrier(0);
        load_w(wring[(2 * h) % R], s0 + R);
        dma_a(c0 + h + kStagesA - 1, (buf + kStagesA - 1) % kStagesA);
      } else if constexpr (F8) {
        compute_f8(wring[(2 * h) % R], wring[(2 * h + 1) % R], buf, c0 + h, parity);
        __builtin_amdgcn_sched_barrier(0);
        load_w(wring[(2 * h) % R], s0 + R);
      } else {
        compute(wring[(2 * h) % R], buf_t{}, j0_t{}, keep_j0);
        __builtin_amdgcn_sched_barrier(0);
        load_w(wring[(2 * h) % R], s0 + R);
        // the buffer chunk c - 1 was read from is free since the last barrier: chunk c + 3 goes there
        dma_a(c0 + h + kStagesA - 1, (buf + kStagesA - 1) % kStagesA);
        __builtin_amdgcn_sched_barrier(0);
        compute(wring[(2 * h + 1) % R], buf_t{}, j1_t{}, std::false_type{});
      }
      __builtin_amdgcn_sched_barrier(0);
      pace_poll(std::integral_constant<int, h & 1>{});
      __builtin_amdgcn_sched_barrier(0);
      store_a(buf ^ 1);
      // ADMA: the 12 loads above (and the two polls) may still be in flight, everything older has landed - among
      // it this wave's part of chunks c + 1 and c + 2; the barrier publishes them
      // (a bare barrier: the fence of __syncthreads would drain every load in flight, since the
      // asynchronous copies count as stores to LDS)
      if constexpr (ADMA) {
        vmem_wait<2 * kNF + kND + kPolls>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      } else {
        __syncthreads();
      }
      pace_collect(std::integral_constant<int, h & 1>{}, c0 + h);
    };
    constexpr int kPeriod = ADMA ? kStagesA : R / 2;  // chunks after which ring slots and buffers repeat
    static_assert(kPeriod == 2 || kPeriod == 4, "unrolled by hand below");
    constexpr std::false_type kFull{};
    int c = 0;
    for (; c + kPeriod <= nfull; c += kPeriod) {
      chunk_step(c, std::integral_constant<int, 0>{}, kFull);
      chunk_step(c, std::integral_constant<int, 1>{}, kFull);
      if constexpr (kPeriod == 4) {
        chunk_step(c, std::integral_constant<int, 2>{}, kFull);
        chunk_step(c, std::integral_constant<int, 3>{}, kFull);
      }
    }
    // the chunks left over (fewer than a period, the half chunk last): same steps, loads past the end are clamped
    auto keep = [&](int chunk) {
      if constexpr (ADMA) return (half_chunk && chunk == nfull) ? 0 : -1;
      else return kFull;
    };
    if (c < nchunks) chunk_step(c, std::integral_constant<int, 0>{}, keep(c));
    if constexpr (kPeriod == 4) {
      if (c + 1 < nchunks) chunk_step(c, std::integral_constant<int, 1>{}, keep(c + 1));
      if (c + 2 < nchunks) chunk_step(c, std::integral_constant<int, 2>{}, keep(c + 2));
      if constexpr (ADMA) {
        if (c + 3 < nchunks) chunk_step(c, std::integral_constant<int, 3>{}, keep(c + 3));
      }
    }

    // (the int8 MFMAs are issued from assembly statements: the compiler does not know that the accumulators come
    // out of the matrix pipe and inserts no wait states before the first VALU instruction that reads them)
    if constexpr (ADMA && I8 && !M32) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    // ---- switch: the finished tile's scales leave LDS first (LDS reads the compiler sees wait
    // for every asynchronous copy in flight, so none may follow start_tile), then the next
    // tile's first loads are requested, then this tile is finished ----
    const Tile done = cur;
    // Registers of a lane: row li of the fragment; channel-in-wave fr * kFragRows + 8 (v / 4) + 4 lg + v % 4
    // for register v of fragment fr (16x16: v < 4).
    constexpr int ANH = SWIGLU ? AN / 2 : AN;
    constexpr int kQuads = kAccRegs / 4;
    float sw[AN][kAccRegs];
    float sa_r[AM];
    if constexpr (I8) {
#pragma unroll
      for (int j = 0; j < AN * kQuads; j += 2) {
        // register quad b of fragment fr, j = fr * kQuads + b: 16x16 fragments lie 64 bytes apart, the quads of a
        // 32x32 fragment 32 bytes. (LDS reads the compiler does not see: it would wait for every load in flight.)
        constexpr int kStride = M32 ? 32 : 64;
        static_assert(M32 ? kFragRows == 32 && kQuads == 4 : kFragRows == 16 && kQuads == 1, "layout of the scale slots");
        const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                                  (lds_ptr_t)&sw_lds[parity][wave * kNF * 16 + lg * 4])) + j * kStride;
        v4f s0, s1 = {0.f, 0.f, 0.f, 0.f};
        if (j + 1 < AN * kQuads) lds_read2_b128<kStride>(s0, s1, addr);
        else lds_read1_b128(s0, addr);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          sw[j / kQuads][4 * (j % kQuads) + q] = s0[q];
          if (j + 1 < AN * kQuads) sw[(j + 1) / kQuads][4 * ((j + 1) % kQuads) + q] = s1[q];
        }
      }
      const uint32_t sa_addr = static_cast<uint32_t>(
          reinterpret_cast<uintptr_t>((lds_ptr_t)&sa_lds[parity][wave_m * 16 * kMF + li]));
#pragma unroll
      for (int mf = 0; mf < AM; mf += 4) {
        if (mf + 3 < AM) {
          lds_read4_b32<4 * kFragRows>(sa_r[mf], sa_r[mf + 1], sa_r[mf + 2], sa_r[mf + 3], sa_addr + mf * 4 * kFragRows);
        } else {
#pragma unroll
          for (int m = mf; m < AM; ++m) lds_read1_b32(sa_r[m], sa_addr + m * 4 * kFragRows);
        }
      }
    }
    // BF16 with expert biases: the four bias values of this lane's channels of every fragment, requested
    // before the next tile's loads so that waiting for them does not wait for those
    [[maybe_unused]] uint2 bias_q[AN];
    if constexpr (BF && !M32 && !SWIGLU) {
      if (p.bias) {
#pragma unroll
        for (int fr = 0; fr < AN; ++fr) {
          bool ok;
          const int c = col_of(done, fr, ok);
          bias_q[fr] = ok ? *reinterpret_cast<const uint2*>(p.bias + static_cast<size_t>(done.e) * p.n + c + lg * 4)
                          : make_uint2(0u, 0u);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (nxt.valid) {
#pragma unroll
      for (int i = 0; i < kNA; ++i) rs[i] = rs_next[i];
      rs_scale = rs_scale_next;
      cur = nxt;
      start_tile(cur, parity ^ 1);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- epilogue of `done`: dequantise, optional SiLU-mul, transpose through LDS, store ----
    const int row_end = min(done.end, done.row0 + kTM);
    bool wok[kNF];
    int col[kNF];  // per 16-channel block of this wave
#pragma unroll
    for (int f = 0; f < kNF; ++f) col[f] = col_of(done, f, wok[f]);
    // the patch is written and read with LDS instructions the compiler does not see (same reason)
    const uint32_t patch_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&patch[wave_id][0]));
    const uint32_t patch_wr = patch_base + static_cast<uint32_t>(li * kPatchPitch + lg * 8);
    [[maybe_unused]] const uint32_t patch_wr_oai = patch_base + static_cast<uint32_t>(li * kPatchPitch + lg * 4);
    // reader side of the patch: lane -> (row, 16-byte vector), consecutive lanes cover a row
    constexpr int kVecPerRow = kOutBytes / 16;        // 2, 4 or 8
    constexpr int kRowsPerRead = kWave / kVecPerRow;  // 32, 16 or 8
    constexpr int kReads = kRowsPerRead >= kFragRows ? 1 : kFragRows / kRowsPerRead;
    const int rd_row = lane / kVecPerRow, rd_vec = lane % kVecPerRow;
    const uint32_t patch_rd =
        patch_base + static_cast<uint32_t>((rd_row & (kFragRows - 1)) * kPatchPitch + rd_vec * 16);
    constexpr bool kDirectStore = !OAI && !M32 && NFH == 1;
    const int out_col0 = (done.nb * kWN + wave) * NFH * 16 / (OAI ? 2 : 1);  // first output channel of this wave
    const int n_out = OAI ? p.n / 2 : n_half;
#pragma unroll
    for (int mf0 = 0; mf0 < AM; mf0 += kPatchGroup) {
      if (mf0 >= live_frags) continue;  // (wave-uniform) fragments without rows of the tile have nothing to store
#pragma unroll
      for (int j = 0; j < kPatchGroup; ++j) {
      const int mf = mf0 + j;
      if (mf >= live_frags) continue;
      float sa = 1.0f;
      if constexpr (I8) sa = sa_r[mf];
      const int r = done.row0 + wave_m * 16 * kMF + mf * kFragRows + li;
#pragma unroll
      for (int fr = 0; fr < ANH; ++fr) {
#pragma unroll
        for (int b = 0; b < kQuads; ++b) {
          float yv[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if constexpr (!I8) yv[q] = acc[mf][fr][4 * b + q];
            else yv[q] = (static_cast<float>(acc[mf][fr][4 * b + q]) * sa) * sw[fr][4 * b + q];
          }
          if (SWIGLU) {
            const int fu = fr + ANH;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float g = F16 ? half_to_f32(f32_to_half(yv[q]))
                                  : bf16_to_f32(f32_to_bf16_hw(yv[q]));  // gate and up are 16-bit values first
              float uf;
              if constexpr (!I8) uf = acc[mf][fu][4 * b + q];
              else uf = (static_cast<float>(acc[mf][fu][4 * b + q]) * sa) * sw[fu][4 * b + q];
              const float u = F16 ? half_to_f32(f32_to_half(uf)) : bf16_to_f32(f32_to_bf16_hw(uf));
              yv[q] = silu_hw(g) * u;
            }
          }
          if constexpr (BF && !M32 && !SWIGLU) {
            if (p.bias) {  // y = bf16(bf16(gemm) + bias), as the sum of two bf16 tensors is
              const uint16_t bv[4] = {static_cast<uint16_t>(bias_q[fr].x), static_cast<uint16_t>(bias_q[fr].x >> 16),
                                      static_cast<uint16_t>(bias_q[fr].y), static_cast<uint16_t>(bias_q[fr].y >> 16)};
#pragma unroll
              for (int q = 0; q < 4; ++q) yv[q] = bf16_to_f32(f32_to_bf16_hw(yv[q])) + bf16_to_f32(bv[q]);
            }
          }
          if constexpr (OAI) {
            // (gate, up, gate, up): two outputs, at channels (fr * 16 + lg * 4) / 2 and + 1 of the wave's output
            const uint32_t o0 = swigluoai_bf16(f32_to_bf16_hw(yv[0]), f32_to_bf16_hw(yv[1]), p.oai_alpha, p.oai_limit);
            const uint32_t o1 = swigluoai_bf16(f32_to_bf16_hw(yv[2]), f32_to_bf16_hw(yv[3]), p.oai_alpha, p.oai_limit);
            asm volatile("ds_write_b32 %0, %1 offset:%2"
                         :
                         : "v"(patch_wr_oai), "v"(o0 | (o1 << 16)), "i"(fr * kFragRows + j * kFragRows * kPatchPitch)
                         : "memory");
          } else {
          // channel of yv[0] within the wave's output: fr * kFragRows + b * 8 + lg * 4
          const uint2 packed = F16 ? make_uint2(pack2_half(yv[0], yv[1]), pack2_half(yv[2], yv[3]))
                                   : make_uint2(pack2_bf16(yv[0], yv[1]), pack2_bf16(yv[2], yv[3]));
          if constexpr (kDirectStore) {
            // a wave that owns one 16-channel output fragment: the four lanes of a row hold its 32 bytes next to
            // each other - the transpose through LDS would write the same 32-byte pieces. (Wider waves keep the
            // transpose: 32-byte pieces where 64 are possible cost the wide down launch 10 % on Qwen3 dims.)
            const int ocol = out_col0 + lg * 4;
            if (r < row_end && ocol < n_out)
              *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + ocol) = packed;
          } else {
          asm volatile("ds_write_b64 %0, %1 offset:%2"
                       :
                       : "v"(patch_wr), "v"(packed), "i"((fr * kFragRows + b * 8) * 2 + j * kFragRows * kPatchPitch)
                       : "memory");
          }
          }
          if constexpr (I8) {
            const int f16 = M32 ? 2 * fr + (b >> 1) : fr;
            const int cofs = M32 ? (b & 1) * 8 + lg * 4 : lg * 4;
            if (p.acc_out && r < row_end && wok[f16]) {
              const v4i lo = {acc[mf][fr][4 * b], acc[mf][fr][4 * b + 1], acc[mf][fr][4 * b + 2], acc[mf][fr][4 * b + 3]};
              *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + col[f16] + cofs) = lo;
              if (SWIGLU) {
                const int fu = fr + ANH;
                const v4i hi = {acc[mf][fu][4 * b], acc[mf][fu][4 * b + 1], acc[mf][fu][4 * b + 2],
                                acc[mf][fu][4 * b + 3]};
                *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + col[f16 + NFH] + cofs) = hi;
              }
            }
          }
        }
      }
      }
      if constexpr (kDirectStore) continue;
      __builtin_amdgcn_wave_barrier();  // a wave's LDS operations execute in order: the reads see the writes
      // every read of the group is requested before the first one is waited for (fragments past the tile's rows
      // are read as well - whatever the patch holds - and not stored: the waits below count every read)
      v4i v[kPatchGroup][kReads];
#pragma unroll
      for (int j = 0; j < kPatchGroup; ++j)
#pragma unroll
        for (int h = 0; h < kReads; ++h)
          asm volatile("ds_read_b128 %0, %1 offset:%2"
                       : "=v"(v[j][h])
                       : "v"(patch_rd), "i"((kReads > 1 ? h * kRowsPerRead * kPatchPitch : 0) + j * kFragRows * kPatchPitch)
                       : "memory");
#pragma unroll
      for (int j = 0; j < kPatchGroup; ++j) {
#pragma unroll
        for (int h = 0; h < kReads; ++h) {
          lds_wait_upto(kPatchGroup * kReads - 1 - (j * kReads + h), v[j][h]);
          const int pr = h * kRowsPerRead + rd_row;
          const int orow = done.row0 + wave_m * 16 * kMF + (mf0 + j) * kFragRows + pr;
          const int ocol = out_col0 + rd_vec * 8;
          if (pr < kFragRows && orow < row_end && ocol < n_out)  // n_out % 8 == 0: a vector of 8 channels is all in or all out
            *reinterpret_cast<v4i*>(p.y + static_cast<size_t>(orow) * p.ldy + ocol) = v[j][h];
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    if (!nxt.valid) break;
  }
  if constexpr (PACE) __hip_atomic_store(my_slot, 0xffffffffu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <TKind KIND, bool SWIGLU, int NF, int R, int WGS, int WM, bool M32 = false, int MF = 8, bool OAI = false,
          bool PACE = false, bool F16 = false, int WN = kWavesT>
int launch_tiled(TiledParams p, int rows, hipStream_t s, int n_cu, const char* what) {
  constexpr int kTM = WM * 16 * MF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int nfh = SWIGLU ? NF / 2 : NF;
  const int n_exp = p.E + (p.w_tail ? 1 : 0);
  p.n_blocks = ceil_div(n_half, WN * nfh * 16);
  const int max_tiles = (rows + p.tail_rows) / kTM + min(n_exp, rows + p.tail_rows);
  p.max_items = p.n_blocks * max_tiles;
  if (PACE) p.m_major = 0;  // paced siblings are neighbours in the list
  // persistent workgroups: WGS per CU
  const int grid = min(min(ceil_div(p.max_items, 8) * 8, ceil_div(WGS * n_cu, 8) * 8), kBoardSlots);
  const size_t dyn = sizeof(int) * (static_cast<size_t>(p.E) + 1 + n_exp + 2);
  if (tracing_kernels())
    note_kernel("tiled_gemm_kernel<%s%s, %s, %dx%d tile, %d waves, %d per CU%s%s%s>%s",
                KIND == TKind::I8 ? "int8" : (KIND == TKind::F8 ? "fp8" : (F16 ? "f16" : "bf16")),
                (KIND != TKind::BF16 && F16) ? " -> f16" : "", SWIGLU ? "SiLU-mul" : (OAI ? "swigluoai" : "plain"), kTM,
                WN * nfh * 16 * (SWIGLU ? 2 : 1), WM * WN, WGS, M32 ? ", 32x32 MFMA" : "",
                PACE ? ", paced siblings" : "", R != 4 ? ", 8-slot weight ring" : "",
                p.pick == 1 ? " [works if few experts overflow the tile, decided on the device]"
                            : (p.pick == 2 ? " [works otherwise]" : ""));
  hipLaunchKernelGGL((tiled_gemm_kernel<KIND, SWIGLU, NF, R, WGS, WM, M32, MF, OAI, PACE, F16, WN>), dim3(grid),
                     dim3(WM * WN * kWave), dyn, s, p);
  return check_launch(what);
}

// Checks shared by both formats; fills n_cu.
int tiled_common(const TiledParams& p, int rows, int* n_cu_out, const char* what) {
  const int n_exp = p.E + (p.w_tail ? 1 : 0);
  // 32-bit buffer offsets: one expert's weights and every source row of the activations
  KMOE_REQUIRE(static_cast<int64_t>(p.n) * p.k < (1ll << 32), KMOE_ERR_SHAPE, "%s: n*k = %lld needs 32-bit offsets", what,
               static_cast<long long>(p.n) * p.k);
  KMOE_REQUIRE((static_cast<int64_t>(rows) + p.tail_src0 + p.tail_rows + 1) * p.lda < (1ll << 32), KMOE_ERR_SHAPE,
               "%s: activations span more than 4 GiB", what);
  KMOE_REQUIRE(n_exp <= kMaxExperts, KMOE_ERR_SHAPE, "%s: E=%d > %d", what, p.E, kMaxExperts - 1);
  KMOE_REQUIRE(p.ldy % 8 == 0 && reinterpret_cast<uintptr_t>(p.y) % 16 == 0, KMOE_ERR_SHAPE,
               "%s: y must be 16-byte aligned with ldy %% 8 == 0 (ldy=%lld)", what, static_cast<long long>(p.ldy));
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
      return fail(KMOE_ERR_LAUNCH, "%s: cannot query the device", what);
    n_cu = prop.multiProcessorCount;
    // KMOE_SPARE_CUS=n (read once): the persistent grids are cut for n fewer CUs, which stay free for a kernel that
    // runs beside these launches on another stream (a collective; the clock probe). Multiples of 8 keep the XCDs even.
    if (const char* spare = getenv("KMOE_SPARE_CUS")) {
      const int n = atoi(spare);
      if (n > 0 && n < n_cu) n_cu -= n;
    }
  }
  *n_cu_out = n_cu;
  return KMOE_OK;
}

// One 8-wave tile of 16 MF rows per workgroup with the eight waves side by side along the channels (32 channels
// each, all rows): no two waves ask for the same weight bytes, and seven MFMA steps of them are on their way per
// wave (8-slot ring of two fragments) - 112 KB of distinct weight bytes in flight per CU against 48 KB with two
// rows of four waves, at twice the LDS fragment reads per MFMA.
template <TKind K, int MF>
int launch_wide(TiledParams& p, int rows, hipStream_t s, int n_cu, const char* what, bool swiglu, bool f16) {
  if (f16)
    return swiglu ? launch_tiled<K, true, 2, 8, 1, 1, false, MF, false, false, true, 8>(p, rows, s, n_cu, what)
                  : launch_tiled<K, false, 2, 8, 1, 1, false, MF, false, false, true, 8>(p, rows, s, n_cu, what);
  return swiglu ? launch_tiled<K, true, 2, 8, 1, 1, false, MF, false, false, false, 8>(p, rows, s, n_cu, what)
                : launch_tiled<K, false, 2, 8, 1, 1, false, MF, false, false, false, 8>(p, rows, s, n_cu, what);
}

// 8-wave tiles of 32 MF rows, one workgroup per CU.
template <TKind K, int MF>
int launch_tall(TiledParams& p, int rows, hipStream_t s, int n_cu, const char* what, bool swiglu, bool f16) {
  if (f16)
    return swiglu ? launch_tiled<K, true, 4, 4, 1, 2, false, MF, false, false, true>(p, rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 1, 2, false, MF, false, false, true>(p, rows, s, n_cu, what);
  return swiglu ? launch_tiled<K, true, 4, 4, 1, 2, false, MF>(p, rows, s, n_cu, what)
                : launch_tiled<K, false, 4, 4, 1, 2, false, MF>(p, rows, s, n_cu, what);
}

// 64-row tiles (MF = 4) when nearly every expert fits one of them (44 rows per expert on average; at 48 the
// 96-row tiles are ahead, Qwen3 layer at 768 tokens 0.169 -> 0.158 ms, at 40 behind, 0.151 vs 0.155 ms): the launch
// is bound by the weight stream, and half the MFMAs, fragment reads and epilogue per weight byte leave more of
// the CU to it (measured, int8 gate_up / down: Qwen3 shape at 32 rows per expert 101 -> 80 us; DeepSeek-V3 shape
// at 32 rows 1426 -> 1284 / 770 -> 683 us). At 64 rows per expert half of the experts need a second tile and
// a second pass over their weights: DeepSeek-V3 gate_up 1434 -> 1585 us, so the switch sits below that.
// Also when 128-row tiles would leave most workgroups without an item (a dense GEMM of a few hundred rows: one
// expert, fp8 [rows,7168] x [4096,7168]: 102 -> 57 us at 128 rows, 105 -> 62 us at 1024, 150 -> 163 us at 4096).
// Variant 6 (and 12) forces 128 rows, 11 forces 64, 13 forces 96.
bool short_tiles(int variant, int rows, int n_experts, int n, bool swiglu, int n_cu, int max_avg_rows = 44) {
  if (variant == 11) return true;
  if (variant == 6 || variant == 8 || (variant >= 12 && variant <= 22)) return false;
  if (ceil_div(rows, n_experts) <= max_avg_rows) return true;
  const int n_blocks = ceil_div(swiglu ? n / 2 : n, kWavesT * (swiglu ? 2 : 4) * 16);
  return static_cast<long long>(rows / 128 + n_experts) * n_blocks < 2ll * n_cu;
}

}  // namespace

// variant 5: 128x256 or 64x256 tiles by the rows per expert (6, 11: one of them), 4-slot weight ring, 2 workgroups
// per CU (the shape in use); 7: 128x128 tiles, 8-slot ring; 8: 256x256 tiles, 8 waves,
// 1 workgroup per CU; 9: 128x256 tiles on the 32x32 MFMA shapes; 12: 128x256 tiles, sibling m-tiles paced
int tiled_gemm_i8(const kmoe_gemm_i8_args* a, hipStream_t s) {
  const char* what = "kmoe_grouped_gemm_i8 (tiled)";
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  TiledParams p{a->a,      a->lda,        a->a_max,      a->row_src, a->src_div,   a->w,         a->w_max, a->lod,
                a->E,      a->n,          a->k,          a->y,       a->ldy,       a->acc_out,   a->w_tail,
                a->w_max_tail, a->tail_row0, a->w_tail ? a->tail_rows : 0, a->tail_src0, 0, 0};
  int n_cu = 0;
  if (int rc = tiled_common(p, a->rows, &n_cu, what)) return rc;
  constexpr TKind K = TKind::I8;
  const int live = expected_rows(a->rows, a->rows_hint);  // (chooses the tile shape; grids and bounds keep a->rows)
  const int avg_rows = ceil_div(live + (a->w_tail ? a->tail_rows : 0), a->E + (a->w_tail ? 1 : 0));
  const bool shorter = short_tiles(a->variant, live, a->E, a->n, swiglu, n_cu);
  // 128-row 4-wave tiles whose sibling m-tiles are paced against each other (see g_board): variant 12, and the
  // second launch of the device-decided pair (variant 17). They were the default where experts have several m-tiles
  // and the launch's weights are far more than the 256 MB memory-side cache holds (a sibling that falls behind
  // fetches its weights from HBM again: DeepSeek-V3 shape at 4096 tokens, bytes fetched by L2 1.49x -> 1.08x of the
  // algorithmic ones, gate_up 1950 -> 1898 us); the evenly split wide tiles below keep the siblings together by
  // construction and are 6-12 % ahead of them at every batch, so no default path launches them any more.
  const long long weight_bytes = static_cast<long long>(a->E + (a->w_tail ? 1 : 0)) * a->n * a->k;
  const bool paced = a->variant == 12 || (a->variant == 17 && avg_rows > 96);
  // 96-row tiles between the two: from 45 to 72 rows per expert nearly every expert still fits one tile, and a
  // quarter of the 128-row tile's MFMAs (all padding there) is saved (Qwen3 shape, layer: 768 tokens 0.169 ->
  // 0.158 ms, 1024 tokens 0.191 -> 0.165 ms; at 80 rows per expert too many experts need a second tile: -4 % on
  // the Qwen3 shape, +1 % on the DeepSeek-V3 one; DeepSeek-V3 shape at 64 rows per expert: -1.6 %).
  const bool mid = a->variant == 13 || (a->variant == 0 && !shorter && avg_rows <= 72);
  // Wide tiles: 128, 192 or 256 rows x 256 channels on EIGHT waves side by side along the channels (32 channels
  // each, all the tile's rows), one workgroup per CU. No two waves of a workgroup ask for the same weight bytes,
  // seven MFMA steps of them are on their way per wave (112 KB of distinct weight bytes in flight per CU, where two
  // workgroups of four waves hold 96 KB of which the co-resident tiles of one expert duplicate a part), a weight
  // fragment feeds up to 16 MFMAs, and a tile that holds an expert whole streams the expert's weights once. Row
  // fragments past an expert's end cost nothing (see frag_pair_i8), so the height only has to be tall enough.
  // An expert's rows are split evenly over its m-tiles (resolve_item), so the tiles of one channel block take about
  // the same time, stay in step on their neighbouring workgroups and share the weight bytes in L2 without pacing.
  // Measured inside the layer (ms per layer call, same box; before = the 4-wave tiles above, two per CU, paced
  // where the weights exceed 1 GiB):
  //   DeepSeek-V3 dims, tokens 2048 / 3072 / 4096 / 6144 / 8192 / 12288 / 16384:
  //     before 2.346 / 2.589 / 2.985 / 3.738 / 4.561 / 6.406 / 8.350
  //     192-row wide 2.230 / 2.379 / 2.605 / 3.437 / 4.312 / 5.740 / 7.332
  //     128-row wide 2.198 / 2.427 / 2.864 / 3.621 / 4.440 / 6.136 / 7.949; 256-row (spills) - / - / - / 3.445 / 4.479 / 6.032 / 7.730
  //     with +1.0 on the logits of 32 experts, 4096 / 8192 tokens: before 2.989 / 4.652, 192-row wide 2.765 / 4.107
  //   Kimi-K2 dims, tokens 2048 / 4096 / 8192: before 3.339 / 3.792 / 5.800, 192-row 3.158 / 3.518 / 4.689, 128-row 3.118 / 3.515 / 5.142
  //   Qwen3 dims, tokens 2048 / 4096 / 6144 / 8192: 96-row 4-wave tiles 0.220 / 0.318 / 0.427 / 0.554,
  //     192-row wide 0.219 / 0.322 / 0.440 / 0.532, 128-row wide 0.238 / 0.333 / 0.454 / 0.582.
  // So: the 128-row wide tile where nearly every expert fits it (average + 3 sqrt(average) rows of a routed expert),
  // the 192-row one everywhere else - one tile for most experts up to 150 rows, evenly split tiles beyond.
  // Before the even split a 192-row tile next to a 32-row one fetched the expert's weights twice (DeepSeek-V3 dims
  // at 7168 tokens: 4.78 ms, now 4.00), which is what the paced 4-wave tiles and a device-decided pair of launches
  // (a wide tile while few experts overflow it, paced tiles otherwise) had been for; the pair remains as variant 17,
  // the paced tiles as variant 12; 19 / 18 / 22 (and 15 / 14 / 8, 16): 128- / 192- / 256-row wide tiles forced.
  // (an expert of up to 3 MiB stays in an XCD's 4 MB L2 while its m-tiles run: their channel blocks go side by side)
  p.m_major = static_cast<long long>(a->n) * a->k <= (3ll << 20) ? 1 : 0;
  const float avg_routed = static_cast<float>(ceil_div(live, a->E));
  const float reach = avg_routed + 3.0f * sqrtf(avg_routed);
  const bool big = weight_bytes > (1ll << 30);
  int wide = 0;  // row fragments of the wide tile (8: 128 rows, 12: 192, 16: 256), 0: none
  bool pair = false;
  switch (a->variant) {
    case 15: case 19: wide = 8; break;
    case 14: case 18: wide = 12; break;
    case 8: case 16: case 22: wide = 16; break;
    default: break;
  }
  if (a->variant == 0 && !shorter && (big || avg_rows > 72)) {
    // (small weights keep the 96-row tiles up to 72 rows per expert: Qwen3 dims at 1024 tokens 0.164 against 0.169)
    wide = reach <= 128.0f ? 8 : 12;
  } else if (a->variant == 17) {
    wide = reach <= 128.0f ? 8 : (reach <= 192.0f ? 12 : 16);
    pair = true;
  }
  if (wide) {
    const bool f16 = a->act_dtype == KMOE_DT_F16;
    p.pick = pair ? 1 : 0;
    p.pick_rows = 16 * wide;
    const int rc = wide == 8 ? launch_wide<K, 8>(p, a->rows, s, n_cu, what, swiglu, f16)
                             : (wide == 12 ? launch_wide<K, 12>(p, a->rows, s, n_cu, what, swiglu, f16)
                                           : launch_wide<K, 16>(p, a->rows, s, n_cu, what, swiglu, f16));
    if (!pair || rc != KMOE_OK) return rc;
    p.pick = 2;  // the launch below works if the wide one left
  }
  if (a->act_dtype == KMOE_DT_F16) {
    // half outputs: the shapes in use (64-, 96-, 128-row and paced 128-row tiles); the tuning variants are bf16 only
    KMOE_REQUIRE(a->variant == 0 || a->variant == 5 || a->variant == 6 || (a->variant >= 11 && a->variant <= 13) ||
                     a->variant == 17 || wide,
                 KMOE_ERR_UNSUPPORTED, "%s: variant %d is not instantiated for half outputs", what, a->variant);
    if (mid)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 6, false, false, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 6, false, false, true>(p, a->rows, s, n_cu, what);
    if (paced)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, true, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, true, true>(p, a->rows, s, n_cu, what);
    if (shorter)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what);
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what);
  }
  // The 128-channel / deep-ring shape is a tuning variant only: measured slower than the
  // 256-channel shape (Qwen3 gate_up 321 vs 299 us, DeepSeek-V3 at 4096 tokens 2292 vs 1913 us):
  // twice the workgroups re-read the activations.
  if (a->variant == 7)
    return swiglu ? launch_tiled<K, true, 2, 8, 2, 1>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 2, 8, 2, 1>(p, a->rows, s, n_cu, what);
  // (the 32x32 shapes are instantiated for the gate_up launch only: without SiLU-mul the 16-register
  // fragments of the plain epilogue do not fit two workgroups per CU)
  if (a->variant == 9 && swiglu) return launch_tiled<K, true, 4, 4, 2, 1, true>(p, a->rows, s, n_cu, what);
  if (mid)  // 96-row tiles
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 6>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 6>(p, a->rows, s, n_cu, what);
  if (paced)
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, true>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, true>(p, a->rows, s, n_cu, what);
  if (shorter)
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what);
  return swiglu ? launch_tiled<K, true, 4, 4, 2, 1>(p, a->rows, s, n_cu, what)
                : launch_tiled<K, false, 4, 4, 2, 1>(p, a->rows, s, n_cu, what);
}

// fp8 block-scaled operands on the same tiles (weights tiled with kmoe_tile_weights_i8: the
// re-arrangement moves bytes and does not care what they encode).
int tiled_gemm_fp8(const kmoe_gemm_fp8_args* a, hipStream_t s) {
  const char* what = "kmoe_grouped_gemm_fp8_block (tiled)";
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  KMOE_REQUIRE(a->k / 128 <= kMaxKBlocks, KMOE_ERR_UNSUPPORTED, "%s: k=%d > %d", what, a->k, 128 * kMaxKBlocks);
  TiledParams p{reinterpret_cast<const int8_t*>(a->a), a->lda, a->a_scale, a->row_src, a->src_div,
                reinterpret_cast<const int8_t*>(a->w), a->w_scale, a->lod, a->E, a->n, a->k, a->y, a->ldy, nullptr,
                reinterpret_cast<const int8_t*>(a->w_tail), a->w_scale_tail, a->tail_row0,
                a->w_tail ? a->tail_rows : 0, a->tail_src0, 0, 0};
  int n_cu = 0;
  if (int rc = tiled_common(p, a->rows, &n_cu, what)) return rc;
  constexpr TKind K = TKind::F8;
  // (64x128 tiles for a dense GEMM of a few rows, twice the work items: 57 -> 42 us on [128,7168] x [4096,7168],
  // still bound by what one workgroup keeps in flight; not instantiated)
  const bool half = a->act_dtype == KMOE_DT_F16;  // half outputs: the same three shapes
  const int live = expected_rows(a->rows, a->rows_hint);
  if (short_tiles(a->variant, live, a->E, a->n, swiglu, n_cu)) {
    if (half)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what);
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what);
  }
  // (Paced sibling m-tiles - variant 12 - had been the default where experts have several m-tiles, the weights are
  // far more than the memory-side cache holds and a tile walks a long K. With an expert's rows split evenly over
  // its m-tiles the plain 128-row tiles are 2-4 % ahead of them at every batch: DeepSeek-V3 dims, layer at 2048 /
  // 4096 / 8192 / 12288 tokens 2.588 / 3.537 / 5.815 / 8.291 ms paced against 2.474 / 3.497 / 5.694 / 7.991.)
  const int avg_rows = ceil_div(live + (a->w_tail ? a->tail_rows : 0), a->E + (a->w_tail ? 1 : 0));
  // 96-row tiles from 45 to 76 rows per expert: the padding rows of a 128-row tile cost this format its scaling work
  // on top of the MFMAs (gate_up GEMM alone, 64 rows per expert: Qwen3 shape 105 -> 85 us, DeepSeek-V3 shape 1515 ->
  // 1407 us; at 80 rows 107 -> 103 and 1541 -> 1508 us; at 90 rows the DeepSeek-V3 shape loses, 1578 -> 1812 us:
  // too many experts need a second tile)
  if (a->variant == 13 || (a->variant == 0 && avg_rows <= 76)) {
    if (half)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 6, false, false, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 6, false, false, true>(p, a->rows, s, n_cu, what);
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 6>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 6>(p, a->rows, s, n_cu, what);
  }
  const long long weight_bytes = static_cast<long long>(a->E + (a->w_tail ? 1 : 0)) * a->n * a->k;
  const int avg_routed = ceil_div(live, a->E);
  // Wide tiles (eight waves side by side, 192 or 128 rows, as for int8) on the ASYNCHRONOUS activation path: chunks
  // and their row scales copied global -> LDS three chunks ahead, every LDS access in assembly, row fragments past a
  // tile's rows not multiplied, an expert's rows split evenly over its tiles. This format gains less from them than
  // int8 (its loop scales every chunk's partial sums, whatever the tile), and only where nearly every expert fills
  // most of one 192-row tile: layer, tokens -> ms against the 4-wave tiles, DeepSeek-V3 dims 3072 / 4096 / 6144 /
  // 8192 / 12288: 2.880 / 3.535 / 4.705 / 5.792 / 8.236 -> 2.881 / 3.326 / 4.653 / 6.001 / 7.989; Kimi-K2 dims 2048 /
  // 4096 / 8192: 3.301 / 4.021 / 6.696 -> 3.501 / 4.360 / 6.322 (128-row wide: 3.330 / 4.050 / 6.693). So by default
  // from 112 to 200 rows per expert with weights beyond 1 GiB; 18 / 19 force the 192- / 128-row wide tile.
  if (a->variant == 18 || (a->variant == 0 && weight_bytes > (1ll << 30) && avg_routed >= 112 && avg_routed <= 200))
    return launch_wide<K, 12>(p, a->rows, s, n_cu, what, swiglu, half);
  if (a->variant == 19) return launch_wide<K, 8>(p, a->rows, s, n_cu, what, swiglu, half);
  // One 8-wave tile of 192 rows per expert on two rows of four waves (register path): variant 14, and the first
  // launch of the device-decided pair (variant 17); the wide tiles above took over where it had been the default.
  const bool by_rule = a->variant == 17 && avg_routed >= 124 && avg_routed <= 168;
  if (a->variant == 14 || by_rule) {
    p.pick = by_rule ? 1 : 0;
    p.pick_rows = 192;
    const int rc = launch_tall<K, 6>(p, a->rows, s, n_cu, what, swiglu, half);
    if (!by_rule || rc != KMOE_OK) return rc;
    p.pick = 2;
  }
  if (a->variant == 8) return launch_tall<K, 8>(p, a->rows, s, n_cu, what, swiglu, half);
  if (a->variant == 12) {
    if (half)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, true, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, true, true>(p, a->rows, s, n_cu, what);
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, true>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, true>(p, a->rows, s, n_cu, what);
  }
  if (half)
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what);
  return swiglu ? launch_tiled<K, true, 4, 4, 2, 1>(p, a->rows, s, n_cu, what)
                : launch_tiled<K, false, 4, 4, 2, 1>(p, a->rows, s, n_cu, what);
}

// bf16 operands: the same tiles on the byte view of the tensors ([E, n, 2k] bytes, tiled with
// kmoe_tile_weights_i8; activations [rows, 2k] bytes).
int tiled_gemm_bf16(const kmoe_gemm_bf16_args* a, hipStream_t s) {
  const char* what = "kmoe_grouped_gemm_bf16 (tiled)";
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  TiledParams p{reinterpret_cast<const int8_t*>(a->a), a->lda * 2, nullptr, a->row_src, a->src_div,
                reinterpret_cast<const int8_t*>(a->w), nullptr, a->lod, a->E, a->n, a->k * 2, a->y, a->ldy, nullptr,
                nullptr, nullptr, 0, 0, 0, 0, 0};
  int n_cu = 0;
  if (int rc = tiled_common(p, a->rows, &n_cu, what)) return rc;
  constexpr TKind K = TKind::BF16;
  p.bias = a->bias;
  p.oai_alpha = a->act_alpha;
  p.oai_limit = a->act_limit;
  const bool shorter = short_tiles(a->variant, expected_rows(a->rows, a->rows_hint), a->E, a->n, swiglu, n_cu, 40);  // measured: at 48 rows per expert the 128-row tiles are 4 % ahead
  if (a->act == KMOE_ACT_SWIGLUOAI)
    return shorter ? launch_tiled<K, false, 4, 4, 2, 1, false, 4, true>(p, a->rows, s, n_cu, what)
                   : launch_tiled<K, false, 4, 4, 2, 1, false, 8, true>(p, a->rows, s, n_cu, what);
  if (a->act_dtype == KMOE_DT_F16) {  // half operands and results (no bias, no interleaved activation: checked by the caller)
    if (shorter)
      return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what)
                    : launch_tiled<K, false, 4, 4, 2, 1, false, 4, false, false, true>(p, a->rows, s, n_cu, what);
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 8, false, false, true>(p, a->rows, s, n_cu, what);
  }
  if (shorter)
    return swiglu ? launch_tiled<K, true, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what)
                  : launch_tiled<K, false, 4, 4, 2, 1, false, 4>(p, a->rows, s, n_cu, what);
  return swiglu ? launch_tiled<K, true, 4, 4, 2, 1>(p, a->rows, s, n_cu, what)
                : launch_tiled<K, false, 4, 4, 2, 1>(p, a->rows, s, n_cu, what);
}

}  // namespace kmoe
