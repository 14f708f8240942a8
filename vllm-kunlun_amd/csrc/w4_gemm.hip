// Grouped GEMM on 4-bit weights and bf16 activations (W4A16): a weight-streaming kernel for the
// decode regime and a kernel on 128-row tiles for the prefill regime (further down). In both the
// packed weights are unpacked in registers and fed to v_mfma_f32_16x16x32_bf16: a quarter of the
// bytes of the bf16 path; the unpacking (23 VALU instructions per 8 weights) is what bounds the
// streaming kernel once the bytes are that few, and what the tile kernel shares among 128 rows.
//
//   weights  [E][n][k/2] bytes, two codes per byte, low nibble first, code c means c - 8
//            (dequant_int4_native, quantization/kernels/quant_ops.py:71-86), re-arranged by
//            kmoe_tile_weights_i8(E, n, k/2): 1 KB blocks of 16 channels x 128 values. Lane
//            16 g + c of a wave reads 16 consecutive bytes of a block: the 32 values
//            k = 128 kb + 32 g + [0, 32) of channel c. Its t-th 4-byte word (8 values) is its
//            operand of the t-th MFMA of the block; the activation lane (g, row) supplies the
//            same 8 values of its row. So one MFMA step covers k = 32 g + 8 t + [0, 8) for
//            g = 0..3 - not a contiguous range, which the sum does not care about.
//   scales   [E][n][k/group] bf16; a group is a multiple of 32 values, so a lane needs ONE
//            scale per block: group (128 kb + 32 g) / group_size of its channel.
//   value    bf16(float(c - 8) * scale), computed as fma(128 + c, scale, -136 scale): both
//            products and their sum are exact in f32 (8-bit x 8-bit mantissas), so the one
//            rounding is the bf16 one - the same bits as unpacking first (kmoe_dequant_w4_bf16).
//   half     (F16 instantiations: activations, scales and results are IEEE half, the dtype
//            dequant_int4_native itself produces) value = half(c - 8) * scale in half
//            arithmetic: the code is OR-ed into the mantissa of 1024.0h (whose last place
//            counts ones), 1032 is subtracted exactly and one packed multiply rounds the
//            product - the reference's own two steps, two values per instruction.
#include <type_traits>

#include "buffer_ops.h"
#include "kmoe_common.h"
#include "pair_scan.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

struct W4Params {
  const uint16_t* a;  // [a_rows, k] bf16
  int64_t lda;
  const int32_t* row_src;
  int32_t src_div;
  const uint8_t* w;       // tiled packed codes
  const uint16_t* scale;  // [E, n, k / gs] bf16
  int32_t gs;
  int32_t gs_shift;       // log2(gs / 32) when gs / 32 is a power of two, else -1
  // Element strides inside the 16 x (k / gs) scales of a fragment (16 channels), which start at channel * (k / gs) in
  // both layouts. KMOE_S_ROWMAJOR: channel k / gs, group 1. KMOE_S_FRAG16 (kmoe_tile_scales_w4): channel 1, group 16 -
  // the scales a wave needs for one block are then 32 to 128 consecutive bytes: one cache line per load instruction
  // where the row-major layout touches 16 (one per channel), and consecutive LDS banks in the wave's copy.
  int32_t s_ch, s_g;
  const int32_t* lod;
  int32_t E, n, k;
  uint16_t* y;
  int64_t ldy;
  StreamScan scan;  // SCAN instantiations of the streaming kernel: the routed pairs' expert ids instead of lod / row_src
};

constexpr int kWaves = 4;

// 128 + (byte J of v) as a float, in one full-rate instruction: v_perm_b32 puts the byte into
// mantissa bits 16-23 of 0x43000000 = 128.0f (whose unit in the last place is 2^-16, so
// bit 16 counts ones). The integer-to-float conversions run at a fraction of that rate.
template <int J>
__device__ inline float byte_plus_128(uint32_t v) {
  // selector bytes, most significant first: byte 3 of the first source, byte J of the second, zero, zero
  return __builtin_bit_cast(float, __builtin_amdgcn_perm(0x43000000u, v, 0x07000c0cu | (static_cast<uint32_t>(J) << 16)));
}

// 8 codes of one 4-byte word -> 8 bf16 values, value 2 j in the low half of register j:
// 3 instructions split the nibbles into bytes, then per value 1 v_perm and 1 fma
// ((128 + c) s - 136 s: both products have at most 16 significant bits and their sum is
// (c - 8) s, so nothing rounds before the bf16 rounding), and 1 rounding per pair
__device__ inline v4i unpack8(uint32_t word, float s, float m136s) {
  const uint32_t lo = word & 0x0f0f0f0fu;         // codes 0, 2, 4, 6 in bytes 0..3
  const uint32_t hi = (word >> 4) & 0x0f0f0f0fu;  // codes 1, 3, 5, 7
  v4i out;
  out[0] = static_cast<int>(pack2_bf16(__builtin_fmaf(byte_plus_128<0>(lo), s, m136s), __builtin_fmaf(byte_plus_128<0>(hi), s, m136s)));
  out[1] = static_cast<int>(pack2_bf16(__builtin_fmaf(byte_plus_128<1>(lo), s, m136s), __builtin_fmaf(byte_plus_128<1>(hi), s, m136s)));
  out[2] = static_cast<int>(pack2_bf16(__builtin_fmaf(byte_plus_128<2>(lo), s, m136s), __builtin_fmaf(byte_plus_128<2>(hi), s, m136s)));
  out[3] = static_cast<int>(pack2_bf16(__builtin_fmaf(byte_plus_128<3>(lo), s, m136s), __builtin_fmaf(byte_plus_128<3>(hi), s, m136s)));
  return out;
}

// The same 8 codes -> 8 half values (c - 8) * s: pair j is (code 2 j, code 2 j + 1) = byte j of lo and of hi.
template <int J>
__device__ inline int unpack2_half(uint32_t lo, uint32_t hi, v2h s2) {
  // bytes, most significant first: zero, byte J of hi, zero, byte J of lo; then the exponent of 1024.0h on both
  const uint32_t bits =
      __builtin_amdgcn_perm(hi, lo, 0x0c000c00u | (static_cast<uint32_t>(4 + J) << 16) | static_cast<uint32_t>(J)) | 0x64006400u;
  const v2h v = (__builtin_bit_cast(v2h, bits) - (v2h){(_Float16)1032.0f, (_Float16)1032.0f}) * s2;
  return __builtin_bit_cast(int, v);
}
__device__ inline v4i unpack8_half(uint32_t word, v2h s2) {
  const uint32_t lo = word & 0x0f0f0f0fu;
  const uint32_t hi = (word >> 4) & 0x0f0f0f0fu;
  v4i out;
  out[0] = unpack2_half<0>(lo, hi, s2);
  out[1] = unpack2_half<1>(lo, hi, s2);
  out[2] = unpack2_half<2>(lo, hi, s2);
  out[3] = unpack2_half<3>(lo, hi, s2);
  return out;
}

// MF: 16-row fragments per pass over the weights; NF: 16-channel fragments per wave;
// D: 128-value blocks of loads in flight per wave; F16: half activations, scales and results.
// SLDS: every wave first copies the scales of its fragments (16 channels x k / group values each, one
// contiguous piece of the scale tensor) into its own part of LDS and reads a block's scale from there.
// Read from global memory per block, a lane's 2-byte scale load touches 16 cache lines per instruction
// (16 channels, rows apart), as many as the weight load next to it moves bytes for: 20 % of the launch.
// SCAN: the launch sorts the routed pairs by expert itself (pair_scan.h): rows and gather indices come from the
// pairs' expert ids, and the workgroups of channel block 0 write what the sort's launch would have.
template <int MF, int NF, bool SWIGLU, int D, bool F16, bool SLDS, bool SCAN = false>
__global__ __launch_bounds__(kWaves* kWave) void w4_stream_kernel(const W4Params p) {
  static_assert(!SCAN || kWaves == kScanWaves, "scan_pairs is written for four waves");
  extern __shared__ uint16_t scale_lds[];  // SLDS: [kWaves][NF][16][groups]
  __shared__ typename std::conditional<SCAN, PairScanLds, int>::type scan_lds;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  constexpr int TM = 16 * MF;
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;
  const int e = blockIdx.y;
  int row_begin, row_end;
  ListedRows listed = {};
  if constexpr (SCAN) {
    listed = scan_pairs(p.scan, e, p.E, scan_lds, blockIdx.x == 0);  // (all four waves: a barrier inside)
    row_begin = listed.begin;
    row_end = listed.end;
  } else {
    row_begin = p.lod[e];
    row_end = p.lod[e + 1];
  }
  if (row_begin >= row_end) return;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int col_base = (blockIdx.x * kWaves + wave) * NFH * 16;
  if (col_base >= n_half) return;
  const int kblocks = p.k / 128;
  const int groups = p.k / p.gs;
  const uint8_t* w_base = p.w + static_cast<size_t>(e) * p.n * (p.k / 2);
  const uint16_t* s_base = p.scale + static_cast<size_t>(e) * p.n * groups;

  // group of this lane's 32 values of block kb: (128 kb + 32 lg) / gs
  auto group_of = [&](int kb) { return p.gs_shift >= 0 ? (4 * kb + lg) >> p.gs_shift : (4 * kb + lg) / (p.gs / 32); };
  const uint8_t* wp[NF];
  const uint16_t* sp[NF];
  int soff[NF];  // SLDS: this lane's channel row in the wave's LDS copy
  bool wok[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    const int ch0 = wok[f] ? col[f] : 0;  // fragments past the last channel read fragment 0: never stored
    wp[f] = w_base + static_cast<size_t>(ch0 / 16) * kblocks * 1024 + lane * 16;
    sp[f] = s_base + static_cast<size_t>(ch0) * groups + li * p.s_ch;
    if constexpr (SLDS) {
      // the wave's own copy; it alone reads it, so no barrier: a wave's LDS accesses complete in order
      uint32_t* dst = reinterpret_cast<uint32_t*>(scale_lds + (wave * NF + f) * 16 * groups);
      const uint32_t* src = reinterpret_cast<const uint32_t*>(s_base + static_cast<size_t>(ch0) * groups);
      for (int i = lane; i < 8 * groups; i += kWave) dst[i] = src[i];
      soff[f] = (wave * NF + f) * 16 * groups + li * p.s_ch;
    }
  }
  if constexpr (SLDS) __builtin_amdgcn_wave_barrier();  // the copies above stay above the reads below

  for (int row0 = row_begin; row0 < row_end; row0 += TM) {
    const uint16_t* ap[MF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      const int rr = r < row_end ? r : row_begin;  // rows past the end read a valid row: never stored
      int src;
      if constexpr (SCAN)
        src = listed.pair(scan_lds, rr - row_begin) / p.src_div;
      else
        src = p.row_src ? p.row_src[rr] / p.src_div : rr;
      ap[mf] = p.a + static_cast<size_t>(src) * p.lda + 32 * lg;
    }
    v4f acc[MF][NF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf)
#pragma unroll
      for (int f = 0; f < NF; ++f) acc[mf][f] = (v4f){0.f, 0.f, 0.f, 0.f};

    v4i wreg[D][NF];
    uint16_t sreg[D][NF];
    v4i areg[D][MF][4];
    auto load_block = [&](int slot, int kb) {
      const int g = group_of(kb);
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        wreg[slot][f] = *reinterpret_cast<const v4i*>(wp[f] + static_cast<size_t>(kb) * 1024);
        if constexpr (!SLDS) sreg[slot][f] = sp[f][g * p.s_g];
      }
#pragma unroll
      for (int mf = 0; mf < MF; ++mf)
#pragma unroll
        for (int t = 0; t < 4; ++t) areg[slot][mf][t] = *reinterpret_cast<const v4i*>(ap[mf] + 128 * kb + 8 * t);
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
      if (d < kblocks) load_block(d, d);

    for (int kb0 = 0; kb0 < kblocks; kb0 += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int kb = kb0 + d;
        if (kb < kblocks) {
#pragma unroll
          for (int f = 0; f < NF; ++f) {
            if constexpr (SLDS) sreg[d][f] = scale_lds[soff[f] + group_of(kb) * p.s_g];
            if constexpr (F16) {
              const _Float16 sh = __builtin_bit_cast(_Float16, sreg[d][f]);
              const v2h s2 = {sh, sh};
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const v4i wv = unpack8_half(static_cast<uint32_t>(wreg[d][f][t]), s2);
#pragma unroll
                for (int mf = 0; mf < MF; ++mf)
                  acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wv),
                                                                      __builtin_bit_cast(v8h, areg[d][mf][t]),
                                                                      acc[mf][f], 0, 0, 0);
              }
            } else {
              const float s = bf16_to_f32(sreg[d][f]);
              const float m136s = -136.0f * s;
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const v4i wv = unpack8(static_cast<uint32_t>(wreg[d][f][t]), s, m136s);
#pragma unroll
                for (int mf = 0; mf < MF; ++mf)
                  acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wv),
                                                                       __builtin_bit_cast(v8bf, areg[d][mf][t]),
                                                                       acc[mf][f], 0, 0, 0);
              }
            }
          }
          if (kb + D < kblocks) load_block(d, kb + D);
        }
      }
    }

    // epilogue: as the bf16 grouped GEMM - round to bf16, optional SiLU-mul on the bf16 values
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      if (r >= row_end) continue;
#pragma unroll
      for (int f = 0; f < NFH; ++f) {
        if (!wok[f]) continue;
        const int c0 = col[f] + lg * 4;
        uint16_t yv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) yv[q] = f32_to_act(acc[mf][f][q], F16);
        if (SWIGLU) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            yv[q] = f32_to_act(silu_hw(act_to_f32(yv[q], F16)) * act_to_f32(f32_to_act(acc[mf][f + NFH][q], F16), F16), F16);
        }
        const uint2 packed = make_uint2(yv[0] | (static_cast<uint32_t>(yv[1]) << 16),
                                        yv[2] | (static_cast<uint32_t>(yv[3]) << 16));
        *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) = packed;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// Prefill regime: tiles of 64, 96 or 128 rows. The unpacking of a weight word is shared by the row fragments of
// the tile (23 VALU instructions against 8 MFMAs of 16 cycles on the tallest), so the kernel is bound by the matrix cores
// like the 16-bit tile kernels while it reads a quarter of their weight bytes. One workgroup: up to 128 sorted
// rows of one expert x 4 waves x NF fragments of 16 channels. Activations are copied global -> LDS
// asynchronously, one 128-value block of K (256 bytes per row) ahead, two buffers; every wave reads its A
// fragments from there. Weights and their scales go global -> registers, one block ahead; they never pass
// through LDS.

// Work item `item` = (m-tile, channel block) when every expert's rows are cut into tiles of kTileRows and the
// items are numbered m-tile by m-tile: expert, first row and channel block (false: no such item). The hardware
// deals workgroups to the 8 XCDs in turn, so workgroup b takes item (b % 8) * ceil(items / 8) + b / 8: the
// workgroups of one XCD, which share an L2, walk consecutive items - the channel blocks of one m-tile (the same
// activation rows) and the m-tiles of one expert (the same weights). Dealt the other way round, every activation
// row was fetched by six L2s (gate_up of the Qwen3 shape at 8192 tokens: 2.2 GB fetched for 0.5 GB of operands).
template <int kTileRows>
__device__ inline bool locate_w4_item(const W4Params& p, int n_blocks, int& e_out, int& row0_out, int& nb_out) {
  const int lane = lane_id();
  const int epl = (p.E + kWave - 1) / kWave;  // experts per lane
  const int e_begin = lane * epl;
  int local = 0;
  for (int i = 0; i < epl; ++i) {
    const int e = e_begin + i;
    if (e < p.E) local += (p.lod[e + 1] - p.lod[e] + kTileRows - 1) / kTileRows;
  }
  int incl = local;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int o = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += o;
  }
  const int items = __shfl(incl, kWave - 1, kWave) * n_blocks;
  const int seg = (items + 7) >> 3;
  const int j = blockIdx.x >> 3;
  const int item = (blockIdx.x & 7) * seg + j;
  if (j >= seg || item >= items) return false;
  const int t = item / n_blocks;
  nb_out = item - t * n_blocks;
  int excl = incl - local;
  int found_e = -1, found_row = 0;
  if (t >= excl && t < incl) {
    for (int i = 0; i < epl; ++i) {
      const int e = e_begin + i;
      if (e >= p.E) break;
      const int lo = p.lod[e];
      const int tiles = (p.lod[e + 1] - lo + kTileRows - 1) / kTileRows;
      if (t < excl + tiles) {
        found_e = e;
        found_row = lo + (t - excl) * kTileRows;
        break;
      }
      excl += tiles;
    }
  }
  const int src_lane = __builtin_ctzll(__ballot(found_e >= 0));
  e_out = __shfl(found_e, src_lane, kWave);
  row0_out = __shfl(found_row, src_lane, kWave);
  return true;
}

// MF: 16-row fragments of a tile (4, 6, 8: 64-, 96- and 128-row tiles). Two workgroups per CU for every height:
// with three, the 64-row instance had 170 registers to live in and lost to the 128-row one (121 against 111 us
// over 4 to 64 rows per expert on the Qwen3 shape); with two it is a quarter ahead where experts fit its tile.
template <int MF, int NF, bool SWIGLU, bool F16, bool SLDS>
__global__ __launch_bounds__(kWaves* kWave, 2) void w4_tile_kernel(const W4Params p) {
  constexpr int kTileRows = 16 * MF;
  extern __shared__ uint16_t scale_lds[];  // SLDS: [kWaves][NF][16][groups], every wave its own part (as in the streaming kernel)
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  constexpr int NA = kTileRows / 4 / kWaves;  // asynchronous copies per wave and block: 4 rows (1 KB) each
  constexpr int kWaveRows = 4 * NA;           // tile rows a wave copies
  constexpr int kBufBytes = kTileRows * 256;
  // Row r of a block sits at r * 256; its 16-byte vector v at position v ^ (r % 16): the 16 rows of a
  // fragment read (same vector, rows r, r + 1, ...) fall on 16 different bank groups without padding, which
  // the asynchronous copies (1 KB of consecutive LDS bytes per instruction) could not write.
  __shared__ __attribute__((aligned(1024))) int8_t lds_a[2][kBufBytes];
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  int e, row0, nb;
  if (!locate_w4_item<kTileRows>(p, (n_half + kWaves * NFH * 16 - 1) / (kWaves * NFH * 16), e, row0, nb)) return;
  const int row_end = min(p.lod[e + 1], row0 + kTileRows);
  const int col_base = (nb * kWaves + wave) * NFH * 16;
  const int kblocks = p.k / 128;
  const int groups = p.k / p.gs;
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(p.a);
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(p.w + static_cast<size_t>(e) * p.n * (p.k / 2));
  const __amdgpu_buffer_rsrc_t s_rsrc = make_rsrc(p.scale + static_cast<size_t>(e) * p.n * groups);
  auto group_of = [&](int kb) { return p.gs_shift >= 0 ? (4 * kb + lg) >> p.gs_shift : (4 * kb + lg) / (p.gs / 32); };

  uint32_t woff[NF], soff[NF];
  bool wok[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    const int ch0 = wok[f] ? col[f] : 0;  // fragments past the last channel read fragment 0: never stored
    woff[f] = static_cast<uint32_t>(ch0 / 16) * kblocks * 1024u + lane * 16u;
    soff[f] = (static_cast<uint32_t>(ch0) * groups + li * p.s_ch) * 2u;
    if constexpr (SLDS) {
      uint16_t* mine = scale_lds + (wave * NF + f) * 16 * groups;
      uint32_t* dst = reinterpret_cast<uint32_t*>(mine);
      const uint32_t* src = reinterpret_cast<const uint32_t*>(p.scale + (static_cast<size_t>(e) * p.n + ch0) * groups);
      for (int i = lane; i < 8 * groups; i += kWave) dst[i] = src[i];
      soff[f] = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)(mine + li * p.s_ch)));  // LDS byte address of the lane's channel
    }
  }
  if constexpr (SLDS) __builtin_amdgcn_wave_barrier();  // the copies above stay above the reads below (a wave's LDS accesses complete in order)
  // copy i of this wave fills tile rows kWaveRows wave + 4 i + lane / 16; the lane fetches the vector that belongs at its position
  uint32_t aoff[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int tr = kWaveRows * wave + 4 * i + lg;
    const int r = row0 + tr;
    const int rr = r < row_end ? r : row0;  // rows past the end read the tile's first row: never stored
    const int src = p.row_src ? p.row_src[rr] / p.src_div : rr;
    aoff[i] = static_cast<uint32_t>(src) * static_cast<uint32_t>(p.lda * 2) + ((li ^ (tr & 15)) << 4);  // < 4 GiB: host-checked
  }
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)&lds_a[0][0]));
  // fragment reads of MFMA step t: row li (+ 16 per fragment: same row % 16), vector 4 lg + t
  uint32_t fa[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) fa[t] = lds_base + li * 256 + (((4 * lg + t) ^ li) << 4);
  v4f acc[MF][NF];
#pragma unroll
  for (int mf = 0; mf < MF; ++mf)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[mf][f] = (v4f){0.f, 0.f, 0.f, 0.f};
  v4i wbuf[2][NF];
  uint16_t sbuf[2][NF];
  auto load_w = [&](v4i(&w)[NF], uint16_t(&sc)[NF], int kb) {
    const uint32_t g2 = static_cast<uint32_t>(group_of(kb) * p.s_g) * 2u;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      w[f] = buffer_load16(w_rsrc, woff[f], static_cast<uint32_t>(kb) * 1024u);
      if constexpr (!SLDS) sc[f] = static_cast<uint16_t>(__builtin_amdgcn_raw_buffer_load_b16(s_rsrc, soff[f] + g2, 0, 0));
    }
    if constexpr (SLDS) {
      // reads the compiler does not see (it would drain the asynchronous copies in flight before them); the wait is
      // part of the statement, so the values are there when it ends
      static_assert(NF == 4, "four scale reads per block");
      uint32_t s0, s1, s2, s3;
      asm volatile(
          "ds_read_u16 %0, %4\n\t"
          "ds_read_u16 %1, %5\n\t"
          "ds_read_u16 %2, %6\n\t"
          "ds_read_u16 %3, %7\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(s0), "=&v"(s1), "=&v"(s2), "=&v"(s3)
          : "v"(soff[0] + g2), "v"(soff[1] + g2), "v"(soff[2] + g2), "v"(soff[3] + g2)
          : "memory");
      sc[0] = static_cast<uint16_t>(s0);
      sc[1] = static_cast<uint16_t>(s1);
      sc[2] = static_cast<uint16_t>(s2);
      sc[3] = static_cast<uint16_t>(s3);
    }
  };
  auto dma_a = [&](int kb, int buf) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
      buffer_load16_to_lds(a_rsrc, (lds_ptr_t)&lds_a[buf][(kWaveRows * wave + 4 * i) * 256], aoff[i], static_cast<uint32_t>(kb) * 256u);
  };
  // one block: word t of a lane's 16 packed bytes is its operand of MFMA step t; the activation lane (lg, row)
  // supplies values 32 lg + 8 t + [0, 8) of the block, i.e. vector 4 lg + t of the row's 16
  auto compute = [&](const v4i(&w)[NF], const uint16_t(&sc)[NF], auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v4i wv[NF];
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        if constexpr (F16) {
          const _Float16 sh = __builtin_bit_cast(_Float16, sc[f]);
          wv[f] = unpack8_half(static_cast<uint32_t>(w[f][t]), (v2h){sh, sh});
        } else {
          const float s = bf16_to_f32(sc[f]);
          wv[f] = unpack8(static_cast<uint32_t>(w[f][t]), s, -136.0f * s);
        }
      }
      // two fragments in flight: the read of fragment mf + 1 leaves before the MFMAs of fragment mf
      v4i af[2];
      af[0] = lds_read16_raw<buf * kBufBytes>(fa[t]);
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) {
        if (mf + 1 < MF) {
          asm volatile("ds_read_b128 %0, %1 offset:%2"
                       : "=v"(af[(mf + 1) & 1])
                       : "v"(fa[t]), "n"(buf * kBufBytes + (mf + 1) * 16 * 256)
                       : "memory");
          lds_wait<1>(af[mf & 1]);
        } else {
          lds_wait<0>(af[mf & 1]);
        }
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          if constexpr (F16)
            acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wv[f]),
                                                                __builtin_bit_cast(v8h, af[mf & 1]), acc[mf][f], 0, 0, 0);
          else
            acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wv[f]),
                                                                 __builtin_bit_cast(v8bf, af[mf & 1]), acc[mf][f], 0, 0, 0);
        }
      }
    }
  };
  // The block after the current one is requested (weights and scales into registers, activations into the other
  // LDS buffer, which every wave finished reading before the barrier that ended the previous stage) before the
  // MFMAs of the current one; the wait at the end covers all of it, the barrier publishes the copies.
  auto stage = [&](int kb, const v4i(&w)[NF], const uint16_t(&sc)[NF], v4i(&w_next)[NF], uint16_t(&sc_next)[NF], auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    if (kb + 1 < kblocks) {
      dma_a(kb + 1, buf ^ 1);
      load_w(w_next, sc_next, kb + 1);
    }
    compute(w, sc, buf_tag);
    vmem_wait<0>();
    __syncthreads();
  };
  dma_a(0, 0);
  load_w(wbuf[0], sbuf[0], 0);
  vmem_wait<0>();
  __syncthreads();
  for (int kb = 0; kb < kblocks; kb += 2) {
    stage(kb, wbuf[0], sbuf[0], wbuf[1], sbuf[1], std::integral_constant<int, 0>{});
    if (kb + 1 < kblocks) stage(kb + 1, wbuf[1], sbuf[1], wbuf[0], sbuf[0], std::integral_constant<int, 1>{});
  }

  // epilogue: as the streaming kernel - round to the activation type, optional SiLU-mul on the rounded values
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) {
    const int r = row0 + mf * 16 + li;
    if (r >= row_end) continue;
#pragma unroll
    for (int f = 0; f < NFH; ++f) {
      if (!wok[f]) continue;
      const int c0 = col[f] + lg * 4;
      uint16_t yv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) yv[q] = f32_to_act(acc[mf][f][q], F16);
      if (SWIGLU) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          yv[q] = f32_to_act(silu_hw(act_to_f32(yv[q], F16)) * act_to_f32(f32_to_act(acc[mf][f + NFH][q], F16), F16), F16);
      }
      const uint2 packed = make_uint2(yv[0] | (static_cast<uint32_t>(yv[1]) << 16),
                                      yv[2] | (static_cast<uint32_t>(yv[3]) << 16));
      *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) = packed;
    }
  }
}

template <int MF, bool SWIGLU>
int launch_w4_tile(const W4Params& p, int rows, bool f16, hipStream_t s) {
  constexpr int NF = 4;
  constexpr int kTileRows = 16 * MF;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  // an upper bound of the work items (m-tiles x channel blocks), a multiple of 8
  const int n_blocks = ceil_div(n_half, kWaves * NFH * 16);
  const int items = (rows / kTileRows + min(p.E, rows)) * n_blocks;
  const dim3 grid(ceil_div(items, 8) * 8);
  // the scales of a wave's fragments in LDS, while two workgroups still fit a CU next to their activation buffers
  const size_t lds = static_cast<size_t>(kWaves) * NF * 16 * (p.k / p.gs) * sizeof(uint16_t);
  if (tracing_kernels())
    note_kernel("w4_tile_kernel<%d-row tiles, %s, %s, group scales in %s>", kTileRows, SWIGLU ? "SiLU-mul" : "plain",
                f16 ? "f16" : "bf16", lds <= 16 * 1024 ? "LDS" : "global memory");
  if (lds <= 16 * 1024) {
    if (f16)
      hipLaunchKernelGGL((w4_tile_kernel<MF, NF, SWIGLU, true, true>), grid, dim3(kWaves * kWave), lds, s, p);
    else
      hipLaunchKernelGGL((w4_tile_kernel<MF, NF, SWIGLU, false, true>), grid, dim3(kWaves * kWave), lds, s, p);
  } else if (f16) {
    hipLaunchKernelGGL((w4_tile_kernel<MF, NF, SWIGLU, true, false>), grid, dim3(kWaves * kWave), 0, s, p);
  } else {
    hipLaunchKernelGGL((w4_tile_kernel<MF, NF, SWIGLU, false, false>), grid, dim3(kWaves * kWave), 0, s, p);
  }
  return check_launch("kmoe_grouped_gemm_w4a16");
}

template <int MF, int NF, bool SWIGLU, int D, bool SCAN = false>
int launch_w4(const W4Params& p, bool f16, hipStream_t s) {
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const dim3 grid(ceil_div(n_half, kWaves * NFH * 16), p.E);
  const size_t lds = static_cast<size_t>(kWaves) * NF * 16 * (p.k / p.gs) * sizeof(uint16_t);
  if (tracing_kernels())
    note_kernel("w4_stream_kernel<%d rows per pass, %d channel fragments per wave, %s, %d blocks in flight, %s, group scales in %s%s>",
                16 * MF, NF, SWIGLU ? "SiLU-mul" : "plain", D, f16 ? "f16" : "bf16", lds <= 32 * 1024 ? "LDS" : "global memory",
                SCAN ? ", sorts the pairs itself" : "");
  if (lds <= 32 * 1024) {  // beyond: many small groups on a long K; the scales stay in global memory
    if (f16)
      hipLaunchKernelGGL((w4_stream_kernel<MF, NF, SWIGLU, D, true, true, SCAN>), grid, dim3(kWaves * kWave), lds, s, p);
    else
      hipLaunchKernelGGL((w4_stream_kernel<MF, NF, SWIGLU, D, false, true, SCAN>), grid, dim3(kWaves * kWave), lds, s, p);
  } else if (f16) {
    hipLaunchKernelGGL((w4_stream_kernel<MF, NF, SWIGLU, D, true, false, SCAN>), grid, dim3(kWaves * kWave), 0, s, p);
  } else {
    hipLaunchKernelGGL((w4_stream_kernel<MF, NF, SWIGLU, D, false, false, SCAN>), grid, dim3(kWaves * kWave), 0, s, p);
  }
  return check_launch("kmoe_grouped_gemm_w4a16");
}

// scales [rows = E * n][groups] -> per 16 rows [groups][16]
__global__ __launch_bounds__(256) void tile_scales_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                         long long total, int groups) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;  // index into dst
  if (i >= total) return;
  const long long frag = i / (16LL * groups);
  const int r = static_cast<int>(i - frag * 16LL * groups);
  const int g = r >> 4, c = r & 15;
  dst[i] = src[(frag * 16 + c) * groups + g];
}

// Rows per pass of the streaming kernel for a launch (1: 16, 2: 32), or 0 where the tile kernel takes over.
int w4_stream_passes(int rows, int rows_hint, int E, int k) {
  const int avg = ceil_div(expected_rows(rows, rows_hint), E);
  // (with K = 2048 the 32-row streaming pass is never the best: 12 rows per expert 75 on 16-row passes, 84 on
  // 32-row passes, 87 on 64-row tiles; 16 rows 99 / 96 / 87)
  const int one_max = k > 4096 ? 10 : 13;
  const int stream_max = k > 4096 ? 20 : 13;
  return avg <= one_max ? 1 : (avg <= stream_max ? 2 : 0);
}

}  // namespace

bool w4_gate_up_streams(int rows, int rows_hint, int E, int k) { return w4_stream_passes(rows, rows_hint, E, k) != 0; }

}  // namespace kmoe

using namespace kmoe;

extern "C" int kmoe_tile_scales_w4(const uint16_t* src, uint16_t* dst, int E, int n, int groups, kmoe_stream_t stream) {
  KMOE_REQUIRE(src && dst && src != dst, KMOE_ERR_NULL, "tile_scales_w4: NULL pointer, or in place");
  KMOE_REQUIRE(E >= 1 && n >= 16 && n % 16 == 0 && groups >= 1, KMOE_ERR_SHAPE, "tile_scales_w4: E=%d n=%d groups=%d", E, n, groups);
  const long long total = static_cast<long long>(E) * n * groups;
  hipLaunchKernelGGL(tile_scales_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, as_stream(stream), src,
                     dst, total, groups);
  return check_launch("kmoe_tile_scales_w4");
}

extern "C" int kmoe_grouped_gemm_w4a16(const kmoe_gemm_w4_args* a, kmoe_stream_t stream) {
  return grouped_gemm_w4a16_checked(a, stream, nullptr);
}

int kmoe::grouped_gemm_w4a16_checked(const kmoe_gemm_w4_args* a, kmoe_stream_t stream, const StreamScan* scan) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "grouped_gemm_w4a16: NULL args");
  KMOE_REQUIRE(a->a && a->w && a->w_scale && (a->lod || scan) && a->y, KMOE_ERR_NULL, "grouped_gemm_w4a16: NULL pointer");
  KMOE_REQUIRE(a->E >= 1 && a->rows >= 0, KMOE_ERR_SHAPE, "grouped_gemm_w4a16: E=%d rows=%d", a->E, a->rows);
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  KMOE_REQUIRE(a->act == KMOE_ACT_NONE || swiglu, KMOE_ERR_UNSUPPORTED, "grouped_gemm_w4a16: act=%d", a->act);
  KMOE_REQUIRE(a->w_layout == KMOE_W_TILED, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_w4a16: the packed weights must be tiled (kmoe_tile_weights_i8 on [E, n, k/2] bytes)");
  KMOE_REQUIRE(a->k >= 128 && a->k % 128 == 0 && a->n >= 16 && a->n % (swiglu ? 32 : 16) == 0, KMOE_ERR_SHAPE,
               "grouped_gemm_w4a16: n=%d k=%d (need k %% 128 == 0, n %% %d == 0)", a->n, a->k, swiglu ? 32 : 16);
  KMOE_REQUIRE(a->group_size >= 32 && a->group_size % 32 == 0 && a->k % a->group_size == 0, KMOE_ERR_SHAPE,
               "grouped_gemm_w4a16: group_size=%d must be a multiple of 32 that divides k=%d", a->group_size, a->k);
  KMOE_REQUIRE(a->lda >= a->k && a->lda % 8 == 0 && reinterpret_cast<uintptr_t>(a->a) % 16 == 0, KMOE_ERR_SHAPE,
               "grouped_gemm_w4a16: activations need 16-byte aligned rows (lda=%lld)", static_cast<long long>(a->lda));
  KMOE_REQUIRE(a->ldy % 4 == 0 && a->ldy >= (swiglu ? a->n / 2 : a->n), KMOE_ERR_SHAPE, "grouped_gemm_w4a16: ldy=%lld",
               static_cast<long long>(a->ldy));
  KMOE_REQUIRE(!a->row_src || a->src_div >= 1, KMOE_ERR_SHAPE, "grouped_gemm_w4a16: src_div=%d", a->src_div);
  KMOE_REQUIRE(reinterpret_cast<uintptr_t>(a->w_scale) % 4 == 0, KMOE_ERR_SHAPE, "grouped_gemm_w4a16: misaligned scales");
  KMOE_REQUIRE(a->act_dtype == KMOE_DT_BF16 || a->act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_w4a16: act_dtype=%d unknown", a->act_dtype);
  const bool f16 = a->act_dtype == KMOE_DT_F16;
  if (a->rows == 0 && !scan) return KMOE_OK;
  const int q = a->group_size / 32;
  int shift = -1;
  if ((q & (q - 1)) == 0)
    for (shift = 0; (1 << shift) < q; ++shift) {}
  KMOE_REQUIRE(a->scale_layout == KMOE_S_ROWMAJOR || a->scale_layout == KMOE_S_FRAG16, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_w4a16: scale_layout=%d unknown", a->scale_layout);
  const int groups = a->k / a->group_size;
  const bool frag16 = a->scale_layout == KMOE_S_FRAG16;
  const W4Params p{a->a, a->lda, a->row_src, a->src_div, a->w, a->w_scale, a->group_size, shift,
                   frag16 ? 1 : groups, frag16 ? 16 : 1, a->lod, a->E, a->n, a->k, a->y, a->ldy,
                   scan ? *scan : StreamScan{}};
  hipStream_t s = as_stream(stream);
  if (scan) {
    // the routed gate_up launch of a decode-sized layer, on the streaming kernel
    const int passes = w4_stream_passes(a->rows, a->rows_hint, a->E, a->k);
    KMOE_REQUIRE(swiglu && a->variant == 0 && a->row_src == nullptr && passes != 0 && scan->ids && scan->lod &&
                     scan->expert_m && scan->moe_index && scan->sorted_src && scan->n_pairs == a->rows &&
                     a->rows <= kStreamScanMaxPairs,
                 KMOE_ERR_UNSUPPORTED, "grouped_gemm_w4a16: not a launch that can sort the pairs itself");
    return passes == 1 ? launch_w4<1, 2, true, 1, true>(p, f16, s) : launch_w4<2, 2, true, 2, true>(p, f16, s);
  }
  int mf = a->variant;
  // the tile kernel reaches a source row (gathered or not: below `rows`) through a 32-bit byte offset
  const bool tile_ok = static_cast<uint64_t>(a->rows) * static_cast<uint64_t>(a->lda) * 2u + static_cast<uint64_t>(a->k) * 2u < (1ull << 32);
  if (mf == 0) {
    // rows an expert gets under uniform routing, with headroom for the spread: an expert with
    // more rows than one pass holds streams (and unpacks) its weights again. From a dozen and a half rows per
    // expert the tile kernel is ahead on its shortest tile, which is mostly padding there (later when K is long:
    // the streaming kernel's waves then live longer per weight byte); the tile grows when too many experts would
    // need a second one (gate_up, Qwen3 shape / Kimi-K2 shape with groups of 32, us: 12 rows per expert streaming
    // 75 against 87 on 64-row tiles, 16 rows 96 / 1976 against 87 / 2196, 21 rows - / 2196 against - / 2225, 24 rows
    // 109 against 82, 32 rows 3176 against 2250; 64-, 96-, 128-row tiles at 44 rows 84 / 99 / 109, at 48 rows
    // 111 / 109 / 120 and 2440 / 2609 / 2918, at 56 rows 111 / 107 / 119 and 2634 / 2614 / 2993, at 64 rows
    // 133 / 109 / 121, at 76 rows 156 / 109 / 122 and 4073 / 2708 / 3113, at 80 rows - / 136 / 127).
    const int avg = ceil_div(expected_rows(a->rows, a->rows_hint), a->E);
    const int passes = w4_stream_passes(a->rows, a->rows_hint, a->E, a->k);
    mf = passes ? passes : (!tile_ok ? 4 : (avg <= 48 ? 64 : (avg <= 76 ? 96 : 128)));
  }
  if (mf == 8) mf = 128;
  if (mf == 64 || mf == 96 || mf == 128)
    KMOE_REQUIRE(tile_ok, KMOE_ERR_SHAPE, "grouped_gemm_w4a16: the tile kernel addresses the activations with 32 bits (rows=%d lda=%lld)",
                 a->rows, static_cast<long long>(a->lda));
  switch (mf) {
    // One block in flight per wave: the registers that saves put more waves on a SIMD (5-6 instead of 3-4), and
    // the unpacking work of one wave hides the loads of the others better than a deeper queue of its own does
    // (Qwen3 decode GEMMs: 52.9 / 31.2 us against 54.2 / 33.1 with two blocks and 55.8 / 34.8 with three).
    case 1: return swiglu ? launch_w4<1, 2, true, 1>(p, f16, s) : launch_w4<1, 2, false, 1>(p, f16, s);
    // tuning variants of the 16-row kernel: 1xy = x fragments per wave, y blocks in flight
    case 123: return swiglu ? launch_w4<1, 2, true, 3>(p, f16, s) : launch_w4<1, 2, false, 3>(p, f16, s);
    case 141: return swiglu ? launch_w4<1, 4, true, 1>(p, f16, s) : launch_w4<1, 4, false, 1>(p, f16, s);
    case 124: return swiglu ? launch_w4<1, 2, true, 4>(p, f16, s) : launch_w4<1, 2, false, 4>(p, f16, s);
    case 142: return swiglu ? launch_w4<1, 4, true, 2>(p, f16, s) : launch_w4<1, 4, false, 2>(p, f16, s);
    case 143: return swiglu ? launch_w4<1, 4, true, 3>(p, f16, s) : launch_w4<1, 4, false, 3>(p, f16, s);
    case 2: return swiglu ? launch_w4<2, 2, true, 2>(p, f16, s) : launch_w4<2, 2, false, 2>(p, f16, s);
    case 4: return swiglu ? launch_w4<4, 2, true, 2>(p, f16, s) : launch_w4<4, 2, false, 2>(p, f16, s);
    case 64: return swiglu ? launch_w4_tile<4, true>(p, a->rows, f16, s) : launch_w4_tile<4, false>(p, a->rows, f16, s);
    case 96: return swiglu ? launch_w4_tile<6, true>(p, a->rows, f16, s) : launch_w4_tile<6, false>(p, a->rows, f16, s);
    case 128: return swiglu ? launch_w4_tile<8, true>(p, a->rows, f16, s) : launch_w4_tile<8, false>(p, a->rows, f16, s);
    default:
      return fail(KMOE_ERR_UNSUPPORTED, "grouped_gemm_w4a16: variant=%d must be 0, 1, 2, 4, 8, 64, 96 or 128 (or a tuning variant)", a->variant);
  }
}
