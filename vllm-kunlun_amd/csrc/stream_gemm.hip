// Weight-streaming W8A8 grouped GEMM for the decode regime (a handful of rows
// per expert): HBM-bound, every weight byte is read once, MFMA is ~5% busy.
//
// Both operands arrive already arranged for v_mfma_i32_16x16x64_i8, so a wave
// needs no LDS, no barrier and no address arithmetic beyond a stride:
//   weights  "tiled": [E][n/16][k/64] blocks of 1 KB; inside a block byte
//            256*g + 16*c + t is channel c (of 16), k = 16*g + t (g = 0..3) —
//            i.e. exactly what lane 16*g + c feeds the MFMA. A wave reads 1 KB
//            of consecutive bytes per MFMA step and the next step's block follows
//            directly: one long sequential stream per 16 output channels.
//   activations "chunk-major": [k/64][rows][64 B], one chunk per MFMA step; lane
//            (g, r) reads bytes [16 g, 16 g + 16) of row r's chunk. Rows of an expert
//            are consecutive (down GEMM: 1 KB of consecutive bytes per step) or a
//            gather of 64-byte pieces (gate_up GEMM: one half cache line per row and
//            step; with 16-byte chunks a gathered load touched four times as many
//            lines, which cost the DeepSeek-V3 gate_up launch 9 %).
// Each wave owns NF channel fragments and keeps D MFMA steps of loads in flight.
#include "kmoe_common.h"
#include "pair_scan.h"
#include "quant_body.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

struct StreamParams {
  const int8_t* a;  // chunk-major [k/64][a_rows][64]
  int32_t a_rows;
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
  int32_t f16;  // outputs (and the rounding of gate and up before SiLU-mul) in IEEE half instead of bf16
  int32_t rotate;  // every wave starts its K range at a step of its own (see stream_gemm_i8)
  StreamScan scan;  // SCAN instantiations: the routed pairs' expert ids instead of lod / row_src
  StreamQuant quant;  // QUANT instantiations: the rows as bf16 / half values instead of codes and row maxes
};

constexpr int kWaves = 4;
constexpr int kQuantStride = kStreamQuantMaxK + 16;  // bytes between the rows of the LDS copy: row li starts 16 li B into the banks

// KS: the workgroup's 4 waves split K KS ways (KS = 1, 2, 4): 4/KS waves own
// different channels, KS waves share channels and add their exact int32 partial
// sums through LDS. More, shorter streams: a finer-grained tail on small layers.
//
// SCAN: the launch does the stable sort by expert itself. Every workgroup reads all the routed pairs' expert ids
// (p.scan.ids, a few KB from L2, a quarter per wave, kScanBatch loads in flight), counts the ids below its expert
// (its first sorted row) and lists the pairs that chose it, in order (its rows): what lod and row_src would have
// told it, after one memory round trip instead of two dependent ones and without the sort's launch before this one.
// The workgroups of channel block 0 also write the sort's outputs (lod, expert_m, moe_index, sorted_src) for the
// launches that follow.
//
// QUANT: the launch quantises its rows itself (the down projection of a decode-sized layer with k <= 1024). Per
// 16-row pass the workgroup's four waves read the pass's live rows as bf16 / half values (p.quant.act), one row
// per wave at a time, and leave absmax and codes - the arithmetic of quant_i8_rows_body, hence its bits - in LDS,
// where the K loop reads its row fragments; a and a_max are not read. The workgroups of channel block 0 also write
// codes (chunk-major) and row maxes where the quantiser's launch would have left them. Built for four waves per
// SIMD (see stream_gemm_i8).
template <int MF, int NF, bool SWIGLU, int D, int KS, bool SCAN = false, bool QUANT = false>
__global__ __launch_bounds__(kWaves* kWave, QUANT ? 4 : 1) void stream_gemm_i8_kernel(const StreamParams p) {
  static_assert(!SCAN || kWaves == kScanWaves, "scan_pairs is written for four waves");
  static_assert(!QUANT || (MF == 1 && KS == 1 && !SWIGLU && !SCAN), "QUANT: the 16-row down-projection shape only");
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  constexpr int TM = 16 * MF;
  constexpr int WN = kWaves / KS;  // waves along the channel dimension
  __shared__ v4i red[KS > 1 ? (KS - 1) * WN * MF * NF * kWave : 1];
  __shared__ typename std::conditional<SCAN, PairScanLds, int>::type scan_lds;
  __shared__ __attribute__((aligned(16))) int8_t qrows[QUANT ? 16 * kQuantStride : 16];
  __shared__ float qmax[16];
  const int lane = lane_id();
  const int wave_id = threadIdx.x >> 6;
  const int wave = wave_id / KS;   // channel group of this wave
  const int wk = wave_id % KS;     // K part of this wave
  const int li = lane & 15;
  const int lg = lane >> 4;
  const bool f16 = p.f16 != 0;

  // blockIdx.y < E: routed expert, all its rows. Beyond: one 16*MF-row slice of the tail expert.
  const bool tail = static_cast<int>(blockIdx.y) >= p.E;
  const int e = tail ? p.E : blockIdx.y;
  const int8_t* w_base = tail ? p.w_tail : p.w + static_cast<size_t>(e) * p.n * p.k;
  const float* w_max = tail ? p.w_max_tail : p.w_max + static_cast<size_t>(e) * p.n;

  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int ksteps = p.k / 64;
  const int col_base = (blockIdx.x * WN + wave) * NFH * 16;
  // whole wave has nothing to do (no barriers when KS == 1; with QUANT it stays for the quantisation and its barriers)
  const bool idle = KS == 1 && col_base >= n_half;
  if (idle && !QUANT && !SCAN) return;
  const int kb_begin = (ksteps * wk) / KS;
  const int kb_end = (ksteps * (wk + 1)) / KS;
  // With p.rotate a wave walks its K range from a start step of its own, wrapping round: int32 sums do not depend
  // on the order, and waves that were dispatched together no longer read addresses that differ by a
  // multiple of the fragment stride.
  const int klen = kb_end - kb_begin;
  const unsigned wave_key = (static_cast<unsigned>(blockIdx.y) * gridDim.x + blockIdx.x) * kWaves + wave_id;
  const int rot = p.rotate && klen > 1 ? static_cast<int>(((wave_key * 2654435761u) >> 12) % static_cast<unsigned>(klen)) : 0;
  auto kb_of = [&](int i) {
    const int s = i + rot;
    return kb_begin + (s >= klen ? s - klen : s);
  };

  const int8_t* wp[NF];
  bool wok[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    const size_t frag = wok[f] ? col[f] / 16 : 0;
    wp[f] = w_base + frag * ksteps * 1024 + lane * 16;
  }
  const size_t a_step = static_cast<size_t>(p.a_rows) * 64;  // bytes between MFMA steps

  // The first weight steps are requested before anything else: their addresses depend on the block's coordinates
  // only, while the rows do on two dependent loads (the expert's row range, then the gather indices). All
  // workgroups of a launch do the same work, so they start and end in rounds, and a round that begins with those
  // loads leaves the memory queue idle for their latency. Done where a wave's K range is short (a workgroup lives
  // a few microseconds: Qwen3 decode down projection 42.8 -> 40.4 us); with long ranges it changes nothing for the
  // better (DeepSeek-V3 decode: +0.4 %), so those keep the plain order.
  const bool w_first = QUANT || klen < 16;
  v4i wreg[D][NF];
  v4i areg[D][MF];
  auto load_w_step = [&](int slot, int kb) {
#pragma unroll
    for (int f = 0; f < NF; ++f)
      wreg[slot][f] = wok[f] ? *reinterpret_cast<const v4i*>(wp[f] + static_cast<size_t>(kb) * 1024)
                             : (v4i){0, 0, 0, 0};
  };
  if (w_first) {
#pragma unroll
    for (int d = 0; d < D; ++d)
      if (d < klen) load_w_step(d, kb_of(d));
  }
  __builtin_amdgcn_sched_barrier(0);

  int row_begin, row_end;
  ListedRows listed = {};  // SCAN: the expert's rows
  if (tail) {
    row_begin = p.tail_row0 + (static_cast<int>(blockIdx.y) - p.E) * TM;
    row_end = min(p.tail_row0 + p.tail_rows, row_begin + TM);
  } else if constexpr (SCAN) {
    listed = scan_pairs(p.scan, e, p.E, scan_lds, blockIdx.x == 0);
    if (idle) return;  // (KS == 1: no barrier after the scan's)
    row_begin = listed.begin;
    row_end = listed.end;
  } else {
    row_begin = p.lod[e];
    row_end = p.lod[e + 1];
  }
  if (SCAN && idle) return;  // (a tail slice's waves without channels; the routed ones left after the barrier)
  if (row_begin >= row_end) return;  // (an expert without rows has asked for a few KB of its weights in vain)

  for (int row0 = row_begin; row0 < row_end; row0 += TM) {
    if (QUANT) {
      if (row0 != row_begin) __syncthreads();  // the pass before has read its fragments
      const int nvec = p.k / 8;  // vectors of 8 values per row: at most 2 per lane
#pragma unroll 1
      for (int q = 0; q < 4; ++q) {
        const int qi = wave_id + 4 * q;
        const int r = row0 + qi;
        if (r >= row_end) break;  // wave-uniform
        const uint4* src = reinterpret_cast<const uint4*>(p.quant.act + static_cast<size_t>(r) * p.quant.ld);
        Pack8 val[2];
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int v = lane + i * kWave;
          if (v < nvec) {
            val[i].v = src[v];
#pragma unroll
            for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(act_to_f32(val[i].h[j], f16)));
          }
        }
        amax = group_max<kWave>(amax);
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int v = lane + i * kWave;
          if (v < nvec) {
            uint32_t w[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              float f = __builtin_rintf(act_to_f32(val[i].h[j], f16) * inv);
              f = fminf(fmaxf(f, -127.0f), 127.0f);
              w[j >> 2] |= static_cast<uint32_t>(static_cast<int>(f) & 0xff) << (8 * (j & 3));
            }
            *reinterpret_cast<uint2*>(&qrows[qi * kQuantStride + v * 8]) = make_uint2(w[0], w[1]);
            if (blockIdx.x == 0)
              *reinterpret_cast<uint2*>(p.quant.codes + (static_cast<size_t>(v >> 3) * p.a_rows + r) * 64 + (v & 7) * 8) =
                  make_uint2(w[0], w[1]);
          }
        }
        if (lane == 0) {
          qmax[qi] = amax;
          if (blockIdx.x == 0) p.quant.amax[r] = amax;
        }
      }
      __syncthreads();
      if (idle) continue;
    }
    const int8_t* ap[MF];
    int srow[MF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      if constexpr (SCAN)
        srow[mf] = r < row_end ? (tail ? p.tail_src0 + r - p.tail_row0 : listed.pair(scan_lds, r - row_begin) / p.src_div) : -1;
      else
        srow[mf] = r < row_end ? (tail ? p.tail_src0 + r - p.tail_row0 : (p.row_src ? p.row_src[r] / p.src_div : r)) : -1;
      // rows past the end read row 0: valid memory, results never stored
      ap[mf] = p.a + static_cast<size_t>(srow[mf] >= 0 ? srow[mf] : 0) * 64 + lg * 16;
    }

    v4i acc[MF][NF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf)
#pragma unroll
      for (int f = 0; f < NF; ++f) acc[mf][f] = (v4i){0, 0, 0, 0};

    auto load_a_step = [&](int slot, int kb) {
      if (QUANT) return;  // (read from LDS where it is used)
#pragma unroll
      for (int mf = 0; mf < MF; ++mf) areg[slot][mf] = *reinterpret_cast<const v4i*>(ap[mf] + kb * a_step);
    };
    auto load_step = [&](int slot, int kb) {
      load_w_step(slot, kb);
      load_a_step(slot, kb);
    };

#pragma unroll
    for (int d = 0; d < D; ++d)
      if (d < klen) {
        if (row0 != row_begin || !w_first) load_w_step(d, kb_of(d));  // (the first pass may have them already)
        load_a_step(d, kb_of(d));
      }

    for (int i0 = 0; i0 < klen; i0 += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int kb = i0 + d;
        if (kb < klen) {
#pragma unroll
          for (int mf = 0; mf < MF; ++mf)
#pragma unroll
            for (int f = 0; f < NF; ++f)
              acc[mf][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                  wreg[d][f],
                  QUANT ? *reinterpret_cast<const v4i*>(&qrows[li * kQuantStride + kb_of(kb) * 64 + lg * 16]) : areg[d][mf],
                  acc[mf][f], 0, 0, 0);
          if (kb + D < klen) load_step(d, kb_of(kb + D));
        }
      }
    }

    if (KS > 1) {  // add the K parts: waves wk > 0 park their sums in LDS, wave wk == 0 collects
      if (wk > 0) {
#pragma unroll
        for (int mf = 0; mf < MF; ++mf)
#pragma unroll
          for (int f = 0; f < NF; ++f)
            red[(((wk - 1) * WN + wave) * MF * NF + mf * NF + f) * kWave + lane] = acc[mf][f];
      }
      __syncthreads();
      if (wk == 0) {
#pragma unroll
        for (int part = 1; part < KS; ++part)
#pragma unroll
          for (int mf = 0; mf < MF; ++mf)
#pragma unroll
            for (int f = 0; f < NF; ++f)
              acc[mf][f] += red[(((part - 1) * WN + wave) * MF * NF + mf * NF + f) * kWave + lane];
      }
      __syncthreads();  // red is reused by the next m-tile
      if (wk > 0) continue;
    }

#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      if (r >= row_end) continue;
      const float sa = (QUANT ? qmax[li] : p.a_max[srow[mf]]) / 127.0f;
#pragma unroll
      for (int f = 0; f < NFH; ++f) {
        if (!wok[f]) continue;
        const int c0 = col[f] + lg * 4;
        uint16_t yv[4];
        auto finish = [&](const v4i& a, int cc, uint16_t(&out)[4]) {
          const float4 wm = *reinterpret_cast<const float4*>(w_max + cc);
          const float sw[4] = {wm.x / 127.0f, wm.y / 127.0f, wm.z / 127.0f, wm.w / 127.0f};
#pragma unroll
          for (int q = 0; q < 4; ++q) out[q] = f32_to_act((static_cast<float>(a[q]) * sa) * sw[q], f16);
          if (p.acc_out) *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + cc) = a;
        };
        finish(acc[mf][f], c0, yv);
        if (SWIGLU) {
          uint16_t uv[4];
          finish(acc[mf][f + NFH], col[f + NFH] + lg * 4, uv);
#pragma unroll
          for (int q = 0; q < 4; ++q) yv[q] = f32_to_act(silu_hw(act_to_f32(yv[q], f16)) * act_to_f32(uv[q], f16), f16);
        }
        const uint2 packed = make_uint2(yv[0] | (static_cast<uint32_t>(yv[1]) << 16),
                                        yv[2] | (static_cast<uint32_t>(yv[3]) << 16));
        *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) = packed;
      }
    }
  }
}

template <int MF, int NF, bool SWIGLU, int D, int KS = 1, bool SCAN = false, bool QUANT = false>
int launch_stream(const StreamParams& p, hipStream_t s) {
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const dim3 grid(ceil_div(n_half, (kWaves / KS) * NFH * 16), p.E + (p.w_tail ? ceil_div(p.tail_rows, 16 * MF) : 0));
  if (tracing_kernels())
    note_kernel("stream_gemm_i8_kernel<%d rows per pass, %d channel fragments per wave, %s, %d steps in flight, K split %d%s%s>",
                16 * MF, NF, SWIGLU ? "SiLU-mul" : "plain", D, KS, SCAN ? ", sorts the pairs itself" : "",
                QUANT ? ", quantises its rows itself" : "");
  hipLaunchKernelGGL((stream_gemm_i8_kernel<MF, NF, SWIGLU, D, KS, SCAN, QUANT>), grid, dim3(kWaves * kWave), 0, s, p);
  return check_launch("kmoe_grouped_gemm_i8 (stream)");
}

// [E][n][k] row-major -> tiled blocks; one thread moves 16 bytes.
__global__ void tile_weights_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst, int n, int k,
                                    long long total_vec) {
  const long long v = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (v >= total_vec) return;
  const int ksteps = k / 64;
  const int lane = static_cast<int>(v & 63);
  const long long blk = v >> 6;  // (e * n/16 + nb) * ksteps + kb
  const int kb = static_cast<int>(blk % ksteps);
  const long long frag = blk / ksteps;  // e * n/16 + nb
  const long long row = frag * 16 + (lane & 15);
  const int kk = kb * 64 + (lane >> 4) * 16;
  *reinterpret_cast<uint4*>(dst + v * 16) = *reinterpret_cast<const uint4*>(src + row * k + kk);
}

}  // namespace

int stream_gemm_i8(const kmoe_gemm_i8_args* a, hipStream_t s, const StreamScan* scan, const StreamQuant* quant) {
  StreamParams p{a->a, a->a_rows, a->a_max, a->row_src, a->src_div, a->w, a->w_max,
                 a->lod, a->E,     a->n,     a->k,       a->y,       a->ldy, a->acc_out,
                 a->w_tail, a->w_max_tail, a->tail_row0, a->tail_rows, a->tail_src0, a->act_dtype == KMOE_DT_F16,
                 // A fragment's blocks are k / 64 KB apart. When that stride is a multiple of 64 KB (k = 4096, 8192:
                 // Mixtral, Qwen3-235B), waves in step hit the same memory channels: measured 5.5 TB/s at k = 8192
                 // and 6.0 at 4096 against 6.5 at 2048; with the rotated start 6.0 and 6.6. Other strides gain
                 // nothing from it (k = 7168: 6.2 either way).
                 a->k % 4096 == 0,
                 scan ? *scan : StreamScan{}, quant ? *quant : StreamQuant{}};
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  if (quant) {
    // the down launch of a decode-sized layer: 16 rows per pass, one wave per K range
    KMOE_REQUIRE(!scan && !swiglu && a->variant == 0 && a->row_src == nullptr && !a->acc_out && quant->act &&
                     quant->codes && quant->amax && quant->ld >= a->k && quant->ld % 8 == 0 &&
                     a->k <= kStreamQuantMaxK && a->k / 64 < 24 &&
                     ceil_div(expected_rows(a->rows, a->rows_hint), a->E) <= 10,
                 KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8 (stream): not a launch that can quantise its rows itself");
    // (Four steps of weights in flight and two channel fragments per wave as in the plain launch. Two steps, or one
    // fragment per wave with 2 / 4 / 8 steps - 5 to 6 waves per SIMD - are 1.6 to 3.3 us slower; 6 and 8 steps with
    // two fragments need more registers than four waves per SIMD leave, and this launch needs the four: built for
    // three it took as long as the quantiser's launch and this one together had. Qwen3 decode, layer: 117.5 us with
    // the quantiser's launch, 117.0 built for three waves, 115.1 for four.)
    return launch_stream<1, 2, false, 4, 1, false, true>(p, s);
  }
  if (scan) {
    // the routed gate_up launch of a decode-sized layer: 16 rows per pass, the three shapes of `case 1` below
    KMOE_REQUIRE(swiglu && a->variant == 0 && a->row_src == nullptr && scan->ids && scan->lod && scan->expert_m &&
                     scan->moe_index && scan->sorted_src && scan->n_pairs == a->rows &&
                     a->rows <= kStreamScanMaxPairs && a->a_rows <= kStreamScanMaxRows,
                 KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8 (stream): not a launch that can sort the pairs itself");
    const int ksteps = p.k / 64;
    const int blocks = p.E * ceil_div(p.n / 2, kWaves * 16);
    if (ksteps >= 24 && blocks < 2048) return launch_stream<1, 2, true, 2, 4, true>(p, s);
    if (ksteps >= 24) return launch_stream<1, 2, true, 4, 2, true>(p, s);
    return launch_stream<1, 2, true, 4, 1, true>(p, s);
  }
  // m-fragments per pass from the rows an expert gets under uniform routing
  int mf = a->variant;
  if (mf == 0) {
    // An expert with more rows than one pass holds streams its weights again: leave headroom
    // over the mean for the spread of a random routing (about +-2 sigma at these sizes).
    const int avg = ceil_div(expected_rows(a->rows, a->rows_hint), a->E);
    mf = avg <= 10 ? 1 : (avg <= 22 ? 2 : (avg <= 48 ? 4 : 8));
  }
  switch (mf) {
    // tuning variants of the 16-row kernel: 1xy = prefetch depth x, K split y
    case 121: return swiglu ? launch_stream<1, 2, true, 2, 1>(p, s) : launch_stream<1, 2, false, 2, 1>(p, s);
    case 181: return swiglu ? launch_stream<1, 2, true, 8, 1>(p, s) : launch_stream<1, 2, false, 8, 1>(p, s);
    case 142: return swiglu ? launch_stream<1, 2, true, 4, 2>(p, s) : launch_stream<1, 2, false, 4, 2>(p, s);
    case 144: return swiglu ? launch_stream<1, 2, true, 4, 4>(p, s) : launch_stream<1, 2, false, 4, 4>(p, s);
    case 122: return swiglu ? launch_stream<1, 2, true, 2, 2>(p, s) : launch_stream<1, 2, false, 2, 2>(p, s);
    case 124: return swiglu ? launch_stream<1, 2, true, 2, 4>(p, s) : launch_stream<1, 2, false, 2, 4>(p, s);
    case 182: return swiglu ? launch_stream<1, 2, true, 8, 2>(p, s) : launch_stream<1, 2, false, 8, 2>(p, s);
    case 1: {
      // Split K across the waves of a workgroup when streams are long enough to share:
      // more, shorter streams balance the tail (measured: +6..12% at k = 2048).
      const int ksteps = p.k / 64;
      const int n_half = swiglu ? p.n / 2 : p.n;
      const int blocks = p.E * ceil_div(n_half, kWaves * (swiglu ? 1 : 2) * 16);
      if (ksteps >= 24 && blocks < 2048)
        return swiglu ? launch_stream<1, 2, true, 2, 4>(p, s) : launch_stream<1, 2, false, 2, 4>(p, s);
      if (ksteps >= 24)
        return swiglu ? launch_stream<1, 2, true, 4, 2>(p, s) : launch_stream<1, 2, false, 4, 2>(p, s);
      return swiglu ? launch_stream<1, 2, true, 4>(p, s) : launch_stream<1, 2, false, 4>(p, s);
    }
    case 2:
      return swiglu ? launch_stream<2, 2, true, 4>(p, s) : launch_stream<2, 2, false, 4>(p, s);
    case 4:
      return swiglu ? launch_stream<4, 2, true, 4>(p, s) : launch_stream<4, 2, false, 4>(p, s);
    case 8:
      return swiglu ? launch_stream<8, 2, true, 2>(p, s) : launch_stream<8, 2, false, 2>(p, s);
    default:
      return fail(KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8 (stream): variant=%d must be 0, 1, 2, 4 or 8", a->variant);
  }
}

}  // namespace kmoe

using namespace kmoe;

extern "C" int kmoe_tile_weights_i8(const int8_t* src, int8_t* dst, int E, int n, int k, kmoe_stream_t stream) {
  KMOE_REQUIRE(src && dst, KMOE_ERR_NULL, "tile_weights_i8: NULL pointer");
  KMOE_REQUIRE(src != dst, KMOE_ERR_SHAPE, "tile_weights_i8: src and dst must differ (not an in-place transform)");
  KMOE_REQUIRE(E >= 1 && n >= 16 && n % 16 == 0 && k >= 64 && k % 64 == 0, KMOE_ERR_SHAPE,
               "tile_weights_i8: E=%d n=%d k=%d (need n %% 16 == 0, k %% 64 == 0)", E, n, k);
  const long long total_vec = static_cast<long long>(E) * n * k / 16;
  hipLaunchKernelGGL(tile_weights_kernel, dim3(static_cast<unsigned>((total_vec + 255) / 256)), dim3(256), 0,
                     as_stream(stream), src, dst, n, k, total_vec);
  return check_launch("kmoe_tile_weights_i8");
}
