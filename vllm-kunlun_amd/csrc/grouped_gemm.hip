// Grouped GEMM over expert-sorted rows on gfx950 MFMA: int8 (W8A8), bf16
// (unquantized) and fp8-e4m3 with 128x128 / 1x128 block scales.
//
// Roles: the WEIGHT fragment is the first MFMA operand (16 output channels x K
// bytes), the ACTIVATION fragment the second (K bytes x 16 sorted rows). A lane
// therefore ends up with 4 consecutive output channels of one row: channel
// 4*(lane/16)+q, row lane%16 — what the dequant / SiLU-mul epilogue (gate and up
// fragments of the same channels sit in the same lane) and an 8-byte store want.
//
// Data movement per workgroup:
//   weights     global -> registers, one 256-byte K chunk per channel row
//               prefetched ahead of the MFMAs that consume it; every wave owns
//               its own output channels, so weights never pass through LDS;
//   activations global (gathered through the sort) -> LDS, double-buffered per
//               K chunk, shared by all waves of the workgroup.
// K is handled in BYTES: a chunk is 256 bytes of a row; MFMA step j consumes
// bytes [j*4*LB, (j+1)*4*LB) of the chunk, lane group g = lane/16 holding bytes
// [g*LB, (g+1)*LB) of the step (LB = 16 for int8/bf16, 32 for fp8).
#include "kmoe_common.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kKC = 256;          // bytes of K per chunk and row
constexpr int kPitch = kKC + 16;  // LDS row pitch: 16 rows of a b128 read fall in 16 different bank groups

enum class Kind { I8, BF16, FP8, F16 };  // F16: the unquantized path on IEEE half operands and results
constexpr const char* kind_name(Kind k) {
  return k == Kind::I8 ? "int8" : (k == Kind::BF16 ? "bf16" : (k == Kind::FP8 ? "fp8" : "f16"));
}

template <Kind K> struct Traits;
template <> struct Traits<Kind::I8> {
  using acc_t = v4i;
  static constexpr int LB = 16;   // bytes per lane and MFMA step
  __device__ static acc_t zero() { return (v4i){0, 0, 0, 0}; }
};
template <> struct Traits<Kind::BF16> {
  using acc_t = v4f;
  static constexpr int LB = 16;
  __device__ static acc_t zero() { return (v4f){0.f, 0.f, 0.f, 0.f}; }
};
template <> struct Traits<Kind::F16> : Traits<Kind::BF16> {};
template <> struct Traits<Kind::FP8> {
  using acc_t = v4f;
  static constexpr int LB = 32;
  __device__ static acc_t zero() { return (v4f){0.f, 0.f, 0.f, 0.f}; }
};

struct GemmParams {
  const int8_t* a;         // activations, rows of kbytes bytes
  int64_t lda;             // row stride in BYTES
  const float* a_max;      // I8: [a_rows] absmax; FP8: [a_rows, k/128] scales; BF16: unused
  const int32_t* row_src;
  int32_t src_div;
  const int8_t* w;         // [E, n, kbytes]
  const float* w_max;      // I8: [E, n] absmax; FP8: [E, n/128, k/128] scales; BF16: unused
  const int32_t* lod;
  int32_t E, n, kbytes;
  uint16_t* y;
  int64_t ldy;             // in elements
  int32_t* acc_out;        // I8 only
  int32_t w_tiled;         // weights in 1 KB MFMA blocks [E][n/16][kbytes/64] (kmoe_tile_weights_i8) instead of row-major.
                           // FP8: an MFMA step takes two consecutive blocks, i.e. lane (g, c) holds k = 16g..16g+15 and
                           // 64+16g..64+16g+15 of the step; the activation fragment takes the same two halves
  const int8_t* w_tail;    // optional extra expert (index E): rows [tail_row0, tail_row0 + tail_rows), identity source
  const float* w_max_tail;
  int32_t tail_row0, tail_rows, tail_src0;
  // BF16 only (the expert-bias branch, ops/_kunlun_ops.py:433-468):
  const uint16_t* bias;    // NULL, or [E, n] bf16 added to the bf16 result (rounded again, as `gemm + bias` in bf16 is)
  int32_t oai;             // 1: out[r, i] = swigluoai(y[r, 2i], y[r, 2i+1]) (interleaved gate/up), n/2 outputs per row
  float oai_alpha, oai_limit;
  int32_t f16;             // I8, FP8: outputs (and the rounding of gate and up before SiLU-mul) in IEEE half instead of bf16
};

// Rows of expert e, with the tail expert (e == E) taken from the host-side range.
__device__ inline int rows_begin(const GemmParams& p, int e) { return e < p.E ? p.lod[e] : p.tail_row0; }
__device__ inline int rows_end(const GemmParams& p, int e) {
  return e < p.E ? p.lod[e + 1] : p.tail_row0 + p.tail_rows;
}

__device__ inline int wave_incl_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int o = __shfl_up(v, off, kWave);
    if (lane >= off) v += o;
  }
  return v;
}

// Finds the expert and first row of m-tile number `t` when every expert's rows
// (the tail expert included) are cut into tiles of TM. Returns false when t is past the last tile.
template <int TM>
__device__ inline bool locate_tile(const GemmParams& p, int t, int& e_out, int& row0_out) {
  const int lane = lane_id();
  const int E = p.E + (p.w_tail ? 1 : 0);
  const int epl = (E + kWave - 1) / kWave;
  const int e_begin = lane * epl;
  int local = 0;
  for (int i = 0; i < epl; ++i) {
    const int e = e_begin + i;
    if (e < E) local += (rows_end(p, e) - rows_begin(p, e) + TM - 1) / TM;
  }
  const int incl = wave_incl_scan(local);
  const int total = __shfl(incl, kWave - 1, kWave);
  if (t >= total) return false;
  int excl = incl - local;
  int found_e = -1, found_row = 0;
  if (t >= excl && t < incl) {
    for (int i = 0; i < epl; ++i) {
      const int e = e_begin + i;
      if (e >= E) break;
      const int lo = rows_begin(p, e);
      const int tiles = (rows_end(p, e) - lo + TM - 1) / TM;
      if (t < excl + tiles) {
        found_e = e;
        found_row = lo + (t - excl) * TM;
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

// MF: 16-row fragments per workgroup tile; NF: 16-channel fragments per wave
// (SWIGLU: NF/2 gate + NF/2 up fragments of the same channels); LOCATE: the
// m-tile comes from blockIdx.y through locate_tile (balanced over skewed
// experts) instead of blockIdx.y being the expert.
template <Kind KIND, int MF, int NF, int WAVES, bool SWIGLU, bool LOCATE>
__global__ __launch_bounds__(WAVES* kWave) void grouped_gemm_kernel(const GemmParams p) {
  using T = Traits<KIND>;
  using acc_t = typename T::acc_t;
  constexpr int LB = T::LB;
  constexpr int kJ = kKC / (4 * LB);  // MFMA steps per chunk
  constexpr int kV = LB / 16;         // 16-byte vectors per lane and step
  constexpr int TM = 16 * MF;
  constexpr int THREADS = WAVES * kWave;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  constexpr int NA = (TM * (kKC / 16) + THREADS - 1) / THREADS;  // activation vectors per thread per chunk
  static_assert(!SWIGLU || NF % 2 == 0, "SwiGLU pairs gate and up fragments");

  __shared__ __attribute__((aligned(16))) int8_t lds_a[2][TM * kPitch];

  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;

  int e, row_begin, row_end;
  if (LOCATE) {
    if (!locate_tile<TM>(p, blockIdx.y, e, row_begin)) return;
    row_end = min(rows_end(p, e), row_begin + TM);
  } else {
    e = blockIdx.y;
    row_begin = rows_begin(p, e);
    row_end = rows_end(p, e);
    if (row_begin >= row_end) return;
  }
  const bool tail = e >= p.E;
  const int8_t* w_base = tail ? p.w_tail : p.w + static_cast<size_t>(e) * p.n * p.kbytes;
  const float* w_aux = tail ? p.w_max_tail : p.w_max;  // I8: + e*n below; FP8: indexed with e

  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int col_base = (blockIdx.x * WAVES + wave) * NFH * 16;

  const int8_t* wp[NF];
  bool wok[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    if (p.w_tiled) {  // 1 KB block (fragment, 64 bytes of K): lane l at l*16
      const size_t frag = wok[f] ? col[f] / 16 : 0;
      wp[f] = w_base + frag * (p.kbytes / 64) * 1024 + lane * 16;
    } else {
      wp[f] = w_base + static_cast<size_t>(wok[f] ? col[f] + li : 0) * p.kbytes + lg * LB;
    }
  }
  const int w_step = p.w_tiled ? 64 * LB : 4 * LB;  // bytes between consecutive MFMA steps of a fragment
  const int w_vec = p.w_tiled ? 1024 : 16;           // bytes between the 16-byte halves of a lane's operand (FP8)
  const int a_lane = p.w_tiled ? 16 : LB;            // activation fragment: byte offset of lane group lg ...
  const int a_vec = p.w_tiled ? 64 : 16;             // ... and of its second half (FP8)
  const int nchunks = (p.kbytes + kKC - 1) / kKC;
  const int kblocks = p.kbytes / 128;  // FP8: scale blocks along K

  for (int row0 = row_begin; row0 < row_end; row0 += TM) {
    const int8_t* ap[NA];
    int a_lds[NA];
    int a_kv[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int v = threadIdx.x + i * THREADS;
      const int r = v >> 4;
      const int kv = v & 15;
      a_kv[i] = kv * 16;
      a_lds[i] = (v < TM * 16) ? r * kPitch + kv * 16 : -1;
      ap[i] = nullptr;
      if (v < TM * 16 && row0 + r < row_end) {
        const int sr = tail ? p.tail_src0 + row0 + r - p.tail_row0 : (p.row_src ? p.row_src[row0 + r] / p.src_div : row0 + r);
        ap[i] = p.a + static_cast<size_t>(sr) * p.lda + kv * 16;
      }
    }
    // source row of this lane's output rows (for scales / maxes)
    int srow[MF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      srow[mf] = r < row_end ? (tail ? p.tail_src0 + r - p.tail_row0 : (p.row_src ? p.row_src[r] / p.src_div : r)) : -1;
    }

    acc_t acc[MF][NF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf)
#pragma unroll
      for (int f = 0; f < NF; ++f) acc[mf][f] = T::zero();

    v4i wbuf[2][NF][kJ][kV];
    v4i areg[NA];

    auto load_w = [&](v4i(&dst)[NF][kJ][kV], int chunk) {
      const int kc = chunk * kKC;
#pragma unroll
      for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int j = 0; j < kJ; ++j)
#pragma unroll
          for (int v = 0; v < kV; ++v) {
            const int koff = kc + j * 4 * LB + v * 16;  // k position (+ lg*LB, folded into wp)
            const size_t off = static_cast<size_t>(chunk * kJ + j) * w_step + v * w_vec;
            dst[f][j][v] = (wok[f] && koff + lg * LB < p.kbytes) ? *reinterpret_cast<const v4i*>(wp[f] + off)
                                                                  : (v4i){0, 0, 0, 0};
          }
    };
    auto load_a = [&](int chunk) {
      const int kc = chunk * kKC;
#pragma unroll
      for (int i = 0; i < NA; ++i)
        areg[i] = (ap[i] && kc + a_kv[i] < p.kbytes) ? *reinterpret_cast<const v4i*>(ap[i] + kc) : (v4i){0, 0, 0, 0};
    };
    auto store_a = [&](int buf) {
#pragma unroll
      for (int i = 0; i < NA; ++i)
        if (a_lds[i] >= 0) *reinterpret_cast<v4i*>(&lds_a[buf][a_lds[i]]) = areg[i];
    };
    auto compute = [&](const v4i(&wcur)[NF][kJ][kV], int buf, int chunk) {
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        v4i af[MF][kV];
#pragma unroll
        for (int mf = 0; mf < MF; ++mf)
#pragma unroll
          for (int v = 0; v < kV; ++v)
            af[mf][v] = *reinterpret_cast<const v4i*>(
                &lds_a[buf][(mf * 16 + li) * kPitch + j * 4 * LB + lg * a_lane + v * a_vec]);
        if constexpr (KIND == Kind::I8) {
#pragma unroll
          for (int mf = 0; mf < MF; ++mf)
#pragma unroll
            for (int f = 0; f < NF; ++f)
              acc[mf][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wcur[f][j][0], af[mf][0], acc[mf][f], 0, 0, 0);
        } else if constexpr (KIND == Kind::BF16) {
#pragma unroll
          for (int mf = 0; mf < MF; ++mf)
#pragma unroll
            for (int f = 0; f < NF; ++f)
              acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wcur[f][j][0]),
                                                                   __builtin_bit_cast(v8bf, af[mf][0]), acc[mf][f], 0,
                                                                   0, 0);
        } else if constexpr (KIND == Kind::F16) {
#pragma unroll
          for (int mf = 0; mf < MF; ++mf)
#pragma unroll
            for (int f = 0; f < NF; ++f)
              acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wcur[f][j][0]),
                                                                  __builtin_bit_cast(v8h, af[mf][0]), acc[mf][f], 0, 0,
                                                                  0);
        } else {
          // one MFMA = one 128-wide scale block: scale the block's partial sum, then add
          const int kb = chunk * kJ + j;
          if (kb < kblocks) {
            float sa[MF];
#pragma unroll
            for (int mf = 0; mf < MF; ++mf)
              sa[mf] = srow[mf] >= 0 ? p.a_max[static_cast<size_t>(srow[mf]) * kblocks + kb] : 0.0f;
#pragma unroll
            for (int f = 0; f < NF; ++f) {
              const float sw =
                  wok[f] ? w_aux[((tail ? 0 : static_cast<size_t>(e) * (p.n / 128)) + col[f] / 128) * kblocks + kb] : 0.0f;
              v8i wv;
              wv.lo = wcur[f][j][0];
              wv.hi = wcur[f][j][1];
#pragma unroll
              for (int mf = 0; mf < MF; ++mf) {
                v8i av;
                av.lo = af[mf][0];
                av.hi = af[mf][1];
                const v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    wv, av, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
                const float s = sa[mf] * sw;
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[mf][f][q] = __builtin_fmaf(blk[q], s, acc[mf][f][q]);
              }
            }
          }
        }
      }
    };
    auto stage = [&](int chunk, const v4i(&wcur)[NF][kJ][kV], v4i(&wnext)[NF][kJ][kV], int buf) {
      const bool more = chunk + 1 < nchunks;
      if (more) {
        load_w(wnext, chunk + 1);
        load_a(chunk + 1);
      }
      compute(wcur, buf, chunk);
      if (more) store_a(buf ^ 1);
      __syncthreads();
    };

    load_w(wbuf[0], 0);
    load_a(0);
    store_a(0);
    __syncthreads();
    for (int c = 0; c < nchunks; c += 2) {
      stage(c, wbuf[0], wbuf[1], 0);
      if (c + 1 < nchunks) stage(c + 1, wbuf[1], wbuf[0], 1);
    }

    // ---- epilogue: dequantise, optional SiLU-mul, store ----
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
      const int r = row0 + mf * 16 + li;
      if (r >= row_end) continue;
      float sa = 1.0f;
      const bool f16 = KIND == Kind::F16 || ((KIND == Kind::I8 || KIND == Kind::FP8) && p.f16 != 0);
      if constexpr (KIND == Kind::I8) sa = p.a_max[srow[mf]] / 127.0f;
#pragma unroll
      for (int f = 0; f < NFH; ++f) {
        if (!wok[f]) continue;
        const int c0 = col[f] + lg * 4;
        uint16_t yv[4];
        auto finish = [&](const acc_t& a, int cc, uint16_t(&out)[4]) {
          if constexpr (KIND == Kind::I8) {
            const float4 wm = *reinterpret_cast<const float4*>(w_aux + (tail ? 0 : static_cast<size_t>(e) * p.n) + cc);
            const float sw[4] = {wm.x / 127.0f, wm.y / 127.0f, wm.z / 127.0f, wm.w / 127.0f};
#pragma unroll
            for (int q = 0; q < 4; ++q) out[q] = f32_to_act((static_cast<float>(a[q]) * sa) * sw[q], f16);
            if (p.acc_out) *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + cc) = a;
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) out[q] = f32_to_act(a[q], f16);
          }
        };
        finish(acc[mf][f], c0, yv);
        if (SWIGLU) {
          uint16_t uv[4];
          finish(acc[mf][f + NFH], col[f + NFH] + lg * 4, uv);
#pragma unroll
          for (int q = 0; q < 4; ++q) yv[q] = f32_to_act(silu_hw(act_to_f32(yv[q], f16)) * act_to_f32(uv[q], f16), f16);
        }
        if constexpr (KIND == Kind::BF16 && !SWIGLU) {
          if (p.bias) {
            const uint2 b4 = *reinterpret_cast<const uint2*>(p.bias + static_cast<size_t>(e) * p.n + c0);
            const uint16_t bv[4] = {static_cast<uint16_t>(b4.x), static_cast<uint16_t>(b4.x >> 16),
                                    static_cast<uint16_t>(b4.y), static_cast<uint16_t>(b4.y >> 16)};
#pragma unroll
            for (int q = 0; q < 4; ++q) yv[q] = f32_to_bf16(bf16_to_f32(yv[q]) + bf16_to_f32(bv[q]));
          }
          if (p.oai) {  // this lane holds (gate, up, gate, up) of output channels c0/2 and c0/2 + 1
            const uint16_t o0 = swigluoai_bf16(yv[0], yv[1], p.oai_alpha, p.oai_limit);
            const uint16_t o1 = swigluoai_bf16(yv[2], yv[3], p.oai_alpha, p.oai_limit);
            *reinterpret_cast<uint32_t*>(p.y + static_cast<size_t>(r) * p.ldy + c0 / 2) =
                o0 | (static_cast<uint32_t>(o1) << 16);
            continue;
          }
        }
        const uint2 packed = make_uint2(yv[0] | (static_cast<uint32_t>(yv[1]) << 16),
                                        yv[2] | (static_cast<uint32_t>(yv[3]) << 16));
        *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) = packed;
      }
    }
  }
}

template <Kind KIND, int MF, int NF, int WAVES, bool SWIGLU, bool LOCATE>
int launch(const GemmParams& p, int rows, hipStream_t s, const char* what) {
  constexpr int TM = 16 * MF;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int grid_x = ceil_div(n_half, WAVES * NFH * 16);
  const int n_exp = p.E + (p.w_tail ? 1 : 0);
  const int grid_y = LOCATE ? (rows + p.tail_rows) / TM + min(n_exp, rows + p.tail_rows) : n_exp;
  if (grid_y == 0) return KMOE_OK;
  if (tracing_kernels())
    note_kernel("grouped_gemm_kernel<%s, %d-row tiles, %d channel fragments per wave, %d waves, %s>", kind_name(KIND), TM, NF,
                WAVES, SWIGLU ? "SiLU-mul" : "plain");
  hipLaunchKernelGGL((grouped_gemm_kernel<KIND, MF, NF, WAVES, SWIGLU, LOCATE>), dim3(grid_x, grid_y),
                     dim3(WAVES * kWave), 0, s, p);
  return check_launch(what);
}

// Tiled weights: from this many rows per expert (on average) the persistent 128-row-tile kernel wins over
// the 16/32/64-row kernels of this file although most of its tile is padding: its weight stream is asynchronous
// and it is bound by the weight bytes either way (measured cross-over: 8 to 16 rows, all three formats).
constexpr int kTiledMinRows = 10;
// variants of the bf16 and fp8 launchers that force the tile kernel: 5 (tile height from the rows per expert),
// 6 (128-row tiles), 11 (64-row tiles)
inline bool tile_variant(int v) { return v == 5 || v == 6 || (v >= 11 && v <= 13); }

template <Kind KIND>
int dispatch(const GemmParams& p, int rows, int live, bool swiglu, int variant, hipStream_t s, const char* what) {
  if (variant == 0) {
    // rows per expert if the routing were uniform; decides streaming vs tiled
    const int avg = ceil_div(live, p.E);
    variant = avg <= 16 ? 1 : (avg <= 48 ? 2 : 3);
  }
  switch (variant) {
    case 1:  // weight streaming: 16-row tiles, one expert per workgroup row
      return swiglu ? launch<KIND, 1, 2, 4, true, false>(p, rows, s, what)
                    : launch<KIND, 1, 1, 4, false, false>(p, rows, s, what);
    case 2:  // 32-row tiles
      return swiglu ? launch<KIND, 2, 2, 4, true, false>(p, rows, s, what)
                    : launch<KIND, 2, 2, 4, false, false>(p, rows, s, what);
    case 3:  // 128-row tiles, work list balanced over experts
      return swiglu ? launch<KIND, 8, 4, 4, true, true>(p, rows, s, what)
                    : launch<KIND, 8, 4, 4, false, true>(p, rows, s, what);
    default:
      return fail(KMOE_ERR_UNSUPPORTED, "%s: variant=%d unknown", what, variant);
  }
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

int grouped_gemm_i8_checked(const kmoe_gemm_i8_args* a, kmoe_stream_t stream, const StreamScan* scan,
                            const StreamQuant* quant) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "grouped_gemm_i8: args is NULL");
  KMOE_REQUIRE(a->a && a->a_max && a->w && a->w_max && (a->lod || scan) && a->y, KMOE_ERR_NULL,
               "grouped_gemm_i8: NULL tensor pointer");
  KMOE_REQUIRE(a->E >= 1 && a->n >= 16 && a->k >= 16 && a->rows >= 0, KMOE_ERR_SHAPE,
               "grouped_gemm_i8: E=%d n=%d k=%d rows=%d", a->E, a->n, a->k, a->rows);
  KMOE_REQUIRE(a->k % 16 == 0, KMOE_ERR_SHAPE, "grouped_gemm_i8: k=%d must be a multiple of 16", a->k);
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  KMOE_REQUIRE(a->act == KMOE_ACT_NONE || swiglu, KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8: act=%d unknown", a->act);
  KMOE_REQUIRE(a->act_dtype == KMOE_DT_BF16 || a->act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_i8: act_dtype=%d unknown", a->act_dtype);
  KMOE_REQUIRE(a->n % (swiglu ? 32 : 16) == 0, KMOE_ERR_SHAPE, "grouped_gemm_i8: n=%d must be a multiple of %d",
               a->n, swiglu ? 32 : 16);
  KMOE_REQUIRE(a->a_layout == KMOE_A_CHUNKED || (a->lda % 16 == 0 && a->lda >= a->k), KMOE_ERR_SHAPE,
               "grouped_gemm_i8: lda=%lld must be a multiple of 16 and >= k", (long long)a->lda);
  const int n_out = swiglu ? a->n / 2 : a->n;
  KMOE_REQUIRE(a->ldy % 4 == 0 && a->ldy >= n_out, KMOE_ERR_SHAPE,
               "grouped_gemm_i8: ldy=%lld must be a multiple of 4 and >= %d", (long long)a->ldy, n_out);
  KMOE_REQUIRE(aligned(a->a, 16) && aligned(a->w, 16) && aligned(a->y, 8) && aligned(a->w_max, 16) &&
                   aligned(a->acc_out, 16),
               KMOE_ERR_SHAPE, "grouped_gemm_i8: misaligned tensor pointer");
  KMOE_REQUIRE(!a->row_src || a->src_div >= 1, KMOE_ERR_SHAPE, "grouped_gemm_i8: src_div=%d < 1", a->src_div);
  KMOE_REQUIRE(!a->w_tail || (a->w_max_tail && a->tail_rows >= 0 && a->tail_row0 >= 0 && aligned(a->w_tail, 16) &&
                              aligned(a->w_max_tail, 16)),
               KMOE_ERR_SHAPE, "grouped_gemm_i8: bad tail expert (w_max_tail, tail_row0=%d, tail_rows=%d)",
               a->tail_row0, a->tail_rows);
  KMOE_REQUIRE(a->w_layout == KMOE_W_ROWMAJOR || (a->w_layout == KMOE_W_TILED && a->k % 64 == 0), KMOE_ERR_SHAPE,
               "grouped_gemm_i8: w_layout=%d (tiled weights need k %% 64 == 0, k=%d)", a->w_layout, a->k);
  if (a->a_layout == KMOE_A_CHUNKED) {
    KMOE_REQUIRE(a->w_layout == KMOE_W_TILED, KMOE_ERR_UNSUPPORTED,
                 "grouped_gemm_i8: chunked activations need tiled weights");
    KMOE_REQUIRE(a->a_rows >= 1, KMOE_ERR_SHAPE, "grouped_gemm_i8: a_rows=%d < 1", a->a_rows);
    if (a->rows == 0 && !(a->w_tail && a->tail_rows > 0) && !scan) return KMOE_OK;
    return stream_gemm_i8(a, as_stream(stream), scan, quant);
  }
  KMOE_REQUIRE(!scan && !quant, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_i8: only the weight-streaming kernel sorts the pairs or quantises its rows itself");
  KMOE_REQUIRE(a->a_layout == KMOE_A_ROWMAJOR, KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8: a_layout=%d unknown",
               a->a_layout);
  if (a->rows == 0 && !(a->w_tail && a->tail_rows > 0)) return KMOE_OK;
  // Tiled weights and more than a few rows per expert: the persistent tile kernel (variants 5-9, 11-16 force it)
  if (a->w_layout == KMOE_W_TILED && a->k >= 128 &&
      ((a->variant >= 5 && a->variant <= 9) || (a->variant >= 11 && a->variant <= 22) ||
       (a->variant == 0 && ceil_div(expected_rows(a->rows, a->rows_hint), a->E) > kTiledMinRows)))
    return tiled_gemm_i8(a, as_stream(stream));
  KMOE_REQUIRE(a->variant < 5, KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8: variants 5-12 need tiled weights and k >= 128");
  GemmParams p{a->a,   a->lda, a->a_max, a->row_src, a->src_div, a->w,   a->w_max,
               a->lod, a->E,   a->n,     a->k,       a->y,       a->ldy, a->acc_out, a->w_layout == KMOE_W_TILED,
               a->w_tail, a->w_max_tail, a->tail_row0, a->w_tail ? a->tail_rows : 0, a->tail_src0, nullptr, 0, 0.f, 0.f,
               a->act_dtype == KMOE_DT_F16};
  return dispatch<Kind::I8>(p, a->rows, expected_rows(a->rows, a->rows_hint), swiglu, a->variant, as_stream(stream), "kmoe_grouped_gemm_i8");
}

}  // namespace kmoe

using namespace kmoe;

extern "C" int kmoe_grouped_gemm_i8(const kmoe_gemm_i8_args* a, kmoe_stream_t stream) {
  return grouped_gemm_i8_checked(a, stream, nullptr);
}

extern "C" int kmoe_grouped_gemm_bf16(const kmoe_gemm_bf16_args* a, kmoe_stream_t stream) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "grouped_gemm_bf16: args is NULL");
  KMOE_REQUIRE(a->a && a->w && a->lod && a->y, KMOE_ERR_NULL, "grouped_gemm_bf16: NULL tensor pointer");
  KMOE_REQUIRE(a->E >= 1 && a->n >= 16 && a->k >= 8 && a->rows >= 0, KMOE_ERR_SHAPE,
               "grouped_gemm_bf16: E=%d n=%d k=%d rows=%d", a->E, a->n, a->k, a->rows);
  KMOE_REQUIRE(a->k % 8 == 0, KMOE_ERR_SHAPE, "grouped_gemm_bf16: k=%d must be a multiple of 8", a->k);
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  const bool oai = a->act == KMOE_ACT_SWIGLUOAI;
  KMOE_REQUIRE(a->act == KMOE_ACT_NONE || swiglu || oai, KMOE_ERR_UNSUPPORTED, "grouped_gemm_bf16: act=%d unknown",
               a->act);
  KMOE_REQUIRE(a->n % (swiglu ? 32 : 16) == 0, KMOE_ERR_SHAPE, "grouped_gemm_bf16: n=%d must be a multiple of %d",
               a->n, swiglu ? 32 : 16);
  KMOE_REQUIRE(!a->bias || (!swiglu && aligned(a->bias, 8)), KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_bf16: a bias goes with act none or swigluoai and must be 8-byte aligned");
  KMOE_REQUIRE(a->lda % 8 == 0 && a->lda >= a->k, KMOE_ERR_SHAPE,
               "grouped_gemm_bf16: lda=%lld must be a multiple of 8 and >= k", (long long)a->lda);
  const int n_out = (swiglu || oai) ? a->n / 2 : a->n;
  KMOE_REQUIRE(a->ldy % 4 == 0 && a->ldy >= n_out, KMOE_ERR_SHAPE,
               "grouped_gemm_bf16: ldy=%lld must be a multiple of 4 and >= %d", (long long)a->ldy, n_out);
  KMOE_REQUIRE(aligned(a->a, 16) && aligned(a->w, 16) && aligned(a->y, 8), KMOE_ERR_SHAPE,
               "grouped_gemm_bf16: misaligned tensor pointer");
  KMOE_REQUIRE(!a->row_src || a->src_div >= 1, KMOE_ERR_SHAPE, "grouped_gemm_bf16: src_div=%d < 1", a->src_div);
  const bool half = a->act_dtype == KMOE_DT_F16;
  KMOE_REQUIRE(half || a->act_dtype == KMOE_DT_BF16, KMOE_ERR_UNSUPPORTED, "grouped_gemm_bf16: act_dtype=%d unknown",
               a->act_dtype);
  KMOE_REQUIRE(!half || (!a->bias && !oai), KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_bf16: expert biases and swigluoai are built for bf16 only");
  if (a->rows == 0) return KMOE_OK;
  KMOE_REQUIRE(a->w_layout == KMOE_W_ROWMAJOR || (a->w_layout == KMOE_W_TILED && a->k % 32 == 0), KMOE_ERR_SHAPE,
               "grouped_gemm_bf16: w_layout=%d (tiled weights need k %% 32 == 0, k=%d)", a->w_layout, a->k);
  // tiled weights and more than a few rows per expert: the persistent tile kernel (variants 5, 6, 11 force it)
  if (a->w_layout == KMOE_W_TILED && a->k >= 64 && a->ldy % 8 == 0 &&
      (tile_variant(a->variant) || (a->variant == 0 && ceil_div(expected_rows(a->rows, a->rows_hint), a->E) > kTiledMinRows)))
    return tiled_gemm_bf16(a, as_stream(stream));
  KMOE_REQUIRE(!tile_variant(a->variant), KMOE_ERR_UNSUPPORTED, "grouped_gemm_bf16: variants 5, 6, 11-13 need tiled weights, k >= 64 and ldy %% 8 == 0");
  GemmParams p{reinterpret_cast<const int8_t*>(a->a), a->lda * 2, nullptr, a->row_src, a->src_div,
               reinterpret_cast<const int8_t*>(a->w), nullptr,    a->lod,  a->E,       a->n,
               a->k * 2,                              a->y,       a->ldy,  nullptr, a->w_layout == KMOE_W_TILED,
               nullptr, nullptr, 0, 0, 0, a->bias, oai ? 1 : 0, a->act_alpha, a->act_limit};
  const int live = expected_rows(a->rows, a->rows_hint);
  if (half) return dispatch<Kind::F16>(p, a->rows, live, swiglu, a->variant, as_stream(stream), "kmoe_grouped_gemm_bf16 (half)");
  return dispatch<Kind::BF16>(p, a->rows, live, swiglu, a->variant, as_stream(stream), "kmoe_grouped_gemm_bf16");
}

extern "C" int kmoe_grouped_gemm_fp8_block(const kmoe_gemm_fp8_args* a, kmoe_stream_t stream) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "grouped_gemm_fp8_block: args is NULL");
  KMOE_REQUIRE(a->a && a->a_scale && a->w && a->w_scale && a->lod && a->y, KMOE_ERR_NULL,
               "grouped_gemm_fp8_block: NULL tensor pointer");
  KMOE_REQUIRE(a->E >= 1 && a->n >= 128 && a->k >= 128 && a->rows >= 0, KMOE_ERR_SHAPE,
               "grouped_gemm_fp8_block: E=%d n=%d k=%d rows=%d", a->E, a->n, a->k, a->rows);
  KMOE_REQUIRE(a->act_dtype == KMOE_DT_BF16 || a->act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_fp8_block: act_dtype=%d unknown", a->act_dtype);
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  KMOE_REQUIRE(a->act == KMOE_ACT_NONE || swiglu, KMOE_ERR_UNSUPPORTED, "grouped_gemm_fp8_block: act=%d unknown",
               a->act);
  KMOE_REQUIRE(a->k % 128 == 0 && a->n % (swiglu ? 256 : 128) == 0, KMOE_ERR_SHAPE,
               "grouped_gemm_fp8_block: k=%d and n=%d must be multiples of 128 (n of 256 with SwiGLU)", a->k, a->n);
  KMOE_REQUIRE(a->lda % 16 == 0 && a->lda >= a->k, KMOE_ERR_SHAPE,
               "grouped_gemm_fp8_block: lda=%lld must be a multiple of 16 and >= k", (long long)a->lda);
  const int n_out = swiglu ? a->n / 2 : a->n;
  KMOE_REQUIRE(a->ldy % 4 == 0 && a->ldy >= n_out, KMOE_ERR_SHAPE,
               "grouped_gemm_fp8_block: ldy=%lld must be a multiple of 4 and >= %d", (long long)a->ldy, n_out);
  KMOE_REQUIRE(aligned(a->a, 16) && aligned(a->w, 16) && aligned(a->y, 8), KMOE_ERR_SHAPE,
               "grouped_gemm_fp8_block: misaligned tensor pointer");
  KMOE_REQUIRE(!a->row_src || a->src_div >= 1, KMOE_ERR_SHAPE, "grouped_gemm_fp8_block: src_div=%d < 1", a->src_div);
  KMOE_REQUIRE(!a->w_tail || (a->w_scale_tail && a->tail_rows >= 0 && a->tail_row0 >= 0 && a->tail_src0 >= 0 &&
                              aligned(a->w_tail, 16)),
               KMOE_ERR_SHAPE, "grouped_gemm_fp8_block: bad tail expert (w_scale_tail, tail_row0=%d, tail_rows=%d)",
               a->tail_row0, a->tail_rows);
  const int tail_rows = a->w_tail ? a->tail_rows : 0;
  if (a->rows == 0 && tail_rows == 0) return KMOE_OK;
  KMOE_REQUIRE(a->w_layout == KMOE_W_ROWMAJOR || a->w_layout == KMOE_W_TILED, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_fp8_block: w_layout=%d unknown", a->w_layout);
  // tiled weights and more than a few rows per expert: the persistent tile kernel (variants 5, 6, 11 force it)
  const bool tall_variant = a->variant == 8 || a->variant == 14 || (a->variant >= 17 && a->variant <= 19);  // 8-wave tiles of 256 / 192 rows; 17: chosen on the device; 18, 19: wide 192- / 128-row tiles
  if (a->w_layout == KMOE_W_TILED && a->k <= 8192 && a->ldy % 8 == 0 &&
      (tile_variant(a->variant) || tall_variant || (a->variant == 0 && ceil_div(expected_rows(a->rows, a->rows_hint), a->E) > kTiledMinRows)))
    return tiled_gemm_fp8(a, as_stream(stream));
  KMOE_REQUIRE(!tile_variant(a->variant) && !tall_variant, KMOE_ERR_UNSUPPORTED,
               "grouped_gemm_fp8_block: variants 5, 6, 8, 11-14 need tiled weights, k <= 8192");
  GemmParams p{reinterpret_cast<const int8_t*>(a->a), a->lda, a->a_scale, a->row_src, a->src_div,
               reinterpret_cast<const int8_t*>(a->w), a->w_scale, a->lod,  a->E,       a->n,
               a->k,                                  a->y,       a->ldy,  nullptr, a->w_layout == KMOE_W_TILED,
               reinterpret_cast<const int8_t*>(a->w_tail), a->w_scale_tail, a->tail_row0, tail_rows, a->tail_src0,
               nullptr, 0, 0.f, 0.f, a->act_dtype == KMOE_DT_F16};
  return dispatch<Kind::FP8>(p, a->rows, expected_rows(a->rows, a->rows_hint), swiglu, a->variant, as_stream(stream), "kmoe_grouped_gemm_fp8_block");
}
