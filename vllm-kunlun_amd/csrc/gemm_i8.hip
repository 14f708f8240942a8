// W8A8 grouped GEMM on gfx950 int8 MFMA (v_mfma_i32_16x16x64_i8).
//
// Roles: the WEIGHT tile is the first MFMA operand (16 output channels x 64 k),
// the ACTIVATION tile the second (64 k x 16 sorted rows). A lane therefore ends
// up with 4 consecutive output channels of one row: channel 4*(lane/16)+q,
// row lane%16 — what the dequant / SiLU-mul epilogue and an 8-byte store want.
//
// Data movement per workgroup:
//   weights     global -> registers, 16 B per lane, one K chunk (256 B per
//               channel row) prefetched ahead of the MFMAs that consume it; every
//               wave owns its own output channels, so weights never need LDS;
//   activations global (gathered through the sort) -> LDS, double-buffered per
//               K chunk, shared by all waves of the workgroup.
// Inside a 256-byte chunk lane group g = lane/16 covers bytes [64g, 64g+64) of
// both operands; MFMA step j uses bytes 64g+16j.. of each. Any assignment of k
// to (group, step) is valid for a dot product as long as both operands agree.
#include "kmoe_common.h"

namespace kmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kKC = 256;           // bytes of K per chunk
constexpr int kJ = kKC / 64;       // MFMA steps per chunk
constexpr int kPitch = kKC + 16;   // LDS row pitch: rows 16 B apart mod 256 -> conflict-free b128 reads

struct GemmParams {
  const int8_t* a;
  int64_t lda;
  const float* a_max;
  const int32_t* row_src;
  int32_t src_div;
  const int8_t* w;
  const float* w_max;
  const int32_t* lod;
  int32_t E, n, k;
  uint16_t* y;
  int64_t ldy;
  int32_t* acc_out;
};

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
// are cut into tiles of TM. Returns false when t is past the last tile.
template <int TM>
__device__ inline bool locate_tile(const int32_t* __restrict__ lod, int E, int t, int& e_out, int& row0_out) {
  const int lane = lane_id();
  const int epl = (E + kWave - 1) / kWave;
  const int e_begin = lane * epl;
  int local = 0;
  for (int i = 0; i < epl; ++i) {
    const int e = e_begin + i;
    if (e < E) local += (lod[e + 1] - lod[e] + TM - 1) / TM;
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
      const int lo = lod[e];
      const int tiles = (lod[e + 1] - lo + TM - 1) / TM;
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
template <int MF, int NF, int WAVES, bool SWIGLU, bool LOCATE>
__global__ __launch_bounds__(WAVES* kWave) void gemm_i8_kernel(const GemmParams p) {
  constexpr int TM = 16 * MF;
  constexpr int THREADS = WAVES * kWave;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;       // fragments per wave in "half space"
  constexpr int NA = (TM * (kKC / 16) + THREADS - 1) / THREADS;  // activation vectors per thread per chunk
  static_assert(!SWIGLU || NF % 2 == 0, "SwiGLU pairs gate and up fragments");

  __shared__ __attribute__((aligned(16))) int8_t lds_a[2][TM * kPitch];

  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;  // row (activations) / channel (weights) inside a fragment
  const int lg = lane >> 4;  // k group

  int e, row_begin, row_end;
  if (LOCATE) {
    if (!locate_tile<TM>(p.lod, p.E, blockIdx.y, e, row_begin)) return;
    row_end = min(p.lod[e + 1], row_begin + TM);
  } else {
    e = blockIdx.y;
    row_begin = p.lod[e];
    row_end = p.lod[e + 1];
    if (row_begin >= row_end) return;
  }

  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int col_base = (blockIdx.x * WAVES + wave) * NFH * 16;

  // per-fragment weight row pointers (channel li of the fragment, k group lg)
  const int8_t* wp[NF];
  bool wok[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int fh = SWIGLU ? f % NFH : f;
    const int c = col_base + fh * 16;
    wok[f] = c < n_half;
    col[f] = (SWIGLU && f >= NFH) ? n_half + c : c;
    wp[f] = p.w + (static_cast<size_t>(e) * p.n + (wok[f] ? col[f] + li : 0)) * p.k + lg * 64;
  }
  const int nchunks = (p.k + kKC - 1) / kKC;

  for (int row0 = row_begin; row0 < row_end; row0 += TM) {
    // activation source pointers for this thread's slots of the LDS tile
    const int8_t* ap[NA];
    int a_lds[NA];
    int a_kv[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int v = threadIdx.x + i * THREADS;
      const int r = v >> 4;  // 16 vectors of 16 B per row and chunk
      const int kv = v & 15;
      a_kv[i] = kv * 16;
      a_lds[i] = (v < TM * 16) ? r * kPitch + kv * 16 : -1;
      ap[i] = nullptr;
      if (v < TM * 16 && row0 + r < row_end) {
        const int sr = p.row_src ? p.row_src[row0 + r] / p.src_div : row0 + r;
        ap[i] = p.a + static_cast<size_t>(sr) * p.lda + kv * 16;
      }
    }

    v4i acc[MF][NF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf)
#pragma unroll
      for (int f = 0; f < NF; ++f) acc[mf][f] = (v4i){0, 0, 0, 0};

    v4i wbuf[2][NF][kJ];
    v4i areg[NA];

    auto load_w = [&](v4i(&dst)[NF][kJ], int chunk) {
      const int kc = chunk * kKC;
#pragma unroll
      for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int j = 0; j < kJ; ++j) {
          const int kk = kc + lg * 64 + j * 16;
          dst[f][j] = (wok[f] && kk < p.k) ? *reinterpret_cast<const v4i*>(wp[f] + kc + j * 16) : (v4i){0, 0, 0, 0};
        }
    };
    auto load_a = [&](int chunk) {
      const int kc = chunk * kKC;
#pragma unroll
      for (int i = 0; i < NA; ++i)
        areg[i] = (ap[i] && kc + a_kv[i] < p.k) ? *reinterpret_cast<const v4i*>(ap[i] + kc) : (v4i){0, 0, 0, 0};
    };
    auto store_a = [&](int buf) {
#pragma unroll
      for (int i = 0; i < NA; ++i)
        if (a_lds[i] >= 0) *reinterpret_cast<v4i*>(&lds_a[buf][a_lds[i]]) = areg[i];
    };
    auto compute = [&](const v4i(&wcur)[NF][kJ], int buf) {
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        v4i af[MF];
#pragma unroll
        for (int mf = 0; mf < MF; ++mf)
          af[mf] = *reinterpret_cast<const v4i*>(&lds_a[buf][(mf * 16 + li) * kPitch + lg * 64 + j * 16]);
#pragma unroll
        for (int mf = 0; mf < MF; ++mf)
#pragma unroll
          for (int f = 0; f < NF; ++f)
            acc[mf][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wcur[f][j], af[mf], acc[mf][f], 0, 0, 0);
      }
    };
    auto stage = [&](int chunk, const v4i(&wcur)[NF][kJ], v4i(&wnext)[NF][kJ], int buf) {
      const bool more = chunk + 1 < nchunks;
      if (more) {
        load_w(wnext, chunk + 1);
        load_a(chunk + 1);
      }
      compute(wcur, buf);
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
      const int sr = p.row_src ? p.row_src[r] / p.src_div : r;
      const float sa = p.a_max[sr] / 127.0f;
#pragma unroll
      for (int f = 0; f < NFH; ++f) {
        if (!wok[f]) continue;
        const int c0 = col[f] + lg * 4;
        const float4 wm = *reinterpret_cast<const float4*>(p.w_max + static_cast<size_t>(e) * p.n + c0);
        const float sw[4] = {wm.x / 127.0f, wm.y / 127.0f, wm.z / 127.0f, wm.w / 127.0f};
        uint16_t yv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) yv[q] = f32_to_bf16((static_cast<float>(acc[mf][f][q]) * sa) * sw[q]);
        if (p.acc_out)
          *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + c0) = acc[mf][f];
        if (SWIGLU) {
          const int fu = f + NFH;
          const int cu = col[fu] + lg * 4;
          const float4 um = *reinterpret_cast<const float4*>(p.w_max + static_cast<size_t>(e) * p.n + cu);
          const float su[4] = {um.x / 127.0f, um.y / 127.0f, um.z / 127.0f, um.w / 127.0f};
          if (p.acc_out)
            *reinterpret_cast<v4i*>(p.acc_out + static_cast<size_t>(r) * p.n + cu) = acc[mf][fu];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint16_t uv = f32_to_bf16((static_cast<float>(acc[mf][fu][q]) * sa) * su[q]);
            yv[q] = f32_to_bf16(silu_fixed(bf16_to_f32(yv[q])) * bf16_to_f32(uv));
          }
        }
        const uint2 packed = make_uint2(yv[0] | (static_cast<uint32_t>(yv[1]) << 16),
                                        yv[2] | (static_cast<uint32_t>(yv[3]) << 16));
        *reinterpret_cast<uint2*>(p.y + static_cast<size_t>(r) * p.ldy + c0) = packed;
      }
    }
  }
}

template <int MF, int NF, int WAVES, bool SWIGLU, bool LOCATE>
int launch(const GemmParams& p, int rows, hipStream_t s) {
  constexpr int TM = 16 * MF;
  constexpr int NFH = SWIGLU ? NF / 2 : NF;
  const int n_half = SWIGLU ? p.n / 2 : p.n;
  const int grid_x = ceil_div(n_half, WAVES * NFH * 16);
  const int grid_y = LOCATE ? rows / TM + min(p.E, rows) : p.E;
  if (grid_y == 0) return KMOE_OK;
  hipLaunchKernelGGL((gemm_i8_kernel<MF, NF, WAVES, SWIGLU, LOCATE>), dim3(grid_x, grid_y), dim3(WAVES * kWave), 0, s,
                     p);
  return check_launch("kmoe_grouped_gemm_i8");
}

}  // namespace
}  // namespace kmoe

using namespace kmoe;

extern "C" int kmoe_grouped_gemm_i8(const kmoe_gemm_i8_args* a, kmoe_stream_t stream) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "grouped_gemm_i8: args is NULL");
  KMOE_REQUIRE(a->a && a->a_max && a->w && a->w_max && a->lod && a->y, KMOE_ERR_NULL,
               "grouped_gemm_i8: NULL tensor pointer");
  KMOE_REQUIRE(a->E >= 1 && a->n >= 16 && a->k >= 16 && a->rows >= 0, KMOE_ERR_SHAPE,
               "grouped_gemm_i8: E=%d n=%d k=%d rows=%d", a->E, a->n, a->k, a->rows);
  KMOE_REQUIRE(a->k % 16 == 0, KMOE_ERR_SHAPE, "grouped_gemm_i8: k=%d must be a multiple of 16", a->k);
  const bool swiglu = a->act == KMOE_ACT_SWIGLU;
  KMOE_REQUIRE(a->act == KMOE_ACT_NONE || swiglu, KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8: act=%d unknown", a->act);
  KMOE_REQUIRE(a->n % (swiglu ? 32 : 16) == 0, KMOE_ERR_SHAPE, "grouped_gemm_i8: n=%d must be a multiple of %d",
               a->n, swiglu ? 32 : 16);
  KMOE_REQUIRE(a->lda % 16 == 0 && a->lda >= a->k, KMOE_ERR_SHAPE,
               "grouped_gemm_i8: lda=%lld must be a multiple of 16 and >= k", (long long)a->lda);
  const int n_out = swiglu ? a->n / 2 : a->n;
  KMOE_REQUIRE(a->ldy % 4 == 0 && a->ldy >= n_out, KMOE_ERR_SHAPE,
               "grouped_gemm_i8: ldy=%lld must be a multiple of 4 and >= %d", (long long)a->ldy, n_out);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(a->a) & 15) == 0 && (reinterpret_cast<uintptr_t>(a->w) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(a->y) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(a->w_max) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(a->acc_out) & 15) == 0,
               KMOE_ERR_SHAPE, "grouped_gemm_i8: misaligned tensor pointer");
  KMOE_REQUIRE(!a->row_src || a->src_div >= 1, KMOE_ERR_SHAPE, "grouped_gemm_i8: src_div=%d < 1", a->src_div);
  if (a->rows == 0) return KMOE_OK;

  GemmParams p{a->a, a->lda, a->a_max, a->row_src, a->src_div, a->w, a->w_max, a->lod,
               a->E, a->n,   a->k,     a->y,       a->ldy,     a->acc_out};
  hipStream_t s = as_stream(stream);
  int variant = a->variant;
  if (variant == 0) {
    // rows per expert if the routing were uniform; decides streaming vs tiled
    const int avg = ceil_div(a->rows, a->E);
    variant = avg <= 16 ? 1 : (avg <= 48 ? 2 : 3);
  }
  switch (variant) {
    case 1:  // weight streaming: 16-row tiles, one expert per workgroup column
      return swiglu ? launch<1, 2, 4, true, false>(p, a->rows, s) : launch<1, 1, 4, false, false>(p, a->rows, s);
    case 2:  // 32-row tiles
      return swiglu ? launch<2, 2, 4, true, false>(p, a->rows, s) : launch<2, 2, 4, false, false>(p, a->rows, s);
    case 3:  // 128-row tiles, work list balanced over experts
      return swiglu ? launch<8, 4, 4, true, true>(p, a->rows, s) : launch<8, 4, 4, false, true>(p, a->rows, s);
    default:
      return fail(KMOE_ERR_UNSUPPORTED, "grouped_gemm_i8: variant=%d unknown", a->variant);
  }
}
