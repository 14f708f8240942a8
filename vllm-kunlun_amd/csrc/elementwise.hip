// Bandwidth-bound stages: per-row int8 quantisation, per-group fp8 quantisation,
// SiLU-and-mul, and the weighted top-K combine. All move 16 bytes per lane.
#include "quant_body.h"

namespace kmoe {
namespace {

template <int TPR, int NV>
__global__ __launch_bounds__(256) void quant_i8_rows_kernel(const uint16_t* __restrict__ x, int64_t ld_x, int R,
                                                           int C, int8_t* __restrict__ q, int64_t ld_q,
                                                           float* __restrict__ row_max, int chunked, int f16) {
  quant_i8_rows_body<TPR, NV>(x, ld_x, R, C, q, ld_q, row_max, chunked, blockIdx.x, f16 != 0);
}

// ---------------------------------------- static and asymmetric int8 (the other modes of scaled_int8_quant)
// one thread: 8 values; scale and zero point of the whole tensor
__global__ __launch_bounds__(256) void quant_i8_static_kernel(const uint16_t* __restrict__ x, int64_t ld_x, int R,
                                                             int C, const float* __restrict__ scale,
                                                             const int32_t* __restrict__ azp, int8_t* __restrict__ q,
                                                             int64_t ld_q, int f16) {
  const int vec_per_row = C / 8;
  const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<long long>(R) * vec_per_row) return;
  const int r = static_cast<int>(idx / vec_per_row), c = static_cast<int>(idx % vec_per_row) * 8;
  const float s = scale[0];
  const int z = azp ? azp[0] : 0;
  Pack8 v;
  v.v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * ld_x + c);
  uint32_t w[2] = {0, 0};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    // (the float is clamped before the conversion so that the int32 sum with the zero point cannot overflow)
    const float f = fminf(fmaxf(__builtin_rintf(act_to_f32(v.h[j], f16 != 0) / s), -2147483000.0f), 2147483000.0f);
    const long long t = static_cast<long long>(static_cast<int>(f)) + z;
    const int qi = static_cast<int>(t < -128 ? -128 : (t > 127 ? 127 : t));
    w[j >> 2] |= static_cast<uint32_t>(qi & 0xff) << (8 * (j & 3));
  }
  *reinterpret_cast<uint2*>(q + static_cast<size_t>(r) * ld_q + c) = make_uint2(w[0], w[1]);
}

// one workgroup per row: min and max, then the codes (the row is read twice; this mode is not on a hot path)
__global__ __launch_bounds__(256) void quant_i8_rows_azp_kernel(const uint16_t* __restrict__ x, int64_t ld_x, int C,
                                                               int8_t* __restrict__ q, int64_t ld_q,
                                                               float* __restrict__ row_scale,
                                                               int32_t* __restrict__ row_azp, int f16) {
  __shared__ float red_lo[4], red_hi[4];
  const int r = blockIdx.x;
  const uint16_t* xr = x + static_cast<size_t>(r) * ld_x;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  for (int c = threadIdx.x; c < C; c += 256) {
    const float f = act_to_f32(xr[c], f16 != 0);
    lo = fminf(lo, f);
    hi = fmaxf(hi, f);
  }
  hi = wave_max(hi);
  lo = -wave_max(-lo);
  if (lane_id() == 0) {
    red_lo[threadIdx.x >> 6] = lo;
    red_hi[threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  lo = fminf(fminf(red_lo[0], red_lo[1]), fminf(red_lo[2], red_lo[3]));
  hi = fmaxf(fmaxf(red_hi[0], red_hi[1]), fmaxf(red_hi[2], red_hi[3]));
  float s = (hi - lo) / 255.0f;
  if (!(s > 0.0f)) s = 1.0f;  // a constant row: every code is the zero point
  const float zf = fminf(fmaxf(__builtin_rintf(-128.0f - lo / s), -2147483000.0f), 2147483000.0f);
  const int z = static_cast<int>(zf);
  for (int c = threadIdx.x; c < C; c += 256) {
    const float f = fminf(fmaxf(__builtin_rintf(act_to_f32(xr[c], f16 != 0) / s), -2147483000.0f), 2147483000.0f);
    const long long t = static_cast<long long>(static_cast<int>(f)) + z;
    q[static_cast<size_t>(r) * ld_q + c] = static_cast<int8_t>(t < -128 ? -128 : (t > 127 ? 127 : t));
  }
  if (threadIdx.x == 0) {
    row_scale[r] = s;
    row_azp[r] = z;
  }
}

// ------------------------------------------------------------- fp8 group128
// OCP e4m3fn encode of two floats, round-to-nearest-even, saturating at 448 (NaN -> the largest
// code of its sign): the conversion instruction of gfx950 (v_cvt_pk_fp8_f32 encodes the OCP format
// there) after an explicit clamp, so that its own overflow handling never comes into play.
__device__ inline uint32_t pack2_e4m3fn(float a, float b) {
  auto clamp = [](float f) {
    f = f != f ? __builtin_copysignf(448.0f, f) : f;
    return __builtin_fminf(__builtin_fmaxf(f, -448.0f), 448.0f);
  };
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(clamp(a), clamp(b), 0, false)) & 0xffffu;
}

// 16 lanes x 8 values = one 128-column group; 4 groups per wave. (Several groups per team, all
// requested up front, measured no faster: the eight IEEE divisions per lane set the pace.)
__global__ __launch_bounds__(256) void quant_fp8_group128_kernel(const uint16_t* __restrict__ x, int64_t ld_x,
                                                                int R, int C, uint8_t* __restrict__ q,
                                                                int64_t ld_q, float* __restrict__ scale, int f16) {
  const int groups_per_row = C / 128;
  const long long total = static_cast<long long>(R) * groups_per_row;
  const long long gid = static_cast<long long>(blockIdx.x) * 16 + (threadIdx.x >> 4);
  const int t = threadIdx.x & 15;
  const bool live = gid < total;
  const int r = live ? static_cast<int>(gid / groups_per_row) : 0;
  const int g = live ? static_cast<int>(gid % groups_per_row) : 0;
  Pack8 val;
  val.v = make_uint4(0, 0, 0, 0);
  if (live) val.v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * ld_x + g * 128 + t * 8);
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(act_to_f32(val.h[j], f16 != 0)));
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
  if (!live) return;
  const float s = amax / 448.0f;
  float f[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = s > 0.0f ? act_to_f32(val.h[j], f16 != 0) / s : 0.0f;
  const uint32_t w[2] = {pack2_e4m3fn(f[0], f[1]) | (pack2_e4m3fn(f[2], f[3]) << 16),
                         pack2_e4m3fn(f[4], f[5]) | (pack2_e4m3fn(f[6], f[7]) << 16)};
  *reinterpret_cast<uint2*>(q + static_cast<size_t>(r) * ld_q + g * 128 + t * 8) = make_uint2(w[0], w[1]);
  if (t == 0) scale[static_cast<size_t>(r) * groups_per_row + g] = s;
}

// ------------------------------------------------------------ silu-and-mul
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint16_t* __restrict__ y, int64_t ld_y, int R,
                                                          int I, uint16_t* __restrict__ out, int64_t ld_out,
                                                          int dt) {
  const bool f16 = dt != 0;
  const int vec_per_row = I / 8;
  const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<long long>(R) * vec_per_row) return;
  const int r = static_cast<int>(idx / vec_per_row);
  const int c = static_cast<int>(idx % vec_per_row) * 8;
  Pack8 g, u, o;
  g.v = *reinterpret_cast<const uint4*>(y + static_cast<size_t>(r) * ld_y + c);
  u.v = *reinterpret_cast<const uint4*>(y + static_cast<size_t>(r) * ld_y + I + c);
#pragma unroll
  for (int j = 0; j < 8; ++j) o.h[j] = f32_to_act(silu_hw(act_to_f32(g.h[j], f16)) * act_to_f32(u.h[j], f16), f16);
  *reinterpret_cast<uint4*>(out + static_cast<size_t>(r) * ld_out + c) = o.v;
}

// silu_hw of every 16-bit activation pattern (see kmoe_silu_table)
__global__ __launch_bounds__(256) void silu_table_kernel(float* __restrict__ table, int dt) {
  const unsigned h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h < 65536u) table[h] = silu_hw(act_to_f32(static_cast<uint16_t>(h), dt != 0));
}

// ----------------------------------------------------------------- combine
constexpr int kMaxTopK = 64;

__global__ __launch_bounds__(256) void combine_kernel(const uint16_t* __restrict__ x, int64_t ld_x,
                                                     const int32_t* __restrict__ moe_index,
                                                     const float* __restrict__ topk_w,
                                                     const float* __restrict__ dq, int K, int H, float out_scale,
                                                     int epilogue, const uint16_t* __restrict__ addend,
                                                     int64_t ld_addend, float addend_scale,
                                                     uint16_t* __restrict__ out, int64_t ld_out, int dt) {
  const bool f16 = dt != 0;
  __shared__ int rows[kMaxTopK];
  __shared__ float wts[kMaxTopK];
  const int m = blockIdx.x;
  if (threadIdx.x < K) {
    const size_t j = static_cast<size_t>(m) * K + threadIdx.x;
    rows[threadIdx.x] = moe_index[j];
    wts[threadIdx.x] = dq ? topk_w[j] * dq[j] : topk_w[j];
  }
  __syncthreads();
  // blockIdx.y: which 2048-column slice of the row (wide rows at small M: more workgroups)
  for (int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8; c < H; c += gridDim.y * blockDim.x * 8) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    constexpr int kBatch = 4;  // rows loaded together: one memory round trip per 4 experts, not per expert
    for (int k0 = 0; k0 < K; k0 += kBatch) {
      Pack8 p[kBatch];
      int r[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        r[i] = k0 + i < K ? rows[k0 + i] : -1;
        p[i].v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(max(r[i], 0)) * ld_x + c);
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        if (r[i] < 0) continue;  // pair without a sorted row contributes nothing (its load read row 0)
        const float w = wts[k0 + i];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(w, act_to_f32(p[i].h[j], f16), acc[j]);
      }
    }
    Pack8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.h[j] = f32_to_act(acc[j], f16);
    if (epilogue) {
      Pack8 a;
      a.v = make_uint4(0, 0, 0, 0);
      if (addend) a.v = *reinterpret_cast<const uint4*>(addend + static_cast<size_t>(m) * ld_addend + c);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // each step rounds to the activation dtype, as the caller's tensor operations would
        const uint16_t scaled = out_scale != 1.0f ? f32_to_act(act_to_f32(o.h[j], f16) * out_scale, f16) : o.h[j];
        const uint16_t add = addend_scale != 1.0f ? f32_to_act(act_to_f32(a.h[j], f16) * addend_scale, f16) : a.h[j];
        o.h[j] = addend ? f32_to_act(act_to_f32(scaled, f16) + act_to_f32(add, f16), f16) : scaled;
      }
    }
    *reinterpret_cast<uint4*>(out + static_cast<size_t>(m) * ld_out + c) = o.v;
  }
}

__global__ void fill_dense_lod_kernel(int32_t* lod2, int rows) {
  if (threadIdx.x == 0) lod2[0] = 0;
  if (threadIdx.x == 1) lod2[1] = rows;
}

// one thread: 8 interleaved inputs (16 B) -> 4 outputs (8 B)
__global__ void swigluoai_and_mul_kernel(const uint16_t* __restrict__ y, int64_t ld_y, int R, int I, float alpha,
                                         float limit, uint16_t* __restrict__ out, int64_t ld_out) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int per_row = I / 4;
  if (i >= static_cast<long long>(R) * per_row) return;
  const int r = static_cast<int>(i / per_row), v = static_cast<int>(i % per_row);
  Pack8 in;
  in.v = *reinterpret_cast<const uint4*>(y + static_cast<size_t>(r) * ld_y + v * 8);
  uint16_t o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = swigluoai_bf16(in.h[2 * j], in.h[2 * j + 1], alpha, limit);
  *reinterpret_cast<uint2*>(out + static_cast<size_t>(r) * ld_out + v * 4) =
      make_uint2(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16));
}

// one thread: 8 packed bytes -> 16 bf16 (or half) values
__global__ void dequant_w4_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ scale, long long rows,
                                  int k, int group_size, uint16_t* __restrict__ out, int f16) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int per_row = k / 16;
  if (i >= rows * per_row) return;
  const long long r = i / per_row;
  const int j0 = static_cast<int>(i % per_row) * 16;
  const uint2 in = *reinterpret_cast<const uint2*>(packed + r * (k / 2) + j0 / 2);
  const uint32_t word[2] = {in.x, in.y};
  const uint16_t* srow = scale + r * (k / group_size);
  uint32_t o[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const uint32_t byte = (word[b >> 2] >> (8 * (b & 3))) & 0xffu;
    const int j = j0 + 2 * b;  // group_size is even: both nibbles of a byte share a scale
    // the product of a 4-bit and an 8-bit (11-bit) significand is exact in f32: one rounding, to the 16-bit type
    const float s = act_to_f32(srow[j / group_size], f16 != 0);
    const uint16_t lo = f32_to_act(static_cast<float>(static_cast<int>(byte & 0xf) - 8) * s, f16 != 0);
    const uint16_t hi = f32_to_act(static_cast<float>(static_cast<int>(byte >> 4) - 8) * s, f16 != 0);
    o[b] = lo | (static_cast<uint32_t>(hi) << 16);
  }
  uint4* dst = reinterpret_cast<uint4*>(out + r * k + j0);
  dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
  dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

}  // namespace

int fill_dense_lod(int32_t* lod2, int rows, hipStream_t stream) {
  hipLaunchKernelGGL(fill_dense_lod_kernel, dim3(1), dim3(64), 0, stream, lod2, rows);
  return check_launch("fill_dense_lod");
}

}  // namespace kmoe

using namespace kmoe;

namespace {
int quant_i8_launch(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q, float* row_max,
                    int chunked, int f16, hipStream_t s, const char* what) {
  if (C <= 32 * 8 * 3 && R >= 2048) {
    // short rows, many of them (the second quantisation of a prefill batch): half a wave per row keeps every lane
    // busy and two rows' loads in flight per wave (Qwen3 shape, 65536 rows of 768: 37 -> 31 us inside the layer)
    hipLaunchKernelGGL((quant_i8_rows_kernel<32, 3>), dim3(ceil_div(R, 8)), dim3(256), 0, s, x, ld_x, R, C, q, ld_q,
                       row_max, chunked, f16);
  } else if (C <= 64 * 8 * 2) {
    hipLaunchKernelGGL((quant_i8_rows_kernel<64, 2>), dim3(ceil_div(R, 4)), dim3(256), 0, s, x, ld_x, R, C, q, ld_q,
                       row_max, chunked, f16);
  } else if (C <= 64 * 8 * 4) {
    hipLaunchKernelGGL((quant_i8_rows_kernel<64, 4>), dim3(ceil_div(R, 4)), dim3(256), 0, s, x, ld_x, R, C, q, ld_q,
                       row_max, chunked, f16);
  } else if (C <= 256 * 8 * 4) {
    hipLaunchKernelGGL((quant_i8_rows_kernel<256, 4>), dim3(R), dim3(256), 0, s, x, ld_x, R, C, q, ld_q, row_max,
                       chunked, f16);
  } else if (C <= 256 * 8 * 8) {
    hipLaunchKernelGGL((quant_i8_rows_kernel<256, 8>), dim3(R), dim3(256), 0, s, x, ld_x, R, C, q, ld_q, row_max,
                       chunked, f16);
  } else if (C <= 256 * 8 * 16) {
    hipLaunchKernelGGL((quant_i8_rows_kernel<256, 16>), dim3(R), dim3(256), 0, s, x, ld_x, R, C, q, ld_q, row_max,
                       chunked, f16);
  } else {  // up to 65536 values: 128 registers of row data per thread
    hipLaunchKernelGGL((quant_i8_rows_kernel<256, 32>), dim3(R), dim3(256), 0, s, x, ld_x, R, C, q, ld_q, row_max,
                       chunked, f16);
  }
  return check_launch(what);
}
}  // namespace

namespace {
int check_dtype(int act_dtype, const char* what) {
  KMOE_REQUIRE(act_dtype == KMOE_DT_BF16 || act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED, "%s: act_dtype=%d unknown",
               what, act_dtype);
  return KMOE_OK;
}
}  // namespace

extern "C" int kmoe_quant_i8_rows(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                                  float* row_max, kmoe_stream_t stream) {
  return kmoe_quant_i8_rows_dt(x, ld_x, R, C, q, ld_q, row_max, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_quant_i8_rows_chunked(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, float* row_max,
                                          kmoe_stream_t stream) {
  return kmoe_quant_i8_rows_chunked_dt(x, ld_x, R, C, q, row_max, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_quant_i8_rows_dt(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                                     float* row_max, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "quant_i8_rows")) return rc;
  KMOE_REQUIRE(x && q && row_max, KMOE_ERR_NULL, "quant_i8_rows: NULL pointer");
  KMOE_REQUIRE(R >= 0 && C >= 8 && C % 8 == 0 && C <= 65536, KMOE_ERR_SHAPE,
               "quant_i8_rows: R=%d C=%d (need C %% 8 == 0, 8 <= C <= 65536)", R, C);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_q % 8 == 0 && ld_x >= C && ld_q >= C, KMOE_ERR_SHAPE,
               "quant_i8_rows: row strides %lld/%lld must be multiples of 8 and >= C", (long long)ld_x,
               (long long)ld_q);
  if (R == 0) return KMOE_OK;
  return quant_i8_launch(x, ld_x, R, C, q, ld_q, row_max, 0, act_dtype, as_stream(stream), "kmoe_quant_i8_rows");
}

extern "C" int kmoe_quant_i8_rows_chunked_dt(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, float* row_max,
                                             int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "quant_i8_rows_chunked")) return rc;
  KMOE_REQUIRE(x && q && row_max, KMOE_ERR_NULL, "quant_i8_rows_chunked: NULL pointer");
  KMOE_REQUIRE(R >= 0 && C >= 64 && C % 64 == 0 && C <= 65536, KMOE_ERR_SHAPE,
               "quant_i8_rows_chunked: R=%d C=%d (need C %% 64 == 0, 64 <= C <= 65536)", R, C);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_x >= C, KMOE_ERR_SHAPE,
               "quant_i8_rows_chunked: row stride %lld must be a multiple of 8 and >= C", (long long)ld_x);
  if (R == 0) return KMOE_OK;
  return quant_i8_launch(x, ld_x, R, C, q, 0, row_max, 1, act_dtype, as_stream(stream), "kmoe_quant_i8_rows_chunked");
}

extern "C" int kmoe_quant_fp8_group128(const uint16_t* x, int64_t ld_x, int R, int C, uint8_t* q, int64_t ld_q,
                                       float* scale, kmoe_stream_t stream) {
  return kmoe_quant_fp8_group128_dt(x, ld_x, R, C, q, ld_q, scale, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_quant_fp8_group128_dt(const uint16_t* x, int64_t ld_x, int R, int C, uint8_t* q, int64_t ld_q,
                                          float* scale, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "quant_fp8_group128")) return rc;
  KMOE_REQUIRE(x && q && scale, KMOE_ERR_NULL, "quant_fp8_group128: NULL pointer");
  KMOE_REQUIRE(R >= 0 && C >= 128 && C % 128 == 0, KMOE_ERR_SHAPE, "quant_fp8_group128: R=%d C=%d (need C %% 128 == 0)",
               R, C);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_q % 8 == 0 && ld_x >= C && ld_q >= C, KMOE_ERR_SHAPE,
               "quant_fp8_group128: row strides %lld/%lld must be multiples of 8 and >= C", (long long)ld_x,
               (long long)ld_q);
  if (R == 0) return KMOE_OK;
  const long long groups = static_cast<long long>(R) * (C / 128);
  hipLaunchKernelGGL(quant_fp8_group128_kernel, dim3(static_cast<unsigned>((groups + 15) / 16)), dim3(256), 0,
                     as_stream(stream), x, ld_x, R, C, q, ld_q, scale, act_dtype == KMOE_DT_F16 ? 1 : 0);
  return check_launch("kmoe_quant_fp8_group128");
}

// ---------------------------------------- asymmetric-activation epilogue on int32 accumulators
// one thread: 4 consecutive channels of one row
__global__ __launch_bounds__(256) void scaled_mm_azp_kernel(const int32_t* __restrict__ acc, int64_t ld_acc, int M, int n,
                                                           const float* __restrict__ scale_a, int sa_rows,
                                                           const float* __restrict__ scale_b, int sb_cols,
                                                           const int32_t* __restrict__ azp_adj,
                                                           const int32_t* __restrict__ azp, const float* __restrict__ bias,
                                                           uint16_t* __restrict__ out, int64_t ld_out, int f16) {
  const int quads = n / 4;
  const long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<long long>(M) * quads) return;
  const int r = static_cast<int>(idx / quads), c = static_cast<int>(idx % quads) * 4;
  const int4 a = *reinterpret_cast<const int4*>(acc + static_cast<size_t>(r) * ld_acc + c);
  const int4 adj = azp_adj ? *reinterpret_cast<const int4*>(azp_adj + c) : make_int4(0, 0, 0, 0);
  const uint32_t z = azp ? static_cast<uint32_t>(azp[r]) : 1u;  // (products and differences wrap like int32 arithmetic)
  const float sa = scale_a[sa_rows ? r : 0];
  const int av[4] = {a.x, a.y, a.z, a.w}, dv[4] = {adj.x, adj.y, adj.z, adj.w};
  uint16_t o[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int t = static_cast<int>(static_cast<uint32_t>(av[q]) - z * static_cast<uint32_t>(dv[q]));
    const float sb = scale_b[sb_cols ? c + q : 0];
    // (no zero point: the operands are maxes, as the int8 GEMM takes them, and meet the sum in its order)
    float v = azp_adj ? sa * (sb * static_cast<float>(t)) : (static_cast<float>(t) * (sa / 127.0f)) * (sb / 127.0f);
    if (bias) v = v + bias[c + q];
    o[q] = f32_to_act(v, f16 != 0);
  }
  *reinterpret_cast<uint2*>(out + static_cast<size_t>(r) * ld_out + c) =
      make_uint2(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16));
}

extern "C" int kmoe_scaled_mm_azp_epilogue(const int32_t* acc, int64_t ld_acc, int M, int n, const float* scale_a,
                                           int scale_a_rows, const float* scale_b, int scale_b_cols,
                                           const int32_t* azp_adj, const int32_t* azp, const float* bias, uint16_t* out,
                                           int64_t ld_out, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "scaled_mm_azp_epilogue")) return rc;
  KMOE_REQUIRE(acc && scale_a && scale_b && out && (azp_adj || !azp), KMOE_ERR_NULL, "scaled_mm_azp_epilogue: NULL pointer");
  KMOE_REQUIRE(M >= 0 && n >= 4 && n % 4 == 0 && ld_acc >= n && ld_acc % 4 == 0 && ld_out >= n && ld_out % 4 == 0,
               KMOE_ERR_SHAPE, "scaled_mm_azp_epilogue: M=%d n=%d strides %lld/%lld (need n %% 4 == 0)", M, n,
               (long long)ld_acc, (long long)ld_out);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(acc) & 15) == 0 && (reinterpret_cast<uintptr_t>(azp_adj) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) & 7) == 0,
               KMOE_ERR_SHAPE, "scaled_mm_azp_epilogue: misaligned tensor pointer");
  if (M == 0) return KMOE_OK;
  const long long total = static_cast<long long>(M) * (n / 4);
  hipLaunchKernelGGL(scaled_mm_azp_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                     acc, ld_acc, M, n, scale_a, scale_a_rows, scale_b, scale_b_cols, azp_adj, azp, bias, out, ld_out,
                     act_dtype == KMOE_DT_F16 ? 1 : 0);
  return check_launch("kmoe_scaled_mm_azp_epilogue");
}

extern "C" int kmoe_quant_i8_static(const uint16_t* x, int64_t ld_x, int R, int C, const float* scale,
                                    const int32_t* azp, int8_t* q, int64_t ld_q, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "quant_i8_static")) return rc;
  KMOE_REQUIRE(x && scale && q, KMOE_ERR_NULL, "quant_i8_static: NULL pointer");
  KMOE_REQUIRE(R >= 0 && C >= 8 && C % 8 == 0 && C <= 65536, KMOE_ERR_SHAPE, "quant_i8_static: R=%d C=%d (need C %% 8 == 0)", R, C);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_x >= C && ld_q % 8 == 0 && ld_q >= C, KMOE_ERR_SHAPE,
               "quant_i8_static: row strides %lld/%lld", (long long)ld_x, (long long)ld_q);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0, KMOE_ERR_SHAPE,
               "quant_i8_static: misaligned tensor pointer");
  if (R == 0) return KMOE_OK;
  const long long n = static_cast<long long>(R) * (C / 8);
  hipLaunchKernelGGL(quant_i8_static_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), x, ld_x, R, C, scale, azp, q, ld_q, act_dtype == KMOE_DT_F16 ? 1 : 0);
  return check_launch("kmoe_quant_i8_static");
}

extern "C" int kmoe_quant_i8_rows_azp(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                                      float* row_scale, int32_t* row_azp, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "quant_i8_rows_azp")) return rc;
  KMOE_REQUIRE(x && q && row_scale && row_azp, KMOE_ERR_NULL, "quant_i8_rows_azp: NULL pointer");
  KMOE_REQUIRE(R >= 0 && C >= 1 && C <= 65536 && ld_x >= C && ld_q >= C, KMOE_ERR_SHAPE,
               "quant_i8_rows_azp: R=%d C=%d strides %lld/%lld", R, C, (long long)ld_x, (long long)ld_q);
  if (R == 0) return KMOE_OK;
  hipLaunchKernelGGL(quant_i8_rows_azp_kernel, dim3(R), dim3(256), 0, as_stream(stream), x, ld_x, C, q, ld_q, row_scale,
                     row_azp, act_dtype == KMOE_DT_F16 ? 1 : 0);
  return check_launch("kmoe_quant_i8_rows_azp");
}

extern "C" int kmoe_dequant_w4_bf16(const uint8_t* packed, const uint16_t* scale, int64_t rows, int k, int group_size,
                                    uint16_t* out, kmoe_stream_t stream) {
  return kmoe_dequant_w4(packed, scale, rows, k, group_size, out, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_dequant_w4(const uint8_t* packed, const uint16_t* scale, int64_t rows, int k, int group_size,
                               uint16_t* out, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "dequant_w4")) return rc;
  KMOE_REQUIRE(packed && scale && out, KMOE_ERR_NULL, "dequant_w4_bf16: NULL pointer");
  KMOE_REQUIRE(rows >= 0 && k >= 16 && k % 16 == 0 && group_size >= 2 && group_size % 2 == 0 && k % group_size == 0,
               KMOE_ERR_SHAPE, "dequant_w4_bf16: rows=%lld k=%d group_size=%d", (long long)rows, k, group_size);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(packed) & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0,
               KMOE_ERR_SHAPE, "dequant_w4_bf16: misaligned tensor pointer");
  if (rows == 0) return KMOE_OK;
  const long long n = rows * (k / 16);
  hipLaunchKernelGGL(dequant_w4_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                     packed, scale, static_cast<long long>(rows), k, group_size, out, act_dtype == KMOE_DT_F16 ? 1 : 0);
  return check_launch("kmoe_dequant_w4_bf16");
}

extern "C" int kmoe_swigluoai_and_mul(const uint16_t* y, int64_t ld_y, int R, int I, float alpha, float limit,
                                      uint16_t* out, int64_t ld_out, kmoe_stream_t stream) {
  KMOE_REQUIRE(y && out, KMOE_ERR_NULL, "swigluoai_and_mul: NULL pointer");
  KMOE_REQUIRE(R >= 0 && I >= 4 && I % 4 == 0, KMOE_ERR_SHAPE, "swigluoai_and_mul: R=%d I=%d (need I %% 4 == 0)", R, I);
  KMOE_REQUIRE(ld_y % 8 == 0 && ld_out % 4 == 0 && ld_y >= 2 * I && ld_out >= I, KMOE_ERR_SHAPE,
               "swigluoai_and_mul: row strides %lld/%lld", (long long)ld_y, (long long)ld_out);
  if (R == 0) return KMOE_OK;
  const long long n = static_cast<long long>(R) * (I / 4);
  hipLaunchKernelGGL(swigluoai_and_mul_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), y, ld_y, R, I, alpha, limit, out, ld_out);
  return check_launch("kmoe_swigluoai_and_mul");
}

extern "C" int kmoe_silu_and_mul(const uint16_t* y, int64_t ld_y, int R, int I, uint16_t* out, int64_t ld_out,
                                 kmoe_stream_t stream) {
  return kmoe_silu_and_mul_dt(y, ld_y, R, I, out, ld_out, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_silu_and_mul_dt(const uint16_t* y, int64_t ld_y, int R, int I, uint16_t* out, int64_t ld_out,
                                    int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "silu_and_mul")) return rc;
  KMOE_REQUIRE(y && out, KMOE_ERR_NULL, "silu_and_mul: NULL pointer");
  KMOE_REQUIRE(R >= 0 && I >= 8 && I % 8 == 0, KMOE_ERR_SHAPE, "silu_and_mul: R=%d I=%d (need I %% 8 == 0)", R, I);
  KMOE_REQUIRE(ld_y % 8 == 0 && ld_out % 8 == 0 && ld_y >= 2 * I && ld_out >= I, KMOE_ERR_SHAPE,
               "silu_and_mul: row strides %lld/%lld", (long long)ld_y, (long long)ld_out);
  if (R == 0) return KMOE_OK;
  const long long n = static_cast<long long>(R) * (I / 8);
  hipLaunchKernelGGL(silu_and_mul_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                     as_stream(stream), y, ld_y, R, I, out, ld_out, act_dtype);
  return check_launch("kmoe_silu_and_mul");
}

extern "C" int kmoe_silu_table(float* table, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "silu_table")) return rc;
  KMOE_REQUIRE(table, KMOE_ERR_NULL, "silu_table: NULL pointer");
  hipLaunchKernelGGL(silu_table_kernel, dim3(65536 / 256), dim3(256), 0, as_stream(stream), table, act_dtype);
  return check_launch("kmoe_silu_table");
}

extern "C" int kmoe_combine(const uint16_t* x, int64_t ld_x, const int32_t* moe_index, const float* topk_w,
                            const float* dequant_scale, int M, int K, int H, float out_scale,
                            const uint16_t* addend, int64_t ld_addend, uint16_t* out, int64_t ld_out,
                            kmoe_stream_t stream) {
  return kmoe_combine_dt(x, ld_x, moe_index, topk_w, dequant_scale, M, K, H, out_scale, addend, ld_addend, 1.0f, out,
                         ld_out, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_combine_dt(const uint16_t* x, int64_t ld_x, const int32_t* moe_index, const float* topk_w,
                               const float* dequant_scale, int M, int K, int H, float out_scale,
                               const uint16_t* addend, int64_t ld_addend, float addend_scale, uint16_t* out,
                               int64_t ld_out, int act_dtype, kmoe_stream_t stream) {
  if (int rc = check_dtype(act_dtype, "combine")) return rc;
  KMOE_REQUIRE(x && moe_index && topk_w && out, KMOE_ERR_NULL, "combine: NULL pointer");
  KMOE_REQUIRE(M >= 0 && K >= 1 && K <= kMaxTopK && H >= 8 && H % 8 == 0, KMOE_ERR_SHAPE,
               "combine: M=%d K=%d H=%d (need 1 <= K <= 64, H %% 8 == 0)", M, K, H);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_out % 8 == 0 && ld_x >= H && ld_out >= H, KMOE_ERR_SHAPE,
               "combine: row strides %lld/%lld", (long long)ld_x, (long long)ld_out);
  KMOE_REQUIRE(!addend || (ld_addend % 8 == 0 && ld_addend >= H), KMOE_ERR_SHAPE, "combine: addend stride %lld",
               (long long)ld_addend);
  if (M == 0) return KMOE_OK;
  const int epilogue = (out_scale != 1.0f || addend) ? 1 : 0;
  hipLaunchKernelGGL(combine_kernel, dim3(M, ceil_div(H, 256 * 8)), dim3(256), 0, as_stream(stream), x, ld_x, moe_index, topk_w,
                     dequant_scale, K, H, out_scale, epilogue, addend, ld_addend, addend ? addend_scale : 1.0f, out, ld_out,
                     act_dtype);
  return check_launch("kmoe_combine");
}
