// Per-row dynamic int8 quantisation as a device function, shared by the stand-alone
// kernel and the fused routing + quantisation launch.
#pragma once
#include "kmoe_common.h"

namespace kmoe {

union Pack8 {  // 8 bf16 (or half) values
  uint4 v;
  uint16_t h[8];
};

// ---------------------------------------------------------------- int8 rows
// TPR threads cooperate on one row (32: two rows per wave); each keeps NV vectors of 8 values in
// registers, so the row is read from memory once.
// Workgroup `block` (256 threads) serves rows block * (256 / TPR) ...
template <int TPR, int NV>
__device__ inline void quant_i8_rows_body(const uint16_t* __restrict__ x, int64_t ld_x, int R, int C,
                                          int8_t* __restrict__ q, int64_t ld_q, float* __restrict__ row_max,
                                          int chunked, int block, bool f16 = false) {
  constexpr int kRowsPerBlock = 256 / TPR;
  __shared__ float red[256 / kWave];
  const int sub = threadIdx.x / TPR;
  const int t = threadIdx.x % TPR;
  const int r = block * kRowsPerBlock + sub;
  const bool live = r < R;
  const int nvec = C / 8;
  Pack8 val[NV];
  float amax = 0.0f;
  if (live) {
    const uint4* src = reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * ld_x);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = t + i * TPR;
      if (v < nvec) {
        val[i].v = src[v];
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(act_to_f32(val[i].h[j], f16)));
      }
    }
  }
  amax = group_max<(TPR < kWave ? TPR : kWave)>(amax);
  if (TPR > kWave) {  // one row per block: combine the waves
    if (lane_id() == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = red[0];
#pragma unroll
    for (int w = 1; w < TPR / kWave; ++w) amax = fmaxf(amax, red[w]);
  }
  if (!live) return;
  const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
  // row-major: vector v of the row; chunk-major [C/64][R][64]: vector v is eighth v%8 of chunk v/8
  uint2* dst = reinterpret_cast<uint2*>(q + static_cast<size_t>(r) * (chunked ? 64 : ld_q));
  const size_t vstride = chunked ? static_cast<size_t>(R) : 0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = t + i * TPR;
    if (v < nvec) {
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float f = __builtin_rintf(act_to_f32(val[i].h[j], f16) * inv);
        f = fminf(fmaxf(f, -127.0f), 127.0f);
        const int qi = static_cast<int>(f);
        w[j >> 2] |= static_cast<uint32_t>(qi & 0xff) << (8 * (j & 3));
      }
      dst[chunked ? (v >> 3) * vstride * 8 + (v & 7) : v] = make_uint2(w[0], w[1]);
    }
  }
  if (t == 0) row_max[r] = amax;
}

}  // namespace kmoe
