// Router GEMM: logits[M,E] (f32) = x[M,H] (bf16) . w_gate[E,H]^T (bf16), f32 accumulation on
// v_mfma_f32_16x16x32_bf16 — the step in front of the routing kernels.
//
// The matrix is small (E <= 1024 rows) and, for decode, so is M: the launch is
// latency-bound, so K is split over workgroups until the grid fills the chip. Each
// split writes its own plane of partial logits; the planes are summed in plane order
// (a fixed order: results do not depend on scheduling) either by a small reduction
// kernel or, inside the fused layer, by the routing kernel as it loads the logits.
// No LDS: a wave owns 64 experts x (16*MF) tokens and reads both operands as MFMA
// fragments straight from L2.
#include "kmoe_common.h"

namespace kmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWavesR = 4;

// MF: 16-token fragments per wave, NF: 16-expert fragments per wave, D: MFMA steps of loads in flight.
// <1,1,8> for small M (many small workgroups, deep prefetch: the launch is latency-bound),
// <4,4,2> for large M (16 MFMAs per 8 fragment loads).
// F16: both operands are IEEE half (v_mfma_f32_16x16x32_f16) instead of bf16.
template <int MF, int NF, int D, bool F16>
__global__ __launch_bounds__(kWavesR* kWave) void router_gemm_kernel(
    const uint16_t* __restrict__ x, int64_t ld_x, const uint16_t* __restrict__ w, int M, int H, int E,
    float* __restrict__ planes, size_t plane_stride, int64_t ld_out, int steps_per_split) {
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;
  const int t0 = blockIdx.x * 16 * MF;
  const int e0 = (blockIdx.y * kWavesR + wave) * NF * 16;
  if (e0 >= E) return;  // whole wave; no barriers in this kernel
  const int ksteps = H / 32;
  const int s_begin = blockIdx.z * steps_per_split;
  const int s_end = min(ksteps, s_begin + steps_per_split);

  // rows past the ends read row 0 (valid memory); their results are never stored
  const uint16_t* wp[NF];
  const uint16_t* xp[MF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int e = e0 + f * 16 + li;
    wp[f] = w + static_cast<size_t>(e < E ? e : 0) * H + lg * 8;
  }
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) {
    const int t = t0 + mf * 16 + li;
    xp[mf] = x + static_cast<size_t>(t < M ? t : 0) * ld_x + lg * 8;
  }
  v4f acc[MF][NF];
#pragma unroll
  for (int mf = 0; mf < MF; ++mf)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[mf][f] = (v4f){0.f, 0.f, 0.f, 0.f};

  v4i wf[D][NF], xf[D][MF];
  auto load = [&](int slot, int s) {
    const int k = min(s, ksteps - 1) * 32;
#pragma unroll
    for (int f = 0; f < NF; ++f) wf[slot][f] = *reinterpret_cast<const v4i*>(wp[f] + k);
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) xf[slot][mf] = *reinterpret_cast<const v4i*>(xp[mf] + k);
  };
  auto fma_step = [&](int slot) {
#pragma unroll
    for (int mf = 0; mf < MF; ++mf)
#pragma unroll
      for (int f = 0; f < NF; ++f)
        if constexpr (F16)
          acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wf[slot][f]),
                                                              __builtin_bit_cast(v8h, xf[slot][mf]), acc[mf][f], 0, 0, 0);
        else
          acc[mf][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wf[slot][f]),
                                                               __builtin_bit_cast(v8bf, xf[slot][mf]), acc[mf][f], 0, 0, 0);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) load(d, s_begin + d);
  for (int s = s_begin; s < s_end; s += D) {  // D steps per trip; step s + D is requested as step s retires
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (s + d < s_end) fma_step(d);
      load(d, s + d + D);
    }
  }

  float* out = planes + blockIdx.z * plane_stride;
#pragma unroll
  for (int mf = 0; mf < MF; ++mf) {
    const int t = t0 + mf * 16 + li;
    if (t >= M) continue;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int e = e0 + f * 16 + lg * 4;
      float* o = out + static_cast<size_t>(t) * ld_out + e;
      if (e + 3 < E && (ld_out & 3) == 0) {
        *reinterpret_cast<v4f*>(o) = acc[mf][f];
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (e + q < E) o[q] = acc[mf][f][q];
      }
    }
  }
}

// logits[m,e] = planes[0][m,e] + planes[1][m,e] + ... in that order
__global__ void router_reduce_kernel(const float* planes, size_t plane_stride, int n_planes, int M, int E,
                                     float* logits, int64_t ld) {  // logits may be plane 0
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<size_t>(M) * E) return;
  const int m = static_cast<int>(i / E), e = static_cast<int>(i % E);
  float v = planes[i];
  for (int p = 1; p < n_planes; ++p) v = v + planes[i + p * plane_stride];
  logits[static_cast<size_t>(m) * ld + e] = v;
}

}  // namespace

// K splits and wave shape for a shape: enough workgroups to fill the chip, at least 4 MFMA
// steps per split, at most 8 planes (the routing kernel reads them all for every logit).
// mf_out: 16-token fragments per wave, 4 (with 4 expert fragments) for large M, else 1 (with 1).
void router_plan(int M, int H, int E, int* ks_out, int* mf_out) {
  const int mf = M >= 512 ? 4 : 1;
  const int nf = mf;
  const int tiles = ceil_div(M, 16 * mf) * ceil_div(E, kWavesR * nf * 16);
  const int ksteps = H / 32;
  int ks = ceil_div(512, max(tiles, 1));
  ks = max(1, min(ks, min(8, max(1, ksteps / 4))));
  *ks_out = ks;
  *mf_out = mf;
}

// Partial planes [ks][M][E] (row stride ld_out) into `planes`; ks == 1 gives the logits themselves.
int router_gemm_planes(const uint16_t* x, int64_t ld_x, const uint16_t* w, int M, int H, int E, float* planes,
                       size_t plane_stride, int64_t ld_out, int ks, int mf, hipStream_t s, bool f16) {
  const int ksteps = H / 32;
  const int steps_per_split = ceil_div(ksteps, ks);
  const int nf = mf;
  const dim3 grid(ceil_div(M, 16 * mf), ceil_div(E, kWavesR * nf * 16), ks);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kWavesR * kWave), 0, s, x, ld_x, w, M, H, E, planes, plane_stride, ld_out,
                       steps_per_split);
  };
  if (mf == 4) {
    if (f16) go(router_gemm_kernel<4, 4, 2, true>);
    else go(router_gemm_kernel<4, 4, 2, false>);
  } else {
    if (f16) go(router_gemm_kernel<1, 1, 8, true>);
    else go(router_gemm_kernel<1, 1, 8, false>);
  }
  return check_launch("kmoe_router_gemm_bf16");
}

int router_reduce(const float* planes, size_t plane_stride, int n_planes, int M, int E, float* out, int64_t ld_out,
                  hipStream_t s) {
  const size_t total = static_cast<size_t>(M) * E;
  hipLaunchKernelGGL(router_reduce_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s, planes,
                     plane_stride, n_planes, M, E, out, ld_out);
  return check_launch("kmoe_router_gemm_bf16 (reduce)");
}

}  // namespace kmoe

using namespace kmoe;

extern "C" size_t kmoe_router_gemm_workspace_bytes(int M, int H, int E) {
  if (M <= 0 || H < 32 || E <= 0) return 256;
  int ks, mf;
  router_plan(M, H, E, &ks, &mf);
  return ks <= 1 ? 256 : align_up(static_cast<size_t>(ks) * M * E * sizeof(float), 256);
}

extern "C" int kmoe_router_gemm_bf16(const uint16_t* x, int64_t ld_x, const uint16_t* w_gate, int M, int H, int E,
                                     float* logits, int64_t ld_logits, void* workspace, size_t workspace_bytes,
                                     kmoe_stream_t stream) {
  return kmoe_router_gemm(x, ld_x, w_gate, M, H, E, logits, ld_logits, workspace, workspace_bytes, KMOE_DT_BF16, stream);
}

extern "C" int kmoe_router_gemm(const uint16_t* x, int64_t ld_x, const uint16_t* w_gate, int M, int H, int E,
                                float* logits, int64_t ld_logits, void* workspace, size_t workspace_bytes,
                                int act_dtype, kmoe_stream_t stream) {
  KMOE_REQUIRE(act_dtype == KMOE_DT_BF16 || act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED,
               "router_gemm: act_dtype=%d unknown", act_dtype);
  const bool f16 = act_dtype == KMOE_DT_F16;
  KMOE_REQUIRE(x && w_gate && logits, KMOE_ERR_NULL, "router_gemm_bf16: NULL pointer");
  KMOE_REQUIRE(M >= 0 && E >= 1 && E <= 1024 && H >= 32 && H % 32 == 0, KMOE_ERR_SHAPE,
               "router_gemm_bf16: M=%d H=%d E=%d (need H %% 32 == 0, 1 <= E <= 1024)", M, H, E);
  KMOE_REQUIRE(ld_x % 8 == 0 && ld_x >= H && ld_logits >= E, KMOE_ERR_SHAPE,
               "router_gemm_bf16: row strides %lld/%lld", (long long)ld_x, (long long)ld_logits);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_gate) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(logits) & 15) == 0,
               KMOE_ERR_SHAPE, "router_gemm_bf16: tensors must be 16-byte aligned");
  if (M == 0) return KMOE_OK;
  int ks, mf;
  router_plan(M, H, E, &ks, &mf);
  hipStream_t s = as_stream(stream);
  if (ks == 1) return router_gemm_planes(x, ld_x, w_gate, M, H, E, logits, 0, ld_logits, 1, mf, s, f16);
  const size_t need = static_cast<size_t>(ks) * M * E * sizeof(float);
  KMOE_REQUIRE(workspace && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
               KMOE_ERR_WORKSPACE, "router_gemm_bf16: workspace of %zu bytes (16-byte aligned) needed, got %zu", need,
               workspace_bytes);
  float* planes = static_cast<float*>(workspace);
  const size_t stride = static_cast<size_t>(M) * E;
  if (int rc = router_gemm_planes(x, ld_x, w_gate, M, H, E, planes, stride, E, ks, mf, s, f16)) return rc;
  return router_reduce(planes, stride, ks, M, E, logits, ld_logits, s);
}
