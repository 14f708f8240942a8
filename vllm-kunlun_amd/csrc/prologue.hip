// Routing and the per-token int8 quantisation of the activations in ONE launch:
// the two are independent (both read only the layer's inputs), so the first
// workgroups route tokens while the rest quantise rows. Saves a launch and its
// drain on the decode path, where each of the two kernels runs for a few
// microseconds; at prefill sizes the latency-bound routing waves run under the
// bandwidth-bound quantisation.
#include "quant_body.h"
#include "routing_body.h"

namespace kmoe {
namespace {

struct RouteArgs {
  const float* logits;  // [planes][M][E]; the logit is the sum over planes, plane 0 first
  int planes;
  size_t plane_stride;
  const float* bias;
  int M, E, K, renorm, n_group, topk_group;
  float scale;
  float* topk_w;
  int32_t* topk_ids;
};
struct QuantArgs {
  const uint16_t* x;
  int64_t ld_x;
  int R, C;
  int8_t* q;
  int64_t ld_q;
  float* row_max;
  int chunked;
  int f16;
};

template <int SLOTS, bool SIGMOID, int TPR, int NV>
__global__ __launch_bounds__(256) void route_quant_kernel(const RouteArgs r, const QuantArgs q, int routing_blocks) {
  extern __shared__ float choice_lds[];  // sigmoid routing: [kWavesPerBlock][E]
  if (static_cast<int>(blockIdx.x) < routing_blocks) {
    if (SIGMOID)
      sigmoid_group_topk_body<SLOTS>(r.logits, r.planes, r.plane_stride, r.bias, r.M, r.E, r.K, r.n_group, r.topk_group, r.scale, r.topk_w,
                                     r.topk_ids, choice_lds, blockIdx.x);
    else
      softmax_topk_body<SLOTS>(r.logits, r.planes, r.plane_stride, r.M, r.E, r.K, r.renorm, r.topk_w, r.topk_ids, blockIdx.x);
  } else {
    quant_i8_rows_body<TPR, NV>(q.x, q.ld_x, q.R, q.C, q.q, q.ld_q, q.row_max, q.chunked,
                                static_cast<int>(blockIdx.x) - routing_blocks, q.f16 != 0);
  }
}

template <int SLOTS, bool SIGMOID, int TPR, int NV>
void launch(const RouteArgs& r, const QuantArgs& q, hipStream_t s) {
  const int routing_blocks = ceil_div(r.M, kWavesPerBlock);
  const int quant_blocks = ceil_div(q.R, 256 / TPR);
  const size_t lds = SIGMOID ? sizeof(float) * kWavesPerBlock * r.E : 0;
  hipLaunchKernelGGL((route_quant_kernel<SLOTS, SIGMOID, TPR, NV>), dim3(routing_blocks + quant_blocks), dim3(256), lds,
                     s, r, q, routing_blocks);
}

template <int SLOTS, bool SIGMOID>
void launch_q(const RouteArgs& r, const QuantArgs& q, hipStream_t s) {
  if (q.C <= 64 * 8 * 4)
    launch<SLOTS, SIGMOID, 64, 4>(r, q, s);
  else
    launch<SLOTS, SIGMOID, 256, 4>(r, q, s);
}

}  // namespace

// Returns KMOE_OK after a launch, a negative code on a launch error, or 1 when the
// arguments are outside what the fused kernel is instantiated for (nothing launched:
// the caller runs the two stand-alone entry points, which also report bad arguments).
int fused_route_quant_i8(const float* logits, int planes, size_t plane_stride, const float* bias, int M, int E, int K, int sigmoid, int renorm,
                         int n_group, int topk_group, float scale, float* topk_w, int32_t* topk_ids,
                         const uint16_t* x, int H, int8_t* xq, float* xmax, int chunked, int f16, hipStream_t s) {
  if (M <= 0 || E < 1 || E > 512 || K < 1 || K > E || K > kWave) return 1;
  if (H < 16 || H % 16 || H > 256 * 8 * 4) return 1;
  if (sigmoid) {
    if (n_group <= 1) {
      n_group = 1;
      topk_group = 1;
    } else if (n_group > kWave || E % n_group || E / n_group < 2 || topk_group < 1 || topk_group > n_group ||
               K > topk_group * (E / n_group)) {
      return 1;
    }
  }
  const RouteArgs r{logits, planes, plane_stride, bias, M, E, K, renorm, n_group, topk_group, scale, topk_w, topk_ids};
  const QuantArgs q{x, H, M, H, xq, chunked ? 0 : H, xmax, chunked, f16};
  const int slots = ceil_div(E, kWave);
  if (sigmoid) {
    if (slots <= 2) launch_q<2, true>(r, q, s);
    else if (slots <= 4) launch_q<4, true>(r, q, s);
    else launch_q<8, true>(r, q, s);
  } else {
    if (slots <= 2) launch_q<2, false>(r, q, s);
    else if (slots <= 4) launch_q<4, false>(r, q, s);
    else launch_q<8, false>(r, q, s);
  }
  return check_launch("kmoe_moe_forward (routing + quantisation)");
}

}  // namespace kmoe
