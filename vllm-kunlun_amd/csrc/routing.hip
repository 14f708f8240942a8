// Routing kernels: softmax top-K and DeepSeek-V3 sigmoid grouped top-K.
// One wave64 per token; expert e of the row lives in lane e % 64, slot e / 64.
#include "routing_body.h"

namespace kmoe {
namespace {

template <int SLOTS>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void softmax_topk_kernel(
    const float* __restrict__ logits, int M, int E, int K, int renorm, float* __restrict__ topk_w,
    int32_t* __restrict__ topk_ids) {
  softmax_topk_body<SLOTS>(logits, 1, 0, M, E, K, renorm, topk_w, topk_ids, blockIdx.x);
}

template <int SLOTS>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void sigmoid_group_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int M, int E, int K,
    int n_group, int topk_group, float scale, float* __restrict__ topk_w,
    int32_t* __restrict__ topk_ids) {
  extern __shared__ float choice_lds[];  // [kWavesPerBlock][E]
  sigmoid_group_topk_body<SLOTS>(logits, 1, 0, bias, M, E, K, n_group, topk_group, scale, topk_w, topk_ids, choice_lds,
                                 blockIdx.x);
}

int check_common(const float* logits, int M, int E, int K, const float* w, const int32_t* ids) {
  KMOE_REQUIRE(logits && w && ids, KMOE_ERR_NULL, "routing: NULL pointer");
  KMOE_REQUIRE(M >= 0, KMOE_ERR_SHAPE, "routing: M=%d < 0", M);
  KMOE_REQUIRE(E >= 1 && E <= kMaxSlots * kWave, KMOE_ERR_SHAPE, "routing: E=%d outside [1,%d]", E,
               kMaxSlots * kWave);
  KMOE_REQUIRE(K >= 1 && K <= E && K <= kWave, KMOE_ERR_SHAPE, "routing: K=%d outside [1,min(E,64)]", K);
  return KMOE_OK;
}

}  // namespace
}  // namespace kmoe

using namespace kmoe;

#define KMOE_SLOT_DISPATCH(E, CALL) \
  do {                              \
    const int slots_ = ceil_div((E), kWave); \
    if (slots_ <= 1) { CALL(1); }   \
    else if (slots_ <= 2) { CALL(2); } \
    else if (slots_ <= 4) { CALL(4); } \
    else if (slots_ <= 8) { CALL(8); } \
    else { CALL(16); }              \
  } while (0)

extern "C" int kmoe_softmax_topk(const float* logits, int M, int E, int K, int renorm, float* topk_w,
                                 int32_t* topk_ids, kmoe_stream_t stream) {
  if (int rc = check_common(logits, M, E, K, topk_w, topk_ids)) return rc;
  if (M == 0) return KMOE_OK;
  const dim3 grid(ceil_div(M, kWavesPerBlock)), block(kWavesPerBlock * kWave);
#define CALL(S)                                                                         \
  hipLaunchKernelGGL(softmax_topk_kernel<S>, grid, block, 0, as_stream(stream), logits, M, E, K, \
                     renorm, topk_w, topk_ids)
  KMOE_SLOT_DISPATCH(E, CALL);
#undef CALL
  return check_launch("kmoe_softmax_topk");
}

extern "C" int kmoe_sigmoid_group_topk_norm(const float* logits, const float* bias, int M, int E, int K,
                                            int n_group, int topk_group, float scale, float* topk_w,
                                            int32_t* topk_ids, kmoe_stream_t stream) {
  if (int rc = check_common(logits, M, E, K, topk_w, topk_ids)) return rc;
  if (n_group <= 1) {
    n_group = 1;
    topk_group = 1;
  } else {
    KMOE_REQUIRE(n_group <= kWave, KMOE_ERR_SHAPE, "routing: n_group=%d > 64", n_group);
    KMOE_REQUIRE(E % n_group == 0, KMOE_ERR_SHAPE, "routing: E=%d not divisible by n_group=%d", E, n_group);
    KMOE_REQUIRE(E / n_group >= 2, KMOE_ERR_SHAPE, "routing: groups of %d experts; need >= 2", E / n_group);
    KMOE_REQUIRE(topk_group >= 1 && topk_group <= n_group, KMOE_ERR_SHAPE,
                 "routing: topk_group=%d outside [1,n_group=%d]", topk_group, n_group);
    KMOE_REQUIRE(K <= topk_group * (E / n_group), KMOE_ERR_SHAPE,
                 "routing: K=%d exceeds the %d experts of the kept groups", K, topk_group * (E / n_group));
  }
  if (M == 0) return KMOE_OK;
  const dim3 grid(ceil_div(M, kWavesPerBlock)), block(kWavesPerBlock * kWave);
  const size_t lds = sizeof(float) * kWavesPerBlock * E;
#define CALL(S)                                                                                  \
  hipLaunchKernelGGL(sigmoid_group_topk_kernel<S>, grid, block, lds, as_stream(stream), logits, bias, \
                     M, E, K, n_group, topk_group, scale, topk_w, topk_ids)
  KMOE_SLOT_DISPATCH(E, CALL);
#undef CALL
  return check_launch("kmoe_sigmoid_group_topk_norm");
}
