// Routing kernels: softmax top-K and DeepSeek-V3 sigmoid grouped top-K.
// One wave64 per token; expert e of the row lives in lane e % 64, slot e / 64.
#include "kmoe_common.h"

namespace kmoe {
namespace {

constexpr int kMaxSlots = 16;  // E <= 1024
constexpr int kWavesPerBlock = 4;

// Picks the K best (score desc, expert id asc) entries of the row held as
// score[s] (expert lane + 64*s); lane k < K returns the k-th winner in my_id.
template <int SLOTS>
__device__ inline void select_topk(const float (&score)[SLOTS], const bool (&eligible)[SLOTS], int K,
                                   int lane, int& my_id) {
  uint64_t key[SLOTS];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) key[s] = eligible[s] ? arg_key(score[s], lane + kWave * s) : 0;
  my_id = -1;
  for (int k = 0; k < K; ++k) {
    uint64_t best = 0;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) best = key[s] > best ? key[s] : best;
    best = wave_max_u64(best);
    const int id = arg_key_index(best);
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
      if (id == lane + kWave * s) key[s] = 0;  // taken
    if (lane == k) my_id = id;
  }
}

template <int SLOTS>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void softmax_topk_kernel(
    const float* __restrict__ logits, int M, int E, int K, int renorm, float* __restrict__ topk_w,
    int32_t* __restrict__ topk_ids) {
  const int lane = lane_id();
  const int m = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (m >= M) return;
  const float* row = logits + static_cast<size_t>(m) * E;

  float v[SLOTS];
  bool ok[SLOTS];
  float mx = -__builtin_inff();
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int e = lane + kWave * s;
    ok[s] = e < E;
    v[s] = ok[s] ? row[e] : -__builtin_inff();
    mx = fmaxf(mx, v[s]);
  }
  mx = wave_max(mx);

  // exp and the row sum: per-lane running sum over slots, then the lane tree.
  float ex[SLOTS];
  float part = 0.0f;
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    ex[s] = ok[s] ? exp_fixed(v[s] - mx) : 0.0f;
    part = part + ex[s];
  }
  const float total = wave_sum_tree(part);

  int my_id;
  select_topk<SLOTS>(v, ok, K, lane, my_id);

  // Lane k owns winner k: fetch its exp from the owning lane/slot.
  float p = 0.0f;
  {
    const int want = my_id >= 0 ? my_id : 0;
    float got = 0.0f;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const float t = __shfl(ex[s], want & (kWave - 1), kWave);
      if ((want >> 6) == s) got = t;
    }
    if (lane < K) p = got / total;
  }
  if (renorm) {
    float denom = 0.0f;
    for (int k = 0; k < K; ++k) denom = denom + __shfl(p, k, kWave);  // k ascending
    p = p / denom;
  }
  if (lane < K) {
    topk_w[static_cast<size_t>(m) * K + lane] = p;
    topk_ids[static_cast<size_t>(m) * K + lane] = my_id;
  }
}

template <int SLOTS>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void sigmoid_group_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int M, int E, int K,
    int n_group, int topk_group, float scale, float* __restrict__ topk_w,
    int32_t* __restrict__ topk_ids) {
  extern __shared__ float choice_lds[];  // [kWavesPerBlock][E]
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int m = blockIdx.x * kWavesPerBlock + wave;
  if (m >= M) return;  // whole wave leaves together; no block-level sync below
  const float* row = logits + static_cast<size_t>(m) * E;
  float* choice = choice_lds + wave * E;

  float sg[SLOTS];  // un-biased sigmoid
  float c[SLOTS];   // score used for choosing
  bool ok[SLOTS];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int e = lane + kWave * s;
    ok[s] = e < E;
    sg[s] = 0.0f;
    c[s] = -__builtin_inff();
    if (ok[s]) {
      sg[s] = sigmoid_fixed(row[e]);
      c[s] = bias ? sg[s] + bias[e] : sg[s];
      choice[e] = c[s];
    }
  }

  if (n_group > 1) {
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
    const int gsize = E / n_group;
    // lane g < n_group: sum of the two largest scores of group g
    float gscore = -__builtin_inff();
    if (lane < n_group) {
      float t1 = -__builtin_inff(), t2 = -__builtin_inff();
      const float* gp = choice + lane * gsize;
      for (int i = 0; i < gsize; ++i) {
        const float x = gp[i];
        if (x > t1) {
          t2 = t1;
          t1 = x;
        } else if (x > t2) {
          t2 = x;
        }
      }
      gscore = t1 + t2;
    }
    uint64_t keep = 0;
    uint64_t gkey = lane < n_group ? arg_key(gscore, lane) : 0;
    for (int t = 0; t < topk_group; ++t) {
      const int bi = arg_key_index(wave_max_u64(gkey));
      if (bi == lane) gkey = 0;
      keep |= static_cast<uint64_t>(1) << (bi & 63);
    }
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const int e = lane + kWave * s;
      if (ok[s]) ok[s] = (keep >> (e / gsize)) & 1u;
    }
  }

  int my_id;
  select_topk<SLOTS>(c, ok, K, lane, my_id);

  float p = 0.0f;
  {
    const int want = my_id >= 0 ? my_id : 0;
    float got = 0.0f;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const float t = __shfl(sg[s], want & (kWave - 1), kWave);
      if ((want >> 6) == s) got = t;
    }
    if (lane < K) p = got;
  }
  float denom = 0.0f;
  for (int k = 0; k < K; ++k) denom = denom + __shfl(p, k, kWave);  // k ascending
  denom = denom + 1e-20f;
  p = (p / denom) * scale;
  if (lane < K) {
    topk_w[static_cast<size_t>(m) * K + lane] = p;
    topk_ids[static_cast<size_t>(m) * K + lane] = my_id;
  }
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
