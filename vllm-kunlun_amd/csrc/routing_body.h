// Routing as device functions (one wave per token; expert e of the row lives in
// lane e % 64, slot e / 64), shared by the stand-alone routing kernels and the
// fused routing + activation-quantisation launch.
#pragma once
#include "kmoe_common.h"

namespace kmoe {

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

// Logit of (token row, expert e): the sum, plane 0 first, of `planes` partial planes that lie
// `plane_stride` floats apart (what a split-K router GEMM leaves); planes == 1: the logit itself.
__device__ inline float load_logit(const float* __restrict__ row, int e, int planes, size_t plane_stride) {
  float v = row[e];
  if (planes > 1) {  // at most 8 planes: request them all, then add in plane order
    float t[7];
#pragma unroll
    for (int p = 1; p < 8; ++p) t[p - 1] = p < planes ? row[e + p * plane_stride] : 0.0f;
#pragma unroll
    for (int p = 1; p < 8; ++p)
      if (p < planes) v = v + t[p - 1];
  }
  return v;
}

// One wave per token: workgroup `block` of kWavesPerBlock waves serves tokens
// block * kWavesPerBlock + wave.
template <int SLOTS>
__device__ inline void softmax_topk_body(const float* __restrict__ logits, int planes, size_t plane_stride, int M,
                                         int E, int K, int renorm, float* __restrict__ topk_w,
                                         int32_t* __restrict__ topk_ids, int block) {
  const int lane = lane_id();
  const int m = block * kWavesPerBlock + (threadIdx.x >> 6);
  if (m >= M) return;
  const float* row = logits + static_cast<size_t>(m) * E;

  float v[SLOTS];
  bool ok[SLOTS];
  float mx = -__builtin_inff();
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int e = lane + kWave * s;
    ok[s] = e < E;
    v[s] = ok[s] ? load_logit(row, e, planes, plane_stride) : -__builtin_inff();
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

// choice_lds: [kWavesPerBlock][E] floats of (dynamic) LDS.
template <int SLOTS>
__device__ inline void sigmoid_group_topk_body(const float* __restrict__ logits, int planes, size_t plane_stride,
                                               const float* __restrict__ bias, int M, int E, int K, int n_group,
                                               int topk_group, float scale,
                                               float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
                                               float* choice_lds, int block) {
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int m = block * kWavesPerBlock + wave;
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
      sg[s] = sigmoid_fixed(load_logit(row, e, planes, plane_stride));
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


}  // namespace kmoe
