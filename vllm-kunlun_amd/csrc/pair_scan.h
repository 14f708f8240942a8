// The stable sort of the routed pairs by expert, done by the workgroups of the launch that consumes it.
//
// A decode-sized layer has a few KB of expert ids (one per routed pair). A workgroup that serves expert e reads
// them all itself - a quarter per wave, kScanBatch loads in flight per lane - counts the ids below e (the first
// sorted row of e) and lists the pairs that chose e, in order (the rows of e): what lod and row_src of the sort's
// launch would have told it, after one memory round trip instead of two dependent ones, and that launch is gone.
// The workgroup the caller names also writes the sort's outputs for the launches that follow.
#pragma once
#include "kmoe_common.h"

namespace kmoe {

constexpr int kScanWaves = 4;  // waves of the workgroups that scan
constexpr int kScanBatch = 4;  // expert ids a lane asks for before it waits (a workgroup: one round trip per 1024 pairs)

struct PairScanLds {
  int list[kScanWaves][kStreamScanMaxRows];  // per quarter of the ids: the pairs of the expert, ascending
  int cnt[kScanWaves], below[kScanWaves];
};

// The rows of one expert as scan_pairs found them: sorted rows [begin, end); the pair behind row begin + i.
struct ListedRows {
  int begin, end;
  int c0, c1, c2;  // lengths of the first three quarters' lists
  __device__ int pair(const PairScanLds& s, int i) const {
    int w = 0;
    if (i >= c0) {
      i -= c0;
      w = 1;
      if (i >= c1) {
        i -= c1;
        w = 2;
        if (i >= c2) {
          i -= c2;
          w = 3;
        }
      }
    }
    return s.list[w][i];
  }
};

// Called by all kScanWaves waves of the workgroup (one barrier inside). `publish`: this workgroup writes lod[e],
// expert_m[e], (for the last expert) lod[E], and moe_index / sorted_src of the expert's pairs.
__device__ inline ListedRows scan_pairs(const StreamScan& sc, int e, int E, PairScanLds& s, bool publish) {
  const int lane = lane_id();
  const int wave_id = threadIdx.x >> 6;
  const int quarter = (sc.n_pairs + kScanWaves * kWave - 1) / (kScanWaves * kWave) * kWave;
  const int q_begin = wave_id * quarter;
  const int q_end = min(sc.n_pairs, q_begin + quarter);
  int below = 0, cnt = 0;  // ids below e; pairs of e so far (wave-uniform)
  for (int base = q_begin; base < q_end; base += kScanBatch * kWave) {
    int id[kScanBatch];
#pragma unroll
    for (int u = 0; u < kScanBatch; ++u) {
      const int j = base + u * kWave + lane;
      id[u] = j < q_end ? sc.ids[j] : 0x7fffffff;
    }
    // (every workgroup of the launch walks all the ids: scalar work wherever it can be, and the listing only for
    // the few groups of 64 ids that hold a pair of this expert)
#pragma unroll
    for (int u = 0; u < kScanBatch; ++u) {
      if (base + u * kWave >= q_end) break;  // wave-uniform
      const bool mine = id[u] == e;
      const uint64_t mb = __ballot(mine);
      if (mb != 0) {
        const int at = cnt + __builtin_popcountll(mb & lanemask_lt());
        if (mine && at < kStreamScanMaxRows) s.list[wave_id][at] = base + u * kWave + lane;
        cnt += __builtin_popcountll(mb);
      }
      below += __builtin_popcountll(__ballot(id[u] < e));
    }
  }
  if (lane == 0) {
    s.cnt[wave_id] = min(cnt, kStreamScanMaxRows);  // (a token picks an expert once: never more rows than tokens)
    s.below[wave_id] = below;
  }
  __syncthreads();
  ListedRows r;
  r.c0 = s.cnt[0];
  r.c1 = s.cnt[1];
  r.c2 = s.cnt[2];
  cnt = min(r.c0 + r.c1 + r.c2 + s.cnt[3], kStreamScanMaxRows);
  r.begin = s.below[0] + s.below[1] + s.below[2] + s.below[3];
  r.end = r.begin + cnt;
  if (publish && wave_id == 0) {
    if (lane == 0) {
      sc.lod[e] = r.begin;
      sc.expert_m[e] = cnt;
      if (e == E - 1) sc.lod[E] = r.end;
    }
    for (int i = lane; i < cnt; i += kWave) {
      const int j = r.pair(s, i);
      sc.moe_index[j] = r.begin + i;
      sc.sorted_src[r.begin + i] = j;
    }
  }
  return r;
}

}  // namespace kmoe
