/*
 * moe_oracle.c — TEST INFRASTRUCTURE, not product code.
 *
 * A plain-C CPU restatement of the quantized fused-MoE computation that
 * baidu/vLLM-Kunlun drives through closed kernels, stage by stage in the order
 * of KunlunCompressedTensorsW8A8Int8MoEMethod.apply_monolithic
 * (vllm_kunlun/quantization/compressed_tensors/compressed_tensors_moe.py:122-291).
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * it; the product library never does.
 *
 * The reference's arithmetic lives in binary wheels (kunlun_ops 0.1.58,
 * xspeedgate_ops 1.1.0; docs/source/installation.md:131-137) that are not in
 * the reference tree, and the reference holds no test or golden vector for this
 * path: PARITY WITH THOSE KERNELS IS UNPINNED. What this file computes is fixed
 * by the call sites (shapes, dtypes, stage order, max-not-scale convention) and
 * by the mathematics; tests/test_oracle_*.py pin every function against closed
 * forms, exact integer arithmetic, brute force and independent torch /
 * transformers restatements.
 *
 * Where the reference leaves a bit-level choice open, this file fixes it once:
 *   - rounding is round-half-to-even everywhere (rintf under the default mode);
 *   - top-k order: score descending, ties to the lower expert id;
 *   - exp() is the fixed fma sequence orc_exp() below (< 2 ulp from libm), so a
 *     device kernel performing the same sequence yields the same bits (routing);
 *   - SiLU of a 16-bit gate value: orc_silu() below, or - under a GPU test - the
 *     device's own table of its 65536 values (see silu_act);
 *   - the softmax row sum adds 64 interleaved partial sums (element e goes to
 *     partial e % 64, in ascending e) with a balanced binary tree;
 *   - dequant is ((float)acc * (a_max/127)) * (w_max/127), left to right;
 *   - no operation is contracted into an fma unless written as fmaf.
 * Build with -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------ scalar pieces */

static inline float bf16_to_f32(uint16_t h) {
  union { uint32_t u; float f; } v;
  v.u = (uint32_t)h << 16;
  return v.f;
}

static inline uint16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  uint32_t u = v.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* IEEE half <-> f32, round to nearest even, overflow to infinity (what every IEEE conversion does) */
static inline float half_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const int ex = (h >> 10) & 0x1f;
  const uint32_t man = h & 0x3ffu;
  union { uint32_t u; float f; } v;
  if (ex == 0) {
    v.f = ldexpf((float)man, -24); /* zero and subnormals: man * 2^-24, exact */
    v.u |= sign;
    return v.f;
  }
  if (ex == 31) {
    v.u = sign | 0x7f800000u | (man << 13);
    return v.f;
  }
  v.u = sign | ((uint32_t)(ex - 15 + 127) << 23) | (man << 13);
  return v.f;
}

static inline uint16_t f32_to_half(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  const uint16_t sign = (uint16_t)((v.u >> 16) & 0x8000u);
  const uint32_t a = v.u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);             /* NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);            /* >= 65536 (and inf): infinity */
  if (a < 0x33000000u) return sign;                                   /* < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
  const int ex = (int)(a >> 23) - 127;                                /* unbiased exponent, -25 .. 15 */
  uint32_t man = (a & 0x7fffffu) | 0x800000u;                         /* 24-bit significand */
  const int shift = ex < -14 ? 13 + (-14 - ex) : 13;                  /* bits dropped (more for subnormal results) */
  const uint32_t kept = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t half_ulp = 1u << (shift - 1);
  uint32_t r = kept + ((rem > half_ulp || (rem == half_ulp && (kept & 1u))) ? 1u : 0u);
  /* normal: r has the implicit bit at position 10 (a carry moves into the exponent, which is right, also into
     infinity at the top); subnormal: r is the mantissa itself (a carry to 0x400 gives the smallest normal) */
  const uint32_t bits = ex < -14 ? r : ((uint32_t)(ex + 15 - 1) << 10) + r;
  return (uint16_t)(sign | bits);
}

/* Activation dtype of the int8 path: bf16 (0) or IEEE half (1) patterns in the 16-bit tensors. The reference
 * runs either (platforms/kunlun.py:350-364; its recipes use float16, ci/scripts/server/start_vllm.sh:26).
 * A switch for the whole library, set by the Python front end before each call. */
static int g_act_f16 = 0;
ORC_API void orc_set_act_dtype(int f16) { g_act_f16 = f16 != 0; }
ORC_API uint16_t orc_f32_to_half(float f) { return f32_to_half(f); }
ORC_API float orc_half_to_f32(uint16_t h) { return half_to_f32(h); }
static inline float act_to_f32(uint16_t h) { return g_act_f16 ? half_to_f32(h) : bf16_to_f32(h); }
static inline uint16_t f32_to_act(float f) { return g_act_f16 ? f32_to_half(f) : f32_to_bf16(f); }

ORC_API float orc_exp(float x) {
  x = fminf(fmaxf(x, -86.0f), 86.0f);
  const float n = rintf(x * 0x1.715476p+0f);
  float r = fmaf(n, -0x1.62e4p-1f, x);
  r = fmaf(n, -0x1.7f7d1cp-20f, r);
  float p = 0x1.a01a02p-13f;
  p = fmaf(p, r, 0x1.6c16c2p-10f);
  p = fmaf(p, r, 0x1.111112p-7f);
  p = fmaf(p, r, 0x1.555556p-5f);
  p = fmaf(p, r, 0x1.555556p-3f);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  return ldexpf(p, (int)n);
}

ORC_API float orc_sigmoid(float x) { return 1.0f / (1.0f + orc_exp(-x)); }
ORC_API float orc_silu(float x) { return x / (1.0f + orc_exp(-x)); }

/* SiLU as the layer applies it: to a gate value that has been rounded to the 16-bit activation type first (the
 * reference's silu_and_mul reads a 16-bit tensor, ops/_custom_ops.py:699-706). A function of 65536 arguments per
 * activation type, so its values can be handed over as a table: the device under test computes SiLU with its
 * hardware's exp2 and reciprocal approximations (within an ulp each, not correctly rounded - no CPU sequence has
 * their bits), and a GPU test installs the device's table (orc_set_silu_table) after holding it against libm.
 * Without a table (CPU-only tests, the golden fixtures) silu is orc_silu above. */
static float g_silu_table[2][65536];
static int g_silu_table_set[2] = {0, 0};
ORC_API void orc_set_silu_table(int f16, const float* table) {
  const int t = f16 != 0;
  g_silu_table_set[t] = table != 0;
  if (table) memcpy(g_silu_table[t], table, sizeof(g_silu_table[t]));
}
static inline float silu_act(uint16_t h) {
  return g_silu_table_set[g_act_f16] ? g_silu_table[g_act_f16][h] : orc_silu(act_to_f32(h));
}

/* K best of score[0..E) among eligible entries: score descending, ties to the
 * lower index. O(E*K) selection; out_ids in selection order. */
static void select_topk(const float* score, const uint8_t* eligible, int E, int K, int32_t* out_ids) {
  uint8_t* taken = (uint8_t*)calloc((size_t)E, 1);
  for (int k = 0; k < K; ++k) {
    int best = -1;
    for (int e = 0; e < E; ++e) {
      if (taken[e] || (eligible && !eligible[e])) continue;
      if (best < 0 || score[e] > score[best]) best = e;
    }
    out_ids[k] = best;
    if (best >= 0) taken[best] = 1;
  }
  free(taken);
}

/* ------------------------------------------------------------------ routing */

/* softmax -> top-K (-> renorm). Follows the call at compressed_tensors_moe.py:151-159
 * (logits already f32, normalised weights, int32 ids) and ops/_kunlun_ops.py:666-671. */
ORC_API void orc_softmax_topk(const float* logits, int M, int E, int K, int renorm, float* topk_w,
                              int32_t* topk_ids) {
  float* ex = (float*)malloc(sizeof(float) * (size_t)E);
  for (int m = 0; m < M; ++m) {
    const float* row = logits + (size_t)m * E;
    float mx = row[0];
    for (int e = 1; e < E; ++e) mx = fmaxf(mx, row[e]);
    float part[64];
    for (int l = 0; l < 64; ++l) part[l] = 0.0f;
    for (int e = 0; e < E; ++e) {
      ex[e] = orc_exp(row[e] - mx);
      part[e & 63] = part[e & 63] + ex[e];
    }
    for (int off = 32; off > 0; off >>= 1)
      for (int l = 0; l < off; ++l) part[l] = part[l] + part[l + off];
    const float total = part[0];
    int32_t* ids = topk_ids + (size_t)m * K;
    float* w = topk_w + (size_t)m * K;
    select_topk(row, NULL, E, K, ids); /* softmax is monotone: choose on the logits */
    for (int k = 0; k < K; ++k) w[k] = ex[ids[k]] / total;
    if (renorm) {
      float denom = 0.0f;
      for (int k = 0; k < K; ++k) denom = denom + w[k];
      for (int k = 0; k < K; ++k) w[k] = w[k] / denom;
    }
  }
  free(ex);
}

/* DeepSeek-V3 grouped top-k with correction bias. Follows the call at
 * compressed_tensors_moe.py:160-170 (args x, bias, n_group, topk_group, scale). */
ORC_API void orc_sigmoid_group_topk_norm(const float* logits, const float* bias, int M, int E, int K, int n_group,
                                         int topk_group, float scale, float* topk_w, int32_t* topk_ids) {
  float* s = (float*)malloc(sizeof(float) * (size_t)E);
  float* c = (float*)malloc(sizeof(float) * (size_t)E);
  uint8_t* ok = (uint8_t*)malloc((size_t)E);
  if (n_group < 1) n_group = 1;
  float* gscore = (float*)malloc(sizeof(float) * (size_t)n_group);
  int32_t* gsel = (int32_t*)malloc(sizeof(int32_t) * (size_t)n_group);
  const int gsize = E / n_group;
  for (int m = 0; m < M; ++m) {
    const float* row = logits + (size_t)m * E;
    for (int e = 0; e < E; ++e) {
      s[e] = orc_sigmoid(row[e]);
      c[e] = bias ? s[e] + bias[e] : s[e];
      ok[e] = 1;
    }
    if (n_group > 1) {
      for (int g = 0; g < n_group; ++g) {
        float t1 = -INFINITY, t2 = -INFINITY;
        for (int i = 0; i < gsize; ++i) {
          const float x = c[g * gsize + i];
          if (x > t1) {
            t2 = t1;
            t1 = x;
          } else if (x > t2) {
            t2 = x;
          }
        }
        gscore[g] = t1 + t2;
      }
      select_topk(gscore, NULL, n_group, topk_group, gsel);
      memset(ok, 0, (size_t)E);
      for (int t = 0; t < topk_group; ++t)
        for (int i = 0; i < gsize; ++i) ok[gsel[t] * gsize + i] = 1;
    }
    int32_t* ids = topk_ids + (size_t)m * K;
    float* w = topk_w + (size_t)m * K;
    select_topk(c, ok, E, K, ids);
    float denom = 0.0f;
    for (int k = 0; k < K; ++k) denom = denom + s[ids[k]];
    denom = denom + 1e-20f;
    for (int k = 0; k < K; ++k) w[k] = (s[ids[k]] / denom) * scale;
  }
  free(s);
  free(c);
  free(ok);
  free(gscore);
  free(gsel);
}

/* -------------------------------------------------------------------- align */

/* Stable counting sort by expert (moe_pre_sorted / moe_pre_small index outputs,
 * compressed_tensors_moe.py:172-207). ids outside [0,E) get moe_index -1. */
ORC_API void orc_align(const int32_t* ids, int P, int E, int32_t* moe_index, int32_t* sorted_src,
                       int32_t* expert_m, int32_t* lod) {
  int32_t* cnt = (int32_t*)calloc((size_t)E, sizeof(int32_t));
  for (int j = 0; j < P; ++j)
    if (ids[j] >= 0 && ids[j] < E) cnt[ids[j]]++;
  lod[0] = 0;
  for (int e = 0; e < E; ++e) lod[e + 1] = lod[e] + cnt[e];
  if (expert_m) memcpy(expert_m, cnt, sizeof(int32_t) * (size_t)E);
  memset(cnt, 0, sizeof(int32_t) * (size_t)E);
  for (int j = 0; j < P; ++j) {
    const int e = ids[j];
    if (e < 0 || e >= E) {
      moe_index[j] = -1;
      continue;
    }
    const int pos = lod[e] + cnt[e]++;
    moe_index[j] = pos;
    if (sorted_src) sorted_src[pos] = j;
  }
  free(cnt);
}

/* gen_block_statistic (compressed_tensors_moe.py:186): per-block histograms. */
ORC_API void orc_block_statistic(const int32_t* ids, int P, int E, int n_blocks, int32_t* out) {
  int per = (P + n_blocks - 1) / n_blocks;
  if (per < 1) per = 1;
  memset(out, 0, sizeof(int32_t) * (size_t)n_blocks * (size_t)E);
  for (int j = 0; j < P; ++j)
    if (ids[j] >= 0 && ids[j] < E) out[(size_t)(j / per) * E + ids[j]]++;
}

/* ------------------------------------------------------------------- quant */

/* quant2d (compressed_tensors_moe.py:224,253): per-row absmax int8; `max` out. */
ORC_API void orc_quant_i8_rows(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                               float* row_max) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < R; ++r) {
    const uint16_t* xr = x + (size_t)r * ld_x;
    float amax = 0.0f;
    for (int c = 0; c < C; ++c) amax = fmaxf(amax, fabsf(act_to_f32(xr[c])));
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    for (int c = 0; c < C; ++c) {
      float f = rintf(act_to_f32(xr[c]) * inv);
      f = fminf(fmaxf(f, -127.0f), 127.0f);
      q[(size_t)r * ld_q + c] = (int8_t)(int)f;
    }
    row_max[r] = amax;
  }
}

/* The other modes of scaled_int8_quant (ops/_custom_ops.py:1633-1657 forwards them to closed kernels; the
 * arithmetic restated here is the one of the vLLM operator of the same name, csrc/quantization/
 * compressed_tensors/int8_quant_kernels.cu): one scale (and zero point) for the tensor, or per row the
 * scale (max - min) / 255 and the zero point rint(-128 - min / scale). IEEE division, round half to even,
 * the zero point added in integers, saturation to [-128, 127]. A constant row takes scale 1 (the upstream
 * kernel divides by zero there). */
static int8_t sat8_ll(long long t) { return (int8_t)(t < -128 ? -128 : (t > 127 ? 127 : t)); }
static long long rint_clamped(float f) {
  f = rintf(f);
  if (!(f > -2147483000.0f)) f = -2147483000.0f; /* also NaN */
  if (f > 2147483000.0f) f = 2147483000.0f;
  return (long long)(int)f;
}
ORC_API void orc_quant_i8_static(const uint16_t* x, int64_t ld_x, int R, int C, float scale, int has_azp, int32_t azp,
                                 int8_t* q, int64_t ld_q) {
  for (int r = 0; r < R; ++r)
    for (int c = 0; c < C; ++c)
      q[(size_t)r * ld_q + c] = sat8_ll(rint_clamped(act_to_f32(x[(size_t)r * ld_x + c]) / scale) + (has_azp ? azp : 0));
}
ORC_API void orc_quant_i8_rows_azp(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                                   float* row_scale, int32_t* row_azp) {
  for (int r = 0; r < R; ++r) {
    const uint16_t* xr = x + (size_t)r * ld_x;
    float lo = INFINITY, hi = -INFINITY;
    for (int c = 0; c < C; ++c) {
      lo = fminf(lo, act_to_f32(xr[c]));
      hi = fmaxf(hi, act_to_f32(xr[c]));
    }
    float s = (hi - lo) / 255.0f;
    if (!(s > 0.0f)) s = 1.0f;
    const long long z = rint_clamped(-128.0f - lo / s);
    for (int c = 0; c < C; ++c) q[(size_t)r * ld_q + c] = sat8_ll(rint_clamped(act_to_f32(xr[c]) / s) + z);
    row_scale[r] = s;
    row_azp[r] = (int32_t)z;
  }
}

/* cutlass_scaled_mm_azp (ops/_custom_ops.py:1756-1771 forwards it to a closed kernel; restated from the vLLM
 * operator of that name, csrc/quantization/cutlass_w8a8): the int8 product in int32, the zero-point correction in
 * int32 (azp == NULL: it is folded into azp_adj), then scale_a * (scale_b * float(t)) + bias in f32, unfused.
 * a [M,k], w [n,k] int8; azp_adj [n]; scale_a: M values (per_row) or one; scale_b: n values (per_col) or one.
 * azp_adj == NULL: torch.ops._C.matmul with a bias (ops/_custom_ops.py:1811-1845) - the symmetric product. */
ORC_API void orc_scaled_mm_azp(const int8_t* a, const int8_t* w, int M, int n, int k, const float* scale_a, int per_row,
                               const float* scale_b, int per_col, const int32_t* azp_adj, const int32_t* azp,
                               const float* bias, uint16_t* out) {
  for (int r = 0; r < M; ++r)
    for (int c = 0; c < n; ++c) {
      int32_t acc = 0;
      for (int i = 0; i < k; ++i) acc += (int32_t)a[(size_t)r * k + i] * (int32_t)w[(size_t)c * k + i];
      const int32_t t = azp_adj ? (int32_t)((uint32_t)acc - (azp ? (uint32_t)azp[r] : 1u) * (uint32_t)azp_adj[c]) : acc;
      float v;
      if (azp_adj) { /* vLLM's epilogue */
        v = scale_b[per_col ? c : 0] * (float)t;
        v = scale_a[per_row ? r : 0] * v;
      } else { /* no zero point: the symmetric product, scales in the order of orc_grouped_gemm_i8 */
        v = (float)t * (scale_a[per_row ? r : 0] / 127.0f); /* the operands are maxes here */
        v = v * (scale_b[per_col ? c : 0] / 127.0f);
      }
      if (bias) v = v + bias[c];
      out[(size_t)r * n + c] = f32_to_act(v);
    }
}

/* OCP e4m3fn encoding by exhaustive nearest-value search (ties to even code). */
static float e4m3fn_value(int code) { /* code in [0,127), positive */
  const int ex = code >> 3, man = code & 7;
  return ex == 0 ? ldexpf((float)man, -9) : ldexpf(1.0f + (float)man / 8.0f, ex - 7);
}

ORC_API uint8_t orc_f32_to_e4m3fn(float f) {
  const uint8_t sign = signbit(f) ? 0x80 : 0;
  const float a = fabsf(f);
  if (!(a < 448.0f)) return (uint8_t)(sign | 0x7e);
  int best = 0;
  double bestd = fabs((double)a - 0.0);
  for (int code = 1; code <= 0x7e; ++code) {
    const double d = fabs((double)a - (double)e4m3fn_value(code));
    if (d < bestd || (d == bestd && (code & 1) == 0 && (best & 1) == 1)) {
      best = code;
      bestd = d;
    }
  }
  return (uint8_t)(sign | best);
}

ORC_API float orc_e4m3fn_to_f32(uint8_t b) {
  const float v = e4m3fn_value(b & 0x7f);
  return (b & 0x80) ? -v : v;
}

/* Per-row, per-128-column fp8 quantisation (no reference counterpart; DeepSeek-V3 recipe). */
ORC_API void orc_quant_fp8_group128(const uint16_t* x, int64_t ld_x, int R, int C, uint8_t* q, int64_t ld_q,
                                    float* scale) {
  const int G = C / 128;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < R; ++r) {
    for (int g = 0; g < G; ++g) {
      const uint16_t* xr = x + (size_t)r * ld_x + g * 128;
      float amax = 0.0f;
      for (int c = 0; c < 128; ++c) amax = fmaxf(amax, fabsf(act_to_f32(xr[c])));
      const float s = amax / 448.0f;
      for (int c = 0; c < 128; ++c)
        q[(size_t)r * ld_q + g * 128 + c] = orc_f32_to_e4m3fn(s > 0.0f ? act_to_f32(xr[c]) / s : 0.0f);
      scale[(size_t)r * G + g] = s;
    }
  }
}

/* -------------------------------------------------------------- grouped GEMM */

__attribute__((target_clones("arch=skylake-avx512", "avx2", "default"))) static int32_t dot_i8(const int8_t* a,
                                                                                    const int8_t* b, int k) {
  int32_t acc = 0;
  for (int i = 0; i < k; ++i) acc += (int32_t)a[i] * (int32_t)b[i];
  return acc;
}

/* moe_fc in its int8 form (compressed_tensors_moe.py:226-238, 263-275): rows
 * [lod[e], lod[e+1]) times weight[e]^T, exact int32, dequant by the two maxes.
 * act = 1 fuses silu_and_mul (ops/_custom_ops.py:699-706; gate = first half). */
ORC_API void orc_grouped_gemm_i8(const int8_t* a, int64_t lda, const float* a_max, const int32_t* row_src,
                                 int src_div, const int8_t* w, const float* w_max, const int32_t* lod, int E,
                                 int n, int k, uint16_t* y, int64_t ldy, int32_t* acc_out, int act) {
  for (int e = 0; e < E; ++e) {
    const int r0 = lod[e], r1 = lod[e + 1];
    const int8_t* we = w + (size_t)e * n * k;
    const float* wm = w_max + (size_t)e * n;
#pragma omp parallel for schedule(static)
    for (int r = r0; r < r1; ++r) {
      const int sr = row_src ? row_src[r] / src_div : r;
      const int8_t* ar = a + (size_t)sr * lda;
      const float sa = a_max[sr] / 127.0f;
      const int half = n / 2;
      if (act == 0) {
        for (int c = 0; c < n; ++c) {
          const int32_t acc = dot_i8(ar, we + (size_t)c * k, k);
          if (acc_out) acc_out[(size_t)r * n + c] = acc;
          if (y) y[(size_t)r * ldy + c] = f32_to_act(((float)acc * sa) * (wm[c] / 127.0f));
        }
      } else {
        for (int c = 0; c < half; ++c) {
          const int32_t ag = dot_i8(ar, we + (size_t)c * k, k);
          const int32_t au = dot_i8(ar, we + (size_t)(half + c) * k, k);
          if (acc_out) {
            acc_out[(size_t)r * n + c] = ag;
            acc_out[(size_t)r * n + half + c] = au;
          }
          const uint16_t yg = f32_to_act(((float)ag * sa) * (wm[c] / 127.0f));
          const uint16_t yu = f32_to_act(((float)au * sa) * (wm[half + c] / 127.0f));
          if (y) y[(size_t)r * ldy + c] = f32_to_act(silu_act(yg) * act_to_f32(yu));
        }
      }
    }
  }
}

/* Router logits in front of the layer: `router_logits, _ = self.gate(hidden_states)`
 * (models/deepseek_v2.py:178-184, 275), the bf16 x bf16 -> fp32 product of
 * ops/fused_moe/router/gate_linear.py:105-108. logits[m,e] = sum_k x[m,k] * w[e,k], every
 * product exact in double and the sum kept in double, rounded to f32 once: the value every
 * f32 summation order approximates. Comparisons with a device result are within the bound
 * (H * 2^-24) * sum_k |x[m,k] * w[e,k]|, which `abs_sum` (optional) returns. Parity unpinned
 * against the reference's closed/absent kernels; pinned against torch's f64 matmul. */
ORC_API void orc_router_gemm(const uint16_t* x, int64_t ld_x, const uint16_t* w, int M, int H, int E, float* logits,
                             float* abs_sum) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    for (int e = 0; e < E; ++e) {
      double s = 0.0, sa = 0.0;
      for (int k = 0; k < H; ++k) {
        const double p = (double)act_to_f32(x[(size_t)m * ld_x + k]) * (double)act_to_f32(w[(size_t)e * H + k]);
        s += p;
        sa += p < 0 ? -p : p;
      }
      logits[(size_t)m * E + e] = (float)s;
      if (abs_sum) abs_sum[(size_t)m * E + e] = (float)sa;
    }
  }
}

/* moe_fc with bf16 x and weight (ops/_kunlun_ops.py:578-585, 595-603, 615-622):
 * f32 accumulation in ascending k, one bf16 rounding. A device MFMA sums in its
 * own order, so comparisons with this function are within tolerance, not exact.
 * After orc_set_act_dtype(1) operands and result are IEEE half (the same method under
 * --dtype float16; products of two halves are exact in f32 as those of two bf16 are). */
ORC_API void orc_grouped_gemm_bf16(const uint16_t* a, int64_t lda, const int32_t* row_src, int src_div,
                                   const uint16_t* w, const int32_t* lod, int E, int n, int k, uint16_t* y,
                                   int64_t ldy, int act) {
  for (int e = 0; e < E; ++e) {
    const int r0 = lod[e], r1 = lod[e + 1];
    const uint16_t* we = w + (size_t)e * n * k;
#pragma omp parallel for schedule(static)
    for (int r = r0; r < r1; ++r) {
      const int sr = row_src ? row_src[r] / src_div : r;
      const uint16_t* ar = a + (size_t)sr * lda;
      const int half = n / 2;
      const int nout = act ? half : n;
      for (int c = 0; c < nout; ++c) {
        float g = 0.0f, u = 0.0f;
        const uint16_t* wg = we + (size_t)c * k;
        for (int i = 0; i < k; ++i) g += act_to_f32(ar[i]) * act_to_f32(wg[i]);
        if (act) {
          const uint16_t* wu = we + (size_t)(half + c) * k;
          for (int i = 0; i < k; ++i) u += act_to_f32(ar[i]) * act_to_f32(wu[i]);
          y[(size_t)r * ldy + c] =
              f32_to_act(silu_act(f32_to_act(g)) * act_to_f32(f32_to_act(u)));
        } else {
          y[(size_t)r * ldy + c] = f32_to_act(g);
        }
      }
    }
  }
}

/* 4-bit weight unpacking (dequant_int4_native, quantization/kernels/quant_ops.py:71-86): low nibble first,
 * code c means c - 8, times the scale of the element's (contiguous) group, one bf16 rounding - or, after
 * orc_set_act_dtype(1), one half rounding of half scales: the reference's (code.to(float16) - 8) * scale. */
ORC_API void orc_dequant_w4_bf16(const uint8_t* packed, const uint16_t* scale, int64_t rows, int k, int group_size,
                                 uint16_t* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int j = 0; j < k; ++j) {
      const uint8_t byte = packed[r * (k / 2) + j / 2];
      const int c = (j & 1) ? (byte >> 4) : (byte & 0xf);
      out[r * k + j] = f32_to_act((float)(c - 8) * act_to_f32(scale[r * (k / group_size) + j / group_size]));
    }
}

/* gpt-oss activation (swigluoai_and_mul, ops/_custom_ops.py:728-742): gate and up interleaved,
 * g = min(gate, limit), u = clamp(up, -limit, limit), out = (u + 1) * g * sigmoid(alpha * g), computed
 * in f32 from the bf16 inputs and rounded once (the reference rounds after each torch op; the
 * difference is inside the bf16 tolerance). */
static inline uint16_t swigluoai_bits(uint16_t gate, uint16_t up, float alpha, float limit) {
  const float g = fminf(bf16_to_f32(gate), limit);
  const float u = fminf(fmaxf(bf16_to_f32(up), -limit), limit);
  const float glu = g * orc_sigmoid(g * alpha);
  return f32_to_bf16((u + 1.0f) * glu);
}

ORC_API void orc_swigluoai_and_mul(const uint16_t* y, int64_t ld_y, int R, int I, float alpha, float limit,
                                   uint16_t* out, int64_t ld_out) {
  for (int r = 0; r < R; ++r)
    for (int i = 0; i < I; ++i)
      out[(size_t)r * ld_out + i] = swigluoai_bits(y[(size_t)r * ld_y + 2 * i], y[(size_t)r * ld_y + 2 * i + 1], alpha, limit);
}

/* The expert-bias branch of KunlunOps.fused_moe (ops/_kunlun_ops.py:433-468) as a grouped GEMM:
 * y = bf16(bf16(a . w^T) + bias[e]) (`gemm + bias` on bf16 tensors rounds twice), then, with
 * act == 2, the gpt-oss activation over interleaved columns (n/2 outputs). bias may be NULL. */
ORC_API void orc_grouped_gemm_bf16_bias(const uint16_t* a, int64_t lda, const int32_t* row_src, int src_div,
                                        const uint16_t* w, const uint16_t* bias, const int32_t* lod, int E, int n,
                                        int k, uint16_t* y, int64_t ldy, int act, float alpha, float limit) {
  for (int e = 0; e < E; ++e) {
    const int r0 = lod[e], r1 = lod[e + 1];
    const uint16_t* we = w + (size_t)e * n * k;
#pragma omp parallel for schedule(static)
    for (int r = r0; r < r1; ++r) {
      const int sr = row_src ? row_src[r] / src_div : r;
      const uint16_t* ar = a + (size_t)sr * lda;
      uint16_t prev = 0;
      for (int c = 0; c < n; ++c) {
        float s = 0.0f;
        const uint16_t* wc = we + (size_t)c * k;
        for (int i = 0; i < k; ++i) s += bf16_to_f32(ar[i]) * bf16_to_f32(wc[i]);
        uint16_t v = f32_to_bf16(s);
        if (bias) v = f32_to_bf16(bf16_to_f32(v) + bf16_to_f32(bias[(size_t)e * n + c]));
        if (act == 2) {
          if (c & 1) y[(size_t)r * ldy + c / 2] = swigluoai_bits(prev, v, alpha, limit);
          prev = v;
        } else {
          y[(size_t)r * ldy + c] = v;
        }
      }
    }
  }
}

/* fp8-e4m3fn block-scaled grouped GEMM (no reference counterpart; DeepSeek-V3 recipe):
 * per 128-wide K block the exact f32 sum of code products, times the activation
 * scale of (row, block) and the weight scale of (channel/128, block); blocks added in
 * ascending order; one bf16 rounding. Device MFMA order differs: tolerance, not exact. */
ORC_API void orc_grouped_gemm_fp8(const uint8_t* a, int64_t lda, const float* a_scale, const int32_t* row_src,
                                  int src_div, const uint8_t* w, const float* w_scale, const int32_t* lod, int E,
                                  int n, int k, uint16_t* y, int64_t ldy, int act) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = orc_e4m3fn_to_f32((uint8_t)i);
  const int kb_n = k / 128, nb_n = n / 128;
  for (int e = 0; e < E; ++e) {
    const int r0 = lod[e], r1 = lod[e + 1];
    const uint8_t* we = w + (size_t)e * n * k;
    const float* ws = w_scale + (size_t)e * nb_n * kb_n;
#pragma omp parallel for schedule(static)
    for (int r = r0; r < r1; ++r) {
      const int sr = row_src ? row_src[r] / src_div : r;
      const uint8_t* ar = a + (size_t)sr * lda;
      const float* as = a_scale + (size_t)sr * kb_n;
      const int half = n / 2;
      const int nout = act ? half : n;
      for (int c = 0; c < nout; ++c) {
        float tot[2] = {0.0f, 0.0f};
        for (int part = 0; part < (act ? 2 : 1); ++part) {
          const int cc = part ? half + c : c;
          const uint8_t* wr = we + (size_t)cc * k;
          float t = 0.0f;
          for (int kb = 0; kb < kb_n; ++kb) {
            float s = 0.0f;
            for (int i = 0; i < 128; ++i) s += lut[ar[kb * 128 + i]] * lut[wr[kb * 128 + i]];
            t = fmaf(s, as[kb] * ws[(size_t)(cc / 128) * kb_n + kb], t);
          }
          tot[part] = t;
        }
        if (act)
          y[(size_t)r * ldy + c] =
              f32_to_act(silu_act(f32_to_act(tot[0])) * act_to_f32(f32_to_act(tot[1])));
        else
          y[(size_t)r * ldy + c] = f32_to_act(tot[0]);
      }
    }
  }
}

/* silu_and_mul on a stored gate_up tensor (compressed_tensors_moe.py:240-243). */
ORC_API void orc_silu_and_mul(const uint16_t* y, int64_t ld_y, int R, int I, uint16_t* out, int64_t ld_out) {
  for (int r = 0; r < R; ++r)
    for (int i = 0; i < I; ++i)
      out[(size_t)r * ld_out + i] = f32_to_act(silu_act(y[(size_t)r * ld_y + i]) *
                                                 act_to_f32(y[(size_t)r * ld_y + I + i]));
}

/* moe_post (compressed_tensors_moe.py:278-290): weighted top-K sum, f32
 * weights, f32 accumulate over ascending k, one bf16 rounding; then the caller
 * epilogue of models/deepseek_v2.py:288-296 when requested. */
ORC_API void orc_combine(const uint16_t* x, int64_t ld_x, const int32_t* moe_index, const float* topk_w,
                         const float* dq, int M, int K, int H, float out_scale, const uint16_t* addend,
                         int64_t ld_addend, float addend_scale, uint16_t* out, int64_t ld_out) {
  const int epilogue = (out_scale != 1.0f) || addend;
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    for (int h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) {
        const size_t j = (size_t)m * K + k;
        const int r = moe_index[j];
        if (r < 0) continue;
        const float wt = dq ? topk_w[j] * dq[j] : topk_w[j];
        acc = fmaf(wt, act_to_f32(x[(size_t)r * ld_x + h]), acc);
      }
      uint16_t o = f32_to_act(acc);
      if (epilogue) {
        /* each step rounds to the activation dtype, as the caller's tensor operations do; the half form
           (models/deepseek_v2.py:286-292) scales the shared output instead of the routed sum */
        if (out_scale != 1.0f) o = f32_to_act(act_to_f32(o) * out_scale);
        if (addend) {
          uint16_t ad = addend[(size_t)m * ld_addend + h];
          if (addend_scale != 1.0f) ad = f32_to_act(act_to_f32(ad) * addend_scale);
          o = f32_to_act(act_to_f32(o) + act_to_f32(ad));
        }
      }
      out[(size_t)m * ld_out + h] = o;
    }
  }
}

/* ------------------------------------------------------------ whole layer */

/* apply_monolithic restated: the eight stages of compressed_tensors_moe.py:151-291
 * (+ shared expert per quantization/kernels/scale_mm.py:52-90 and the caller
 * epilogue models/deepseek_v2.py:288-296). Optional outputs expose the
 * intermediates the parity tests compare bit for bit. scoring: 0 softmax, 1 sigmoid. */
ORC_API void orc_forward_w8a8(int M, int H, int E, int K, int I, int scoring, int renorm, int n_group,
                              int topk_group, float routed_scale, const float* logits, const float* bias,
                              const uint16_t* x, const int8_t* w13, const float* w13_max, const int8_t* w2,
                              const float* w2_max, int I_shared, const int8_t* ws13, const float* ws13_max,
                              const int8_t* ws2, const float* ws2_max, float out_scale, float shared_scale,
                              uint16_t* out,
                              /* optional intermediates (NULL to skip) */
                              float* o_topk_w, int32_t* o_topk_ids, int32_t* o_moe_index, int32_t* o_lod,
                              int8_t* o_actq, float* o_actmax, uint16_t* o_down) {
  const int P = M * K;
  float* topk_w = (float*)malloc(sizeof(float) * (size_t)(P ? P : 1));
  int32_t* topk_ids = (int32_t*)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
  int32_t* moe_index = (int32_t*)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
  int32_t* sorted_src = (int32_t*)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
  int32_t* lod = (int32_t*)malloc(sizeof(int32_t) * (size_t)(E + 1));
  int8_t* xq = (int8_t*)malloc((size_t)M * H + 1);
  float* xmax = (float*)malloc(sizeof(float) * (size_t)(M ? M : 1));
  uint16_t* act = (uint16_t*)malloc(sizeof(uint16_t) * ((size_t)P * I + 1));
  int8_t* actq = (int8_t*)malloc((size_t)P * I + 1);
  float* actmax = (float*)malloc(sizeof(float) * (size_t)(P ? P : 1));
  uint16_t* down = (uint16_t*)malloc(sizeof(uint16_t) * ((size_t)P * H + 1));

  if (scoring == 0)
    orc_softmax_topk(logits, M, E, K, renorm, topk_w, topk_ids);
  else
    orc_sigmoid_group_topk_norm(logits, bias, M, E, K, n_group, topk_group, routed_scale, topk_w, topk_ids);
  orc_align(topk_ids, P, E, moe_index, sorted_src, NULL, lod);
  /* quant2d of the expanded rows == quant of each token row once */
  orc_quant_i8_rows(x, H, M, H, xq, H, xmax);
  orc_grouped_gemm_i8(xq, H, xmax, sorted_src, K, w13, w13_max, lod, E, 2 * I, H, act, I, NULL, 1);
  orc_quant_i8_rows(act, I, P, I, actq, I, actmax);
  orc_grouped_gemm_i8(actq, I, actmax, NULL, 1, w2, w2_max, lod, E, H, I, down, H, NULL, 0);

  uint16_t* sh_out = NULL;
  if (I_shared > 0) {
    const int Is = I_shared;
    const int32_t dlod[2] = {0, M};
    uint16_t* sact = (uint16_t*)malloc(sizeof(uint16_t) * ((size_t)M * Is + 1));
    int8_t* sq = (int8_t*)malloc((size_t)M * Is + 1);
    float* smax = (float*)malloc(sizeof(float) * (size_t)(M ? M : 1));
    sh_out = (uint16_t*)malloc(sizeof(uint16_t) * ((size_t)M * H + 1));
    orc_grouped_gemm_i8(xq, H, xmax, NULL, 1, ws13, ws13_max, dlod, 1, 2 * Is, H, sact, Is, NULL, 1);
    orc_quant_i8_rows(sact, Is, M, Is, sq, Is, smax);
    orc_grouped_gemm_i8(sq, Is, smax, NULL, 1, ws2, ws2_max, dlod, 1, H, Is, sh_out, H, NULL, 0);
    free(sact);
    free(sq);
    free(smax);
  }
  orc_combine(down, H, moe_index, topk_w, NULL, M, K, H, out_scale, sh_out, H, shared_scale, out, H);

  if (o_topk_w) memcpy(o_topk_w, topk_w, sizeof(float) * (size_t)P);
  if (o_topk_ids) memcpy(o_topk_ids, topk_ids, sizeof(int32_t) * (size_t)P);
  if (o_moe_index) memcpy(o_moe_index, moe_index, sizeof(int32_t) * (size_t)P);
  if (o_lod) memcpy(o_lod, lod, sizeof(int32_t) * (size_t)(E + 1));
  if (o_actq) memcpy(o_actq, actq, (size_t)P * I);
  if (o_actmax) memcpy(o_actmax, actmax, sizeof(float) * (size_t)P);
  if (o_down) memcpy(o_down, down, sizeof(uint16_t) * (size_t)P * H);
  free(topk_w);
  free(topk_ids);
  free(moe_index);
  free(sorted_src);
  free(lod);
  free(xq);
  free(xmax);
  free(act);
  free(actq);
  free(actmax);
  free(down);
  free(sh_out);
}
