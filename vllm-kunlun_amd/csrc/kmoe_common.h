// Shared device/host helpers for libkmoe (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kmoe.h"

namespace kmoe {

// Rows a launch expects to be live: `rows` bounds the sorted rows (grids and buffers are sized by it), the hint of
// the argument blocks (0: none) says how many of them the caller expects to exist - an expert-parallel share
// sorts only the pairs routed to its own experts. Kernels are CHOSEN by it; every choice is correct for any count.
inline int expected_rows(int rows, int hint) { return hint > 0 && hint < rows ? hint : rows; }

constexpr int kWave = 64;

// ---- error plumbing (host) -------------------------------------------------
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
// The calling thread's record of launched GEMM kernels (kmoe_trace_kernels): a launcher notes the kernel it chose.
bool tracing_kernels();
void note_kernel(const char* fmt, ...);
// Writes {0, rows} to lod2: the row offsets of a dense (single-expert) GEMM.
int fill_dense_lod(int32_t* lod2, int rows, hipStream_t stream);
// Weight-streaming int8 GEMM (tiled weights, chunk-major activations); arguments already validated.
// With `scan` (the layer's routed gate_up launch at decode sizes) the launch sorts the routed pairs by expert
// itself: it reads the pairs' expert ids instead of lod / row_src (args->lod and args->row_src are ignored; the
// gather divisor is args->src_div) and leaves what the sort would have left: lod [E+1], expert_m [E],
// moe_index [n_pairs], sorted_src [n_pairs]. Every id must lie in [0, E).
struct StreamScan {
  const int32_t* ids;
  int32_t n_pairs;
  int32_t* lod;
  int32_t* expert_m;
  int32_t* moe_index;
  int32_t* sorted_src;
};
constexpr int kStreamScanMaxPairs = 4096;
constexpr int kStreamScanMaxRows = 512;  // tokens: no expert gets more rows than that
// With `quant` (the layer's down launch at decode sizes, k <= kStreamQuantMaxK) the launch quantises its rows
// itself: it reads them as bf16 / half values (act, row stride ld; args->act_dtype) instead of args->a / a_max and
// leaves codes (chunk-major [k/64][args->a_rows][64]) and row maxes where the quantiser's launch would have.
struct StreamQuant {
  const uint16_t* act;
  int64_t ld;
  int8_t* codes;
  float* amax;
};
constexpr int kStreamQuantMaxK = 1024;
int stream_gemm_i8(const kmoe_gemm_i8_args* args, hipStream_t stream, const StreamScan* scan = nullptr,
                   const StreamQuant* quant = nullptr);
// kmoe_grouped_gemm_i8 with the options above for the layer's own launches.
int grouped_gemm_i8_checked(const kmoe_gemm_i8_args* args, kmoe_stream_t stream, const StreamScan* scan,
                            const StreamQuant* quant = nullptr);
// kmoe_grouped_gemm_w4a16 with `scan` for the layer's routed gate_up launch where it runs on the streaming kernel
// (w4_gate_up_streams says whether a launch of these dimensions does).
int grouped_gemm_w4a16_checked(const kmoe_gemm_w4_args* args, kmoe_stream_t stream, const StreamScan* scan);
bool w4_gate_up_streams(int rows, int rows_hint, int E, int k);
// Persistent 128-row-tile GEMMs for many rows per expert (tiled weights, row-major activations);
// arguments already validated.
int tiled_gemm_i8(const kmoe_gemm_i8_args* args, hipStream_t stream);
int tiled_gemm_fp8(const kmoe_gemm_fp8_args* args, hipStream_t stream);
int tiled_gemm_bf16(const kmoe_gemm_bf16_args* args, hipStream_t stream);
// Routing + per-token int8 quantisation of x [M,H] in one launch. Returns 1 (nothing launched)
// when the arguments are outside its instantiations: the caller then uses the two entry points.
int fused_route_quant_i8(const float* logits, int planes, size_t plane_stride, const float* bias, int M, int E, int K, int sigmoid, int renorm,
                         int n_group, int topk_group, float scale, float* topk_w, int32_t* topk_ids,
                         const uint16_t* x, int H, int8_t* xq, float* xmax, int chunked, int f16, hipStream_t stream);

// Router GEMM pieces for the fused layer: the split (ks planes, mf*16 tokens per wave) chosen for
// a shape, and the launch that leaves the partial planes [ks][M][E] (ks == 1: the logits).
void router_plan(int M, int H, int E, int* ks_out, int* mf_out);
int router_gemm_planes(const uint16_t* x, int64_t ld_x, const uint16_t* w, int M, int H, int E, float* planes,
                       size_t plane_stride, int64_t ld_out, int ks, int mf, hipStream_t stream, bool f16 = false);
// out[m,e] = planes[0][m,e] + planes[1][m,e] + ... (that order); out may be plane 0 itself.
int router_reduce(const float* planes, size_t plane_stride, int n_planes, int M, int E, float* out, int64_t ld_out,
                  hipStream_t stream);

#define KMOE_REQUIRE(cond, code, ...) \
  do {                                \
    if (!(cond)) return ::kmoe::fail((code), __VA_ARGS__); \
  } while (0)

// ---- bf16 <-> f32, bit-exact round-to-nearest-even --------------------------
__host__ __device__ inline float bf16_to_f32(uint16_t h) {
  union { uint32_t u; float f; } v;
  v.u = static_cast<uint32_t>(h) << 16;
  return v.f;
}

__host__ __device__ inline uint16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  uint32_t u = v.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);  // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// Device-only: the gfx950 conversion instruction (v_cvt_pk_bf16_f32, round to nearest
// even) — same bits as f32_to_bf16 for every finite input, one instruction per pair.
typedef float kmoe_v2f __attribute__((ext_vector_type(2)));
typedef __bf16 kmoe_v2bf __attribute__((ext_vector_type(2)));
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((kmoe_v2f){lo, hi}, kmoe_v2bf));
}
__device__ inline uint16_t f32_to_bf16_hw(float f) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f)); }

// ---- activation dtype: bf16 or IEEE half, chosen per call (a wave-uniform flag) ----------
// Both are 16-bit patterns in uint16_t tensors. Conversions are round-to-nearest-even; a value
// beyond the half range becomes infinity, as in every IEEE conversion.
__device__ inline float half_to_f32(uint16_t h) { return static_cast<float>(__builtin_bit_cast(_Float16, h)); }
// (The empty asm keeps the f32 value as it is: without it the compiler folds a preceding f32 multiplication into
// a mixed-precision instruction that rounds the exact product to half ONCE, which differs from rounding it to
// f32 first - the sequence the result contract fixes - whenever the f32 rounding lands on a half tie.)
__device__ inline uint16_t f32_to_half(float f) {
  asm("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}
__device__ inline float act_to_f32(uint16_t h, bool f16) { return f16 ? half_to_f32(h) : bf16_to_f32(h); }
__device__ inline uint16_t f32_to_act(float f, bool f16) { return f16 ? f32_to_half(f) : f32_to_bf16(f); }
typedef _Float16 kmoe_v2h __attribute__((ext_vector_type(2)));
__device__ inline uint32_t pack2_half(float lo, float hi) {
  asm("" : "+v"(lo));
  asm("" : "+v"(hi));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((kmoe_v2f){lo, hi}, kmoe_v2h));
}

// ---- fixed-sequence transcendental -----------------------------------------
// exp(x) as one fixed sequence of IEEE single operations (mul, round-to-even,
// fma, exact power-of-two scaling), so that a CPU restatement performing the
// same sequence gives the same bits. Argument clamped to [-86, 86] so neither
// the result nor 1/(1+result) leaves the normal range. Error < 2 ulp.
__device__ inline float exp_fixed(float x) {
  x = fminf(fmaxf(x, -86.0f), 86.0f);
  const float n = __builtin_rintf(x * 0x1.715476p+0f);            // x * log2(e)
  float r = __builtin_fmaf(n, -0x1.62e4p-1f, x);                  // - n * ln2_hi
  r = __builtin_fmaf(n, -0x1.7f7d1cp-20f, r);                     // - n * ln2_lo
  float p = 0x1.a01a02p-13f;                                      // 1/5040
  p = __builtin_fmaf(p, r, 0x1.6c16c2p-10f);                      // 1/720
  p = __builtin_fmaf(p, r, 0x1.111112p-7f);                       // 1/120
  p = __builtin_fmaf(p, r, 0x1.555556p-5f);                       // 1/24
  p = __builtin_fmaf(p, r, 0x1.555556p-3f);                       // 1/6
  p = __builtin_fmaf(p, r, 0.5f);
  p = __builtin_fmaf(p, r, 1.0f);
  p = __builtin_fmaf(p, r, 1.0f);
  return __builtin_ldexpf(p, static_cast<int>(n));
}

__device__ inline float sigmoid_fixed(float x) { return 1.0f / (1.0f + exp_fixed(-x)); }

// ---- SiLU of the GEMM epilogues ----------------------------------------------
// silu(g) = g / (1 + e^-g) on the hardware's transcendental unit: v_exp_f32 (2^t) and v_rcp_f32, each within
// one ulp, five instructions in all - the fixed-sequence exp and an IEEE divide cost thirty and were a sixth of
// the prefill gate_up launch. The two instructions are not correctly rounded, so no CPU sequence gives their
// bits; but SiLU is only ever applied to a 16-BIT activation value (gate is rounded to bf16 / half first, as the
// reference's silu_and_mul reads a 16-bit tensor), i.e. to one of 65536 arguments per activation type:
// kmoe_silu_table writes this function's result for every one of them, which is how a checker follows it bit
// for bit. Every kernel calls THIS function, so a token's result does not depend on the kernel that computes it.
// Arguments below -87 count as -87 (1 + 2^t and its reciprocal stay in the normal range; the result there,
// -1.4e-36, is 0 for every purpose, also for g = -inf, which would otherwise give inf x 0).
__device__ inline float silu_hw(float g) {
  const float gc = fmaxf(g, -87.0f);
  const float d = 1.0f + __builtin_amdgcn_exp2f(gc * -0x1.715476p+0f);  // 1 + 2^(-g log2(e))
  return gc * __builtin_amdgcn_rcpf(d);
}
// gpt-oss activation on a (gate, up) pair of bf16 values, one rounding at the end:
// g = min(gate, limit), u = clamp(up, -limit, limit), out = (u + 1) * g * sigmoid(alpha * g)
// (reference: swigluoai_and_mul, ops/_custom_ops.py:728-742).
__device__ inline uint16_t swigluoai_bf16(uint16_t gate, uint16_t up, float alpha, float limit) {
  const float g = fminf(bf16_to_f32(gate), limit);
  const float u = fminf(fmaxf(bf16_to_f32(up), -limit), limit);
  const float glu = g * sigmoid_fixed(g * alpha);
  return f32_to_bf16((u + 1.0f) * glu);
}

// ---- wave64 helpers ---------------------------------------------------------
__device__ inline int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}
// max over aligned groups of G lanes (G a power of two up to 64)
template <int G>
__device__ inline float group_max(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Butterfly sum: every lane ends with the same bits (each step adds the same
// two numbers on both sides). Equivalent to the balanced binary tree
// t[l] = t[l] + t[l + off], off = 32,16,...,1, over the 64 lane values.
__device__ inline float wave_sum_tree(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = v + __shfl_xor(v, off, kWave);
  return v;
}

__device__ inline int wave_sum_int(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// (value, index) argmax with ties to the lower index; all lanes get the winner.
__device__ inline void wave_argmax(float& v, int& idx) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, kWave);
    const int oi = __shfl_xor(idx, off, kWave);
    if (ov > v || (ov == v && oi < idx)) {
      v = ov;
      idx = oi;
    }
  }
}

// ---- wave-wide arg-max on packed keys, over DPP (no LDS crossbar) ------------
// A float maps to an unsigned int with the same order (-0 counts as +0); the key
// is (ordered value << 32) | ~index, so the largest key is the largest value
// and, among equal values, the lowest index. Key 0 means "no candidate".
__device__ inline uint32_t ordered_bits(float v) {
  union { float f; uint32_t u; } b;
  b.f = v + 0.0f;
  return (b.u & 0x80000000u) ? ~b.u : (b.u | 0x80000000u);
}
__device__ inline uint64_t arg_key(float v, int idx) {
  return (static_cast<uint64_t>(ordered_bits(v)) << 32) | static_cast<uint32_t>(~static_cast<uint32_t>(idx));
}
__device__ inline int arg_key_index(uint64_t key) { return static_cast<int>(~static_cast<uint32_t>(key)); }

template <int CTRL, int ROW_MASK>
__device__ inline uint64_t dpp_max_step(uint64_t k) {
  const uint32_t lo = static_cast<uint32_t>(k), hi = static_cast<uint32_t>(k >> 32);
  const uint32_t olo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
  const uint32_t ohi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
  const uint64_t o = (static_cast<uint64_t>(ohi) << 32) | olo;
  return o > k ? o : k;
}
// Max of a 64-bit key over the 64 lanes; every lane gets the result.
__device__ inline uint64_t wave_max_u64(uint64_t k) {
  k = dpp_max_step<0xB1, 0xf>(k);   // quad_perm [1,0,3,2]
  k = dpp_max_step<0x4E, 0xf>(k);   // quad_perm [2,3,0,1]
  k = dpp_max_step<0x141, 0xf>(k);  // row_half_mirror
  k = dpp_max_step<0x140, 0xf>(k);  // row_mirror: every lane of a 16-lane row holds the row max
  k = dpp_max_step<0x142, 0xa>(k);  // row_bcast15 into rows 1 and 3
  k = dpp_max_step<0x143, 0xc>(k);  // row_bcast31 into rows 2 and 3: lane 63 holds the wave max
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(k), 63);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(k >> 32), 63);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

__device__ inline uint64_t lanemask_lt() {
  return (static_cast<uint64_t>(1) << lane_id()) - 1;
}

inline hipStream_t as_stream(kmoe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace kmoe
