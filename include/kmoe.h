/*
 * kmoe.h — C ABI of libkmoe.so: the MI355X (gfx950) quantized fused-MoE path.
 *
 * Every entry point takes raw DEVICE pointers plus explicit sizes, enqueues
 * hand-written HIP kernels on the given stream and returns at once:
 *   - returns KMOE_OK (0) or a negative KMOE_ERR_* code; never throws;
 *   - never allocates or frees device memory, never synchronises the stream
 *     (scratch comes in through `workspace` arguments sized by the
 *     *_workspace_bytes functions), so calls can be captured into a HIP graph;
 *   - enqueues on the given stream ONLY. The one exception is asked for per call:
 *     kmoe_moe_forward with KMOE_FLAG_SIDE_STREAM in kmoe_moe_args.flags may run
 *     the shared expert on a second stream of the library's (see the flag);
 *   - kmoe_last_error() gives the text of the calling thread's last failure.
 * A `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *
 * State the library keeps per process and GPU, besides its code: (1) a pacing
 * board of 128 KiB inside the device image (the persistent tile GEMM's workgroups
 * post their progress there so that tiles reading the same weight bytes stay in
 * step; every wait on it is bounded and no result depends on it, so launches that
 * overlap on one GPU - two streams, two layers - share it safely and at worst pace
 * each other badly); (2) the 64 MiB buffer of kmoe_moe_forward_static; (3) with
 * KMOE_FLAG_SIDE_STREAM, one stream and two events, created by the first call
 * that asks for them outside a capture.
 *
 * Each function cites the reference interface (baidu/vLLM-Kunlun, paths under
 * vllm_kunlun/) whose closed-source kernel it stands in for.
 *
 * Conventions shared by all functions
 *   M tokens, H hidden, E experts, K experts per token, I intermediate size,
 *   P = M*K routed (token, slot) pairs, flat pair index j = m*K + k.
 *   "sorted row" r in [0,P): position of a pair after the stable sort by
 *   expert id; rows of expert e are [lod[e], lod[e+1]).
 *   bf16 tensors are uint16_t bit patterns; rounding is round-to-nearest-even.
 *   int8 quantisation carries the row ABSMAX ("max"), not a scale: the value
 *   represented by q is q * max / 127 (reference: quantization/kernels/
 *   scale_mm.py:43-50, compressed_tensors_moe.py:116-120).
 */
#ifndef KMOE_H
#define KMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KMOE_OK 0
#define KMOE_ERR_NULL (-1)        /* a required pointer is NULL            */
#define KMOE_ERR_SHAPE (-2)       /* a size is out of range / inconsistent */
#define KMOE_ERR_UNSUPPORTED (-3) /* valid request this build cannot serve */
#define KMOE_ERR_WORKSPACE (-4)   /* workspace missing or too small        */
#define KMOE_ERR_LAUNCH (-5)      /* the HIP runtime refused a launch      */

typedef void* kmoe_stream_t;

/* Activation dtype of the int8 and unquantized paths: the 16-bit tensors (x, intermediates, out; the
 * weights of the unquantized path) hold bf16 or IEEE half patterns. The reference runs its deployment recipes with --dtype float16 (ci/scripts/server/start_vllm.sh:26;
 * platforms/kunlun.py:350-364 admits float16 and bfloat16). Functions without an act_dtype argument take bf16. */
#define KMOE_DT_BF16 0
#define KMOE_DT_F16 1

/* Text of the last error raised on the calling thread ("" if none). */
const char* kmoe_last_error(void);
/* Library version string, e.g. "kmoe 0.1 gfx950". */
const char* kmoe_version(void);
/* Diagnostics, no counterpart in the reference. kmoe_trace_kernels(1) clears the calling thread's record and starts
 * noting the GEMM kernel of every GEMM launch made on this thread (by the GEMM entry points and inside
 * kmoe_moe_forward), as the launcher chose it: name and template arguments, one per line in launch order, e.g.
 * "tiled_gemm_kernel<int8, SiLU-mul, 128x256 tile, 4 waves, 2 per CU>". kmoe_trace_kernels(0) stops noting and
 * keeps the record. kmoe_traced_kernels() returns the record (at most 4 KiB, valid until this thread's next
 * kmoe_trace_kernels(1)). Costs one thread-local test per launch while off. */
void kmoe_trace_kernels(int on);
const char* kmoe_traced_kernels(void);

/* ------------------------------------------------------------------ routing */

/*
 * Softmax top-K routing. Replaces kunlun_ops.moe_softmax_topk (renorm=0;
 * ops/_custom_ops.py:781-790, called ops/_kunlun_ops.py:666-668) and
 * kunlun_ops.moe_softmax_topk_norm (renorm=1; ops/_custom_ops.py:1084-1094,
 * called quantization/compressed_tensors/compressed_tensors_moe.py:152-159).
 *   logits [M,E] f32 -> topk_w [M,K] f32, topk_ids [M,K] i32.
 * ids: the K largest logits per row, descending, ties -> lower expert id.
 * w = softmax(logits)[ids]; with renorm, divided by their sum over K.
 * Limits: 1 <= K <= min(E,64), E <= 1024.
 */
int kmoe_softmax_topk(const float* logits, int M, int E, int K, int renorm,
                      float* topk_w, int32_t* topk_ids, kmoe_stream_t stream);

/*
 * DeepSeek-V3 "noaux_tc" routing. Replaces kunlun_ops.moe_sigmoid_group_topk_norm
 * (ops/_custom_ops.py:1351-1371, called compressed_tensors_moe.py:160-170 and
 * ops/_kunlun_ops.py:421-431; prototype csrc/xops.h:153-160).
 *   s = sigmoid(logits); c = s + bias (bias may be NULL = 0);
 *   group score = sum of the 2 largest c in the group; keep the topk_group
 *   best groups (ties -> lower group); take the K largest c among their
 *   experts (ties -> lower id); w = s[ids] / (sum_k s[ids] + 1e-20) * scale.
 * n_group <= 1 disables the group stage. Limits as above, n_group <= 64,
 * E % n_group == 0, E / n_group >= 2, K <= topk_group * E / n_group.
 */
int kmoe_sigmoid_group_topk_norm(const float* logits, const float* bias, int M,
                                 int E, int K, int n_group, int topk_group,
                                 float scale, float* topk_w, int32_t* topk_ids,
                                 kmoe_stream_t stream);

/* -------------------------------------------------------------------- align */

/*
 * Per-block histogram of expert ids. Replaces kunlun_ops.gen_block_statistic
 * (ops/_custom_ops.py:1123-1125, called compressed_tensors_moe.py:186).
 * Block b of n_blocks counts the pairs j in [b*ceil(P/n_blocks), ...).
 *   topk_ids [P] i32 -> block_statistic [n_blocks,E] i32 (overwritten).
 */
int kmoe_block_statistic(const int32_t* topk_ids, int P, int E, int n_blocks,
                         int32_t* block_statistic, kmoe_stream_t stream);

/* Scratch bytes kmoe_align needs for P pairs and E experts. */
size_t kmoe_align_workspace_bytes(int P, int E);

/*
 * Stable counting sort of the routed pairs by expert. Replaces the index part
 * of kunlun_ops.moe_pre_sorted (ops/_custom_ops.py:1144-1163, called
 * compressed_tensors_moe.py:188-196) and xspeedgate_ops.moe_pre_small
 * (compressed_tensors_moe.py:199-207).
 *   topk_ids [P] i32 (all in [0,E)) ->
 *   moe_index [P]   : sorted row of pair j              (reference: moe_index)
 *   sorted_src [P]  : pair j that sits in sorted row r   (inverse; may be NULL)
 *   expert_m [E]    : rows per expert                    (may be NULL)
 *   lod [E+1]       : exclusive prefix sum of expert_m   (sorted_tokens_num_lod)
 * Limits: E <= 1024, P <= 2^24.
 */
int kmoe_align(const int32_t* topk_ids, int P, int E, int32_t* moe_index,
               int32_t* sorted_src, int32_t* expert_m, int32_t* lod,
               void* workspace, size_t workspace_bytes, kmoe_stream_t stream);

/*
 * The same sort for an expert-parallel share: the ids are global and this launch owns the experts
 * [first_expert, first_expert + E) of them - the id shift of the reference's expert-parallel loop
 * (experts_id = ep_rank * num_local_experts + i, ops/_kunlun_ops.py:677-689). Pairs routed elsewhere get no
 * sorted row (moe_index = -1, which kmoe_combine skips); lod counts the local pairs only.
 */
int kmoe_align_local(const int32_t* topk_ids, int P, int E, int first_expert, int32_t* moe_index,
                     int32_t* sorted_src, int32_t* expert_m, int32_t* lod,
                     void* workspace, size_t workspace_bytes, kmoe_stream_t stream);

/*
 * Gather of activation rows into sorted order: the data part of
 * kunlun_ops.moe_pre_sorted (output moe_expand, compressed_tensors_moe.py:173-196).
 *   dst[r, :] = src[sorted_src[r] / K, :]   for r in [0,P); 16-bit elements,
 *   H % 8 == 0, rows 16-byte aligned.
 */
int kmoe_gather_rows(const uint16_t* src, int64_t ld_src,
                     const int32_t* sorted_src, int P, int K, int H,
                     uint16_t* dst, int64_t ld_dst, kmoe_stream_t stream);

/* ------------------------------------------------------ activation quantise */

/*
 * Per-row dynamic symmetric int8. Replaces kunlun_ops.quant2d
 * (ops/_custom_ops.py:1912-1924, called compressed_tensors_moe.py:224,253; and
 * through _C.scaled_int8_quant, ops/_custom_ops.py:1633-1657).
 *   x [R,C] bf16 -> q [R,C] i8, row_max [R] f32 (absmax of the row);
 *   q = clamp(rne(x * (127 / row_max)), -127, 127); an all-zero row gives q=0, max=0.
 * Limits: C % 8 == 0, C <= 65536, ld_x % 8 == 0, ld_q % 8 == 0.
 */
int kmoe_quant_i8_rows(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q,
                       int64_t ld_q, float* row_max, kmoe_stream_t stream);

/*
 * Same quantisation, codes written "chunk-major": q is [C/64][R][64], i.e. code
 * (r, c) sits at ((c/64)*R + r)*64 + c%64 — the activation layout of the
 * weight-streaming GEMM (KMOE_A_CHUNKED): the 64 bytes of a row that one MFMA step
 * consumes are contiguous, the rows of a step next to each other.
 * Limits as above, and C % 64 == 0.
 */
int kmoe_quant_i8_rows_chunked(const uint16_t* x, int64_t ld_x, int R, int C,
                               int8_t* q, float* row_max, kmoe_stream_t stream);

/* The two functions above for either activation dtype (KMOE_DT_*). */
int kmoe_quant_i8_rows_dt(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                          float* row_max, int act_dtype, kmoe_stream_t stream);
int kmoe_quant_i8_rows_chunked_dt(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q,
                                  float* row_max, int act_dtype, kmoe_stream_t stream);

/*
 * The other modes of torch.ops._C.scaled_int8_quant (ops/_custom_ops.py:1633-1657), which the reference hands
 * to xspeedgate_ops.static_scaled_int8_quant / dynamic_scaled_int8_quant (closed). Their arithmetic is the one
 * of the vLLM operator of the same name that the reference's scheme classes are written against
 * (csrc/quantization/compressed_tensors/int8_quant_kernels.cu):
 *   static:           q = sat8( rint(x / scale[0]) (+ azp[0]) )             one f32 scale (and zero point) per tensor
 *   dynamic + azp:    per row: s = (max - min) / 255 (1 for a constant row), azp = rint(-128 - min / s),
 *                     q = sat8( rint(x / s) + azp ); row_scale[r] = s, row_azp[r] = azp
 * with IEEE division, round-half-even and saturation to [-128, 127] (the sum with the zero point in int32).
 * x [R,C] in act_dtype; scale, azp: device pointers. Limits: C % 8 == 0, C <= 65536.
 */
int kmoe_quant_i8_static(const uint16_t* x, int64_t ld_x, int R, int C, const float* scale, const int32_t* azp,
                         int8_t* q, int64_t ld_q, int act_dtype, kmoe_stream_t stream);
int kmoe_quant_i8_rows_azp(const uint16_t* x, int64_t ld_x, int R, int C, int8_t* q, int64_t ld_q,
                           float* row_scale, int32_t* row_azp, int act_dtype, kmoe_stream_t stream);

/*
 * Epilogue of torch.ops._C.cutlass_scaled_mm_azp (ops/_custom_ops.py:1756-1771, closed in the reference; called by
 * KunlunScaledMMLinearKernel.apply_weights for asymmetric activations, quantization/kernels/scale_mm.py:70-82) on
 * the int32 accumulators of an int8 GEMM (acc_out of kmoe_grouped_gemm_i8). The arithmetic is the one of the vLLM
 * operator of that name (csrc/quantization/cutlass_w8a8, ScaledEpilogueBiasAzp / ...AzpToken):
 *   t = acc[r,c] - azp[r] * azp_adj[c]   (int32; azp == NULL: t = acc[r,c] - azp_adj[c], the zero point of a static
 *                                         scheme being folded into azp_adj)
 *   out[r,c] = dt( scale_a[r or 0] * (scale_b[c or 0] * float(t)) + bias[c] )      f32, products and sum unfused
 * azp_adj [n] int32: the sums of the weight codes over k per output channel. scale_a: one f32 per row
 * (scale_a_rows != 0) or one for the tensor; scale_b: one per channel (scale_b_cols != 0) or one; bias [n] f32 or NULL.
 * azp_adj == NULL (then azp must be NULL too) is the symmetric product with a bias, torch.ops._C.matmul(..., bias=)
 * (ops/_custom_ops.py:1811-1845; caller scale_mm.py:83-90): t = acc, and the scales meet it in the order of
 * kmoe_grouped_gemm_i8 and in its convention - scale_a and scale_b then hold the MAXES (x_pc_max, w_pc_max) and are
 * divided by 127 here: out = dt( (float(t) * (scale_a / 127)) * (scale_b / 127) + bias ), so that a zero bias
 * changes nothing.
 */
int kmoe_scaled_mm_azp_epilogue(const int32_t* acc, int64_t ld_acc, int M, int n, const float* scale_a, int scale_a_rows,
                                const float* scale_b, int scale_b_cols, const int32_t* azp_adj, const int32_t* azp,
                                const float* bias, uint16_t* out, int64_t ld_out, int act_dtype, kmoe_stream_t stream);

/*
 * Per-row, per-128-column-group dynamic fp8-e4m3fn (OCP). No counterpart in the
 * reference (its fp8 ops are empty stubs, ops/_custom_ops.py:44-89); follows
 * the DeepSeek-V3 block-scaled recipe.
 *   x [R,C] bf16 -> q [R,C] e4m3fn bytes, scale [R, C/128] f32;
 *   scale = absmax/448 (absmax 0 -> scale 0, q 0); q = e4m3fn_rne_sat(x / scale).
 * Limits: C % 128 == 0.
 */
int kmoe_quant_fp8_group128(const uint16_t* x, int64_t ld_x, int R, int C,
                            uint8_t* q, int64_t ld_q, float* scale,
                            kmoe_stream_t stream);
/* The same with x in act_dtype (KMOE_DT_BF16 or KMOE_DT_F16). */
int kmoe_quant_fp8_group128_dt(const uint16_t* x, int64_t ld_x, int R, int C,
                               uint8_t* q, int64_t ld_q, float* scale, int act_dtype,
                               kmoe_stream_t stream);

/* ------------------------------------------------------------- grouped GEMM */

#define KMOE_ACT_NONE 0
#define KMOE_ACT_SWIGLU 1 /* out[r,i] = silu(y[r,i]) * y[r,i+n/2], i < n/2 */
#define KMOE_ACT_SWIGLUOAI 2 /* bf16 only: out[r,i] = (u+1) * g * sigmoid(alpha*g), g = min(y[r,2i], limit),
                                u = clamp(y[r,2i+1], -limit, limit), i < n/2 (gate/up interleaved) */

typedef struct kmoe_gemm_i8_args {
  const int8_t* a;        /* [a_rows, k] quantised activations, row stride lda  */
  int64_t lda;
  const float* a_max;     /* [a_rows] absmax of each activation row             */
  const int32_t* row_src; /* NULL: sorted row r reads a[r]. Else it reads
                             a[row_src[r] / src_div] (gather through the sort)  */
  int32_t src_div;        /* >= 1                                               */
  const int8_t* w;        /* [E, n, k] weights, k contiguous                    */
  const float* w_max;     /* [E, n] absmax of each output channel               */
  const int32_t* lod;     /* [E+1] row offsets per expert (device)              */
  int32_t E, n, k;
  int32_t rows;           /* capacity = lod[E] upper bound (P)                  */
  uint16_t* y;            /* bf16 [rows, n] (act none) or [rows, n/2] (SwiGLU)  */
  int64_t ldy;
  int32_t* acc_out;       /* NULL, or int32 [rows, n]: raw accumulators         */
  int32_t act;            /* KMOE_ACT_*                                         */
  int32_t variant;        /* 0 = choose from the shape. Tuning and tests: 1-3 LDS-staged 16/32/64-row
                             kernels; with tiled weights 5 = tile kernel (6: 128-row tiles, 11: 64-row
                             tiles, 13: 96-row tiles, 7, 9: other tile shapes, 12: 128-row tiles whose m-tiles of
                             one expert and channel block keep in step so that they share the weight bytes in L2;
                             19, 18, 22: wide tiles of 128, 192, 256 rows - eight waves side by side along the
                             channels, one workgroup per CU (15, 14, 8 and 16 are older names of 19, 18, 22); 17: a
                             wide-tile launch and a paced 128-row-tile launch, of which the row counts decide on the
                             device which one works; 0 takes 64- / 96-row tiles for few rows per expert and the 128- or
                             192-row wide tiles beyond, an expert's rows split evenly over its tiles; all need k >= 128); with
                             chunked activations 1, 2, 4, 8 = 16-row fragments per pass of the streaming kernel */
  int32_t w_layout;       /* KMOE_W_ROWMAJOR, or KMOE_W_TILED (kmoe_tile_weights_i8) */
  int32_t a_layout;       /* KMOE_A_ROWMAJOR, or KMOE_A_CHUNKED: a is [k/64][a_rows][64]
                             (kmoe_quant_i8_rows_chunked); needs w_layout TILED   */
  int32_t a_rows;         /* rows of the chunked activation array               */
  /* Optional "tail expert": one more expert (e.g. a dense shared expert run in the
     same launch) whose weights live outside w. Its rows are [tail_row0, tail_row0 +
     tail_rows) — host values, not in lod — and row r of it reads activation row
     tail_src0 + r - tail_row0 (row_src is not consulted). NULL w_tail: none.      */
  const int8_t* w_tail;   /* [n, k], same layout as w                           */
  const float* w_max_tail; /* [n]                                                */
  int32_t tail_row0, tail_rows, tail_src0;
  int32_t act_dtype;      /* KMOE_DT_*: dtype of y (and of the rounding of gate and up before SiLU-mul) */
  int32_t rows_hint;      /* 0, or the rows the caller expects to be live when `rows` is only their bound (an
                             expert-parallel share): chooses the kernel, never the result          */
} kmoe_gemm_i8_args;

#define KMOE_W_ROWMAJOR 0
#define KMOE_W_TILED 1
/* layouts of the group scales of packed 4-bit weights (kmoe_gemm_w4_args.scale_layout) */
#define KMOE_S_ROWMAJOR 0
#define KMOE_S_FRAG16 1
#define KMOE_A_ROWMAJOR 0
#define KMOE_A_CHUNKED 1

/*
 * Re-arranges int8 weights [E,n,k] (k contiguous) into MFMA-ready 1 KB blocks
 * [E][n/16][k/64][4][16][16]: block byte 256*g + 16*c + t holds channel 16*nb + c,
 * k = 64*kb + 16*g + t. Done once after loading (the reference's hook for load-time
 * work is process_weights_after_loading, compressed_tensors_moe.py:116-120); the
 * values and every result are unchanged, only the streaming pattern is.
 * dst must not alias src. Limits: n % 16 == 0, k % 64 == 0.
 */
int kmoe_tile_weights_i8(const int8_t* src, int8_t* dst, int E, int n, int k,
                         kmoe_stream_t stream);

/*
 * W8A8 grouped GEMM. Replaces kunlun_ops.moe_fc in its int8 form
 * (ops/_custom_ops.py:1204-1244, called compressed_tensors_moe.py:226-238 and
 * 263-275; prototype csrc/xops.h:230-239) and, with E=1, the dense
 * kunlun_ops.matmul with x_pc_max/w_pc_max (ops/_custom_ops.py:1811-1845,
 * called quantization/kernels/scale_mm.py:83-90).
 * For each expert e and sorted row r in [lod[e], lod[e+1]):
 *   acc[r,c] = sum_k a[src(r),k] * w[e,c,k]                      (int32, exact)
 *   y[r,c]   = bf16( float(acc) * (a_max[src(r)]/127) * (w_max[e,c]/127) )
 * With KMOE_ACT_SWIGLU the bf16 y is never stored: the kernel stores
 *   bf16( silu(float(y[r,i])) * float(y[r,i+n/2]) ),  silu(t) = t/(1+exp(-t)).
 * Limits: k % 16 == 0, n % 16 == 0 (SwiGLU: n % 32 == 0), 16-byte aligned rows.
 */
int kmoe_grouped_gemm_i8(const kmoe_gemm_i8_args* args, kmoe_stream_t stream);

typedef struct kmoe_gemm_bf16_args {
  const uint16_t* a;      /* [a_rows, k] bf16 activations, row stride lda (elements) */
  int64_t lda;
  const int32_t* row_src; /* as in kmoe_gemm_i8_args                                  */
  int32_t src_div;
  const uint16_t* w;      /* [E, n, k] bf16 weights, k contiguous                     */
  const int32_t* lod;     /* [E+1]                                                    */
  int32_t E, n, k, rows;
  uint16_t* y;            /* bf16 [rows, n] or [rows, n/2] with SwiGLU                */
  int64_t ldy;
  int32_t act;
  int32_t variant;
  int32_t w_layout;       /* KMOE_W_ROWMAJOR, or KMOE_W_TILED: the BYTES of w ([E, n, 2k])
                             re-arranged by kmoe_tile_weights_i8(E, n, 2k); needs k % 32 == 0 */
  /* the expert-bias branch of KunlunOps.fused_moe (ops/_kunlun_ops.py:433-468): */
  const uint16_t* bias;   /* NULL, or [E, n] bf16: y = bf16(bf16(gemm) + bias), before the activation;
                             with KMOE_ACT_NONE or KMOE_ACT_SWIGLUOAI                  */
  float act_alpha, act_limit; /* KMOE_ACT_SWIGLUOAI (the reference uses 1.702 and 7.0)    */
  int32_t act_dtype;      /* KMOE_DT_BF16, or KMOE_DT_F16: a, w and y are IEEE half (the
                             unquantized method under --dtype float16); without bias / SWIGLUOAI */
  int32_t rows_hint;      /* 0, or the rows the caller expects to be live when `rows` is only their bound (an
                             expert-parallel share): chooses the kernel, never the result          */
} kmoe_gemm_bf16_args;

/*
 * Unquantized grouped GEMM: kunlun_ops.moe_fc with bf16 x and weight
 * (ops/_kunlun_ops.py:578-585, 595-603, 615-622; act="SWISH_GLU" at :595-603).
 *   y[r,c] = bf16( sum_k float(a[src(r),k]) * float(w[e,c,k]) ), f32 accumulation
 *   on MFMA (summation order is the hardware's; compare within tolerance); with
 *   act_dtype = KMOE_DT_F16 the same on half operands (v_mfma_f32_16x16x32_f16) with a
 *   half result.
 * Limits: k % 8 == 0, n % 16 == 0 (SwiGLU: n % 32 == 0).
 */
int kmoe_grouped_gemm_bf16(const kmoe_gemm_bf16_args* args, kmoe_stream_t stream);

typedef struct kmoe_gemm_fp8_args {
  const uint8_t* a;       /* [a_rows, k] e4m3fn activations, row stride lda           */
  int64_t lda;
  const float* a_scale;   /* [a_rows, k/128] per-row, per-128-column scales           */
  const int32_t* row_src;
  int32_t src_div;
  const uint8_t* w;       /* [E, n, k] e4m3fn weights                                 */
  const float* w_scale;   /* [E, n/128, k/128] one scale per 128x128 block            */
  const int32_t* lod;
  int32_t E, n, k, rows;
  uint16_t* y;
  int64_t ldy;
  int32_t act;
  int32_t variant;
  int32_t w_layout;       /* KMOE_W_ROWMAJOR, or KMOE_W_TILED: the bytes of w re-arranged
                             by kmoe_tile_weights_i8 (which moves bytes whatever they
                             encode); needs k % 128 == 0, always true here          */
  /* Optional "tail expert", as in kmoe_gemm_i8_args: one more expert whose weights live
     outside w (a dense shared expert run in the same launch). Its rows are
     [tail_row0, tail_row0 + tail_rows) of y and read a rows tail_src0 + i (no gather). */
  const uint8_t* w_tail;      /* NULL, or [n, k] in w_layout                          */
  const float* w_scale_tail;  /* [n/128, k/128]                                       */
  int32_t tail_row0, tail_rows, tail_src0;
  int32_t act_dtype;          /* KMOE_DT_BF16, or KMOE_DT_F16: y (and the rounding of gate and up before
                                 SiLU-mul) in IEEE half                                */
  int32_t rows_hint;      /* 0, or the rows the caller expects to be live when `rows` is only their bound (an
                             expert-parallel share): chooses the kernel, never the result          */
} kmoe_gemm_fp8_args;

/*
 * fp8-e4m3fn block-scaled grouped GEMM (DeepSeek-V3 recipe). The reference has no
 * fp8 MoE (platforms/kunlun.py:350-364 rejects fp8; moe_fc only exposes the
 * scale_n/scale_k arguments, ops/_custom_ops.py:1218-1221).
 *   y[r,c] = bf16( sum_kb [ sum_{k in kb} a[src(r),k]*w[e,c,k] ] * a_scale[src(r),kb] * w_scale[e,c/128,kb] )
 * with kb the 128-wide K blocks, f32 accumulation.
 * Limits: k % 128 == 0, n % 128 == 0 (SwiGLU: n % 256 == 0).
 */
int kmoe_grouped_gemm_fp8_block(const kmoe_gemm_fp8_args* args, kmoe_stream_t stream);

typedef struct kmoe_gemm_w4_args {
  const uint16_t* a;      /* [a_rows, k] bf16 activations, row stride lda (elements)  */
  int64_t lda;
  const int32_t* row_src; /* as in kmoe_gemm_i8_args                                  */
  int32_t src_div;
  const uint8_t* w;       /* [E, n, k/2] packed 4-bit codes: two per byte, low nibble first,
                             code c means c - 8; the bytes re-arranged by
                             kmoe_tile_weights_i8(E, n, k/2) (w_layout = KMOE_W_TILED)  */
  const uint16_t* w_scale;/* [E, n, k/group_size] bf16                                */
  int32_t group_size;     /* values per scale along k: a multiple of 32 that divides k
                             (k itself: one scale per output channel)                 */
  const int32_t* lod;     /* [E+1]                                                    */
  int32_t E, n, k, rows;
  uint16_t* y;            /* bf16 [rows, n] or [rows, n/2] with SwiGLU                */
  int64_t ldy;
  int32_t act;            /* KMOE_ACT_NONE or KMOE_ACT_SWIGLU                         */
  int32_t variant;        /* 0 = from the shape; 1, 2, 4 = 16-row fragments per pass of the
                             streaming kernel; 64, 96, 128 = the tile kernel (prefill) with tiles
                             of that many rows (8 = 128)                              */
  int32_t w_layout;       /* KMOE_W_TILED                                             */
  int32_t act_dtype;      /* KMOE_DT_BF16, or KMOE_DT_F16: a, w_scale and y are IEEE half and the
                             weight values are half((code - 8) * scale), what
                             dequant_int4_native (quant_ops.py:71-86) itself computes  */
  int32_t scale_layout;   /* KMOE_S_ROWMAJOR: w_scale as the checkpoint holds it, [E, n, k/group_size];
                             KMOE_S_FRAG16: re-arranged by kmoe_tile_scales_w4 (same bytes in total) */
  int32_t rows_hint;      /* 0, or the rows the caller expects to be live when `rows` is only their bound (an
                             expert-parallel share): chooses the kernel, never the result          */
} kmoe_gemm_w4_args;

/*
 * 4-bit weight-only grouped GEMM (W4A16). The reference unpacks the packed tensors to
 * fp16 inside every call (dequant_int4_native, quantization/kernels/quant_ops.py:71-86,
 * called compressed_tensors_moe.py:320-327) and then runs the unquantized moe_fc; this
 * entry point reads the packed weights once and unpacks them in registers:
 *   y[r,c] = bf16( sum_k float(a[src(r),k]) * float(bf16((code[e,c,k] - 8) * scale[e,c,k/group])) )
 * i.e. the bf16 grouped GEMM on the weights kmoe_dequant_w4_bf16 would produce, with
 * f32 accumulation on MFMA (compare within tolerance). Two kernels: a weight-streaming
 * one for the decode regime (an expert with more rows than one pass holds streams its
 * weights again) and, from two dozen rows per expert, one on 128-row tiles that shares
 * the unpacking of a weight among the tile's rows; both sum in the same order and give
 * the same bits.
 * Limits: k % 128 == 0, n % 16 == 0 (SwiGLU: n % 32 == 0), tiled weights; the tile
 * kernel needs rows * lda * 2 < 4 GiB (else the streaming kernel serves every size).
 */
int kmoe_grouped_gemm_w4a16(const kmoe_gemm_w4_args* args, kmoe_stream_t stream);

/*
 * Load-time re-arrangement of the group scales of packed 4-bit weights (no counterpart in the
 * reference, whose closed kernels take the checkpoint layout): [E, n, groups] -> per 16 output
 * channels [groups][16]. The scales one MFMA block needs (16 channels x the 1 to 4 groups the
 * block's 128 values fall into) are then 32 to 128 consecutive bytes instead of 16 pieces a row
 * apart: the form to hand to kmoe_grouped_gemm_w4a16 / kmoe_moe_forward where a channel has more
 * scales than a workgroup can hold in LDS (long k, small groups). Not in place. n % 16 == 0.
 */
int kmoe_tile_scales_w4(const uint16_t* src, uint16_t* dst, int E, int n, int groups, kmoe_stream_t stream);

/*
 * The gpt-oss activation on a stored, interleaved gate_up result. Replaces
 * torch.ops._C.swigluoai_and_mul (ops/_custom_ops.py:728-742).
 *   y [R,2I] bf16 -> out [R,I] bf16, out[r,i] = (u+1) * g * sigmoid(alpha*g),
 *   g = min(y[r,2i], limit), u = clamp(y[r,2i+1], -limit, limit).
 */
int kmoe_swigluoai_and_mul(const uint16_t* y, int64_t ld_y, int R, int I, float alpha,
                           float limit, uint16_t* out, int64_t ld_out, kmoe_stream_t stream);

/*
 * SiLU-and-mul on a stored gate_up result. Replaces kunlun_ops.swiglu
 * (ops/_custom_ops.py:699-706, called compressed_tensors_moe.py:240-243).
 *   y [R,2I] bf16 -> out [R,I] bf16 = bf16( silu(y[:, :I]) * y[:, I:] ).
 */
int kmoe_silu_and_mul(const uint16_t* y, int64_t ld_y, int R, int I,
                      uint16_t* out, int64_t ld_out, kmoe_stream_t stream);
/* ... for either activation dtype (KMOE_DT_*). */
int kmoe_silu_and_mul_dt(const uint16_t* y, int64_t ld_y, int R, int I, uint16_t* out, int64_t ld_out,
                         int act_dtype, kmoe_stream_t stream);

/*
 * The device's SiLU, tabulated: table[h] (f32, 65536 entries) = silu of the 16-bit activation pattern h in
 * act_dtype, computed by the very function every GEMM epilogue and kmoe_silu_and_mul use. No counterpart in the
 * reference; it exists for checkers. The kernels compute silu(g) = g / (1 + e^-g) on the hardware's exp2 and
 * reciprocal instructions (each within one ulp, not correctly rounded), applied to the gate value AFTER it has been
 * rounded to the activation type, as the reference's silu_and_mul (ops/_custom_ops.py:699-706) reads a 16-bit
 * tensor. A CPU restatement that looks silu up in this table therefore reproduces the kernels' outputs bit for
 * bit, and the table itself is what to hold against a libm silu (within 4e-6 relative).
 */
int kmoe_silu_table(float* table, int act_dtype, kmoe_stream_t stream);

/*
 * Shader-clock probe, a measurement aid with no counterpart in the reference. n_workgroups (1..64) single-wave
 * workgroups each run `reps` (2..1048576) runs of fixed length in shader clocks - odd runs 8 x s_sleep 127, even
 * runs a chain of 2048 dependent v_fma_f32 - and write three int64 per run to samples[(workgroup * reps + run) * 3]:
 * the 100 MHz counter at the start, the run's duration in ticks of that counter (10 ns), and the run's duration in
 * s_memtime ticks. Launched on a second stream beside a kernel under test: the s_memtime ticks of a run stay the
 * same whatever runs beside it while its 10-ns duration stretches when the chip lowers the shader clock under load,
 * so ticks / duration is the clock the kernel under test really gets. The persistent tile kernels occupy every CU;
 * the environment variable KMOE_SPARE_CUS=n (read once per process) cuts their grids for n fewer CUs, so that the
 * probe's waves (or a collective's) find a place beside them.
 */
int kmoe_clock_probe(int64_t* samples, int n_workgroups, int reps, kmoe_stream_t stream);

/*
 * Un-permute + weighted top-K sum. Replaces kunlun_ops.moe_post
 * (ops/_custom_ops.py:1316-1324, called compressed_tensors_moe.py:278-290).
 *   out[m,h] = bf16( sum_k topk_w[m,k] * dq[m,k] * float(x[moe_index[m*K+k], h]) )
 * f32 accumulation, k ascending; dequant_scale (dq) may be NULL (= 1).
 * Optional caller epilogue (models/deepseek_v2.py:288-296), applied when
 * out_scale != 1 or addend != NULL:
 *   out = bf16( float(bf16(float(out) * out_scale)) + float(addend[m,h]) ).
 */
int kmoe_combine(const uint16_t* x, int64_t ld_x, const int32_t* moe_index,
                 const float* topk_w, const float* dequant_scale, int M, int K,
                 int H, float out_scale, const uint16_t* addend,
                 int64_t ld_addend, uint16_t* out, int64_t ld_out,
                 kmoe_stream_t stream);
/*
 * ... for either activation dtype (KMOE_DT_*), and with a factor on the addend: the half-precision form of
 * the caller epilogue (models/deepseek_v2.py:286-292) keeps the routed sum unscaled and multiplies the
 * shared expert's output by 1/routed_scaling_factor instead:
 *   out = dt( float(dt(float(out) * out_scale)) + float(dt(float(addend[m,h]) * addend_scale)) ),
 * a factor of exactly 1 skipping its multiplication and rounding.
 */
int kmoe_combine_dt(const uint16_t* x, int64_t ld_x, const int32_t* moe_index,
                    const float* topk_w, const float* dequant_scale, int M, int K,
                    int H, float out_scale, const uint16_t* addend, int64_t ld_addend,
                    float addend_scale, uint16_t* out, int64_t ld_out, int act_dtype,
                    kmoe_stream_t stream);

/*
 * Unpacks 4-bit weights to bf16 once, at load time. Replaces dequant_int4_native
 * (quantization/kernels/quant_ops.py:71-86), which KunlunCompressedTensorsWNA16MoEMethod.apply
 * runs on the whole weight tensor in EVERY forward call (compressed_tensors_moe.py:320-327).
 * packed [rows, k/2] bytes, low nibble = element 2j, high nibble = element 2j+1, unsigned code c
 * means c - 8; scale [rows, k/group_size] bf16 (group_size == k: one scale per row):
 *   out[r, j] = bf16( float(c - 8) * float(scale[r, j / group_size]) ).
 * (The reference tiles its scale tensor along k with Tensor.repeat, which equals this for one
 * scale per row; for several groups per row this function follows the contiguous groups of the
 * compressed-tensors format.) Limits: k % 16 == 0, group_size % 2 == 0, k % group_size == 0.
 */
int kmoe_dequant_w4_bf16(const uint8_t* packed, const uint16_t* scale, int64_t rows, int k,
                         int group_size, uint16_t* out, kmoe_stream_t stream);
/* The same with scale and out in act_dtype (KMOE_DT_*). KMOE_DT_F16 is the reference's own
 * arithmetic: (code.to(float16) - 8) * scale, one rounding to half. */
int kmoe_dequant_w4(const uint8_t* packed, const uint16_t* scale, int64_t rows, int k,
                    int group_size, uint16_t* out, int act_dtype, kmoe_stream_t stream);

/* ---------------------------------------------------------------- router GEMM */

/*
 * Router logits: logits[M,E] (f32) = x[M,H] (bf16) . w_gate[E,H]^T (bf16), accumulated in
 * f32. Replaces the gate projection in front of the layer: GateLinear.forward /
 * ops.router_gemm_bf16_fp32 (ops/fused_moe/router/gate_linear.py:91-116), called as
 * `router_logits, _ = self.gate(hidden_states)` (models/deepseek_v2.py:178-184, 275).
 * K is split over workgroups for small M; the partial planes (in `workspace`,
 * kmoe_router_gemm_workspace_bytes) are added in a fixed order, so the result does not
 * depend on scheduling. Limits: H % 32 == 0, E <= 1024, 16-byte aligned tensors.
 */
size_t kmoe_router_gemm_workspace_bytes(int M, int H, int E);
int kmoe_router_gemm_bf16(const uint16_t* x, int64_t ld_x, const uint16_t* w_gate,
                          int M, int H, int E, float* logits, int64_t ld_logits,
                          void* workspace, size_t workspace_bytes, kmoe_stream_t stream);
/* ... with x and w_gate in either dtype (KMOE_DT_*; both the same). */
int kmoe_router_gemm(const uint16_t* x, int64_t ld_x, const uint16_t* w_gate,
                     int M, int H, int E, float* logits, int64_t ld_logits,
                     void* workspace, size_t workspace_bytes, int act_dtype, kmoe_stream_t stream);

/* ------------------------------------------------------------ fused forward */

#define KMOE_SCORE_SOFTMAX 0
#define KMOE_SCORE_SIGMOID 1

#define KMOE_FMT_INT8 0      /* int8 weights + per-channel max, per-token int8 activations   */
#define KMOE_FMT_FP8_BLOCK 1 /* e4m3fn weights + 128x128 block scales, 1x128 activation scales */
#define KMOE_FMT_BF16 2      /* bf16 weights, no quantisation                                 */
#define KMOE_FMT_W4A16 3     /* packed 4-bit weights + bf16 group scales, bf16 activations
                                (kmoe_grouped_gemm_w4a16); no shared expert, no bias     */

typedef struct kmoe_moe_args {
  /* shape */
  int32_t M, H, E, K, I;
  int32_t format;        /* KMOE_FMT_*                                           */
  /* routing */
  int32_t scoring;       /* KMOE_SCORE_*                                        */
  int32_t renormalize;   /* softmax only: divide the K weights by their sum     */
  int32_t n_group, topk_group; /* sigmoid only; n_group <= 1: no group stage    */
  float routed_scale;    /* sigmoid only: multiplies the routing weights        */
  const float* logits;   /* [M,E] f32, or NULL with w_gate set: the layer then computes
                            them itself (kmoe_router_gemm_bf16 without the reduction
                            pass: the routing kernel adds the partial planes)     */
  const float* bias;     /* [E] f32 correction bias or NULL                     */
  /* activations and routed expert weights */
  const uint16_t* x;     /* [M,H] bf16                                          */
  const void* w13;       /* [E,2I,H] int8 / e4m3fn / bf16                       */
  const float* w13_max;  /* INT8: [E,2I] absmax. FP8: [E,2I/128,H/128] scales. BF16: NULL */
  const void* w2;        /* [E,H,I]                                             */
  const float* w2_max;   /* INT8: [E,H]. FP8: [E,H/128,I/128]. BF16: NULL       */
  /* optional dense shared expert in the same format (I_shared = 0: none) */
  int32_t I_shared;
  const void* ws13;      /* [2*I_shared,H]                                      */
  const float* ws13_max; /* INT8: [2*I_shared]. FP8: [2*I_shared/128,H/128]     */
  const void* ws2;       /* [H,I_shared]                                        */
  const float* ws2_max;  /* INT8: [H]. FP8: [H/128,I_shared/128]                */
  /* caller epilogue: out = routed*out_scale (+ shared) */
  float out_scale;
  uint16_t* out;         /* [M,H] bf16                                          */
  /* optional profiling: NULL, or 2*KMOE_N_STAGES hipEvent_t handles; entry 2s is
     recorded on the stream before stage s and entry 2s+1 after it (NULL entries
     are skipped). Leave NULL under graph capture.                             */
  void* const* stage_events;
  int32_t w_layout;      /* KMOE_W_TILED if w13, w2 went through kmoe_tile_weights_i8;
                            else KMOE_W_ROWMAJOR                                   */
  const uint16_t* w_gate; /* NULL, or [E,H] bf16 router weight (used when logits is NULL) */
  /* BF16 only, the expert-bias branch (ops/_kunlun_ops.py:433-468): */
  const uint16_t* w13_bias; /* NULL, or [E,2I] bf16                                   */
  const uint16_t* w2_bias;  /* NULL, or [E,H] bf16                                    */
  int32_t activation;    /* KMOE_ACT_SWIGLU (0 means the same) or KMOE_ACT_SWIGLUOAI: w13
                            then holds gate and up rows interleaved               */
  float act_alpha, act_limit;
  int32_t ws_layout;     /* layout of ws13, ws2 (KMOE_W_*): a shared expert whose sizes do not allow
                            tiling (k % 64) stays row-major next to tiled routed experts  */
  /* W4A16 only: w13 / w2 hold the packed codes ([E,2I,H/2], [E,H,I/2] bytes, tiled) */
  const uint16_t* w13_scale; /* [E,2I,H/group_size] bf16                               */
  const uint16_t* w2_scale;  /* [E,H,I/group_size] bf16                                */
  int32_t group_size;    /* a multiple of 32 dividing H and I (one value for both tensors) */
  int32_t act_dtype;     /* KMOE_DT_* of x, out (and w_gate, shared-expert output): half goes with every format
                            (KMOE_FMT_BF16: the weights are then half too, and no biases, no SWIGLUOAI;
                            KMOE_FMT_W4A16: the group scales are then half) */
  float shared_scale;    /* caller epilogue for half activations (models/deepseek_v2.py:286-292: the routed sum stays
                            unscaled and the shared expert's output is multiplied by 1/routed_scaling_factor):
                            out = dt( dt(routed * out_scale) + dt(shared * shared_scale) ); 0 means 1 */
  int32_t tile_variant;  /* INT8 and FP8_BLOCK, tuning: 0, or the `variant` (int8: 5-22; fp8: 5, 6, 8, 11-14, 17-19) handed to
                            the two routed GEMMs when the batch runs on the tile kernel (more than 10 rows per
                            expert); ignored otherwise */
  int32_t w_scale_layout; /* W4A16: KMOE_S_* of w13_scale and w2_scale                                  */
  /* An expert-parallel share (ops/_kunlun_ops.py:640-696: each rank holds num_local_experts of the experts and
     computes what the pairs routed to them contribute; the sum over ranks is the caller's all-reduce). The routing
     runs over E_global experts (logits [M,E_global], bias [E_global], w_gate [E_global,H]; K <= E_global); the
     weights are those of the E experts [first_expert, first_expert + E). 0 / 0: one GPU holds every expert. */
  int32_t E_global, first_expert;
  int32_t flags;         /* KMOE_FLAG_* or'ed together; 0: none                                            */
} kmoe_moe_args;

/* kmoe_moe_args.flags.
 * KMOE_FLAG_SIDE_STREAM: a shared expert that cannot ride in the routed launches (a width other than the routed
 * experts'; the fp8 layer at decode sizes) may run on a second stream of the library's own (one per GPU, default
 * priority, non-blocking, created by the first such call that is not being captured), forked from `stream` by an
 * event after the first quantisation and joined back by an event before the combine: the caller still sees one
 * stream's worth of ordering, and under capture the fork and join become graph edges. Without the flag (the default)
 * everything is enqueued on `stream`. The environment variable KMOE_SIDE_STREAM overrides the flag for the whole
 * process (0: never, 1: as if every call set it); it is read once. Ignored with stage_events and by
 * kmoe_moe_forward_static. */
#define KMOE_FLAG_SIDE_STREAM 1

/* Decode-sized int8 batches (at most 10 rows per expert, tiled weights): two of the layer's small launches are folded
 * into the GEMM launches. The gate_up launch sorts the routed pairs by expert itself (every workgroup scans the pairs'
 * expert ids; up to 4096 pairs and 512 tokens, one GPU holding every expert) and writes moe_index, sorted_src,
 * expert_m and lod as the sort's launch would (so does the gate_up launch of KMOE_FMT_W4A16 where it runs on that
 * format's streaming kernel); the down launch quantises its rows itself (rows up to 1024 values)
 * and writes actq and actmax as the quantiser's launch would. Same bits, same workspace contents, two launches
 * fewer; KMOE_STAGE_ALIGN / KMOE_STAGE_QUANT2 then bracket nothing. The environment variables KMOE_SORT_IN_GEMM=0
 * and KMOE_QUANT_IN_GEMM=0 (read once per process) keep the launches apart: for measurements. */

#define KMOE_STAGE_ROUTING 0
#define KMOE_STAGE_ALIGN 1
#define KMOE_STAGE_QUANT1 2
#define KMOE_STAGE_GEMM1 3 /* gate_up + SiLU-mul */
#define KMOE_STAGE_QUANT2 4
#define KMOE_STAGE_GEMM2 5 /* down */
#define KMOE_STAGE_SHARED 6
#define KMOE_STAGE_COMBINE 7
#define KMOE_N_STAGES 8

/* Byte offsets of the intermediates kmoe_moe_forward keeps in its workspace.
 * An int8 shared expert as wide as the routed experts (I_shared == I) is run as
 * one more expert of the routed launches: its rows are [P, P+M) of act / actq /
 * actmax / down, and the sh_* slots stay empty.
 * xq/actq hold int8 or e4m3fn codes; xmax/actmax hold row maxes (INT8) or
 * per-128-column scales (FP8); all four are unused for BF16. */
typedef struct kmoe_moe_layout {
  size_t total_bytes;
  size_t topk_w, topk_ids, moe_index, sorted_src, expert_m, lod, align_ws;
  size_t xq, xmax, act, actq, actmax, down;
  size_t sh_lod, sh_act, sh_actq, sh_actmax, sh_out;
  size_t codes_chunked; /* 1: xq/actq/sh_actq are chunk-major [C/64][rows][64] (the
                           weight-streaming decode path), 0: row-major [rows][C] */
  size_t logit_planes;  /* partial router logits [planes][M][E] f32 (w_gate given)   */
  size_t n_logit_planes;
} kmoe_moe_layout;

/* Workspace layout (and total size) for a shape; only the shape and format fields of args are read. */
int kmoe_moe_workspace_layout(const kmoe_moe_args* args, kmoe_moe_layout* layout);

/*
 * The whole layer: routing -> align -> activation quant -> gate_up GEMM with
 * fused SiLU-mul -> activation quant -> down GEMM -> weighted combine
 * (+ shared expert, + caller epilogue). Replaces, for KMOE_FMT_INT8,
 * KunlunCompressedTensorsW8A8Int8MoEMethod.apply_monolithic
 * (compressed_tensors_moe.py:122-291) with the shared expert of
 * KunlunScaledMMLinearKernel.apply_weights (quantization/kernels/scale_mm.py:52-90);
 * for KMOE_FMT_BF16, KunlunOps.fused_moe (ops/_kunlun_ops.py:377-637). KMOE_FMT_FP8_BLOCK
 * has no counterpart in the reference. Results are bit-identical to running the
 * stage functions above one by one.
 */
int kmoe_moe_forward(const kmoe_moe_args* args, void* workspace,
                     size_t workspace_bytes, kmoe_stream_t stream);

/*
 * kmoe_moe_forward without a workspace argument. No counterpart in the reference: it is for
 * callers that cannot allocate device memory for a workspace (code that is being captured
 * into a HIP graph, serving loops and harnesses that forbid hipMalloc). The intermediates live
 * in a buffer of KMOE_STATIC_WORKSPACE_BYTES that is part of the library's device image (every
 * GPU the library runs on holds it until the process ends); a shape whose
 * kmoe_moe_workspace_layout().total_bytes exceeds it is refused with KMOE_ERR_WORKSPACE.
 * Allocates nothing, same results as kmoe_moe_forward bit for bit. Call it with the stream's
 * device current. All calls on one GPU share the one buffer: calls that may overlap on a GPU
 * (two streams, two threads) race; the buffer keeps the last call's intermediates.
 * The buffer's device address is looked up once per GPU, by the first kmoe_moe_forward or
 * kmoe_moe_forward_static call on that GPU whose stream is not being captured (the lookup is
 * not a stream operation). A captured call that would be the first is refused with
 * KMOE_ERR_UNSUPPORTED: make one call on the GPU outside the capture before.
 */
#define KMOE_STATIC_WORKSPACE_BYTES (64u << 20)
int kmoe_moe_forward_static(const kmoe_moe_args* args, kmoe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KMOE_H */
