// Host side of libkmoe: error state, and the fused layer call that strings the
// stage kernels together on one stream out of one caller-owned workspace.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "kmoe_common.h"

namespace kmoe {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// ---- record of the GEMM kernels a thread launches (kmoe_trace_kernels) ----
static thread_local bool g_trace_on = false;
static thread_local char g_trace[4096] = "";
static thread_local size_t g_trace_len = 0;

bool tracing_kernels() { return g_trace_on; }
void note_kernel(const char* fmt, ...) {
  if (!g_trace_on || g_trace_len + 2 >= sizeof(g_trace)) return;
  va_list ap;
  va_start(ap, fmt);
  const int n = vsnprintf(g_trace + g_trace_len, sizeof(g_trace) - g_trace_len - 1, fmt, ap);
  va_end(ap);
  if (n < 0) return;
  g_trace_len = g_trace_len + static_cast<size_t>(n) < sizeof(g_trace) - 2 ? g_trace_len + static_cast<size_t>(n)
                                                                           : sizeof(g_trace) - 2;
  g_trace[g_trace_len++] = '\n';
  g_trace[g_trace_len] = '\0';
}

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return KMOE_OK;
  return fail(KMOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
}

}  // namespace kmoe

using namespace kmoe;

extern "C" const char* kmoe_last_error(void) { return g_error; }
extern "C" const char* kmoe_version(void) { return "kmoe 0.3 gfx950"; }
extern "C" void kmoe_trace_kernels(int on) {
  if (on) {
    g_trace[0] = '\0';
    g_trace_len = 0;
  }
  g_trace_on = on != 0;
}
extern "C" const char* kmoe_traced_kernels(void) { return g_trace; }

namespace {

// formats whose GEMMs read the bf16 activations themselves (no activation quantisation)
bool bf16_activations(int format) { return format == KMOE_FMT_BF16 || format == KMOE_FMT_W4A16; }

int check_shape(const kmoe_moe_args* a) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "moe_forward: args is NULL");
  KMOE_REQUIRE(a->M >= 0 && a->H >= 16 && a->E >= 1 && a->K >= 1 && a->I >= 16, KMOE_ERR_SHAPE,
               "moe_forward: M=%d H=%d E=%d K=%d I=%d", a->M, a->H, a->E, a->K, a->I);
  KMOE_REQUIRE(a->format == KMOE_FMT_INT8 || a->format == KMOE_FMT_FP8_BLOCK || a->format == KMOE_FMT_BF16 ||
                   a->format == KMOE_FMT_W4A16,
               KMOE_ERR_UNSUPPORTED, "moe_forward: format=%d unknown", a->format);
  if (a->format == KMOE_FMT_W4A16) {
    KMOE_REQUIRE(a->I_shared == 0, KMOE_ERR_UNSUPPORTED, "moe_forward: no shared expert with 4-bit weights");
    KMOE_REQUIRE(a->w_layout == KMOE_W_TILED, KMOE_ERR_UNSUPPORTED, "moe_forward: 4-bit weights must be tiled");
    KMOE_REQUIRE(a->group_size >= 32 && a->group_size % 32 == 0 && a->H % a->group_size == 0 &&
                     a->I % a->group_size == 0,
                 KMOE_ERR_SHAPE, "moe_forward: group_size=%d must be a multiple of 32 dividing H=%d and I=%d",
                 a->group_size, a->H, a->I);
  }
  const int mult = a->format == KMOE_FMT_FP8_BLOCK || a->format == KMOE_FMT_W4A16 ? 128 : 16;
  KMOE_REQUIRE(a->H % mult == 0 && a->I % mult == 0, KMOE_ERR_SHAPE,
               "moe_forward: H=%d and I=%d must be multiples of %d", a->H, a->I, mult);
  const int Eg = a->E_global > 0 ? a->E_global : a->E;
  KMOE_REQUIRE(a->K <= Eg && a->K <= 64 && a->E <= 1024 && Eg <= 1024, KMOE_ERR_SHAPE,
               "moe_forward: K=%d E=%d E_global=%d out of range", a->K, a->E, Eg);
  KMOE_REQUIRE(a->first_expert >= 0 && a->first_expert + a->E <= Eg, KMOE_ERR_SHAPE,
               "moe_forward: experts [%d, %d) are not among the %d the routing runs over", a->first_expert,
               a->first_expert + a->E, Eg);
  KMOE_REQUIRE(a->I_shared >= 0 && a->I_shared % mult == 0, KMOE_ERR_SHAPE,
               "moe_forward: I_shared=%d must be a non-negative multiple of %d", a->I_shared, mult);
  KMOE_REQUIRE(static_cast<long long>(a->M) * a->K <= (1 << 24), KMOE_ERR_SHAPE, "moe_forward: M*K too large");
  KMOE_REQUIRE(a->act_dtype == KMOE_DT_BF16 || a->act_dtype == KMOE_DT_F16, KMOE_ERR_UNSUPPORTED,
               "moe_forward: act_dtype=%d unknown", a->act_dtype);
  KMOE_REQUIRE(a->act_dtype == KMOE_DT_BF16 || a->format != KMOE_FMT_BF16 ||
                   (!a->w13_bias && !a->w2_bias && a->activation != KMOE_ACT_SWIGLUOAI),
               KMOE_ERR_UNSUPPORTED, "moe_forward: expert biases and swigluoai are built for bf16 only");
  // elements in 64 bytes of a weight row
  const int row64 = a->format == KMOE_FMT_BF16 ? 32 : (a->format == KMOE_FMT_W4A16 ? 128 : 64);
  KMOE_REQUIRE(a->w_layout == KMOE_W_ROWMAJOR ||
                   (a->w_layout == KMOE_W_TILED && a->H % row64 == 0 && a->I % row64 == 0),
               KMOE_ERR_SHAPE, "moe_forward: w_layout=%d needs H, I multiples of %d", a->w_layout, row64);
  KMOE_REQUIRE(a->I_shared == 0 || a->ws_layout == KMOE_W_ROWMAJOR ||
                   (a->ws_layout == KMOE_W_TILED && a->H % row64 == 0 && a->I_shared % row64 == 0),
               KMOE_ERR_SHAPE, "moe_forward: ws_layout=%d needs H, I_shared multiples of %d", a->ws_layout, row64);
  return KMOE_OK;
}

// The weight-streaming decode path (chunk-major codes, no row tiles) against the persistent tile kernel:
// the stream kernels re-read the weights once per 16-64 rows of an expert, so their time grows with the rows
// per expert; the tile kernel's hardly does. Measured cross-over with 64-row tiles: 10-12 rows per expert on
// both the Qwen3 and the DeepSeek-V3 shape.
// Pairs this launch expects to land on its own experts: all of them, or the share of an expert-parallel rank under
// uniform routing (the kernels are chosen by the rows per expert; any choice is correct for any routing).
long long local_pairs(const kmoe_moe_args* a) {
  const long long P = static_cast<long long>(a->M) * a->K;
  return a->E_global > a->E ? (P * a->E + a->E_global - 1) / a->E_global : P;
}

// KMOE_SORT_IN_GEMM=0 (read once) keeps the sort a launch of its own on the weight-streaming path too.
bool scan_allowed() {
  static const bool on = [] {
    const char* v = getenv("KMOE_SORT_IN_GEMM");
    return !(v && v[0] == '0');
  }();
  return on;
}

// KMOE_QUANT_IN_GEMM=0 (read once) keeps the second quantisation a launch of its own there.
bool quant_in_gemm_allowed() {
  static const bool on = [] {
    const char* v = getenv("KMOE_QUANT_IN_GEMM");
    return !(v && v[0] == '0');
  }();
  return on;
}

bool use_stream_path(const kmoe_moe_args* a) {
  const long long P = local_pairs(a);
  // a row-major shared expert cannot read the chunk-major codes this path quantises x into
  return a->format == KMOE_FMT_INT8 && a->w_layout == KMOE_W_TILED && (P + a->E - 1) / a->E <= 10 && a->M <= 1024 &&
         (a->I_shared == 0 || a->ws_layout == KMOE_W_TILED);
}

// A shared expert of the routed experts' width runs inside the routed GEMM launches
// as one more ("tail") expert over rows [P, P+M): no extra launches, and its few
// workgroups overlap the routed experts' instead of leaving most CUs idle.
// fp8: only where the routed experts run on the tile kernel (more than 10 rows per expert). With fewer
// rows the routed launch uses the 16-row LDS-staged kernel, which would stream the tail expert's weights once
// per 16 token rows (measured at 128 tokens: gate_up +260 us against 57 us for a launch of its own).
bool fold_shared(const kmoe_moe_args* a) {
  if (a->I_shared <= 0 || a->I_shared != a->I || a->ws_layout != a->w_layout) return false;
  if (a->format == KMOE_FMT_INT8) return true;
  const long long P = local_pairs(a);
  return a->format == KMOE_FMT_FP8_BLOCK && a->w_layout == KMOE_W_TILED && a->H <= 8192 && a->I <= 8192 &&
         (P + a->E - 1) / a->E > 10;
}

// One expert-MLP pass (gate_up + SiLU-mul, requantise, down) over `rows` rows in
// the layer's format. `x_rows` is what the first GEMM reads: quantised codes, or
// the bf16 activations themselves for KMOE_FMT_BF16.
struct MlpPass {
  int format;
  const void* x_rows;      // [*, H]
  const float* x_aux;      // row maxes / group scales (NULL for bf16)
  const int32_t* row_src;  // gather for the first GEMM (NULL: identity)
  int src_div;
  const void *w13, *w2;
  const float *w13_aux, *w2_aux;
  const int32_t* lod;
  int E, H, I, rows;
  int rows_hint;   // 0, or the rows expected to be live (an expert-parallel share): see kmoe_gemm_*_args
  uint16_t* act;   // [rows, I] bf16
  void* actq;      // [rows, I] codes
  float* act_aux;  // [rows] or [rows, I/128]
  uint16_t* out;   // [rows, H] bf16
  int w_layout;    // KMOE_W_*
  bool stream;     // INT8 + tiled weights: chunk-major codes and the weight-streaming GEMM
  int x_count;     // rows of x_rows (chunk-major addressing)
  // INT8, FP8 tail expert (folded shared expert): rows [rows, rows + tail_rows) of act/actq/out
  const void *w13_tail, *w2_tail;
  const float *w13_aux_tail, *w2_aux_tail;
  int tail_rows;
  // BF16 expert-bias branch
  const uint16_t *w13_bias, *w2_bias;
  int oai;  // 1: gate_up rows interleaved, gpt-oss activation
  float act_alpha, act_limit;
  // W4A16: group scales of the packed weights
  const uint16_t *w13_scale, *w2_scale;
  int group_size, scale_layout;
  int variant;  // INT8: kernel variant of the two GEMMs (0: from the shape)
  int act_dtype;  // INT8, BF16: KMOE_DT_* of x_rows' source, act and out (BF16: of the weights too)
  // INT8 weight-streaming path: the gate_up launch sorts the routed pairs itself (row_src is then NULL and lod is
  // what that launch writes)
  const StreamScan* scan;
  bool quant_in_gemm;  // the down launch quantises its rows itself: no launch between the two GEMMs
};

int run_gemm(const MlpPass& m, bool first, kmoe_stream_t stream) {
  const int n = first ? 2 * m.I : m.H;
  const int k = first ? m.H : m.I;
  const void* a = first ? m.x_rows : (bf16_activations(m.format) ? static_cast<const void*>(m.act) : m.actq);
  const float* a_aux = first ? m.x_aux : m.act_aux;
  const void* w = first ? m.w13 : m.w2;
  const float* w_aux = first ? m.w13_aux : m.w2_aux;
  uint16_t* y = first ? m.act : m.out;
  const int64_t ldy = first ? m.I : m.H;
  const int act = first ? KMOE_ACT_SWIGLU : KMOE_ACT_NONE;
  const int32_t* row_src = first ? m.row_src : nullptr;
  const int src_div = first ? m.src_div : 1;
  if (m.format == KMOE_FMT_INT8) {
    kmoe_gemm_i8_args g = {};
    g.a = static_cast<const int8_t*>(a);
    g.lda = k;
    g.a_max = a_aux;
    g.row_src = row_src;
    g.src_div = src_div;
    g.w = static_cast<const int8_t*>(w);
    g.w_max = w_aux;
    g.lod = m.lod;
    g.E = m.E;
    g.n = n;
    g.k = k;
    g.rows = m.rows;
    g.rows_hint = m.rows_hint;
    g.y = y;
    g.ldy = ldy;
    g.act = act;
    g.w_layout = m.w_layout;
    g.variant = m.variant;
    g.act_dtype = m.act_dtype;
    if (m.stream) {
      g.a_layout = KMOE_A_CHUNKED;
      g.a_rows = first ? m.x_count : m.rows + m.tail_rows;
    }
    if (m.tail_rows > 0) {
      g.w_tail = static_cast<const int8_t*>(first ? m.w13_tail : m.w2_tail);
      g.w_max_tail = first ? m.w13_aux_tail : m.w2_aux_tail;
      g.tail_row0 = m.rows;
      g.tail_rows = m.tail_rows;
      g.tail_src0 = first ? 0 : m.rows;  // gate_up reads token rows, down reads its own act rows
    }
    const StreamQuant quant{m.act, m.I, static_cast<int8_t*>(m.actq), m.act_aux};
    return grouped_gemm_i8_checked(&g, stream, first ? m.scan : nullptr, !first && m.quant_in_gemm ? &quant : nullptr);
  }
  if (m.format == KMOE_FMT_FP8_BLOCK) {
    kmoe_gemm_fp8_args g = {};
    g.a = static_cast<const uint8_t*>(a);
    g.lda = k;
    g.a_scale = a_aux;
    g.row_src = row_src;
    g.src_div = src_div;
    g.w = static_cast<const uint8_t*>(w);
    g.w_scale = w_aux;
    g.act_dtype = m.act_dtype;
    g.lod = m.lod;
    g.E = m.E;
    g.n = n;
    g.k = k;
    g.rows = m.rows;
    g.rows_hint = m.rows_hint;
    g.y = y;
    g.ldy = ldy;
    g.act = act;
    g.w_layout = m.w_layout;
    g.variant = m.variant;
    if (m.tail_rows > 0) {
      g.w_tail = static_cast<const uint8_t*>(first ? m.w13_tail : m.w2_tail);
      g.w_scale_tail = first ? m.w13_aux_tail : m.w2_aux_tail;
      g.tail_row0 = m.rows;
      g.tail_rows = m.tail_rows;
      g.tail_src0 = first ? 0 : m.rows;  // gate_up reads token rows, down reads its own act rows
    }
    return kmoe_grouped_gemm_fp8_block(&g, stream);
  }
  if (m.format == KMOE_FMT_W4A16) {
    kmoe_gemm_w4_args g = {};
    g.a = static_cast<const uint16_t*>(a);
    g.lda = k;
    g.row_src = row_src;
    g.src_div = src_div;
    g.w = static_cast<const uint8_t*>(w);
    g.w_scale = first ? m.w13_scale : m.w2_scale;
    g.group_size = m.group_size;
    g.scale_layout = m.scale_layout;
    g.lod = m.lod;
    g.E = m.E;
    g.n = n;
    g.k = k;
    g.rows = m.rows;
    g.rows_hint = m.rows_hint;
    g.y = y;
    g.ldy = ldy;
    g.act = act;
    g.w_layout = m.w_layout;
    g.act_dtype = m.act_dtype;
    return grouped_gemm_w4a16_checked(&g, stream, first ? m.scan : nullptr);
  }
  kmoe_gemm_bf16_args g = {};
  g.a = static_cast<const uint16_t*>(a);
  g.lda = k;
  g.row_src = row_src;
  g.src_div = src_div;
  g.w = static_cast<const uint16_t*>(w);
  g.lod = m.lod;
  g.E = m.E;
  g.n = n;
  g.k = k;
  g.rows = m.rows;
  g.rows_hint = m.rows_hint;
  g.y = y;
  g.ldy = ldy;
  g.act = first && m.oai ? KMOE_ACT_SWIGLUOAI : act;
  g.w_layout = m.w_layout;
  g.bias = first ? m.w13_bias : m.w2_bias;
  g.act_alpha = m.act_alpha;
  g.act_limit = m.act_limit;
  g.act_dtype = m.act_dtype;
  return kmoe_grouped_gemm_bf16(&g, stream);
}

template <class Mark>
int run_mlp(const MlpPass& m, kmoe_stream_t stream, Mark&& mark) {
  int rc;
  const char* whose = m.row_src || m.scan ? "routed experts" : "shared expert";
  mark(KMOE_STAGE_GEMM1, 0);
  if (tracing_kernels()) note_kernel("[gate_up, %s]", whose);
  rc = run_gemm(m, true, stream);
  if (rc) return rc;
  mark(KMOE_STAGE_GEMM1, 1);
  mark(KMOE_STAGE_QUANT2, 0);
  if (m.format == KMOE_FMT_INT8 && m.quant_in_gemm) {
    // (the down launch does it)
  } else if (m.format == KMOE_FMT_INT8) {
    const int qrows = m.rows + m.tail_rows;
    rc = m.stream ? kmoe_quant_i8_rows_chunked_dt(m.act, m.I, qrows, m.I, static_cast<int8_t*>(m.actq), m.act_aux,
                                                  m.act_dtype, stream)
                  : kmoe_quant_i8_rows_dt(m.act, m.I, qrows, m.I, static_cast<int8_t*>(m.actq), m.I, m.act_aux,
                                          m.act_dtype, stream);
  } else if (m.format == KMOE_FMT_FP8_BLOCK) {
    rc = kmoe_quant_fp8_group128_dt(m.act, m.I, m.rows + m.tail_rows, m.I, static_cast<uint8_t*>(m.actq), m.I, m.act_aux,
                                    m.act_dtype, stream);
  }
  if (rc) return rc;
  mark(KMOE_STAGE_QUANT2, 1);
  mark(KMOE_STAGE_GEMM2, 0);
  if (tracing_kernels()) note_kernel("[down, %s]", whose);
  rc = run_gemm(m, false, stream);
  if (rc) return rc;
  mark(KMOE_STAGE_GEMM2, 1);
  return KMOE_OK;
}

}  // namespace

extern "C" int kmoe_moe_workspace_layout(const kmoe_moe_args* a, kmoe_moe_layout* L) {
  if (int rc = check_shape(a)) return rc;
  KMOE_REQUIRE(L, KMOE_ERR_NULL, "moe_workspace_layout: layout is NULL");
  const size_t M = a->M, H = a->H, E = a->E, K = a->K, I = a->I, P = M * K, Is = a->I_shared;
  const bool quant = !bf16_activations(a->format);
  const bool fp8 = a->format == KMOE_FMT_FP8_BLOCK;
  const bool fold = fold_shared(a);
  const size_t R = P + (fold ? M : 0);  // rows of the routed intermediates (+ folded shared expert rows)
  const size_t Ms = fold ? 0 : (Is ? M : 0);  // rows of the separate shared-expert intermediates
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off += align_up(bytes ? bytes : 1, 256);
    return at;
  };
  L->topk_w = take(P * 4);
  L->topk_ids = take(P * 4);
  L->moe_index = take(P * 4);
  L->sorted_src = take(P * 4);
  L->expert_m = take(E * 4);
  L->lod = take((E + 1) * 4);
  L->align_ws = take(kmoe_align_workspace_bytes(static_cast<int>(P), a->E));
  L->xq = take(quant ? M * H : 0);
  L->xmax = take(quant ? M * 4 * (fp8 ? H / 128 : 1) : 0);
  L->act = take(R * I * 2);
  L->actq = take(quant ? R * I : 0);
  L->actmax = take(quant ? R * 4 * (fp8 ? I / 128 : 1) : 0);
  L->down = take(R * H * 2);
  L->sh_lod = take(2 * 4);
  L->sh_act = take(Ms * Is * 2);
  L->sh_actq = take(quant ? Ms * Is : 0);
  L->sh_actmax = take(quant ? Ms * 4 * (fp8 ? Is / 128 : 1) : 0);
  L->sh_out = take(Ms * H * 2);
  int ks = 0, mf = 0;
  if (a->w_gate && a->H % 32 == 0) router_plan(a->M, a->H, a->E_global > 0 ? a->E_global : a->E, &ks, &mf);
  L->n_logit_planes = ks;
  L->logit_planes = take(ks ? static_cast<size_t>(ks) * M * (a->E_global > 0 ? a->E_global : E) * 4 : 0);
  L->total_bytes = off;
  L->codes_chunked = use_stream_path(a) ? 1 : 0;
  return KMOE_OK;
}

namespace {

// A shared expert that cannot ride in the routed launches (another width; the fp8 decode kernels) is a chain of
// small launches that depends on the layer's input only. It runs on a stream of the library's own, forked from
// the caller's stream after the first quantisation and joined back before the combine, so that it hides under
// the routed GEMMs instead of adding its launches' latencies to the layer (DeepSeek-V3 fp8 decode: 85 us of
// 1.86 ms). Only for calls that ask for it (KMOE_FLAG_SIDE_STREAM): by default every launch goes to the caller's
// stream. One stream and two events per GPU, created on the first call that wants them and is not being
// captured (default priority, non-blocking); work of consecutive calls is ordered on it like on any stream.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  bool failed = false;
};
constexpr int kSideDevices = 64;
SideStream g_side[kSideDevices];
std::mutex g_side_mutex;

// Whether this call may use the side stream: KMOE_FLAG_SIDE_STREAM of the call, unless the environment variable
// KMOE_SIDE_STREAM (read once) says 0 (never) or 1 (always).
bool wants_side_stream(const kmoe_moe_args* a) {
  static const int forced = [] {
    const char* v = getenv("KMOE_SIDE_STREAM");
    return (v && v[0]) ? (v[0] != '0' ? 1 : 0) : -1;
  }();
  return forced >= 0 ? forced == 1 : (a->flags & KMOE_FLAG_SIDE_STREAM) != 0;
}

// The side stream of the current device, or NULL: not created yet while the caller's stream is being captured (a
// capture must not be the first to ask), or the runtime refused.
SideStream* side_stream(hipStream_t main) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kSideDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_side_mutex);
  SideStream& sd = g_side[dev];
  if (sd.stream) return &sd;
  if (sd.failed) return nullptr;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(main, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (hipStreamCreateWithFlags(&sd.stream, hipStreamNonBlocking) != hipSuccess ||
      hipEventCreateWithFlags(&sd.fork, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&sd.join, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    sd.failed = true;
    sd.stream = nullptr;
    return nullptr;
  }
  return &sd;
}

int moe_forward_impl(const kmoe_moe_args* a, void* workspace, size_t workspace_bytes, kmoe_stream_t stream,
                     bool may_fork);
void learn_static_workspace(hipStream_t stream);

}  // namespace

extern "C" int kmoe_moe_forward(const kmoe_moe_args* a, void* workspace, size_t workspace_bytes,
                                kmoe_stream_t stream) {
  learn_static_workspace(as_stream(stream));  // (so that a later captured kmoe_moe_forward_static finds the address)
  return moe_forward_impl(a, workspace, workspace_bytes, stream, true);
}

namespace {

int moe_forward_impl(const kmoe_moe_args* a, void* workspace, size_t workspace_bytes, kmoe_stream_t stream,
                     bool may_fork) {
  kmoe_moe_layout L;
  if (int rc = kmoe_moe_workspace_layout(a, &L)) return rc;
  if (a->M == 0) return KMOE_OK;
  const bool quant = !bf16_activations(a->format);
  KMOE_REQUIRE((a->logits || a->w_gate) && a->x && a->w13 && a->w2 && a->out, KMOE_ERR_NULL,
               "moe_forward: NULL tensor pointer");
  KMOE_REQUIRE(a->logits || (a->H % 32 == 0 && (reinterpret_cast<uintptr_t>(a->w_gate) & 15) == 0 &&
                             (reinterpret_cast<uintptr_t>(a->x) & 15) == 0),
               KMOE_ERR_SHAPE, "moe_forward: the router GEMM needs H %% 32 == 0 and 16-byte aligned x, w_gate");
  KMOE_REQUIRE(!quant || (a->w13_max && a->w2_max), KMOE_ERR_NULL, "moe_forward: weight max/scale pointers are NULL");
  KMOE_REQUIRE(a->format != KMOE_FMT_W4A16 || (a->w13_scale && a->w2_scale), KMOE_ERR_NULL,
               "moe_forward: group scale pointers are NULL");
  KMOE_REQUIRE(a->I_shared == 0 || (a->ws13 && a->ws2 && (!quant || (a->ws13_max && a->ws2_max))), KMOE_ERR_NULL,
               "moe_forward: shared expert pointers are NULL");
  KMOE_REQUIRE(a->scoring == KMOE_SCORE_SOFTMAX || a->scoring == KMOE_SCORE_SIGMOID, KMOE_ERR_UNSUPPORTED,
               "moe_forward: scoring=%d unknown", a->scoring);
  KMOE_REQUIRE(a->activation == 0 || a->activation == KMOE_ACT_SWIGLU ||
                   (a->activation == KMOE_ACT_SWIGLUOAI && a->format == KMOE_FMT_BF16),
               KMOE_ERR_UNSUPPORTED, "moe_forward: activation=%d (swigluoai goes with bf16 weights only)", a->activation);
  KMOE_REQUIRE((!a->w13_bias && !a->w2_bias) || a->format == KMOE_FMT_BF16, KMOE_ERR_UNSUPPORTED,
               "moe_forward: expert biases go with bf16 weights only");
  KMOE_REQUIRE(!a->w13_bias || a->activation == KMOE_ACT_SWIGLUOAI, KMOE_ERR_UNSUPPORTED,
               "moe_forward: a gate_up bias goes with the swigluoai activation");
  KMOE_REQUIRE(workspace, KMOE_ERR_WORKSPACE, "moe_forward: workspace is NULL (need %zu bytes)", L.total_bytes);
  KMOE_REQUIRE(workspace_bytes >= L.total_bytes, KMOE_ERR_WORKSPACE, "moe_forward: workspace %zu < %zu bytes",
               workspace_bytes, L.total_bytes);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, KMOE_ERR_WORKSPACE,
               "moe_forward: workspace must be 256-byte aligned");

  char* ws = static_cast<char*>(workspace);
  auto at = [&](size_t off) { return static_cast<void*>(ws + off); };
  float* topk_w = static_cast<float*>(at(L.topk_w));
  int32_t* topk_ids = static_cast<int32_t*>(at(L.topk_ids));
  int32_t* moe_index = static_cast<int32_t*>(at(L.moe_index));
  int32_t* sorted_src = static_cast<int32_t*>(at(L.sorted_src));
  int32_t* lod = static_cast<int32_t*>(at(L.lod));
  const int M = a->M, H = a->H, E = a->E, K = a->K, I = a->I, P = M * K;
  const int Eg = a->E_global > 0 ? a->E_global : E;  // experts the routing runs over (an expert-parallel share: more than E)
  int rc = KMOE_OK;
  auto mark = [&](int stage, int end) {
    if (!a->stage_events) return;
    void* ev = a->stage_events[2 * stage + end];
    if (ev) (void)hipEventRecord(static_cast<hipEvent_t>(ev), as_stream(stream));
  };

  // 0. router logits if the caller handed over the gate weight instead: split-K partial planes,
  //    which the routing kernel adds up as it loads them (timed as part of the routing stage)
  const bool stream_mode = use_stream_path(a);
  bool quant_done = false;
  mark(KMOE_STAGE_ROUTING, 0);
  const float* logits = a->logits;
  int planes = 1;
  size_t plane_stride = 0;
  if (!logits) {
    int mf = 0;
    router_plan(M, H, Eg, &planes, &mf);
    float* buf = static_cast<float*>(at(L.logit_planes));
    plane_stride = static_cast<size_t>(M) * Eg;
    rc = router_gemm_planes(a->x, H, a->w_gate, M, H, Eg, buf, plane_stride, Eg, planes, mf, as_stream(stream),
                            a->act_dtype == KMOE_DT_F16);
    if (rc) return rc;
    logits = buf;
  }
  // 1. routing; on the int8 decode path together with step 3 (independent work, one launch)
  if (a->format == KMOE_FMT_INT8) {
    rc = fused_route_quant_i8(logits, planes, plane_stride, a->bias, M, Eg, K, a->scoring == KMOE_SCORE_SIGMOID, a->renormalize, a->n_group,
                              a->topk_group, a->routed_scale, topk_w, topk_ids, a->x, H, static_cast<int8_t*>(at(L.xq)),
                              static_cast<float*>(at(L.xmax)), stream_mode ? 1 : 0, a->act_dtype == KMOE_DT_F16,
                              as_stream(stream));
    if (rc < 0) return rc;
    quant_done = rc == KMOE_OK;
    rc = KMOE_OK;
  }
  if (!quant_done && planes > 1) {  // the stand-alone routing kernels take finished logits: add the planes into plane 0
    rc = router_reduce(logits, plane_stride, planes, M, Eg, static_cast<float*>(at(L.logit_planes)), Eg, as_stream(stream));
    if (rc) return rc;
  }
  if (quant_done) {
    // both done
  } else if (a->scoring == KMOE_SCORE_SOFTMAX) {
    rc = kmoe_softmax_topk(logits, M, Eg, K, a->renormalize, topk_w, topk_ids, stream);
  } else {
    rc = kmoe_sigmoid_group_topk_norm(logits, a->bias, M, Eg, K, a->n_group, a->topk_group, a->routed_scale, topk_w,
                                      topk_ids, stream);
  }
  if (rc) return rc;
  mark(KMOE_STAGE_ROUTING, 1);
  // 2. stable sort of the routed pairs by expert. On the weight-streaming path (a few rows per expert) the gate_up
  // launch does it in its prologue and writes the same four arrays: one launch and its round trips less
  // (Qwen3 decode: 4.8 us of 125). Not for an expert-parallel share (pairs of other ranks' experts get no row).
  mark(KMOE_STAGE_ALIGN, 0);
  const StreamScan scan{topk_ids, P, lod, static_cast<int32_t*>(at(L.expert_m)), moe_index, sorted_src};
  const bool streams = stream_mode || (a->format == KMOE_FMT_W4A16 && a->w_layout == KMOE_W_TILED &&
                                       w4_gate_up_streams(P, 0, E, H));
  const bool scan_in_gemm = streams && Eg == E && a->first_expert == 0 && P <= kStreamScanMaxPairs &&
                            M <= kStreamScanMaxRows && scan_allowed();
  if (!scan_in_gemm) {
    rc = kmoe_align_local(topk_ids, P, E, a->first_expert, moe_index, sorted_src, static_cast<int32_t*>(at(L.expert_m)), lod,
                          at(L.align_ws), kmoe_align_workspace_bytes(P, E), stream);
    if (rc) return rc;
  }
  mark(KMOE_STAGE_ALIGN, 1);
  // 3. quantise each TOKEN row once (the reference quantises the K-times expanded copy; same values)
  mark(KMOE_STAGE_QUANT1, 0);
  const void* x_rows = a->x;
  if (quant_done) {
    x_rows = at(L.xq);
  } else if (a->format == KMOE_FMT_INT8) {
    rc = stream_mode ? kmoe_quant_i8_rows_chunked_dt(a->x, H, M, H, static_cast<int8_t*>(at(L.xq)),
                                                     static_cast<float*>(at(L.xmax)), a->act_dtype, stream)
                     : kmoe_quant_i8_rows_dt(a->x, H, M, H, static_cast<int8_t*>(at(L.xq)), H,
                                             static_cast<float*>(at(L.xmax)), a->act_dtype, stream);
    x_rows = at(L.xq);
  } else if (a->format == KMOE_FMT_FP8_BLOCK) {
    rc = kmoe_quant_fp8_group128_dt(a->x, H, M, H, static_cast<uint8_t*>(at(L.xq)), H, static_cast<float*>(at(L.xmax)),
                                    a->act_dtype, stream);
    x_rows = at(L.xq);
  }
  if (rc) return rc;
  mark(KMOE_STAGE_QUANT1, 1);

  // 4-6. routed experts: gate_up GEMM (+SiLU-mul, rows gathered through the sort), requantise, down GEMM
  MlpPass routed = {};
  routed.format = a->format;
  routed.x_rows = x_rows;
  routed.x_aux = quant ? static_cast<const float*>(at(L.xmax)) : nullptr;
  routed.row_src = scan_in_gemm ? nullptr : sorted_src;
  routed.scan = scan_in_gemm ? &scan : nullptr;
  routed.src_div = K;
  routed.w13 = a->w13;
  routed.w2 = a->w2;
  routed.w13_aux = a->w13_max;
  routed.w2_aux = a->w2_max;
  routed.lod = lod;
  routed.E = E;
  routed.H = H;
  routed.I = I;
  routed.rows = P;
  routed.rows_hint = a->E_global > E ? static_cast<int>(local_pairs(a)) : 0;
  routed.act = static_cast<uint16_t*>(at(L.act));
  routed.actq = at(L.actq);
  routed.act_aux = static_cast<float*>(at(L.actmax));
  routed.out = static_cast<uint16_t*>(at(L.down));
  routed.w_layout = a->w_layout;
  routed.w13_scale = a->w13_scale;
  routed.w2_scale = a->w2_scale;
  routed.group_size = a->group_size;
  routed.scale_layout = a->w_scale_layout;
  routed.act_dtype = a->act_dtype;
  if (a->format == KMOE_FMT_BF16) {
    routed.w13_bias = a->w13_bias;
    routed.w2_bias = a->w2_bias;
    routed.oai = a->activation == KMOE_ACT_SWIGLUOAI;
    routed.act_alpha = a->act_alpha;
    routed.act_limit = a->act_limit;
  }
  routed.stream = stream_mode;
  // Down projections up to 1024 wide quantise their rows in the launch's prologue (Qwen3 decode: one 4.5 us launch
  // and its gap less); wider rows would not fit the workgroup's LDS copy next to three resident workgroups per CU.
  routed.quant_in_gemm = stream_mode && I <= kStreamQuantMaxK && quant_in_gemm_allowed();
  routed.x_count = M;
  if (a->format == KMOE_FMT_INT8 && !stream_mode && a->w_layout == KMOE_W_TILED && a->tile_variant >= 5 &&
      a->tile_variant <= 22 && (local_pairs(a) + E - 1) / E > 10 && H >= 128 && I >= 128)
    routed.variant = a->tile_variant;
  const int tv = a->tile_variant;
  if (a->format == KMOE_FMT_FP8_BLOCK && a->w_layout == KMOE_W_TILED && (local_pairs(a) + E - 1) / E > 10 &&
      (tv == 5 || tv == 6 || tv == 8 || (tv >= 11 && tv <= 14) || (tv >= 17 && tv <= 19)))
    routed.variant = tv;
  const bool fold = fold_shared(a);
  if (fold) {
    routed.w13_tail = a->ws13;
    routed.w2_tail = a->ws2;
    routed.w13_aux_tail = a->ws13_max;
    routed.w2_aux_tail = a->ws2_max;
    routed.tail_rows = M;
  }
  // 7. dense shared expert on all M rows: the grouped GEMM with a single expert whose lod is {0, M}. With a side
  // stream it is enqueued there BEFORE the routed pass (it reads x / its codes only) and joined after it.
  const uint16_t* shared_out = fold ? routed.out + static_cast<size_t>(P) * H : nullptr;
  const bool own_pass = a->I_shared > 0 && !fold;
  SideStream* side =
      own_pass && may_fork && !a->stage_events && wants_side_stream(a) ? side_stream(as_stream(stream)) : nullptr;
  auto shared_pass = [&](kmoe_stream_t st) -> int {
    int32_t* dense_lod = static_cast<int32_t*>(at(L.sh_lod));
    int rcs = fill_dense_lod(dense_lod, stream_mode ? 0 : M, as_stream(st));  // (streaming path: see below)
    if (rcs) return rcs;
    MlpPass sh = routed;
    // the expert-bias branch belongs to the routed experts only: a dense shared MLP has no per-expert
    // bias and uses the plain SiLU-mul over [gate | up] rows
    sh.w13_bias = nullptr;
    sh.w2_bias = nullptr;
    sh.oai = 0;
    sh.tail_rows = 0;
    sh.row_src = nullptr;
    sh.scan = nullptr;
    sh.quant_in_gemm = false;
    sh.src_div = 1;
    sh.w13 = a->ws13;
    sh.w2 = a->ws2;
    sh.w_layout = a->ws_layout;
    sh.w13_aux = a->ws13_max;
    sh.w2_aux = a->ws2_max;
    sh.lod = dense_lod;
    sh.E = 1;
    sh.I = a->I_shared;
    sh.rows = M;
    sh.rows_hint = 0;
    sh.variant = 0;  // (a tuning variant of the routed GEMMs does not apply to the dense pass)
    if (stream_mode) {
      // On the weight-streaming path a dense expert is best run as the launch's TAIL expert: the kernel cuts
      // a tail's rows into 16- or 32-row slices for as many workgroups, while one routed expert with M rows
      // is one column of workgroups that walks its rows in passes (measured at 64 tokens, hidden 2048:
      // the pass of a shared expert of intermediate size 1536 took 56 us, now 22; of size 6144, 97 -> 36 us).
      // The routed expert list is then one expert without rows.
      sh.rows = 0;
      sh.tail_rows = M;
      sh.w13_tail = a->ws13;
      sh.w2_tail = a->ws2;
      sh.w13_aux_tail = a->ws13_max;
      sh.w2_aux_tail = a->ws2_max;
      sh.variant = M <= 128 ? 1 : (M <= 256 ? 2 : 4);  // rows per slice: 16, 32, 64
    }
    sh.act = static_cast<uint16_t*>(at(L.sh_act));
    sh.actq = at(L.sh_actq);
    sh.act_aux = static_cast<float*>(at(L.sh_actmax));
    sh.out = static_cast<uint16_t*>(at(L.sh_out));
    rcs = run_mlp(sh, st, [](int, int) {});
    if (rcs) return rcs;
    shared_out = sh.out;
    return KMOE_OK;
  };
  if (side) {
    // (record and wait are one step under the lock: the events are shared by every caller on this GPU, and a
    // wait refers to the event's latest record)
    auto hand_over = [](hipEvent_t ev, hipStream_t from, hipStream_t to) {
      std::lock_guard<std::mutex> lock(g_side_mutex);
      hipError_t err = hipEventRecord(ev, from);
      if (err == hipSuccess) err = hipStreamWaitEvent(to, ev, 0);
      return err;
    };
    hipError_t e = hand_over(side->fork, as_stream(stream), side->stream);
    KMOE_REQUIRE(e == hipSuccess, KMOE_ERR_LAUNCH, "moe_forward: fork to the side stream: %s", hipGetErrorString(e));
    const int rc_side = shared_pass(side->stream);
    rc = rc_side ? rc_side : run_mlp(routed, stream, mark);
    // joined in any case, after the routed pass is in the caller's stream: a captured side stream must come back
    // to the stream it forked from
    e = hand_over(side->join, side->stream, as_stream(stream));
    if (rc) return rc;
    KMOE_REQUIRE(e == hipSuccess, KMOE_ERR_LAUNCH, "moe_forward: join of the side stream: %s", hipGetErrorString(e));
  } else {
    rc = run_mlp(routed, stream, mark);
    if (rc) return rc;
  }
  mark(KMOE_STAGE_SHARED, 0);
  if (own_pass && !side) {
    rc = shared_pass(stream);
    if (rc) return rc;
  }
  mark(KMOE_STAGE_SHARED, 1);
  // 8. weighted combine (+ caller epilogue)
  mark(KMOE_STAGE_COMBINE, 0);
  // shared_scale == 0 (a zeroed field) means 1
  rc = kmoe_combine_dt(static_cast<uint16_t*>(at(L.down)), H, moe_index, topk_w, nullptr, M, K, H, a->out_scale,
                       shared_out, H, a->shared_scale == 0.0f ? 1.0f : a->shared_scale, a->out, H, a->act_dtype,
                       stream);
  mark(KMOE_STAGE_COMBINE, 1);
  return rc;
}

}  // namespace

// ---- the layer for callers that cannot hand over a workspace -------------------------------
// kmoe_moe_forward with its workspace in a file-scope device array. The array's name is only a
// host-side handle: its device address is asked for once per GPU (each GPU holds its own copy at
// its own address) and that address is what the kernels get.
static __device__ __align__(256) unsigned char scratch[KMOE_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current GPU. It is looked up once per GPU, by the first call whose stream is
// not being captured (the lookup is not a stream operation and may be what makes the runtime load the array); a
// captured call that finds it missing is refused.
int static_workspace(void** out, hipStream_t stream) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail(KMOE_ERR_LAUNCH, "moe_forward_static: hipGetDevice: %s", hipGetErrorString(err));
  KMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, KMOE_ERR_UNSUPPORTED, "moe_forward_static: device %d (at most %d)", dev,
               kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
    KMOE_REQUIRE(cap == hipStreamCaptureStatusNone, KMOE_ERR_UNSUPPORTED,
                 "moe_forward_static: the built-in buffer's address on device %d is not known yet and this stream is "
                 "being captured: call kmoe_moe_forward or kmoe_moe_forward_static once outside the capture first",
                 dev);
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !p)
      return fail(KMOE_ERR_LAUNCH, "moe_forward_static: hipGetSymbolAddress on device %d: %s", dev,
                  hipGetErrorString(err));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return KMOE_OK;
}

// Looks the address up on behalf of later captured calls; failures (a capture in progress, a runtime error) are
// left for kmoe_moe_forward_static to report.
void learn_static_workspace(hipStream_t stream) {
  static thread_local int known_dev = -1;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if (dev == known_dev) return;
  void* p = nullptr;
  char saved[sizeof(g_error)];
  memcpy(saved, g_error, sizeof(saved));
  if (static_workspace(&p, stream) == KMOE_OK) known_dev = dev;
  else memcpy(g_error, saved, sizeof(saved));  // not this call's failure
}

}  // namespace

extern "C" int kmoe_moe_forward_static(const kmoe_moe_args* a, kmoe_stream_t stream) {
  kmoe_moe_layout L;
  if (int rc = kmoe_moe_workspace_layout(a, &L)) return rc;
  KMOE_REQUIRE(L.total_bytes <= static_cast<size_t>(KMOE_STATIC_WORKSPACE_BYTES), KMOE_ERR_WORKSPACE,
               "moe_forward_static: this shape needs %zu bytes of scratch, the built-in buffer holds %zu "
               "(use kmoe_moe_forward with a workspace of the caller's)",
               L.total_bytes, static_cast<size_t>(KMOE_STATIC_WORKSPACE_BYTES));
  void* ws = nullptr;
  if (int rc = static_workspace(&ws, as_stream(stream))) return rc;
  // every slot of the layout is written by the stage that owns it before anything reads it, so
  // the last call's contents need no clearing
  return moe_forward_impl(a, ws, KMOE_STATIC_WORKSPACE_BYTES, stream, false);  // no second stream: nothing is created here
}
