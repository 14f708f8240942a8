// Host side of libkmoe: error state, and the fused W8A8 layer call that strings
// the stage kernels together on one stream out of one caller-owned workspace.
#include <cstdarg>
#include <cstdio>

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

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return KMOE_OK;
  return fail(KMOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
}

}  // namespace kmoe

using namespace kmoe;

extern "C" const char* kmoe_last_error(void) { return g_error; }
extern "C" const char* kmoe_version(void) { return "kmoe 0.1 gfx950"; }

namespace {

int check_shape(const kmoe_w8a8_args* a) {
  KMOE_REQUIRE(a, KMOE_ERR_NULL, "forward_w8a8: args is NULL");
  KMOE_REQUIRE(a->M >= 0 && a->H >= 16 && a->E >= 1 && a->K >= 1 && a->I >= 16, KMOE_ERR_SHAPE,
               "forward_w8a8: M=%d H=%d E=%d K=%d I=%d", a->M, a->H, a->E, a->K, a->I);
  KMOE_REQUIRE(a->H % 16 == 0 && a->I % 16 == 0, KMOE_ERR_SHAPE, "forward_w8a8: H=%d and I=%d must be multiples of 16",
               a->H, a->I);
  KMOE_REQUIRE(a->K <= a->E && a->K <= 64 && a->E <= 1024, KMOE_ERR_SHAPE, "forward_w8a8: K=%d E=%d out of range", a->K,
               a->E);
  KMOE_REQUIRE(a->I_shared >= 0 && a->I_shared % 16 == 0, KMOE_ERR_SHAPE,
               "forward_w8a8: I_shared=%d must be a non-negative multiple of 16", a->I_shared);
  KMOE_REQUIRE(static_cast<long long>(a->M) * a->K <= (1 << 24), KMOE_ERR_SHAPE, "forward_w8a8: M*K too large");
  return KMOE_OK;
}

}  // namespace

extern "C" int kmoe_w8a8_workspace_layout(const kmoe_w8a8_args* a, kmoe_w8a8_layout* L) {
  if (int rc = check_shape(a)) return rc;
  KMOE_REQUIRE(L, KMOE_ERR_NULL, "w8a8_workspace_layout: layout is NULL");
  const size_t M = a->M, H = a->H, E = a->E, K = a->K, I = a->I, P = M * K, Is = a->I_shared;
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
  L->xq = take(M * H);
  L->xmax = take(M * 4);
  L->act = take(P * I * 2);
  L->actq = take(P * I);
  L->actmax = take(P * 4);
  L->down = take(P * H * 2);
  L->sh_lod = take(2 * 4);
  L->sh_act = take(M * Is * 2);
  L->sh_actq = take(M * Is);
  L->sh_actmax = take(M * 4);
  L->sh_out = take(Is ? M * H * 2 : 0);
  L->total_bytes = off;
  return KMOE_OK;
}

extern "C" int kmoe_forward_w8a8(const kmoe_w8a8_args* a, void* workspace, size_t workspace_bytes,
                                 kmoe_stream_t stream) {
  kmoe_w8a8_layout L;
  if (int rc = kmoe_w8a8_workspace_layout(a, &L)) return rc;
  if (a->M == 0) return KMOE_OK;
  KMOE_REQUIRE(a->logits && a->x && a->w13 && a->w13_max && a->w2 && a->w2_max && a->out, KMOE_ERR_NULL,
               "forward_w8a8: NULL tensor pointer");
  KMOE_REQUIRE(a->I_shared == 0 || (a->ws13 && a->ws13_max && a->ws2 && a->ws2_max), KMOE_ERR_NULL,
               "forward_w8a8: shared expert pointers are NULL");
  KMOE_REQUIRE(a->scoring == KMOE_SCORE_SOFTMAX || a->scoring == KMOE_SCORE_SIGMOID, KMOE_ERR_UNSUPPORTED,
               "forward_w8a8: scoring=%d unknown", a->scoring);
  KMOE_REQUIRE(workspace, KMOE_ERR_WORKSPACE, "forward_w8a8: workspace is NULL (need %zu bytes)", L.total_bytes);
  KMOE_REQUIRE(workspace_bytes >= L.total_bytes, KMOE_ERR_WORKSPACE, "forward_w8a8: workspace %zu < %zu bytes",
               workspace_bytes, L.total_bytes);
  KMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, KMOE_ERR_WORKSPACE,
               "forward_w8a8: workspace must be 256-byte aligned");

  char* ws = static_cast<char*>(workspace);
  auto at = [&](size_t off) { return static_cast<void*>(ws + off); };
  float* topk_w = static_cast<float*>(at(L.topk_w));
  int32_t* topk_ids = static_cast<int32_t*>(at(L.topk_ids));
  int32_t* moe_index = static_cast<int32_t*>(at(L.moe_index));
  int32_t* sorted_src = static_cast<int32_t*>(at(L.sorted_src));
  int32_t* lod = static_cast<int32_t*>(at(L.lod));
  int8_t* xq = static_cast<int8_t*>(at(L.xq));
  float* xmax = static_cast<float*>(at(L.xmax));
  const int M = a->M, H = a->H, E = a->E, K = a->K, I = a->I, P = M * K;
  int rc;
  auto mark = [&](int stage, int end) {
    if (!a->stage_events) return;
    void* ev = a->stage_events[2 * stage + end];
    if (ev) (void)hipEventRecord(static_cast<hipEvent_t>(ev), as_stream(stream));
  };

  // 1. routing
  mark(KMOE_STAGE_ROUTING, 0);
  if (a->scoring == KMOE_SCORE_SOFTMAX) {
    rc = kmoe_softmax_topk(a->logits, M, E, K, a->renormalize, topk_w, topk_ids, stream);
  } else {
    rc = kmoe_sigmoid_group_topk_norm(a->logits, a->bias, M, E, K, a->n_group, a->topk_group, a->routed_scale, topk_w,
                                      topk_ids, stream);
  }
  if (rc) return rc;
  mark(KMOE_STAGE_ROUTING, 1);
  // 2. stable sort of the routed pairs by expert
  mark(KMOE_STAGE_ALIGN, 0);
  rc = kmoe_align(topk_ids, P, E, moe_index, sorted_src, static_cast<int32_t*>(at(L.expert_m)), lod, at(L.align_ws),
                  kmoe_align_workspace_bytes(P, E), stream);
  if (rc) return rc;
  mark(KMOE_STAGE_ALIGN, 1);
  mark(KMOE_STAGE_QUANT1, 0);
  // 3. one int8 row per TOKEN (the reference quantises the K-times expanded copy; same values)
  rc = kmoe_quant_i8_rows(a->x, H, M, H, xq, H, xmax, stream);
  if (rc) return rc;
  mark(KMOE_STAGE_QUANT1, 1);
  mark(KMOE_STAGE_GEMM1, 0);
  // 4. gate_up GEMM with dequant + SiLU-mul epilogue; rows gathered through the sort
  kmoe_gemm_i8_args g1 = {};
  g1.a = xq;
  g1.lda = H;
  g1.a_max = xmax;
  g1.row_src = sorted_src;
  g1.src_div = K;
  g1.w = a->w13;
  g1.w_max = a->w13_max;
  g1.lod = lod;
  g1.E = E;
  g1.n = 2 * I;
  g1.k = H;
  g1.rows = P;
  g1.y = static_cast<uint16_t*>(at(L.act));
  g1.ldy = I;
  g1.act = KMOE_ACT_SWIGLU;
  rc = kmoe_grouped_gemm_i8(&g1, stream);
  if (rc) return rc;
  mark(KMOE_STAGE_GEMM1, 1);
  mark(KMOE_STAGE_QUANT2, 0);
  // 5. requantise the activation rows
  rc = kmoe_quant_i8_rows(static_cast<uint16_t*>(at(L.act)), I, P, I, static_cast<int8_t*>(at(L.actq)), I,
                          static_cast<float*>(at(L.actmax)), stream);
  if (rc) return rc;
  mark(KMOE_STAGE_QUANT2, 1);
  mark(KMOE_STAGE_GEMM2, 0);
  // 6. down GEMM
  kmoe_gemm_i8_args g2 = {};
  g2.a = static_cast<int8_t*>(at(L.actq));
  g2.lda = I;
  g2.a_max = static_cast<float*>(at(L.actmax));
  g2.w = a->w2;
  g2.w_max = a->w2_max;
  g2.lod = lod;
  g2.E = E;
  g2.n = H;
  g2.k = I;
  g2.rows = P;
  g2.y = static_cast<uint16_t*>(at(L.down));
  g2.ldy = H;
  g2.act = KMOE_ACT_NONE;
  rc = kmoe_grouped_gemm_i8(&g2, stream);
  if (rc) return rc;
  mark(KMOE_STAGE_GEMM2, 1);

  // 7. dense shared expert on all M rows: one "expert" whose lod is [0, M]
  mark(KMOE_STAGE_SHARED, 0);
  const uint16_t* shared_out = nullptr;
  if (a->I_shared > 0) {
    const int Is = a->I_shared;
    // the dense call is the grouped GEMM with a single expert whose lod is {0, M}
    int32_t* dense_lod = static_cast<int32_t*>(at(L.sh_lod));
    rc = fill_dense_lod(dense_lod, M, as_stream(stream));
    if (rc) return rc;
    kmoe_gemm_i8_args s1 = {};
    s1.a = xq;
    s1.lda = H;
    s1.a_max = xmax;
    s1.w = a->ws13;
    s1.w_max = a->ws13_max;
    s1.lod = dense_lod;
    s1.E = 1;
    s1.n = 2 * Is;
    s1.k = H;
    s1.rows = M;
    s1.y = static_cast<uint16_t*>(at(L.sh_act));
    s1.ldy = Is;
    s1.act = KMOE_ACT_SWIGLU;
    rc = kmoe_grouped_gemm_i8(&s1, stream);
    if (rc) return rc;
    rc = kmoe_quant_i8_rows(static_cast<uint16_t*>(at(L.sh_act)), Is, M, Is, static_cast<int8_t*>(at(L.sh_actq)), Is,
                            static_cast<float*>(at(L.sh_actmax)), stream);
    if (rc) return rc;
    kmoe_gemm_i8_args s2 = {};
    s2.a = static_cast<int8_t*>(at(L.sh_actq));
    s2.lda = Is;
    s2.a_max = static_cast<float*>(at(L.sh_actmax));
    s2.w = a->ws2;
    s2.w_max = a->ws2_max;
    s2.lod = dense_lod;
    s2.E = 1;
    s2.n = H;
    s2.k = Is;
    s2.rows = M;
    s2.y = static_cast<uint16_t*>(at(L.sh_out));
    s2.ldy = H;
    s2.act = KMOE_ACT_NONE;
    rc = kmoe_grouped_gemm_i8(&s2, stream);
    if (rc) return rc;
    shared_out = static_cast<uint16_t*>(at(L.sh_out));
  }
  mark(KMOE_STAGE_SHARED, 1);
  // 8. weighted combine (+ caller epilogue)
  mark(KMOE_STAGE_COMBINE, 0);
  rc = kmoe_combine(static_cast<uint16_t*>(at(L.down)), H, moe_index, topk_w, nullptr, M, K, H, a->out_scale,
                      shared_out, H, a->out, H, stream);
  mark(KMOE_STAGE_COMBINE, 1);
  return rc;
}
