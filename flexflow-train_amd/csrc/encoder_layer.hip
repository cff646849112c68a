// One transformer encoder layer (forward + backward) as a sequence of the
// operator entry points, in the order the reference's local executor would
// run the layer's ops (forward in topological order, backward in reverse).
// Host code only: every arithmetic step is one of the ffk_* kernels.
#include "ffk_common.h"
#include "fused_ops.h"
#include "colreduce.h"
#include "gemm.h"
#include <stdlib.h>

namespace ffk {

struct LayerWs {
  // forward activations kept for backward
  size_t h1, mean1, rstd1, attn_out, attn_drop, x1, h2, mean2, rstd2;
  size_t f1, act1, act1_drop, f2, f2_drop, pre2;
  // backward scratch
  size_t g_f2, g_act1_drop, g_act1, g_f1, g_h2, g_x1, g_attn, g_h1, g_tmp;
  size_t mha_reserve, ln_ws, ln_ws_b, lin_ws, lin_ws_b;  // two of each: their column sums are reduced together at the end
  size_t total;
};

static size_t a256(size_t x) { return (x + 255) & ~(size_t)255; }

static ffk_mha_desc_t mha_desc(ffk_encoder_layer_desc_t const *d) {
  ffk_mha_desc_t m;
  int64_t const hd = d->d_model / d->heads;
  m.num_samples = d->batch;
  m.num_heads = d->heads;
  m.q_size = m.k_size = m.v_size = d->d_model;
  m.q_proj_size = m.k_proj_size = m.v_proj_size = hd;
  m.o_proj_size = d->d_model;
  m.qo_seq_length = m.kv_seq_length = d->seq;
  m.scale = d->attn_scale;
  m.causal = d->causal;
  return m;
}

static LayerWs layout(ffk_encoder_layer_desc_t const *d, int dtype) {
  LayerWs L;
  size_t const es = dtype_size(dtype);
  size_t const T = (size_t)(d->batch * d->seq);
  size_t const td = a256(T * (size_t)d->d_model * es);
  size_t const tf = a256(T * (size_t)d->d_ff * es);
  size_t const tr = a256(T * sizeof(float));
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += bytes; return o; };
  L.h1 = take(td); L.mean1 = take(tr); L.rstd1 = take(tr);
  L.attn_out = take(td); L.attn_drop = take(td); L.x1 = take(td);
  L.h2 = take(td); L.mean2 = take(tr); L.rstd2 = take(tr);
  L.f1 = take(tf); L.act1 = take(tf); L.act1_drop = take(tf);
  L.f2 = take(td); L.f2_drop = take(td); L.pre2 = take(td);
  L.g_f2 = take(td); L.g_act1_drop = take(tf); L.g_act1 = take(tf); L.g_f1 = take(tf);
  L.g_h2 = take(td); L.g_x1 = take(td); L.g_attn = take(td); L.g_h1 = take(td); L.g_tmp = take(td);
  ffk_mha_desc_t m = mha_desc(d);
  L.mha_reserve = take(a256(ffk_mha_reserve_bytes(&m, dtype)));
  L.ln_ws = take(a256(ffk_layer_norm_backward_workspace_bytes((int64_t)T, d->d_model)));
  L.ln_ws_b = take(a256(ffk_layer_norm_backward_workspace_bytes((int64_t)T, d->d_model)));
  size_t l1 = ffk_linear_backward_workspace_bytes(dtype, FFK_ACT_RELU, 1, (int64_t)T, d->d_ff);
  size_t l2 = ffk_linear_backward_workspace_bytes(dtype, FFK_ACT_NONE, 1, (int64_t)T, d->d_model);
  L.lin_ws = take(a256(l1 > l2 ? l1 : l2));
  L.lin_ws_b = take(a256(l1 > l2 ? l1 : l2));
  L.total = off;
  return L;
}

static int check_layer(char const *who, int dtype, ffk_encoder_layer_desc_t const *d) {
  FFK_REQUIRE(d != nullptr, "%s: NULL descriptor", who);
  FFK_REQUIRE(dtype == FFK_BF16, "%s: dtype %d not supported (bf16 only)", who, dtype);
  FFK_REQUIRE(d->batch > 0 && d->seq > 0 && d->d_model > 0 && d->heads > 0 && d->d_ff > 0,
              "%s: non-positive size", who);
  FFK_REQUIRE(d->d_model % d->heads == 0, "%s: d_model not divisible by heads", who);
  FFK_REQUIRE(d->activation == FFK_ACT_RELU || d->activation == FFK_ACT_GELU,
              "%s: Unhandled activation function %d", who, d->activation);
  return FFK_OK;
}

// FFK_OPTION_LAYER_UNFUSED != 0 runs every op of the layer as its own kernel
// (the plain operator sequence); the default fuses neighbours where the result
// is bit-identical.  For tests that compare the two.
static bool layer_fusion_enabled() { return option(FFK_OPTION_LAYER_UNFUSED) == 0; }

// out = residual + dropout(in): one fused pass when possible, else dropout
// into `scratch` followed by the element-wise add.
static int dropout_then_add(ffk_stream_t st, int dtype, void const *in, void *scratch,
                            void const *residual, void *out, int64_t n, float rate,
                            uint64_t seed) {
  if (layer_fusion_enabled() && dropout_fusable(dtype, in, residual, out, n, 0)) {
    return dropout_add_residual(as_stream(st), dtype, in, residual, out, n, rate, seed, 0);
  }
  int rc = ffk_dropout_forward(st, dtype, in, scratch, n, rate, seed, 0);
  if (rc != FFK_OK) return rc;
  return ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, scratch, residual, out, n, n, n);
}

#define FFK_TRY(expr)                                                          \
  do {                                                                         \
    int rc__ = (expr);                                                         \
    if (rc__ != FFK_OK) return rc__;                                           \
  } while (0)

}  // namespace ffk

using namespace ffk;

extern "C" size_t ffk_encoder_layer_workspace_bytes(ffk_encoder_layer_desc_t const *d, int dtype) {
  if (d == nullptr || dtype_size(dtype) == 0) return 0;
  return layout(d, dtype).total;
}

extern "C" int ffk_encoder_layer_forward(ffk_stream_t st, int dtype,
                                         ffk_encoder_layer_desc_t const *d,
                                         ffk_encoder_layer_params_t const *w,
                                         void const *x, void *y, void *workspace,
                                         size_t workspace_bytes) {
  FFK_TRY(check_layer("encoder_layer_forward", dtype, d));
  FFK_REQUIRE(w && x && y, "encoder_layer_forward: NULL argument");
  LayerWs L = layout(d, dtype);
  if (workspace == nullptr || workspace_bytes < L.total) {
    return fail(FFK_ERR_WORKSPACE, "encoder_layer_forward: workspace of %zu bytes needed, %zu given",
                L.total, workspace_bytes);
  }
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  int64_t const T = d->batch * d->seq, E = d->d_model, F = d->d_ff;
  ffk_mha_desc_t m = mha_desc(d);
  float const p = d->dropout_rate;
  bool const gelu = d->activation == FFK_ACT_GELU;
  auto mean = [&](size_t o) { return reinterpret_cast<float *>(ws + o); };

  void const *attn_in = x;
  if (d->pre_layer_norm) {
    FFK_TRY(ffk_layer_norm_forward(st, dtype, x, ws + L.h1, w->ln1_gamma, w->ln1_beta,
                                   mean(L.mean1), mean(L.rstd1), T, E, d->ln_eps));
    attn_in = ws + L.h1;
  }
  FFK_TRY(ffk_mha_forward(st, dtype, &m, attn_in, attn_in, attn_in, w->attn_weight, ws + L.attn_out,
                          ws + L.mha_reserve, L.ln_ws - L.mha_reserve));
  void const *attn_res = ws + L.attn_out;
  void *ffn_in;
  if (d->pre_layer_norm) {
    // x1 = dropout(attn) + x (the reference's encoder applies no dropout here)
    int rc = FFK_ERR_UNSUPPORTED;
    if (layer_fusion_enabled()) {
      rc = dropout_add_layer_norm_forward(as_stream(st), dtype, ws + L.attn_out, x, ws + L.x1, ws + L.h2, w->ln2_gamma,
                                          w->ln2_beta, mean(L.mean2), mean(L.rstd2), T, E, d->ln_eps, p, d->seed + 0, 0);
      if (rc != FFK_OK && rc != FFK_ERR_UNSUPPORTED) return rc;
    }
    if (rc == FFK_ERR_UNSUPPORTED) {
      FFK_TRY(dropout_then_add(st, dtype, ws + L.attn_out, ws + L.attn_drop, x, ws + L.x1, T * E, p, d->seed + 0));
      FFK_TRY(ffk_layer_norm_forward(st, dtype, ws + L.x1, ws + L.h2, w->ln2_gamma, w->ln2_beta,
                                     mean(L.mean2), mean(L.rstd2), T, E, d->ln_eps));
    }
    ffn_in = ws + L.h2;
  } else {
    // h1 = attn + x ; x1 = LN1(h1)
    FFK_TRY(ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, attn_res, x, ws + L.h1, T * E, T * E, T * E));
    FFK_TRY(ffk_layer_norm_forward(st, dtype, ws + L.h1, ws + L.x1, w->ln1_gamma, w->ln1_beta,
                                   mean(L.mean1), mean(L.rstd1), T, E, d->ln_eps));
    ffn_in = ws + L.x1;
  }
  // dense(d_ff, activation) -> dropout -> dense(d_model) -> dropout
  if (gelu) {
    // (The GEMM could apply GELU and the dropout while it stores its tile --
    // linear_gelu_dropout_forward -- but every CU reaches the store of its one
    // tile at the same time, nothing overlaps the extra arithmetic, and the
    // launch measured 55.6 us against 37.7 + 15.1 us for the two kernels here.)
    FFK_TRY(ffk_linear_forward(st, dtype, FFK_ACT_NONE, ffn_in, ws + L.f1, w->w1, w->b1, T, E, F));
  } else {
    FFK_TRY(ffk_linear_forward(st, dtype, FFK_ACT_RELU, ffn_in, ws + L.act1, w->w1, w->b1, T, E, F));
  }
  if (gelu && layer_fusion_enabled() &&
      dropout_fusable(dtype, ws + L.f1, nullptr, ws + L.act1_drop, T * F, 0)) {
    // GELU's own output is not needed again: backward reads the pre-activation
    FFK_TRY(gelu_dropout_forward(as_stream(st), dtype, ws + L.f1, ws + L.act1_drop, T * F, p, d->seed + 1, 0));
  } else {
    if (gelu) FFK_TRY(ffk_element_unary_forward(st, dtype, FFK_OP_GELU, 0.0f, ws + L.f1, ws + L.act1, T * F));
    FFK_TRY(ffk_dropout_forward(st, dtype, ws + L.act1, ws + L.act1_drop, T * F, p, d->seed + 1, 0));
  }
  // x1 + dropout(dense(d_model)): the dropout and the addition ride on the GEMM's tile store
  // where that kernel exists (backward reads neither the Linear's nor the dropout's output)
  void *const ffn_sum = d->pre_layer_norm ? y : static_cast<void *>(ws + L.pre2);
  int sum_rc = FFK_ERR_UNSUPPORTED;
  if (layer_fusion_enabled()) {
    sum_rc = linear_dropout_add_forward(as_stream(st), dtype, ws + L.act1_drop, ws + L.x1, ffn_sum, w->w2, w->b2,
                                        T, F, E, p, d->seed + 2, 0);
    if (sum_rc != FFK_OK && sum_rc != FFK_ERR_UNSUPPORTED) return sum_rc;
  }
  if (sum_rc != FFK_OK) {
    FFK_TRY(ffk_linear_forward(st, dtype, FFK_ACT_NONE, ws + L.act1_drop, ws + L.f2, w->w2, w->b2, T, F, E));
    FFK_TRY(dropout_then_add(st, dtype, ws + L.f2, ws + L.f2_drop, ws + L.x1, ffn_sum, T * E, p, d->seed + 2));
  }
  if (!d->pre_layer_norm) {
    FFK_TRY(ffk_layer_norm_forward(st, dtype, ws + L.pre2, y, w->ln2_gamma, w->ln2_beta,
                                   mean(L.mean2), mean(L.rstd2), T, E, d->ln_eps));
  }
  return FFK_OK;
}

extern "C" int ffk_encoder_layer_backward(ffk_stream_t st, int dtype,
                                          ffk_encoder_layer_desc_t const *d,
                                          ffk_encoder_layer_params_t const *w,
                                          ffk_encoder_layer_params_t const *g,
                                          void const *x, void const *dy, void *dx,
                                          void *workspace, size_t workspace_bytes) {
  FFK_TRY(check_layer("encoder_layer_backward", dtype, d));
  FFK_REQUIRE(w && g && x && dy && dx, "encoder_layer_backward: NULL argument");
  LayerWs L = layout(d, dtype);
  if (workspace == nullptr || workspace_bytes < L.total) {
    return fail(FFK_ERR_WORKSPACE, "encoder_layer_backward: workspace of %zu bytes needed, %zu given",
                L.total, workspace_bytes);
  }
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  int64_t const T = d->batch * d->seq, E = d->d_model, F = d->d_ff;
  ffk_mha_desc_t m = mha_desc(d);
  float const p = d->dropout_rate;
  bool const gelu = d->activation == FFK_ACT_GELU;
  auto mean = [&](size_t o) { return reinterpret_cast<float *>(ws + o); };
  size_t const ln_ws_bytes = L.ln_ws_b - L.ln_ws, lin_ws_bytes = L.lin_ws_b - L.lin_ws;
  int const wacc = d->overwrite_weight_grads ? 0 : (FFK_ACC_WEIGHT | FFK_ACC_BIAS);
  int const mha_mode = d->overwrite_weight_grads ? FFK_MHA_OVERWRITE_WEIGHT_GRAD : 0;
  bool const ln_acc = !d->overwrite_weight_grads;  // LayerNorm gamma / beta gradients follow the same switch
  int const ln_mode = ln_acc ? FFK_LN_ACC_PARAMS : 0;

  // The four small column reductions of this pass (two bias gradients, two pairs of LayerNorm
  // parameter gradients) are collected and run as one launch at the end: each is a few
  // microseconds of launch latency for almost no work.  Their producers get scratch of their own.
  ColreduceBatch reductions;
  struct Collect {
    ColreduceBatch *saved;
    explicit Collect(ColreduceBatch *b) : saved(tl_colreduce_batch) { tl_colreduce_batch = b; }
    ~Collect() { tl_colreduce_batch = saved; }
  } collect(layer_fusion_enabled() ? &reductions : tl_colreduce_batch);

  // ---- tail: y = x1 + f2_drop (pre-LN) or y = LN2(x1 + f2_drop) (post-LN)
  void const *g_sum = dy;  // gradient of (x1 + f2_drop)
  if (!d->pre_layer_norm) {
    FFK_TRY(ffk_layer_norm_backward(st, dtype, dy, ws + L.pre2, mean(L.mean2), mean(L.rstd2), w->ln2_gamma,
                                    ws + L.g_tmp, g->ln2_gamma, g->ln2_beta, T, E, ws + L.ln_ws, ln_ws_bytes, ln_mode));
    g_sum = ws + L.g_tmp;
  }
  // ---- FFN backward
  // The dropout behind the second FFN Linear: its backward also sums its result's columns, the
  // Linear's bias gradient, in the same pass (the Linear's backward below then has none to compute).
  void *b2_grad = g->b2;
  {
    int rc = FFK_ERR_UNSUPPORTED;
    DropoutParams dp;
    FFK_TRY(make_dropout_params("encoder_layer_backward", p, d->seed + 2, 0, dp));
    if (layer_fusion_enabled() && b2_grad != nullptr) {
      rc = dropout_backward_colsum(as_stream(st), dtype, g_sum, ws + L.g_f2, T, E, b2_grad, (wacc & FFK_ACC_BIAS) != 0,
                                   reinterpret_cast<float *>(ws + L.lin_ws), dp);
      if (rc != FFK_OK && rc != FFK_ERR_UNSUPPORTED) return rc;
    }
    if (rc == FFK_OK) {
      b2_grad = nullptr;
    } else {
      FFK_TRY(ffk_dropout_backward(st, dtype, g_sum, ws + L.g_f2, T * E, p, d->seed + 2, 0, 0));
    }
  }
  int g_f1_rc = FFK_ERR_UNSUPPORTED;
  bool b1_done = false;  // the first Linear's bias gradient already computed
  // The two FFN weight gradients, [E,F] and [F,E] over the same T rows, are off the path of the
  // input gradients and each is one 128x128 tile per CU at this layer's sizes: both go out as one
  // launch behind the first Linear's input gradient (the same kernel and tile each would run on
  // alone, so the same bits; one launch and one tail fewer).
  void const *ffn_in = d->pre_layer_norm ? ws + L.h2 : ws + L.x1;
  GemmProblem const dw2_problem = {E, F, ws + L.g_f2, E, ws + L.act1_drop, F, g->w2, F};
  GemmProblem const dw1_problem = {F, E, ws + L.g_f1, F, ffn_in, E, g->w1, E};
  bool const pair_dw = gelu && layer_fusion_enabled() && g->w1 != nullptr && g->w2 != nullptr &&
                       (E / 128) * (F / 128) >= kNumCU / 2 &&
                       gemm_pair_supported(dtype, true, false, T, dw2_problem, dw1_problem);
  bool dw_pending = false;  // both weight gradients still to be computed, as a pair
  if (gelu && layer_fusion_enabled()) {
    // the dropout's and GELU's backward ride on the tile store of the input-gradient GEMM
    // (52.7 us against 37.7 + 18.4 us: the separate kernel moves three tensors, this one adds one read)
    // ... and so do the column sums of what it stores, the first Linear's bias gradient
    if (g->b1 != nullptr) {
      g_f1_rc = linear_backward_dropout_gelu(as_stream(st), dtype, ws + L.g_f2, ws + L.act1_drop, ws + L.f1,
                                             ws + L.g_f1, w->w2, pair_dw ? nullptr : g->w2, b2_grad, T, F, E, ws + L.lin_ws,
                                             lin_ws_bytes, wacc, p, d->seed + 1, 0, g->b1,
                                             reinterpret_cast<float *>(ws + L.lin_ws_b), (wacc & FFK_ACC_BIAS) != 0);
      b1_done = g_f1_rc == FFK_OK;
    }
    if (g_f1_rc == FFK_ERR_UNSUPPORTED) {
      g_f1_rc = linear_backward_dropout_gelu(as_stream(st), dtype, ws + L.g_f2, ws + L.act1_drop, ws + L.f1,
                                             ws + L.g_f1, w->w2, pair_dw ? nullptr : g->w2, b2_grad, T, F, E, ws + L.lin_ws,
                                             lin_ws_bytes, wacc, p, d->seed + 1, 0);
    }
    if (g_f1_rc != FFK_OK && g_f1_rc != FFK_ERR_UNSUPPORTED) return g_f1_rc;
    dw_pending = pair_dw && g_f1_rc == FFK_OK;  // refused: nothing was launched, the separate operators follow
  }
  bool const g_f1_ready = g_f1_rc == FFK_OK;
  if (!g_f1_ready) {
    FFK_TRY(ffk_linear_backward(st, dtype, FFK_ACT_NONE, 0, ws + L.f2, ws + L.g_f2, ws + L.act1_drop,
                                ws + L.g_act1_drop, w->w2, g->w2, b2_grad, T, F, E, ws + L.lin_ws, lin_ws_bytes,
                                wacc));
  }
  bool const fuse_gelu_bwd = g_f1_ready || (gelu && layer_fusion_enabled() &&
                             dropout_fusable(dtype, ws + L.g_act1_drop, ws + L.f1, ws + L.g_f1, T * F, 0));
  if (g_f1_ready) {
  } else if (fuse_gelu_bwd) {
    FFK_TRY(dropout_backward_gelu_backward(as_stream(st), dtype, ws + L.g_act1_drop, ws + L.f1, ws + L.g_f1,
                                           T * F, p, d->seed + 1, 0));
  } else {
    FFK_TRY(ffk_dropout_backward(st, dtype, ws + L.g_act1_drop, ws + L.g_act1, T * F, p, d->seed + 1, 0, 0));
  }
  if (gelu) {
    if (!fuse_gelu_bwd) {
      FFK_TRY(ffk_element_unary_backward(st, dtype, FFK_OP_GELU, 0.0f, ws + L.act1, ws + L.g_act1, ws + L.f1,
                                         ws + L.g_f1, T * F, 0));
    }
    FFK_TRY(ffk_linear_backward(st, dtype, FFK_ACT_NONE, 0, ws + L.f1, ws + L.g_f1, ffn_in, ws + L.g_h2,
                                w->w1, dw_pending ? nullptr : g->w1, b1_done ? nullptr : g->b1, T, E, F,
                                ws + L.lin_ws_b, lin_ws_bytes, wacc));
    if (dw_pending) {
      FFK_TRY(gemm_dispatch_pair(as_stream(st), dtype, true, false, T, dw2_problem, dw1_problem,
                                 (wacc & FFK_ACC_WEIGHT) != 0));
    }
  } else {
    FFK_TRY(ffk_linear_backward(st, dtype, FFK_ACT_RELU, 0, ws + L.act1, ws + L.g_act1, ffn_in, ws + L.g_h2,
                                w->w1, g->w1, g->b1, T, E, F, ws + L.lin_ws_b, lin_ws_bytes, wacc));
  }
  // ---- gradient reaching x1
  bool g_attn_ready = false;  // the attention branch's dropout backward already done
  if (d->pre_layer_norm) {
    // g_x1 = LN2_backward(g_h2) + dy
    int rc = FFK_ERR_UNSUPPORTED;
    if (layer_fusion_enabled()) {
      // ... and g_attn = dropout_backward(g_x1) on the way, when the mask comes in whole blocks
      bool const with_drop = T * E % 8 == 0 && E % 8 == 0;
      rc = layer_norm_backward_add_residual(as_stream(st), dtype, ws + L.g_h2, ws + L.x1, mean(L.mean2),
                                            mean(L.rstd2), w->ln2_gamma, dy, ws + L.g_x1, g->ln2_gamma,
                                            g->ln2_beta, T, E, ws + L.ln_ws, ln_ws_bytes,
                                            with_drop ? ws + L.g_attn : nullptr, p, d->seed + 0, 0, ln_acc);
      if (rc != FFK_OK && rc != FFK_ERR_UNSUPPORTED) return rc;
      g_attn_ready = rc == FFK_OK && with_drop;
    }
    if (rc == FFK_ERR_UNSUPPORTED) {
      FFK_TRY(ffk_layer_norm_backward(st, dtype, ws + L.g_h2, ws + L.x1, mean(L.mean2), mean(L.rstd2), w->ln2_gamma,
                                      ws + L.g_x1, g->ln2_gamma, g->ln2_beta, T, E, ws + L.ln_ws, ln_ws_bytes, ln_mode));
      FFK_TRY(ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, ws + L.g_x1, dy, ws + L.g_x1, T * E, T * E, T * E));
    }
  } else {
    FFK_TRY(ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, ws + L.g_h2, g_sum, ws + L.g_x1, T * E, T * E, T * E));
  }
  // ---- attention block backward
  void const *g_attn_res;  // gradient of (attn (+dropout) + x)
  if (d->pre_layer_norm) {
    g_attn_res = ws + L.g_x1;
    if (!g_attn_ready) FFK_TRY(ffk_dropout_backward(st, dtype, g_attn_res, ws + L.g_attn, T * E, p, d->seed + 0, 0, 0));
    FFK_TRY(ffk_mha_backward(st, dtype, &m, ws + L.h1, ws + L.g_h1, ws + L.h1, nullptr, ws + L.h1, nullptr,
                             w->attn_weight, g->attn_weight, ws + L.g_attn, ws + L.mha_reserve,
                             L.ln_ws - L.mha_reserve, mha_mode));
    // dx = LN1_backward(g_h1) + g_x1
    int rc = FFK_ERR_UNSUPPORTED;
    if (layer_fusion_enabled()) {
      rc = layer_norm_backward_add_residual(as_stream(st), dtype, ws + L.g_h1, x, mean(L.mean1), mean(L.rstd1),
                                            w->ln1_gamma, g_attn_res, dx, g->ln1_gamma, g->ln1_beta, T, E,
                                            ws + L.ln_ws_b, ln_ws_bytes, nullptr, 0.0f, 0, 0, ln_acc);
      if (rc != FFK_OK && rc != FFK_ERR_UNSUPPORTED) return rc;
    }
    if (rc == FFK_ERR_UNSUPPORTED) {
      FFK_TRY(ffk_layer_norm_backward(st, dtype, ws + L.g_h1, x, mean(L.mean1), mean(L.rstd1), w->ln1_gamma, dx,
                                      g->ln1_gamma, g->ln1_beta, T, E, ws + L.ln_ws_b, ln_ws_bytes, ln_mode));
      FFK_TRY(ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, dx, g_attn_res, dx, T * E, T * E, T * E));
    }
  } else {
    FFK_TRY(ffk_layer_norm_backward(st, dtype, ws + L.g_x1, ws + L.h1, mean(L.mean1), mean(L.rstd1), w->ln1_gamma,
                                    ws + L.g_attn, g->ln1_gamma, g->ln1_beta, T, E, ws + L.ln_ws_b, ln_ws_bytes, ln_mode));
    g_attn_res = ws + L.g_attn;
    FFK_TRY(ffk_mha_backward(st, dtype, &m, x, dx, x, nullptr, x, nullptr, w->attn_weight, g->attn_weight,
                             g_attn_res, ws + L.mha_reserve, L.ln_ws - L.mha_reserve, mha_mode));
    FFK_TRY(ffk_element_binary_forward(st, dtype, FFK_OP_EW_ADD, dx, g_attn_res, dx, T * E, T * E, T * E));
  }
  FFK_HIP(colreduce_flush(as_stream(st), reductions));
  return FFK_OK;
}

// ---------------------------------------------------------------------------
// The same collection for callers that sequence the operators themselves.
// ---------------------------------------------------------------------------
static thread_local ffk::ColreduceBatch tl_caller_batch;

extern "C" int ffk_column_reductions_begin(void) {
  tl_caller_batch.count = 0;
  tl_caller_batch.dtype = -1;
  ffk::tl_colreduce_batch = &tl_caller_batch;
  return FFK_OK;
}

extern "C" int ffk_column_reductions_end(ffk_stream_t stream) {
  if (ffk::tl_colreduce_batch != &tl_caller_batch) return FFK_OK;  // nothing was begun on this thread
  ffk::tl_colreduce_batch = nullptr;
  FFK_HIP(ffk::colreduce_flush(as_stream(stream), tl_caller_batch));
  return FFK_OK;
}

