// MultiHeadAttention forward/backward for gfx950: projection GEMMs around the
// fused attention core (reference: one cudnnMultiHeadAttnForward /
// BackwardData / BackwardWeights call each, lib/kernels/src/cuda/ops/
// attention_kernels.cu:215-303).
//
// Weight blob: [ W_Q | W_K | W_V | W_O ] with W_Q = [heads*qProj, qSize]
// (head-major rows), W_K = [heads*kProj, kSize], W_V = [heads*vProj, vSize],
// W_O = [oProj, heads*vProj], all row-major.  qProj = kProj (the reference
// asserts it, src/cuda/ops/attention_kernels.cu:61); vProj is free.  When
// query, key and value are the same tensor the three input projections run as
// one GEMM against the contiguous [heads*(2*qProj + vProj), size] block and the
// core reads the fused buffer through strides.  FLOAT (the reference's data
// type) and BF16; the core is attention_f32.hip / attention.hip /
// attention_gen.hip.
//
// Reserve space layout (bytes, each region 256-byte aligned):
//   QKV projections | context | lse | delta | d(context) | d(QKV projections)
#include "gemm.h"

namespace ffk {

struct MhaLayout {
  int64_t TQ, TK;                 // tokens: B*Sq, B*Skv
  int64_t nQ, nK, nV, nC;         // elements of each projected tensor / context
  size_t off_qkv, off_ctx, off_lse, off_delta, off_dctx, off_dqkv, total;
  int64_t wq, wk, wv, wo;         // weight offsets (elements)
};

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

static MhaLayout make_layout(ffk_mha_desc_t const *d, size_t es) {
  MhaLayout L;
  L.TQ = d->num_samples * d->qo_seq_length;
  L.TK = d->num_samples * d->kv_seq_length;
  L.nQ = L.TQ * d->num_heads * d->q_proj_size;
  L.nK = L.TK * d->num_heads * d->k_proj_size;
  L.nV = L.TK * d->num_heads * d->v_proj_size;
  L.nC = L.TQ * d->num_heads * d->v_proj_size;
  size_t off = 0;
  L.off_qkv = off;   off += align256((size_t)(L.nQ + L.nK + L.nV) * es);
  L.off_ctx = off;   off += align256((size_t)L.nC * es);
  L.off_lse = off;   off += align256((size_t)(d->num_samples * d->num_heads * d->qo_seq_length) * 4);
  L.off_delta = off; off += align256((size_t)(d->num_samples * d->num_heads * d->qo_seq_length) * 4);
  L.off_dctx = off;  off += align256((size_t)L.nC * es);
  L.off_dqkv = off;  off += align256((size_t)(L.nQ + L.nK + L.nV) * es);
  L.total = off;
  L.wq = 0;
  L.wk = L.wq + d->num_heads * d->q_proj_size * d->q_size;
  L.wv = L.wk + d->num_heads * d->k_proj_size * d->k_size;
  L.wo = L.wv + d->num_heads * d->v_proj_size * d->v_size;
  return L;
}

static int check_mha(char const *who, int dtype, ffk_mha_desc_t const *d) {
  FFK_REQUIRE(d != nullptr, "%s: NULL descriptor", who);
  FFK_REQUIRE(dtype == FFK_BF16 || dtype == FFK_FLOAT, "%s: dtype %d not supported (FLOAT or BF16)", who, dtype);
  FFK_REQUIRE(d->num_samples > 0 && d->num_heads > 0 && d->q_size > 0 && d->k_size > 0 &&
                  d->v_size > 0 && d->o_proj_size > 0 && d->qo_seq_length > 0 && d->kv_seq_length > 0,
              "%s: non-positive size", who);
  FFK_REQUIRE(d->q_proj_size == d->k_proj_size, "%s: qProjSize must equal kProjSize", who);
  FFK_REQUIRE(d->q_proj_size > 0 && d->v_proj_size > 0, "%s: non-positive projection size", who);
  int64_t const unit = dtype == FFK_BF16 ? 8 : 4;
  FFK_REQUIRE(d->q_proj_size <= 256 && d->q_proj_size % unit == 0 && d->v_proj_size <= 256 &&
                  d->v_proj_size % unit == 0,
              "%s: projection size %lld / %lld not supported (multiples of %lld up to 256)", who,
              (long long)d->q_proj_size, (long long)d->v_proj_size, (long long)unit);
  return FFK_OK;
}

// The reserve layout depends on the descriptor alone, so a backward call finds
// what the forward call wrote whatever the caller's pointers are: with equal
// input widths and sequence lengths the three projections are the column
// blocks of ONE [tokens, heads*(2*qProj + vProj)] buffer (the core reads them
// through strides), otherwise three dense tensors one after the other.
static bool is_interleaved(ffk_mha_desc_t const *d) {
  return d->q_size == d->k_size && d->k_size == d->v_size && d->qo_seq_length == d->kv_seq_length;
}
// Self-attention on one tensor: the three input projections are one GEMM.
static bool is_aliased(ffk_mha_desc_t const *d, void const *q, void const *k, void const *v) {
  return q == k && k == v && is_interleaved(d);
}

static ffk_attention_desc_t core_desc(ffk_mha_desc_t const *d, bool fused) {
  int64_t const H = d->num_heads, Dq = d->q_proj_size, Dv = d->v_proj_size;
  ffk_attention_desc_t a;
  a.batch = d->num_samples;
  a.heads = H;
  a.seq_q = d->qo_seq_length;
  a.seq_kv = d->kv_seq_length;
  a.head_dim = Dq;
  a.v_head_dim = Dv;
  int64_t const row = H * (2 * Dq + Dv);
  a.q_seq_stride = a.k_seq_stride = fused ? row : H * Dq;
  a.v_seq_stride = fused ? row : H * Dv;
  a.q_batch_stride = d->qo_seq_length * a.q_seq_stride;
  a.k_batch_stride = d->kv_seq_length * a.k_seq_stride;
  a.v_batch_stride = d->kv_seq_length * a.v_seq_stride;
  a.o_seq_stride = H * Dv;
  a.o_batch_stride = d->qo_seq_length * H * Dv;
  a.scale = d->scale;
  a.causal = d->causal;
  return a;
}

}  // namespace ffk

using namespace ffk;

extern "C" size_t ffk_mha_weight_elements(ffk_mha_desc_t const *d) {
  if (d == nullptr) return 0;
  return (size_t)(d->num_heads * (d->q_proj_size * d->q_size + d->k_proj_size * d->k_size +
                                  d->v_proj_size * d->v_size + d->v_proj_size * d->o_proj_size));
}

extern "C" size_t ffk_mha_reserve_bytes(ffk_mha_desc_t const *d, int dtype) {
  if (d == nullptr || dtype_size(dtype) == 0) return 0;
  return make_layout(d, dtype_size(dtype)).total;
}

extern "C" int ffk_mha_forward(ffk_stream_t stream, int dtype,
                               ffk_mha_desc_t const *d, void const *query,
                               void const *key, void const *value,
                               void const *weight, void *output, void *reserve,
                               size_t reserve_bytes) {
  int rc = check_mha("mha_forward", dtype, d);
  if (rc != FFK_OK) return rc;
  FFK_REQUIRE(query && key && value && weight && output, "mha_forward: NULL tensor");
  size_t const es = dtype_size(dtype);
  MhaLayout L = make_layout(d, es);
  if (reserve == nullptr || reserve_bytes < L.total) {
    return fail(FFK_ERR_WORKSPACE, "mha_forward: reserve space of %zu bytes needed, %zu given",
                L.total, reserve_bytes);
  }
  hipStream_t st = as_stream(stream);
  uint8_t *rs = static_cast<uint8_t *>(reserve);
  uint8_t const *w = static_cast<uint8_t const *>(weight);
  int64_t const H = d->num_heads, HDq = H * d->q_proj_size, HDv = H * d->v_proj_size;
  int64_t const row = 2 * HDq + HDv;  // the interleaved buffer's row: [ Q | K | V ]
  bool const fused = is_interleaved(d);
  uint8_t *qkv = rs + L.off_qkv;
  GemmEpilogue ep;
  void const *qp, *kp, *vp;
  if (is_aliased(d, query, key, value)) {
    // [T, row] = X . [W_Q; W_K; W_V]^T
    rc = gemm_dispatch(st, dtype, false, true, L.TQ, row, d->q_size, query, d->q_size,
                       w + L.wq * es, d->q_size, qkv, row, ep);
    if (rc != FFK_OK) return rc;
    qp = qkv;
    kp = qkv + HDq * es;
    vp = qkv + 2 * HDq * es;
  } else {
    uint8_t *Q = qkv, *K = fused ? qkv + HDq * es : qkv + L.nQ * es, *V = fused ? qkv + 2 * HDq * es : K + L.nK * es;
    rc = gemm_dispatch(st, dtype, false, true, L.TQ, HDq, d->q_size, query, d->q_size,
                       w + L.wq * es, d->q_size, Q, fused ? row : HDq, ep);
    if (rc != FFK_OK) return rc;
    rc = gemm_dispatch(st, dtype, false, true, L.TK, HDq, d->k_size, key, d->k_size,
                       w + L.wk * es, d->k_size, K, fused ? row : HDq, ep);
    if (rc != FFK_OK) return rc;
    rc = gemm_dispatch(st, dtype, false, true, L.TK, HDv, d->v_size, value, d->v_size,
                       w + L.wv * es, d->v_size, V, fused ? row : HDv, ep);
    if (rc != FFK_OK) return rc;
    qp = Q; kp = K; vp = V;
  }
  ffk_attention_desc_t a = core_desc(d, fused);
  rc = ffk_attention_forward(stream, dtype, &a, qp, kp, vp, rs + L.off_ctx,
                             reinterpret_cast<float *>(rs + L.off_lse));
  if (rc != FFK_OK) return rc;
  // output[T, oProj] = context[T, H*vProj] . W_O[oProj, H*vProj]^T
  return gemm_dispatch(st, dtype, false, true, L.TQ, d->o_proj_size, HDv, rs + L.off_ctx, HDv,
                       w + L.wo * es, HDv, output, d->o_proj_size, ep);
}

extern "C" int ffk_mha_backward(ffk_stream_t stream, int dtype,
                                ffk_mha_desc_t const *d, void const *query,
                                void *query_grad, void const *key,
                                void *key_grad, void const *value,
                                void *value_grad, void const *weight,
                                void *weight_grad, void const *output_grad,
                                void *reserve, size_t reserve_bytes,
                                int accumulate) {
  int rc = check_mha("mha_backward", dtype, d);
  if (rc != FFK_OK) return rc;
  FFK_REQUIRE(query && key && value && weight && output_grad, "mha_backward: NULL tensor");
  size_t const es = dtype_size(dtype);
  MhaLayout L = make_layout(d, es);
  if (reserve == nullptr || reserve_bytes < L.total) {
    return fail(FFK_ERR_WORKSPACE, "mha_backward: reserve space of %zu bytes needed, %zu given",
                L.total, reserve_bytes);
  }
  hipStream_t st = as_stream(stream);
  uint8_t *rs = static_cast<uint8_t *>(reserve);
  uint8_t const *w = static_cast<uint8_t const *>(weight);
  uint8_t *dw = static_cast<uint8_t *>(weight_grad);
  int64_t const H = d->num_heads, HDq = H * d->q_proj_size, HDv = H * d->v_proj_size;
  int64_t const row = 2 * HDq + HDv;  // the interleaved buffers' row: [ Q | K | V ]
  bool const fused = is_interleaved(d);
  bool const aliased = is_aliased(d, query, key, value);
  // one tensor, three roles: its gradient is the sum of the three, which needs
  // either all three outputs or query_grad alone
  FFK_REQUIRE(!aliased || (key_grad == nullptr) == (value_grad == nullptr),
              "mha_backward: query, key and value are one tensor: pass both key_grad and value_grad, or "
              "neither (their gradients are then added into query_grad)");
  uint8_t *qkv = rs + L.off_qkv, *dqkv = rs + L.off_dqkv;
  uint8_t *ctx = rs + L.off_ctx, *dctx = rs + L.off_dctx;
  GemmEpilogue over, acc, in_ep;
  acc.accumulate = (accumulate & FFK_MHA_OVERWRITE_WEIGHT_GRAD) == 0;
  in_ep.accumulate = (accumulate & FFK_MHA_ACC_INPUT_GRADS) != 0;

  // d(context) = dOut . W_O ; dW_O += dOut^T . context
  rc = gemm_dispatch(st, dtype, false, false, L.TQ, HDv, d->o_proj_size, output_grad,
                     d->o_proj_size, w + L.wo * es, HDv, dctx, HDv, over);
  if (rc != FFK_OK) return rc;
  // The two weight gradients of a self-attention block (output projection and
  // folded Q/K/V projection) have the same reduction length and each leaves
  // part of the chip idle: where the library can, they run as ONE launch after
  // the core's backward.
  bool const folded = aliased && key_grad == nullptr && value_grad == nullptr;
  GemmProblem const wo_grad = {d->o_proj_size, HDv, output_grad, d->o_proj_size, ctx, HDv,
                               dw != nullptr ? dw + L.wo * es : nullptr, HDv};
  GemmProblem const wqkv_grad = {row, d->q_size, dqkv, row, query, d->q_size,
                                 dw != nullptr ? dw + L.wq * es : nullptr, d->q_size};
  bool const paired = dw != nullptr && folded && gemm_pair_supported(dtype, true, false, L.TQ, wqkv_grad, wo_grad);
  if (dw != nullptr && !paired) {
    // d(QKV projections) is not written before the core's backward: until
    // then it serves as split-K scratch for this small-output, long-K GEMM.
    GemmEpilogue acc_o = acc;
    acc_o.splitk_ws = dqkv;
    acc_o.splitk_ws_bytes = L.total - L.off_dqkv;
    rc = gemm_dispatch(st, dtype, true, false, d->o_proj_size, HDv, L.TQ, output_grad,
                       d->o_proj_size, ctx, HDv, dw + L.wo * es, HDv, acc_o);
    if (rc != FFK_OK) return rc;
  }

  ffk_attention_desc_t a = core_desc(d, fused);
  void const *qp, *kp, *vp;
  void *dqp, *dkp, *dvp;
  if (fused) {
    qp = qkv; kp = qkv + HDq * es; vp = qkv + 2 * HDq * es;
    dqp = dqkv; dkp = dqkv + HDq * es; dvp = dqkv + 2 * HDq * es;
  } else {
    qp = qkv; kp = qkv + L.nQ * es; vp = qkv + (L.nQ + L.nK) * es;
    dqp = dqkv; dkp = dqkv + L.nQ * es; dvp = dqkv + (L.nQ + L.nK) * es;
  }
  // The core writes dQ/dK/dV with the same strides it reads Q/K/V with.
  rc = ffk_attention_backward(stream, dtype, &a, qp, kp, vp, ctx, dctx,
                              reinterpret_cast<float const *>(rs + L.off_lse),
                              reinterpret_cast<float *>(rs + L.off_delta), dqp, dkp, dvp);
  if (rc != FFK_OK) return rc;

  if (folded) {
    // dX (+)= dQKV[T,row] . [W_Q; W_K; W_V]  and  dW_QKV += dQKV^T . X
    if (query_grad != nullptr) {
      rc = gemm_dispatch(st, dtype, false, false, L.TQ, d->q_size, row, dqkv, row,
                         w + L.wq * es, d->q_size, query_grad, d->q_size, in_ep);
      if (rc != FFK_OK) return rc;
    }
    if (paired) {
      return gemm_dispatch_pair(st, dtype, true, false, L.TQ, wqkv_grad, wo_grad, acc.accumulate);
    }
    if (dw != nullptr) {
      rc = gemm_dispatch(st, dtype, true, false, row, d->q_size, L.TQ, dqkv, row, query,
                         d->q_size, dw + L.wq * es, d->q_size, acc);
      if (rc != FFK_OK) return rc;
    }
    return FFK_OK;
  }
  struct Part {
    void const *x; void *dx; void const *dp; int64_t T, size, woff, HD;
  } parts[3] = {
      {query, query_grad, dqp, L.TQ, d->q_size, L.wq, HDq},
      {key, key_grad, dkp, L.TK, d->k_size, L.wk, HDq},
      {value, value_grad, dvp, L.TK, d->v_size, L.wv, HDv},
  };
  for (int i = 0; i < 3; i++) {
    Part const &pt = parts[i];
    int64_t const HD = pt.HD, ld = fused ? row : HD;
    if (pt.dx != nullptr) {
      rc = gemm_dispatch(st, dtype, false, false, pt.T, pt.size, HD, pt.dp, ld,
                         w + pt.woff * es, pt.size, pt.dx, pt.size, in_ep);
      if (rc != FFK_OK) return rc;
    }
    if (dw != nullptr) {
      rc = gemm_dispatch(st, dtype, true, false, HD, pt.size, pt.T, pt.dp, ld, pt.x, pt.size,
                         dw + pt.woff * es, pt.size, acc);
      if (rc != FFK_OK) return rc;
    }
  }
  return FFK_OK;
}
