/*
 * ffk_oracle.h -- CPU restatement of the reference's per-device operator
 * arithmetic.  TEST INFRASTRUCTURE ONLY: it is the checker for the gfx950
 * kernels (tests, the smoke check and the CPU-baseline leg of the benchmark);
 * the product library never calls it.
 *
 * All tensors are host float arrays in dense row-major order unless noted.
 * "bf16 mode" of a function means: its float inputs already hold
 * bf16-representable values, arithmetic is done in fp32/fp64 and results are
 * rounded to bf16 (round-to-nearest-even) exactly where the device kernel
 * stores bf16.
 *
 * Pinning status of each function is listed at the top of ffk_oracle.c.
 */
#ifndef FFK_ORACLE_H
#define FFK_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- helpers ---- */
void orc_set_num_threads(int n);
int orc_get_max_threads(void);
float orc_round_bf16(float x);
void orc_round_bf16_array(float *x, int64_t n);
int64_t orc_offset(int64_t const *dims, int rank, int64_t const *coord);

/* ---- tensor_accessor_* primitives (2-D fp32) ---- */
void orc_matmul(float const *lhs, float const *rhs, float *out, int64_t M,
                int64_t K, int64_t N);
void orc_transpose(float const *in, float *out, int64_t rows, int64_t cols);
void orc_broadcast(float const *in, int64_t const *in_dims, int in_rank,
                   float *out, int64_t const *out_dims, int out_rank);
void orc_reduce_dim(float const *in, int64_t const *dims, int rank, int dim,
                    float *out);
void orc_relu(float const *in, float *out, int64_t n);
void orc_scale(float const *in, float c, float *out, int64_t n);
void orc_add(float const *a, float const *b, float *out, int64_t n);

/* ---- Linear ---- */
/* activation: -1 none, 0 relu (others unsupported on the reference CPU path;
 * 1 sigmoid and 2 tanh are provided from the reference GPU helpers). */
int orc_linear_forward(int activation, float const *input, float *output,
                       float const *weight, float const *bias, int64_t batch,
                       int64_t in_dim, int64_t out_dim);
int orc_linear_backward(int activation, int relu_grad_mode,
                        float const *output, float const *output_grad,
                        float const *input, float *input_grad,
                        float const *weight, float *weight_grad,
                        float *bias_grad, int64_t batch, int64_t in_dim,
                        int64_t out_dim);
void orc_linear_l2_regularizer_grad(float const *weight, float *weight_grad,
                                    int64_t n, float lambda);
/* C[M,N] = op(A).op(B) accumulated in double, for GEMM checks at any size. */
void orc_gemm_f64(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                  float const *A, float const *B, float *C);

/* ---- element-wise ---- */
int orc_element_unary_forward(int op, float scalar, float const *in, float *out,
                              int64_t n);
int orc_element_unary_backward(int op, float scalar, float const *out,
                               float const *out_grad, float const *in,
                               float *in_grad, int64_t n, int accumulate);
int orc_element_binary_forward(int op, float const *lhs, float const *rhs,
                               float *out, int64_t n, int64_t nl, int64_t nr);
int orc_element_binary_backward(int op, float const *out_grad,
                                float const *lhs, float const *rhs,
                                float *lhs_grad, float *rhs_grad, int64_t n,
                                int accumulate);

/* ---- LayerNorm ---- */
void orc_layer_norm_forward(float const *x, float *y, float const *gamma,
                            float const *beta, float *mean, float *rstd,
                            int64_t M, int64_t N, float eps);
void orc_layer_norm_backward(float const *dy, float const *x,
                             float const *mean, float const *rstd,
                             float const *gamma, float *dx, float *dgamma,
                             float *dbeta, int64_t M, int64_t N,
                             int accumulate_dx);

/* ---- Softmax over the middle dim of [outer, dim, inner] ---- */
void orc_softmax_forward(float const *x, float *y, int64_t outer, int64_t dim,
                         int64_t inner);
void orc_softmax_backward(float const *y, float const *dy, float *dx,
                          int64_t outer, int64_t dim, int64_t inner);

/* ---- Dropout (Philox4x32-10 counter stream) ---- */
void orc_philox4x32_10(uint32_t const ctr[4], uint32_t const key[2],
                       uint32_t out[4]);
void orc_dropout_mask(uint8_t *mask, int64_t n, float rate, uint64_t seed,
                      uint64_t offset);
void orc_dropout_forward(float const *x, float *y, int64_t n, float rate,
                         uint64_t seed, uint64_t offset);
void orc_dropout_backward(float const *dy, float *dx, int64_t n, float rate,
                          uint64_t seed, uint64_t offset, int accumulate);

/* ---- Embedding ---- */
/* indices as int64 host array; aggr: -1 none (bag must be 1), 0 sum, 1 avg. */
int orc_embedding_forward(int64_t const *indices, float *out,
                          float const *weight, int aggr, int64_t num_bags,
                          int64_t bag, int64_t dim, int64_t num_entries);
/* weight_grad += ...; rows visited in ascending position order, fp32 adds. */
int orc_embedding_backward(int64_t const *indices, float const *out_grad,
                           float *weight_grad, int aggr, int64_t num_bags,
                           int64_t bag, int64_t dim, int64_t num_entries);
/* same, accumulated in double and rounded once (order-free reference). */
int orc_embedding_backward_f64(int64_t const *indices, float const *out_grad,
                               float *weight_grad, int aggr, int64_t num_bags,
                               int64_t bag, int64_t dim, int64_t num_entries);

/* ---- attention core and MultiHeadAttention ---- */
/* q [B,Sq,H,D], k [B,Skv,H,D], v [B,Skv,H,Dv] (dense), o [B,Sq,H,Dv],
 * lse [B,H,Sq].  bf16_mode: round P to bf16 before the PV product and O at the
 * store. */
void orc_attention_forward(float const *q, float const *k, float const *v,
                           float *o, float *lse, int64_t B, int64_t H,
                           int64_t Sq, int64_t Skv, int64_t D, int64_t Dv,
                           float scale, int causal, int bf16_mode);
void orc_attention_backward(float const *q, float const *k, float const *v,
                            float const *d_o, float *dq, float *dk, float *dv,
                            int64_t B, int64_t H, int64_t Sq, int64_t Skv,
                            int64_t D, int64_t Dv, float scale, int causal);

typedef struct {
  int64_t num_samples, num_heads;
  int64_t q_size, k_size, v_size;
  int64_t q_proj_size, k_proj_size, v_proj_size, o_proj_size;
  int64_t qo_seq_length, kv_seq_length;
  float scale;
  int causal;
} orc_mha_desc_t;

/* weight blob [W_Q | W_K | W_V | W_O] as described in include/ffk.h. */
void orc_mha_forward(orc_mha_desc_t const *d, float const *query,
                     float const *key, float const *value, float const *weight,
                     float *output, int bf16_mode);
/* grads are overwritten (dq, dk, dv) / accumulated into (dweight). */
void orc_mha_backward(orc_mha_desc_t const *d, float const *query,
                      float const *key, float const *value,
                      float const *weight, float const *output_grad,
                      float *dquery, float *dkey, float *dvalue,
                      float *dweight, int bf16_mode);

void orc_sgd_update(float lr, float momentum, int nesterov, float weight_decay,
                    float const *grad, int64_t n, int replicas, float *w,
                    float *v);
void orc_adam_update(float alpha_t, float beta1, float beta2, float weight_decay,
                     float epsilon, float const *grad, int64_t n, int replicas,
                     float *w, float *vv, float *mm);
void orc_sparse_cce_loss_backward(float *dlogit, float const *logit,
                                  int const *label, int64_t volume,
                                  int64_t num_samples, int64_t num_classes,
                                  int k, float scale_factor);
void orc_difference_loss_backward(float *dlogit, float const *logit,
                                  float const *label, int64_t volume,
                                  float scale_factor);
void orc_identity_loss_backward(float *dloss, int64_t volume, float scale_factor);

/* ---- Concat: out [num_blocks, sum blk], in[i] [num_blocks, blk[i]] ---- */
void orc_concat_forward(float *out, float const *const *in, int64_t const *blk,
                        int n, int64_t num_blocks);
void orc_concat_backward(float const *dout, float *const *din,
                         int64_t const *blk, int n, int64_t num_blocks,
                         int accumulate);

/* ---- Transpose: out dim i = in dim perm[i] (dims outermost first) ---- */
void orc_transpose_nd(float const *in, float *out, int nd, int64_t const *in_dim,
                      int const *perm, int accumulate);
/* ---- Gather along the middle dim of [outer, dim, stride] ---- */
void orc_gather_forward(float const *in, int64_t const *index, float *out,
                        int64_t outer, int64_t in_dim, int64_t out_dim,
                        int64_t stride);
void orc_gather_backward(float const *dout, int64_t const *index, float *din,
                         int64_t outer, int64_t in_dim, int64_t out_dim,
                         int64_t stride);

#ifdef __cplusplus
}
#endif
#endif
