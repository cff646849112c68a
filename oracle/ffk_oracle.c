/*
 * ffk_oracle.c -- CPU restatement (the parity oracle) of the reference's
 * per-device operator arithmetic.  TEST INFRASTRUCTURE ONLY; never linked
 * into, loaded by or called from the product library.
 *
 * What each function follows, and what pins it:
 *
 *  orc_offset                 lib/kernels/src/kernels/accessor.cc:15-33
 *      pinned: KAT lib/kernels/test/src/kernels/accessor.cc:25-66
 *  orc_matmul                 tensor_accessor_binary_ops.cc:111-141 (k-inner
 *      fp32 accumulate)       pinned: Linear KATs below; brute force fp64
 *  orc_transpose/broadcast/reduce_dim/relu/scale
 *                             tensor_accessor_unary_ops.cc:14-244
 *      pinned: KATs lib/kernels/test/src/kernels/tensor_accessor_unary_ops.cc:11-177
 *  orc_linear_forward/backward (activation none)
 *                             linear_kernels_cpu.cc:12-94
 *      pinned: KATs lib/kernels/test/src/kernels/linear_kernels_cpu.cc:11-174
 *  orc_linear_backward, RELU  relu_grad_mode 1 = linear_kernels_cpu.cc:46-52,65-71
 *      (source text only -- no reference test runs an activation through the
 *      kernel: PARITY UNPINNED by the reference's tests); mode 0 =
 *      cuda_helper.cu:60-64, pinned by finite differences.
 *  orc_linear_l2_regularizer_grad   src/cuda/ops/linear_kernels.cu:269-290
 *      (dW = 1 dW + lambda W once per backward call); no reference test runs a
 *      regulariser (PARITY UNPINNED there); pinned by the closed form: it is
 *      the gradient of lambda/2 |W|^2, checked by finite differences, and
 *      with a zero output gradient a Linear backward leaves exactly lambda W.
 *  orc_element_unary_*        src/cuda/ops/element_unary_kernels.cu:104-250
 *      the reference has no test for this op (PARITY UNPINNED there); pinned
 *      here by closed forms / libm and finite differences.
 *  orc_element_binary_*       src/cuda/ops/element_binary_kernels.cu:27-81
 *      no reference test (PARITY UNPINNED there); pinned by closed forms.
 *  orc_layer_norm_*           src/cuda/ops/layer_norm_kernels.cu:69-181
 *      reference test has no assertion; pinned by invariants (row mean 0,
 *      var 1; sum dx = 0; sum dx*xhat = 0), finite differences and
 *      torch.nn.functional.layer_norm in fp64.
 *  orc_softmax_*              cudnnSoftmaxForward semantics
 *      (src/cuda/ops/softmax_kernels.cu:45-78); pinned by row sums, shift
 *      invariance, torch.softmax fp64, finite differences.
 *  orc_philox4x32_10          Random123 Philox4x32-10 (Salmon et al., SC'11)
 *      pinned: the published known-answer vectors (tests/golden/philox_kat.json)
 *  orc_dropout_*              stream defined by this build (the reference's
 *      generator is cuDNN's opaque one: PARITY UNPINNED by the reference);
 *      pinned: mask is a pure function of Philox; keep-rate within 5 sigma.
 *  orc_embedding_*            src/cuda/embedding_kernels.cu:48-317
 *      no reference test (PARITY UNPINNED there); pinned by brute force /
 *      torch.nn.functional.embedding_bag.
 *  orc_attention_*, orc_mha_* cudnnMultiHeadAttn* semantics as called from
 *      src/cuda/ops/attention_kernels.cu:73-92,224,261,285.  The arithmetic
 *      lives in closed-source cuDNN 8.9 and the reference test only checks
 *      "non-zero": PARITY UNPINNED by the reference.  Pinned here by the
 *      textbook definition: torch scaled_dot_product_attention in fp64,
 *      softmax row sums, causal independence, finite differences.
 *  orc_sgd_update             src/cuda/optimizer_kernels.cu:23-44 and the CPU
 *      composition src/kernels/optimizer_kernels_cpu.cc:10-60 (every tensor op
 *      separately rounded, which is what -ffp-contract=off gives here).  The
 *      reference has no test for it (PARITY UNPINNED there); pinned by
 *      torch.optim.SGD (the kernel cites it) in fp64 and by special cases
 *      (lr = 0, momentum = 0, weight_decay = 0 reduce to textbook steps).
 *  orc_adam_update            src/cuda/optimizer_kernels.cu:111-133 (the CPU
 *      version is NOT_IMPLEMENTED in the reference; no test: PARITY UNPINNED
 *      there).  Pinned by the closed form in fp64 and by the first step from
 *      zero state, where W moves by alpha_t*(1-b1)*g / (sqrt((1-b2) g^2)+eps).
 *  orc_*_loss_backward        src/cuda/loss_function_kernels.cu:21-139
 *      no reference test (PARITY UNPINNED there); pinned by the closed forms
 *      (gradient of mean softmax-cross-entropy w.r.t. the softmax output path
 *      the reference uses: logit - onehot, times the scale).
 *      Also pinned by a five-step trajectory against torch.optim.Adam with
 *      epsilon = 0 (where the two forms coincide) and, for the losses, by
 *      autograd of the loss each kernel differentiates.
 *  orc_concat_*               src/cuda/ops/concat_kernels.cu:22-97 with
 *      copy_with_stride / add_with_stride (src/cuda/cuda_helper.cu:160-173).
 *      The reference's test only asserts non-zero output (PARITY UNPINNED
 *      there); pinned by numpy.concatenate and by split-after-concat.
 *  orc_transpose_nd           src/cuda/ops/transpose_kernels.cu:27-110 (the
 *      intended `out = in` over the same stride walk; the reference's kernel
 *      adds into uninitialised memory) and the CPU helper
 *      tensor_accessor_transpose (src/kernels/tensor_accessor_unary_ops.cc),
 *      whose known-answer test (test/src/kernels/tensor_accessor_unary_ops.cc)
 *      is among the golden vectors.  Also pinned by numpy.transpose.
 *  orc_gather_*               src/cuda/ops/gather_kernels.cu:23-82; the
 *      reference has no value test (PARITY UNPINNED there); pinned by
 *      numpy.take_along_axis and numpy.add.at.
 *  orc_cast_*                 src/kernels/cast_kernels_cpu.cc:6-20
 *      the reference tests only compare its GPU and CPU kernels on random
 *      data; pinned by numpy astype on exactly representable values and on
 *      rounding boundaries.
 */
#include "ffk_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* OperatorType ordinals (lib/op-attrs/include/op-attrs/operator_type.dtg.toml:12-94) */
enum {
  OP_SCALAR_MULTIPLY = 8, OP_SCALAR_ADD = 9, OP_SCALAR_TRUE_DIV = 11,
  OP_SCALAR_SUB = 12, OP_RELU = 13, OP_IDENTITY = 14, OP_SIGMOID = 15,
  OP_TANH = 16, OP_ELU = 17, OP_EW_ADD = 28, OP_EW_MUL = 29, OP_EW_SUB = 35,
  OP_EW_DIV = 36, OP_EW_MAX = 40, OP_EW_MIN = 41, OP_EXP = 56, OP_SIN = 61,
  OP_COS = 62, OP_GELU = 67, OP_RSQRT = 70, OP_POW = 71,
  OP_GELU_REFERENCE_GRAD = 1067
};

/* ------------------------------------------------------------------ helpers */

/* Threads for the loops marked parallel (matrix products by row, attention by
 * (batch, head)); 1 = the reference's single-threaded CPU evaluation.  Results
 * are the same bits for any count. */
void orc_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n > 0 ? n : 1);
#else
  (void)n;
#endif
}
int orc_get_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

float orc_round_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    u = (u | 0x00400000u) & 0xffff0000u;
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
  }
  memcpy(&x, &u, 4);
  return x;
}

void orc_round_bf16_array(float *x, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    x[i] = orc_round_bf16(x[i]);
  }
}

/* accessor.cc:15-33: row-major offset, dim 0 outermost */
int64_t orc_offset(int64_t const *dims, int rank, int64_t const *coord) {
  int64_t offset = 0;
  int64_t multiplier = 1;
  for (int i = rank - 1; i >= 0; i--) {
    if (coord[i] < 0 || coord[i] >= dims[i]) {
      return -1;
    }
    offset += coord[i] * multiplier;
    multiplier *= dims[i];
  }
  return offset;
}

/* ----------------------------------------------- tensor_accessor primitives */

/* tensor_accessor_binary_ops.cc:126-138 */
void orc_matmul(float const *lhs, float const *rhs, float *out, int64_t M,
                int64_t K, int64_t N) {
  /* rows are independent: threads change who computes an element, not how */
#pragma omp parallel for schedule(static) if (M * N * K > 1000000)
  for (int64_t i = 0; i < M; i++) {
    for (int64_t j = 0; j < N; j++) {
      float accum = 0.0f;
      for (int64_t k = 0; k < K; k++) {
        accum += lhs[i * K + k] * rhs[k * N + j];
      }
      out[i * N + j] = accum;
    }
  }
}

/* tensor_accessor_unary_ops.cc:109-127 */
void orc_transpose(float const *in, float *out, int64_t rows, int64_t cols) {
  for (int64_t i = 0; i < rows; i++) {
    for (int64_t j = 0; j < cols; j++) {
      out[j * rows + i] = in[i * cols + j];
    }
  }
}

/* tensor_accessor_unary_ops.cc:56-70: numpy-style broadcast (trailing dims
 * aligned, size-1 dims repeat). */
void orc_broadcast(float const *in, int64_t const *in_dims, int in_rank,
                   float *out, int64_t const *out_dims, int out_rank) {
  int64_t total = 1;
  for (int i = 0; i < out_rank; i++) {
    total *= out_dims[i];
  }
  int64_t coord[8];
  for (int64_t idx = 0; idx < total; idx++) {
    int64_t rem = idx;
    for (int i = out_rank - 1; i >= 0; i--) {
      coord[i] = rem % out_dims[i];
      rem /= out_dims[i];
    }
    int64_t off = 0, mult = 1;
    for (int i = in_rank - 1; i >= 0; i--) {
      int oi = i + (out_rank - in_rank);
      int64_t c = in_dims[i] == 1 ? 0 : coord[oi];
      off += c * mult;
      mult *= in_dims[i];
    }
    out[idx] = in[off];
  }
}

/* tensor_accessor_unary_ops.cc:174-192: sum over one dim, visiting inputs in
 * row-major order */
void orc_reduce_dim(float const *in, int64_t const *dims, int rank, int dim,
                    float *out) {
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < dim; i++) {
    outer *= dims[i];
  }
  for (int i = dim + 1; i < rank; i++) {
    inner *= dims[i];
  }
  int64_t R = dims[dim];
  for (int64_t i = 0; i < outer * inner; i++) {
    out[i] = 0.0f;
  }
  for (int64_t o = 0; o < outer; o++) {
    for (int64_t r = 0; r < R; r++) {
      for (int64_t i = 0; i < inner; i++) {
        out[o * inner + i] += in[(o * R + r) * inner + i];
      }
    }
  }
}

/* tensor_accessor_unary_ops.cc:32-45 (note `>=`) */
void orc_relu(float const *in, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    out[i] = in[i] >= 0 ? in[i] : 0;
  }
}

void orc_scale(float const *in, float c, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    out[i] = in[i] * c;
  }
}

void orc_add(float const *a, float const *b, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    out[i] = a[i] + b[i];
  }
}

/* -------------------------------------------------------------------- Linear */

/* linear_kernels_cpu.cc:12-43 */
int orc_linear_forward(int activation, float const *input, float *output,
                       float const *weight, float const *bias, int64_t batch,
                       int64_t in_dim, int64_t out_dim) {
  float *wt = (float *)malloc(sizeof(float) * (size_t)(in_dim * out_dim + 1));
  orc_transpose(weight, wt, out_dim, in_dim); /* -> [in, out] */
  orc_matmul(input, wt, output, batch, in_dim, out_dim);
  free(wt);
  if (bias) {
    int64_t bd[1] = {out_dim};
    int64_t od[2] = {batch, out_dim};
    float *bb = (float *)malloc(sizeof(float) * (size_t)(batch * out_dim + 1));
    orc_broadcast(bias, bd, 1, bb, od, 2);
    orc_add(output, bb, output, batch * out_dim);
    free(bb);
  }
  switch (activation) {
    case -1:
      break;
    case 0:
      orc_relu(output, output, batch * out_dim);
      break;
    case 1: /* sigmoid (not on the reference CPU path) */
      for (int64_t i = 0; i < batch * out_dim; i++) {
        output[i] = (float)(1.0 / (1.0 + exp(-(double)output[i])));
      }
      break;
    case 2:
      for (int64_t i = 0; i < batch * out_dim; i++) {
        output[i] = (float)tanh((double)output[i]);
      }
      break;
    default:
      return 1; /* the reference PANICs: "Unhandled activation function" */
  }
  return 0;
}

/* linear_kernels_cpu.cc:54-94 */
int orc_linear_backward(int activation, int relu_grad_mode,
                        float const *output, float const *output_grad,
                        float const *input, float *input_grad,
                        float const *weight, float *weight_grad,
                        float *bias_grad, int64_t batch, int64_t in_dim,
                        int64_t out_dim) {
  int64_t n = batch * out_dim;
  float *g = (float *)malloc(sizeof(float) * (size_t)(n + 1));
  switch (activation) {
    case -1:
      memcpy(g, output_grad, sizeof(float) * (size_t)n);
      break;
    case 0:
      for (int64_t i = 0; i < n; i++) {
        if (relu_grad_mode == 1) {
          /* single_element_relu_bwd applied to output_grad itself,
           * linear_kernels_cpu.cc:46-52,69-71 */
          g[i] = output_grad[i] > 0 ? 1.0f : 0.0f;
        } else {
          /* reluBackward, cuda_helper.cu:60-64 */
          g[i] = output[i] > 0.0f ? output_grad[i] : 0.0f;
        }
      }
      break;
    case 1: /* sigmoid_backward_function, cuda_helper.cu:87-91 */
      for (int64_t i = 0; i < n; i++) {
        g[i] = output_grad[i] * output[i] * (1.0f - output[i]);
      }
      break;
    case 2:
      for (int64_t i = 0; i < n; i++) {
        g[i] = output_grad[i] * (1.0f - output[i] * output[i]);
      }
      break;
    default:
      free(g);
      return 1;
  }
  if (input_grad) {
    orc_matmul(g, weight, input_grad, batch, out_dim, in_dim);
  }
  if (weight_grad) {
    float *xt = (float *)malloc(sizeof(float) * (size_t)(batch * in_dim + 1));
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(in_dim * out_dim + 1));
    orc_transpose(input, xt, batch, in_dim);            /* [in, batch] */
    orc_matmul(xt, g, tmp, in_dim, batch, out_dim);     /* [in, out]   */
    orc_transpose(tmp, weight_grad, in_dim, out_dim);   /* [out, in]   */
    free(xt);
    free(tmp);
  }
  if (bias_grad) {
    int64_t d[2] = {batch, out_dim};
    orc_reduce_dim(g, d, 2, 0, bias_grad);
  }
  free(g);
  return 0;
}

/* linear_kernels.cu:269-290: cublasSgeam(alpha = 1, dW, beta = lambda, W) -> dW */
void orc_linear_l2_regularizer_grad(float const *weight, float *weight_grad,
                                    int64_t n, float lambda) {
  for (int64_t i = 0; i < n; i++) {
    weight_grad[i] = 1.0f * weight_grad[i] + lambda * weight[i];
  }
}

void orc_gemm_f64(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                  float const *A, float const *B, float *C) {
#pragma omp parallel for schedule(static) if (M * N * K > 1000000)
  for (int64_t i = 0; i < M; i++) {
    for (int64_t j = 0; j < N; j++) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; k++) {
        double a = trans_a ? A[k * M + i] : A[i * K + k];
        double b = trans_b ? B[j * K + k] : B[k * N + j];
        acc += a * b;
      }
      C[i * N + j] = (float)acc;
    }
  }
}

/* -------------------------------------------------------------- element-wise */

/* element_unary_kernels.cu:104-170; relu/sigmoid/tanh/elu = cuDNN activation
 * definitions (element_unary_kernels.cu:58-86). Math in double, cast to T,
 * as the reference's GELU line does. */
int orc_element_unary_forward(int op, float s, float const *in, float *out,
                              int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double x = in[i];
    double r;
    switch (op) {
      case OP_SCALAR_MULTIPLY: r = (double)(in[i] * s); break;
      case OP_SCALAR_ADD: r = (double)(in[i] + s); break;
      case OP_SCALAR_SUB: r = (double)(in[i] - s); break;
      case OP_SCALAR_TRUE_DIV: r = (double)(in[i] / s); break;
      case OP_POW: r = pow(x, (double)s); break;
      case OP_EXP: r = exp(x); break;
      case OP_IDENTITY: r = x; break;
      case OP_GELU_REFERENCE_GRAD:
      case OP_GELU: r = x * 0.5 * erfc(-x * M_SQRT1_2); break;
      case OP_RSQRT: r = 1.0 / sqrt(x); break;
      case OP_SIN: r = sin(x); break;
      case OP_COS: r = cos(x); break;
      case OP_RELU: r = x > 0 ? x : 0; break;
      case OP_SIGMOID: r = 1.0 / (1.0 + exp(-x)); break;
      case OP_TANH: r = tanh(x); break;
      case OP_ELU: r = x > 0 ? x : (double)s * (exp(x) - 1.0); break;
      default: return 1;
    }
    out[i] = (float)r;
  }
  return 0;
}

/* element_unary_kernels.cu:172-250.  accumulate: -1 = the reference's per-op
 * behaviour (`=` for POW, GELU, RSQRT; `+=` otherwise), 0 / 1 = forced. */
int orc_element_unary_backward(int op, float s, float const *out,
                               float const *out_grad, float const *in,
                               float *in_grad, int64_t n, int accumulate) {
  int acc = accumulate;
  if (acc < 0) {
    acc = !(op == OP_POW || op == OP_GELU || op == OP_GELU_REFERENCE_GRAD ||
            op == OP_RSQRT);
  }
  for (int64_t i = 0; i < n; i++) {
    double x = in[i], y = out[i], dy = out_grad[i];
    double g;
    switch (op) {
      case OP_SCALAR_MULTIPLY: g = dy * s; break;
      case OP_SCALAR_ADD: g = dy; break;
      case OP_SCALAR_SUB: g = dy; break;
      case OP_SCALAR_TRUE_DIV: g = dy / s; break;
      case OP_POW: g = dy * s * pow(x, (double)s - 1.0); break;
      case OP_EXP: g = dy * exp(x); break;
      case OP_IDENTITY: g = dy; break;
      case OP_GELU: /* true derivative Phi(x) + x phi(x) */
        g = dy * (0.5 * erfc(-x * M_SQRT1_2) +
                  x * exp(-0.5 * x * x) / sqrt(2.0 * M_PI));
        break;
      case OP_GELU_REFERENCE_GRAD: /* literal element_unary_kernels.cu:226-231 */
        g = dy * (0.5 * erfc(-x * M_SQRT1_2) -
                  0.5 * M_SQRT1_2 * x * exp(-x * x * 0.5));
        break;
      case OP_RSQRT: g = -0.5 * dy * y * y * y; break;
      case OP_SIN: g = dy * cos(x); break;
      case OP_COS: g = dy * -sin(x); break;
      case OP_RELU: g = x > 0 ? dy : 0; break;
      case OP_SIGMOID: g = dy * y * (1.0 - y); break;
      case OP_TANH: g = dy * (1.0 - y * y); break;
      case OP_ELU: g = x > 0 ? dy : dy * (y + s); break;
      default: return 1;
    }
    in_grad[i] = acc ? (float)((double)in_grad[i] + g) : (float)g;
  }
  return 0;
}

int orc_element_binary_forward(int op, float const *lhs, float const *rhs,
                               float *out, int64_t n, int64_t nl, int64_t nr) {
  for (int64_t i = 0; i < n; i++) {
    float l = lhs[i % nl], r = rhs[i % nr];
    switch (op) {
      case OP_EW_ADD: out[i] = l + r; break;
      case OP_EW_SUB: out[i] = l - r; break;
      case OP_EW_MUL: out[i] = l * r; break;
      case OP_EW_DIV: out[i] = l / r; break;
      case OP_EW_MAX: out[i] = l >= r ? l : r; break;
      case OP_EW_MIN: out[i] = l <= r ? l : r; break;
      default: return 1;
    }
  }
  return 0;
}

/* element_binary_kernels.cu:27-81 with alpha = 1, beta = accumulate */
int orc_element_binary_backward(int op, float const *g, float const *lhs,
                                float const *rhs, float *dl, float *dr,
                                int64_t n, int accumulate) {
  float beta = accumulate ? 1.0f : 0.0f;
  for (int64_t i = 0; i < n; i++) {
    float ol = accumulate ? dl[i] : 0.0f;
    float orr = accumulate ? dr[i] : 0.0f;
    switch (op) {
      case OP_EW_ADD:
        dl[i] = g[i] + beta * ol;
        dr[i] = g[i] + beta * orr;
        break;
      case OP_EW_SUB:
        dl[i] = g[i] + beta * ol;
        dr[i] = -g[i] + beta * orr;
        break;
      case OP_EW_MUL:
        dl[i] = g[i] * rhs[i] + beta * ol;
        dr[i] = g[i] * lhs[i] + beta * orr;
        break;
      case OP_EW_DIV:
        dl[i] = g[i] / rhs[i] + beta * ol;
        dr[i] = -g[i] * lhs[i] / (rhs[i] * rhs[i]) + beta * orr;
        break;
      case OP_EW_MAX:
        dl[i] = (lhs[i] >= rhs[i]) ? g[i] + beta * ol : beta * ol;
        dr[i] = (rhs[i] >= lhs[i]) ? g[i] + beta * orr : beta * orr;
        break;
      case OP_EW_MIN:
        dl[i] = (lhs[i] <= rhs[i]) ? g[i] + beta * ol : beta * ol;
        dr[i] = (rhs[i] <= lhs[i]) ? g[i] + beta * orr : beta * orr;
        break;
      default:
        return 1;
    }
  }
  return 0;
}

/* ----------------------------------------------------------------- LayerNorm */

/* layer_norm_kernels.cu:69-112: biased variance max(E[x^2]-mean^2, 0),
 * rstd = rsqrt(var + eps).  Row sums are taken in double so the oracle is the
 * more exact side of the comparison. */
void orc_layer_norm_forward(float const *x, float *y, float const *gamma,
                            float const *beta, float *mean, float *rstd,
                            int64_t M, int64_t N, float eps) {
  for (int64_t i = 0; i < M; i++) {
    double s1 = 0.0, s2 = 0.0;
    for (int64_t j = 0; j < N; j++) {
      double v = x[i * N + j];
      s1 += v;
      s2 += v * v;
    }
    double scale = 1.0 / (double)N;
    double mu = s1 * scale;
    double var = s2 * scale - mu * mu;
    if (var < 0) {
      var = 0;
    }
    double rs = 1.0 / sqrt(var + (double)eps);
    if (mean) {
      mean[i] = (float)mu;
    }
    if (rstd) {
      rstd[i] = (float)rs;
    }
    for (int64_t j = 0; j < N; j++) {
      double g = gamma ? gamma[j] : 1.0;
      double b = beta ? beta[j] : 0.0;
      y[i * N + j] = (float)(((double)x[i * N + j] - mu) * rs * g + b);
    }
  }
}

/* layer_norm_kernels.cu:115-181 (ds/db, fused params c1/c2, dX) and :184-214
 * (dgamma/dbeta column sums) */
void orc_layer_norm_backward(float const *dy, float const *x,
                             float const *mean, float const *rstd,
                             float const *gamma, float *dx, float *dgamma,
                             float *dbeta, int64_t M, int64_t N,
                             int accumulate_dx) {
  double *dg = (double *)calloc((size_t)N + 1, sizeof(double));
  double *db = (double *)calloc((size_t)N + 1, sizeof(double));
  for (int64_t i = 0; i < M; i++) {
    double ds = 0.0, dbs = 0.0;
    double mu = mean[i], rs = rstd[i];
    for (int64_t j = 0; j < N; j++) {
      double g = gamma ? gamma[j] : 1.0;
      double d = dy[i * N + j], v = x[i * N + j];
      ds += d * v * g;
      dbs += d * g;
      dg[j] += d * (v - mu) * rs;
      db[j] += d;
    }
    double s = 1.0 / (double)N;
    double c1 = (dbs * mu - ds) * rs * rs * rs * s;
    double c2 = -(c1 * mu + dbs * rs * s);
    if (dx) {
      for (int64_t j = 0; j < N; j++) {
        double g = gamma ? gamma[j] : 1.0;
        double v = rs * dy[i * N + j] * g + c1 * x[i * N + j] + c2;
        dx[i * N + j] =
            accumulate_dx ? (float)((double)dx[i * N + j] + v) : (float)v;
      }
    }
  }
  for (int64_t j = 0; j < N; j++) {
    if (dgamma) {
      dgamma[j] = (float)dg[j];
    }
    if (dbeta) {
      dbeta[j] = (float)db[j];
    }
  }
  free(dg);
  free(db);
}

/* ------------------------------------------------------------------- Softmax */

void orc_softmax_forward(float const *x, float *y, int64_t outer, int64_t dim,
                         int64_t inner) {
  for (int64_t o = 0; o < outer; o++) {
    for (int64_t i = 0; i < inner; i++) {
      float const *xp = x + o * dim * inner + i;
      float *yp = y + o * dim * inner + i;
      double mx = -INFINITY;
      for (int64_t c = 0; c < dim; c++) {
        if (xp[c * inner] > mx) {
          mx = xp[c * inner];
        }
      }
      double sum = 0.0;
      for (int64_t c = 0; c < dim; c++) {
        sum += exp((double)xp[c * inner] - mx);
      }
      for (int64_t c = 0; c < dim; c++) {
        yp[c * inner] = (float)(exp((double)xp[c * inner] - mx) / sum);
      }
    }
  }
}

void orc_softmax_backward(float const *y, float const *dy, float *dx,
                          int64_t outer, int64_t dim, int64_t inner) {
  for (int64_t o = 0; o < outer; o++) {
    for (int64_t i = 0; i < inner; i++) {
      int64_t base = o * dim * inner + i;
      double dot = 0.0;
      for (int64_t c = 0; c < dim; c++) {
        dot += (double)y[base + c * inner] * (double)dy[base + c * inner];
      }
      for (int64_t c = 0; c < dim; c++) {
        dx[base + c * inner] = (float)((double)y[base + c * inner] *
                                       ((double)dy[base + c * inner] - dot));
      }
    }
  }
}

/* ------------------------------------------------------------------- Dropout */

static inline void mulhilo32(uint32_t a, uint32_t b, uint32_t *hi,
                             uint32_t *lo) {
  uint64_t p = (uint64_t)a * (uint64_t)b;
  *hi = (uint32_t)(p >> 32);
  *lo = (uint32_t)p;
}

/* Philox4x32-10 as published (Salmon, Moraes, Dror, Shaw: "Parallel random
 * numbers: as easy as 1, 2, 3", SC'11; Random123 philox.h): multipliers
 * 0xD2511F53 / 0xCD9E8D57, Weyl key increments 0x9E3779B9 / 0xBB67AE85. */
void orc_philox4x32_10(uint32_t const ctr_in[4], uint32_t const key_in[2],
                       uint32_t out[4]) {
  uint32_t c[4] = {ctr_in[0], ctr_in[1], ctr_in[2], ctr_in[3]};
  uint32_t k[2] = {key_in[0], key_in[1]};
  for (int r = 0; r < 10; r++) {
    uint32_t hi0, lo0, hi1, lo1;
    mulhilo32(0xD2511F53u, c[0], &hi0, &lo0);
    mulhilo32(0xCD9E8D57u, c[2], &hi1, &lo1);
    uint32_t n0 = hi1 ^ c[1] ^ k[0];
    uint32_t n1 = lo1;
    uint32_t n2 = hi0 ^ c[3] ^ k[1];
    uint32_t n3 = lo0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
    k[0] += 0x9E3779B9u;
    k[1] += 0xBB67AE85u;
  }
  out[0] = c[0]; out[1] = c[1]; out[2] = c[2]; out[3] = c[3];
}

static uint32_t dropout_threshold(float rate) {
  double t = ceil((double)rate * 65536.0);
  if (t < 0) {
    t = 0;
  }
  if (t > 65536.0) {
    t = 65536.0;
  }
  return (uint32_t)t;
}

/* element i (global index e = offset + i): counter (e/8 lo, e/8 hi, 0, 0),
 * key (seed lo, seed hi); the element's 16 bits are half (e%8)%2 (0 = low) of
 * word (e%8)/2; kept iff they are >= ceil(rate * 2^16). */
void orc_dropout_mask(uint8_t *mask, int64_t n, float rate, uint64_t seed,
                      uint64_t offset) {
  uint32_t thr = dropout_threshold(rate);
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint64_t cached_block = ~(uint64_t)0;
  uint32_t w[4] = {0, 0, 0, 0};
  for (int64_t i = 0; i < n; i++) {
    uint64_t e = offset + (uint64_t)i;
    uint64_t blk = e >> 3;
    if (blk != cached_block) {
      uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), 0u, 0u};
      orc_philox4x32_10(ctr, key, w);
      cached_block = blk;
    }
    uint32_t h = (uint32_t)(e & 7);
    uint32_t word = w[h >> 1];
    uint32_t half = (h & 1) ? (word >> 16) : (word & 0xffffu);
    mask[i] = (half >= thr) ? 1 : 0;
  }
}

void orc_dropout_forward(float const *x, float *y, int64_t n, float rate,
                         uint64_t seed, uint64_t offset) {
  uint8_t *m = (uint8_t *)malloc((size_t)n + 1);
  orc_dropout_mask(m, n, rate, seed, offset);
  float scale = 1.0f / (1.0f - rate);
  for (int64_t i = 0; i < n; i++) {
    y[i] = m[i] ? x[i] * scale : 0.0f;
  }
  free(m);
}

void orc_dropout_backward(float const *dy, float *dx, int64_t n, float rate,
                          uint64_t seed, uint64_t offset, int accumulate) {
  uint8_t *m = (uint8_t *)malloc((size_t)n + 1);
  orc_dropout_mask(m, n, rate, seed, offset);
  float scale = 1.0f / (1.0f - rate);
  for (int64_t i = 0; i < n; i++) {
    float g = m[i] ? dy[i] * scale : 0.0f;
    dx[i] = accumulate ? dx[i] + g : g;
  }
  free(m);
}

/* ----------------------------------------------------------------- Embedding */

/* embedding_kernels.cu:48-125 (true AVG: sum / bag) */
int orc_embedding_forward(int64_t const *idx, float *out, float const *w,
                          int aggr, int64_t num_bags, int64_t bag, int64_t dim,
                          int64_t num_entries) {
  if (aggr < 0 && bag != 1) {
    return 1;
  }
  for (int64_t b = 0; b < num_bags; b++) {
    for (int64_t d = 0; d < dim; d++) {
      float acc = 0.0f;
      for (int64_t j = 0; j < bag; j++) {
        int64_t row = idx[b * bag + j];
        if (row < 0 || row >= num_entries) {
          return 2;
        }
        acc = acc + w[row * dim + d];
      }
      if (aggr == 1) {
        acc = acc * (1.0f / (float)bag);
      }
      out[b * dim + d] = acc;
    }
  }
  return 0;
}

/* embedding_kernels.cu:128-317 with the atomics replaced by ordered adds */
int orc_embedding_backward(int64_t const *idx, float const *g, float *dw,
                           int aggr, int64_t num_bags, int64_t bag, int64_t dim,
                           int64_t num_entries) {
  float scale = aggr == 1 ? 1.0f / (float)bag : 1.0f;
  for (int64_t b = 0; b < num_bags; b++) {
    for (int64_t j = 0; j < bag; j++) {
      int64_t row = idx[b * bag + j];
      if (row < 0 || row >= num_entries) {
        return 2;
      }
      for (int64_t d = 0; d < dim; d++) {
        float v = aggr == 1 ? g[b * dim + d] * scale : g[b * dim + d];
        dw[row * dim + d] += v;
      }
    }
  }
  return 0;
}

int orc_embedding_backward_f64(int64_t const *idx, float const *g, float *dw,
                               int aggr, int64_t num_bags, int64_t bag,
                               int64_t dim, int64_t num_entries) {
  double *acc = (double *)calloc((size_t)(num_entries * dim) + 1, sizeof(double));
  float scale = aggr == 1 ? 1.0f / (float)bag : 1.0f;
  for (int64_t b = 0; b < num_bags; b++) {
    for (int64_t j = 0; j < bag; j++) {
      int64_t row = idx[b * bag + j];
      if (row < 0 || row >= num_entries) {
        free(acc);
        return 2;
      }
      for (int64_t d = 0; d < dim; d++) {
        float v = aggr == 1 ? g[b * dim + d] * scale : g[b * dim + d];
        acc[row * dim + d] += (double)v;
      }
    }
  }
  for (int64_t i = 0; i < num_entries * dim; i++) {
    dw[i] = (float)((double)dw[i] + acc[i]);
  }
  free(acc);
  return 0;
}

/* ----------------------------------------------------------------- attention */

#define QI(b, s, h, d, S, H, D) ((((b) * (S) + (s)) * (H) + (h)) * (D) + (d))

/* q, k: [B, S, H, D]; v, o: [B, S, H, Dv] (the value head size may differ from
 * the query/key head size: vProjSize vs qProjSize in attention_kernels.cu:78-80).
 * Every (batch, head) pair is independent and is computed by one thread in a
 * fixed order, so the result does not depend on the thread count. */
void orc_attention_forward(float const *q, float const *k, float const *v,
                           float *o, float *lse, int64_t B, int64_t H,
                           int64_t Sq, int64_t Skv, int64_t D, int64_t Dv,
                           float scale, int causal, int bf16_mode) {
#pragma omp parallel for schedule(dynamic) if (B * H * Sq * Skv > 100000)
  for (int64_t bh = 0; bh < B * H; bh++) {
    int64_t const b = bh / H, h = bh % H;
    double *p = (double *)malloc(sizeof(double) * (size_t)(Skv + 1));
    for (int64_t i = 0; i < Sq; i++) {
      int64_t lim = causal ? (i + 1 < Skv ? i + 1 : Skv) : Skv;
      double mx = -INFINITY;
      for (int64_t j = 0; j < lim; j++) {
        double s = 0.0;
        for (int64_t d = 0; d < D; d++) {
          s += (double)q[QI(b, i, h, d, Sq, H, D)] *
               (double)k[QI(b, j, h, d, Skv, H, D)];
        }
        s *= (double)scale;
        p[j] = s;
        if (s > mx) {
          mx = s;
        }
      }
      double sum = 0.0;
      for (int64_t j = 0; j < lim; j++) {
        p[j] = exp(p[j] - mx);
        sum += p[j];
      }
      if (lse) {
        lse[(b * H + h) * Sq + i] = (float)(mx + log(sum));
      }
      if (bf16_mode) {
        /* the device rounds the unnormalised probabilities to bf16 before
         * the PV product and divides by the fp32 row sum after */
        for (int64_t j = 0; j < lim; j++) {
          p[j] = (double)orc_round_bf16((float)p[j]);
        }
      }
      for (int64_t d = 0; d < Dv; d++) {
        double acc = 0.0;
        for (int64_t j = 0; j < lim; j++) {
          acc += p[j] * (double)v[QI(b, j, h, d, Skv, H, Dv)];
        }
        float r = (float)(acc / sum);
        o[QI(b, i, h, d, Sq, H, Dv)] = bf16_mode ? orc_round_bf16(r) : r;
      }
    }
    free(p);
  }
}

void orc_attention_backward(float const *q, float const *k, float const *v,
                            float const *d_o, float *dq, float *dk, float *dv,
                            int64_t B, int64_t H, int64_t Sq, int64_t Skv,
                            int64_t D, int64_t Dv, float scale, int causal) {
  double *dqa = (double *)calloc((size_t)(B * Sq * H * D) + 1, sizeof(double));
  double *dka = (double *)calloc((size_t)(B * Skv * H * D) + 1, sizeof(double));
  double *dva = (double *)calloc((size_t)(B * Skv * H * Dv) + 1, sizeof(double));
  /* a (batch, head) pair touches only its own slices of the accumulators */
#pragma omp parallel for schedule(dynamic) if (B * H * Sq * Skv > 100000)
  for (int64_t bh = 0; bh < B * H; bh++) {
    int64_t const b = bh / H, h = bh % H;
    double *p = (double *)malloc(sizeof(double) * (size_t)(Skv + 1));
    double *dp = (double *)malloc(sizeof(double) * (size_t)(Skv + 1));
    for (int64_t i = 0; i < Sq; i++) {
      int64_t lim = causal ? (i + 1 < Skv ? i + 1 : Skv) : Skv;
      double mx = -INFINITY;
      for (int64_t j = 0; j < lim; j++) {
        double s = 0.0;
        for (int64_t d = 0; d < D; d++) {
          s += (double)q[QI(b, i, h, d, Sq, H, D)] *
               (double)k[QI(b, j, h, d, Skv, H, D)];
        }
        p[j] = s * (double)scale;
        if (p[j] > mx) {
          mx = p[j];
        }
      }
      double sum = 0.0;
      for (int64_t j = 0; j < lim; j++) {
        p[j] = exp(p[j] - mx);
        sum += p[j];
      }
      double dot = 0.0; /* sum_j P_ij dP_ij */
      for (int64_t j = 0; j < lim; j++) {
        p[j] /= sum;
        double t = 0.0;
        for (int64_t d = 0; d < Dv; d++) {
          t += (double)d_o[QI(b, i, h, d, Sq, H, Dv)] *
               (double)v[QI(b, j, h, d, Skv, H, Dv)];
        }
        dp[j] = t;
        dot += p[j] * t;
      }
      for (int64_t j = 0; j < lim; j++) {
        double ds = p[j] * (dp[j] - dot) * (double)scale;
        for (int64_t d = 0; d < D; d++) {
          dqa[QI(b, i, h, d, Sq, H, D)] +=
              ds * (double)k[QI(b, j, h, d, Skv, H, D)];
          dka[QI(b, j, h, d, Skv, H, D)] +=
              ds * (double)q[QI(b, i, h, d, Sq, H, D)];
        }
        for (int64_t d = 0; d < Dv; d++) {
          dva[QI(b, j, h, d, Skv, H, Dv)] +=
              p[j] * (double)d_o[QI(b, i, h, d, Sq, H, Dv)];
        }
      }
    }
    free(p);
    free(dp);
  }
  for (int64_t i = 0; i < B * Sq * H * D; i++) {
    dq[i] = (float)dqa[i];
  }
  for (int64_t i = 0; i < B * Skv * H * D; i++) {
    dk[i] = (float)dka[i];
  }
  for (int64_t i = 0; i < B * Skv * H * Dv; i++) {
    dv[i] = (float)dva[i];
  }
  free(dqa); free(dka); free(dva);
}

/* ------------------------------------------------------- MultiHeadAttention */

static void maybe_round(float *x, int64_t n, int bf16_mode) {
  if (bf16_mode) {
    orc_round_bf16_array(x, n);
  }
}

/* out = softmax(scale (q W_Q^T)(k W_K^T)^T)(v W_V^T) W_O^T per head,
 * concatenated over heads before W_O (cudnnMultiHeadAttnForward as set up in
 * attention_kernels.cu:73-92: no biases, no dropout, full window). */
void orc_mha_forward(orc_mha_desc_t const *d, float const *query,
                     float const *key, float const *value, float const *weight,
                     float *output, int bf16_mode) {
  int64_t B = d->num_samples, H = d->num_heads;
  int64_t Sq = d->qo_seq_length, Skv = d->kv_seq_length;
  int64_t Dq = d->q_proj_size, Dk = d->k_proj_size, Dv = d->v_proj_size;
  float const *wq = weight;
  float const *wk = wq + H * Dq * d->q_size;
  float const *wv = wk + H * Dk * d->k_size;
  float const *wo = wv + H * Dv * d->v_size;
  float *Q = (float *)malloc(sizeof(float) * (size_t)(B * Sq * H * Dq + 1));
  float *K = (float *)malloc(sizeof(float) * (size_t)(B * Skv * H * Dk + 1));
  float *V = (float *)malloc(sizeof(float) * (size_t)(B * Skv * H * Dv + 1));
  float *C = (float *)malloc(sizeof(float) * (size_t)(B * Sq * H * Dv + 1));
  orc_gemm_f64(0, 1, B * Sq, H * Dq, d->q_size, query, wq, Q);
  orc_gemm_f64(0, 1, B * Skv, H * Dk, d->k_size, key, wk, K);
  orc_gemm_f64(0, 1, B * Skv, H * Dv, d->v_size, value, wv, V);
  maybe_round(Q, B * Sq * H * Dq, bf16_mode);
  maybe_round(K, B * Skv * H * Dk, bf16_mode);
  maybe_round(V, B * Skv * H * Dv, bf16_mode);
  /* the reference asserts kProjSize == qProjSize (attention_kernels.cu:61);
   * the value head size is its own */
  orc_attention_forward(Q, K, V, C, NULL, B, H, Sq, Skv, Dq, Dv, d->scale,
                        d->causal, bf16_mode);
  orc_gemm_f64(0, 1, B * Sq, d->o_proj_size, H * Dv, C, wo, output);
  maybe_round(output, B * Sq * d->o_proj_size, bf16_mode);
  free(Q); free(K); free(V); free(C);
}

void orc_mha_backward(orc_mha_desc_t const *d, float const *query,
                      float const *key, float const *value,
                      float const *weight, float const *output_grad,
                      float *dquery, float *dkey, float *dvalue,
                      float *dweight, int bf16_mode) {
  int64_t B = d->num_samples, H = d->num_heads;
  int64_t Sq = d->qo_seq_length, Skv = d->kv_seq_length;
  int64_t Dq = d->q_proj_size, Dk = d->k_proj_size, Dv = d->v_proj_size;
  int64_t nq = H * Dq * d->q_size, nk = H * Dk * d->k_size;
  int64_t nv = H * Dv * d->v_size, no = d->o_proj_size * H * Dv;
  float const *wq = weight;
  float const *wk = wq + nq;
  float const *wv = wk + nk;
  float const *wo = wv + nv;
  int64_t TQ = B * Sq, TK = B * Skv;
  float *Q = (float *)malloc(sizeof(float) * (size_t)(TQ * H * Dq + 1));
  float *K = (float *)malloc(sizeof(float) * (size_t)(TK * H * Dk + 1));
  float *V = (float *)malloc(sizeof(float) * (size_t)(TK * H * Dv + 1));
  float *C = (float *)malloc(sizeof(float) * (size_t)(TQ * H * Dv + 1));
  float *dC = (float *)malloc(sizeof(float) * (size_t)(TQ * H * Dv + 1));
  float *dQ = (float *)malloc(sizeof(float) * (size_t)(TQ * H * Dq + 1));
  float *dK = (float *)malloc(sizeof(float) * (size_t)(TK * H * Dk + 1));
  float *dV = (float *)malloc(sizeof(float) * (size_t)(TK * H * Dv + 1));
  orc_gemm_f64(0, 1, TQ, H * Dq, d->q_size, query, wq, Q);
  orc_gemm_f64(0, 1, TK, H * Dk, d->k_size, key, wk, K);
  orc_gemm_f64(0, 1, TK, H * Dv, d->v_size, value, wv, V);
  maybe_round(Q, TQ * H * Dq, bf16_mode);
  maybe_round(K, TK * H * Dk, bf16_mode);
  maybe_round(V, TK * H * Dv, bf16_mode);
  orc_attention_forward(Q, K, V, C, NULL, B, H, Sq, Skv, Dq, Dv, d->scale,
                        d->causal, bf16_mode);
  /* dC = dOut . W_O ; dW_O += dOut^T . C */
  orc_gemm_f64(0, 0, TQ, H * Dv, d->o_proj_size, output_grad, wo, dC);
  maybe_round(dC, TQ * H * Dv, bf16_mode);
  float *tmp = (float *)malloc(sizeof(float) *
                               (size_t)((nq > nk ? nq : nk) + nv + no + 1));
  orc_gemm_f64(1, 0, d->o_proj_size, H * Dv, TQ, output_grad, C, tmp);
  for (int64_t i = 0; i < no; i++) {
    dweight[nq + nk + nv + i] += tmp[i];
  }
  orc_attention_backward(Q, K, V, dC, dQ, dK, dV, B, H, Sq, Skv, Dq, Dv,
                         d->scale, d->causal);
  maybe_round(dQ, TQ * H * Dq, bf16_mode);
  maybe_round(dK, TK * H * Dk, bf16_mode);
  maybe_round(dV, TK * H * Dv, bf16_mode);
  /* input grads: dquery = dQ . W_Q etc.; weight grads: dW_Q += dQ^T . query */
  orc_gemm_f64(0, 0, TQ, d->q_size, H * Dq, dQ, wq, dquery);
  orc_gemm_f64(0, 0, TK, d->k_size, H * Dk, dK, wk, dkey);
  orc_gemm_f64(0, 0, TK, d->v_size, H * Dv, dV, wv, dvalue);
  orc_gemm_f64(1, 0, H * Dq, d->q_size, TQ, dQ, query, tmp);
  for (int64_t i = 0; i < nq; i++) {
    dweight[i] += tmp[i];
  }
  orc_gemm_f64(1, 0, H * Dk, d->k_size, TK, dK, key, tmp);
  for (int64_t i = 0; i < nk; i++) {
    dweight[nq + i] += tmp[i];
  }
  orc_gemm_f64(1, 0, H * Dv, d->v_size, TK, dV, value, tmp);
  for (int64_t i = 0; i < nv; i++) {
    dweight[nq + nk + i] += tmp[i];
  }
  free(tmp);
  free(Q); free(K); free(V); free(C); free(dC); free(dQ); free(dK); free(dV);
}

/* ------------------------------------------------------- optimizer updates */

void orc_sgd_update(float lr, float momentum, int nesterov, float weight_decay,
                    float const *grad, int64_t n, int replicas, float *w,
                    float *v) {
  for (int64_t i = 0; i < n; i++) {
    float g = grad[i];
    for (int r = 1; r < replicas; r++) {
      g = g + grad[(int64_t)r * n + i];
    }
    float t = weight_decay * w[i];
    float gt = g + t;
    if (momentum > 0.0f) {
      float vm = v[i] * momentum;
      float vn = vm + gt;
      v[i] = vn;
      if (nesterov) {
        float mv = momentum * vn;
        gt = gt + mv;
      } else {
        gt = vn;
      }
    }
    float step = lr * gt;
    w[i] = w[i] - step;
  }
}

void orc_adam_update(float alpha_t, float beta1, float beta2, float weight_decay,
                     float epsilon, float const *grad, int64_t n, int replicas,
                     float *w, float *vv, float *mm) {
  for (int64_t i = 0; i < n; i++) {
    float g = grad[i];
    for (int r = 1; r < replicas; r++) {
      g = g + grad[(int64_t)r * n + i];
    }
    float t = weight_decay * w[i];
    float gt = g + t;
    float a = beta1 * mm[i];
    float c1 = 1.0f - beta1;
    float b = c1 * gt;
    float mt = a + b;
    float c = beta2 * vv[i];
    float c2 = 1.0f - beta2;
    float d = c2 * gt;
    float e = d * gt;
    float vt = c + e;
    mm[i] = mt;
    vv[i] = vt;
    float num = alpha_t * mt;
    float den = sqrtf(vt) + epsilon;
    float q = num / den;
    w[i] = w[i] - q;
  }
}

/* ------------------------------------------------------------ loss backward */

void orc_sparse_cce_loss_backward(float *dlogit, float const *logit,
                                  int const *label, int64_t volume,
                                  int64_t num_samples, int64_t num_classes,
                                  int k, float scale_factor) {
  /* copy, subtract 1 at the label, scale by scale_factor * k */
  memcpy(dlogit, logit, sizeof(float) * (size_t)volume);
  for (int64_t i = 0; i < num_samples; i++) {
    int64_t l = label[i / k];
    if (l >= 0 && l < num_classes) {
      dlogit[i * num_classes + l] -= 1.0f;
    }
  }
  float s = scale_factor * (float)k;
  for (int64_t i = 0; i < volume; i++) {
    dlogit[i] = dlogit[i] * s;
  }
}

void orc_difference_loss_backward(float *dlogit, float const *logit,
                                  float const *label, int64_t volume,
                                  float scale_factor) {
  for (int64_t i = 0; i < volume; i++) {
    float d = logit[i] - label[i];
    dlogit[i] = d * scale_factor;
  }
}

void orc_identity_loss_backward(float *dloss, int64_t volume, float scale_factor) {
  for (int64_t i = 0; i < volume; i++) {
    dloss[i] = 1.0f * scale_factor;
  }
}

/* ------------------------------------------------------------------ concat */
void orc_concat_forward(float *out, float const *const *in, int64_t const *blk,
                        int n, int64_t num_blocks) {
  int64_t out_blk = 0;
  for (int i = 0; i < n; i++) {
    out_blk += blk[i];
  }
  int64_t offset = 0;
  for (int i = 0; i < n; i++) {
    /* copy_with_stride(output + offset, input, num_blocks, out_blk, blk[i]) */
    for (int64_t b = 0; b < num_blocks; b++) {
      for (int64_t j = 0; j < blk[i]; j++) {
        out[b * out_blk + offset + j] = in[i][b * blk[i] + j];
      }
    }
    offset += blk[i];
  }
}

void orc_concat_backward(float const *dout, float *const *din,
                         int64_t const *blk, int n, int64_t num_blocks,
                         int accumulate) {
  int64_t out_blk = 0;
  for (int i = 0; i < n; i++) {
    out_blk += blk[i];
  }
  int64_t offset = 0;
  for (int i = 0; i < n; i++) {
    /* add_with_stride(input_grad, output_grad + offset, ...) */
    for (int64_t b = 0; b < num_blocks; b++) {
      for (int64_t j = 0; j < blk[i]; j++) {
        float g = dout[b * out_blk + offset + j];
        float *d = &din[i][b * blk[i] + j];
        *d = accumulate ? *d + g : g;
      }
    }
    offset += blk[i];
  }
}

/* --------------------------------------------------------------- transpose */
void orc_transpose_nd(float const *in, float *out, int nd, int64_t const *in_dim,
                      int const *perm, int accumulate) {
  int64_t in_stride[8], out_dim[8], idx[8];
  int64_t s = 1, total = 1;
  for (int i = nd - 1; i >= 0; i--) {
    in_stride[i] = s;
    s *= in_dim[i];
  }
  for (int i = 0; i < nd; i++) {
    out_dim[i] = in_dim[perm[i]];
    total *= out_dim[i];
    idx[i] = 0;
  }
  for (int64_t o = 0; o < total; o++) {
    int64_t src = 0;
    for (int i = 0; i < nd; i++) {
      src += idx[i] * in_stride[perm[i]];
    }
    out[o] = accumulate ? out[o] + in[src] : in[src];
    for (int i = nd - 1; i >= 0; i--) { /* next output coordinate, row-major */
      if (++idx[i] < out_dim[i]) {
        break;
      }
      idx[i] = 0;
    }
  }
}

/* ------------------------------------------------------------------ gather */
void orc_gather_forward(float const *in, int64_t const *index, float *out,
                        int64_t outer, int64_t in_dim, int64_t out_dim,
                        int64_t stride) {
  int64_t total = outer * out_dim * stride;
  for (int64_t o = 0; o < total; o++) {
    int64_t outer_index = o / (stride * out_dim);
    int64_t left_over = o % stride;
    int64_t j = index[o];
    out[o] = (j >= 0 && j < in_dim)
                 ? in[outer_index * (stride * in_dim) + j * stride + left_over]
                 : 0.0f;
  }
}

void orc_gather_backward(float const *dout, int64_t const *index, float *din,
                         int64_t outer, int64_t in_dim, int64_t out_dim,
                         int64_t stride) {
  int64_t total = outer * out_dim * stride;
  for (int64_t o = 0; o < total; o++) {
    int64_t outer_index = o / (stride * out_dim);
    int64_t left_over = o % stride;
    int64_t j = index[o];
    if (j >= 0 && j < in_dim) {
      din[outer_index * (stride * in_dim) + j * stride + left_over] += dout[o];
    }
  }
}
