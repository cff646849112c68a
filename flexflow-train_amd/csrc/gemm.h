// Internal GEMM interface shared by Linear, the attention projections and the
// public ffk_gemm entry point.
#pragma once
#include "ffk_common.h"
#include "dropout_rng.h"

namespace ffk {

struct GemmEpilogue {
  void const *bias = nullptr;  // [N] in the GEMM dtype, added to every row
  int activation = FFK_ACT_NONE;
  bool accumulate = false;     // C += result instead of C = result
  // Optional fp32 scratch for split-K (used when the output has too few tiles
  // to occupy the chip); gemm_splitk_workspace_bytes() says how much helps.
  void *splitk_ws = nullptr;
  size_t splitk_ws_bytes = 0;
  // Optional element-wise operators applied to the output tile while it is
  // written (bf16 only, see gemm_tail_supported).  With a tail the GEMM gives
  // the bits of the separate kernels run after it:
  //   kTailGeluDropout     C = result (kept: backward reads the pre-activation),
  //                        tail_out = dropout(GELU(C))
  //   kTailDropoutGeluGrad C = dropout_backward(result) * GELU'(tail_in); the
  //                        plain result is not stored
  //   kTailDropoutAdd      C = tail_in + dropout(result); the plain result is
  //                        not stored
  // tail_in / tail_out are dense [M, N] tensors, the dropout stream is indexed
  // by m * N + n from tail_dropout.offset.
  enum Tail { kTailNone = 0, kTailGeluDropout = 1, kTailDropoutGeluGrad = 2, kTailDropoutAdd = 3 };
  int tail = kTailNone;
  void const *tail_in = nullptr;
  void *tail_out = nullptr;
  DropoutParams tail_dropout = {};
  // kTailDropoutGeluGrad, optional: the GEMM also leaves the partial column
  // sums of what it stores (colsum_partials_elems(M, N) floats, the partials
  // colsum_dispatch would compute from the stored tensor); colsum_finish adds
  // them up into the column sums (+)= out.
  float *tail_colsum_partials = nullptr;
};
int colsum_finish(hipStream_t stream, int dtype, float const *partials, int64_t M, int64_t N, void *out,
                  bool accumulate);

// Whether gemm_dispatch can run this GEMM with ep.tail (it fails otherwise).
bool gemm_tail_supported(int dtype, bool trans_a, bool trans_b, int64_t M, int64_t N,
                         int64_t K, void const *A, int64_t lda, void const *B, int64_t ldb,
                         void const *C, int64_t ldc, GemmEpilogue const &ep);

// C[M,N] (+)= op(A) . op(B), fp32 accumulation.
//   trans_a == false: A is [M,K] row-major (lda = K); true: A is [K,M] (lda = M)
//   trans_b == false: B is [K,N] row-major (ldb = N); true: B is [N,K] (ldb = K)
// lda/ldb/ldc are row strides in elements (>= the dense value), so strided
// views (column slices of a fused buffer) can be used directly.
int gemm_dispatch(hipStream_t stream, int dtype, bool trans_a, bool trans_b,
                  int64_t M, int64_t N, int64_t K, void const *A, int64_t lda,
                  void const *B, int64_t ldb, void *C, int64_t ldc,
                  GemmEpilogue const &ep);

// Two GEMMs of the same kind (same transposes, same reduction length K, no
// bias or activation, same accumulate switch) in ONE launch: for two outputs
// that each leave part of the chip idle (the two weight gradients of an
// attention block).  Each problem's result is the bits of gemm_dispatch on it
// alone with the 128x128 tile.  gemm_pair_supported says whether the pair
// runs (BF16, outputs multiples of 128, K a multiple of 64, 16-byte aligned
// operands); gemm_dispatch_pair fails otherwise.
struct GemmProblem {
  int64_t M, N;
  void const *A;
  int64_t lda;
  void const *B;
  int64_t ldb;
  void *C;
  int64_t ldc;
};
bool gemm_pair_supported(int dtype, bool trans_a, bool trans_b, int64_t K, GemmProblem const &p0,
                         GemmProblem const &p1);
int gemm_dispatch_pair(hipStream_t stream, int dtype, bool trans_a, bool trans_b, int64_t K,
                       GemmProblem const &p0, GemmProblem const &p1, bool accumulate);

// Scratch bytes with which a bf16 GEMM of this shape would split its reduction
// (0: it would not).
size_t gemm_splitk_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K);

// out[N] (+)= sum over the M rows of X[M,N] (ldx row stride); `partials` is
// fp32 scratch of colsum_partials_elems(M, N) floats.
int64_t colsum_partials_elems(int64_t M, int64_t N);
// dx[M,N] = dropout_backward(dy) and colsum (+)= its column sums (the bias
// gradient of the Linear whose output the dropout follows), one pass over dy.
// The sums are taken over dx as stored, in the order colsum_dispatch uses, so
// they are the bits of the two separate kernels.  FFK_ERR_UNSUPPORTED (nothing
// launched, no message) when the shape has no vector kernel.
int dropout_backward_colsum(hipStream_t stream, int dtype, void const *dy, void *dx, int64_t M,
                            int64_t N, void *colsum, bool accumulate, float *partials,
                            DropoutParams const &drop);
int colsum_dispatch(hipStream_t stream, int dtype, void const *X, int64_t ldx,
                    int64_t M, int64_t N, void *out, bool accumulate,
                    float *partials);

}  // namespace ffk
