"""Linear / GEMM parity: HIP kernels through the C ABI against the oracle."""
import json
import os
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def test_linear_reference_kat_fp32(ffk, golden_dir):
    k = json.load(open(os.path.join(golden_dir, "linear_kat.json")))
    say("linear KAT 4x3 . 3x2 fp32")
    x = to_dev(np.array(k["input"], np.float32), torch)
    w = to_dev(np.array(k["projection"], np.float32), torch)
    b = to_dev(np.array(k["bias"], np.float32), torch)
    y = ffk.linear_forward(x, w, b)
    assert np.array_equal(to_np(y), np.array(k["output"], np.float32))
    dy = to_dev(np.array(k["output_grad"], np.float32), torch)
    dx, dw, db = torch.zeros_like(x), torch.zeros_like(w), torch.zeros_like(b)
    ffk.linear_backward(y, dy, x, w, dx, dw, db)
    assert np.array_equal(to_np(dx), np.array(k["input_grad"], np.float32))
    assert np.array_equal(to_np(dw), np.array(k["projection_grad"], np.float32))
    assert np.array_equal(to_np(db), np.array(k["bias_grad"], np.float32))


def _cfg1_inputs(seed=0, batch=32, in_dim=64, out_dim=128):
    g = rng(seed)
    x = g.uniform(-1, 1, (batch, in_dim)).astype(np.float32)
    w = (g.standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
    b = (g.standard_normal((out_dim,)) * 0.02).astype(np.float32)
    dy = g.standard_normal((batch, out_dim)).astype(np.float32)
    return x, w, b, dy


@pytest.mark.parametrize("relu_grad_mode", [0, 1])
def test_linear_config1_fp32_relu(ffk, oracle, relu_grad_mode):
    """BASELINE config 1: fp32 [32,64] . [128,64]^T + bias, ReLU; both readings
    of the ReLU gradient (reference GPU helper / reference CPU text)."""
    x, w, b, dy = _cfg1_inputs()
    say("linear cfg1 fp32 relu mode", relu_grad_mode)
    y_ref = oracle.linear_forward(x, w, b, activation=0)
    dx_ref, dw_ref, db_ref = oracle.linear_backward(y_ref, dy, x, w, activation=0,
                                                    relu_grad_mode=relu_grad_mode)
    xd, wd, bd, dyd = (to_dev(a, torch) for a in (x, w, b, dy))
    y = ffk.linear_forward(xd, wd, bd, activation=ffk.ACT_RELU)
    assert_close(to_np(y), y_ref, FP32_RTOL, "y")
    dx, dw, db = torch.zeros_like(xd), torch.zeros_like(wd), torch.zeros_like(bd)
    ffk.linear_backward(y, dyd, xd, wd, dx, dw, db, activation=ffk.ACT_RELU,
                        relu_grad_mode=relu_grad_mode)
    assert_close(to_np(dx), dx_ref, FP32_RTOL, "dx")
    assert_close(to_np(dw), dw_ref, FP32_RTOL, "dw")
    assert_close(to_np(db), db_ref, FP32_RTOL, "db")
    # accumulate (reference GPU beta = 1): a second call doubles the gradients
    ffk.linear_backward(y, dyd, xd, wd, dx, dw, db, activation=ffk.ACT_RELU,
                        relu_grad_mode=relu_grad_mode, accumulate=True)
    assert_close(to_np(dx), 2 * dx_ref, FP32_RTOL, "dx acc")
    assert_close(to_np(dw), 2 * dw_ref, FP32_RTOL, "dw acc")
    assert_close(to_np(db), 2 * db_ref, FP32_RTOL, "db acc")


@pytest.mark.parametrize("shape", [(1, 1, 1), (5, 3, 7), (33, 65, 129), (70, 17, 64), (128, 256, 96)])
@pytest.mark.parametrize("act", [-1, 0, 1, 2])
def test_linear_fp32_ragged(ffk, oracle, shape, act):
    batch, in_dim, out_dim = shape
    say("linear fp32 ragged", shape, "act", act)
    x, w, b, dy = _cfg1_inputs(seed=batch * 1000 + in_dim, batch=batch, in_dim=in_dim, out_dim=out_dim)
    w = w * 20
    y_ref = oracle.linear_forward(x, w, b, activation=act)
    dx_ref, dw_ref, db_ref = oracle.linear_backward(y_ref, dy, x, w, activation=act)
    xd, wd, bd, dyd = (to_dev(a, torch) for a in (x, w, b, dy))
    y = ffk.linear_forward(xd, wd, bd, activation=act)
    assert_close(to_np(y), y_ref, FP32_RTOL, "y")
    dx, dw, db = torch.zeros_like(xd), torch.zeros_like(wd), torch.zeros_like(bd)
    ffk.linear_backward(to_dev(y_ref, torch), dyd, xd, wd, dx, dw, db, activation=act)
    assert_close(to_np(dx), dx_ref, FP32_RTOL, "dx")
    assert_close(to_np(dw), dw_ref, FP32_RTOL, "dw")
    assert_close(to_np(db), db_ref, FP32_RTOL, "db")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(32, 64, 128), (7, 5, 3), (128, 1024, 512)])
def test_linear_backward_with_l2_regularizer(ffk, oracle, dtype, shape):
    """Linear backward followed by the regulariser's term (linear_kernels.cu:269-290):
    dW = (dW + g^T x) + lambda W, twice in a row as the reference's accumulating path runs it."""
    batch, in_dim, out_dim = shape
    lam = 0.25
    say("linear backward + L2 regulariser", dtype, shape)
    x, w, b, dy = _cfg1_inputs(seed=3, batch=batch, in_dim=in_dim, out_dim=out_dim)
    w = w * 20
    bf = dtype == "bf16"
    if bf:
        x, w, dy = bf16_round(x), bf16_round(w), bf16_round(dy)
    rnd = bf16_round if bf else (lambda a: a)
    _, dw1, _ = oracle.linear_backward(None, dy, x, w)
    want1 = rnd(oracle.linear_l2_regularizer_grad(w, rnd(dw1), lam))
    want2 = rnd(oracle.linear_l2_regularizer_grad(w, rnd(want1 + dw1), lam))
    tt = torch.bfloat16 if bf else torch.float32
    xd, wd, dyd = (to_dev(a, torch, tt) for a in (x, w, dy))
    dw = torch.zeros_like(wd)
    ffk.linear_backward(None, dyd, xd, wd, None, dw, None, accumulate=True)
    ffk.linear_l2_regularizer_grad(wd, dw, lam)
    tol = BF16_RTOL if bf else FP32_RTOL
    assert_close(to_np(dw), want1, tol, "dw + lambda w")
    ffk.linear_backward(None, dyd, xd, wd, None, dw, None, accumulate=True)
    ffk.linear_l2_regularizer_grad(wd, dw, lam)
    assert_close(to_np(dw), want2, tol, "second call")
    # the term alone, on a gradient of zeros, is lambda W to the last bit in fp32
    z = torch.zeros_like(wd)
    ffk.linear_l2_regularizer_grad(wd, z, lam)
    if not bf:
        assert np.array_equal(to_np(z), oracle.linear_l2_regularizer_grad(w, np.zeros_like(w), lam))


@pytest.mark.parametrize("act", [-1, 0, 1, 2])
@pytest.mark.parametrize("shape", [(32, 64, 128), (70, 17, 65), (1, 1, 1), (300, 200, 130), (1024, 96, 80), (1100, 64, 72)])
def test_small_fp32_backward_in_one_launch_equals_the_general_path(ffk, oracle, shape, act):
    """A small fp32 backward with all three gradients runs as ONE launch (activation gradient,
    both products and the bias sums as jobs of one grid); asked for one gradient at a time the
    same entry point takes the general path (one kernel per product).  Same values either way,
    both against the oracle, with and without accumulation.  The last shape's batch is beyond
    the reduction depth the one-launch kernel takes: both calls go the general way."""
    batch, in_dim, out_dim = shape
    say("small fp32 linear backward, one launch vs general", shape, "act", act)
    x, w, b, dy = _cfg1_inputs(seed=11 + batch, batch=batch, in_dim=in_dim, out_dim=out_dim)
    w = w * 20
    y_ref = oracle.linear_forward(x, w, b, activation=act)
    dx_ref, dw_ref, db_ref = oracle.linear_backward(y_ref, dy, x, w, activation=act)
    xd, wd, yd, dyd = (to_dev(a, torch) for a in (x, w, y_ref, dy))
    one = [torch.full_like(xd, 0.5), torch.full_like(wd, 0.25), torch.full((out_dim,), 2.0, device="cuda")]
    ffk.linear_backward(yd, dyd, xd, wd, *one, activation=act, accumulate=True)
    sep = [torch.full_like(xd, 0.5), torch.full_like(wd, 0.25), torch.full((out_dim,), 2.0, device="cuda")]
    ffk.linear_backward(yd, dyd, xd, wd, sep[0], None, None, activation=act, accumulate=True)
    ffk.linear_backward(yd, dyd, xd, wd, None, sep[1], sep[2], activation=act, accumulate=True)
    for got, gen, want, base, name in zip(one, sep, (dx_ref, dw_ref, db_ref), (0.5, 0.25, 2.0), ("dx", "dw", "db")):
        assert_close(to_np(got), want + base, FP32_RTOL, name + " (one launch)")
        assert_close(to_np(got), to_np(gen), FP32_RTOL, name + " one launch vs general")
    # storing mode ignores what the tensors held
    ffk.linear_backward(yd, dyd, xd, wd, *one, activation=act, accumulate=False)
    for got, want, name in zip(one, (dx_ref, dw_ref, db_ref), ("dx", "dw", "db")):
        assert_close(to_np(got), want, FP32_RTOL, name + " stored")


def test_linear_no_bias_and_skipped_grads(ffk, oracle):
    x, w, b, dy = _cfg1_inputs(seed=5, batch=16, in_dim=24, out_dim=40)
    say("linear fp32 no bias / NULL grads")
    y_ref = oracle.linear_forward(x, w, None)
    xd, wd, dyd = (to_dev(a, torch) for a in (x, w, dy))
    y = ffk.linear_forward(xd, wd, None)
    assert_close(to_np(y), y_ref, FP32_RTOL, "y")
    dx_ref, dw_ref, _ = oracle.linear_backward(y_ref, dy, x, w, use_bias=False)
    dw = torch.zeros_like(wd)
    ffk.linear_backward(y, dyd, xd, wd, None, dw, None)
    assert_close(to_np(dw), dw_ref, FP32_RTOL, "dw")
    dx = torch.zeros_like(xd)
    ffk.linear_backward(y, dyd, xd, wd, dx, None, None)
    assert_close(to_np(dx), dx_ref, FP32_RTOL, "dx")


def test_linear_errors(ffk):
    x = torch.zeros((4, 4), device="cuda")
    with pytest.raises(ffk.FFKError, match="Unhandled activation"):
        ffk.linear_forward(x, x, None, activation=9)
    # (a small fp32 backward with all gradients asked for runs as one launch and needs no scratch;
    # without the input gradient it takes the general path, which does)
    with pytest.raises(ffk.FFKError, match="workspace"):
        ffk.check(ffk.lib().ffk_linear_backward(0, ffk.FLOAT, ffk.ACT_RELU, 0, x.data_ptr(), x.data_ptr(),
                                                x.data_ptr(), None, x.data_ptr(), x.data_ptr(), None,
                                                4, 4, 4, None, 0, 0))
    with pytest.raises(ffk.FFKError, match="output needed"):
        ffk.check(ffk.lib().ffk_linear_backward(0, ffk.FLOAT, ffk.ACT_RELU, 0, None, x.data_ptr(),
                                                x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), None,
                                                4, 4, 4, None, 0, 0))


@pytest.mark.parametrize("trans_a,trans_b", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(128, 128, 64), (256, 384, 192), (64, 64, 64), (200, 72, 40), (8, 8, 8),
                                 (130, 258, 136), (512, 1024, 256)])
def test_gemm_bf16(ffk, oracle, trans_a, trans_b, mnk):
    M, N, K = mnk
    say("gemm bf16", mnk, "ta", trans_a, "tb", trans_b)
    g = rng(M * 7 + N * 3 + K)
    A = bf16_round(g.standard_normal((K, M) if trans_a else (M, K)))
    B = bf16_round(g.standard_normal((N, K) if trans_b else (K, N)))
    want = oracle.gemm_f64(A, B, trans_a, trans_b)
    Ad, Bd = to_dev(A, torch, torch.bfloat16), to_dev(B, torch, torch.bfloat16)
    C = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    ffk.gemm(Ad, Bd, C, trans_a, trans_b)
    # exact products, fp32 accumulation, one bf16 rounding at the store
    assert_close(to_np(C), want, 2.0 ** -8, "C")
    C0 = bf16_round(g.standard_normal((M, N)))
    Cd = to_dev(C0, torch, torch.bfloat16)
    ffk.gemm(Ad, Bd, Cd, trans_a, trans_b, accumulate=True)
    assert_close(to_np(Cd), want + C0, 2.0 ** -7, "C accumulate")


F32_GEMM_SHAPES = [  # M, N, K: whole tiles, ragged edges in every direction, one k quad, both tile widths
    (128, 128, 32), (300, 260, 100), (128, 132, 4), (1000, 192, 36), (256, 64, 68), (1152, 2048, 64), (4096, 8192, 40),
]


@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("mnk", F32_GEMM_SHAPES)
def test_gemm_fp32_tiled(ffk, oracle, trans_a, trans_b, mnk):
    """The fp32 kernel with 128-row tiles (operands read 16 bytes at a time) against the fp64
    product, and against the bounds-checked 64x64 kernel, which adds every element's products in
    the same order: equal bits.  The general kernel is reached through a view whose rows start
    4 bytes off 16-byte alignment."""
    M, N, K = mnk
    if M * N > 2 ** 24 and (trans_a or not trans_b):
        pytest.skip("the largest shape once")
    say("gemm fp32 tiled", mnk, "ta", trans_a, "tb", trans_b)
    name = ffk.gemm_kernel_name(ffk.FLOAT, trans_a, trans_b, M, N, K)
    assert name.startswith("gemm_f32_tiled_kernel"), name
    g = rng(3 * M + 5 * N + K)
    A = g.standard_normal((K, M) if trans_a else (M, K)).astype(np.float32)
    B = g.standard_normal((N, K) if trans_b else (K, N)).astype(np.float32)
    Ad, Bd = to_dev(A, torch), to_dev(B, torch)
    C = torch.full((M, N), 7.0, device="cuda")
    ffk.gemm(Ad, Bd, C, trans_a, trans_b)
    if M * N <= 2 ** 22:
        want = oracle.gemm_f64(A, B, trans_a, trans_b)
        assert_close(to_np(C), want, FP32_RTOL, "C")
    else:
        rows = np.sort(g.choice(M, 24, replace=False))
        A_rows = np.ascontiguousarray(A[:, rows] if trans_a else A[rows])
        assert_close(to_np(C[torch.from_numpy(rows).cuda()]), oracle.gemm_f64(A_rows, B, trans_a, trans_b), FP32_RTOL, "C rows")
    # the same product by the general kernel: operands shifted one float off alignment
    def shifted(t):
        flat = torch.empty((t.numel() + 1,), device="cuda")
        v = flat[1:].view(t.shape)
        v.copy_(t)
        return v
    A1, B1 = shifted(Ad), shifted(Bd)
    C1 = torch.full((M, N), 7.0, device="cuda")
    ffk.check(ffk.lib().ffk_gemm(ffk.current_stream(), ffk.FLOAT, int(trans_a), int(trans_b), M, N, K,
                                 A1.data_ptr(), B1.data_ptr(), C1.data_ptr(), 0))
    assert torch.equal(C, C1)
    # accumulate: C += product, old contents read once
    C0 = g.standard_normal((M, N)).astype(np.float32)
    Cd, Cd1 = to_dev(C0, torch), to_dev(C0, torch)
    ffk.gemm(Ad, Bd, Cd, trans_a, trans_b, accumulate=True)
    ffk.check(ffk.lib().ffk_gemm(ffk.current_stream(), ffk.FLOAT, int(trans_a), int(trans_b), M, N, K,
                                 A1.data_ptr(), B1.data_ptr(), Cd1.data_ptr(), 1))
    assert torch.equal(Cd, Cd1)
    assert torch.equal(Cd, C + to_dev(C0, torch))


@pytest.mark.parametrize("act", [-1, 0, 1, 2, 3])
def test_linear_fp32_tiled_bias_and_activation(ffk, oracle, act):
    """A fp32 Linear large enough for the tiled kernel: bias and every activation on its store."""
    batch, in_dim, out_dim = 520, 136, 384
    say("linear fp32 tiled", (batch, in_dim, out_dim), "act", act)
    assert ffk.gemm_kernel_name(ffk.FLOAT, False, True, batch, out_dim, in_dim, True, act).startswith("gemm_f32_tiled_kernel")
    x, w, b, dy = _cfg1_inputs(seed=31, batch=batch, in_dim=in_dim, out_dim=out_dim)
    w = w * 10
    if act == 3:  # the reference's Linear has no GELU; this one is Linear -> ElementUnary GELU
        y_ref = oracle.element_unary_forward(ffk.OP["GELU"], oracle.linear_forward(x, w, b, activation=-1))
    else:
        y_ref = oracle.linear_forward(x, w, b, activation=act)
    xd, wd, bd, dyd = (to_dev(a, torch) for a in (x, w, b, dy))
    y = ffk.linear_forward(xd, wd, bd, activation=act)
    assert_close(to_np(y), y_ref, FP32_RTOL, "y")
    if act != 3:  # GELU has no backward on the Linear
        dx_ref, dw_ref, db_ref = oracle.linear_backward(y_ref, dy, x, w, activation=act)
        dx, dw, db = torch.zeros_like(xd), torch.zeros_like(wd), torch.zeros_like(bd)
        ffk.linear_backward(to_dev(y_ref, torch), dyd, xd, wd, dx, dw, db, activation=act)
        assert_close(to_np(dx), dx_ref, FP32_RTOL, "dx")
        assert_close(to_np(dw), dw_ref, FP32_RTOL, "dw")
        assert_close(to_np(db), db_ref, FP32_RTOL, "db")


@pytest.mark.parametrize("mnk", [(7, 5, 3), (33, 9, 12), (16, 24, 20)])
def test_gemm_bf16_unaligned_shapes_take_the_plain_kernel(ffk, oracle, mnk):
    M, N, K = mnk
    say("gemm bf16 unaligned", mnk)
    g = rng(99)
    A = bf16_round(g.standard_normal((M, K)))
    B = bf16_round(g.standard_normal((N, K)))
    want = oracle.gemm_f64(A, B, False, True)
    C = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ffk.gemm(to_dev(A, torch, torch.bfloat16), to_dev(B, torch, torch.bfloat16), C, False, True)
    assert_close(to_np(C), want, 2.0 ** -8, "C")


@pytest.mark.parametrize("act", [-1, 0])
def test_linear_bf16(ffk, oracle, act):
    batch, in_dim, out_dim = 256, 192, 384
    say("linear bf16", (batch, in_dim, out_dim), "act", act)
    g = rng(21)
    x = bf16_round(g.standard_normal((batch, in_dim)))
    w = bf16_round(g.standard_normal((out_dim, in_dim)) * 0.05)
    b = bf16_round(g.standard_normal((out_dim,)) * 0.05)
    dy = bf16_round(g.standard_normal((batch, out_dim)))
    y_ref = bf16_round(oracle.linear_forward(x, w, b, activation=act))
    xd, wd, bd, dyd = (to_dev(a, torch, torch.bfloat16) for a in (x, w, b, dy))
    y = ffk.linear_forward(xd, wd, bd, activation=act)
    assert_close(to_np(y), y_ref, BF16_RTOL, "y")
    dx_ref, dw_ref, db_ref = oracle.linear_backward(to_np(y), dy, x, w, activation=act)
    dx, dw, db = torch.zeros_like(xd), torch.zeros_like(wd), torch.zeros_like(bd)
    ffk.linear_backward(y, dyd, xd, wd, dx, dw, db, activation=act)
    assert_close(to_np(dx), dx_ref, BF16_RTOL, "dx")
    assert_close(to_np(dw), dw_ref, BF16_RTOL, "dw")
    assert_close(to_np(db), db_ref, BF16_RTOL, "db")


# Shapes that tile exactly take the pipelined direct-to-LDS kernels: 128x128
# tiles when that yields >= 128 workgroups, 256x256 tiles from 192 workgroups.
PIPE_SHAPES = [(2048, 2048, 512), (1024, 2048, 320), (4096, 3072, 256), (3072, 4096, 192)]


@pytest.mark.parametrize("trans_a,trans_b", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", PIPE_SHAPES)
def test_gemm_bf16_pipelined_tiles(ffk, oracle, trans_a, trans_b, mnk):
    M, N, K = mnk
    say("gemm bf16 pipelined", mnk, "ta", trans_a, "tb", trans_b)
    g = rng(M + 3 * N + 7 * K)
    A = bf16_round(g.standard_normal((K, M) if trans_a else (M, K)))
    B = bf16_round(g.standard_normal((N, K) if trans_b else (K, N)))
    Ad, Bd = to_dev(A, torch, torch.bfloat16), to_dev(B, torch, torch.bfloat16)
    C = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    ffk.gemm(Ad, Bd, C, trans_a, trans_b)
    Cn = to_np(C)
    # (1) the oracle on a sample of rows and on a sample of columns
    rows = np.sort(g.choice(M, 40, replace=False))
    cols = np.sort(g.choice(N, 40, replace=False))
    A_rows = np.ascontiguousarray(A[:, rows] if trans_a else A[rows])
    B_cols = np.ascontiguousarray(B[cols] if trans_b else B[:, cols])
    assert_close(Cn[rows], oracle.gemm_f64(A_rows, B, trans_a, trans_b), 2.0 ** -8, "C rows")
    assert_close(Cn[:, cols], oracle.gemm_f64(A, B_cols, trans_a, trans_b), 2.0 ** -8, "C cols")
    # (2) every element, through linearity: C v = A (B v)
    v = g.standard_normal((N,))
    A64 = (A.T if trans_a else A).astype(np.float64)
    B64 = (B.T if trans_b else B).astype(np.float64)
    want = A64 @ (B64 @ v)
    got = Cn.astype(np.float64) @ v
    bound = 2.0 ** -8 * (np.abs(A64) @ (np.abs(B64) @ np.abs(v)))
    assert np.all(np.abs(got - want) <= bound + 1e-6)
    # (3) accumulate adds to the old contents with a single rounding
    C0 = bf16_round(g.standard_normal((M, N)))
    Cd = to_dev(C0, torch, torch.bfloat16)
    ffk.gemm(Ad, Bd, Cd, trans_a, trans_b, accumulate=True)
    assert_close(to_np(Cd)[rows], oracle.gemm_f64(A_rows, B, trans_a, trans_b) + C0[rows], 2.0 ** -7, "C acc")


# Reductions from 2048 on take 256x256 tiles with one wave per SIMD (128x128 wave tiles, two 64-deep
# stages); the option forces that kernel onto short reductions too: one, two and three k-tiles
# exercise its prologue and drain, 33 an odd count in the steady loop.
WIDE_SHAPES = [(2048, 2048, 64), (2048, 2048, 128), (2048, 2048, 192), (4096, 3072, 2112)]


@pytest.mark.parametrize("trans_a,trans_b", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", WIDE_SHAPES)
def test_gemm_bf16_one_wave_per_simd(ffk, oracle, trans_a, trans_b, mnk):
    M, N, K = mnk
    say("gemm bf16 one wave per SIMD", mnk, "ta", trans_a, "tb", trans_b)
    g = rng(5 * M + 3 * N + K)
    A = bf16_round(g.standard_normal((K, M) if trans_a else (M, K)))
    B = bf16_round(g.standard_normal((N, K) if trans_b else (K, N)))
    C0 = bf16_round(g.standard_normal((M, N)))
    Ad, Bd = to_dev(A, torch, torch.bfloat16), to_dev(B, torch, torch.bfloat16)
    out = {}
    try:
        for variant in (264, 256):
            ffk.set_option(ffk.OPTION_GEMM_VARIANT, variant)
            C = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
            ffk.gemm(Ad, Bd, C, trans_a, trans_b)
            Cacc = to_dev(C0, torch, torch.bfloat16)
            ffk.gemm(Ad, Bd, Cacc, trans_a, trans_b, accumulate=True)
            out[variant] = (C, Cacc)
    finally:
        ffk.set_option(ffk.OPTION_GEMM_VARIANT, 0)
    Cn = to_np(out[264][0])
    rows = np.sort(g.choice(M, 24, replace=False))
    cols = np.sort(g.choice(N, 24, replace=False))
    A_rows = np.ascontiguousarray(A[:, rows] if trans_a else A[rows])
    B_cols = np.ascontiguousarray(B[cols] if trans_b else B[:, cols])
    assert_close(Cn[rows], oracle.gemm_f64(A_rows, B, trans_a, trans_b), 2.0 ** -8, "C rows")
    assert_close(Cn[:, cols], oracle.gemm_f64(A, B_cols, trans_a, trans_b), 2.0 ** -8, "C cols")
    # both kernels add the k-steps up in the same order: every element agrees to the bit
    assert torch.equal(out[264][0], out[256][0])
    assert torch.equal(out[264][1], out[256][1])
    assert_close(to_np(out[264][1])[rows], oracle.gemm_f64(A_rows, B, trans_a, trans_b) + C0[rows], 2.0 ** -7, "C acc")


@pytest.mark.parametrize("mnk", [(512, 384, 1024), (256, 384, 2048), (4096, 3072, 1024)])
@pytest.mark.parametrize("bias", [False, True])
def test_gemm_bf16_256x192_tile(ffk, oracle, mnk, bias):
    """The 256x192 tile (one wave per SIMD, 128x96 wave tiles) that the fused Q/K/V projection's
    [4096, 3072] output takes so that its tiles cover the chip in one whole round: option 192
    forces it at any fitting size; against the oracle on sampled rows and columns, and bit for
    bit against the 128x128-tile kernel (every pipelined kernel adds the k-steps in the same
    order).  At [4096, 3072] the dispatch must pick it by itself."""
    M, N, K = mnk
    say("gemm bf16 256x192 tile", mnk, "bias", bias)
    g = rng(7 * M + N + K)
    A = bf16_round(g.standard_normal((M, K)))
    B = bf16_round(g.standard_normal((N, K)) * 0.05)
    bv = bf16_round(g.standard_normal((N,))) if bias else None
    Ad, Bd = to_dev(A, torch, torch.bfloat16), to_dev(B, torch, torch.bfloat16)
    bd = to_dev(bv, torch, torch.bfloat16) if bias else None
    out = {}
    try:
        for variant in (192, 128):
            ffk.set_option(ffk.OPTION_GEMM_VARIANT, variant)
            out[variant] = ffk.linear_forward(Ad, Bd, bd)
            name = ffk.gemm_kernel_name(ffk.BF16, False, True, M, N, K, has_bias=bias)
            assert name.startswith("gemm_bf16_pipe_kernel<256,192,128,96," if variant == 192 else "gemm_bf16_pipe_kernel<128,128,"), name
    finally:
        ffk.set_option(ffk.OPTION_GEMM_VARIANT, 0)
    assert torch.equal(out[192], out[128])
    Cn = to_np(out[192])
    rows = np.sort(g.choice(M, 16, replace=False))
    cols = np.sort(g.choice(N, 16, replace=False))
    want_r = oracle.gemm_f64(np.ascontiguousarray(A[rows]), B, False, True) + (bv if bias else 0.0)
    want_c = oracle.gemm_f64(A, np.ascontiguousarray(B[cols]), False, True) + (bv[cols] if bias else 0.0)
    assert_close(Cn[rows], want_r, 2.0 ** -8, "C rows")
    assert_close(Cn[:, cols], want_c, 2.0 ** -8, "C cols")
    if mnk == (4096, 3072, 1024):
        assert ffk.gemm_kernel_name(ffk.BF16, False, True, M, N, K, has_bias=bias).startswith(
            "gemm_bf16_pipe_kernel<256,192,128,96,")
        assert torch.equal(ffk.linear_forward(Ad, Bd, bd), out[192])


@pytest.mark.parametrize("act", [-1, 0])
def test_linear_bf16_pipelined(ffk, oracle, act):
    """Linear at a size whose three products all take the pipelined kernels
    (NT forward with bias/activation epilogue, NN and TN backward)."""
    batch, in_dim, out_dim = 2048, 1024, 2048
    say("linear bf16 pipelined", (batch, in_dim, out_dim), "act", act)
    g = rng(23)
    x = bf16_round(g.standard_normal((batch, in_dim)))
    w = bf16_round(g.standard_normal((out_dim, in_dim)) * 0.03)
    b = bf16_round(g.standard_normal((out_dim,)) * 0.5)
    dy = bf16_round(g.standard_normal((batch, out_dim)))
    xd, wd, bd, dyd = (to_dev(a, torch, torch.bfloat16) for a in (x, w, b, dy))
    y = ffk.linear_forward(xd, wd, bd, activation=act)
    rows = np.sort(g.choice(batch, 32, replace=False))
    y_ref = oracle.linear_forward(x[rows], w, b, activation=act)
    assert_close(to_np(y)[rows], y_ref, BF16_RTOL, "y rows")
    yn = to_np(y)
    dx, dw, db = torch.zeros_like(xd), torch.zeros_like(wd), torch.zeros_like(bd)
    ffk.linear_backward(y, dyd, xd, wd, dx, dw, db, activation=act)
    gmat = dy * (yn > 0) if act == 0 else dy
    assert_close(to_np(dx)[rows], oracle.gemm_f64(np.ascontiguousarray(gmat[rows]), w), BF16_RTOL, "dx rows")
    orows = np.sort(g.choice(out_dim, 32, replace=False))
    dw_ref = oracle.gemm_f64(np.ascontiguousarray(gmat[:, orows]), x, trans_a=True)
    assert_close(to_np(dw)[orows], dw_ref, BF16_RTOL, "dw rows")
    assert_close(to_np(db), gmat.astype(np.float64).sum(0), BF16_RTOL, "db")


def test_collected_column_reductions_equal_immediate_ones(ffk):
    """Between ffk_column_reductions_begin and _end the bias gradients are not written; _end
    writes all of them with one launch, and they equal the ones computed call by call."""
    say("collected column reductions")
    g = rng(77)
    bt = torch.bfloat16
    cases = []
    for (batch, in_dim, out_dim) in [(512, 256, 384), (300, 128, 1000), (64, 64, 32)]:
        x = to_dev(bf16_round(g.standard_normal((batch, in_dim)).astype(np.float32)), torch, bt)
        w = to_dev(bf16_round(g.standard_normal((out_dim, in_dim)).astype(np.float32) * 0.1), torch, bt)
        dy = to_dev(bf16_round(g.standard_normal((batch, out_dim)).astype(np.float32)), torch, bt)
        cases.append((x, w, dy))
    want = []
    for x, w, dy in cases:
        db = torch.zeros((w.shape[0],), dtype=bt, device="cuda")
        ffk.linear_backward(dy, dy, x, w, db=db, accumulate=0)
        want.append(db)
    got = [torch.full((w.shape[0],), 7.0, dtype=bt, device="cuda") for _, w, _ in cases]
    keep = []  # every collected call needs workspace of its own until _end
    ffk.check(ffk.lib().ffk_column_reductions_begin())
    try:
        for (x, w, dy), db in zip(cases, got):
            need = ffk.lib().ffk_linear_backward_workspace_bytes(ffk.BF16, ffk.ACT_NONE, 1, x.shape[0], w.shape[0])
            ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
            keep.append(ws)
            ffk.linear_backward(dy, dy, x, w, db=db, accumulate=0, workspace=ws)
        torch.cuda.synchronize()
        assert all(bool((db == 7.0).all()) for db in got)  # nothing written yet
    finally:
        ffk.check(ffk.lib().ffk_column_reductions_end(ffk.current_stream()))
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    # _end without _begin is a no-op
    ffk.check(ffk.lib().ffk_column_reductions_end(ffk.current_stream()))



FUSED_TAIL_SHAPES = [  # (batch, in_dim, out_dim) of the forward Linear
    (2048, 1024, 2048),  # 128x128 tiles, 256 of them (and 128 for the second Linear)
    (1024, 192, 2048),   # 128x128 tiles, fewer k-tiles than pipeline stages
    (3072, 256, 4096),   # 256x256 tiles in both directions
    (4096, 4096, 1024),  # the second Linear on 256x256 tiles
]


@pytest.mark.parametrize("batch,in_dim,out_dim", FUSED_TAIL_SHAPES)
def test_linear_with_gelu_and_dropout_on_the_tile_store_equals_separate_operators(ffk, batch, in_dim, out_dim):
    """ffk_linear_gelu_dropout_forward and ffk_linear_backward_dropout_gelu give the bits of
    Linear -> GELU -> Dropout and of Linear backward -> Dropout backward -> GELU backward."""
    say("linear with GELU and dropout on the tile store %s" % ((batch, in_dim, out_dim),))
    g = rng(batch + in_dim)
    bt = torch.bfloat16
    rate, seed, offset = 0.1, 987654321, 4096
    x = to_dev(bf16_round(g.standard_normal((batch, in_dim)).astype(np.float32)), torch, bt)
    w = to_dev(bf16_round(g.standard_normal((out_dim, in_dim)).astype(np.float32) / np.sqrt(in_dim)), torch, bt)
    b = to_dev(bf16_round(g.standard_normal((out_dim,)).astype(np.float32)), torch, bt)
    # forward
    y_sep = torch.empty((batch, out_dim), dtype=bt, device="cuda")
    ffk.linear_forward(x, w, b, ffk.ACT_NONE, y_sep)
    act = ffk.element_unary_forward(ffk.OP["GELU"], y_sep)
    dropped_sep = ffk.dropout_forward(act, rate, seed, offset)
    y, dropped = ffk.linear_gelu_dropout_forward(x, w, b, rate, seed, offset)
    assert torch.equal(y.view(torch.int16), y_sep.view(torch.int16))
    assert torch.equal(dropped.view(torch.int16), dropped_sep.view(torch.int16))
    assert 0.05 < float((dropped == 0).float().mean()) < 0.15
    # the second Linear with its dropout and the residual addition: [batch, out_dim] -> [batch, in_dim]
    w_down = to_dev(bf16_round(g.standard_normal((in_dim, out_dim)).astype(np.float32) * 0.05), torch, bt)
    b_down = to_dev(bf16_round(g.standard_normal((in_dim,)).astype(np.float32)), torch, bt)
    if batch * in_dim >= 128 * 128 * 128 and in_dim % 128 == 0:
        y2 = torch.empty((batch, in_dim), dtype=bt, device="cuda")
        ffk.linear_forward(dropped, w_down, b_down, ffk.ACT_NONE, y2)
        want = ffk.dropout_add_forward(y2, x, rate, seed + 1, offset)
        got = ffk.linear_dropout_add_forward(dropped, x, w_down, b_down, rate, seed + 1, offset)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # backward of the Linear that consumes `dropped`: [batch, out_dim] -> [batch, in_dim]
    w2 = to_dev(bf16_round(g.standard_normal((in_dim, out_dim)).astype(np.float32) * 0.1), torch, bt)
    dy2 = to_dev(bf16_round(g.standard_normal((batch, in_dim)).astype(np.float32)), torch, bt)
    d_dropped = torch.empty_like(dropped)
    dw_sep = torch.empty_like(w2)
    db_sep = torch.empty((in_dim,), dtype=bt, device="cuda")
    ffk.linear_backward(dy2, dy2, dropped, w2, dx=d_dropped, dw=dw_sep, db=db_sep, accumulate=0)
    dx_sep = ffk.dropout_gelu_backward(d_dropped, y, rate, seed, offset)
    dw = torch.empty_like(w2)
    db = torch.empty_like(db_sep)
    dx = ffk.linear_backward_dropout_gelu(dy2, dropped, y, w2, rate, seed, offset, dw=dw, db=db)
    assert torch.equal(dx.view(torch.int16), dx_sep.view(torch.int16))
    assert torch.equal(dw.view(torch.int16), dw_sep.view(torch.int16))
    assert torch.equal(db.view(torch.int16), db_sep.view(torch.int16))
    # ... and with the first Linear's bias gradient summed on the same tile store
    db1_sep = torch.empty((out_dim,), dtype=bt, device="cuda")
    ffk.linear_backward(None, dx_sep, x, w, dx=None, dw=None, db=db1_sep, accumulate=0)
    db1 = torch.full_like(db1_sep, 5.0)
    try:
        dx = ffk.linear_backward_dropout_gelu_bias_grad(dy2, dropped, y, w2, rate, seed, db1, offset, dw=dw, db=db)
    except ffk.FFKError as e:
        assert "no fused kernel" in str(e) and (batch, in_dim, out_dim) != (4096, 1024, 4096)
        return
    assert torch.equal(dx.view(torch.int16), dx_sep.view(torch.int16))
    assert torch.equal(dw.view(torch.int16), dw_sep.view(torch.int16))
    assert torch.equal(db.view(torch.int16), db_sep.view(torch.int16))
    assert torch.equal(db1.view(torch.int16), db1_sep.view(torch.int16))
    ffk.linear_backward_dropout_gelu_bias_grad(dy2, dropped, y, w2, rate, seed, db1, offset, dw=dw, db=db,
                                               accumulate_gelu_bias=True)
    ffk.linear_backward(None, dx_sep, x, w, dx=None, dw=None, db=db1_sep, accumulate=4)  # FFK_ACC_BIAS
    assert torch.equal(db1.view(torch.int16), db1_sep.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("batch,out_dim", [(4096, 1024), (512, 4096), (100, 64), (33, 8), (7, 5)])
def test_dropout_backward_with_the_bias_gradient_equals_separate_operators(ffk, dtype, batch, out_dim):
    """ffk_dropout_backward_bias_grad: the bits of ffk_dropout_backward followed by the column sums
    ffk_linear_backward takes for the bias gradient; shapes without such a kernel are refused."""
    say("dropout backward with bias gradient", dtype, (batch, out_dim))
    g = rng(batch + out_dim)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    dy = to_dev(rnd(g.standard_normal((batch, out_dim)).astype(np.float32)), torch, dtype)
    rate, seed, offset = 0.1, 4242, 64
    dx_sep = ffk.dropout_backward(dy, rate, seed, offset)
    x = torch.zeros((batch, 8), dtype=dtype, device="cuda")
    w = torch.zeros((out_dim, 8), dtype=dtype, device="cuda")
    db_sep = torch.empty((out_dim,), dtype=dtype, device="cuda")
    ffk.linear_backward(None, dx_sep, x, w, dx=None, dw=None, db=db_sep, accumulate=0)
    db = torch.full_like(db_sep, 3.0)
    try:
        dx = ffk.dropout_backward_bias_grad(dy, rate, seed, db, offset)
    except ffk.FFKError as e:
        assert "no fused kernel" in str(e) and (batch, out_dim) not in ((4096, 1024), (512, 4096))
        return
    assert torch.equal(dx, dx_sep) and torch.equal(db, db_sep)
    ffk.dropout_backward_bias_grad(dy, rate, seed, db, offset, accumulate_bias=True)
    ffk.linear_backward(None, dx_sep, x, w, dx=None, dw=None, db=db_sep, accumulate=4)  # FFK_ACC_BIAS
    assert torch.equal(db, db_sep)


def test_linear_with_fused_tail_refuses_shapes_without_a_kernel(ffk):
    say("linear with fused tail: unsupported shapes")
    bt = torch.bfloat16
    x = torch.zeros((100, 64), dtype=bt, device="cuda")
    w = torch.zeros((128, 64), dtype=bt, device="cuda")
    b = torch.zeros((128,), dtype=bt, device="cuda")
    with pytest.raises(ffk.FFKError, match="no fused kernel"):
        ffk.linear_gelu_dropout_forward(x, w, b, 0.1, 1)
    xf = torch.zeros((2048, 256), dtype=torch.float32, device="cuda")
    wf = torch.zeros((2048, 256), dtype=torch.float32, device="cuda")
    bf = torch.zeros((2048,), dtype=torch.float32, device="cuda")
    with pytest.raises(ffk.FFKError, match="no fused kernel"):
        ffk.linear_gelu_dropout_forward(xf, wf, bf, 0.1, 1)
    with pytest.raises(ffk.FFKError, match="no fused kernel"):
        ffk.linear_backward_dropout_gelu(x, torch.zeros((100, 128), dtype=bt, device="cuda"),
                                         torch.zeros((100, 128), dtype=bt, device="cuda"),
                                         torch.zeros((64, 128), dtype=bt, device="cuda"), 0.1, 1)


@pytest.mark.gpu
def test_matrix_rate_probe_runs_and_counts_its_flops(ffk):
    """The measurement aid: finite sums out, the flops of the launch as documented, bad arguments refused."""
    say("probe_mfma_bf16")
    out = torch.empty((256 * 256,), device="cuda")
    flops = ffk.probe_mfma_bf16(10, out)
    torch.cuda.synchronize()
    assert flops == 256 * 4 * 10 * 16 * 2.0 * 32 * 32 * 16
    assert bool(torch.isfinite(out).all()) and float(out.abs().max()) > 0
    rc = ffk.lib().ffk_probe_mfma_bf16(ffk.current_stream(), 10, 1, ffk.ptr(out), 1024, None)
    assert rc == ffk.ERR_INVALID
    rc = ffk.lib().ffk_probe_mfma_bf16(ffk.current_stream(), 0, 1, ffk.ptr(out), out.numel() * 4, None)
    assert rc == ffk.ERR_INVALID
