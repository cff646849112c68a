"""LayerNorm / Softmax parity against the oracle."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


LN_SHAPES = [(1, 8), (3, 5), (7, 64), (33, 1024), (64, 4096), (5, 100), (9, 8192), (2, 20000), (130, 768)]


@pytest.mark.parametrize("shape", LN_SHAPES)
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("affine", [True, False])
def test_layer_norm(ffk, oracle, shape, dtype, affine):
    M, N = shape
    say("layer_norm", shape, dtype, "affine", affine)
    g = rng(M * 31 + N)
    x = (g.standard_normal((M, N)) * 1.5 + 0.3).astype(np.float32)
    dy = g.standard_normal((M, N)).astype(np.float32)
    gamma = (1 + 0.1 * g.standard_normal((N,))).astype(np.float32) if affine else None
    beta = (0.1 * g.standard_normal((N,))).astype(np.float32) if affine else None
    dx0 = g.standard_normal((M, N)).astype(np.float32)
    tdt, rtol = (torch.float32, 2e-5) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        x, dy, dx0 = bf16_round(x), bf16_round(dy), bf16_round(dx0)
        if affine:
            gamma, beta = bf16_round(gamma), bf16_round(beta)
    eps = 1e-5
    y_ref, mean_ref, rstd_ref = oracle.layer_norm_forward(x, gamma, beta, eps)
    xd, dyd = to_dev(x, torch, tdt), to_dev(dy, torch, tdt)
    gd = to_dev(gamma, torch, tdt) if affine else None
    bd = to_dev(beta, torch, tdt) if affine else None
    y, mean, rstd = ffk.layer_norm_forward(xd, gd, bd, eps)
    assert_close(to_np(y), y_ref, rtol, "y")
    assert_close(to_np(mean), mean_ref, 2e-5, "mean")
    assert_close(to_np(rstd), rstd_ref, 2e-5, "rstd")
    dx_ref, dg_ref, db_ref = oracle.layer_norm_backward(dy, x, mean_ref, rstd_ref, gamma)
    dx = torch.zeros_like(xd)
    dg = torch.zeros((N,), dtype=tdt, device="cuda")
    db = torch.zeros((N,), dtype=tdt, device="cuda")
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dx, dg, db)
    assert_close(to_np(dx), dx_ref, rtol * 2, "dx")
    assert_close(to_np(dg), dg_ref, rtol * 2, "dgamma")
    assert_close(to_np(db), db_ref, rtol * 2, "dbeta")
    dxa = to_dev(dx0, torch, tdt)
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dxa, dg, db, accumulate=True)
    want, _, _ = oracle.layer_norm_backward(dy, x, mean_ref, rstd_ref, gamma, dx_init=dx0)
    assert_close(to_np(dxa), want, rtol * 2, "dx accumulate")


def test_layer_norm_many_rows_bf16(ffk, oracle):
    """More rows than persistent workgroups: exercises the row loop and the
    partial-sum reduction of dgamma/dbeta (config-2 shape [4096, 1024])."""
    M, N = 4096, 1024
    say("layer_norm many rows", (M, N))
    g = rng(77)
    x = bf16_round(g.standard_normal((M, N)))
    dy = bf16_round(g.standard_normal((M, N)))
    gamma = bf16_round(1 + 0.02 * g.standard_normal((N,)))
    beta = bf16_round(0.02 * g.standard_normal((N,)))
    y_ref, mean_ref, rstd_ref = oracle.layer_norm_forward(x, gamma, beta, 1e-5)
    dx_ref, dg_ref, db_ref = oracle.layer_norm_backward(dy, x, mean_ref, rstd_ref, gamma)
    bt = torch.bfloat16
    xd, dyd, gd, bd = (to_dev(a, torch, bt) for a in (x, dy, gamma, beta))
    y, mean, rstd = ffk.layer_norm_forward(xd, gd, bd, 1e-5)
    assert_close(to_np(y), y_ref, BF16_RTOL, "y")
    dx, dg, db = torch.zeros_like(xd), torch.zeros_like(gd), torch.zeros_like(bd)
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dx, dg, db)
    assert_close(to_np(dx), dx_ref, BF16_RTOL, "dx")
    assert_close(to_np(dg), dg_ref, BF16_RTOL, "dgamma")
    assert_close(to_np(db), db_ref, BF16_RTOL, "dbeta")


@pytest.mark.parametrize("shape", [(33, 1024), (64, 4096), (130, 768), (7, 64), (9, 8192), (4096, 1024)])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_layer_norm_backward_residual_is_copy_then_accumulate(ffk, shape, dtype):
    """input_grad = residual + gradient in one kernel has the bits of copying residual into
    input_grad and letting the plain backward add into it (whose values the oracle checks
    above); with a dropout the third output has the bits of ffk_dropout_backward on the sum."""
    M, N = shape
    say("layer_norm backward residual", shape, dtype)
    g = rng(M + N)
    td = torch.float32 if dtype == "fp32" else torch.bfloat16
    rnd = (lambda a: a.astype(np.float32)) if dtype == "fp32" else bf16_round
    x, dy, res = (rnd(g.standard_normal((M, N))) for _ in range(3))
    gamma = rnd(1 + 0.02 * g.standard_normal((N,)))
    beta = rnd(0.02 * g.standard_normal((N,)))
    xd, dyd, rd, gd, bd = (to_dev(a, torch, td) for a in (x, dy, res, gamma, beta))
    _, mean, rstd = ffk.layer_norm_forward(xd, gd, bd, 1e-5)
    dx0, dg0, db0 = rd.clone(), torch.zeros_like(gd), torch.zeros_like(bd)
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dx0, dg0, db0, accumulate=True)
    dx1, dg1, db1 = torch.full_like(xd, 7.0), torch.zeros_like(gd), torch.zeros_like(bd)
    ffk.layer_norm_backward_residual(dyd, xd, mean, rstd, gd, rd, dx1, dg1, db1)
    assert torch.equal(dx0, dx1) and torch.equal(dg0, dg1) and torch.equal(db0, db1)
    if dtype == "bf16":
        rate, seed, offset = 0.1, 1234, 8 * 5
        dx2, dropped = torch.empty_like(xd), torch.empty_like(xd)
        ffk.layer_norm_backward_residual(dyd, xd, mean, rstd, gd, rd, dx2, dg1, db1, dropped=dropped, rate=rate,
                                         seed=seed, offset=offset)
        assert torch.equal(dx0, dx2)
        assert torch.equal(dropped, ffk.dropout_backward(dx0, rate, seed, offset))
        # parameter gradients added into what is there
        dg3, db3 = dg0.clone(), db0.clone()
        ffk.layer_norm_backward_residual(dyd, xd, mean, rstd, gd, rd, dx2, dg3, db3, accumulate_params=True)
        dg4, db4 = dg0.clone(), db0.clone()
        ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dx0.clone(), dg4, db4, accumulate=3)
        assert torch.equal(dg3, dg4) and torch.equal(db3, db4)


@pytest.mark.parametrize("shape", [(33, 1024), (64, 4096), (130, 768), (7, 64), (4096, 1024)])
def test_dropout_add_layer_norm_forward_is_the_three_operators(ffk, shape):
    M, N = shape
    say("dropout + add + layer_norm forward", shape)
    g = rng(M * 3 + N)
    bt = torch.bfloat16
    x, res = (to_dev(bf16_round(g.standard_normal((M, N))), torch, bt) for _ in range(2))
    gamma = to_dev(bf16_round(1 + 0.02 * g.standard_normal((N,))), torch, bt)
    beta = to_dev(bf16_round(0.02 * g.standard_normal((N,))), torch, bt)
    rate, seed, offset = 0.1, 99, 16
    total, y, mean, rstd = ffk.dropout_add_layer_norm_forward(x, res, gamma, beta, 1e-5, rate, seed, offset)
    want_total = ffk.dropout_add_forward(x, res, rate, seed, offset)
    want_y, want_mean, want_rstd = ffk.layer_norm_forward(want_total, gamma, beta, 1e-5)
    assert torch.equal(total, want_total) and torch.equal(y, want_y)
    assert torch.equal(mean, want_mean) and torch.equal(rstd, want_rstd)


def test_layer_norm_fused_forms_refuse_what_they_cannot_run(ffk):
    """Rows that are no multiple of 8 elements have no one-pass kernel: FFK_ERR_UNSUPPORTED, nothing written."""
    bt = torch.bfloat16
    x = torch.zeros((4, 100), device="cuda", dtype=bt)
    gamma = torch.ones((100,), device="cuda", dtype=bt)
    m = torch.zeros((4,), device="cuda")
    dx = torch.full_like(x, 3.0)
    ws = torch.empty((ffk.lib().ffk_layer_norm_backward_workspace_bytes(4, 100),), dtype=torch.uint8, device="cuda")
    rc = ffk.lib().ffk_layer_norm_backward_residual(0, ffk.BF16, x.data_ptr(), x.data_ptr(), m.data_ptr(), m.data_ptr(),
                                                    gamma.data_ptr(), x.data_ptr(), dx.data_ptr(), None, None, 4, 100,
                                                    ws.data_ptr(), ws.numel(), 0, None, 0.0, 0, 0)
    assert rc == ffk.ERR_UNSUPPORTED
    y = torch.full_like(x, 3.0)
    rc = ffk.lib().ffk_dropout_add_layer_norm_forward(0, ffk.BF16, x.data_ptr(), x.data_ptr(), dx.data_ptr(), y.data_ptr(),
                                                      gamma.data_ptr(), gamma.data_ptr(), m.data_ptr(), m.data_ptr(), 4, 100,
                                                      1e-5, 0.1, 1, 0)
    assert rc == ffk.ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert bool((dx == 3.0).all()) and bool((y == 3.0).all())


def test_layer_norm_workspace_error(ffk):
    x = torch.zeros((8, 64), device="cuda")
    m = torch.zeros((8,), device="cuda")
    with pytest.raises(ffk.FFKError, match="workspace"):
        ffk.check(ffk.lib().ffk_layer_norm_backward(0, ffk.FLOAT, x.data_ptr(), x.data_ptr(), m.data_ptr(),
                                                    m.data_ptr(), None, x.data_ptr(), None, None, 8, 64,
                                                    None, 0, 0))


SM_SHAPES = [(1, 1, 1), (5, 7, 1), (33, 64, 1), (17, 2048, 1), (4, 4096, 1), (3, 16384, 1), (2, 50000, 1),
             (3, 5, 7), (2, 10, 64), (4, 3, 1000), (6, 1000, 1)]


@pytest.mark.parametrize("shape", SM_SHAPES)
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_softmax(ffk, oracle, shape, dtype):
    outer, dim, inner = shape
    say("softmax", shape, dtype)
    g = rng(outer * 13 + dim)
    x = (g.standard_normal(shape) * 4).astype(np.float32)
    dy = g.standard_normal(shape).astype(np.float32)
    tdt, rtol = (torch.float32, 2e-5) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        x, dy = bf16_round(x), bf16_round(dy)
    y_ref = oracle.softmax_forward(x, outer, dim, inner)
    xd = to_dev(x, torch, tdt)
    y = ffk.softmax_forward(xd, outer, dim, inner)
    assert_close(to_np(y), y_ref, rtol, "y")
    yn = to_np(y)
    dx_ref = oracle.softmax_backward(yn, dy, outer, dim, inner)
    dx = ffk.softmax_backward(y, to_dev(dy, torch, tdt), outer, dim, inner)
    assert_close(to_np(dx), dx_ref, rtol * 2, "dx")
    # the reference's own backward is a copy (softmax_kernels.cu:68-78)
    dxc = ffk.softmax_backward_copy(to_dev(dy, torch, tdt))
    assert np.array_equal(to_np(dxc), dy)


def test_softmax_config3_rows_sum_to_one(ffk):
    """BASELINE config 3: last-dim softmax of [128,2048,2048] bf16 logits
    N(0,4^2); size-independent properties at the full size."""
    say("softmax cfg3 full size")
    outer, dim = 128 * 2048, 2048
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.randn((outer, dim), device="cuda", generator=gen) * 4).to(torch.bfloat16)
    y = ffk.softmax_forward(x, outer, dim, 1)
    sums = y.float().sum(-1)
    assert float((sums - 1).abs().max()) < 2e-2
    assert float(y.min()) >= 0
    # argmax preserved, shift invariance
    assert torch.equal(y.float().argmax(-1)[:4096], x.float().argmax(-1)[:4096])
    dy = torch.randn((outer, dim), device="cuda", generator=gen).to(torch.bfloat16)
    dx = ffk.softmax_backward(y, dy, outer, dim, 1)
    assert float(dx.float().sum(-1).abs().max()) < 5e-2   # rows of dx sum to 0
