"""The LayerNorm backward entry point that allocates nothing
(ffk_layer_norm_backward_static) against ffk_layer_norm_backward, through the
C ABI, and both against the oracle.  Runs last: a fault in the per-device
scratch array must not hide the other tests."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _case(ffk, oracle, M, N, dtype, same_grid):
    say("layer_norm_backward_static", (M, N), dtype)
    g = rng(M * 7 + N)
    x = (g.standard_normal((M, N)) * 1.5 + 0.3).astype(np.float32)
    dy = g.standard_normal((M, N)).astype(np.float32)
    gamma = (1 + 0.1 * g.standard_normal((N,))).astype(np.float32)
    beta = (0.1 * g.standard_normal((N,))).astype(np.float32)
    tdt, rtol = (torch.float32, 2e-5) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        x, dy, gamma, beta = bf16_round(x), bf16_round(dy), bf16_round(gamma), bf16_round(beta)
    xd, dyd, gd, bd = (to_dev(a, torch, tdt) for a in (x, dy, gamma, beta))
    _, mean, rstd = ffk.layer_norm_forward(xd, gd, bd, 1e-5)
    want = [torch.full_like(xd, 7.0), torch.full_like(gd, 7.0), torch.full_like(gd, 7.0)]
    got = [torch.full_like(xd, -3.0), torch.full_like(gd, -3.0), torch.full_like(gd, -3.0)]
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, *want)
    torch.cuda.synchronize()
    # free device memory as the driver reports it (hipMemGetInfo): it also sees an allocation
    # made inside the library, which torch's own counter would not
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    ffk.layer_norm_backward_static(dyd, xd, mean, rstd, gd, *got)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated during the call"
    # dX never depends on how many workgroups walk the rows
    assert torch.equal(got[0], want[0]), "dx bits differ"
    if same_grid:
        assert torch.equal(got[1], want[1]) and torch.equal(got[2], want[2]), "parameter gradient bits differ"
    else:
        assert_close(to_np(got[1]), to_np(want[1]), rtol, "dgamma vs the workspace entry point")
        assert_close(to_np(got[2]), to_np(want[2]), rtol, "dbeta vs the workspace entry point")
    if M * N <= (1 << 22):
        _, mean_ref, rstd_ref = oracle.layer_norm_forward(x, gamma, beta, 1e-5)[0:3]
        dx_ref, dg_ref, db_ref = oracle.layer_norm_backward(dy, x, mean_ref, rstd_ref, gamma)
        assert_close(to_np(got[0]), dx_ref, rtol * 2, "dx vs oracle")
        assert_close(to_np(got[1]), dg_ref, rtol * 2, "dgamma vs oracle")
        assert_close(to_np(got[2]), db_ref, rtol * 2, "dbeta vs oracle")
    # accumulate form
    acc_w, acc_g = torch.ones_like(xd), torch.ones_like(xd)
    ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, acc_w, want[1], want[2], accumulate=True)
    ffk.layer_norm_backward_static(dyd, xd, mean, rstd, gd, acc_g, got[1], got[2], accumulate=True)
    torch.cuda.synchronize()
    assert torch.equal(acc_w, acc_g), "accumulated dx bits differ"


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_static_scratch_two_calls_second_smaller(ffk, oracle, dtype):
    # the larger call fills the array; the smaller one after it must not see
    # what the first left there
    _case(ffk, oracle, 4096, 1024, dtype, same_grid=True)
    _case(ffk, oracle, 130, 768, dtype, same_grid=True)
    _case(ffk, oracle, 3, 8, dtype, same_grid=True)


def test_static_scratch_fewer_workgroups_than_the_workspace_form(ffk, oracle):
    # N 4096: the array holds 256 partial rows, the workspace form uses 512
    _case(ffk, oracle, 2048, 4096, "bf16", same_grid=False)
    _case(ffk, oracle, 600, 4096, "fp32", same_grid=False)
    _case(ffk, oracle, 64, 16384, "bf16", same_grid=True)  # 64 rows: one workgroup each in both
    # rows the vector kernels do not take use no scratch at all
    _case(ffk, oracle, 5, 100, "fp32", same_grid=True)


def test_static_scratch_inside_a_collecting_region(ffk, oracle):
    # between _begin and _end the workspace form defers its column sums; this
    # one must not (the next call overwrites its partial sums)
    g = rng(5)
    tdt = torch.bfloat16
    cases = []
    for M, N in ((512, 1024), (256, 1024)):
        x = bf16_round(g.standard_normal((M, N)))
        dy = bf16_round(g.standard_normal((M, N)))
        gamma = bf16_round(1 + 0.1 * g.standard_normal((N,)))
        xd, dyd, gd = (to_dev(a, torch, tdt) for a in (x, dy, gamma))
        _, mean, rstd = ffk.layer_norm_forward(xd, gd, gd, 1e-5)
        cases.append((dyd, xd, mean, rstd, gd))
    got = []
    ffk.check(ffk.lib().ffk_column_reductions_begin())
    try:
        for dyd, xd, mean, rstd, gd in cases:
            dx, dg, db = torch.empty_like(xd), torch.zeros_like(gd), torch.zeros_like(gd)
            ffk.layer_norm_backward_static(dyd, xd, mean, rstd, gd, dx, dg, db)
            got.append((dx, dg, db))
    finally:
        ffk.check(ffk.lib().ffk_column_reductions_end(ffk.current_stream()))
    torch.cuda.synchronize()
    for (dyd, xd, mean, rstd, gd), (dx, dg, db) in zip(cases, got):
        dx2, dg2, db2 = torch.empty_like(xd), torch.zeros_like(gd), torch.zeros_like(gd)
        ffk.layer_norm_backward(dyd, xd, mean, rstd, gd, dx2, dg2, db2)
        torch.cuda.synchronize()
        assert torch.equal(dx, dx2) and torch.equal(dg, dg2) and torch.equal(db, db2)


def test_static_scratch_in_a_collecting_region_with_shared_parameters(ffk):
    """Two LayerNorms that share gamma / beta gradients inside one collecting region: the
    workspace form first (its column sums are collected), the static form after it (its own run
    at once).  In storing mode the later call's values must be what the tensors hold at the
    end, as outside a region; in accumulating mode the sum of both."""
    g = rng(6)
    tdt = torch.bfloat16
    N = 1024
    cases = []
    for M in (384, 512):
        x = bf16_round(g.standard_normal((M, N)))
        dy = bf16_round(g.standard_normal((M, N)))
        gamma = bf16_round(1 + 0.1 * g.standard_normal((N,)))
        xd, dyd, gd = (to_dev(a, torch, tdt) for a in (x, dy, gamma))
        _, mean, rstd = ffk.layer_norm_forward(xd, gd, gd, 1e-5)
        cases.append((dyd, xd, mean, rstd, gd))
    alone = []
    for c in cases:
        dx, dg, db = torch.empty_like(c[1]), torch.zeros((N,), dtype=tdt, device="cuda"), torch.zeros((N,), dtype=tdt, device="cuda")
        ffk.layer_norm_backward(*c, dx, dg, db)
        alone.append((dg, db))
    for accumulate in (0, ffk.LN_ACC_PARAMS):
        dg, db = torch.zeros((N,), dtype=tdt, device="cuda"), torch.zeros((N,), dtype=tdt, device="cuda")
        ffk.check(ffk.lib().ffk_column_reductions_begin())
        try:
            ffk.layer_norm_backward(*cases[0], torch.empty_like(cases[0][1]), dg, db, accumulate=accumulate)
            ffk.layer_norm_backward_static(*cases[1], torch.empty_like(cases[1][1]), dg, db, accumulate=accumulate)
        finally:
            ffk.check(ffk.lib().ffk_column_reductions_end(ffk.current_stream()))
        torch.cuda.synchronize()
        if accumulate == 0:
            assert torch.equal(dg, alone[1][0]) and torch.equal(db, alone[1][1]), "the later call must win"
        else:
            # (the second call adds its fp32 sums to the first call's stored bf16 values: equal to
            # the sum of the two stored results up to one rounding of the second term)
            want_g = alone[0][0].float() + alone[1][0].float()
            want_b = alone[0][1].float() + alone[1][1].float()
            assert_close(to_np(dg), to_np(want_g), 2.0 ** -7, "both calls must add (dgamma)")
            assert_close(to_np(db), to_np(want_b), 2.0 ** -7, "both calls must add (dbeta)")
            assert not torch.equal(dg, alone[1][0]), "the first call's sums were lost"


def test_static_scratch_rejects_a_flag_that_is_no_mask(ffk):
    x = torch.zeros((2, 64), dtype=torch.bfloat16, device="cuda")
    m = torch.zeros((2,), dtype=torch.float32, device="cuda")
    rc = ffk.lib().ffk_layer_norm_backward_static(0, ffk.BF16, x.data_ptr(), x.data_ptr(), m.data_ptr(), m.data_ptr(),
                                                  None, x.data_ptr(), None, None, 2, 64, -1)
    assert rc == 1 and b"not a mask" in ffk.lib().ffk_last_error()


def test_static_scratch_rejects_rows_beyond_the_limit(ffk):
    N = 16384 + 8
    x = torch.zeros((2, N), dtype=torch.bfloat16, device="cuda")
    m = torch.zeros((2,), dtype=torch.float32, device="cuda")
    rc = ffk.lib().ffk_layer_norm_backward_static(0, ffk.BF16, x.data_ptr(), x.data_ptr(), m.data_ptr(),
                                                  m.data_ptr(), None, x.data_ptr(), None, None, 2, N, 0)
    assert rc == 4  # FFK_ERR_WORKSPACE
    assert b"exceed the limit" in ffk.lib().ffk_last_error()
