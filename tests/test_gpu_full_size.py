"""The benchmark configurations at their FULL sizes against the oracle.

The small-shape tests pick other template instantiations and grids than the
sizes the kernels are timed at; these run the timed shapes.  The oracle sees a
sample (rows, columns, bags) where the whole tensor would take minutes, and
size-independent invariants cover every element."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu
BT = torch.bfloat16


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def zipf_ids(g, n, vocab, s=1.1):
    p = 1.0 / np.arange(1, vocab + 1) ** s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, g.random(n)), vocab - 1)


def dev_randn(shape, seed, dtype=BT, scale=1.0):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=gen) * scale).to(dtype)


def test_layer_norm_config3(ffk, oracle):
    """LayerNorm over [16384, 4096] bf16, eps 1e-5: 64 sampled rows against the oracle, the
    parameter gradients against fp64 column sums over all rows."""
    M, N = 16384, 4096
    say("layer norm full size", (M, N))
    x, dy = dev_randn((M, N), 1), dev_randn((M, N), 2)
    gamma = (1 + 0.1 * dev_randn((N,), 3, torch.float32)).to(BT)
    beta = (0.1 * dev_randn((N,), 4, torch.float32)).to(BT)
    y, mean, rstd = ffk.layer_norm_forward(x, gamma, beta, 1e-5)
    dx = torch.empty_like(x)
    dg, db = torch.empty_like(gamma), torch.empty_like(gamma)
    ffk.layer_norm_backward(dy, x, mean, rstd, gamma, dx, dg, db)
    torch.cuda.synchronize()
    g = rng(11)
    rows = np.sort(np.concatenate([g.choice(M, 60, replace=False), [0, 1, M - 2, M - 1]]))
    ridx = torch.from_numpy(rows).cuda()
    xs, dys = to_np(x[ridx]), to_np(dy[ridx])
    gn, bn = to_np(gamma), to_np(beta)
    y_ref, mean_ref, rstd_ref = oracle.layer_norm_forward(xs, gn, bn, 1e-5)
    assert_close(to_np(y[ridx]), y_ref, BF16_RTOL, "y rows")
    assert_close(to_np(mean[ridx]), mean_ref, 2e-5, "mean rows")
    assert_close(to_np(rstd[ridx]), rstd_ref, 2e-5, "rstd rows")
    dx_ref, _, _ = oracle.layer_norm_backward(dys, xs, mean_ref, rstd_ref, gn)
    assert_close(to_np(dx[ridx]), dx_ref, BF16_RTOL, "dx rows")
    # every row: sum_j dx = 0 and sum_j dx * xhat = 0 (to bf16 rounding of dx)
    xd = x.double()
    mean64 = xd.mean(dim=1)
    rstd64 = 1.0 / torch.sqrt(xd.var(dim=1, unbiased=False) + 1e-5)
    assert float((mean.double() - mean64).abs().max()) < 2e-5
    assert float(((rstd.double() - rstd64) / rstd64).abs().max()) < 2e-5
    xhat = (xd - mean64[:, None]) * rstd64[:, None]
    dxd = dx.double()
    scale = dxd.abs().sum(dim=1)
    assert float((dxd.sum(dim=1).abs() / scale).max()) < 2e-3
    assert float(((dxd * xhat).sum(dim=1).abs() / scale).max()) < 4e-3
    # dgamma / dbeta: fp64 column sums over all 16384 rows
    dg_ref = (dy.double() * xhat).sum(dim=0).cpu().numpy()
    db_ref = dy.double().sum(dim=0).cpu().numpy()
    assert_close(to_np(dg), dg_ref, BF16_RTOL, "dgamma")
    assert_close(to_np(db), db_ref, BF16_RTOL, "dbeta")
    assert torch.isfinite(y.float()).all() and torch.isfinite(dx.float()).all()


@pytest.mark.parametrize("op_name", ["add", "mul"])
def test_element_binary_config3(ffk, oracle, op_name):
    """ElementBinary add / mul on [16384, 4096] bf16, forward and backward: the oracle on a
    sampled block of rows, closed forms in fp64 over every element."""
    M, N = 16384, 4096
    op = ffk.OP["EW_ADD" if op_name == "add" else "EW_MUL"]
    say("element binary full size", op_name, (M, N))
    a, b, gy = dev_randn((M, N), 5), dev_randn((M, N), 6), dev_randn((M, N), 7)
    out = ffk.element_binary_forward(op, a, b)
    da, dbt = torch.empty_like(a), torch.empty_like(a)
    ffk.element_binary_backward(op, gy, a, b, da, dbt)
    torch.cuda.synchronize()
    af, bf, gf = a.float(), b.float(), gy.float()
    if op_name == "add":
        assert torch.equal(out, (af + bf).to(BT))
        assert torch.equal(da, gy) and torch.equal(dbt, gy)
    else:
        assert torch.equal(out, (af * bf).to(BT))
        assert torch.equal(da, (gf * bf).to(BT)) and torch.equal(dbt, (gf * af).to(BT))
    r0 = 8191
    sl = slice(r0, r0 + 16)
    an, bn, gn = to_np(a[sl]), to_np(b[sl]), to_np(gy[sl])
    assert_close(to_np(out[sl]), oracle.element_binary_forward(op, an, bn), BF16_RTOL, "out block")
    dl_ref, dr_ref = oracle.element_binary_backward(op, gn, an, bn)
    assert_close(to_np(da[sl]), dl_ref, BF16_RTOL, "dlhs block")
    assert_close(to_np(dbt[sl]), dr_ref, BF16_RTOL, "drhs block")


def test_embedding_config4_tokens(ffk, oracle):
    """65 536 Zipf(1.1) int32 token ids over V 50257 x D 1024: fp32 table, bf16 output and
    output gradient.  Gather bit-exact; deterministic scatter-add bit-exact against the
    oracle's fp32 loop; sorted and atomic paths within 1e-5 of the fp64 sum."""
    V, D, n = 50257, 1024, 65536
    say("embedding tokens full size", (V, D, n))
    g = rng(4)
    ids = zipf_ids(g, n, V).astype(np.int32)
    table = dev_randn((V, D), 8, torch.float32, 0.02)
    dy = dev_randn((n, D), 9)
    idd = to_dev(ids, torch, torch.int32)
    out = ffk.embedding_forward(idd, table, out_dtype=BT)
    assert torch.equal(out, table[idd.long()].to(BT))          # a gather is a copy of rounded rows
    sample = np.sort(g.choice(n, 512, replace=False))
    want = bf16_round(oracle.embedding_forward(ids[sample], to_np(table)))
    assert np.array_equal(to_np(out[torch.from_numpy(sample).cuda()]), want)
    # backward: the oracle's loop over all 65 536 x 1024 additions
    dyn = to_np(dy)
    same_order = oracle.embedding_backward(ids, dyn, V)
    dw = torch.zeros((V, D), device="cuda")
    ffk.embedding_backward(idd, dy, dw, deterministic=True)
    assert np.array_equal(to_np(dw), same_order), "deterministic scatter-add differs from the ordered fp32 sums"
    exact = oracle.embedding_backward(ids, dyn, V, f64=True)
    for mode, kw in (("sorted", dict(workspace=True)), ("atomic", dict(workspace=False))):
        dw = torch.zeros((V, D), device="cuda")
        ffk.embedding_backward(idd, dy, dw, **kw)
        assert_close(to_np(dw), exact, FP32_RTOL, "dW " + mode)
    # untouched rows stay zero; what was added is what came in
    touched = np.zeros(V, bool)
    touched[ids] = True
    assert not to_np(dw)[~touched].any()


def test_embedding_config4_dlrm_table(ffk, oracle):
    """One DLRM table, 1 M x 128 fp32, 16 384 sum bags of 32 Zipf ids: forward bit-exact on
    sampled bags (the oracle sums a bag left to right like the kernel), backward against
    numpy's add.at on the touched rows."""
    V, D, B, bag = 1_000_000, 128, 16384, 32
    say("embedding DLRM table full size", (V, D, B, bag))
    g = rng(6)
    ids = zipf_ids(g, B * bag, V).reshape(B, bag).astype(np.int64)
    table = dev_randn((V, D), 10, torch.float32)
    idd = to_dev(ids, torch, torch.int64)
    out = ffk.embedding_forward(idd, table, aggr=0)
    sample = np.sort(g.choice(B, 256, replace=False))
    rows = np.unique(ids[sample])
    remap = {int(r): i for i, r in enumerate(rows)}
    small_ids = np.vectorize(remap.get)(ids[sample])
    small_table = to_np(table[torch.from_numpy(rows).cuda()])
    want = oracle.embedding_forward(small_ids, small_table, aggr=0)
    assert np.array_equal(to_np(out[torch.from_numpy(sample).cuda()]), want)
    # all bags: fp64 sum of the looked-up rows
    ref_all = table[idd.reshape(-1)].double().reshape(B, bag, D).sum(dim=1)
    assert float((out.double() - ref_all).abs().max() / ref_all.abs().max()) < 1e-6
    dy = dev_randn((B, D), 12, torch.float32)
    touched = np.unique(ids)
    pos = np.searchsorted(touched, ids.reshape(-1))
    want_rows = np.zeros((touched.size, D), np.float64)
    np.add.at(want_rows, pos, np.repeat(to_np(dy).astype(np.float64), bag, axis=0))
    tidx = torch.from_numpy(touched).cuda()
    for mode, kw in (("sorted", dict(workspace=True)), ("deterministic", dict(deterministic=True)),
                     ("atomic", dict(workspace=False))):
        dw = torch.zeros((V, D), device="cuda")
        ffk.embedding_backward(idd, dy, dw, aggr=0, **kw)
        # the hottest row receives about 50 000 gradient rows; with atomics they are added one
        # by one in fp32 in arrival order, whose rounding error grows with the run length
        # (the sorted paths add partial sums of 16), so that path gets 1e-4
        assert_close(to_np(dw[tidx]), want_rows, 1e-4 if mode == "atomic" else FP32_RTOL, "dW touched rows " + mode)
        assert float(dw.double().sum()) == pytest.approx(float(dy.double().sum()) * bag, rel=1e-6)
        assert int((dw != 0).any(dim=1).sum()) <= touched.size


@pytest.mark.parametrize("trans_a,trans_b", [(False, True), (False, False), (True, False)])
def test_gemm_config5_projection(ffk, oracle, trans_a, trans_b):
    """The projection GEMMs of config 5: M 16384, N 4096, K 4096 forward (NT), input gradient
    (NN); weight gradient (TN) M 4096, N 4096, K 16384.  Sampled rows and columns against
    the fp64 oracle, every element through linearity."""
    M, N, K = (4096, 4096, 16384) if trans_a else (16384, 4096, 4096)
    say("gemm config 5", (M, N, K), "ta", trans_a, "tb", trans_b)
    A = dev_randn((K, M) if trans_a else (M, K), 13)
    B = dev_randn((N, K) if trans_b else (K, N), 14, scale=0.02)
    C = torch.full((M, N), 3.0, dtype=BT, device="cuda")
    ffk.gemm(A, B, C, trans_a, trans_b)
    torch.cuda.synchronize()
    g = rng(15)
    rows = np.sort(g.choice(M, 24, replace=False))
    cols = np.sort(g.choice(N, 24, replace=False))
    ridx, cidx = torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda()
    An, Bn = to_np(A), to_np(B)
    A_rows = np.ascontiguousarray(An[:, rows] if trans_a else An[rows])
    B_cols = np.ascontiguousarray(Bn[cols] if trans_b else Bn[:, cols])
    assert_close(to_np(C[ridx]), oracle.gemm_f64(A_rows, Bn, trans_a, trans_b), 2.0 ** -8, "C rows")
    assert_close(to_np(C[:, cidx]), oracle.gemm_f64(An, B_cols, trans_a, trans_b), 2.0 ** -8, "C cols")
    v = torch.randn((N,), device="cuda", dtype=torch.float64)
    A64 = (A.t() if trans_a else A).double()
    B64 = (B.t() if trans_b else B).double()
    want = A64 @ (B64 @ v)
    got = C.double() @ v
    bound = 2.0 ** -8 * (A64.abs() @ (B64.abs() @ v.abs()))
    assert bool(((got - want).abs() <= bound + 1e-6).all())
