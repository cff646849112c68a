"""Embedding gather / scatter-add parity against the oracle."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def zipf_ids(g, n, vocab, s=1.1):
    """Zipf(s) over [0, vocab) by inverse CDF."""
    p = 1.0 / np.arange(1, vocab + 1) ** s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, g.random(n)), vocab - 1)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("wdt,odt", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                     (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("V,D,n", [(10, 4, 7), (1000, 128, 513), (50257, 1024, 4096), (97, 33, 50)])
def test_gather_bit_exact(ffk, oracle, idt, wdt, odt, V, D, n):
    say("embedding gather", idt, wdt, odt, (V, D, n))
    g = rng(V + D)
    w = (g.standard_normal((V, D)) * 0.02).astype(np.float32)
    if wdt == torch.bfloat16:
        w = bf16_round(w)
    ids = zipf_ids(g, n, V)
    want = oracle.embedding_forward(ids, w)
    if odt == torch.bfloat16:
        want = bf16_round(want)
    out = ffk.embedding_forward(to_dev(ids, torch, idt), to_dev(w, torch, wdt), out_dtype=odt)
    assert np.array_equal(to_np(out), want)   # a gather is a copy: bit-exact


@pytest.mark.parametrize("aggr", [0, 1])
@pytest.mark.parametrize("V,D,B,bag", [(1000, 128, 64, 32), (100, 16, 9, 5), (5000, 128, 1024, 32), (50, 7, 3, 1)])
def test_bag_forward(ffk, oracle, aggr, V, D, B, bag):
    say("embedding bag fwd", aggr, (V, D, B, bag))
    g = rng(B + bag)
    w = g.standard_normal((V, D)).astype(np.float32)
    ids = zipf_ids(g, B * bag, V).reshape(B, bag)
    want = oracle.embedding_forward(ids, w, aggr=aggr)
    out = ffk.embedding_forward(to_dev(ids, torch, torch.int64), to_dev(w, torch), aggr=aggr)
    # same left-to-right fp32 summation order as the oracle: bit-exact
    assert np.array_equal(to_np(out), want)


@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,D,n", [(10, 4, 7), (1000, 128, 2000), (50257, 1024, 2048), (97, 33, 50)])
def test_scatter_add(ffk, oracle, gdt, V, D, n):
    say("embedding scatter-add", gdt, (V, D, n))
    g = rng(V * 3 + n)
    ids = zipf_ids(g, n, V)
    dy = g.standard_normal((n, D)).astype(np.float32)
    if gdt == torch.bfloat16:
        dy = bf16_round(dy)
    dw0 = g.standard_normal((V, D)).astype(np.float32)
    want = oracle.embedding_backward(ids, dy, V, f64=True, dw_init=dw0)
    dw = to_dev(dw0, torch)
    ffk.embedding_backward(to_dev(ids, torch, torch.int32), to_dev(dy, torch, gdt), dw)
    # fp32 atomics: order-dependent rounding, checked against the fp64 sum
    assert_close(to_np(dw), want, FP32_RTOL, "dW")


@pytest.mark.parametrize("aggr", [0, 1])
def test_bag_backward(ffk, oracle, aggr):
    V, D, B, bag = 2000, 128, 256, 32
    say("embedding bag bwd", aggr)
    g = rng(5)
    ids = zipf_ids(g, B * bag, V).reshape(B, bag)
    dy = g.standard_normal((B, D)).astype(np.float32)
    want = oracle.embedding_backward(ids, dy, V, aggr=aggr, f64=True)
    dw = torch.zeros((V, D), device="cuda")
    ffk.embedding_backward(to_dev(ids, torch, torch.int64), to_dev(dy, torch), dw, aggr=aggr)
    assert_close(to_np(dw), want, FP32_RTOL, "dW")


def test_out_of_range_ids_are_skipped_and_errors(ffk):
    say("embedding invalid ids")
    w = torch.ones((10, 8), device="cuda")
    ids = torch.tensor([1, 10, -1, 3], dtype=torch.int64, device="cuda")
    out = ffk.embedding_forward(ids, w)
    assert out[0].sum() == 8 and out[1].sum() == 0 and out[2].sum() == 0 and out[3].sum() == 8
    dw = torch.zeros((10, 8), device="cuda")
    ffk.embedding_backward(ids, torch.ones((4, 8), device="cuda"), dw)
    assert dw.sum() == 16
    with pytest.raises(ffk.FFKError, match="bag must be 1"):
        ffk.check(ffk.lib().ffk_embedding_forward(0, ffk.INT64, ffk.FLOAT, ffk.FLOAT, ids.data_ptr(),
                                                  out.data_ptr(), w.data_ptr(), ffk.AGGR_NONE, 2, 2, 8, 10))
    # empty input is a no-op
    ffk.check(ffk.lib().ffk_embedding_forward(0, ffk.INT64, ffk.FLOAT, ffk.FLOAT, None, None, None,
                                              ffk.AGGR_NONE, 0, 1, 8, 10))


@pytest.mark.parametrize("mode", ["atomic", "sorted", "deterministic"])
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,D,B,bag", [(300, 1024, 5000, 1), (50, 64, 2300, 3), (1000, 100, 700, 4),
                                       (4000, 192, 2049, 2), (7, 256, 4096, 1), (20, 8, 5, 1)])
def test_scatter_add_modes(ffk, oracle, mode, idt, gdt, V, D, B, bag):
    """The three backward paths on the same inputs: plain atomics (no scratch),
    sorted runs summed in registers (scratch given), and the deterministic
    variant.  Ragged ends, row widths below and above one wave, heavy
    duplication (runs far longer than a walker's chunk), ids outside the table."""
    say("embedding scatter-add", mode, idt, gdt, (V, D, B, bag))
    g = rng(V + D + B)
    ids = zipf_ids(g, B * bag, V).reshape(B, bag)
    bad = g.random(ids.shape) < 0.01
    ids_dev = np.where(bad, np.where(g.random(ids.shape) < 0.5, -1, V + 5), ids)
    dy = g.standard_normal((B, D)).astype(np.float32)
    if gdt == torch.bfloat16:
        dy = bf16_round(dy)
    aggr = 0 if bag > 1 else -1
    # expected: invalid lookups contribute nothing (checked against the oracle
    # on the all-valid ids, then used with the invalid ones masked out)
    rows = np.repeat(np.arange(B), bag).reshape(B, bag)
    all_valid = np.zeros((V, D), dtype=np.float64)
    np.add.at(all_valid, ids.reshape(-1), dy[rows.reshape(-1)].astype(np.float64))
    assert_close(all_valid, oracle.embedding_backward(ids, dy, V, aggr=aggr, f64=True), 1e-6,
                 "test-side expectation vs oracle")
    want = np.zeros((V, D), dtype=np.float64)
    ok = ~bad
    np.add.at(want, ids[ok], dy[rows[ok]].astype(np.float64))
    kw = dict(atomic=dict(workspace=False), sorted=dict(workspace=True),
              deterministic=dict(deterministic=True))[mode]
    dw = torch.zeros((V, D), device="cuda")
    ffk.embedding_backward(to_dev(ids_dev, torch, idt), to_dev(dy, torch, gdt), dw, aggr=aggr, **kw)
    assert_close(to_np(dw), want, FP32_RTOL, "dW")
    if mode == "deterministic":
        # every row summed in ascending lookup order from zero: the oracle's
        # fp32 loop does the same additions in the same order -> same bits
        ids_masked = np.where(bad, V, ids)   # the oracle skips out-of-range ids
        same = oracle.embedding_backward(ids_masked, dy, V + 1, aggr=aggr)[:V]
        assert np.array_equal(to_np(dw), same)
        dw2 = torch.zeros((V, D), device="cuda")
        ffk.embedding_backward(to_dev(ids_dev, torch, idt), to_dev(dy, torch, gdt), dw2, aggr=aggr, **kw)
        assert torch.equal(dw, dw2)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("dt,ndt", [(torch.float16, np.float16), (torch.float64, np.float64)])
@pytest.mark.parametrize("aggr,V,D,B,bag", [(-1, 97, 33, 50, 1), (0, 1000, 128, 64, 32), (1, 100, 17, 9, 5),
                                            (1, 40, 8, 700, 4)])
def test_half_and_double_tables(ffk, oracle, idt, dt, ndt, aggr, V, D, B, bag):
    """The reference's HALF and DOUBLE instantiations: table, output and gradients of one type, all
    arithmetic in that type.  Forward: the bag is summed entry by entry, so the oracle's order
    is the device's and random data must match to the bit.  Backward: the atomics' order is
    free, so the gradients are eighths of small integers, whose sums are exact in half whatever
    the order (|sum| <= 700 * 4 * 2 / 8 < 2048 / 8 steps) -- bit-exact again."""
    say("embedding HALF/DOUBLE tables", idt, dt, (aggr, V, D, B, bag))
    g = rng(V + B + bag)
    w = g.standard_normal((V, D)).astype(ndt)
    ids = zipf_ids(g, B * bag, V).reshape(B, bag) if aggr >= 0 else zipf_ids(g, B, V)
    want = oracle.embedding_forward_typed(ids, w, aggr=aggr)
    wd, idd = torch.from_numpy(w).cuda(), to_dev(ids, torch, idt)
    out = ffk.embedding_forward(idd, wd, aggr=aggr)
    assert out.dtype == dt
    assert np.array_equal(out.cpu().numpy(), want)
    # backward: exact sums; AVG's factor half(1/bag) is exact for bag 4 and rounds for bag 5, and is
    # applied to the gradient once per bag, before the adds, in the oracle as on the device
    dy = (g.integers(-2, 3, (ids.shape[0], D)) * (bag if aggr == 1 and bag == 4 else 1) / 8.0).astype(ndt)
    init = (g.integers(-4, 5, (V, D)) / 4.0).astype(ndt)
    if aggr == 1 and bag == 5:
        # half(1/5) times an eighth is not a short binary fraction: keep every row's lookups few
        # enough that order cannot matter by giving each lookup its own row
        ids = g.permutation(V)[:B * bag].reshape(B, bag) if B * bag <= V else ids
        idd = to_dev(ids, torch, idt)
    want_dw = oracle.embedding_backward_typed(ids, dy, V, aggr=aggr, dw_init=init)
    dw = torch.from_numpy(init).cuda()
    ffk.embedding_backward_typed(idd, torch.from_numpy(dy).cuda(), dw, aggr=aggr)
    assert dw.dtype == dt
    assert np.array_equal(dw.cpu().numpy(), want_dw)


def test_half_and_double_tables_errors(ffk):
    w = torch.ones((10, 8), device="cuda", dtype=torch.float16)
    ids = torch.tensor([1, 10, -1, 3], dtype=torch.int64, device="cuda")
    out = ffk.embedding_forward(ids, w)  # ids outside the table are skipped, as for the other types
    assert out[0].sum() == 8 and out[1].sum() == 0 and out[2].sum() == 0
    dw = torch.zeros((10, 8), device="cuda", dtype=torch.float16)
    ffk.embedding_backward_typed(ids, torch.ones((4, 8), device="cuda", dtype=torch.float16), dw)
    assert dw.sum() == 16
    # FLOAT goes to the fp32 entry point; bf16 has no typed form (its gradients accumulate in fp32)
    dwf = torch.zeros((10, 8), device="cuda")
    ffk.embedding_backward_typed(ids, torch.ones((4, 8), device="cuda"), dwf)
    assert dwf.sum() == 16
    with pytest.raises(ffk.FFKError, match="not supported"):
        ffk.embedding_backward_typed(ids, torch.ones((4, 8), device="cuda", dtype=torch.bfloat16),
                                     torch.zeros((10, 8), device="cuda", dtype=torch.bfloat16))
    with pytest.raises(ffk.FFKError, match="not supported"):  # table and output types must agree
        ffk.embedding_forward(ids, w, out_dtype=torch.float32)
