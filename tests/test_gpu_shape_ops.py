"""Transpose and Gather through the C ABI against the oracle.  Transpose moves bits (and
makes one fp32 add per element when accumulating): exact.  Gather forward is exact;
its backward adds with atomics in an order that varies, so fp32 tolerance 1e-5."""
import itertools
import sys

import numpy as np
import pytest
import torch

from util import assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


CASES = [
    ((2, 3, 4, 5), None),            # every permutation
    ((64, 96), [(1, 0)]),            # plain 2-D, whole tiles and a ragged one
    ((70, 130), [(1, 0)]),
    ((8, 512, 16, 64), [(0, 2, 1, 3), (0, 2, 3, 1), (3, 2, 1, 0)]),   # the head split of attention
    ((3, 1, 40, 1, 24), [(2, 1, 0, 3, 4), (4, 3, 2, 1, 0)]),          # extents of one
    ((5,), [(0,)]),
]


@pytest.mark.parametrize("shape,perms", CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transpose_forward_backward(ffk, oracle, shape, perms, dtype):
    g = rng(5)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    x = rnd(g.standard_normal(shape).astype(np.float32))
    xd = to_dev(x, torch, dtype)
    for perm in (perms or list(itertools.permutations(range(len(shape))))):
        say("transpose", shape, perm, dtype)
        out = ffk.transpose_forward(xd, perm)
        want = oracle.transpose_nd(x, perm)
        assert tuple(out.shape) == want.shape
        assert np.array_equal(to_np(out), want), perm
        # backward: the inverse permutation of the output gradient, added or stored
        dout = rnd(g.standard_normal(want.shape).astype(np.float32))
        old = rnd(g.standard_normal(shape).astype(np.float32))
        inverse = np.argsort(perm)
        for accumulate in (True, False):
            din = to_dev(old, torch, dtype)
            ffk.transpose_backward(to_dev(dout, torch, dtype), din, perm, accumulate=accumulate)
            ref = np.transpose(dout, inverse) + (old if accumulate else 0.0)
            assert np.array_equal(to_np(din), rnd(ref.astype(np.float32))), (perm, accumulate)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.bool, torch.float16, torch.float64])
def test_transpose_moves_any_data_type(ffk, dtype):
    say("transpose", dtype)
    x = (torch.arange(6 * 70 * 9, device="cuda").reshape(6, 70, 9) % (2 if dtype == torch.bool else 1000)).to(dtype)
    for perm in ((2, 0, 1), (0, 2, 1), (1, 0, 2)):
        assert torch.equal(ffk.transpose_forward(x, perm), x.permute(perm).contiguous())
    with pytest.raises(ffk.FFKError, match="not a permutation"):
        ffk.transpose_forward(x, (0, 0, 1))
    if dtype not in (torch.float32, torch.bfloat16):
        with pytest.raises(ffk.FFKError, match="adding supports"):
            ffk.transpose_backward(x.permute(1, 0, 2).contiguous(), torch.zeros_like(x), (1, 0, 2), accumulate=True)


@pytest.mark.parametrize("rows,in_dim,picks", [(5, 33, 17), (64, 4096, 1024), (9, 4100, 4100), (3, 20000, 5000), (7, 16384, 2048),
                                               (4, 1000, 100)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64, torch.bool])
def test_gather_along_the_last_dim(ffk, oracle, rows, in_dim, picks, dtype):
    """Rows picked from densely go through LDS (whole-row staging, vector or element loads), long
    or sparsely picked rows straight from memory: both move values bit for bit."""
    say("gather along the last dim", (rows, in_dim, picks), dtype)
    g = rng(rows + in_dim)
    x = g.integers(-1000, 1000, size=(rows, in_dim)).astype(np.float32)
    idx = g.integers(0, in_dim, size=(rows, picks))
    idx.flat[::53] = in_dim                   # out-of-range entries read 0
    idx.flat[::59] = -3
    xd = to_dev(x, torch).to(dtype) if dtype != torch.bool else to_dev(x, torch) > 0
    out = ffk.gather_forward(xd, to_dev(idx, torch, torch.int64), 1)
    want = oracle.gather_forward(xd.to(torch.float32).cpu().numpy(), idx, 1)   # values as the type holds them
    assert np.array_equal(out.to(torch.float32).cpu().numpy(), want)


@pytest.mark.parametrize("rows,in_dim,picks", [(5, 33, 17), (64, 4096, 1024), (9, 4100, 300), (3, 20000, 5000), (7, 16384, 2048),
                                               (4, 1000, 10)])
@pytest.mark.parametrize("itype", [torch.int32, torch.int64])
def test_gather_backward_along_the_last_dim(ffk, oracle, rows, in_dim, picks, itype):
    """Rows summed in LDS and rows added to with memory atomics give the reference's sums; integer-valued
    gradients make them exact whatever the order of the adds, and unpicked elements keep their bits."""
    say("gather backward along the last dim", (rows, in_dim, picks), itype)
    g = rng(rows + in_dim + 1)
    idx = g.integers(0, in_dim, size=(rows, picks))
    idx[:, : picks // 2] = idx[:, picks // 2: picks // 2 * 2] // 7   # repeated targets
    idx.flat[::53] = in_dim
    idx.flat[::59] = -3
    dout = g.integers(-64, 64, size=(rows, picks)).astype(np.float32)
    old = g.integers(-64, 64, size=(rows, in_dim)).astype(np.float32)
    old.flat[::5] = -0.0
    din = to_dev(old, torch)
    ffk.gather_backward(to_dev(dout, torch), to_dev(idx, torch, itype), din, 1)
    want = oracle.gather_backward(dout, idx, old, 1)
    got = to_np(din)
    assert np.array_equal(got, want)
    untouched = np.ones_like(old, dtype=bool)
    ok = (idx >= 0) & (idx < in_dim)
    untouched[np.nonzero(ok)[0], idx[ok]] = False
    assert np.array_equal(got.view(np.uint32)[untouched], old.view(np.uint32)[untouched])


def test_gather_along_the_last_dim_at_the_benchmarked_size(ffk):
    """[16384,4096] -> [16384,1024] as kernel_bench.py times it: the forward moves the values torch.gather
    moves, the backward gives the sums of torch's scatter_add_ (integer-valued gradients: exact in any order)."""
    say("gather [16384,4096] -> [16384,1024]")
    gen = torch.Generator(device="cuda").manual_seed(5)
    src = torch.randn((16384, 4096), device="cuda", generator=gen)
    idx = torch.randint(0, 4096, (16384, 1024), device="cuda", generator=gen)
    out = ffk.gather_forward(src, idx.to(torch.int32), 1)
    assert torch.equal(out, torch.gather(src, 1, idx))
    dout = torch.randint(-8, 8, (16384, 1024), device="cuda", generator=gen).to(torch.float32)
    old = torch.randint(-8, 8, (16384, 4096), device="cuda", generator=gen).to(torch.float32)
    din = old.clone()
    ffk.gather_backward(dout, idx.to(torch.int32), din, 1)
    assert torch.equal(din, old.scatter_add(1, idx, dout))


@pytest.mark.parametrize("dim", [0, 1, 2])
@pytest.mark.parametrize("itype", [torch.int32, torch.int64])
def test_gather_forward_backward(ffk, oracle, dim, itype):
    say("gather", dim, itype)
    g = rng(6)
    x = g.standard_normal((7, 33, 20)).astype(np.float32)
    shape = list(x.shape)
    shape[dim] = 11
    idx = g.integers(0, x.shape[dim], size=shape)
    idx.flat[::97] = -1                       # out-of-range entries read 0 and scatter nothing
    out = ffk.gather_forward(to_dev(x, torch), to_dev(idx, torch, itype), dim)
    assert np.array_equal(to_np(out), oracle.gather_forward(x, idx, dim))
    dout = g.standard_normal(shape).astype(np.float32)
    old = g.standard_normal(x.shape).astype(np.float32)
    din = to_dev(old, torch)
    ffk.gather_backward(to_dev(dout, torch), to_dev(idx, torch, itype), din, dim)
    assert_close(to_np(din), oracle.gather_backward(dout, idx, old, dim), 1e-5, "gather backward")
    # bf16 values move bit for bit
    xb = bf16_round(x)
    outb = ffk.gather_forward(to_dev(xb, torch, torch.bfloat16), to_dev(idx, torch, itype), dim)
    assert np.array_equal(to_np(outb), oracle.gather_forward(xb, idx, dim))
