"""Concat through the C ABI against the oracle: bit-exact (a move, and one fp32 add per
element in the accumulating backward)."""
import sys

import numpy as np
import pytest
import torch

from util import bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("shapes,axis", [
    ([(2, 4)] * 4, 0),                       # the reference test's shapes
    ([(4, 2)] * 4, 1),
    ([(3, 5, 2), (3, 1, 2), (3, 7, 2)], 1),   # not a multiple of 16 bytes: element-wise path
    ([(64, 128)] * 27, 1),                   # DLRM interaction: 26 sparse features + the dense one
    ([(300, 64), (300, 256), (300, 8)], -1),  # 16-byte path, ragged
    ([(5,), (0,), (2,)], 0),                 # an empty input
    ([(2, 3, 4)] * 70, 1),                   # more inputs than one launch takes
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_concat_forward_backward(ffk, oracle, shapes, axis, dtype):
    say("concat", shapes[:3], len(shapes), axis, dtype)
    g = rng(3)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    ins = [rnd(g.standard_normal(s).astype(np.float32)) for s in shapes]
    dev = [to_dev(a, torch, dtype) for a in ins]
    out = ffk.concat_forward(dev, axis)
    want = oracle.concat_forward(ins, axis)
    assert tuple(out.shape) == want.shape
    assert np.array_equal(to_np(out), want)
    dout = rnd(g.standard_normal(want.shape).astype(np.float32))
    old = [rnd(g.standard_normal(s).astype(np.float32)) for s in shapes]
    for accumulate in (True, False):
        grads = [to_dev(a, torch, dtype) for a in old]
        ffk.concat_backward(to_dev(dout, torch, dtype), grads, axis, accumulate=accumulate)
        ref = oracle.concat_backward(dout, old, axis, accumulate=accumulate)
        for got, r in zip(grads, ref):
            assert np.array_equal(to_np(got), rnd(r))


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.bool, torch.float16, torch.float64])
def test_concat_moves_any_data_type(ffk, dtype):
    say("concat", dtype)
    parts = [(torch.arange(3 * n, device="cuda").reshape(3, n) % 2 if dtype == torch.bool
              else torch.arange(3 * n, device="cuda").reshape(3, n)).to(dtype) for n in (5, 1, 8)]
    out = ffk.concat_forward(parts, 1)
    assert torch.equal(out, torch.cat(parts, dim=1))
    back = [torch.zeros_like(p) for p in parts]
    ffk.concat_backward(out, back, 1, accumulate=False)
    for a, b in zip(parts, back):
        assert torch.equal(a, b)
    if dtype not in (torch.float32, torch.bfloat16):
        with pytest.raises(ffk.FFKError, match="accumulating backward"):
            ffk.concat_backward(out, back, 1, accumulate=True)


def test_concat_on_unaligned_views(ffk, oracle):
    say("concat unaligned")
    g = rng(4)
    a = g.standard_normal((8, 16)).astype(np.float32)
    b = g.standard_normal((8, 32)).astype(np.float32)
    da = torch.empty(8 * 16 + 1, device="cuda")[1:].view(8, 16)   # 4 bytes past a 16-byte boundary
    da.copy_(to_dev(a, torch))
    out = ffk.concat_forward([da, to_dev(b, torch)], 1)
    assert np.array_equal(to_np(out), np.concatenate([a, b], axis=1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_split_is_concat_read_the_other_way(ffk, oracle, dtype):
    say("split", dtype)
    g = rng(8)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    x = rnd(g.standard_normal((6, 29, 8)).astype(np.float32))
    sizes = [5, 1, 16, 7]
    outs = ffk.split_forward(to_dev(x, torch, dtype), sizes, 1)
    for got, want in zip(outs, np.split(x, np.cumsum(sizes)[:-1], axis=1)):
        assert np.array_equal(to_np(got), want)
    douts = [rnd(g.standard_normal(o.shape).astype(np.float32)) for o in outs]
    old = rnd(g.standard_normal(x.shape).astype(np.float32))
    for accumulate in (True, False):
        din = to_dev(old, torch, dtype)
        ffk.split_backward([to_dev(d, torch, dtype) for d in douts], din, 1, accumulate=accumulate)
        want = oracle.concat_forward(douts, 1) + (old if accumulate else 0.0)
        assert np.array_equal(to_np(din), rnd(want.astype(np.float32)))
