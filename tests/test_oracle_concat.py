"""Pins the oracle's Concat restatement (the reference's test only asserts non-zero
output): numpy.concatenate on the reference test's shapes and on ragged inputs, and
split-after-concat for the backward."""
import numpy as np
import pytest

from util import rng


@pytest.mark.parametrize("shapes,axis", [
    ([(2, 4)] * 4, 0),                      # test_concat_kernel.cc: 4 inputs, axis 0
    ([(4, 2)] * 4, 1),                      # ... axis 1
    ([(3, 5, 2), (3, 1, 2), (3, 7, 2)], 1),  # ragged along the axis, trailing dim behind it
    ([(6, 3), (6, 9)], -1),
    ([(5,), (0,), (2,)], 0),                # an empty input
])
def test_concat_forward_is_numpy_concatenate(oracle, shapes, axis):
    g = rng(1)
    ins = [g.standard_normal(s).astype(np.float32) for s in shapes]
    assert np.array_equal(oracle.concat_forward(ins, axis), np.concatenate(ins, axis=axis))


def test_concat_backward_splits_the_gradient_and_adds(oracle):
    g = rng(2)
    shapes = [(3, 5, 2), (3, 1, 2), (3, 7, 2)]
    dout = g.standard_normal((3, 13, 2)).astype(np.float32)
    old = [g.standard_normal(s).astype(np.float32) for s in shapes]
    pieces = np.split(dout, [5, 6], axis=1)
    got = oracle.concat_backward(dout, old, 1, accumulate=True)
    for a, o, p in zip(got, old, pieces):
        assert np.array_equal(a, o + p)
    got = oracle.concat_backward(dout, old, 1, accumulate=False)
    for a, p in zip(got, pieces):
        assert np.array_equal(a, p)
    # forward then backward from zero gives the inputs back
    ins = [g.standard_normal(s).astype(np.float32) for s in shapes]
    back = oracle.concat_backward(oracle.concat_forward(ins, 1), [np.zeros_like(a) for a in ins], 1)
    for a, b in zip(ins, back):
        assert np.array_equal(a, b)
