"""Pins the oracle's Transpose and Gather restatements: the reference's own known-answer
vector for the 2-D transpose (tensor_accessor_transpose), numpy.transpose on every
permutation of a 4-D tensor, numpy.take_along_axis / numpy.add.at for Gather."""
import itertools
import json
import os

import numpy as np
import pytest

from util import rng


def test_transpose_reference_kat(oracle, golden_dir):
    t = json.load(open(os.path.join(golden_dir, "tensor_accessor_kat.json")))["transpose"]
    got = oracle.transpose_nd(np.array(t["input"], dtype=np.float32), (1, 0))
    assert np.array_equal(got, np.array(t["output"], dtype=np.float32))


def test_transpose_every_permutation_of_four_dims(oracle):
    x = rng(1).standard_normal((2, 3, 4, 5)).astype(np.float32)
    for perm in itertools.permutations(range(4)):
        assert np.array_equal(oracle.transpose_nd(x, perm), np.transpose(x, perm)), perm
    # accumulate: into + permuted
    into = rng(2).standard_normal((5, 2, 4, 3)).astype(np.float32)
    assert np.array_equal(oracle.transpose_nd(x, (3, 0, 2, 1), into=into), into + np.transpose(x, (3, 0, 2, 1)))


@pytest.mark.parametrize("dim", [0, 1, 2, -1])
def test_gather_is_take_along_axis(oracle, dim):
    g = rng(3)
    x = g.standard_normal((4, 6, 5)).astype(np.float32)
    shape = list(x.shape)
    shape[dim] = 3
    idx = g.integers(0, x.shape[dim], size=shape)
    assert np.array_equal(oracle.gather_forward(x, idx, dim), np.take_along_axis(x, idx, axis=dim))
    dout = g.standard_normal(shape).astype(np.float32)
    want = np.zeros_like(x, dtype=np.float64)
    d = dim if dim >= 0 else 3 + dim
    coords = list(np.indices(shape))
    coords[d] = idx
    np.add.at(want, tuple(coords), dout.astype(np.float64))
    got = oracle.gather_backward(dout, idx, np.zeros_like(x), dim)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
