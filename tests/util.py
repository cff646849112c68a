"""Shared helpers for the parity tests."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def to_dev(a, torch, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def bf16_round(a):
    """Round a float32 array to bf16-representable values (RNE), on the host."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32).numpy()


def to_np(t):
    import torch
    return t.detach().to(torch.float32).cpu().numpy()


# Tolerances stated by the task: fp32 within 1e-5 relative, bf16 within 2e-2
# relative.  "Relative" is taken against the tensor's scale (max |expected|),
# with the usual elementwise rtol on top, so values near zero are not held to
# an absolute precision the datatype cannot deliver.
FP32_RTOL = 1e-5
BF16_RTOL = 2e-2


def assert_close(actual, expected, rtol, what="", max_bad_frac=0.0):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    scale = np.max(np.abs(expected)) if expected.size else 0.0
    atol = rtol * max(scale, 1e-30)
    err = np.abs(actual - expected)
    bound = atol + rtol * np.abs(expected)
    bad = err > bound
    if bad.sum() > max_bad_frac * bad.size:
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            "%s: %d/%d elements out of tolerance (rtol %g); worst at %s: got %r want %r"
            % (what, int(bad.sum()), bad.size, rtol, i, actual[i], expected[i]))
