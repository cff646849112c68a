"""Pins the oracle's optimizer / loss-backward restatements (the reference has
no test for them): closed forms in fp64, torch.optim.SGD (which the reference
kernel cites as its model), and special cases that a dropped term, a swapped
operand or a wrong sign would break."""
import numpy as np
import pytest

from util import rng


def test_sgd_matches_torch_optim_sgd(oracle):
    import torch
    g = rng(1)
    for momentum, nesterov, wd in [(0.0, False, 0.0), (0.9, False, 0.0), (0.9, True, 1e-2), (0.5, False, 0.1)]:
        w0 = g.standard_normal(257).astype(np.float32)
        p = torch.nn.Parameter(torch.tensor(w0, dtype=torch.float64))
        opt = torch.optim.SGD([p], lr=0.05, momentum=momentum, nesterov=nesterov, weight_decay=wd)
        w, v = w0.copy(), (np.zeros_like(w0) if momentum > 0 else None)
        for step in range(4):
            grad = g.standard_normal(257).astype(np.float32)
            p.grad = torch.tensor(grad, dtype=torch.float64)
            opt.step()
            w, v = oracle.sgd_update(w, grad, 0.05, momentum, nesterov, wd, v)
            np.testing.assert_allclose(w, p.detach().numpy(), rtol=2e-6, atol=2e-6)


def test_sgd_special_cases(oracle):
    g = rng(2)
    w0 = g.standard_normal(100).astype(np.float32)
    grad = g.standard_normal(100).astype(np.float32)
    # lr = 0 leaves the weights, but still updates the momentum buffer
    w, v = oracle.sgd_update(w0, grad, 0.0, 0.9, False, 0.0, np.ones(100, np.float32))
    assert np.array_equal(w, w0)
    np.testing.assert_allclose(v, 0.9 + grad, rtol=1e-6)
    # plain step
    w, _ = oracle.sgd_update(w0, grad, 0.5)
    np.testing.assert_allclose(w, w0 - 0.5 * grad, rtol=1e-6, atol=1e-7)
    # weight decay alone (zero gradient) shrinks the weights by lr * wd
    w, _ = oracle.sgd_update(w0, np.zeros(100, np.float32), 0.1, weight_decay=0.5)
    np.testing.assert_allclose(w, w0 * (1 - 0.05), rtol=1e-6, atol=1e-7)
    # replicas are summed before the step
    two = np.concatenate([grad, 2 * grad])
    w, _ = oracle.sgd_update(w0, two, 0.5, replicas=2)
    np.testing.assert_allclose(w, w0 - 1.5 * grad, rtol=1e-6, atol=1e-6)


def test_adam_closed_form(oracle):
    g = rng(3)
    w0 = g.standard_normal(300).astype(np.float32)
    m0 = (g.standard_normal(300) * 0.1).astype(np.float32)
    v0 = (g.random(300) * 0.1).astype(np.float32)
    grad = g.standard_normal(300).astype(np.float32)
    a, b1, b2, wd, eps = 1e-2, 0.9, 0.99, 0.05, 1e-6
    w, m, v = oracle.adam_update(w0, grad, m0, v0, a, b1, b2, wd, eps)
    gt = grad.astype(np.float64) + wd * w0.astype(np.float64)
    mt = b1 * m0 + (1 - b1) * gt
    vt = b2 * v0 + (1 - b2) * gt * gt
    np.testing.assert_allclose(m, mt, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(v, vt, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(w, w0 - a * mt / (np.sqrt(vt) + eps), rtol=2e-6, atol=1e-6)
    # first step from zero state: the move is alpha_t (1-b1) g / (sqrt(1-b2) |g| + eps)
    z = np.zeros(300, np.float32)
    w1, _, _ = oracle.adam_update(w0, grad, z, z, a, b1, b2, 0.0, 0.0)
    np.testing.assert_allclose(w0 - w1, a * (1 - b1) / np.sqrt(1 - b2) * np.sign(grad), rtol=1e-4)


def test_loss_backward_closed_forms(oracle):
    g = rng(4)
    B, C = 12, 7
    logit = g.random((B, C)).astype(np.float32)
    label = g.integers(0, C, size=B)
    scale = 1.0 / B
    want = logit.astype(np.float64).copy()
    want[np.arange(B), label] -= 1.0
    got = oracle.sparse_cce_loss_backward(logit, label, B, C, 1, scale)
    np.testing.assert_allclose(got, want * scale, rtol=1e-6, atol=1e-7)
    # k > 1: k consecutive rows share a label and the scale grows by k
    k = 3
    lab2 = g.integers(0, C, size=B // k)
    want = logit.astype(np.float64).copy()
    want[np.arange(B), np.repeat(lab2, k)] -= 1.0
    got = oracle.sparse_cce_loss_backward(logit, lab2, B, C, k, scale)
    np.testing.assert_allclose(got, want * scale * k, rtol=1e-6, atol=1e-7)
    lab = g.random((B, C)).astype(np.float32)
    np.testing.assert_allclose(oracle.difference_loss_backward(logit, lab, 0.25),
                               (logit.astype(np.float64) - lab) * 0.25, rtol=1e-6, atol=1e-7)
    assert np.array_equal(oracle.identity_loss_backward((5, 3), 0.125), np.full((5, 3), 0.125, np.float32))


def test_adam_trajectory_matches_torch_optim_adam(oracle):
    """With epsilon = 0 the reference's form (alpha_t = alpha sqrt(1 - b2^t) / (1 - b1^t) folded
    into the step, lib/pcg/src/pcg/optimizer_attrs.cc:6-26) is algebraically torch.optim.Adam's
    bias-corrected step, L2 weight decay included; five steps of both must agree."""
    import torch
    g = rng(5)
    w0 = g.standard_normal(200).astype(np.float32)
    grads = [g.standard_normal(200).astype(np.float32) for _ in range(5)]
    alpha, b1, b2, wd = 1e-2, 0.9, 0.99, 0.03
    p = torch.nn.Parameter(torch.tensor(w0, dtype=torch.float64))
    opt = torch.optim.Adam([p], lr=alpha, betas=(b1, b2), eps=0.0, weight_decay=wd)
    w = w0.copy()
    m = np.zeros(200, np.float32)
    v = np.zeros(200, np.float32)
    beta1_t, beta2_t = 1.0, 1.0
    for grad in grads:
        # the attrs as they stand after get_optimizer_attrs_for_next_iter has run t times
        beta1_t *= b1
        beta2_t *= b2
        alpha_t = alpha * np.sqrt(1 - beta2_t) / (1 - beta1_t)
        w, m, v = oracle.adam_update(w, grad, m, v, alpha_t, b1, b2, wd, 0.0)
        p.grad = torch.tensor(grad, dtype=torch.float64)
        opt.step()
    np.testing.assert_allclose(w, p.detach().numpy(), rtol=2e-5, atol=2e-6)


def test_loss_backward_is_the_gradient_of_the_loss(oracle):
    """Autograd of the loss each kernel differentiates: cross-entropy of softmax outputs with
    respect to the pre-softmax scores (the kernels are handed the softmax output as `logit`),
    and the mean squared error."""
    import torch
    g = rng(6)
    B, C = 9, 11
    z = torch.tensor(g.standard_normal((B, C)), dtype=torch.float64, requires_grad=True)
    label = g.integers(0, C, size=B)
    torch.nn.functional.cross_entropy(z, torch.tensor(label), reduction="mean").backward()
    probs = torch.softmax(z.detach(), dim=1).numpy().astype(np.float32)
    got = oracle.sparse_cce_loss_backward(probs, label, B, C, 1, 1.0 / B)
    np.testing.assert_allclose(got, z.grad.numpy(), rtol=1e-5, atol=1e-7)
    # dense labels: soft targets that sum to one
    soft = g.random((B, C))
    soft /= soft.sum(axis=1, keepdims=True)
    z.grad = None
    (-(torch.tensor(soft) * torch.log_softmax(z, dim=1)).sum(dim=1).mean()).backward()
    got = oracle.difference_loss_backward(probs, soft.astype(np.float32), 1.0 / B)
    np.testing.assert_allclose(got, z.grad.numpy(), rtol=1e-5, atol=1e-7)
    x = torch.tensor(g.standard_normal((B, C)), dtype=torch.float64, requires_grad=True)
    target = g.standard_normal((B, C))
    torch.nn.functional.mse_loss(x, torch.tensor(target)).backward()
    got = oracle.difference_loss_backward(x.detach().numpy().astype(np.float32), target.astype(np.float32), 2.0 / (B * C))
    np.testing.assert_allclose(got, x.grad.numpy(), rtol=1e-5, atol=1e-7)
