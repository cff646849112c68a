"""SGD / Adam updates, loss-function backward and Cast against the oracle.
These kernels round every fp32 operation separately, like the reference's CPU
evaluation, so fp32 results are compared bit for bit."""
import sys

import numpy as np
import pytest
import torch

from util import bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("n", [1, 7, 1024, 100003])
@pytest.mark.parametrize("momentum,nesterov,wd", [(0.0, False, 0.0), (0.9, False, 0.0), (0.9, True, 0.01),
                                                  (0.5, False, 0.1)])
def test_sgd_update_bit_exact(ffk, oracle, n, momentum, nesterov, wd):
    say("sgd", n, momentum, nesterov, wd)
    g = rng(n + int(momentum * 10))
    w0 = g.standard_normal(n).astype(np.float32)
    v0 = g.standard_normal(n).astype(np.float32) if momentum > 0 else None
    grad = g.standard_normal(n).astype(np.float32)
    w_ref, v_ref = oracle.sgd_update(w0, grad, 0.05, momentum, nesterov, wd, v0)
    w = to_dev(w0, torch)
    v = to_dev(v0, torch) if v0 is not None else None
    lowp = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    ffk.sgd_update(w, to_dev(grad, torch), 0.05, momentum, nesterov, wd, v, weight_lowp=lowp)
    assert np.array_equal(to_np(w), w_ref)
    if v is not None:
        assert np.array_equal(to_np(v), v_ref)
    assert np.array_equal(to_np(lowp), bf16_round(w_ref))


def test_sgd_update_bf16_gradient_and_replicas(ffk, oracle):
    say("sgd bf16 grad, 3 replicas")
    g = rng(5)
    n = 4096
    w0 = g.standard_normal(n).astype(np.float32)
    grad = bf16_round(g.standard_normal(3 * n))
    w_ref, _ = oracle.sgd_update(w0, grad, 0.1, replicas=3)
    w = to_dev(w0, torch)
    ffk.sgd_update(w, to_dev(grad, torch, torch.bfloat16), 0.1, num_replicas=3)
    assert np.array_equal(to_np(w), w_ref)


def test_sgd_update_errors(ffk):
    w = torch.zeros(8, device="cuda")
    g = torch.zeros(8, device="cuda")
    with pytest.raises(ffk.FFKError, match="sgd_v must be given exactly when momentum"):
        ffk.sgd_update(w, g, 0.1, momentum=0.9)
    with pytest.raises(ffk.FFKError, match="sgd_v must be given exactly when momentum"):
        ffk.sgd_update(w, g, 0.1, momentum=0.0, sgd_v=torch.zeros(8, device="cuda"))
    with pytest.raises(ffk.FFKError, match="not supported"):
        ffk.sgd_update(w, torch.zeros(8, device="cuda", dtype=torch.float64), 0.1)


@pytest.mark.parametrize("n", [3, 4096, 100003])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_adam_update_bit_exact(ffk, oracle, n, gdt):
    say("adam", n, gdt)
    g = rng(n)
    w0 = g.standard_normal(n).astype(np.float32)
    m0 = (g.standard_normal(n) * 0.1).astype(np.float32)
    v0 = (g.random(n) * 0.1).astype(np.float32)
    grad = g.standard_normal(n).astype(np.float32)
    if gdt == torch.bfloat16:
        grad = bf16_round(grad)
    args = dict(alpha_t=1e-2, beta1=0.9, beta2=0.99, weight_decay=0.05, epsilon=1e-6)
    w_ref, m_ref, v_ref = oracle.adam_update(w0, grad, m0, v0, **args)
    w, m, v = to_dev(w0, torch), to_dev(m0, torch), to_dev(v0, torch)
    ffk.adam_update(w, to_dev(grad, torch, gdt), m, v, **args)
    assert np.array_equal(to_np(m), m_ref)
    assert np.array_equal(to_np(v), v_ref)
    assert np.array_equal(to_np(w), w_ref)


@pytest.mark.parametrize("C", [1000, 1003, 3, 1])
def test_loss_backward_bit_exact(ffk, oracle, C):
    say("loss backward", C)
    g = rng(9)
    B = 96
    logit = g.random((B, C)).astype(np.float32)
    label = g.integers(0, C, size=B).astype(np.int32)
    scale = 1.0 / B
    want = oracle.sparse_cce_loss_backward(logit, label, B, C, 1, scale)
    got = ffk.sparse_categorical_crossentropy_loss_backward(to_dev(logit, torch), to_dev(label, torch, torch.int32),
                                                            B, C, 1, scale)
    assert np.array_equal(to_np(got), want)
    k = 4
    lab2 = g.integers(0, C, size=B // k).astype(np.int32)
    want = oracle.sparse_cce_loss_backward(logit, lab2, B, C, k, scale)
    got = ffk.sparse_categorical_crossentropy_loss_backward(to_dev(logit, torch), to_dev(lab2, torch, torch.int32),
                                                            B, C, k, scale)
    assert np.array_equal(to_np(got), want)
    lab = g.random((B, C)).astype(np.float32)
    for kind, s in (("categorical_crossentropy", scale), ("mean_squared_error_avg", 2.0 / (B * C))):
        want = oracle.difference_loss_backward(logit, lab, s)
        got = ffk.difference_loss_backward(kind, to_dev(logit, torch), to_dev(lab, torch), s)
        assert np.array_equal(to_np(got), want), kind
    got = ffk.identity_loss_backward(to_dev(logit, torch), scale)
    assert np.array_equal(to_np(got), oracle.identity_loss_backward(logit.shape, scale))
    with pytest.raises(ffk.FFKError, match="bad sizes"):
        ffk.check(ffk.lib().ffk_identity_loss_backward(0, got.data_ptr(), got.data_ptr(), 10, 11, 1.0))


NP = {torch.bool: np.bool_, torch.int32: np.int32, torch.int64: np.int64, torch.float16: np.float16,
      torch.float32: np.float32, torch.float64: np.float64}


@pytest.mark.parametrize("idt", [torch.bool, torch.int32, torch.int64, torch.float16, torch.float32,
                                 torch.float64, torch.bfloat16])
@pytest.mark.parametrize("odt", [torch.bool, torch.int32, torch.int64, torch.float16, torch.float32,
                                 torch.float64, torch.bfloat16])
def test_cast_forward_backward(ffk, oracle, idt, odt):
    say("cast", idt, odt)
    g = rng(3)
    n = 1003
    # small integers and halves: exactly representable in every type, so the
    # conversion itself (not a rounding choice) is what is checked ...
    vals = g.integers(-64, 64, size=n).astype(np.float64) / (1.0 if idt in (torch.int32, torch.int64, torch.bool) else 2.0)
    if idt == torch.bool:
        vals = (vals > 0).astype(np.float64)
    x = torch.tensor(vals, dtype=torch.float64).to(idt).cuda()
    src = x.cpu().to(torch.float64).numpy()
    if odt == torch.bool:
        want = src != 0
    elif odt in (torch.int32, torch.int64):
        want = np.trunc(src)          # static_cast truncates toward zero
    else:
        want = src
    out = torch.empty(n, dtype=odt, device="cuda")
    ffk.cast_forward(x, out)
    assert np.array_equal(out.cpu().to(torch.float64).numpy(), want.astype(np.float64))
    # ... backward adds the cast gradient to what is there
    old = torch.tensor(g.integers(0, 2 if odt == torch.bool else 8, size=n), dtype=torch.float64).to(odt).cuda()
    acc = old.clone()
    ffk.cast_backward(x, acc)
    if odt == torch.bool:
        want_b = (want != 0) | (old.cpu().numpy() != 0)
    else:
        want_b = want.astype(np.float64) + old.cpu().to(torch.float64).numpy()
    assert np.array_equal(acc.cpu().to(torch.float64).numpy(), want_b.astype(np.float64))


def test_cast_rounding_to_bf16_and_half(ffk, oracle):
    say("cast rounding")
    g = rng(11)
    x = g.standard_normal(4096).astype(np.float32)
    out = torch.empty(4096, dtype=torch.bfloat16, device="cuda")
    ffk.cast_forward(to_dev(x, torch), out)
    assert np.array_equal(to_np(out), bf16_round(x))        # round to nearest even
    outh = torch.empty(4096, dtype=torch.float16, device="cuda")
    ffk.cast_forward(to_dev(x, torch), outh)
    assert np.array_equal(outh.cpu().numpy(), oracle.cast(x, np.float16))
    outd = torch.empty(4096, dtype=torch.float64, device="cuda")
    ffk.cast_forward(to_dev(x, torch), outd)
    assert np.array_equal(outd.cpu().numpy(), oracle.cast(x, np.float64))


def test_cast_and_loss_on_unaligned_views(ffk, oracle):
    say("cast / loss, pointers off the 16-byte grid")
    g = rng(12)
    n = 777
    x = g.standard_normal(n + 1).astype(np.float32)
    xd = to_dev(x, torch)[1:]                       # 4 bytes past a 16-byte boundary
    out = torch.empty(n + 3, dtype=torch.bfloat16, device="cuda")[3:]
    ffk.cast_forward(xd, out)
    assert np.array_equal(to_np(out), bf16_round(x[1:]))
    acc = to_dev(x, torch)[1:].clone()
    accv = torch.zeros(n + 1, device="cuda")[1:]
    accv.copy_(acc)
    ffk.cast_backward(out, accv)
    assert np.array_equal(to_np(accv), bf16_round(x[1:]) + x[1:])
    B, C = 7, 111
    logit = g.random(B * C + 1).astype(np.float32)
    lab = g.random(B * C).astype(np.float32)
    label = g.integers(0, C, size=B).astype(np.int32)
    ld = to_dev(logit, torch)[1:]
    want = oracle.sparse_cce_loss_backward(logit[1:].reshape(B, C), label, B, C, 1, 0.25)
    got = ffk.sparse_categorical_crossentropy_loss_backward(ld, to_dev(label, torch, torch.int32), B, C, 1, 0.25)
    assert np.array_equal(to_np(got).reshape(B, C), want)
    want = oracle.difference_loss_backward(logit[1:], lab, 0.25)
    got = ffk.difference_loss_backward("categorical_crossentropy", ld, to_dev(lab, torch), 0.25)
    assert np.array_equal(to_np(got), want)
