"""Pins the oracle functions the reference's tests leave open, against what the
mathematics fixes: library routines in fp64 (torch on the CPU), invariants,
finite differences and brute force.  CPU only."""
import numpy as np
import pytest
import torch

from util import rng

F = torch.nn.functional
OP = dict(SCALAR_MULTIPLY=8, SCALAR_ADD=9, SCALAR_TRUE_DIV=11, SCALAR_SUB=12, RELU=13,
          IDENTITY=14, SIGMOID=15, TANH=16, ELU=17, EW_ADD=28, EW_MUL=29, EW_SUB=35,
          EW_DIV=36, EW_MAX=40, EW_MIN=41, EXP=56, SIN=61, COS=62, GELU=67, RSQRT=70,
          POW=71, GELU_REFERENCE_GRAD=1067)


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


def test_matmul_and_gemm_f64_brute_force(oracle):
    g = rng(1)
    A = g.standard_normal((7, 5)).astype(np.float32)
    B = g.standard_normal((5, 9)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.allclose(oracle.matmul(A, B), want, rtol=1e-6, atol=1e-6)
    assert np.allclose(oracle.gemm_f64(A, B), want, rtol=1e-7, atol=1e-7)
    assert np.allclose(oracle.gemm_f64(A.T.copy(), B, trans_a=True), want, rtol=1e-7, atol=1e-7)
    assert np.allclose(oracle.gemm_f64(A, B.T.copy(), trans_b=True), want, rtol=1e-7, atol=1e-7)
    # a transposed operand must not be mistaken for the plain one
    assert not np.allclose(oracle.gemm_f64(A[:5, :5], B[:5, :5].copy(), trans_b=True),
                           A[:5, :5].astype(np.float64) @ B[:5, :5].astype(np.float64))


def test_linear_relu_modes(oracle):
    g = rng(2)
    x = g.uniform(-1, 1, (6, 5)).astype(np.float32)
    w = g.standard_normal((4, 5)).astype(np.float32)
    b = g.standard_normal((4,)).astype(np.float32)
    dy = g.standard_normal((6, 4)).astype(np.float32)
    y = oracle.linear_forward(x, w, b, activation=0)
    pre = x.astype(np.float64) @ w.T.astype(np.float64) + b
    assert np.allclose(y, np.maximum(pre, 0), atol=1e-6)
    # mode 0 (GPU semantics) is the true gradient: compare with autograd
    xt, wt, bt = t64(x).requires_grad_(), t64(w).requires_grad_(), t64(b).requires_grad_()
    F.relu(F.linear(xt, wt, bt)).backward(t64(dy))
    dx, dw, db = oracle.linear_backward(y, dy, x, w, activation=0, relu_grad_mode=0)
    assert np.allclose(dx, xt.grad.numpy(), atol=1e-5)
    assert np.allclose(dw, wt.grad.numpy(), atol=1e-5)
    assert np.allclose(db, bt.grad.numpy(), atol=1e-5)
    # mode 1 (reference CPU text): the processed gradient is [dy > 0]
    gmask = (dy > 0).astype(np.float32)
    dx1, dw1, db1 = oracle.linear_backward(y, dy, x, w, activation=0, relu_grad_mode=1)
    assert np.allclose(dx1, gmask @ w, atol=1e-5)
    assert np.allclose(dw1, gmask.T @ x, atol=1e-5)
    assert np.allclose(db1, gmask.sum(0), atol=1e-5)
    with pytest.raises(ValueError):
        oracle.linear_forward(x, w, b, activation=3)  # the reference PANICs on GELU


def test_linear_l2_regularizer_grad_is_the_gradient_of_the_penalty(oracle):
    """dW' = dW + lambda W: lambda W is the gradient of lambda/2 |W|^2 (autograd), it is added
    to what the tensor holds (not stored over it, not scaled into it), and it uses W, not dW."""
    g = rng(12)
    w = g.standard_normal((4, 5)).astype(np.float32)
    dw = g.standard_normal((4, 5)).astype(np.float32)
    lam = 0.37
    wt = t64(w).requires_grad_()
    (0.5 * lam * (wt * wt).sum()).backward()
    got = oracle.linear_l2_regularizer_grad(w, dw, lam)
    assert np.allclose(got, dw + wt.grad.numpy(), atol=1e-6)
    assert np.allclose(oracle.linear_l2_regularizer_grad(w, np.zeros_like(w), lam), lam * w, atol=1e-7)
    assert np.array_equal(oracle.linear_l2_regularizer_grad(w, dw, 0.0), dw)
    # a full backward with a zero output gradient leaves exactly lambda W behind the GEMM
    x = g.standard_normal((6, 5)).astype(np.float32)
    _, dw0, _ = oracle.linear_backward(None, np.zeros((6, 4), np.float32), x, w)
    assert np.allclose(oracle.linear_l2_regularizer_grad(w, dw0, lam), lam * w, atol=1e-7)


@pytest.mark.parametrize("name,fn,scalar", [
    ("EXP", torch.exp, 0.0), ("IDENTITY", lambda v: v * 1.0, 0.0),
    ("GELU", lambda v: F.gelu(v), 0.0), ("RSQRT", torch.rsqrt, 0.0),
    ("SIN", torch.sin, 0.0), ("COS", torch.cos, 0.0), ("RELU", F.relu, 0.0),
    ("SIGMOID", torch.sigmoid, 0.0), ("TANH", torch.tanh, 0.0),
    ("ELU", lambda v: F.elu(v, alpha=0.7), 0.7),
    ("SCALAR_MULTIPLY", lambda v: v * 1.7, 1.7), ("SCALAR_ADD", lambda v: v + 1.7, 1.7),
    ("SCALAR_SUB", lambda v: v - 1.7, 1.7), ("SCALAR_TRUE_DIV", lambda v: v / 1.7, 1.7),
    ("POW", lambda v: v ** 1.7, 1.7),
])
def test_unary_against_autograd(oracle, name, fn, scalar):
    g = rng(3)
    x = g.uniform(0.2, 2.0, (64,)) if name in ("RSQRT", "POW") else g.uniform(-3, 3, (64,))
    x = x.astype(np.float32)
    dy = g.standard_normal((64,)).astype(np.float32)
    xt = t64(x).requires_grad_()
    yt = fn(xt)
    yt.backward(t64(dy))
    y = oracle.element_unary_forward(OP[name], x, scalar)
    assert np.allclose(y, yt.detach().numpy(), rtol=2e-6, atol=1e-6), name
    dx = oracle.element_unary_backward(OP[name], y, dy, x, scalar=scalar, accumulate=0)
    assert np.allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-5), name
    # reference accumulate rule: `=` for GELU/POW/RSQRT, `+=` otherwise
    init = g.standard_normal((64,)).astype(np.float32)
    dx2 = oracle.element_unary_backward(OP[name], y, dy, x, dx_init=init, scalar=scalar, accumulate=-1)
    base = 0.0 if name in ("GELU", "POW", "RSQRT") else init
    assert np.allclose(dx2, base + xt.grad.numpy(), rtol=1e-5, atol=1e-5), name


def test_gelu_reference_grad_is_the_literal_formula(oracle):
    x = np.linspace(-3, 3, 41).astype(np.float32)
    dy = np.ones_like(x)
    y = oracle.element_unary_forward(OP["GELU"], x)
    got = oracle.element_unary_backward(OP["GELU_REFERENCE_GRAD"], y, dy, x)
    xd = x.astype(np.float64)
    from math import erfc
    want = np.array([0.5 * erfc(-v * 2 ** -0.5) - 0.5 * 2 ** -0.5 * v * np.exp(-v * v / 2) for v in xd])
    assert np.allclose(got, want, atol=1e-6)
    true = oracle.element_unary_backward(OP["GELU"], y, dy, x)
    assert not np.allclose(got, true, atol=1e-3)  # the two formulas do differ


@pytest.mark.parametrize("name", ["EW_ADD", "EW_SUB", "EW_MUL"])
@pytest.mark.parametrize("shapes", [((6, 5, 8), (8,), (6, 5, 8)), ((7, 12), (7, 12), (12,)), ((4, 3, 10), (3, 10), (10,))])
def test_element_binary_broadcast_gradients_against_autograd(oracle, name, shapes):
    """A trailing-dims operand is what torch broadcasts too: its gradient is autograd's reduction."""
    out_shape, ls, rs = shapes
    g = np.random.default_rng(5)
    l64, r64 = g.standard_normal(ls), g.standard_normal(rs)
    dy = g.standard_normal(out_shape).astype(np.float32)
    fn = dict(EW_ADD=torch.add, EW_SUB=torch.sub, EW_MUL=torch.mul)[name]
    lt = torch.tensor(l64.astype(np.float32), dtype=torch.float64, requires_grad=True)
    rt = torch.tensor(r64.astype(np.float32), dtype=torch.float64, requires_grad=True)
    fn(lt.expand(out_shape), rt.expand(out_shape)).backward(torch.tensor(dy, dtype=torch.float64))
    dl, dr = oracle.element_binary_backward_broadcast(OP[name], dy, l64.astype(np.float32), r64.astype(np.float32))
    assert dl.shape == ls and dr.shape == rs
    assert np.allclose(dl, lt.grad.numpy(), rtol=1e-6, atol=1e-6)
    assert np.allclose(dr, rt.grad.numpy(), rtol=1e-6, atol=1e-6)
    # accumulate adds to what was there
    i1, i2 = g.standard_normal(ls).astype(np.float32), g.standard_normal(rs).astype(np.float32)
    dl2, dr2 = oracle.element_binary_backward_broadcast(OP[name], dy, l64.astype(np.float32), r64.astype(np.float32),
                                                        i1, i2, accumulate=1)
    assert np.allclose(dl2, lt.grad.numpy() + i1, rtol=1e-6, atol=1e-6)
    assert np.allclose(dr2, rt.grad.numpy() + i2, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("name", ["EW_ADD", "EW_SUB", "EW_MUL", "EW_DIV", "EW_MAX", "EW_MIN"])
def test_binary_against_autograd(oracle, name):
    g = rng(4)
    l = g.uniform(0.5, 2, (5, 8)).astype(np.float32)
    r = g.uniform(0.5, 2, (5, 8)).astype(np.float32)
    dy = g.standard_normal((5, 8)).astype(np.float32)
    fn = dict(EW_ADD=torch.add, EW_SUB=torch.sub, EW_MUL=torch.mul, EW_DIV=torch.div,
              EW_MAX=torch.maximum, EW_MIN=torch.minimum)[name]
    lt, rt = t64(l).requires_grad_(), t64(r).requires_grad_()
    out = fn(lt, rt)
    out.backward(t64(dy))
    assert np.allclose(oracle.element_binary_forward(OP[name], l, r), out.detach().numpy(), rtol=1e-6)
    dl, dr = oracle.element_binary_backward(OP[name], dy, l, r)
    assert np.allclose(dl, lt.grad.numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(dr, rt.grad.numpy(), rtol=1e-5, atol=1e-6)
    i1, i2 = g.standard_normal((5, 8)).astype(np.float32), g.standard_normal((5, 8)).astype(np.float32)
    dl2, dr2 = oracle.element_binary_backward(OP[name], dy, l, r, i1, i2, accumulate=1)
    assert np.allclose(dl2, i1 + lt.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(dr2, i2 + rt.grad.numpy(), rtol=1e-5, atol=1e-5)
    # bias-style broadcast of the rhs
    rb = r[0]
    assert np.allclose(oracle.element_binary_forward(OP[name], l, rb, l.shape),
                       fn(t64(l), t64(rb)).numpy(), rtol=1e-6)


def test_layer_norm_against_torch_and_invariants(oracle):
    g = rng(5)
    M, N = 9, 48
    x = (g.standard_normal((M, N)) * 2 + 0.5).astype(np.float32)
    gamma = g.standard_normal((N,)).astype(np.float32)
    beta = g.standard_normal((N,)).astype(np.float32)
    dy = g.standard_normal((M, N)).astype(np.float32)
    eps = 1e-5
    y, mean, rstd = oracle.layer_norm_forward(x, gamma, beta, eps)
    xt, gt, bt = t64(x).requires_grad_(), t64(gamma).requires_grad_(), t64(beta).requires_grad_()
    yt = F.layer_norm(xt, (N,), gt, bt, eps)
    yt.backward(t64(dy))
    assert np.allclose(y, yt.detach().numpy(), atol=1e-5)
    assert np.allclose(mean, x.astype(np.float64).mean(1), atol=1e-6)
    assert np.allclose(rstd, 1 / np.sqrt(x.astype(np.float64).var(1) + eps), rtol=1e-6)
    y1, _, _ = oracle.layer_norm_forward(x, None, None, eps)
    assert np.allclose(y1.mean(1), 0, atol=1e-5) and np.allclose(y1.var(1), 1, atol=1e-3)
    dx, dg, db = oracle.layer_norm_backward(dy, x, mean, rstd, gamma)
    assert np.allclose(dx, xt.grad.numpy(), atol=2e-5)
    assert np.allclose(dg, gt.grad.numpy(), atol=2e-5)
    assert np.allclose(db, bt.grad.numpy(), atol=2e-5)
    assert np.allclose(dx.sum(1), 0, atol=1e-4)            # sum_j dx = 0
    assert np.allclose((dx * y1).sum(1), 0, atol=1e-4)     # sum_j dx * xhat = 0
    init = g.standard_normal((M, N)).astype(np.float32)
    dx2, _, _ = oracle.layer_norm_backward(dy, x, mean, rstd, gamma, dx_init=init)
    assert np.allclose(dx2, init + xt.grad.numpy(), atol=3e-5)


@pytest.mark.parametrize("shape", [(6, 33, 1), (3, 7, 5)])
def test_softmax_against_torch(oracle, shape):
    g = rng(6)
    outer, dim, inner = shape
    x = (g.standard_normal(shape) * 4).astype(np.float32)
    dy = g.standard_normal(shape).astype(np.float32)
    y = oracle.softmax_forward(x, outer, dim, inner)
    xt = t64(x).requires_grad_()
    yt = torch.softmax(xt, dim=1)
    yt.backward(t64(dy))
    assert np.allclose(y, yt.detach().numpy(), atol=1e-6)
    assert np.allclose(y.sum(1), 1, atol=1e-5)
    assert np.allclose(oracle.softmax_forward(x + 3.0, outer, dim, inner), y, atol=1e-6)
    dx = oracle.softmax_backward(y, dy, outer, dim, inner)
    assert np.allclose(dx, xt.grad.numpy(), atol=1e-6)


def test_dropout_stream_properties(oracle):
    n, rate, seed = 200000, 0.1, 12345
    m = oracle.dropout_mask(n, rate, seed)
    keep = m.mean()
    sigma = np.sqrt(rate * (1 - rate) / n)
    assert abs(keep - (1 - rate)) < 5 * sigma
    # pure function of (seed, offset + i): a shifted window equals a slice
    assert np.array_equal(oracle.dropout_mask(1000, rate, seed, offset=37), m[37:1037])
    assert not np.array_equal(oracle.dropout_mask(n, rate, seed + 1), m)
    # element e uses 16 bits of block e / 8: half (e % 8) % 2 of word (e % 8) / 2, threshold ceil(rate * 2^16)
    thr = int(np.ceil(np.float32(rate).astype(np.float64) * 2 ** 16))
    for e in (0, 1, 2, 3, 4, 7, 8, 9, 1022, 1023):
        w = oracle.philox4x32_10([e // 8, 0, 0, 0], [seed & 0xffffffff, seed >> 32])
        word = int(w[(e % 8) // 2])
        half = (word >> 16) if e % 2 else (word & 0xffff)
        assert m[e] == (1 if half >= thr else 0)
    x = rng(7).standard_normal((n,)).astype(np.float32)
    y = oracle.dropout_forward(x, rate, seed)
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(rate))
    assert np.array_equal(y, np.where(m == 1, x * scale, np.float32(0)))
    assert np.array_equal(oracle.dropout_backward(x, rate, seed), y)
    assert oracle.dropout_mask(100, 0.0, seed).all() and not oracle.dropout_mask(100, 1.0, seed).any()


def test_embedding_against_torch(oracle):
    g = rng(8)
    V, D, B, bag = 50, 12, 17, 5
    w = g.standard_normal((V, D)).astype(np.float32)
    idx = g.integers(0, V, (B,))
    assert np.array_equal(oracle.embedding_forward(idx, w), w[idx])
    bags = g.integers(0, V, (B, bag))
    want_sum = F.embedding_bag(torch.from_numpy(bags), t64(w), mode="sum").numpy()
    want_avg = F.embedding_bag(torch.from_numpy(bags), t64(w), mode="mean").numpy()
    assert np.allclose(oracle.embedding_forward(bags, w, aggr=0), want_sum, atol=1e-5)
    assert np.allclose(oracle.embedding_forward(bags, w, aggr=1), want_avg, atol=1e-5)
    dy = g.standard_normal((B, D)).astype(np.float32)
    for aggr, mode in ((0, "sum"), (1, "mean")):
        wt = t64(w).requires_grad_()
        F.embedding_bag(torch.from_numpy(bags), wt, mode=mode).backward(t64(dy))
        assert np.allclose(oracle.embedding_backward(bags, dy, V, aggr=aggr), wt.grad.numpy(), atol=1e-5)
        assert np.allclose(oracle.embedding_backward(bags, dy, V, aggr=aggr, f64=True), wt.grad.numpy(), atol=1e-5)
    wt = t64(w).requires_grad_()
    F.embedding(torch.from_numpy(idx), wt).backward(t64(dy))
    assert np.allclose(oracle.embedding_backward(idx, dy, V), wt.grad.numpy(), atol=1e-5)
    with pytest.raises(ValueError):
        oracle.embedding_forward(np.array([V]), w)


@pytest.mark.parametrize("dt", [np.float16, np.float64])
def test_typed_embedding_against_torch_and_the_fp32_restatement(oracle, dt):
    """The HALF / DOUBLE restatements (numpy) against torch's embedding_bag in float64 and against
    the C fp32 restatement on data whose sums are exact in every type (eighths of small integers),
    where the three must agree to the bit; then what only arithmetic in the table's own type gives."""
    g = rng(81)
    V, D, B, bag = 40, 6, 13, 4
    w = (g.integers(-32, 33, (V, D)) / 8.0).astype(dt)
    bags = g.integers(0, V, (B, bag))
    dy = (g.integers(-16, 17, (B, D)) / 4.0).astype(dt)
    for aggr, mode in ((0, "sum"), (1, "mean")):  # bag = 4: the average is exact too
        want = F.embedding_bag(torch.from_numpy(bags), t64(w.astype(np.float64)), mode=mode).numpy()
        got = oracle.embedding_forward_typed(bags, w, aggr=aggr)
        assert got.dtype == dt and np.array_equal(got.astype(np.float64), want)
        assert np.array_equal(got.astype(np.float32), oracle.embedding_forward(bags, w.astype(np.float32), aggr=aggr))
        wt = t64(w.astype(np.float64)).requires_grad_()
        F.embedding_bag(torch.from_numpy(bags), wt, mode=mode).backward(t64(dy.astype(np.float64)))
        dw = oracle.embedding_backward_typed(bags, dy, V, aggr=aggr)
        assert dw.dtype == dt and np.array_equal(dw.astype(np.float64), wt.grad.numpy())
        assert np.array_equal(dw.astype(np.float32), oracle.embedding_backward(bags, dy.astype(np.float32), V, aggr=aggr))
    idx = g.integers(0, V, (B,))
    assert np.array_equal(oracle.embedding_forward_typed(idx, w), w[idx])
    # accumulation into what weight_grad held
    init = np.full((V, D), 0.5, dt)
    assert np.array_equal(oracle.embedding_backward_typed(idx, dy, V, dw_init=init),
                          oracle.embedding_backward_typed(idx, dy, V) + dt(0.5))
    with pytest.raises(ValueError):
        oracle.embedding_forward_typed(np.array([V]), w)
    if dt == np.float16:
        # a bag summed in half: 2048 + 1 is a tie that rounds back to 2048 each time; in fp32 it is 2050
        w2 = np.array([[2048.0], [1.0]], np.float16)
        assert oracle.embedding_forward_typed(np.array([[0, 1, 1]]), w2, aggr=0)[0, 0] == 2048.0
        assert oracle.embedding_forward(np.array([[0, 1, 1]]), w2.astype(np.float32), aggr=0)[0, 0] == 2050.0
        # AVG's factor is half(1/3) = 0.333251953125, not a division
        assert oracle.embedding_forward_typed(np.array([[0, 0, 0]]), np.array([[1.0]], np.float16), aggr=1)[0, 0] \
            == np.float16(np.float16(3.0) * np.float16(np.float32(1.0) / np.float32(3.0)))
    else:
        # double keeps what fp32 loses
        w2 = np.array([[2.0 ** 30], [2.0 ** -30]], np.float64)
        assert oracle.embedding_forward_typed(np.array([[0, 1]]), w2, aggr=0)[0, 0] == 2.0 ** 30 + 2.0 ** -30


@pytest.mark.parametrize("Dv", [8, 5, 12])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_against_torch_sdpa(oracle, causal, Dv):
    """Dv != D: the value head size (vProjSize) is independent of the query/key one."""
    g = rng(9)
    B, S, H, D = 2, 11, 3, 8
    q, k = (g.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(2))
    v, do = (g.standard_normal((B, S, H, Dv)).astype(np.float32) for _ in range(2))
    scale = 0.31
    o, lse = oracle.attention_forward(q, k, v, scale, causal)
    qt, kt, vt = (t64(a).transpose(1, 2).requires_grad_() for a in (q, k, v))
    ot = F.scaled_dot_product_attention(qt, kt, vt, is_causal=causal, scale=scale)
    ot.backward(t64(do).transpose(1, 2))
    assert np.allclose(o, ot.detach().transpose(1, 2).numpy(), atol=1e-5)
    s = torch.einsum("bhqd,bhkd->bhqk", qt, kt).detach() * scale
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    assert np.allclose(lse, torch.logsumexp(s, -1).numpy(), atol=1e-5)
    dq, dk, dv = oracle.attention_backward(q, k, v, do, scale, causal)
    assert np.allclose(dq, qt.grad.transpose(1, 2).numpy(), atol=1e-5)
    assert np.allclose(dk, kt.grad.transpose(1, 2).numpy(), atol=1e-5)
    assert np.allclose(dv, vt.grad.transpose(1, 2).numpy(), atol=1e-5)
    if causal:  # out[t] must not depend on inputs after t
        k2, v2 = k.copy(), v.copy()
        k2[:, 6:] += 1.0
        v2[:, 6:] -= 2.0
        o2, _ = oracle.attention_forward(q, k2, v2, scale, True)
        assert np.array_equal(o2[:, :6], o[:, :6])


@pytest.mark.parametrize("causal", [False, True])
def test_attention_bf16_mode_against_torch_with_rounded_probabilities(oracle, causal):
    """bf16_mode is the mode every bf16 device test compares with: the unnormalised
    probabilities exp(s - max) are rounded to bf16 before the PV product, the row sum is taken
    over the unrounded ones, and the output is rounded to bf16.  The same composition, step by
    step, in torch fp64."""
    g = rng(19)
    B, Sq, Skv, H, D = 2, 9, 13, 2, 8
    def bf(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    q, k, v = (bf(g.standard_normal(s)) for s in ((B, Sq, H, D), (B, Skv, H, D), (B, Skv, H, D)))
    scale = 0.4
    o, lse = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=True)
    qt, kt, vt = (t64(a).transpose(1, 2) for a in (q, k, v))
    s = torch.einsum("bhqd,bhkd->bhqk", qt, kt) * scale
    if causal:  # key j visible to query i iff j <= i
        s = s.masked_fill(torch.triu(torch.ones(Sq, Skv, dtype=torch.bool), 1), float("-inf"))
    p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
    p_rounded = p.to(torch.float32).to(torch.bfloat16).to(torch.float64)
    want = torch.einsum("bhqk,bhkd->bhqd", p_rounded, vt) / p.sum(dim=-1, keepdim=True)
    want = want.to(torch.float32).to(torch.bfloat16).to(torch.float32).transpose(1, 2).numpy()
    # the same bits, except where an fp64 value sits within an fp32 rounding of a bf16 tie
    diff = np.abs(o - want)
    assert (diff > 0).mean() < 0.01 and diff.max() <= np.abs(want).max() * 2.0 ** -7
    assert np.allclose(lse, torch.logsumexp(s, -1).numpy(), atol=1e-5)
    # and it is not the unrounded mode
    o32, _ = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=False)
    assert not np.array_equal(o, o32)


@pytest.mark.parametrize("Dv", [4, 6])
def test_mha_against_torch_composition(oracle, Dv):
    g = rng(10)
    B, Sq, Skv, H, E, Dh = 2, 6, 7, 3, 10, 4
    desc = oracle.mha_desc(B, H, E, E + 1, E + 2, Dh, Dh, Dv, E, Sq, Skv, scale=0.5, causal=False)
    q = g.standard_normal((B, Sq, E)).astype(np.float32)
    k = g.standard_normal((B, Skv, E + 1)).astype(np.float32)
    v = g.standard_normal((B, Skv, E + 2)).astype(np.float32)
    nq, nk, nv, no = H * Dh * E, H * Dh * (E + 1), H * Dv * (E + 2), E * H * Dv
    w = (g.standard_normal((nq + nk + nv + no,)) * 0.3).astype(np.float32)
    dout = g.standard_normal((B, Sq, E)).astype(np.float32)
    out = oracle.mha_forward(desc, q, k, v, w)
    qt, kt, vt, wt = (t64(a).requires_grad_() for a in (q, k, v, w))
    wq = wt[:nq].view(H * Dh, E)
    wk = wt[nq:nq + nk].view(H * Dh, E + 1)
    wv = wt[nq + nk:nq + nk + nv].view(H * Dv, E + 2)
    wo = wt[nq + nk + nv:].view(E, H * Dv)
    Q = (qt @ wq.T).view(B, Sq, H, Dh).transpose(1, 2)
    K = (kt @ wk.T).view(B, Skv, H, Dh).transpose(1, 2)
    Vv = (vt @ wv.T).view(B, Skv, H, Dv).transpose(1, 2)
    ctx = F.scaled_dot_product_attention(Q, K, Vv, scale=0.5).transpose(1, 2).reshape(B, Sq, H * Dv)
    ot = ctx @ wo.T
    ot.backward(t64(dout))
    assert np.allclose(out, ot.detach().numpy(), atol=1e-5)
    dq, dk, dv, dw = oracle.mha_backward(desc, q, k, v, w, dout)
    assert np.allclose(dq, qt.grad.numpy(), atol=2e-5)
    assert np.allclose(dk, kt.grad.numpy(), atol=2e-5)
    assert np.allclose(dv, vt.grad.numpy(), atol=2e-5)
    assert np.allclose(dw, wt.grad.numpy(), atol=5e-5)


def test_thread_count_does_not_change_a_bit(oracle):
    """The oracle's parallel loops (matrix products by row, attention by (batch, head)) give
    every output element to one thread in the serial order."""
    g = rng(33)
    A = g.standard_normal((130, 90)).astype(np.float32)
    Bm = g.standard_normal((90, 110)).astype(np.float32)
    B, S, H, D = 2, 70, 4, 8
    q, k, v, do = (g.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(4))
    before = oracle.max_threads()
    try:
        oracle.set_num_threads(1)
        one = [oracle.matmul(A, Bm), oracle.gemm_f64(A, Bm), *oracle.attention_forward(q, k, v, 0.3, True),
               *oracle.attention_backward(q, k, v, do, 0.3, True)]
        oracle.set_num_threads(4)
        four = [oracle.matmul(A, Bm), oracle.gemm_f64(A, Bm), *oracle.attention_forward(q, k, v, 0.3, True),
                *oracle.attention_backward(q, k, v, do, 0.3, True)]
    finally:
        oracle.set_num_threads(before)
    for a, b in zip(one, four):
        assert np.array_equal(a, b)


def test_round_bf16_matches_torch(oracle):
    x = np.concatenate([rng(11).standard_normal(1000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, 1e-40], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.round_bf16(x), want)
