"""ElementUnary / ElementBinary / Dropout parity against the oracle."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu

UNARY = ["SCALAR_MULTIPLY", "SCALAR_ADD", "SCALAR_SUB", "SCALAR_TRUE_DIV", "POW", "EXP", "IDENTITY",
         "GELU", "RSQRT", "SIN", "COS", "RELU", "SIGMOID", "TANH", "ELU"]
BINARY = ["EW_ADD", "EW_SUB", "EW_MUL", "EW_DIV", "EW_MAX", "EW_MIN"]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _unary_input(name, n, seed):
    g = rng(seed)
    if name in ("RSQRT", "POW"):
        return g.uniform(0.2, 2.0, (n,)).astype(np.float32)
    return g.uniform(-3, 3, (n,)).astype(np.float32)


@pytest.mark.parametrize("name", UNARY + ["GELU_REFERENCE_GRAD"])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("n", [1, 1000, 4096 * 33 + 5])
def test_unary(ffk, oracle, name, dtype, n):
    say("unary", name, dtype, n)
    op = ffk.OP[name]
    scalar = 1.7
    x = _unary_input(name, n, 31)
    dy = rng(32).standard_normal((n,)).astype(np.float32)
    dx0 = rng(33).standard_normal((n,)).astype(np.float32)
    tdt, rtol = (torch.float32, 2e-5) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        x, dy, dx0 = bf16_round(x), bf16_round(dy), bf16_round(dx0)
    y_ref = oracle.element_unary_forward(op, x, scalar)
    xd = to_dev(x, torch, tdt)
    y = ffk.element_unary_forward(op, xd, scalar)
    assert_close(to_np(y), y_ref, rtol, "y")
    for acc in (-1, 0, 1):
        dx = to_dev(dx0, torch, tdt)
        ffk.element_unary_backward(op, y, to_dev(dy, torch, tdt), xd, dx, scalar, accumulate=acc)
        want = oracle.element_unary_backward(op, to_np(y), dy, x, dx_init=dx0, scalar=scalar, accumulate=acc)
        assert_close(to_np(dx), want, rtol, "dx acc=%d" % acc)


def test_unary_unaligned_pointer_and_empty(ffk, oracle):
    say("unary unaligned/empty")
    base = torch.zeros(1030, device="cuda")
    x = rng(1).standard_normal(1025).astype(np.float32)
    base[3:1028] = torch.from_numpy(x).cuda()
    view = base[3:1028]
    out = torch.zeros(1031, device="cuda")[5:1030]
    ffk.check(ffk.lib().ffk_element_unary_forward(ffk.current_stream(), ffk.FLOAT, ffk.OP["EXP"], 0.0,
                                                  view.data_ptr(), out.data_ptr(), 1025))
    assert_close(to_np(out), oracle.element_unary_forward(ffk.OP["EXP"], x), 2e-5, "exp unaligned")
    ffk.check(ffk.lib().ffk_element_unary_forward(ffk.current_stream(), ffk.FLOAT, ffk.OP["EXP"], 0.0,
                                                  None, None, 0))
    with pytest.raises(ffk.FFKError):
        ffk.element_unary_forward(4242, base)


@pytest.mark.parametrize("name", BINARY)
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(1,), (37, 19), (257, 1024)])
def test_binary(ffk, oracle, name, dtype, shape):
    say("binary", name, dtype, shape)
    op = ffk.OP[name]
    g = rng(41)
    l = g.uniform(0.5, 2, shape).astype(np.float32)
    r = g.uniform(0.5, 2, shape).astype(np.float32)
    dy = g.standard_normal(shape).astype(np.float32)
    i1 = g.standard_normal(shape).astype(np.float32)
    i2 = g.standard_normal(shape).astype(np.float32)
    tdt, rtol = (torch.float32, FP32_RTOL) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        l, r, dy, i1, i2 = (bf16_round(a) for a in (l, r, dy, i1, i2))
    ld, rd, dyd = (to_dev(a, torch, tdt) for a in (l, r, dy))
    out = ffk.element_binary_forward(op, ld, rd)
    assert_close(to_np(out), oracle.element_binary_forward(op, l, r), rtol, "out")
    for acc in (0, 1):
        dl, dr = to_dev(i1, torch, tdt), to_dev(i2, torch, tdt)
        ffk.element_binary_backward(op, dyd, ld, rd, dl, dr, accumulate=bool(acc))
        wl, wr = oracle.element_binary_backward(op, dy, l, r, i1, i2, accumulate=acc)
        assert_close(to_np(dl), wl, rtol, "dl acc=%d" % acc)
        assert_close(to_np(dr), wr, rtol, "dr acc=%d" % acc)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_binary_broadcast_rhs(ffk, oracle, dtype):
    say("binary broadcast", dtype)
    g = rng(43)
    l = g.standard_normal((65, 48)).astype(np.float32)
    r = g.standard_normal((48,)).astype(np.float32)
    tdt, rtol = (torch.float32, FP32_RTOL) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        l, r = bf16_round(l), bf16_round(r)
    out = ffk.element_binary_forward(ffk.OP["EW_ADD"], to_dev(l, torch, tdt), to_dev(r, torch, tdt))
    assert_close(to_np(out), oracle.element_binary_forward(ffk.OP["EW_ADD"], l, r, l.shape), rtol, "bcast")
    r5 = r[:7].copy()  # 65 * 48 is not a multiple of 7: not broadcastable
    with pytest.raises(ffk.FFKError, match="broadcast"):
        ffk.element_binary_forward(ffk.OP["EW_ADD"], to_dev(l, torch, tdt), to_dev(r5, torch, tdt),
                                   out=torch.empty((65, 48), dtype=tdt, device="cuda"))


@pytest.mark.parametrize("name", ["EW_ADD", "EW_SUB", "EW_MUL"])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shapes", [((65, 48), (65, 48), (48,)), ((300, 7, 130), (130,), (300, 7, 130)),
                                    ((1000, 70), (70,), (70,)), ((5, 3, 64), (3, 64), (64,))])
def test_binary_broadcast_gradients(ffk, oracle, name, dtype, shapes):
    """The reference's broadcast_inputLHS / broadcast_inputRHS branches: a smaller operand's
    gradient is the sum over the output elements it was broadcast to."""
    out_shape, ls, rs = shapes
    say("binary broadcast gradients", name, dtype, shapes)
    op = ffk.OP[name]
    g = rng(47)
    l = g.uniform(0.5, 2, ls).astype(np.float32)
    r = g.uniform(0.5, 2, rs).astype(np.float32)
    dy = g.standard_normal(out_shape).astype(np.float32)
    i1 = g.standard_normal(ls).astype(np.float32)
    i2 = g.standard_normal(rs).astype(np.float32)
    tdt, rtol = (torch.float32, FP32_RTOL) if dtype == "fp32" else (torch.bfloat16, BF16_RTOL)
    if dtype == "bf16":
        l, r, dy, i1, i2 = (bf16_round(a) for a in (l, r, dy, i1, i2))
    ld, rd, dyd = (to_dev(a, torch, tdt) for a in (l, r, dy))
    for acc in (0, 1):
        dl, dr = to_dev(i1, torch, tdt), to_dev(i2, torch, tdt)
        ffk.element_binary_backward_broadcast(op, dyd, ld, rd, dl, dr, accumulate=bool(acc))
        wl, wr = oracle.element_binary_backward_broadcast(op, dy, l, r, i1, i2, accumulate=acc)
        assert_close(to_np(dl), wl, rtol, "dl acc=%d" % acc)
        assert_close(to_np(dr), wr, rtol, "dr acc=%d" % acc)
    # one gradient only, as the reference allows
    dr = to_dev(i2, torch, tdt)
    ffk.element_binary_backward_broadcast(op, dyd, ld, rd, None, dr, accumulate=False)
    assert_close(to_np(dr), oracle.element_binary_backward_broadcast(op, dy, l, r)[1], rtol, "dr alone")
    # twice the same call: the same bits (fixed summation order)
    dr2 = to_dev(i2, torch, tdt)
    ffk.element_binary_backward_broadcast(op, dyd, ld, rd, None, dr2, accumulate=False)
    assert torch.equal(dr, dr2)


def test_binary_broadcast_gradients_refusals(ffk):
    x = torch.ones((8, 4), device="cuda")
    b = torch.ones((4,), device="cuda")
    with pytest.raises(ffk.FFKError, match="no broadcast gradient"):
        ffk.element_binary_backward_broadcast(ffk.OP["EW_MAX"], x, x, b, torch.empty_like(x), torch.empty_like(b))
    with pytest.raises(ffk.FFKError, match="broadcast"):
        ffk.element_binary_backward_broadcast(ffk.OP["EW_ADD"], x, x, torch.ones((3,), device="cuda"),
                                              torch.empty_like(x), torch.empty((3,), device="cuda"))


@pytest.mark.parametrize("n,offset", [(1, 0), (4099, 0), (65536 + 3, 8), (5000, 3), (70001, 1 << 33)])
@pytest.mark.parametrize("rate", [0.1, 0.5, 0.0, 1.0])
def test_dropout_mask_bit_exact(ffk, oracle, n, offset, rate):
    say("dropout mask", n, offset, rate)
    seed = 0x123456789ABCDEF
    m = ffk.dropout_mask(n, rate, seed, offset)
    assert np.array_equal(m.cpu().numpy(), oracle.dropout_mask(n, rate, seed, offset))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("n,offset", [(4096 * 9, 0), (12345, 0), (12345, 5), (3, 2)])
def test_dropout_forward_backward(ffk, oracle, dtype, n, offset):
    say("dropout", dtype, n, offset)
    rate, seed = 0.1, 12345
    x = rng(51).standard_normal((n,)).astype(np.float32)
    dx0 = rng(52).standard_normal((n,)).astype(np.float32)
    tdt = torch.float32 if dtype == "fp32" else torch.bfloat16
    if dtype == "bf16":
        x, dx0 = bf16_round(x), bf16_round(dx0)
    xd = to_dev(x, torch, tdt)
    y = ffk.dropout_forward(xd, rate, seed, offset)
    want = oracle.dropout_forward(x, rate, seed, offset)
    if dtype == "bf16":
        want = bf16_round(want)
    # mask bit-exact => zeros in exactly the same places; kept values equal
    assert np.array_equal(to_np(y) == 0, want == 0) or np.array_equal(to_np(y), want)
    assert np.array_equal(to_np(y), want)
    dx = ffk.dropout_backward(xd, rate, seed, offset)
    assert np.array_equal(to_np(dx), want)
    dxa = to_dev(dx0, torch, tdt)
    ffk.dropout_backward(xd, rate, seed, offset, dx=dxa, accumulate=True)
    wa = oracle.dropout_backward(x, rate, seed, offset, dx_init=dx0)
    if dtype == "bf16":
        wa = bf16_round(wa)
    assert np.array_equal(to_np(dxa), wa)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_dropout_fused_with_neighbour_equals_separate_operators(ffk, dtype):
    """The three fused dropout entries against the separate entries run one after the other
    (bit for bit), and their refusal of operands the vector kernels cannot take."""
    say("dropout fused pairs", dtype)
    n, rate, seed, offset = 4096 * 24, 0.1, 777, 16
    tdt = torch.float32 if dtype == "fp32" else torch.bfloat16
    g = rng(61)
    x = to_dev(g.standard_normal((n,)).astype(np.float32), torch, tdt)
    r = to_dev(g.standard_normal((n,)).astype(np.float32), torch, tdt)
    dy = to_dev(g.standard_normal((n,)).astype(np.float32), torch, tdt)
    gelu = ffk.OP["GELU"]
    want = ffk.element_binary_forward(ffk.OP["EW_ADD"], ffk.dropout_forward(x, rate, seed, offset), r)
    assert torch.equal(ffk.dropout_add_forward(x, r, rate, seed, offset), want)
    want = ffk.dropout_forward(ffk.element_unary_forward(gelu, x), rate, seed, offset)
    assert torch.equal(ffk.gelu_dropout_forward(x, rate, seed, offset), want)
    act = ffk.element_unary_forward(gelu, x)
    want = ffk.element_unary_backward(gelu, act, ffk.dropout_backward(dy, rate, seed, offset), x, torch.empty_like(x),
                                      accumulate=0)
    assert torch.equal(ffk.dropout_gelu_backward(dy, x, rate, seed, offset), want)
    with pytest.raises(ffk.FFKError, match="fusable"):
        ffk.gelu_dropout_forward(x[: n - 1], rate, seed, offset)
    with pytest.raises(ffk.FFKError, match="fusable"):
        ffk.dropout_add_forward(x, r, rate, seed, offset + 3)


def test_dropout_full_size_statistics(ffk):
    """BASELINE config 3 size [16384, 4096] bf16, p = 0.1: keep rate within
    5 sigma, kept values scaled by 1/(1-p), backward mask == forward mask."""
    say("dropout cfg3 full size")
    n = 16384 * 4096
    x = torch.ones((n,), dtype=torch.bfloat16, device="cuda")
    y = ffk.dropout_forward(x, 0.1, 12345)
    kept = (y != 0)
    rate = kept.float().mean().item()
    sigma = (0.1 * 0.9 / n) ** 0.5
    assert abs(rate - 0.9) < 5 * sigma + 1e-7
    vals = y[kept]
    assert torch.all(vals == vals[0]) and abs(vals[0].item() - 1 / 0.9) < 1e-2
    dx = ffk.dropout_backward(x, 0.1, 12345)
    assert torch.equal(dx, y)
    m = ffk.dropout_mask(n, 0.1, 12345)
    assert torch.equal(m.bool(), kept)
