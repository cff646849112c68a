"""Fused attention core and MultiHeadAttention parity against the oracle."""
import sys

import numpy as np
import pytest
import torch

from util import BF16_RTOL, FP32_RTOL, assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu
BT = torch.bfloat16


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


SHAPES = [  # B, H, Sq, Skv, D (, Dv)
    (1, 1, 8, 8, 64), (2, 3, 11, 11, 64), (1, 2, 100, 100, 128), (2, 2, 129, 129, 64),
    (1, 4, 256, 256, 128), (1, 2, 300, 300, 64), (1, 1, 64, 200, 64), (2, 1, 160, 96, 128),
    # the head size of the reference's transformer and BERT builders (transformer.cc:37-38, bert.cc:64-65)
    (1, 2, 70, 70, 256), (2, 2, 129, 200, 256), (1, 1, 300, 300, 256),
    # a value head size of its own (vdim != kdim), and head sizes that are no power of two
    (1, 2, 100, 100, 64, 128), (2, 1, 129, 96, 128, 64), (1, 2, 40, 72, 256, 64), (1, 1, 65, 65, 64, 256),
    (1, 2, 50, 50, 32), (1, 2, 90, 130, 96), (1, 3, 33, 33, 40, 72), (1, 1, 140, 140, 200, 8),
]


def _dv(shape):
    return shape[5] if len(shape) > 5 else shape[4]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_core(ffk, oracle, shape, causal):
    # causal with Sq != Skv: key j is visible to query i iff j <= i (the mask is aligned top-left)
    B, H, Sq, Skv, D = shape[:5]
    Dv = _dv(shape)
    say("attention core", shape, "causal", causal)
    g = rng(Sq * 7 + D + int(causal))
    q = bf16_round(g.standard_normal((B, Sq, H, D)))
    k = bf16_round(g.standard_normal((B, Skv, H, D)))
    v = bf16_round(g.standard_normal((B, Skv, H, Dv)))
    do = bf16_round(g.standard_normal((B, Sq, H, Dv)))
    scale = 1.0 / np.sqrt(D)
    o_ref, lse_ref = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=True)
    qd, kd, vd, dod = (to_dev(a, torch, BT) for a in (q, k, v, do))
    o, lse = ffk.attention_forward(qd, kd, vd, scale, causal)
    assert_close(to_np(o), o_ref, BF16_RTOL, "O")
    assert_close(to_np(lse), lse_ref, 1e-3, "lse")
    dq_ref, dk_ref, dv_ref = oracle.attention_backward(q, k, v, do, scale, causal)
    dq, dk, dv = ffk.attention_backward(qd, kd, vd, o, dod, lse, scale, causal)
    assert_close(to_np(dq), dq_ref, BF16_RTOL, "dQ")
    assert_close(to_np(dk), dk_ref, BF16_RTOL, "dK")
    assert_close(to_np(dv), dv_ref, BF16_RTOL, "dV")


# Forward kernel: 256 query rows per workgroup, 64 per wavefront in two halves, 64 keys per tile.
# Shapes around those sizes (blocks that end inside a half, a last key tile of 1 and of 63, more
# keys than queries and the reverse), under both masks.
FWD_SHAPES = [(1, 2, 600, 600, 128), (1, 1, 257, 705, 64), (1, 1, 513, 513, 128), (2, 1, 33, 449, 128), (1, 2, 320, 65, 64)]


@pytest.mark.parametrize("variant", [2, 1])
@pytest.mark.parametrize("shape", FWD_SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_forward_kernels(ffk, oracle, shape, causal, variant):
    """Both forward kernels at every shape (option 2: 64 query rows per wavefront, option 1: 32;
    the default picks by size)."""
    B, H, Sq, Skv, D = shape
    say("attention forward", shape, "causal", causal, "variant", variant)
    g = rng(Sq * 3 + Skv + D + int(causal))
    q = bf16_round(g.standard_normal((B, Sq, H, D)))
    k = bf16_round(g.standard_normal((B, Skv, H, D)))
    v = bf16_round(g.standard_normal((B, Skv, H, D)))
    scale = 1.0 / np.sqrt(D)
    o_ref, lse_ref = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=True)
    ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, variant)
    try:
        o, lse = ffk.attention_forward(*(to_dev(a, torch, BT) for a in (q, k, v)), scale, causal)
    finally:
        ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 0)
    assert_close(to_np(o), o_ref, BF16_RTOL, "O")
    assert_close(to_np(lse), lse_ref, 1e-3, "lse")


@pytest.mark.parametrize("shape", FWD_SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_backward_kernels(ffk, oracle, shape, causal):
    """The tuned backward kernels (dQ; dK/dV streaming 64-row query tiles as two pipelined halves)
    against the oracle; nothing in them is atomic, so a second run gives the same bits."""
    B, H, Sq, Skv, D = shape
    say("attention backward", shape, "causal", causal)
    g = rng(Sq * 5 + Skv + D + int(causal))
    q = bf16_round(g.standard_normal((B, Sq, H, D)))
    k = bf16_round(g.standard_normal((B, Skv, H, D)))
    v = bf16_round(g.standard_normal((B, Skv, H, D)))
    do = bf16_round(g.standard_normal((B, Sq, H, D)))
    scale = 1.0 / np.sqrt(D)
    qd, kd, vd, dod = (to_dev(a, torch, BT) for a in (q, k, v, do))
    o, lse = ffk.attention_forward(qd, kd, vd, scale, causal)
    grads = ffk.attention_backward(qd, kd, vd, o, dod, lse, scale, causal)
    again = ffk.attention_backward(qd, kd, vd, o, dod, lse, scale, causal)
    dq_ref, dk_ref, dv_ref = oracle.attention_backward(q, k, v, do, scale, causal)
    for name, got, want in zip(("dQ", "dK", "dV"), grads, (dq_ref, dk_ref, dv_ref)):
        assert_close(to_np(got), want, BF16_RTOL, name)
    for name, a, b in zip(("dQ", "dK", "dV"), grads, again):
        assert torch.equal(a, b), name


@pytest.mark.parametrize("causal", [False, True])
def test_attention_forward_growing_scores(ffk, oracle, causal):
    """Keys grow along the sequence, so every tile raises the row maxima: by less than the
    kernel's threshold for moving its reference point in the first half of the sequence
    (probabilities above 1 are then summed), by more in the second."""
    B, H, S, D = 1, 2, 1024, 128
    say("attention growing scores, causal", causal)
    g = rng(77 + int(causal))
    q = bf16_round(np.abs(g.standard_normal((B, S, H, D))) * 0.5)
    ramp = np.where(np.arange(S) < S // 2, 1.0 + np.arange(S) / S, 1.5 + 12.0 * (np.arange(S) - S // 2) / S)
    k = bf16_round(np.abs(g.standard_normal((B, S, H, D))) * ramp[None, :, None, None] * 0.25)
    v = bf16_round(g.standard_normal((B, S, H, D)))
    scale = 1.0 / np.sqrt(D)
    o_ref, lse_ref = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=True)
    ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 2)  # the kernel with the lazily moved reference point
    try:
        o, lse = ffk.attention_forward(*(to_dev(a, torch, BT) for a in (q, k, v)), scale, causal)
    finally:
        ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 0)
    assert_close(to_np(o), o_ref, BF16_RTOL, "O")
    assert_close(to_np(lse), lse_ref, 1e-3, "lse")


F32_SHAPES = [  # B, H, Sq, Skv, D (, Dv)
    (1, 1, 8, 8, 64), (2, 3, 11, 11, 32), (1, 2, 100, 100, 128), (2, 2, 129, 129, 64), (1, 2, 40, 40, 4),
    (1, 4, 256, 256, 128), (1, 2, 300, 300, 48), (1, 1, 64, 200, 64), (2, 1, 160, 96, 100), (1, 3, 70, 33, 20),
    (1, 2, 70, 70, 256), (2, 2, 129, 200, 256), (1, 1, 200, 140, 132),
    (1, 2, 100, 100, 64, 128), (2, 1, 129, 96, 128, 36), (1, 2, 40, 72, 256, 64), (1, 1, 65, 65, 16, 256),
]


@pytest.mark.parametrize("shape", F32_SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_core_fp32(ffk, oracle, shape, causal):
    """The fp32 core behind the reference's float MultiHeadAttention signature."""
    B, H, Sq, Skv, D = shape[:5]
    Dv = _dv(shape)
    say("attention core fp32", shape, "causal", causal)
    g = rng(Sq * 5 + D + int(causal))
    q, k, v, do = (g.standard_normal(s).astype(np.float32)
                   for s in ((B, Sq, H, D), (B, Skv, H, D), (B, Skv, H, Dv), (B, Sq, H, Dv)))
    scale = 1.0 / np.sqrt(D)
    o_ref, lse_ref = oracle.attention_forward(q, k, v, scale, causal, bf16_mode=False)
    qd, kd, vd, dod = (to_dev(a, torch) for a in (q, k, v, do))
    o, lse = ffk.attention_forward(qd, kd, vd, scale, causal)
    assert_close(to_np(o), o_ref, FP32_RTOL, "O")
    assert_close(to_np(lse), lse_ref, FP32_RTOL, "lse")
    dq_ref, dk_ref, dv_ref = oracle.attention_backward(q, k, v, do, scale, causal)
    dq, dk, dv = ffk.attention_backward(qd, kd, vd, o, dod, lse, scale, causal)
    assert_close(to_np(dq), dq_ref, FP32_RTOL, "dQ")
    assert_close(to_np(dk), dk_ref, FP32_RTOL, "dK")
    assert_close(to_np(dv), dv_ref, FP32_RTOL, "dV")


def test_attention_reference_scale_one(ffk, oracle):
    """The reference configures cuDNN with smScalar = 1.0 (attention_kernels.cu:76)."""
    say("attention scale 1.0")
    g = rng(3)
    B, H, S, D = 1, 2, 40, 64
    q = bf16_round(g.standard_normal((B, S, H, D)) * 0.3)
    k = bf16_round(g.standard_normal((B, S, H, D)) * 0.3)
    v = bf16_round(g.standard_normal((B, S, H, D)))
    o_ref, _ = oracle.attention_forward(q, k, v, 1.0, False, bf16_mode=True)
    o, _ = ffk.attention_forward(*(to_dev(a, torch, BT) for a in (q, k, v)), 1.0, False)
    assert_close(to_np(o), o_ref, BF16_RTOL, "O")


def test_attention_strided_views(ffk, oracle):
    """q/k/v interleaved in one [B, S, 3*H*D] buffer, addressed through strides."""
    say("attention strided")
    g = rng(4)
    B, H, S, D = 2, 2, 70, 64
    qkv = bf16_round(g.standard_normal((B, S, 3, H, D)))
    do = bf16_round(g.standard_normal((B, S, H, D)))
    q, k, v = (np.ascontiguousarray(qkv[:, :, i]) for i in range(3))
    scale = 0.125
    o_ref, _ = oracle.attention_forward(q, k, v, scale, True, bf16_mode=True)
    dq_ref, dk_ref, dv_ref = oracle.attention_backward(q, k, v, do, scale, True)
    buf = to_dev(qkv, torch, BT)
    row = 3 * H * D
    desc = ffk.AttentionDesc(B, H, S, S, D, S * row, row, S * row, row, S * row, row, S * H * D, H * D,
                             scale, 1)
    es = 2
    o = torch.empty((B, S, H, D), dtype=BT, device="cuda")
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    base = buf.data_ptr()
    st = ffk.current_stream()
    ffk.check(ffk.lib().ffk_attention_forward(st, ffk.BF16, desc, base, base + H * D * es, base + 2 * H * D * es,
                                              o.data_ptr(), lse.data_ptr()))
    assert_close(to_np(o), o_ref, BF16_RTOL, "O")
    dbuf = torch.zeros_like(buf)
    delta = torch.empty_like(lse)
    dod = to_dev(do, torch, BT)
    db = dbuf.data_ptr()
    ffk.check(ffk.lib().ffk_attention_backward(st, ffk.BF16, desc, base, base + H * D * es, base + 2 * H * D * es,
                                               o.data_ptr(), dod.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                                               db, db + H * D * es, db + 2 * H * D * es))
    d = to_np(dbuf)
    assert_close(d[:, :, 0], dq_ref, BF16_RTOL, "dQ")
    assert_close(d[:, :, 1], dk_ref, BF16_RTOL, "dK")
    assert_close(d[:, :, 2], dv_ref, BF16_RTOL, "dV")


def test_attention_errors(ffk):
    q = torch.zeros((1, 8, 2, 264), dtype=BT, device="cuda")
    with pytest.raises(ffk.FFKError, match="head_dim"):
        ffk.attention_forward(q, q, q, 1.0, False)
    q = torch.zeros((1, 8, 2, 36), dtype=BT, device="cuda")  # strides of 72 are fine, the head size is no multiple of 8
    with pytest.raises(ffk.FFKError, match="head_dim"):
        ffk.attention_forward(q, q, q, 1.0, False)
    q32 = torch.zeros((1, 8, 1, 260), dtype=torch.float32, device="cuda")
    with pytest.raises(ffk.FFKError, match="head_dim"):
        ffk.attention_forward(q32, q32, q32, 1.0, False)
    q16 = torch.zeros((1, 8, 1, 64), dtype=torch.float16, device="cuda")
    desc = ffk.attention_desc_bshd(q16, q16, 1.0, False)
    rc = ffk.lib().ffk_attention_forward(0, ffk.HALF, desc, q16.data_ptr(), q16.data_ptr(), q16.data_ptr(),
                                         q16.data_ptr(), None)
    assert rc == 1 and b"dtype" in ffk.lib().ffk_last_error()


def test_attention_config5_causal_prefix(ffk, oracle):
    """BASELINE config 5 (B 4, S 4096, H 32, hd 128, causal) at full size.
    Causality makes the first P queries a function of the first P keys only,
    so the oracle on that prefix is the exact expectation for the full run;
    dK/dV of the LAST keys depend only on the last queries likewise."""
    B, H, S, D = 4, 32, 4096, 128
    say("attention cfg5 full size")
    gen = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, do = (torch.randn((B, S, H, D), device="cuda", generator=gen).to(BT) for _ in range(4))
    scale = 1.0 / np.sqrt(D)
    o, lse = ffk.attention_forward(q, k, v, scale, True)
    P = 192
    for (b, h) in ((0, 0), (3, 31)):
        qs, ks, vs = (to_np(t[b:b + 1, :P, h:h + 1]) for t in (q, k, v))
        o_ref, lse_ref = oracle.attention_forward(qs, ks, vs, scale, True, bf16_mode=True)
        assert_close(to_np(o[b:b + 1, :P, h:h + 1]), o_ref, BF16_RTOL, "O prefix")
        assert_close(to_np(lse[b, h, :P]), lse_ref[0, 0], 1e-3, "lse prefix")
    assert torch.isfinite(o.float()).all()
    dq, dk, dv = ffk.attention_backward(q, k, v, o, do, lse, scale, True)
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all()
    # dQ of the first P queries depends on the first P keys only
    b, h = 1, 7
    qs, ks, vs, dos = (to_np(t[b:b + 1, :P, h:h + 1]) for t in (q, k, v, do))
    dq_ref, _, _ = oracle.attention_backward(qs, ks, vs, dos, scale, True)
    assert_close(to_np(dq[b:b + 1, :P, h:h + 1]), dq_ref, BF16_RTOL, "dQ prefix")
    # dV/dK of the last T keys: only queries >= S-T see them, but those queries
    # attend to all keys; check with the oracle on the last-T queries x all keys
    T = 8
    qs = to_np(q[b:b + 1, S - T:, h:h + 1])
    dos = to_np(do[b:b + 1, S - T:, h:h + 1])
    ks, vs = to_np(k[b:b + 1, :, h:h + 1]), to_np(v[b:b + 1, :, h:h + 1])
    # causal mask for a suffix of queries = explicit per-row limits: emulate by
    # running non-causal on each row's visible keys
    dv_ref = np.zeros((T, D), np.float64)
    dk_ref = np.zeros((T, D), np.float64)
    for i in range(T):
        lim = S - T + i + 1
        _, dkr, dvr = oracle.attention_backward(qs[:, i:i + 1], ks[:, :lim], vs[:, :lim], dos[:, i:i + 1],
                                                scale, False)
        dk_ref[: i + 1] += dkr[0, S - T:lim, 0]
        dv_ref[: i + 1] += dvr[0, S - T:lim, 0]
    assert_close(to_np(dk[b, S - T:, h]), dk_ref, BF16_RTOL, "dK suffix")
    assert_close(to_np(dv[b, S - T:, h]), dv_ref, BF16_RTOL, "dV suffix")


def test_mha_config5_block_causal_prefix(ffk, oracle):
    """BASELINE config 5 as ONE MultiHeadAttention call: batch 4, seq 4096, embed 4096, 32 heads x
    128, causal, the four [16384,4096]x[4096,4096] projections around the core, forward and
    backward (the reference's cudnnMultiHeadAttnForward / BackwardData / BackwardWeights,
    attention_kernels.cu:215-303).  Under the causal mask the first P tokens of a sequence are a
    function of its first P tokens only, so the oracle on that prefix is the exact expectation for
    output[b, :P].  For the backward the upstream gradient is zero outside the prefix of sequence
    b0: every intermediate gradient is then zero outside that prefix (queries before P see only
    keys before P), so dquery[b0, :P] and the WHOLE weight gradient equal the oracle's on the
    prefix, and dquery is exactly zero everywhere else.  A second backward with a dense random
    upstream gradient must stay finite and, by linearity, contain the first one's weight gradient
    when the two upstream gradients are added."""
    B, S, H, Dh = 4, 4096, 32, 128
    E = H * Dh
    P, b0 = 96, 2
    say("mha cfg5 block, causal prefix", (B, S, E, H, Dh))
    scale = 1.0 / np.sqrt(Dh)
    gen = torch.Generator(device="cuda").manual_seed(55)
    x = torch.randn((B, S, E), device="cuda", generator=gen).to(BT)
    desc = ffk.mha_desc(B, H, E, E, E, Dh, Dh, Dh, E, S, S, scale, True)
    nw = ffk.lib().ffk_mha_weight_elements(desc)
    assert nw == 4 * E * E
    w = (torch.randn((nw,), device="cuda", generator=gen) * 0.02).to(BT)
    reserve = ffk.mha_reserve(desc, ffk.BF16)
    out = ffk.mha_forward(desc, x, x, x, w, reserve)
    assert torch.isfinite(out.float()).all()
    odesc = oracle.mha_desc(1, H, E, E, E, Dh, Dh, Dh, E, P, P, scale, True)
    wn = to_np(w)
    for b in (0, b0):
        xs = to_np(x[b:b + 1, :P])
        out_ref = oracle.mha_forward(odesc, xs, xs, xs, wn, bf16_mode=True)
        assert_close(to_np(out[b:b + 1, :P]), out_ref, BF16_RTOL, "output prefix, sequence %d" % b)
    # backward, upstream gradient confined to the prefix of sequence b0
    dout = torch.zeros((B, S, E), device="cuda", dtype=BT)
    dout[b0, :P] = torch.randn((P, E), device="cuda", generator=gen).to(BT)
    dx = torch.full_like(x, 3.0)
    dw = torch.full_like(w, 3.0)
    ffk.mha_backward(desc, x, dx, x, None, x, None, w, dw, dout, reserve,
                     accumulate=ffk.MHA_OVERWRITE_WEIGHT_GRAD)
    xs = to_np(x[b0:b0 + 1, :P])
    dq_ref, dk_ref, dv_ref, dw_ref = oracle.mha_backward(odesc, xs, xs, xs, wn, to_np(dout[b0:b0 + 1, :P]),
                                                         bf16_mode=True)
    assert_close(to_np(dx[b0:b0 + 1, :P]), dq_ref + dk_ref + dv_ref, BF16_RTOL, "dquery prefix")
    assert_close(to_np(dw), dw_ref, BF16_RTOL, "dweight (whole)")
    rest = dx.clone()
    rest[b0, :P] = 0
    assert not rest.any(), "gradient outside the prefix must be exactly zero"
    # dense upstream gradient: finite; linear in the upstream gradient
    dout2 = torch.randn((B, S, E), device="cuda", generator=gen).to(BT)
    dx2, dw2 = torch.empty_like(x), torch.empty_like(w)
    ffk.mha_backward(desc, x, dx2, x, None, x, None, w, dw2, dout2, reserve,
                     accumulate=ffk.MHA_OVERWRITE_WEIGHT_GRAD)
    assert torch.isfinite(dx2.float()).all() and torch.isfinite(dw2.float()).all()
    dout3 = (dout2.float() + dout.float()).to(BT)
    dw3 = torch.empty_like(w)
    ffk.mha_backward(desc, x, dx2, x, None, x, None, w, dw3, dout3, reserve,
                     accumulate=ffk.MHA_OVERWRITE_WEIGHT_GRAD)
    # dout3 is dout2 + dout up to one bf16 rounding of the P x E prefix entries
    assert_close(to_np(dw3), to_np(dw2) + to_np(dw), BF16_RTOL, "weight gradient is linear in the upstream gradient")


MHA_CASES = [  # B, Sq, Skv, H, E(q), Ek, Ev, Dh, oProj, self-attention? (, vProj)
    (2, 20, 20, 4, 64, 64, 64, 64, 64, True),
    (2, 33, 33, 2, 128, 128, 128, 64, 96, True),
    (1, 24, 40, 2, 64, 72, 80, 64, 64, False),
    (2, 64, 64, 2, 256, 256, 256, 128, 256, True),
    (2, 64, 64, 12, 768, 768, 768, 64, 768, True),  # both weight gradients in one two-problem GEMM launch
    (2, 24, 24, 2, 64, 64, 64, 64, 64, False),      # three tensors of one shape: one interleaved projection buffer
    # the reference's default transformer layer: 512 features, 8 heads, kdim = vdim = 2048 / 8 = 256
    # (lib/models/src/models/transformer/transformer.cc:37-38)
    (2, 40, 40, 8, 512, 512, 512, 256, 512, True),
    (1, 24, 40, 2, 64, 72, 80, 256, 64, False),
    # vdim != kdim (lib/op-attrs/src/op-attrs/ops/attention.cc:23-37 leaves both free)
    (2, 33, 33, 2, 128, 128, 128, 64, 96, True, 128),
    (2, 24, 24, 2, 64, 64, 64, 128, 64, False, 64),
    (1, 24, 40, 2, 64, 72, 80, 64, 64, False, 256),
    (2, 20, 20, 3, 96, 96, 96, 40, 96, True, 24),
]
MHA_CASES_FP32 = MHA_CASES[:4] + MHA_CASES[6:] + [
    (2, 20, 20, 4, 64, 64, 64, 16, 64, True),   # head sizes the bf16 core does not take
    (1, 24, 40, 2, 64, 72, 80, 40, 56, False),
    (2, 24, 24, 2, 64, 64, 64, 32, 64, False),
]


def _mha_case(ffk, oracle, case, causal, fp32):
    B, Sq, Skv, H, E, Ek, Ev, Dh, oP, self_attn = case[:10]
    Dv = case[10] if len(case) > 10 else Dh
    say("mha", "fp32" if fp32 else "bf16", case, "causal", causal)
    BT, BF16_RTOL, dtype = (torch.float32, FP32_RTOL, ffk.FLOAT) if fp32 else (torch.bfloat16, 2e-2, ffk.BF16)
    bf16_round = (lambda a: np.asarray(a, dtype=np.float32)) if fp32 else globals()["bf16_round"]
    g = rng(Sq + E + int(causal))
    scale = 1.0 / np.sqrt(Dh)
    query = bf16_round(g.standard_normal((B, Sq, E)))
    key = query if self_attn else bf16_round(g.standard_normal((B, Skv, Ek)))
    value = query if self_attn else bf16_round(g.standard_normal((B, Skv, Ev)))
    odesc = oracle.mha_desc(B, H, E, Ek, Ev, Dh, Dh, Dv, oP, Sq, Skv, scale, causal)
    desc = ffk.mha_desc(B, H, E, Ek, Ev, Dh, Dh, Dv, oP, Sq, Skv, scale, causal)
    nw = ffk.lib().ffk_mha_weight_elements(desc)
    assert nw == H * Dh * (E + Ek) + H * Dv * Ev + oP * H * Dv
    w = bf16_round(g.standard_normal((nw,)) * (2.0 / np.sqrt(E)))
    dout = bf16_round(g.standard_normal((B, Sq, oP)))
    out_ref = oracle.mha_forward(odesc, query, key, value, w, bf16_mode=not fp32)
    dq_ref, dk_ref, dv_ref, dw_ref = oracle.mha_backward(odesc, query, key, value, w, dout, bf16_mode=not fp32)

    qd = to_dev(query, torch, BT)
    kd = qd if self_attn else to_dev(key, torch, BT)
    vd = qd if self_attn else to_dev(value, torch, BT)
    wd, doutd = to_dev(w, torch, BT), to_dev(dout, torch, BT)
    reserve = ffk.mha_reserve(desc, dtype)
    out = ffk.mha_forward(desc, qd, kd, vd, wd, reserve)
    assert_close(to_np(out), out_ref, BF16_RTOL, "out")
    dw = torch.zeros_like(wd)
    dq = torch.full_like(qd, 3.0)  # input gradients are stored, not added to
    if self_attn:
        # key/value alias query: their gradients fold into query_grad
        ffk.mha_backward(desc, qd, dq, kd, None, vd, None, wd, dw, doutd, reserve)
        assert_close(to_np(dq), dq_ref + dk_ref + dv_ref, BF16_RTOL, "dquery (folded)")
    else:
        dk, dv = torch.full_like(kd, 3.0), torch.full_like(vd, 3.0)
        ffk.mha_backward(desc, qd, dq, kd, dk, vd, dv, wd, dw, doutd, reserve)
        assert_close(to_np(dq), dq_ref, BF16_RTOL, "dquery")
        assert_close(to_np(dk), dk_ref, BF16_RTOL, "dkey")
        assert_close(to_np(dv), dv_ref, BF16_RTOL, "dvalue")
    assert_close(to_np(dw), dw_ref, BF16_RTOL, "dweight")
    # weight_grad accumulates (CUDNN_WGRAD_MODE_ADD): a second call doubles it
    dq2 = torch.zeros_like(qd)
    if self_attn:
        ffk.mha_backward(desc, qd, dq2, kd, None, vd, None, wd, dw, doutd, reserve)
    else:
        ffk.mha_backward(desc, qd, dq2, kd, torch.zeros_like(kd), vd, torch.zeros_like(vd), wd, dw, doutd, reserve)
    assert_close(to_np(dw), 2 * dw_ref, BF16_RTOL, "dweight accumulated")


@pytest.mark.parametrize("case", MHA_CASES)
@pytest.mark.parametrize("causal", [False, True])
def test_mha(ffk, oracle, case, causal):
    _mha_case(ffk, oracle, case, causal, fp32=False)


@pytest.mark.parametrize("case", MHA_CASES_FP32)
@pytest.mark.parametrize("causal", [False, True])
def test_mha_fp32(ffk, oracle, case, causal):
    """FLOAT is the data type of the reference's own entry points (attention_kernels.h:12-51)."""
    _mha_case(ffk, oracle, case, causal, fp32=True)


def test_mha_accumulate_input_grads(ffk, oracle):
    say("mha input gradients added on request")
    B, S, H, E, Dh = 1, 16, 2, 64, 64
    g = rng(9)
    x = g.standard_normal((B, S, E)).astype(np.float32)
    odesc = oracle.mha_desc(B, H, E, E, E, Dh, Dh, Dh, E, S, S, 0.125, False)
    desc = ffk.mha_desc(B, H, E, E, E, Dh, Dh, Dh, E, S, S, 0.125, False)
    w = (g.standard_normal((ffk.lib().ffk_mha_weight_elements(desc),)) * 0.2).astype(np.float32)
    dout = g.standard_normal((B, S, E)).astype(np.float32)
    dq_ref, dk_ref, dv_ref, _ = oracle.mha_backward(odesc, x, x, x, w, dout)
    xd, wd, dd = to_dev(x, torch), to_dev(w, torch), to_dev(dout, torch)
    reserve = ffk.mha_reserve(desc, ffk.FLOAT)
    ffk.mha_forward(desc, xd, xd, xd, wd, reserve)
    dq = torch.full_like(xd, 2.0)
    ffk.mha_backward(desc, xd, dq, xd, None, xd, None, wd, torch.zeros_like(wd), dd, reserve, accumulate=True)
    assert_close(to_np(dq), 2.0 + dq_ref + dk_ref + dv_ref, FP32_RTOL, "dquery added")
    # one tensor in three roles: key_grad without value_grad has no meaning
    with pytest.raises(ffk.FFKError, match="one tensor"):
        ffk.mha_backward(desc, xd, dq, xd, torch.zeros_like(xd), xd, None, wd, torch.zeros_like(wd), dd, reserve)


def test_mha_separate_grads_when_aliased(ffk, oracle):
    say("mha aliased, separate grads")
    B, S, H, E, Dh = 1, 16, 2, 64, 64
    g = rng(8)
    x = bf16_round(g.standard_normal((B, S, E)))
    odesc = oracle.mha_desc(B, H, E, E, E, Dh, Dh, Dh, E, S, S, 0.125, False)
    desc = ffk.mha_desc(B, H, E, E, E, Dh, Dh, Dh, E, S, S, 0.125, False)
    w = bf16_round(g.standard_normal((ffk.lib().ffk_mha_weight_elements(desc),)) * 0.2)
    dout = bf16_round(g.standard_normal((B, S, E)))
    dq_ref, dk_ref, dv_ref, _ = oracle.mha_backward(odesc, x, x, x, w, dout, bf16_mode=True)
    xd, wd, dd = to_dev(x, torch, BT), to_dev(w, torch, BT), to_dev(dout, torch, BT)
    reserve = ffk.mha_reserve(desc, ffk.BF16)
    ffk.mha_forward(desc, xd, xd, xd, wd, reserve)
    dq, dk, dv = (torch.zeros_like(xd) for _ in range(3))
    dw = torch.zeros_like(wd)
    ffk.mha_backward(desc, xd, dq, xd, dk, xd, dv, wd, dw, dd, reserve)
    assert_close(to_np(dq), dq_ref, BF16_RTOL, "dq")
    assert_close(to_np(dk), dk_ref, BF16_RTOL, "dk")
    assert_close(to_np(dv), dv_ref, BF16_RTOL, "dv")


def test_mha_errors(ffk):
    desc = ffk.mha_desc(1, 2, 64, 64, 64, 64, 64, 64, 64, 8, 8)
    x = torch.zeros((1, 8, 64), dtype=BT, device="cuda")
    w = torch.zeros((ffk.lib().ffk_mha_weight_elements(desc),), dtype=BT, device="cuda")
    small = torch.zeros((16,), dtype=torch.uint8, device="cuda")
    with pytest.raises(ffk.FFKError, match="reserve"):
        ffk.mha_forward(desc, x, x, x, w, small)
    bad = ffk.mha_desc(1, 2, 64, 64, 64, 44, 44, 44, 64, 8, 8)
    with pytest.raises(ffk.FFKError, match="projection size"):
        ffk.mha_forward(bad, x, x, x, w, ffk.mha_reserve(desc, ffk.BF16))
    bad = ffk.mha_desc(1, 2, 64, 64, 64, 64, 128, 64, 64, 8, 8)
    with pytest.raises(ffk.FFKError, match="qProjSize must equal kProjSize"):
        ffk.mha_forward(bad, x, x, x, w, ffk.mha_reserve(desc, ffk.BF16))
    bad = ffk.mha_desc(1, 2, 64, 64, 64, 260, 260, 260, 64, 8, 8)
    x32, w32 = x.float(), torch.zeros((ffk.lib().ffk_mha_weight_elements(bad),), dtype=torch.float32, device="cuda")
    with pytest.raises(ffk.FFKError, match="projection size"):
        ffk.mha_forward(bad, x32, x32, x32, w32, ffk.mha_reserve(bad, ffk.FLOAT))
