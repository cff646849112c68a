"""Transformer encoder layer forward+backward (BASELINE config 2 structure)
against the layer composed from oracle operators."""
import sys

import numpy as np
import pytest
import torch

from layer_oracle import layer_forward_backward, make_params
from util import assert_close, bf16_round, rng, to_dev, to_np

pytestmark = pytest.mark.gpu
BT = torch.bfloat16


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_device(ffk, cfg, params, x, dy, overwrite_weight_grads=False):
    desc = ffk.EncoderLayerDesc(cfg["batch"], cfg["seq"], cfg["d_model"], cfg["heads"], cfg["d_ff"],
                                cfg["p"], cfg["seed"], cfg["eps"], cfg["scale"], int(cfg["causal"]),
                                int(cfg["pre_ln"]), ffk.ACT_GELU if cfg["gelu"] else ffk.ACT_RELU,
                                int(overwrite_weight_grads))
    wt = {k: to_dev(v, torch, BT) for k, v in params.items()}
    # storing mode must not care what the gradient tensors hold
    gt = {k: (torch.full_like(v, 3.0) if overwrite_weight_grads else torch.zeros_like(v)) for k, v in wt.items()}
    xd, dyd = to_dev(x, torch, BT), to_dev(dy, torch, BT)
    y, dx = torch.empty_like(xd), torch.empty_like(xd)
    ws = ffk.encoder_layer_workspace(desc, ffk.BF16)
    W, G = ffk.encoder_layer_params(wt), ffk.encoder_layer_params(gt)
    ffk.encoder_layer_forward(desc, W, xd, y, ws)
    ffk.encoder_layer_backward(desc, W, G, xd, dyd, dx, ws)
    torch.cuda.synchronize()
    return to_np(y), to_np(dx), {k: to_np(v) for k, v in gt.items()}


@pytest.mark.parametrize("pre_ln,gelu", [(True, True), (False, False)])
@pytest.mark.parametrize("p", [0.0, 0.1])
def test_encoder_layer_small(ffk, oracle, pre_ln, gelu, p):
    cfg = dict(batch=2, seq=48, d_model=128, heads=2, d_ff=256, p=p, seed=1234, eps=1e-5,
               scale=1.0 / 8.0, causal=False, pre_ln=pre_ln, gelu=gelu)
    say("encoder layer", cfg)
    g = rng(17)
    params = make_params(g, cfg, bf16_round)
    # larger weights than N(0, 0.02) so that every branch contributes visibly
    for k in ("attn_weight", "w1", "w2"):
        params[k] = bf16_round(params[k] * 4)
    x = bf16_round(g.standard_normal((cfg["batch"], cfg["seq"], cfg["d_model"])))
    dy = bf16_round(g.standard_normal(x.shape))
    y_ref, dx_ref, g_ref = layer_forward_backward(oracle, cfg, params, x, dy)
    y, dx, grads = run_device(ffk, cfg, params, x, dy)
    # every tensor within the bf16 tolerance of 2e-2 (measured: at most 0.17 of that bound,
    # through a dozen chained bf16 roundings, both variants)
    assert_close(y, y_ref, 2e-2, "y")
    assert_close(dx, dx_ref, 2e-2, "dx")
    for k in g_ref:
        assert_close(grads[k].reshape(g_ref[k].shape), g_ref[k], 2e-2, "grad " + k)


def test_encoder_layer_config2_shape_runs_and_is_deterministic(ffk):
    """BASELINE config 2 at full size: B 8, S 512, d 1024, H 16, FFN 4096,
    pre-LN, GELU, dropout 0.1.  Size-independent checks: finite outputs,
    bit-identical repeat (no atomics on this path), dropout really drops."""
    cfg = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096, p=0.1, seed=7, eps=1e-5,
               scale=0.125, causal=False, pre_ln=True, gelu=True)
    say("encoder layer cfg2 full size")
    g = rng(2)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((8, 512, 1024)))
    dy = bf16_round(g.standard_normal(x.shape))
    y1, dx1, g1 = run_device(ffk, cfg, params, x, dy)
    y2, dx2, g2 = run_device(ffk, cfg, params, x, dy)
    assert np.isfinite(y1).all() and np.isfinite(dx1).all()
    assert np.array_equal(y1, y2) and np.array_equal(dx1, dx2)
    for k in g1:
        assert np.isfinite(g1[k]).all() and np.array_equal(g1[k], g2[k]), k
    cfg0 = dict(cfg, p=0.0)
    y0, _, _ = run_device(ffk, cfg0, params, x, dy)
    assert not np.array_equal(y0, y1)


def test_encoder_layer_config2_full_size_against_the_oracle_on_one_sequence(ffk, oracle):
    """BASELINE config 2 at full size against the oracle.  The layer mixes tokens only inside a
    sequence, and the dropout streams are indexed by flat element position, so sequence 0 of the
    batch of 8 (the first 512 x 1024 elements of every activation) is what the oracle computes for
    a batch of that one sequence with the same weights, seeds and upstream gradient: y[0] and dx[0]
    are compared with it.  This runs the kernels the full size dispatches to (the pipelined GEMMs
    with the element-wise tails, the paired weight-gradient launches, split-K), which the small
    layer tests do not reach.  The weight gradients sum over all 8 sequences; they are covered at
    this size by the bit-equality with the one-kernel-per-operator sequence below."""
    cfg = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096, p=0.1, seed=7, eps=1e-5,
               scale=0.125, causal=False, pre_ln=True, gelu=True)
    say("encoder layer cfg2 full size vs oracle on sequence 0")
    g = rng(2)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((8, 512, 1024)))
    dy = bf16_round(g.standard_normal(x.shape))
    y, dx, _ = run_device(ffk, cfg, params, x, dy)
    cfg1 = dict(cfg, batch=1)
    y_ref, dx_ref, _ = layer_forward_backward(oracle, cfg1, params, x[:1], dy[:1])
    assert_close(y[:1], y_ref, 2e-2, "y[0]")
    assert_close(dx[:1], dx_ref, 2e-2, "dx[0]")
    # and the other sequences are not copies of sequence 0
    assert not np.array_equal(y[1], y[0])


@pytest.mark.parametrize("shape", ["small", "config2"])
@pytest.mark.parametrize("pre_ln,gelu", [(True, True), (False, True), (False, False)])
def test_fused_layer_equals_operator_sequence(ffk, shape, pre_ln, gelu):
    """The layer entry points fuse neighbouring ops (GELU into the GEMM
    epilogue, dropout into the residual add, dropout backward into GELU
    backward, the residual add into LayerNorm backward).  With the option
    FFK_OPTION_LAYER_UNFUSED set the same entry points run one kernel per
    operator; both must give the same bits."""
    if shape == "small":
        cfg = dict(batch=2, seq=64, d_model=128, heads=2, d_ff=256)
    else:
        cfg = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096)
    cfg.update(p=0.1, seed=99, eps=1e-5, scale=0.125, causal=False, pre_ln=pre_ln, gelu=gelu)
    say("fused vs operator sequence", cfg)
    g = rng(5)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((cfg["batch"], cfg["seq"], cfg["d_model"])))
    dy = bf16_round(g.standard_normal(x.shape))
    ffk.set_option(ffk.OPTION_LAYER_UNFUSED, 1)
    try:
        y_u, dx_u, g_u = run_device(ffk, cfg, params, x, dy)
    finally:
        ffk.set_option(ffk.OPTION_LAYER_UNFUSED, 0)
    y_f, dx_f, g_f = run_device(ffk, cfg, params, x, dy)
    assert np.array_equal(y_u, y_f)
    assert np.array_equal(dx_u, dx_f)
    for k in g_u:
        assert np.array_equal(g_u[k], g_f[k]), k


def test_split_k_weight_gradient_matches_unsplit(ffk):
    """At config 2 the attention output projection's weight gradient
    ([1024 x 1024] output, reduction over 4096 tokens) runs as a split-K GEMM
    with fp32 partial sums.  FFK_OPTION_GEMM_VARIANT = 128 forces the same tile
    configuration without the split; the two differ only in fp32 summation
    order, so the bf16 results agree to a rounding step."""
    cfg = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096, p=0.1, seed=3, eps=1e-5,
               scale=0.125, causal=False, pre_ln=True, gelu=True)
    say("split-K vs unsplit", cfg)
    g = rng(8)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((8, 512, 1024)))
    dy = bf16_round(g.standard_normal(x.shape))
    ffk.set_option(ffk.OPTION_GEMM_VARIANT, 128)
    try:
        _, _, g_plain = run_device(ffk, cfg, params, x, dy)
    finally:
        ffk.set_option(ffk.OPTION_GEMM_VARIANT, 0)
    _, _, g_split = run_device(ffk, cfg, params, x, dy)
    E = 1024
    wo_plain = g_plain["attn_weight"][3 * E * E:]
    wo_split = g_split["attn_weight"][3 * E * E:]
    assert np.abs(wo_plain).max() > 0
    assert_close(wo_split, wo_plain, 1e-2, "dW_O split-K vs unsplit")


@pytest.mark.parametrize("pre_ln,gelu", [(True, True), (False, False)])
def test_stored_weight_gradients_equal_added_into_zero(ffk, pre_ln, gelu):
    """overwrite_weight_grads stores every weight gradient: the same bits as adding into
    cleared tensors, whatever the tensors held before."""
    cfg = dict(batch=2, seq=48, d_model=128, heads=2, d_ff=256, p=0.1, seed=99, eps=1e-5,
               scale=1.0 / 8.0, causal=False, pre_ln=pre_ln, gelu=gelu)
    say("stored weight gradients", cfg)
    g = rng(23)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((cfg["batch"], cfg["seq"], cfg["d_model"])))
    dy = bf16_round(g.standard_normal(x.shape))
    y0, dx0, g0 = run_device(ffk, cfg, params, x, dy)
    y1, dx1, g1 = run_device(ffk, cfg, params, x, dy, overwrite_weight_grads=True)
    assert np.array_equal(y0, y1) and np.array_equal(dx0, dx1)
    for k in g0:
        assert np.any(g0[k] != 0), k
        assert np.array_equal(g0[k], g1[k]), k


@pytest.mark.parametrize("pre_ln,gelu", [(True, True), (False, False)])
@pytest.mark.parametrize("fused", [True, False])
def test_weight_gradients_add_up_over_two_backward_calls(ffk, pre_ln, gelu, fused):
    """Without overwrite_weight_grads every weight gradient is added into (micro-batch
    accumulation): two backward calls leave twice one call's gradient in every tensor,
    the LayerNorm parameters included."""
    cfg = dict(batch=2, seq=48, d_model=128, heads=2, d_ff=256, p=0.1, seed=5, eps=1e-5,
               scale=1.0 / 8.0, causal=False, pre_ln=pre_ln, gelu=gelu)
    say("weight gradients over two calls", cfg, "fused", fused)
    g = rng(29)
    params = make_params(g, cfg, bf16_round)
    x = bf16_round(g.standard_normal((cfg["batch"], cfg["seq"], cfg["d_model"])))
    dy = bf16_round(g.standard_normal(x.shape))
    desc = ffk.EncoderLayerDesc(cfg["batch"], cfg["seq"], cfg["d_model"], cfg["heads"], cfg["d_ff"],
                                cfg["p"], cfg["seed"], cfg["eps"], cfg["scale"], 0, int(pre_ln),
                                ffk.ACT_GELU if gelu else ffk.ACT_RELU, 0)
    wt = {k: to_dev(v, torch, torch.float32).to(BT) for k, v in params.items()}
    xd, dyd = to_dev(x, torch, BT), to_dev(dy, torch, BT)
    y, dx = torch.empty_like(xd), torch.empty_like(xd)
    ws = ffk.encoder_layer_workspace(desc, ffk.BF16)
    W = ffk.encoder_layer_params(wt)
    ffk.set_option(ffk.OPTION_LAYER_UNFUSED, 0 if fused else 1)
    try:
        ffk.encoder_layer_forward(desc, W, xd, y, ws)
        once = {k: torch.zeros_like(v) for k, v in wt.items()}
        ffk.encoder_layer_backward(desc, W, ffk.encoder_layer_params(once), xd, dyd, dx, ws)
        twice = {k: torch.zeros_like(v) for k, v in wt.items()}
        G2 = ffk.encoder_layer_params(twice)
        ffk.encoder_layer_backward(desc, W, G2, xd, dyd, dx, ws)
        ffk.encoder_layer_backward(desc, W, G2, xd, dyd, dx, ws)
    finally:
        ffk.set_option(ffk.OPTION_LAYER_UNFUSED, 0)
    torch.cuda.synchronize()
    for k in once:
        a, b = to_np(once[k]), to_np(twice[k])
        assert np.any(a != 0), k
        # g + g is exact in bf16 up to the rounding of the second addition's operand
        assert_close(b, 2 * a, 1e-2, "twice " + k)
