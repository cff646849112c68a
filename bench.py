"""Headline benchmark: transformer encoder layer forward+backward tokens/s on
one MI355X (BASELINE config 2: bf16, batch 8, seq 512, d_model 1024, 16 heads,
FFN 4096 GELU, pre-LayerNorm, dropout 0.1; synthetic N(0,1) activations and
N(0,0.02) weights).

    python bench.py --gpus 1 --steps K --warmup W [--config N]

Prints one JSON line.  Besides the whole-step throughput it reports
  check        : before anything is timed, a small layer is compared with the
                 CPU oracle, and the full-size step's outputs must be finite
                 and bit-identical over two runs (their checksums are printed);
  roofline     : the dominant kernel (the bf16 MFMA GEMM of the first FFN
                 projection, [4096,1024] x [4096,1024]^T), timed live with HIP
                 events on the launch stream, against the 2.5 PFLOP/s dense
                 bf16 MFMA peak;
  device_copy  : a plain device copy's GB/s, measured in the same run, beside
                 the 8 TB/s vendor figure;
  mfma_loop    : the matrix rate every SIMD sustains issuing bf16 MFMAs back
                 to back from registers, measured in the same run, beside the
                 2.5 PFLOP/s vendor figure (roofline.frac_of_measured_mfma_loop
                 restates the dominant kernel's fraction against it);
  clock_settle : the untimed steps run before the warm-up steps, until the
                 shader clock has reached the state it then holds;
  cpu_baseline : the CPU oracle's restatement of the same layer, timed on the
                 host cores on a bounded sample (one sequence of 128 tokens of
                 the same layer), scaled to tokens/s.
--config 1, 3, 4 or 5 measures one of the other BASELINE configurations
instead (per-kernel times against their roofline, and the oracle timed beside
them on a stated sub-shape); config 2 is the default and the headline.
"""
import argparse
import ctypes
import hashlib
import importlib.util
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))


def _load(name, path):
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def _oracle():
    return _load("ffk_oracle", os.path.join(ROOT, "oracle", "oracle.py"))


def _oracle_one_core():
    """The oracle for the cpu_baseline legs: one thread, like the reference's CPU kernels."""
    oracle = _oracle()
    oracle.set_num_threads(1)
    return oracle


CFG = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096, p=0.1, seed=20240, eps=1e-5,
           scale=1.0 / 8.0, causal=False, pre_ln=True, gelu=True)
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "ffn_up_gemm_hbm_traffic.md")


SETTLE_SECONDS = 0.2


def settle_clocks(fn, least=0, seconds=SETTLE_SECONDS):
    """Runs fn untimed, at least `least` times and for at least `seconds`: the card's shader clock
    needs some tens of milliseconds of sustained load to reach the state it then holds (launches
    in the first 50 ms after an idle spell measure 10-20% slow, 40 consecutive launches of one
    kernel show the time falling launch by launch), and a timed region that starts inside that
    ramp measures the ramp.  Returns the number of calls made."""
    import torch
    n = 0
    t0 = time.perf_counter()
    while n < least or time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        n += 20
        torch.cuda.synchronize()
    return n


def event_timer(ffk):
    """us per call of fn, HIP events on the stream the entry points are launched on."""
    lib = ffk.lib()

    def run(fn, iters=50, warm=5):
        stream = ffk.current_stream()
        e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
        ffk.check(lib.ffk_event_create(ctypes.byref(e0)))
        ffk.check(lib.ffk_event_create(ctypes.byref(e1)))
        settle_clocks(fn, warm)
        ffk.check(lib.ffk_event_record(e0, stream))
        for _ in range(iters):
            fn()
        ffk.check(lib.ffk_event_record(e1, stream))
        ffk.check(lib.ffk_event_synchronize(e1))
        ms = ctypes.c_float()
        ffk.check(lib.ffk_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        lib.ffk_event_destroy(e0)
        lib.ffk_event_destroy(e1)
        return ms.value / iters * 1e3
    return run


def make_device_state(ffk, torch, cfg):
    bt = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(1)
    desc = ffk.EncoderLayerDesc(cfg["batch"], cfg["seq"], cfg["d_model"], cfg["heads"], cfg["d_ff"],
                                cfg["p"], cfg["seed"], cfg["eps"], cfg["scale"], int(cfg["causal"]),
                                int(cfg["pre_ln"]), ffk.ACT_GELU if cfg["gelu"] else ffk.ACT_RELU,
                                1)  # every weight gradient is stored, not added: nothing to clear per step
    shapes = ffk.encoder_layer_param_shapes(desc)
    wt = {}
    for name, shape in shapes.items():
        t = torch.randn(shape, device="cuda", generator=gen) * 0.02
        if name.endswith("gamma"):
            t = t + 1.0
        wt[name] = t.to(bt)
    # all weight gradients live in one flat buffer (16-byte aligned slices)
    sizes = {k: (v.numel() + 7) // 8 * 8 for k, v in wt.items()}
    flat = torch.zeros((sum(sizes.values()),), dtype=bt, device="cuda")
    gt, off = {}, 0
    for k, v in wt.items():
        gt[k] = flat[off:off + v.numel()].view(v.shape)
        off += sizes[k]
    T = cfg["batch"] * cfg["seq"]
    x = torch.randn((T, cfg["d_model"]), device="cuda", generator=gen).to(bt)
    dy = torch.randn((T, cfg["d_model"]), device="cuda", generator=gen).to(bt)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    ws = ffk.encoder_layer_workspace(desc, ffk.BF16)
    return dict(desc=desc, wt=wt, gt=gt, grad_flat=flat, x=x, dy=dy, y=y, dx=dx, ws=ws,
                W=ffk.encoder_layer_params(wt), G=ffk.encoder_layer_params(gt))


def step(ffk, st):
    # one training step of the layer: forward, backward (which stores fresh weight gradients)
    ffk.encoder_layer_forward(st["desc"], st["W"], st["x"], st["y"], st["ws"])
    ffk.encoder_layer_backward(st["desc"], st["W"], st["G"], st["x"], st["dy"], st["dx"], st["ws"])


def check_before_timing(ffk, torch, st):
    """(1) a small layer of the same structure against the CPU oracle, through the same entry
    points; (2) the full-size step: finite outputs, and the same bits on a second run."""
    import numpy as np
    oracle = _oracle()
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from layer_oracle import layer_forward_backward, make_params
    from util import assert_close, bf16_round, to_dev, to_np
    cfg = dict(CFG, batch=2, seq=32, d_model=128, heads=2, d_ff=256, seed=99)
    g = np.random.default_rng(0)
    params = make_params(g, cfg, bf16_round)
    for k in ("attn_weight", "w1", "w2"):
        params[k] = bf16_round(params[k] * 4)
    x = bf16_round(g.standard_normal((2, 32, 128)))
    dy = bf16_round(g.standard_normal(x.shape))
    y_ref, dx_ref, g_ref = layer_forward_backward(oracle, cfg, params, x, dy)
    bt = torch.bfloat16
    desc = ffk.EncoderLayerDesc(2, 32, 128, 2, 256, cfg["p"], 99, cfg["eps"], cfg["scale"], 0, 1, ffk.ACT_GELU, 1)
    wt = {k: to_dev(v, torch, bt) for k, v in params.items()}
    gt = {k: torch.zeros_like(v) for k, v in wt.items()}
    xd, dyd = to_dev(x, torch, bt), to_dev(dy, torch, bt)
    y, dx = torch.empty_like(xd), torch.empty_like(xd)
    ws = ffk.encoder_layer_workspace(desc, ffk.BF16)
    W, G = ffk.encoder_layer_params(wt), ffk.encoder_layer_params(gt)
    ffk.encoder_layer_forward(desc, W, xd, y, ws)
    ffk.encoder_layer_backward(desc, W, G, xd, dyd, dx, ws)
    torch.cuda.synchronize()
    assert_close(to_np(y), y_ref, 2e-2, "bench check: y of the small layer")
    assert_close(to_np(dx), dx_ref, 2e-2, "bench check: dx of the small layer")
    assert_close(to_np(gt["w1"]), g_ref["w1"], 2e-2, "bench check: dW1 of the small layer")

    def checksum(t):
        f = t.double()
        return [float(f.sum()), float(f.abs().sum())]

    step(ffk, st)
    torch.cuda.synchronize()
    first = [checksum(st["y"]), checksum(st["dx"]), checksum(st["grad_flat"])]
    nonfinite = int((~torch.isfinite(st["y"].float())).sum() + (~torch.isfinite(st["dx"].float())).sum() +
                    (~torch.isfinite(st["grad_flat"].float())).sum())
    assert nonfinite == 0, "bench check: %d non-finite values in the step's outputs" % nonfinite
    y1, dx1 = st["y"].clone(), st["dx"].clone()
    step(ffk, st)
    torch.cuda.synchronize()
    assert torch.equal(y1, st["y"]) and torch.equal(dx1, st["dx"]), "bench check: the step is not reproducible"
    assert first[0][1] > 0 and first[1][1] > 0 and first[2][1] > 0, "bench check: an output is all zero"
    return {"small_layer_vs_oracle": "ok (y, dx, dW1 within 2e-2)", "nonfinite": 0, "repeatable_bits": True,
            "sum_abs_sum": {"y": first[0], "dx": first[1], "weight_grads": first[2]}}


def dominant_kernel_traffic():
    """HBM bytes one launch of the dominant kernel moves, from the `rocprofv3 --pmc FETCH_SIZE`
    and `--pmc WRITE_SIZE` runs kept in profiles/ffn_up_gemm_hbm_traffic.md.  That file names
    the hash of the GEMM source the counters were taken with; for any other source the
    figure is stale and None is reported."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    m_bytes = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
    m_hash = re.search(r"gemm_source_sha256:\s*([0-9a-f]{64})", text)
    if not m_bytes or not m_hash:
        return None
    src = os.path.join(ROOT, "flexflow-train_amd", "csrc", "gemm.hip")
    if hashlib.sha256(open(src, "rb").read()).hexdigest() != m_hash.group(1):
        return None
    return int(m_bytes.group(1))


def time_dominant_kernel(ffk, torch, cfg, iters=50, calibration_copy=False):
    """The FFN up-projection (Linear forward with bias, [4096,1024] x
    [4096,1024]^T) at its real shape, HIP events on the stream the kernel is
    launched on.  calibration_copy also launches one element-wise copy of
    256 MiB (read 256 MiB, write 256 MiB) for scaling HBM traffic counters."""
    T, E, F = cfg["batch"] * cfg["seq"], cfg["d_model"], cfg["d_ff"]
    bt = torch.bfloat16
    A = torch.randn((T, E), device="cuda").to(bt)
    B = (torch.randn((F, E), device="cuda") * 0.02).to(bt)
    bias = (torch.randn((F,), device="cuda") * 0.02).to(bt)
    C = torch.empty((T, F), device="cuda", dtype=bt)
    if calibration_copy:
        src = torch.randn((128 << 20,), device="cuda").to(bt)  # 256 MiB of bf16
        dst = torch.empty_like(src)
        ffk.element_unary_forward(ffk.OP["IDENTITY"], src, out=dst)
    us = event_timer(ffk)(lambda: ffk.linear_forward(A, B, bias, ffk.ACT_NONE, C), iters)
    sec = us * 1e-6
    flops = 2.0 * T * F * E
    return dict(bound="mfma", achieved=flops / sec / 1e12, peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s",
                frac=flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                traffic=dominant_kernel_traffic(),
                # asked of the library's own dispatch for this shape, not written down here
                kernel="%s (FFN up-projection, M%d N%d K%d, bias)"
                       % (ffk.gemm_kernel_name(ffk.BF16, False, True, T, F, E, has_bias=True), T, F, E),
                us_per_launch=us)


def measure_mfma_loop(ffk, torch):
    """The library's probe: every SIMD issues bf16 32x32x16 matrix instructions back to back from
    registers.  What it reaches is the ceiling for a GEMM on this card at the clock it sustains."""
    out = torch.empty((256 * 256,), device="cuda")
    flops = ffk.probe_mfma_bf16(2000, out)
    us = event_timer(ffk)(lambda: ffk.probe_mfma_bf16(2000, out), 20)
    return {"TFLOP/s": flops / us / 1e6, "vendor_peak_TFLOP/s": MFMA_BF16_PEAK_TFLOPS,
            "what": "256 CUs x 4 waves, 32000 back-to-back 32x32x16 bf16 MFMAs each on random operands in registers"}


def measure_device_copy(ffk, torch):
    """A plain copy of 256 MiB (the library's element-wise identity), GB/s of read + written bytes."""
    src = torch.randn((128 << 20,), device="cuda").to(torch.bfloat16)
    dst = torch.empty_like(src)
    us = event_timer(ffk)(lambda: ffk.element_unary_forward(ffk.OP["IDENTITY"], src, out=dst), 20)
    return {"GB/s": 2.0 * src.numel() * 2 / us / 1e3, "vendor_peak_GB/s": HBM_PEAK_GBPS,
            "what": "element-wise identity over 256 MiB bf16, read + write"}


def cpu_baseline(cfg):
    """The oracle's layer on a bounded sample: 1 sequence x 128 tokens of the
    same layer (same widths), single thread, scaled to tokens/s."""
    import numpy as np
    oracle = _oracle_one_core()
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from layer_oracle import layer_forward_backward, make_params
    small = dict(cfg, batch=1, seq=128)
    g = np.random.default_rng(0)
    rb = oracle.round_bf16
    params = make_params(g, small, rb)
    x = rb(g.standard_normal((1, 128, cfg["d_model"])))
    dy = rb(g.standard_normal(x.shape))
    t0 = time.perf_counter()
    layer_forward_backward(oracle, small, params, x, dy)
    dt = time.perf_counter() - t0
    return dict(value=128 / dt, unit="tokens/s", cores=1, kind="port",
                sample="oracle layer fwd+bwd on 1 sequence x 128 tokens (same d_model/heads/FFN), "
                       "%.1f s; attention cost per token is lower than at seq 512" % dt)


# ---------------------------------------------------------------------------
# The other BASELINE configurations (--config 1, 3, 4, 5): per-kernel times
# against the roofline, with the oracle timed beside them on a stated sub-shape.
# ---------------------------------------------------------------------------
def _kernel_row(name, us, bytes_=None, flops=None, peak_tflops=MFMA_BF16_PEAK_TFLOPS):
    row = {"kernel": name, "us": us}
    if bytes_ is not None:
        row.update(bound="hbm", achieved=bytes_ / us / 1e3, peak=HBM_PEAK_GBPS, unit="GB/s",
                   frac=bytes_ / us / 1e3 / HBM_PEAK_GBPS)
    if flops is not None:
        row.update(bound="mfma", achieved=flops / us / 1e6, peak=peak_tflops, unit="TFLOP/s",
                   frac=flops / us / 1e6 / peak_tflops)
    return row


def _cpu_time(fn, min_seconds=1.0, max_reps=100000):
    """Seconds per call of fn on one host core."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or reps >= max_reps:
            return dt / reps


def config1(ffk, torch, with_cpu):
    """Linear fwd+bwd, fp32, input [32,64], weight [128,64] + bias, ReLU: the one case the
    reference runs on its CPU path (linear_kernels_cpu.cc:12-94); the oracle is that path."""
    import numpy as np
    g = np.random.default_rng(1)
    batch, in_dim, out_dim = 32, 64, 128
    x = g.uniform(-1, 1, (batch, in_dim)).astype(np.float32)
    w = (g.standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
    b = (g.standard_normal((out_dim,)) * 0.02).astype(np.float32)
    dy = g.standard_normal((batch, out_dim)).astype(np.float32)
    xd, wd, bd, dyd = (torch.from_numpy(a).cuda() for a in (x, w, b, dy))
    y = torch.empty((batch, out_dim), device="cuda")
    dx, dw, db = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(bd)
    need = ffk.lib().ffk_linear_backward_workspace_bytes(ffk.FLOAT, ffk.ACT_RELU, 1, batch, out_dim)
    ws = torch.empty((max(need, 1),), dtype=torch.uint8, device="cuda")
    timer = event_timer(ffk)
    fwd = lambda: ffk.linear_forward(xd, wd, bd, ffk.ACT_RELU, y)
    bwd = lambda: ffk.linear_backward(y, dyd, xd, wd, dx, dw, db, activation=ffk.ACT_RELU, workspace=ws)
    us_f, us_b = timer(fwd, 200, 20), timer(bwd, 200, 20)
    f_fwd = 2.0 * batch * in_dim * out_dim
    rows = [_kernel_row("Linear fp32 forward [32,64]x[128,64]^T + bias + ReLU", us_f, flops=f_fwd,
                        peak_tflops=MFMA_FP32_PEAK_TFLOPS),
            _kernel_row("Linear fp32 backward (dX, dW, db)", us_b, flops=2 * f_fwd, peak_tflops=MFMA_FP32_PEAK_TFLOPS)]
    out = {"value": batch / ((us_f + us_b) * 1e-6), "unit": "samples/s", "ms_per_step": (us_f + us_b) * 1e-3,
           "dtype": "f32", "kernels": rows,
           "config": {"workload": "single Linear fwd+bwd, fp32, input [32,64], weight [128,64] + bias, ReLU "
                                  "(BASELINE config 1); launch-latency bound: 0.5 MFLOP per pass"}}
    if with_cpu:
        oracle = _oracle_one_core()
        yc = oracle.linear_forward(x, w, b, activation=0)
        t_f = _cpu_time(lambda: oracle.linear_forward(x, w, b, activation=0))
        t_b = _cpu_time(lambda: oracle.linear_backward(yc, dy, x, w, activation=0))
        out["cpu_baseline"] = {"value": batch / (t_f + t_b), "unit": "samples/s", "cores": 1, "kind": "port",
                               "sample": "the whole workload: oracle linear forward %.1f us, backward %.1f us per call"
                                         % (t_f * 1e6, t_b * 1e6)}
    return out


def config3(ffk, torch, with_cpu):
    """Bandwidth-bound op set, bf16: LayerNorm [16384,4096], Softmax [128,2048,2048] over the last dim,
    ElementBinary add / mul and Dropout p = 0.1 on [16384,4096], forward and backward."""
    bt = torch.bfloat16
    timer = event_timer(ffk)
    M, N = 16384, 4096
    n = M * N
    rows = []
    a, b = torch.randn(n, device="cuda").to(bt), torch.randn(n, device="cuda").to(bt)
    o, da, db = torch.empty_like(a), torch.empty_like(a), torch.empty_like(a)
    ADD, MUL = ffk.OP["EW_ADD"], ffk.OP["EW_MUL"]
    rows.append(_kernel_row("ElementBinary add fwd", timer(lambda: ffk.element_binary_forward(ADD, a, b, out=o), 20), bytes_=6 * n))
    rows.append(_kernel_row("ElementBinary mul fwd", timer(lambda: ffk.element_binary_forward(MUL, a, b, out=o), 20), bytes_=6 * n))
    rows.append(_kernel_row("ElementBinary add bwd", timer(lambda: ffk.element_binary_backward(ADD, o, a, b, da, db), 20), bytes_=6 * n))
    rows.append(_kernel_row("ElementBinary mul bwd", timer(lambda: ffk.element_binary_backward(MUL, o, a, b, da, db), 20), bytes_=10 * n))
    rows.append(_kernel_row("Dropout p=0.1 fwd", timer(lambda: ffk.dropout_forward(a, 0.1, 12345, out=o), 20), bytes_=4 * n))
    rows.append(_kernel_row("Dropout p=0.1 bwd", timer(lambda: ffk.dropout_backward(a, 0.1, 12345, dx=o), 20), bytes_=4 * n))
    x, dy = a.view(M, N), b.view(M, N)
    gam, bet = torch.ones(N, device="cuda", dtype=bt), torch.zeros(N, device="cuda", dtype=bt)
    y, dx = o.view(M, N), da.view(M, N)
    mean, rstd = torch.empty(M, device="cuda"), torch.empty(M, device="cuda")
    dg, dbe = torch.empty_like(gam), torch.empty_like(gam)
    ws = torch.empty(ffk.lib().ffk_layer_norm_backward_workspace_bytes(M, N), dtype=torch.uint8, device="cuda")
    rows.append(_kernel_row("LayerNorm fwd [16384,4096]", timer(lambda: ffk.layer_norm_forward(x, gam, bet, 1e-5, y, mean, rstd), 20), bytes_=4 * n))
    rows.append(_kernel_row("LayerNorm bwd [16384,4096]", timer(lambda: ffk.layer_norm_backward(dy, x, mean, rstd, gam, dx, dg, dbe, workspace=ws), 20), bytes_=6 * n))
    del a, b, o, da, db
    outer, dim = 128 * 2048, 2048
    sx = (torch.randn((outer, dim), device="cuda") * 4).to(bt)
    sy, sdy, sdx = torch.empty_like(sx), torch.randn((outer, dim), device="cuda").to(bt), torch.empty_like(sx)
    rows.append(_kernel_row("Softmax fwd [128,2048,2048]", timer(lambda: ffk.softmax_forward(sx, outer, dim, 1, out=sy), 10), bytes_=4 * outer * dim))
    rows.append(_kernel_row("Softmax bwd [128,2048,2048]", timer(lambda: ffk.softmax_backward(sy, sdy, outer, dim, 1, dx=sdx), 10), bytes_=6 * outer * dim))
    total_bytes = sum(r["achieved"] * r["us"] * 1e3 for r in rows)
    total_us = sum(r["us"] for r in rows)
    out = {"value": total_bytes / total_us / 1e3, "unit": "GB/s", "ms_per_step": total_us * 1e-3, "dtype": "bf16",
           "kernels": rows,
           "config": {"workload": "LayerNorm [16384,4096] eps 1e-5, Softmax last dim of [128,2048,2048] logits N(0,4^2), "
                                  "ElementBinary add/mul and Dropout p=0.1 on [16384,4096], fwd+bwd, bf16 (BASELINE "
                                  "config 3); value = algorithmic bytes of all ten launches / their summed time"}}
    if with_cpu:
        import numpy as np
        oracle = _oracle_one_core()
        g = np.random.default_rng(3)
        frac = 64  # 1/64 of the rows of every tensor
        m = M // frac
        xa, xb = oracle.round_bf16(g.standard_normal((m, N))), oracle.round_bf16(g.standard_normal((m, N)))
        gm, be = np.ones(N, np.float32), np.zeros(N, np.float32)
        sm = oracle.round_bf16(g.standard_normal((outer // frac, dim)) * 4)

        def work():
            for op in (28, 29):
                oracle.element_binary_forward(op, xa, xb)
                oracle.element_binary_backward(op, xa, xa, xb)
            oracle.dropout_forward(xa, 0.1, 12345)
            oracle.dropout_backward(xa, 0.1, 12345)
            yy, mu, rs = oracle.layer_norm_forward(xa, gm, be, 1e-5)
            oracle.layer_norm_backward(xb, xa, mu, rs, gm)
            p = oracle.softmax_forward(sm, outer // frac, dim, 1)
            oracle.softmax_backward(p, sm, outer // frac, dim, 1)
        t = _cpu_time(work, 3.0)
        out["cpu_baseline"] = {"value": total_bytes / (t * frac) / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "the same ten operators on 1/64 of the rows of every tensor (%.2f s), time "
                                         "scaled by 64: extrapolated" % t}
    return out


def _zipf(n, vocab, seed, s=1.1):
    import numpy as np
    p = 1.0 / np.arange(1, vocab + 1) ** s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, np.random.default_rng(seed).random(n)), vocab - 1)


def config4(ffk, torch, with_cpu):
    """Embedding gather fwd + scatter-add bwd: V 50257 x D 1024 fp32 table, 65 536 int32 Zipf(1.1) ids, bf16
    output gradient; one DLRM table of 1 M x 128 with 16 384 sum bags of 32 ids (the eight tables are
    eight such calls)."""
    bt = torch.bfloat16
    timer = event_timer(ffk)
    V, D, n = 50257, 1024, 65536
    w = torch.randn((V, D), device="cuda") * 0.02
    ids_np = _zipf(n, V, 0)
    ids = torch.from_numpy(ids_np).to(torch.int32).cuda()
    dy = torch.randn((n, D), device="cuda").to(bt)
    dw = torch.zeros((V, D), device="cuda")
    uniq = int(torch.unique(ids).numel())
    rows = []
    gather_bytes = n * 4 + uniq * D * 4 + n * D * 2
    scatter_bytes = n * 4 + n * D * 2 + uniq * D * 8
    rows.append(_kernel_row("Embedding gather 65536 ids (fp32 table -> bf16)", timer(lambda: ffk.embedding_forward(ids, w, out_dtype=bt), 20), bytes_=gather_bytes))
    rows.append(_kernel_row("Embedding scatter-add, sorted (sort included)", timer(lambda: ffk.embedding_backward(ids, dy, dw, workspace=True), 20), bytes_=scatter_bytes))
    rows.append(_kernel_row("Embedding scatter-add, atomics only", timer(lambda: ffk.embedding_backward(ids, dy, dw, workspace=False), 20), bytes_=scatter_bytes))
    V2, D2, B, bag = 1000000, 128, 16384, 32
    w2 = torch.randn((V2, D2), device="cuda")
    bids_np = _zipf(B * bag, V2, 1).reshape(B, bag)
    bids = torch.from_numpy(bids_np).to(torch.int64).cuda()
    uniq2 = int(torch.unique(bids).numel())
    dy2, dw2 = torch.randn((B, D2), device="cuda"), torch.zeros((V2, D2), device="cuda")
    bag_f = B * bag * 8 + uniq2 * D2 * 4 + B * D2 * 4
    bag_b = B * bag * 8 + B * D2 * 4 + uniq2 * D2 * 8
    rows.append(_kernel_row("DLRM bag fwd, 1M x 128, 16384 bags of 32", timer(lambda: ffk.embedding_forward(bids, w2, aggr=0), 20), bytes_=bag_f))
    rows.append(_kernel_row("DLRM bag bwd, sorted (sort included)", timer(lambda: ffk.embedding_backward(bids, dy2, dw2, aggr=0, workspace=True), 20), bytes_=bag_b))
    rows.append(_kernel_row("DLRM bag bwd, atomics only", timer(lambda: ffk.embedding_backward(bids, dy2, dw2, aggr=0, workspace=False), 20), bytes_=bag_b))
    step_us = rows[0]["us"] + rows[1]["us"] + 8 * (rows[3]["us"] + rows[4]["us"])
    lookups = n + 8 * B * bag
    out = {"value": lookups / (step_us * 1e-6), "unit": "lookups/s", "ms_per_step": step_us * 1e-3, "dtype": "f32",
           "kernels": rows,
           "config": {"workload": "token embedding gather + sorted scatter-add (65 536 ids) and 8 DLRM tables' bag fwd + "
                                  "sorted bwd (8 x 16 384 x 32 ids), BASELINE config 4; one table is timed and counted "
                                  "eight times; bytes count touched rows once (%d and %d unique rows)" % (uniq, uniq2)}}
    if with_cpu:
        oracle = _oracle_one_core()
        wn, dyn = w.cpu().numpy(), dy.float().cpu().numpy()
        sub = 4096  # 1/16 of the token ids
        t_tok = _cpu_time(lambda: (oracle.embedding_forward(ids_np[:sub], wn),
                                   oracle.embedding_backward(ids_np[:sub], dyn[:sub], V)), 2.0)
        w2n, dy2n = w2.cpu().numpy(), dy2.cpu().numpy()
        sb = 1024  # 1/16 of one table's bags
        t_bag = _cpu_time(lambda: (oracle.embedding_forward(bids_np[:sb], w2n, aggr=0),
                                   oracle.embedding_backward(bids_np[:sb], dy2n[:sb], V2, aggr=0)), 2.0)
        t_all = t_tok * (n / sub) + 8 * t_bag * (B / sb)
        out["cpu_baseline"] = {"value": lookups / t_all, "unit": "lookups/s", "cores": 1, "kind": "port",
                               "sample": "oracle gather + scatter-add on 4096 of the token ids (%.3f s) and on 1024 bags of "
                                         "one DLRM table (%.3f s, including clearing its 512 MB gradient), scaled to the "
                                         "whole workload: extrapolated" % (t_tok, t_bag)}
    return out


def config5(ffk, torch, with_cpu):
    """Causal multi-head attention fwd+bwd, bf16: batch 4, seq 4096, 32 heads x 128, with the four projection
    GEMMs [16384,4096] x [4096,4096], as ONE MultiHeadAttention forward + backward call pair (the block);
    the kernels of the block timed one by one stand beside it."""
    bt = torch.bfloat16
    timer = event_timer(ffk)
    B, H, S, D = 4, 32, 4096, 128
    T, E = B * S, H * D
    scale = 1.0 / math.sqrt(D)
    f_attn = 4.0 * B * H * S * S * D * 0.5
    f_gemm = 2.0 * T * E * E
    flops = 3.5 * f_attn + 12 * f_gemm
    # the block: query = key = value = x, so the three input projections are one GEMM
    x = torch.randn((B, S, E), device="cuda").to(bt)
    desc = ffk.mha_desc(B, H, E, E, E, D, D, D, E, S, S, scale, True)
    w = (torch.randn((ffk.lib().ffk_mha_weight_elements(desc),), device="cuda") * 0.02).to(bt)
    dout = torch.randn((B, S, E), device="cuda").to(bt)
    reserve = ffk.mha_reserve(desc, ffk.BF16)
    out, dx, dw = torch.empty_like(x), torch.empty_like(x), torch.empty_like(w)

    def block():
        ffk.mha_forward(desc, x, x, x, w, reserve, out=out)
        ffk.mha_backward(desc, x, dx, x, None, x, None, w, dw, dout, reserve, accumulate=ffk.MHA_OVERWRITE_WEIGHT_GRAD)

    block()
    torch.cuda.synchronize()
    nonfinite = int((~torch.isfinite(out.float())).sum()) + int((~torch.isfinite(dx.float())).sum()) + \
        int((~torch.isfinite(dw.float())).sum())
    t_fwd = timer(lambda: ffk.mha_forward(desc, x, x, x, w, reserve, out=out), 10)
    t_blk = timer(block, 10)
    rows = [_kernel_row("MultiHeadAttention forward (block: QKV projection, causal core, output projection)", t_fwd,
                        flops=f_attn + 4 * f_gemm),
            _kernel_row("MultiHeadAttention forward + backward (block)", t_blk, flops=flops)]
    step_us = rows[1]["us"]
    del x, w, dout, reserve, out, dx, dw
    q, k, v, do = (torch.randn((B, S, H, D), device="cuda").to(bt) for _ in range(4))
    o, lse = ffk.attention_forward(q, k, v, scale, True)
    rows += [_kernel_row("attention fwd, causal", timer(lambda: ffk.attention_forward(q, k, v, scale, True), 10), flops=f_attn),
             _kernel_row("attention bwd, causal", timer(lambda: ffk.attention_backward(q, k, v, o, do, lse, scale, True), 10), flops=2.5 * f_attn)]
    del q, k, v, do, o
    X = torch.randn((T, E), device="cuda").to(bt)
    W = (torch.randn((E, E), device="cuda") * 0.02).to(bt)
    Y, dW = torch.empty((T, E), device="cuda", dtype=bt), torch.empty((E, E), device="cuda", dtype=bt)
    rows.append(_kernel_row("projection forward  NT M16384 N4096 K4096", timer(lambda: ffk.gemm(X, W, Y, False, True), 10), flops=f_gemm))
    rows.append(_kernel_row("projection dX       NN M16384 N4096 K4096", timer(lambda: ffk.gemm(X, W, Y, False, False), 10), flops=f_gemm))
    rows.append(_kernel_row("projection dW       TN M4096 N4096 K16384", timer(lambda: ffk.gemm(X, Y, dW, True, False), 10), flops=f_gemm))
    out = {"value": T / (step_us * 1e-6), "unit": "tokens/s", "ms_per_step": step_us * 1e-3, "dtype": "bf16",
           "kernels": rows, "step_tflops": flops / step_us / 1e6, "nonfinite": nonfinite,
           "config": {"workload": "causal multi-head attention fwd+bwd as one block, batch 4, seq 4096, 32 heads x 128, with "
                                  "its four projection GEMMs [16384,4096]x[4096,4096] (BASELINE config 5): one step = "
                                  "ffk_mha_forward + ffk_mha_backward on one tensor as query, key and value; the rows "
                                  "after the first two time the block's kernels one by one",
                      "algorithmic_tflop_per_step": flops / 1e12}}
    if with_cpu:
        import numpy as np
        oracle = _oracle_one_core()
        g = np.random.default_rng(5)
        s_sub = 1024  # one (batch, head) at a quarter of the sequence: cost is quadratic in the length
        qs, ks, vs, dos = (oracle.round_bf16(g.standard_normal((1, s_sub, 1, D))) for _ in range(4))
        t0 = time.perf_counter()
        oracle.attention_forward(qs, ks, vs, scale, True, bf16_mode=True)
        oracle.attention_backward(qs, ks, vs, dos, scale, True)
        t_attn = (time.perf_counter() - t0) * (S / s_sub) ** 2 * B * H
        m_sub = 32  # rows of the projection input
        Xs, Ws = oracle.round_bf16(g.standard_normal((m_sub, E))), oracle.round_bf16(g.standard_normal((E, E)) * 0.02)
        t0 = time.perf_counter()
        oracle.gemm_f64(Xs, Ws, False, True)
        t_gemm = (time.perf_counter() - t0) * (T / m_sub) * 12
        out["cpu_baseline"] = {"value": T / (t_attn + t_gemm), "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": "oracle attention fwd+bwd on one (batch, head) at seq 1024, scaled by 16 x 128; one "
                                         "oracle GEMM of 32 rows scaled to the twelve [16384,4096,4096] products: extrapolated "
                                         "(%.0f s + %.0f s of CPU time for the whole workload)" % (t_attn, t_gemm)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5],
                    help="BASELINE configuration to measure (2 = the headline transformer layer)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-seconds", type=float, default=SETTLE_SECONDS,
                    help="untimed steps run for this long before the warm-up steps (0: none)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant kernel's timing loop and a 256 MiB calibration "
                         "copy (for rocprofv3 counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every kernel here runs on a single MI355X and no "
                 "collective is built; run with --gpus 1")
    import torch
    ffk = _load("flexflow_train_amd", os.path.join(ROOT, "flexflow-train_amd", "__init__.py"))
    ffk.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.roofline_only:
        print(json.dumps({"roofline": time_dominant_kernel(ffk, torch, CFG, calibration_copy=True)}))
        return
    if args.config != 2:
        fn = {1: config1, 3: config3, 4: config4, 5: config5}[args.config]
        body = fn(ffk, torch, not args.no_cpu_baseline)
        out = {"metric": "per-kernel time and fraction of the HBM / MFMA roofline, BASELINE config %d" % args.config,
               "n_gpus": 1, "steps": 1, "warmup": 0, "higher_is_better": True, "scaling": "weak",
               "vs_baseline": None, "data": "synthetic"}
        out.update(body)
        print(json.dumps(out))
        return
    st = make_device_state(ffk, torch, CFG)
    check = check_before_timing(ffk, torch, st)
    settled = settle_clocks(lambda: step(ffk, st), seconds=args.settle_seconds) if args.settle_seconds > 0 else 0
    for _ in range(args.warmup):
        step(ffk, st)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(ffk, st)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tokens = CFG["batch"] * CFG["seq"]
    ms = dt / args.steps * 1e3
    roof = time_dominant_kernel(ffk, torch, CFG)
    out = {
        "metric": "transformer-layer fwd+bwd tokens/s on 1 GPU",
        "value": tokens / (dt / args.steps),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "transformer encoder layer fwd+bwd, bf16/fp32-accumulate: batch 8, "
                               "seq 512, d_model 1024, 16 heads, FFN 4096 GELU, pre-LayerNorm, "
                               "dropout 0.1 (BASELINE config 2)",
                   "tokens_per_step": tokens, "algorithmic_gflop_per_step": 335.0},
        "step_tflops": 335.0e9 / (dt / args.steps) / 1e12,
        "clock_settle": {"untimed_steps_before_warmup": settled, "seconds": args.settle_seconds,
                         "why": "the shader clock ramps for tens of ms after idle; value is the steady state"},
        "check": check,
        "roofline": roof,
        "device_copy": measure_device_copy(ffk, torch),
        "mfma_loop": measure_mfma_loop(ffk, torch),
    }
    out["roofline"]["frac_of_measured_mfma_loop"] = roof["achieved"] / out["mfma_loop"]["TFLOP/s"]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(CFG)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
