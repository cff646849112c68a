"""Headline benchmark: transformer encoder layer forward+backward tokens/s on
one MI355X (BASELINE config 2: bf16, batch 8, seq 512, d_model 1024, 16 heads,
FFN 4096 GELU, pre-LayerNorm, dropout 0.1; synthetic N(0,1) activations and
N(0,0.02) weights).

    python bench.py --gpus 1 --steps K --warmup W

Prints one JSON line.  Besides the whole-step throughput it reports
  roofline     : the dominant kernel (the bf16 MFMA GEMM of the first FFN
                 projection, [4096,1024] x [4096,1024]^T), timed live with HIP
                 events on the launch stream, against the 2.5 PFLOP/s dense
                 bf16 MFMA peak;
  cpu_baseline : the CPU oracle's restatement of the same layer, timed on the
                 host cores on a bounded sample (one sequence of 128 tokens of
                 the same layer), scaled to tokens/s.
"""
import argparse
import importlib.util
import json
import os
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


CFG = dict(batch=8, seq=512, d_model=1024, heads=16, d_ff=4096, p=0.1, seed=20240, eps=1e-5,
           scale=1.0 / 8.0, causal=False, pre_ln=True, gelu=True)
MFMA_BF16_PEAK_TFLOPS = 2500.0


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


# HBM bytes one launch of the dominant kernel moves, from `rocprofv3 --pmc
# FETCH_SIZE` and `--pmc WRITE_SIZE` runs of `bench.py --roofline-only`, each
# counter scaled by what it reads for the 256 MiB copy kernel that the same run
# launches (profiles/ffn_up_gemm_hbm_traffic.md holds the runs and the factors).
DOMINANT_KERNEL_TRAFFIC_BYTES = 84141236  # 48.2 MiB fetched + 32 MiB written; 48 MiB algorithmic


def time_dominant_kernel(ffk, torch, cfg, iters=50, calibration_copy=False):
    """The FFN up-projection (Linear forward with bias, [4096,1024] x
    [4096,1024]^T) at its real shape, HIP events on the stream the kernel is
    launched on.  calibration_copy also launches one element-wise copy of
    256 MiB (read 256 MiB, write 256 MiB) for scaling HBM traffic counters."""
    import ctypes
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
    lib = ffk.lib()
    stream = ffk.current_stream()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    ffk.check(lib.ffk_event_create(ctypes.byref(e0)))
    ffk.check(lib.ffk_event_create(ctypes.byref(e1)))
    for _ in range(5):
        ffk.linear_forward(A, B, bias, ffk.ACT_NONE, C)
    ffk.check(lib.ffk_event_record(e0, stream))
    for _ in range(iters):
        ffk.linear_forward(A, B, bias, ffk.ACT_NONE, C)
    ffk.check(lib.ffk_event_record(e1, stream))
    ffk.check(lib.ffk_event_synchronize(e1))
    ms = ctypes.c_float()
    ffk.check(lib.ffk_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    lib.ffk_event_destroy(e0)
    lib.ffk_event_destroy(e1)
    sec = ms.value / iters * 1e-3
    flops = 2.0 * T * F * E
    return dict(bound="mfma", achieved=flops / sec / 1e12, peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s",
                frac=flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                traffic=DOMINANT_KERNEL_TRAFFIC_BYTES,
                kernel="gemm_bf16_pipe_kernel<256,256,128,64,32,4,1,false,true,0,false> "
                       "(FFN up-projection, M%d N%d K%d, bias)" % (T, F, E),
                us_per_launch=sec * 1e6)


def cpu_baseline(cfg):
    """The oracle's layer on a bounded sample: 1 sequence x 128 tokens of the
    same layer (same widths), single thread, scaled to tokens/s."""
    import numpy as np
    oracle = _load("ffk_oracle", os.path.join(ROOT, "oracle", "oracle.py"))
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    st = make_device_state(ffk, torch, CFG)
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
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(CFG)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
