"""Per-kernel measurements at the shapes of the baseline configurations.

    python kernel_bench.py [group ...]

Groups: gemm (config 2 and config 5 projection GEMMs), bandwidth (config 3:
LayerNorm, Softmax, ElementBinary, Dropout, plus GELU), embedding (config 4:
token gather / scatter-add, DLRM bags), attention (config 5 and the config 2
core), update (optimizer steps, Cast and loss backward over a parameter-sized
buffer), shape (Concat, Transpose, Gather).  Every line gives the mean launch time over the timed iterations
(HIP events on torch's current stream, which is the stream the entry points are
given) and the ALGORITHMIC bytes or flops of the op divided by that time,
against 8 TB/s HBM or the 2.5 PFLOP/s dense bf16 MFMA peak.  Inputs are
synthetic (seeded normal / Zipf) and already resident in HBM.
"""
import importlib.util
import math
import time
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("flexflow_train_amd",
                                               os.path.join(HERE, "flexflow-train_amd", "__init__.py"))
ffk = importlib.util.module_from_spec(_spec)
sys.modules["flexflow_train_amd"] = ffk
_spec.loader.exec_module(ffk)
BT = torch.bfloat16
HBM_PEAK = 8e12
MFMA_PEAK = 2.5e15


SETTLE_SECONDS = 0.1   # --settle=S on the command line; 0 for counter runs, whose clock does not matter


def timeit(fn, iters=20, warm=5, settle=None):
    settle = SETTLE_SECONDS if settle is None else settle
    # at least `warm` calls and `settle` seconds of untimed load first: the shader clock takes tens
    # of milliseconds of sustained work to reach the state it then holds, and the first launches
    # after an idle spell (building the next case's tensors is one) run 10-20% slow
    n, t0 = 0, time.perf_counter()
    while n < warm or time.perf_counter() - t0 < settle:
        fn()
        n += 1
        if n % 10 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters * 1e-3


def report(name, t, bytes_=None, flops=None):
    msg = "%-46s %9.1f us" % (name, t * 1e6)
    if bytes_:
        msg += "  %8.1f GB/s    (%5.1f%% of 8 TB/s)" % (bytes_ / t / 1e9, bytes_ / t / HBM_PEAK * 100)
    if flops:
        msg += "  %8.1f TFLOP/s (%5.1f%% of 2.5 PFLOP/s)" % (flops / t / 1e12, flops / t / MFMA_PEAK * 100)
    print(msg, flush=True)


def zipf(n, vocab, s=1.1, seed=0):
    p = 1.0 / np.arange(1, vocab + 1) ** s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, np.random.default_rng(seed).random(n)), vocab - 1)


def bench_gemm():
    # (M, N, K, trans_a, trans_b): forward (NT), input-gradient (NN) and
    # weight-gradient (TN) GEMMs of the config 2 layer, then config 5's projections
    shapes = [(4096, 3072, 1024, 0, 1), (4096, 1024, 1024, 0, 1), (4096, 4096, 1024, 0, 1), (4096, 1024, 4096, 0, 1),
              (4096, 4096, 1024, 0, 0), (4096, 1024, 4096, 0, 0), (4096, 1024, 3072, 0, 0), (4096, 1024, 1024, 0, 0),
              (1024, 4096, 4096, 1, 0), (4096, 1024, 4096, 1, 0), (3072, 1024, 4096, 1, 0), (1024, 1024, 4096, 1, 0),
              (16384, 4096, 4096, 0, 1), (16384, 4096, 4096, 0, 0), (4096, 4096, 16384, 1, 0)]
    for (M, N, K, ta, tb) in shapes:
        A = torch.randn((K, M) if ta else (M, K), device="cuda").to(BT)
        B = torch.randn((N, K) if tb else (K, N), device="cuda").to(BT)
        C = torch.empty((M, N), device="cuda", dtype=BT)
        t = timeit(lambda: ffk.gemm(A, B, C, bool(ta), bool(tb)))
        report("gemm bf16 M%d N%d K%d %s%s" % (M, N, K, "T" if ta else "N", "T" if tb else "N"), t,
               flops=2.0 * M * N * K)
        if K >= 1024 and M % 256 == 0 and N % 256 == 0 and (M // 256) * (N // 256) >= 192:
            # the eight-wave 256x256 kernel that the one-wave-per-SIMD kernel replaced at these sizes
            ffk.set_option(ffk.OPTION_GEMM_VARIANT, 256)
            try:
                t = timeit(lambda: ffk.gemm(A, B, C, bool(ta), bool(tb)))
            finally:
                ffk.set_option(ffk.OPTION_GEMM_VARIANT, 0)
            report("  previous kernel (8 waves, 4 x 32-deep stages)", t, flops=2.0 * M * N * K)
        # the vendor library on the same operands (hipBLASLt, reached through torch.matmul), for scale
        At, Bt = (A.t() if ta else A), (B.t() if tb else B)
        t = timeit(lambda: torch.matmul(At, Bt, out=C))
        report("  vendor library (torch.matmul)", t, flops=2.0 * M * N * K)


def bench_gemm_fp32():
    # the reference's own data type: Linear shapes of the config 2 layer in fp32 (v_mfma_f32_32x32x2f32,
    # 157.3 TFLOP/s dense peak), and a large square
    for (M, N, K, ta, tb) in [(4096, 4096, 1024, 0, 1), (4096, 1024, 4096, 0, 1), (4096, 1024, 4096, 0, 0),
                              (1024, 4096, 4096, 1, 0), (8192, 8192, 8192, 0, 1)]:
        A = torch.randn((K, M) if ta else (M, K), device="cuda")
        B = torch.randn((N, K) if tb else (K, N), device="cuda")
        C = torch.empty((M, N), device="cuda")
        iters = 5 if M * N * K > 2 ** 36 else 20
        t = timeit(lambda: ffk.gemm(A, B, C, bool(ta), bool(tb)), iters=iters)
        print("%-46s %9.1f us  %8.1f TFLOP/s (%5.1f%% of 157.3 TFLOP/s)  %s" % (
            "gemm fp32 M%d N%d K%d %s%s" % (M, N, K, "T" if ta else "N", "T" if tb else "N"), t * 1e6,
            2.0 * M * N * K / t / 1e12, 2.0 * M * N * K / t / 157.3e12 * 100,
            ffk.gemm_kernel_name(ffk.FLOAT, bool(ta), bool(tb), M, N, K)), flush=True)
        At, Bt = (A.t() if ta else A), (B.t() if tb else B)
        t = timeit(lambda: torch.matmul(At, Bt, out=C), iters=iters)
        print("%-46s %9.1f us  %8.1f TFLOP/s (%5.1f%% of 157.3 TFLOP/s)" % (
            "  vendor library (torch.matmul)", t * 1e6, 2.0 * M * N * K / t / 1e12, 2.0 * M * N * K / t / 157.3e12 * 100), flush=True)


def bench_fused_linear():
    # Config 2's feed-forward block (4096 tokens, 1024 -> 4096 -> 1024): each Linear with the
    # element-wise operators around it as separate launches and on the GEMM's tile store
    T, E, F, rate, seed = 4096, 1024, 4096, 0.1, 2024
    L = ffk.lib()
    st = ffk.current_stream()
    p = ffk.ptr
    x = torch.randn((T, E), device="cuda").to(BT)
    w1 = (torch.randn((F, E), device="cuda") * 0.03).to(BT)
    b1 = torch.zeros((F,), device="cuda", dtype=BT)
    w2 = (torch.randn((E, F), device="cuda") * 0.015).to(BT)
    b2 = torch.zeros((E,), device="cuda", dtype=BT)
    h, act = torch.empty((T, F), device="cuda", dtype=BT), torch.empty((T, F), device="cuda", dtype=BT)
    y, out = torch.empty((T, E), device="cuda", dtype=BT), torch.empty((T, E), device="cuda", dtype=BT)
    dy = torch.randn((T, E), device="cuda").to(BT)
    dact, dh = torch.empty_like(act), torch.empty_like(h)
    need = L.ffk_linear_backward_workspace_bytes(ffk.BF16, ffk.ACT_NONE, 0, T, E)
    ws = torch.empty((max(need, 1),), dtype=torch.uint8, device="cuda")

    def up_separate():
        ffk.linear_forward(x, w1, b1, ffk.ACT_NONE, h)
        ffk.check(L.ffk_gelu_dropout_forward(st, ffk.BF16, p(h), p(act), T * F, rate, seed, 0))

    def up_tail():
        ffk.check(L.ffk_linear_gelu_dropout_forward(st, ffk.BF16, p(x), p(h), p(act), p(w1), p(b1), T, E, F,
                                                    rate, seed, 0))

    def down_separate():
        ffk.linear_forward(act, w2, b2, ffk.ACT_NONE, y)
        ffk.check(L.ffk_dropout_add_forward(st, ffk.BF16, p(y), p(x), p(out), T * E, rate, seed, 0))

    def down_tail():
        ffk.check(L.ffk_linear_dropout_add_forward(st, ffk.BF16, p(act), p(x), p(out), p(w2), p(b2), T, F, E,
                                                   rate, seed, 0))

    def grad_separate():
        ffk.check(L.ffk_linear_backward(st, ffk.BF16, ffk.ACT_NONE, 0, None, p(dy), p(act), p(dact), p(w2), None,
                                        None, T, F, E, p(ws), need, 0))
        ffk.check(L.ffk_dropout_gelu_backward(st, ffk.BF16, p(dact), p(h), p(dh), T * F, rate, seed, 0))

    def grad_tail():
        ffk.check(L.ffk_linear_backward_dropout_gelu(st, ffk.BF16, p(dy), p(act), p(h), p(dh), p(w2), None, None,
                                                     T, F, E, p(ws), need, 0, rate, seed, 0))

    flops = 2.0 * T * E * F
    up_separate()  # h, act hold finite values for the backward timings
    for name, fn in [("Linear 1024->4096, GELU+Dropout: 2 launches", up_separate),
                     ("Linear 1024->4096, GELU+Dropout: on the tile store", up_tail),
                     ("Linear 4096->1024, Dropout+add: 2 launches", down_separate),
                     ("Linear 4096->1024, Dropout+add: on the tile store", down_tail),
                     ("Linear 4096->1024 dX, Dropout/GELU bwd: 2 launches", grad_separate),
                     ("Linear 4096->1024 dX, Dropout/GELU bwd: tile store", grad_tail)]:
        report(name, timeit(fn), flops=flops)


def bench_bandwidth():
    n = 16384 * 4096
    a = torch.randn(n, device="cuda").to(BT)
    b = torch.randn(n, device="cuda").to(BT)
    o = torch.empty_like(a)
    da, db = torch.zeros_like(a), torch.zeros_like(a)
    t = timeit(lambda: o.copy_(a))
    report("device copy (torch) [16384,4096] bf16", t, bytes_=4 * n)
    t = timeit(lambda: ffk.element_binary_forward(ffk.OP["EW_ADD"], a, b, out=o))
    report("ElementBinary add fwd", t, bytes_=6 * n)
    t = timeit(lambda: ffk.element_binary_forward(ffk.OP["EW_MUL"], a, b, out=o))
    report("ElementBinary mul fwd", t, bytes_=6 * n)
    t = timeit(lambda: ffk.element_binary_backward(ffk.OP["EW_ADD"], o, a, b, da, db))
    report("ElementBinary add bwd", t, bytes_=6 * n)
    t = timeit(lambda: ffk.element_binary_backward(ffk.OP["EW_MUL"], o, a, b, da, db))
    report("ElementBinary mul bwd", t, bytes_=10 * n)
    t = timeit(lambda: ffk.element_unary_forward(ffk.OP["GELU"], a, out=o))
    report("ElementUnary GELU fwd", t, bytes_=4 * n)
    t = timeit(lambda: ffk.element_unary_backward(ffk.OP["GELU"], o, b, a, da))
    report("ElementUnary GELU bwd", t, bytes_=6 * n)
    t = timeit(lambda: ffk.dropout_forward(a, 0.1, 12345, out=o))
    report("Dropout p=0.1 fwd", t, bytes_=4 * n)
    t = timeit(lambda: ffk.dropout_backward(a, 0.1, 12345, dx=o))
    report("Dropout p=0.1 bwd", t, bytes_=4 * n)
    for (M, N) in [(16384, 4096), (4096, 1024)]:
        x = torch.randn((M, N), device="cuda").to(BT)
        dy = torch.randn((M, N), device="cuda").to(BT)
        g = torch.ones(N, device="cuda", dtype=BT)
        beta = torch.zeros(N, device="cuda", dtype=BT)
        y = torch.empty_like(x)
        mean, rstd = torch.empty(M, device="cuda"), torch.empty(M, device="cuda")
        dx, dg, dbeta = torch.empty_like(x), torch.empty_like(g), torch.empty_like(beta)
        ws = torch.empty(ffk.lib().ffk_layer_norm_backward_workspace_bytes(M, N), dtype=torch.uint8, device="cuda")
        t = timeit(lambda: ffk.layer_norm_forward(x, g, beta, 1e-5, y, mean, rstd))
        report("LayerNorm fwd [%d,%d]" % (M, N), t, bytes_=4 * M * N)
        t = timeit(lambda: ffk.layer_norm_backward(dy, x, mean, rstd, g, dx, dg, dbeta, workspace=ws))
        report("LayerNorm bwd [%d,%d]" % (M, N), t, bytes_=6 * M * N)
    outer, dim = 128 * 2048, 2048
    x = (torch.randn((outer, dim), device="cuda") * 4).to(BT)
    y = torch.empty_like(x)
    dy = torch.randn((outer, dim), device="cuda").to(BT)
    dx = torch.empty_like(x)
    t = timeit(lambda: ffk.softmax_forward(x, outer, dim, 1, out=y), iters=10)
    report("Softmax fwd [128,2048,2048]", t, bytes_=4 * outer * dim)
    t = timeit(lambda: ffk.softmax_backward(y, dy, outer, dim, 1, dx=dx), iters=10)
    report("Softmax bwd [128,2048,2048]", t, bytes_=6 * outer * dim)


def bench_embedding():
    V, D, n = 50257, 1024, 65536
    w = torch.randn((V, D), device="cuda") * 0.02
    ids = torch.from_numpy(zipf(n, V)).to(torch.int32).cuda()
    dy = torch.randn((n, D), device="cuda").to(BT)
    dw = torch.zeros((V, D), device="cuda")
    uniq = int(torch.unique(ids).numel())
    t = timeit(lambda: ffk.embedding_forward(ids, w, out_dtype=BT))
    report("Embedding gather 65536 ids (fp32 -> bf16)", t, bytes_=n * 4 + uniq * D * 4 + n * D * 2)
    scatter_bytes = n * 4 + n * D * 2 + uniq * D * 8
    t = timeit(lambda: ffk.embedding_backward(ids, dy, dw, workspace=True))
    report("Embedding scatter-add, sorted (with sort)", t, bytes_=scatter_bytes)
    t = timeit(lambda: ffk.embedding_backward(ids, dy, dw, workspace=False))
    report("Embedding scatter-add, atomics only", t, bytes_=scatter_bytes)
    V, D, B, bag = 1000000, 128, 16384, 32
    w = torch.randn((V, D), device="cuda")
    ids = torch.from_numpy(zipf(B * bag, V)).to(torch.int64).cuda().view(B, bag)
    uniq = int(torch.unique(ids).numel())
    t = timeit(lambda: ffk.embedding_forward(ids, w, aggr=0))
    report("DLRM bag fwd 1M x 128, 16384 bags of 32", t, bytes_=B * bag * 8 + uniq * D * 4 + B * D * 4)
    dy = torch.randn((B, D), device="cuda")
    dw = torch.zeros((V, D), device="cuda")
    bag_bytes = B * bag * 8 + B * D * 4 + uniq * D * 8
    t = timeit(lambda: ffk.embedding_backward(ids, dy, dw, aggr=0, workspace=True))
    report("DLRM bag bwd, sorted (with sort)", t, bytes_=bag_bytes)
    t = timeit(lambda: ffk.embedding_backward(ids, dy, dw, aggr=0, workspace=False))
    report("DLRM bag bwd, atomics only", t, bytes_=bag_bytes)


def bench_attention():
    for (B, H, S, D, causal) in [(4, 32, 4096, 128, True), (4, 32, 4096, 128, False), (8, 16, 512, 64, False)]:
        q, k, v, do = (torch.randn((B, S, H, D), device="cuda").to(BT) for _ in range(4))
        scale = 1.0 / math.sqrt(D)
        o, lse = ffk.attention_forward(q, k, v, scale, causal)
        f = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0)
        t = timeit(lambda: ffk.attention_forward(q, k, v, scale, causal), iters=10)
        report("attention fwd B%d H%d S%d D%d causal=%d" % (B, H, S, D, causal), t, flops=f)
        t = timeit(lambda: ffk.attention_backward(q, k, v, o, do, lse, scale, causal), iters=10)
        report("attention bwd B%d H%d S%d D%d causal=%d" % (B, H, S, D, causal), t, flops=2.5 * f)
        # the other forward kernel at this size: 32 query rows per wavefront, then 64 whatever the size
        try:
            ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 1)
            t = timeit(lambda: ffk.attention_forward(q, k, v, scale, causal), iters=10)
            report("  forward, 32 query rows per wavefront", t, flops=f)
            ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 2)
            t = timeit(lambda: ffk.attention_forward(q, k, v, scale, causal), iters=10)
            report("  forward, 64 query rows per wavefront", t, flops=f)
        finally:
            ffk.set_option(ffk.OPTION_ATTENTION_VARIANT, 0)
    # the kernels for every other head size (multiples of 8 up to 256, value heads of their own
    # size): 32 query rows per wavefront, head size padded to the next of 32 / 64 / 128 / 256
    for (B, H, S, Dq, Dv, dt) in [(4, 8, 2048, 256, 256, BT), (4, 16, 2048, 96, 64, BT), (4, 16, 2048, 80, 80, BT),
                                  (2, 8, 1024, 256, 256, torch.float32), (2, 8, 1024, 64, 64, torch.float32)]:
        q, k = (torch.randn((B, S, H, Dq), device="cuda").to(dt) for _ in range(2))
        v, do = (torch.randn((B, S, H, Dv), device="cuda").to(dt) for _ in range(2))
        scale = 1.0 / math.sqrt(Dq)
        o, lse = ffk.attention_forward(q, k, v, scale, False)
        f = 2.0 * B * H * S * S * (Dq + Dv)
        tag = "B%d H%d S%d Dq%d Dv%d %s" % (B, H, S, Dq, Dv, "bf16" if dt == BT else "fp32")
        t = timeit(lambda: ffk.attention_forward(q, k, v, scale, False), iters=10)
        report("attention fwd " + tag, t, flops=f)
        t = timeit(lambda: ffk.attention_backward(q, k, v, o, do, lse, scale, False), iters=10)
        report("attention bwd " + tag, t, flops=2.5 * f)


def bench_small_linear():
    # fp32 Linear at sizes where a launch costs more than the arithmetic: the forward is one
    # launch of 64x64 tiles, the whole backward (dX, dW, bias sums) one launch
    for (batch, in_dim, out_dim, act) in [(32, 64, 128, ffk.ACT_RELU), (256, 256, 256, ffk.ACT_NONE), (1024, 512, 512, ffk.ACT_RELU)]:
        x = torch.randn((batch, in_dim), device="cuda")
        w = torch.randn((out_dim, in_dim), device="cuda") * 0.1
        b = torch.randn((out_dim,), device="cuda")
        y = torch.empty((batch, out_dim), device="cuda")
        dy = torch.randn((batch, out_dim), device="cuda")
        dx, dw, db = torch.empty_like(x), torch.empty_like(w), torch.empty_like(b)
        ffk.linear_forward(x, w, b, act, out=y)
        t = timeit(lambda: ffk.linear_forward(x, w, b, act, out=y), iters=50)
        report("Linear fp32 fwd [%d,%d]x[%d,%d]^T act %d" % (batch, in_dim, out_dim, in_dim, act), t, flops=2.0 * batch * in_dim * out_dim)
        ws = torch.empty((max(1, ffk.lib().ffk_linear_backward_workspace_bytes(ffk.FLOAT, act, 1, batch, out_dim)),),
                         dtype=torch.uint8, device="cuda")
        t = timeit(lambda: ffk.linear_backward(y, dy, x, w, dx, dw, db, act, workspace=ws), iters=50)
        report("Linear fp32 bwd (one launch)", t, flops=4.0 * batch * in_dim * out_dim)


def bench_update():
    # 64 Mi parameters: a few encoder layers' worth; the config 2 layer alone (12.6 M)
    # is over in a handful of microseconds
    n = 64 << 20
    w = torch.randn(n, device="cuda")
    g = torch.randn(n, device="cuda")
    gb = g.to(BT)
    v = torch.zeros(n, device="cuda")
    m = torch.zeros(n, device="cuda")
    wl = torch.empty(n, device="cuda", dtype=BT)
    t = timeit(lambda: ffk.sgd_update(w, g, 0.01))
    report("SGD plain, fp32 grad", t, bytes_=12 * n)
    t = timeit(lambda: ffk.sgd_update(w, g, 0.01, 0.9, True, 1e-4, sgd_v=v))
    report("SGD momentum+nesterov, fp32 grad", t, bytes_=20 * n)
    t = timeit(lambda: ffk.sgd_update(w, gb, 0.01, 0.9, True, 1e-4, sgd_v=v, weight_lowp=wl))
    report("SGD momentum, bf16 grad, bf16 weight copy out", t, bytes_=20 * n)
    t = timeit(lambda: ffk.adam_update(w, g, m, v, 1e-3, weight_decay=1e-2))
    report("Adam, fp32 grad", t, bytes_=28 * n)
    t = timeit(lambda: ffk.adam_update(w, gb, m, v, 1e-3, weight_decay=1e-2, weight_lowp=wl))
    report("Adam, bf16 grad, bf16 weight copy out", t, bytes_=28 * n)
    t = timeit(lambda: ffk.cast_forward(w, wl))
    report("Cast fp32 -> bf16", t, bytes_=6 * n)
    t = timeit(lambda: ffk.cast_backward(wl, g))
    report("Cast backward bf16 -> fp32 (accumulating)", t, bytes_=10 * n)
    samples, classes = 4096, 50257
    logit = torch.rand((samples, classes), device="cuda")
    label = torch.randint(0, classes, (samples,), device="cuda", dtype=torch.int32)
    out = torch.empty_like(logit)
    t = timeit(lambda: ffk.sparse_categorical_crossentropy_loss_backward(logit, label, samples, classes, 1,
                                                                         1.0 / samples, out=out))
    report("sparse CCE loss backward [4096, 50257]", t, bytes_=8 * samples * classes)


def bench_shape():
    # the data-movement operators around the hot path: DLRM's interaction concat (27 parts of
    # [16384, 128]) and a wide one, head split / merge transposes of configs 2 and 5, a 2-D
    # transpose, a gather along the vocabulary (one logit per token)
    parts = [torch.randn((16384, 128), device="cuda").to(BT) for _ in range(27)]
    cat = torch.empty((16384, 27 * 128), device="cuda", dtype=BT)
    grads = [torch.empty_like(p) for p in parts]
    t = timeit(lambda: ffk.concat_forward(parts, 1, out=cat))
    report("Concat 27 x [16384,128] bf16 fwd", t, bytes_=2 * cat.numel() * 2)
    t = timeit(lambda: ffk.concat_backward(cat, grads, 1, accumulate=False))
    report("Concat 27 x [16384,128] bf16 bwd (store)", t, bytes_=2 * cat.numel() * 2)
    t = timeit(lambda: ffk.concat_backward(cat, grads, 1, accumulate=True))
    report("Concat 27 x [16384,128] bf16 bwd (add)", t, bytes_=3 * cat.numel() * 2)
    wide = [torch.randn((4096, 4096), device="cuda").to(BT) for _ in range(4)]
    wcat = torch.empty((4096, 16384), device="cuda", dtype=BT)
    t = timeit(lambda: ffk.concat_forward(wide, 1, out=wcat))
    report("Concat 4 x [4096,4096] bf16 fwd", t, bytes_=2 * wcat.numel() * 2)
    for (B, S, H, D) in [(8, 512, 16, 64), (4, 4096, 32, 128)]:
        x = torch.randn((B, S, H, D), device="cuda").to(BT)
        y = torch.empty((B, H, S, D), device="cuda", dtype=BT)
        t = timeit(lambda: ffk.transpose_forward(x, (0, 2, 1, 3), out=y))
        report("Transpose [%d,%d,%d,%d] -> (0,2,1,3) bf16" % (B, S, H, D), t, bytes_=2 * x.numel() * 2)
    x = torch.randn((16384, 4096), device="cuda").to(BT)
    y = torch.empty((4096, 16384), device="cuda", dtype=BT)
    t = timeit(lambda: ffk.transpose_forward(x, (1, 0), out=y))
    report("Transpose [16384,4096] -> (1,0) bf16", t, bytes_=2 * x.numel() * 2)
    g = torch.zeros((16384, 4096), device="cuda", dtype=BT)
    t = timeit(lambda: ffk.transpose_backward(y, g, (1, 0), accumulate=True))
    report("Transpose backward (adds) [16384,4096] bf16", t, bytes_=3 * x.numel() * 2)
    xf = torch.randn((16384, 4096), device="cuda")
    yf = torch.empty((4096, 16384), device="cuda")
    t = timeit(lambda: ffk.transpose_forward(xf, (1, 0), out=yf))
    report("Transpose [16384,4096] -> (1,0) fp32", t, bytes_=2 * xf.numel() * 4)
    logits = torch.randn((16384, 50257), device="cuda")
    idx = torch.randint(0, 50257, (16384, 1), device="cuda", dtype=torch.int64)
    out = torch.empty((16384, 1), device="cuda")
    t = timeit(lambda: ffk.gather_forward(logits, idx, 1, out=out))
    report("Gather 1 of 50257 per row, 16384 rows (fp32)", t, bytes_=16384 * (8 + 64 + 4))
    idx2 = torch.randint(0, 4096, (16384, 1024), device="cuda", dtype=torch.int32)
    src = torch.randn((16384, 4096), device="cuda")
    out2 = torch.empty((16384, 1024), device="cuda")
    t = timeit(lambda: ffk.gather_forward(src, idx2, 1, out=out2))
    report("Gather [16384,4096] -> [16384,1024] along dim 1 (fp32)", t, bytes_=idx2.numel() * (4 + 4) + src.numel() * 4)
    gin = torch.zeros_like(src)
    t = timeit(lambda: ffk.gather_backward(out2, idx2, gin, 1))
    report("Gather backward (row sums in LDS) [16384,1024] -> [16384,4096]", t, bytes_=idx2.numel() * (4 + 4 + 8))


GROUPS = dict(gemm=bench_gemm, gemm_fp32=bench_gemm_fp32, fused_linear=bench_fused_linear, bandwidth=bench_bandwidth, embedding=bench_embedding, attention=bench_attention, small_linear=bench_small_linear,
              update=bench_update, shape=bench_shape)

if __name__ == "__main__":
    ffk.lib()
    assert torch.cuda.is_available(), "kernel_bench.py needs a GPU"
    names = []
    for a in sys.argv[1:]:
        if a.startswith("--settle="):
            SETTLE_SECONDS = float(a.split("=", 1)[1])
        else:
            names.append(a)
    for name in names or list(GROUPS):
        GROUPS[name]()
