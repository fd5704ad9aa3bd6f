#!/usr/bin/env python3
"""Benchmark of the Winograd-ReLU conv layer (winograd2x2_imTrans + winograd2x2_conv) on one MI355X.

A step is one pass of the hot path over one synthetic batch, inputs resident in HBM:
  TI = winograd2x2_imTrans(x, relu)      [B,H,W,C] -> [16,B,nH,nW,C]
  y  = winograd2x2_conv(TI, W)           [16,B,nH,nW,C] x [16,C,K] -> [B,2nH,2nW,K]
Default workload: ResNet-18 conv3 stage, N=64, 28x28x128 -> 128, fp32, Winograd-domain ReLU
on, weights magnitude-pruned to 20 % density (values only: the contraction is dense, as in
the reference, winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:80-85).

Prints one JSON line.  `value` is the effective direct-convolution rate 18*N*H*W*C*K / step
time.  `roofline` describes the MFMA kernel (32*M*C*K flop per launch), `roofline_imtrans`
the transform kernel (4*B*H*W*C + 64*M*C bytes per launch); both use the average launch
duration measured with HIP events on the launching stream.  `cpu_baseline` times the CPU
oracle (OpenMP C restatement of the same three stages) on this host's cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "sparse-winograd-cnn_amd")
for _p in (ROOT, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# Memory traffic per launch (bytes) behind the L2s, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per
# dispatch) and scaled by what the same counters read for a 128 MiB copy: FETCH_SIZE x 2.00, WRITE_SIZE x 1.00
# (the tables of profiles/conv_imtrans_*.md; tests/test_bench_contract.py checks these literals against them).  Keyed
# by the kernel variant that was profiled: a run whose launcher picked another
# one, or a configuration that was not profiled, reports null.
MEASURED_TRAFFIC = {
    # (workload, precision, op): (kernel variant, bytes)
    ("cfg3", "fp32", "conv"): ("wide48", (58014.0 * 2 + 25088.0) * 1024),        # algorithmic 129.5 MB
    ("cfg3", "fp32", "imtrans"): (None, (12575.0 * 2 + 100423.9) * 1024),         # algorithmic 128.45 MB
    ("cfg2", "fp32", "conv"): ("tall16", (108090.0 * 2 + 50176.0) * 1024),       # algorithmic 257.2 MB
    ("cfg2", "fp32", "imtrans"): (None, (25126.2 * 2 + 200811.9) * 1024),
    ("cfg4a", "fp32", "conv"): ("wide48x64", (43381.5 * 2 + 12544.0) * 1024),    # algorithmic 68.4 MB
    ("cfg4a", "fp32", "imtrans"): (None, (6431.2 * 2 + 50176.0) * 1024),
    ("cfg4b", "fp32", "conv"): ("short16", (83452.0 * 2 + 8192.0) * 1024),       # algorithmic 58.7 MB
    ("cfg4b", "fp32", "imtrans"): (None, (3175.0 * 2 + 32768.0) * 1024),
    ("cfg3", "bf16_stored", "conv"): ("stored-tall", (30373.5 * 2 + 25088.0) * 1024),    # algorithmic 77.6 MB
    ("cfg3", "bf16_stored", "imtrans"): (None, (12584.0 * 2 + 50176.0) * 1024),
    ("cfg2", "bf16_stored", "conv"): ("stored-tall", (60294.8 * 2 + 50176.0) * 1024),
    ("cfg2", "bf16_stored", "imtrans"): (None, (25128.0 * 2 + 100352.0) * 1024),
    ("cfg4a", "bf16_stored", "conv"): ("stored-split", (23787.0 * 2 + 12544.0) * 1024),
    ("cfg4a", "bf16_stored", "imtrans"): (None, (6312.0 * 2 + 25088.0) * 1024),
    ("cfg4b", "bf16_stored", "conv"): ("stored-spread", (24747.7 * 2 + 24576.0) * 1024),   # both kernels
    ("cfg4b", "bf16_stored", "imtrans"): (None, (3176.0 * 2 + 16384.0) * 1024),
}


def measured_traffic(workload, precision, op, variant=None):
    """Bytes per launch from the table above if `variant` is the kernel variant that was profiled, else None."""
    entry = MEASURED_TRAFFIC.get((workload, precision, op))
    if entry is None or (entry[0] is not None and entry[0] != variant):
        return None
    return round(entry[1])


HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, datasheet
FP32_MFMA_PEAK_TF = 157.3  # MI355X dense fp32 matrix, datasheet
BF16_MFMA_PEAK_TF = 2500.0

# name: (B, H, W, C, K, weight density, input kind)
WORKLOADS = {
    "cfg1": (1, 16, 16, 64, 64, 1.0, "normal"),
    "cfg2": (64, 56, 56, 64, 64, 0.3, "halfnormal"),
    "cfg3": (64, 28, 28, 128, 128, 0.2, "normal"),
    "cfg4a": (64, 14, 14, 256, 256, 0.1, "normal"),
    "cfg4b": (64, 7, 7, 512, 512, 0.1, "normal"),
}
SEEDS = {"cfg1": 100, "cfg2": 200, "cfg3": 300, "cfg4a": 400, "cfg4b": 410}


def make_inputs(name):
    import numpy as np
    from winograd_weights import gen_prune_mask

    B, H, W, C, K, density, kind = WORKLOADS[name]
    seed = SEEDS[name]
    x = np.random.default_rng(seed).standard_normal((B, H, W, C)).astype(np.float32)
    if kind == "halfnormal":
        x = np.maximum(x, 0)
    w = (np.random.default_rng(seed + 1).standard_normal((16, C, K)) * 0.05).astype(np.float32)
    if density < 1.0:
        gen_prune_mask(w, density)
    return x, w


def time_loop(fn, iters, torch):
    """Average duration of `iters` back-to-back calls, by HIP events on the current stream (ms)."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / iters


def cpu_baseline(name, x, w, budget_s):
    """The oracle's three stages on the host cores; returns (dict, ti_ref, y_ref)."""
    import numpy as np

    import oracle

    B, H, W, C, K = WORKLOADS[name][:5]
    nH, nW = (H + 1) // 2, (W + 1) // 2
    flops = 18.0 * B * H * W * C * K
    times, stages = [], None
    t_begin = time.perf_counter()
    ti = y = None
    while True:
        t0 = time.perf_counter()
        ti = oracle.imtrans(x, relu=True)
        t1 = time.perf_counter()
        p = oracle.gemm16(ti, w)
        t2 = time.perf_counter()
        y = oracle.output_transform(p, B, nH, nW)
        t3 = time.perf_counter()
        times.append(t3 - t0)
        if stages is None or t3 - t0 <= min(times):
            stages = (t1 - t0, t2 - t1, t3 - t2)
        if len(times) >= 9 or (time.perf_counter() - t_begin) > budget_s and len(times) >= 3:
            break
    med = float(np.median(times))
    return {
        "value": round(flops / med / 1e9, 2),
        "unit": "GFLOP/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "sample": "%d full %s steps (whole batch), median; best-step stages imtrans/gemm/output = %.1f/%.1f/%.1f ms"
                  % (len(times), name, stages[0] * 1e3, stages[1] * 1e3, stages[2] * 1e3),
        "ms_per_step": round(med * 1e3, 2),
    }, ti, y


def bench_resnet(args, torch, dev):
    """benchmark config 5: full ResNet-18-var forward, all 16 3x3 convs through the ops, random-init weights
    magnitude-pruned per layer (30/20/10/10 % density by stage), input ~N(0,1) [N,224,224,3]."""
    import numpy as np

    import resnet18_var
    from winograd_weights import gen_prune_mask

    rng = np.random.default_rng(500)
    density = {"2": 0.3, "3": 0.2, "4": 0.1, "5": 0.1}
    model = resnet18_var.ResNet18Var(precision=args.precision)
    for lname, conv in zip(resnet18_var.winograd_layer_names(), model.winograd_convs()):
        w = conv.W.data.numpy().copy()
        conv.mask = torch.from_numpy(gen_prune_mask(w, density[lname[len("Winograd_W")]]))
    model = model.to(dev)
    N = args.batch
    image = torch.from_numpy(rng.standard_normal((N, 224, 224, 3)).astype(np.float32)).to(dev)
    # 18*N*H*W*C*K over the 16 Winograd layers at the sizes the model runs them (56, 28, 14, 14)
    sizes = {"2": 56, "3": 28, "4": 14, "5": 14}
    flops = sum(18.0 * N * sizes[n[len("Winograd_W")]] ** 2 * c.in_channel * c.out_channel
                for n, c in zip(resnet18_var.winograd_layer_names(), model.winograd_convs()))
    with torch.no_grad():
        for _ in range(max(args.warmup // 4, 2)):
            logits = model(image)
        torch.cuda.synchronize()
        steps = max(args.steps // 10, 5)
        t0 = time.perf_counter()
        for _ in range(steps):
            logits = model(image)
        torch.cuda.synchronize()
        ms_eager = (time.perf_counter() - t0) * 1e3 / steps
        # The same forward replayed from one captured HIP graph: about a hundred launches per forward
        # (ops of this library and stock PyTorch ones) stop costing host time.  The replay is only
        # reported if three replays, with eager work between them, each reproduce the eager logits.
        ms_graph = None
        if args.graph:
            try:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    model(image)
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    logits_g = model(image)
                ok = True
                for _ in range(3):
                    eager = model(image)
                    torch.cuda.synchronize()
                    graph.replay()
                    torch.cuda.synchronize()
                    ok = ok and bool(torch.equal(logits_g, eager))
                if ok:
                    t0 = time.perf_counter()
                    for _ in range(steps):
                        graph.replay()
                    torch.cuda.synchronize()
                    ms_graph = (time.perf_counter() - t0) * 1e3 / steps
                else:
                    print("bench.py: graph replays of the cfg5 forward differ from the eager result; not reported",
                          file=sys.stderr)
            except RuntimeError as e:  # a stock op that cannot be captured
                print("bench.py: cfg5 forward not captured: %s" % e, file=sys.stderr)
                torch.cuda.synchronize()
    ms = ms_eager if ms_graph is None or ms_eager <= ms_graph else ms_graph
    print(json.dumps({
        "metric": "ResNet-18-var Winograd-ReLU forward (config 5), effective conv GFLOP/s of its 16 3x3 layers",
        "value": round(flops / (ms * 1e-3) / 1e9, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": steps,
        "warmup": max(args.warmup // 4, 2), "ms_per_step": round(ms, 3), "images_per_s": round(N / (ms * 1e-3), 1),
        "launch": "eager" if ms == ms_eager else "graph replay",
        "ms_per_step_eager": round(ms_eager, 3), "ms_per_step_graph": None if ms_graph is None else round(ms_graph, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"fp32": "f32", "bf16": "bf16 operands, f32 accumulate",
                  "bf16_stored": "bf16 operands (stored as bf16), f32 accumulate"}[args.precision], "data": "synthetic",
        "config": {"workload": "cfg5: ResNet-18-var forward, N=%d, 224x224x3, whole model time incl. stock "
                               "PyTorch conv1/1x1/BN/pool/FC" % N, "gemm_precision": args.precision},
        "logits_finite": bool(torch.isfinite(logits).all()),
    }))


# (label, N, H = W, C, K): the layer shapes of ResNet-18-var (imagenet-resnet-transWino-prune.py:117-211) at batch 64
# and 128, benchmark configs 4a/4b, and a handful of shapes outside the model.
SWEEP_SHAPES = [(("N%d %dx%d %d->%d" % (n, hw, hw, c, k)), n, hw, c, k)
                for n in (64, 128)
                for hw, c, k in ((56, 64, 64), (28, 64, 128), (28, 128, 128), (14, 128, 256), (14, 256, 256), (14, 256, 512),
                                 (14, 512, 512))] + [
    ("cfg4b N64 7x7 512->512", 64, 7, 512, 512), ("N32 28x28 128->128", 32, 28, 128, 128), ("N16 56x56 64->64", 16, 56, 64, 64),
    ("N8 112x112 32->32", 8, 112, 32, 32), ("N48 20x20 192->96", 48, 20, 192, 96), ("N256 14x14 128->128", 256, 14, 128, 128),
    ("N4 56x56 256->64", 4, 56, 256, 64), ("N100 10x10 320->160", 100, 10, 320, 160),
    ("N24 28x28 96->192", 24, 28, 96, 192), ("N12 14x14 1024->256", 12, 14, 1024, 256), ("N200 8x8 64->320", 200, 8, 64, 320),
    ("N2 224x224 32->64", 2, 224, 32, 64), ("N64 12x12 384->384", 64, 12, 384, 384)]
TILINGS = ("ring32", "ring16", "tall16", "short16", "wide48", "wide48x64")


def bench_sweep(args, torch, dev):
    """For every shape: the fp32 convolution kernel under each tiling it is eligible for (forced through
    swc_winograd2x2_conv_force_tiling) and under the launcher's own choice.  One JSON line; `rows` holds the table."""
    import swc_hip
    L = swc_hip.lib()
    stream = torch.cuda.current_stream().cuda_stream
    rows, worst = [], 0.0
    for label, N, hw, C, K in SWEEP_SHAPES:
        nH = nW = (hw + 1) // 2
        ti = torch.relu(torch.randn(16, N, nH, nW, C, device=dev))
        w = torch.randn(16, C, K, device=dev) * 0.05
        y = torch.empty(N, 2 * nH, 2 * nW, K, device=dev)

        def call():
            if L.swc_winograd2x2_conv(ti.data_ptr(), w.data_ptr(), y.data_ptr(), None, None, C, N, nH, nW, K, 1, 1, stream) != 0:
                raise RuntimeError("the conv launcher failed")

        iters = max(args.steps // 4, 20)
        times = {}
        for name in TILINGS:
            if L.swc_winograd2x2_conv_force_tiling(name.encode()) != 0:
                raise RuntimeError("unknown tiling %s" % name)
            call()
            if L.swc_winograd2x2_conv_last_kernel().decode() != name:
                continue   # not eligible for this shape: the launcher fell back
            for _ in range(3):
                call()
            times[name] = time_loop(call, iters, torch)
        L.swc_winograd2x2_conv_force_tiling(None)
        call()
        pick = L.swc_winograd2x2_conv_last_kernel().decode()
        for _ in range(3):
            call()
        t_pick = time_loop(call, iters, torch)
        best = min(times, key=times.get)
        # the launcher's choice measured in the same way as the forced runs (same kernel as times[pick])
        t_pick = min(t_pick, times.get(pick, t_pick))
        over = t_pick / times[best] - 1.0
        worst = max(worst, over)
        rows.append({"shape": label, "pick": pick, "best": best, "us_pick": round(t_pick * 1e3, 1),
                     "us": {k: round(v * 1e3, 1) for k, v in times.items()}, "pick_over_best_pct": round(100 * over, 1),
                     "mfma_frac_pick": round(32.0 * N * nH * nW * C * K / (t_pick * 1e-3) / 1e12 / FP32_MFMA_PEAK_TF, 3)})
        del ti, w, y
    print(json.dumps({"metric": "fp32 conv kernel time per tiling, launcher's pick against the best", "unit": "us",
                      "value": round(100 * worst, 1), "value_is": "worst pick_over_best_pct over the rows",
                      "n_gpus": 1, "higher_is_better": False, "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["cfg5", "sweep", "layer"],
                    help="cfg1-cfg4b: one layer; cfg5: the whole ResNet-18-var forward (16 Winograd layers), N=128; "
                         "sweep: the fp32 conv kernel under every tiling over the model's layer shapes and a few others; "
                         "layer: one layer of the shape given with --layer")
    ap.add_argument("--layer", default="128,14,512,512,0.1", metavar="N,HW,C,K[,density]",
                    help="shape of --workload layer (input N x HW x HW x C, K filters, N(0,1) input, weights pruned to "
                         "`density`): e.g. the ResNet-18-var layers at the model's batch, for profiles of one kernel")
    ap.add_argument("--batch", type=int, default=128, help="batch size of the cfg5 forward")
    ap.add_argument("--precision", default="fp32", choices=["fp32", "bf16", "bf16_stored"],
                    help="fp32 (the reference's arithmetic); bf16: GEMM operands rounded to bf16 inside the conv "
                         "kernel; bf16_stored: the transformed activations are also written and read as bf16")
    ap.add_argument("--no-workspace", action="store_true",
                    help="bf16_stored: call the convolution without its scratch buffer (swc_winograd2x2_conv_bf16in)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg and the parity gate")
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds of CPU work for cpu_baseline")
    ap.add_argument("--backward", action="store_true",
                    help="also time the two gradient ops (conv grad: dP transform + the dW and dTI batched GEMMs; "
                         "imTrans grad through the fused ReLU) and add a `backward` object to the line")
    ap.add_argument("--no-rotate", dest="rotate", action="store_false",
                    help="skip the extra timing over cycled buffer sets (Infinity Cache defeated)")
    ap.add_argument("--rotate-only", action="store_true",
                    help="run only the loops over cycled buffer sets and print their timings: the run to put under "
                         "rocprofv3 for counters of the cold-buffer case")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="time only eager launches; by default the K steps are also replayed from one captured HIP "
                         "graph and, when that is faster, `value`/`ms_per_step` are the replayed figure "
                         "(`ms_per_step_eager` keeps the other)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="run five 128 MiB device-to-device copies and exit: the known-size kernel that the "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters are scaled against")
    args = ap.parse_args()
    if args.copy_probe:
        import torch
        a = torch.ones(32 * 1024 * 1024, device="cuda")
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes_read": a.numel() * 4, "copy_probe_bytes_written": a.numel() * 4}))
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on one GPU only; --gpus %d is not supported (the forward pass "
                 "shards over the batch with no exchange step, so N GPUs are N independent copies of this run)"
                 % args.gpus)

    import numpy as np
    import torch

    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans

    swc_hip.lib()  # fail loudly if the HIP library is not built
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    prop = torch.cuda.get_device_properties(dev)
    print("device: %s, %d CUs, %.0f MHz, %.0f GiB" % (prop.name, prop.multi_processor_count,
          getattr(prop, "clock_rate", 0) / 1e3, prop.total_memory / 2 ** 30), file=sys.stderr)

    name = args.workload
    if name == "layer":
        f = args.layer.split(",")
        n_, hw_, c_, k_ = (int(v) for v in f[:4])
        WORKLOADS["layer"] = (n_, hw_, hw_, c_, k_, float(f[4]) if len(f) > 4 else 1.0, "normal")
        SEEDS["layer"] = 500
    if name == "cfg5":
        return bench_resnet(args, torch, dev)
    if name == "sweep":
        return bench_sweep(args, torch, dev)
    B, H, W, C, K, density, kind = WORKLOADS[name]
    nH, nW = (H + 1) // 2, (W + 1) // 2
    M = B * nH * nW
    x_np, w_np = make_inputs(name)
    x = torch.from_numpy(x_np).to(dev)
    w = torch.from_numpy(w_np).to(dev)
    stored = args.precision == "bf16_stored"
    ti = torch.empty(16, B, nH, nW, C, device=dev, dtype=torch.bfloat16 if stored else torch.float32)
    y = torch.empty(B, 2 * nH, 2 * nW, K, device=dev)

    # The timed loop calls the launcher-level C entry points directly with prebuilt arguments
    # (the Python op wrappers re-validate shapes on every call, which costs more host time
    # than the transform kernel runs for).  The wrappers are exercised once, for the record.
    L = swc_hip.lib()
    stream = torch.cuda.current_stream().cuda_stream
    xp, wp, tip, yp = x.data_ptr(), w.data_ptr(), ti.data_ptr(), y.data_ptr()
    if stored:
        from winograd2x2_conv.winograd2x2_conv import winograd2x2_weights_bf16
        w16 = winograd2x2_weights_bf16(w)   # prepared once, like W*mask
        w16p = w16.data_ptr()
        winograd2x2_imTrans(x, relu=True, out=ti, out_dtype=torch.bfloat16)
        winograd2x2_conv(ti, w16, out=y)

        def call_imtrans(a, b, st):
            return L.swc_winograd2x2_imtrans_bf16out(a, None, None, b, C, B, H, W, 1, 1, 1, st)

        # the launcher's scratch buffer (what tmp_data_buffer is to the reference's launcher), allocated once
        ws_floats = 0 if args.no_workspace else L.swc_winograd2x2_conv_bf16in_workspace_floats(C, B, nH, nW, K)
        ws = torch.empty(max(ws_floats, 1), dtype=torch.float32, device=dev)
        wsp = ws.data_ptr() if ws_floats else None

        def call_conv(b, c, st):
            return L.swc_winograd2x2_conv_bf16in_ws(b, w16p, c, None, None, None, 0, wsp, ws_floats, C, B, nH, nW, K, 1, 1, st)
    else:
        conv_entry = L.swc_winograd2x2_conv if args.precision == "fp32" else L.swc_winograd2x2_conv_bf16
        winograd2x2_imTrans(x, relu=True, out=ti)
        winograd2x2_conv(ti, w, precision=args.precision, out=y)

        def call_imtrans(a, b, st):
            return L.swc_winograd2x2_imtrans(a, b, C, B, H, W, 1, 1, 1, st)

        def call_conv(b, c, st):
            return conv_entry(b, wp, c, None, None, C, B, nH, nW, K, 1, 1, st)

    def f_imtrans():
        if call_imtrans(xp, tip, stream) != 0:
            raise RuntimeError("the imTrans launcher failed")

    def f_conv():
        if call_conv(tip, yp, stream) != 0:
            raise RuntimeError("the conv launcher failed")

    def step():
        f_imtrans()
        f_conv()

    # the same layer as one kernel: fp32 (swc_winograd2x2_relu_conv) or bf16 operands (swc_winograd2x2_relu_conv_bf16)
    def call_fused():
        if stored:
            return L.swc_winograd2x2_relu_conv_bf16(xp, None, None, w16p, yp, None, None, None, C, B, H, W, K, 1, 1, 1,
                                                    stream)
        return L.swc_winograd2x2_relu_conv(xp, wp, yp, C, B, H, W, K, 1, 1, 1, stream)

    fused_ok = args.precision != "bf16" and call_fused() == 0

    def f_fused():
        if call_fused() != 0:
            raise RuntimeError("the fused-layer launcher failed")

    def rotated_timings():
        """The kernels over buffer sets that are cycled, so that consecutive launches cannot be served from the
        256 MB Infinity Cache: together the sets are larger than it."""
        set_bytes = (x.numel() + y.numel()) * 4 + ti.numel() * ti.element_size()
        n_sets = max(2, -(-3 * 256 * 2 ** 20 // set_bytes))
        if n_sets * set_bytes >= 64 * 2 ** 30:
            return None
        sets = [(x.clone(), torch.empty_like(ti), torch.empty_like(y)) for _ in range(n_sets)]
        for xs, ts, ys in sets:
            call_imtrans(xs.data_ptr(), ts.data_ptr(), stream)
        ptrs = [(a.data_ptr(), b.data_ptr(), c.data_ptr()) for a, b, c in sets]
        state = {"i": 0}

        def nxt():
            state["i"] = (state["i"] + 1) % n_sets
            return ptrs[state["i"]]

        def r_imtrans():
            a, b, _ = nxt()
            if call_imtrans(a, b, stream) != 0:
                raise RuntimeError("the imTrans launcher failed")

        def r_conv():
            _, b, c = nxt()
            if call_conv(b, c, stream) != 0:
                raise RuntimeError("the conv launcher failed")

        def r_step():
            a, b, c = nxt()
            if call_imtrans(a, b, stream) != 0 or call_conv(b, c, stream) != 0:
                raise RuntimeError("step failed")

        # Every set is touched twice by every kernel before anything is timed (the first touch of freshly allocated
        # memory pays for its page mappings), and each figure is the median of three timed loops; the minimum is
        # reported beside it.
        for f in (r_imtrans, r_conv, r_step):
            time_loop(f, 2 * n_sets, torch)
        iters = max(args.steps, 2 * n_sets)
        runs = {k: sorted(time_loop(f, iters, torch) for _ in range(3))
                for k, f in (("ms_imtrans", r_imtrans), ("ms_conv", r_conv), ("ms_step", r_step))}
        out_r = {"buffer_sets": n_sets, "MB_per_set": round(set_bytes / 1e6, 1), "timed_loops": 3}
        for k, v in runs.items():
            out_r[k] = round(v[1], 5)
            out_r[k + "_min"] = round(v[0], 5)
        return out_r

    if args.rotate_only:
        print(json.dumps({"workload": name, "gemm_precision": args.precision, "rotated_buffers": rotated_timings()}))
        return

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # The same K steps captured once into a HIP graph and replayed: what a caller whose loop is
    # launch-bound would run (the launchers allocate nothing and never synchronise, so they capture).
    ms_step_graph = None
    if args.graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for _ in range(args.steps):
                    if call_imtrans(xp, tip, cs) != 0 or call_conv(tip, yp, cs) != 0:
                        raise RuntimeError("a launcher refused the capture stream")
            graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            ms_step_graph = (time.perf_counter() - t0) * 1e3 / args.steps
        except Exception as e:  # capture unavailable: the eager figure stands
            print("bench.py: HIP graph capture failed (%s); eager timing only" % e, file=sys.stderr)
            ms_step_graph = None

    # The same step through the Python surface the reference's callers use (winograd2x2_imTrans(...) and
    # winograd2x2_conv(...), ResNet-18-var/winograd_imtrans.py:16-17, winograd_conv.py:28): shape checks, output
    # allocation and one C call per op on every call.
    if stored:
        def py_step():
            return winograd2x2_conv(winograd2x2_imTrans(x, relu=True, out_dtype=torch.bfloat16), w16)
    else:
        def py_step():
            return winograd2x2_conv(winograd2x2_imTrans(x, relu=True), w, precision=args.precision)
    for _ in range(args.warmup):
        py_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        py_step()
    t_host = time.perf_counter() - t0
    torch.cuda.synchronize()
    ms_step_python = (time.perf_counter() - t0) * 1e3 / args.steps
    us_host_python = t_host * 1e6 / args.steps   # host time per step alone (the launches are asynchronous)

    # Per-kernel average launch durations, HIP events on the launching (current) stream.
    ms_imtrans = time_loop(f_imtrans, args.steps, torch)
    ms_conv = time_loop(f_conv, args.steps, torch)
    ms_pair = time_loop(step, args.steps, torch)
    ms_fused = time_loop(f_fused, args.steps, torch) if fused_ok else None

    rotated = rotated_timings() if args.rotate else None
    if fused_ok:
        y_fused = y.clone()
        step()  # leave the two-op result in y for the parity gate
    torch.cuda.synchronize()

    direct_flops = 18.0 * B * H * W * C * K
    gemm_flops = 32.0 * M * C * K
    ti_el = 2.0 if stored else 4.0   # bytes per element of TI (and of the weights the conv reads)
    imtrans_bytes = 4.0 * B * H * W * C + 16.0 * ti_el * M * C
    conv_bytes = 16.0 * ti_el * M * C + 16.0 * ti_el * C * K + 16.0 * M * K
    tf_conv = gemm_flops / (ms_conv * 1e-3) / 1e12
    gbs_imtrans = imtrans_bytes / (ms_imtrans * 1e-3) / 1e9
    gbs_conv = conv_bytes / (ms_conv * 1e-3) / 1e9
    if args.precision == "fp32":
        # fp32 MFMA bounds the contraction (arithmetic intensity 51 flop/B at conv3, ridge 19.7)
        conv_roofline = {"kernel": "winograd2x2_conv (16 GEMMs + fused A^T m A), fp32 MFMA, tiling %s"
                                   % L.swc_winograd2x2_conv_last_kernel().decode(), "bound": "mfma",
                         "achieved": round(tf_conv, 2), "peak": FP32_MFMA_PEAK_TF, "unit": "TFLOP/s",
                         "frac": round(tf_conv / FP32_MFMA_PEAK_TF, 4)}
    else:
        # with bf16 operands the ridge is ~310 flop/B: every ResNet-18 shape is bound by reading TI
        conv_roofline = {"kernel": "winograd2x2_conv (16 GEMMs + fused A^T m A), bf16 MFMA, %s TI"
                                   % ("bf16-stored" if stored else "fp32-stored"), "bound": "hbm",
                         "achieved": round(gbs_conv, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs_conv / HBM_PEAK_GBS, 4),
                         "mfma_TFLOPs": round(tf_conv, 2), "mfma_peak_TFLOPs": BF16_MFMA_PEAK_TF}
    if rotated is not None:
        conv_roofline["frac_rotated"] = round(conv_roofline["frac"] * ms_conv / rotated["ms_conv"], 4)
    conv_variant = L.swc_winograd2x2_conv_last_kernel().decode()
    conv_roofline.update({"traffic": measured_traffic(name, args.precision, "conv", conv_variant), "kernel_variant": conv_variant,
                          "algorithmic_flop_per_launch": gemm_flops, "algorithmic_bytes_per_launch": conv_bytes})

    ms_best = ms_step if ms_step_graph is None else min(ms_step, ms_step_graph)
    out = {
        "metric": "effective conv GFLOP/s + imTrans HBM GB/s, ResNet-18 conv3 batch 64, 1 MI355X",
        "value": round(direct_flops / (ms_best * 1e-3) / 1e9, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_best, 5),
        "launch": "hip graph replay of the K steps" if ms_best != ms_step else "eager",
        "ms_per_step_eager": round(ms_step, 5),
        "ms_per_step_graph": None if ms_step_graph is None else round(ms_step_graph, 5),
        "ms_per_step_python_ops": round(ms_step_python, 5),
        "python_ops_host_us_per_step": round(us_host_python, 1),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"fp32": "f32", "bf16": "bf16 operands, f32 accumulate",
                  "bf16_stored": "bf16 operands (stored as bf16), f32 accumulate"}[args.precision],
        "data": "synthetic",
        "config": {
            "workload": "%s: winograd2x2_imTrans(+ReLU) + winograd2x2_conv, N=%d %dx%dx%d -> %d, fp32 NHWC, "
                        "weights [16,%d,%d] at %.0f%% density" % (name, B, H, W, C, K, C, K, density * 100),
            "tiles_M": M,
            "input": kind,
            "gemm_precision": args.precision,
        },
        "imtrans_GBps": round(gbs_imtrans, 1),
        "conv_TFLOPs": round(tf_conv, 2),
        "ms_imtrans": round(ms_imtrans, 5),
        "ms_conv": round(ms_conv, 5),
        "ms_pair_events": round(ms_pair, 5),
        "rotated_buffers": rotated,
        "roofline": conv_roofline,
        # the same layer as one kernel (swc_winograd2x2_relu_conv): TI never reaches memory
        "fused_layer": None if not fused_ok else {
            "ms": round(ms_fused, 5),
            "effective_direct_conv_GFLOPs": round(direct_flops / (ms_fused * 1e-3) / 1e9, 1),
            "mfma_TFLOPs": round(gemm_flops / (ms_fused * 1e-3) / 1e12, 2),
            "mfma_frac": round(gemm_flops / (ms_fused * 1e-3) / 1e12 /
                               (BF16_MFMA_PEAK_TF if stored else FP32_MFMA_PEAK_TF), 4),
            "algorithmic_bytes_per_launch": 4.0 * B * H * W * C + 16.0 * (2.0 if stored else 4.0) * C * K + 16.0 * M * K,
            "hbm_frac": round((4.0 * B * H * W * C + 16.0 * (2.0 if stored else 4.0) * C * K + 16.0 * M * K) /
                              (ms_fused * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "max_abs_diff_vs_two_op": float((y_fused - y).abs().max()),
        },
        "roofline_imtrans": {
            "kernel": "winograd2x2_imTrans + ReLU",
            "bound": "hbm",
            "achieved": round(gbs_imtrans, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs_imtrans / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic(name, "bf16_stored" if stored else "fp32", "imtrans"),
            "algorithmic_bytes_per_launch": imtrans_bytes,
            # the same kernel over cycled buffer sets: nothing it touches is in the Infinity Cache
            "achieved_rotated": None if rotated is None else round(imtrans_bytes / (rotated["ms_imtrans"] * 1e-3) / 1e9, 1),
            "frac_rotated": None if rotated is None else round(imtrans_bytes / (rotated["ms_imtrans"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        },
    }

    if args.backward:
        dy = torch.randn(B, 2 * nH, 2 * nW, K, device=dev)
        dti, dw = torch.empty_like(ti), torch.empty_like(w)
        tmp = torch.empty(16 * M * K, device=dev)
        dx = torch.empty(B, H, W, C, device=dev)
        ptr = lambda t: t.data_ptr()  # noqa: E731

        def f_conv_grad():
            if L.swc_winograd2x2_conv_grad(tip, wp, ptr(dy), ptr(dti), ptr(dw), ptr(tmp), None, C, B, 2 * nH, 2 * nW, K,
                                           1, 1, stream) != 0:
                raise RuntimeError("swc_winograd2x2_conv_grad failed")

        def f_imtrans_grad():   # ReLU mask read from the forward result (TI)
            if L.swc_winograd2x2_imtrans_grad(ptr(dti), tip, ptr(dx), C, B, H, W, 1, 1, stream) != 0:
                raise RuntimeError("swc_winograd2x2_imtrans_grad failed")

        def f_imtrans_grad_input():   # ReLU mask recomputed from the forward input: what the autograd path calls
            if L.swc_winograd2x2_imtrans_grad_relu_input(ptr(dti), xp, ptr(dx), C, B, H, W, 1, 1, stream) != 0:
                raise RuntimeError("swc_winograd2x2_imtrans_grad_relu_input failed")

        for _ in range(3):
            f_conv_grad()
            f_imtrans_grad()
            f_imtrans_grad_input()
        iters = max(args.steps // 4, 10)
        ms_cg = time_loop(f_conv_grad, iters, torch)
        ms_ig = time_loop(f_imtrans_grad, iters, torch)
        ms_igx = time_loop(f_imtrans_grad_input, iters, torch)
        dx_bytes = 4.0 * B * H * W * C
        out["backward"] = {
            "ms_conv_grad": round(ms_cg, 5),
            "conv_grad_TFLOPs": round(2 * gemm_flops / (ms_cg * 1e-3) / 1e12, 2),  # two GEMMs of 32*M*C*K each
            # reads dT and the forward input (64*M*C + |X| bytes), writes dX
            "ms_imtrans_grad": round(ms_igx, 5),
            "imtrans_grad_GBps": round((64.0 * M * C + 2 * dx_bytes) / (ms_igx * 1e-3) / 1e9, 1),
            # reads dT and the forward result as the mask source (2 * 64*M*C bytes), writes dX
            "ms_imtrans_grad_mask_from_output": round(ms_ig, 5),
            "imtrans_grad_mask_from_output_GBps": round((128.0 * M * C + dx_bytes) / (ms_ig * 1e-3) / 1e9, 1),
        }

        # Shapes the MFMA kernels of the backward pass do not take run a plain 16-batch GEMM (scalar fma, 32x32
        # tiles): one shape whose K is no multiple of 32 (dTI falls back) and one whose M is no multiple of 32 (dW).
        fallback = []
        for fb_B, fb_n, fb_C, fb_K in ((8, 9, 128, 72), (3, 7, 128, 128)):
            fb_M = fb_B * fb_n * fb_n
            f_ti = torch.relu(torch.randn(16, fb_B, fb_n, fb_n, fb_C, device=dev))
            f_w = torch.randn(16, fb_C, fb_K, device=dev) * 0.05
            f_dy = torch.randn(fb_B, 2 * fb_n, 2 * fb_n, fb_K, device=dev)
            f_dti, f_dw, f_tmp = torch.empty_like(f_ti), torch.empty_like(f_w), torch.empty(16 * fb_M * fb_K, device=dev)

            def f_fallback():
                if L.swc_winograd2x2_conv_grad(ptr(f_ti), ptr(f_w), ptr(f_dy), ptr(f_dti), ptr(f_dw), ptr(f_tmp), None, fb_C,
                                               fb_B, 2 * fb_n, 2 * fb_n, fb_K, 1, 1, stream) != 0:
                    raise RuntimeError("swc_winograd2x2_conv_grad failed")
            for _ in range(3):
                f_fallback()
            ms_fb = time_loop(f_fallback, iters, torch)
            fallback.append({"shape": "B%d %dx%d tiles %d->%d (M=%d)" % (fb_B, fb_n, fb_n, fb_C, fb_K, fb_M),
                             "ms_conv_grad": round(ms_fb, 5),
                             "TFLOPs": round(64.0 * fb_M * fb_C * fb_K / (ms_fb * 1e-3) / 1e12, 2)})
        out["backward"]["plain_gemm_fallback"] = fallback

    if not args.no_cpu:
        cpu, ti_ref, y32_ref = cpu_baseline(name, x_np, w_np, args.cpu_budget)
        out["cpu_baseline"] = cpu
        # Parity gate on the very buffers that were timed.
        import oracle
        ti_gpu = ti.float().cpu().numpy()
        y_gpu = y.cpu().numpy()
        if stored:   # the transform is rounded once to bf16 as it is stored; the weights once when prepared
            ti_ref = oracle.round_bf16(ti_ref)
            y_ref = oracle.conv(ti_ref, oracle.round_bf16(w_np), acc64=True)
            y32_ref = oracle.conv(ti_ref, oracle.round_bf16(w_np))
        else:
            y_ref = oracle.conv(ti_ref, w_np, acc64=True)
        den = float(np.max(np.abs(y_ref)))
        out["parity"] = {
            "imtrans_bit_exact": bool(np.array_equal(ti_gpu, ti_ref)),
            "relu_zero_mask_equal": bool(np.array_equal(ti_gpu == 0, ti_ref == 0)),
            "conv_max_rel_err": float(np.max(np.abs(y_gpu - y_ref)) / den),
            "conv_l1_rel_err": float(np.sum(np.abs(y_gpu - y_ref)) / (np.sum(np.abs(y_gpu)) + np.sum(np.abs(y_ref)))),
            "cpu_fp32_oracle_max_rel_err": float(np.max(np.abs(y32_ref - y_ref)) / den),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
