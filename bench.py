"""Headline benchmark: one BERT-large encoder layer (fp16, B=8, S=512, hidden 1024, 16 heads, FFN 4096),
forward + autodiff backward through the "hip" library-node implementations, on one MI355X.

Prints ONE JSON line (see the keys below). `value` is ms per forward+backward step with all inputs
resident in HBM: W warm-up steps, then exactly K timed steps between two synchronisations; ahead of the warm-up steps
the program runs untimed for 40 ms so that the GPU's clock has settled under this load (`settle`). `roofline` describes the dominant kernel (the fp16 MFMA GEMM): algorithmic FLOPs of
all contraction launches of a step divided by their summed HIP-event durations. `hbm_nodes` does the
same against the HBM roofline for the memory-bound nodes. `cpu_baseline` is the C++ / OpenMP restatement of the
reference's pure expansions (oracle/bert_layer_loops.cpp) timed on this host, with the NumPy + BLAS form beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# Bytes that cross the L2 <-> fabric boundary for the 11 GEMM launches of one step: rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE (one run each, of `bench.py --steps 3 --warmup 2 --no-cpu-baseline --calibrate-copy`), each
# scaled by what the same counter reads for the 128 MiB copy kernel of --calibrate-copy (FETCH_SIZE x 2.000,
# WRITE_SIZE x 1.000). Measured, not computed here: it goes stale when the GEMM tiling changes, so the tile selection
# it was measured with is part of the value and is compared with the library's at run time.
GEMM_TRAFFIC_BYTES_PER_STEP = {"fetched": 833.6e6, "written": 184.6e6,
                               "measured_with": "tile configurations 4 (256x256) / 5 and 7 (128x128, four / two stages) / 9 chosen by "
                                                "the library, interleaved K loop; profiles/bert_layer_fwd_bwd_hbm_traffic.md"}

METRIC = "BERT-large encoder layer fp16 fwd+bwd ms/iter at 1 GPU; % MFMA & HBM roofline"
B, S, H, HEADS, FFN = 8, 512, 1024, 16, 4096


def build_program(device, gelu_epilogue=False, reuse_transients=True):
    import torch
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import CompiledSDFG
    from daceml_amd.transformation import fusion

    sdfg = graphs.bert_encoder_layer(B, S, H, HEADS, FFN, torch.float16, eps=1e-12)
    fusion.auto_optimize(sdfg, training=True, gelu_epilogue=gelu_epilogue)
    add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + graphs.BERT_PARAM_NAMES,
                      grad_dtypes={n: torch.float32 for n in graphs.BERT_PARAM_NAMES})
    fusion.optimize_backward(sdfg)
    return CompiledSDFG(sdfg, device=device, reuse_transients=reuse_transients)


def synthetic_inputs(device):
    """Seeded synthetic data of the config's shape: x, dy ~ N(0,1); weights N(0, 0.02), biases 0, LN 1/0."""
    import numpy as np
    import torch
    from daceml_amd import graphs
    p = graphs.bert_init_params(H, FFN, 1234 + 4)
    rng = np.random.default_rng(1234 + 5)
    x = rng.standard_normal((B, S, H)).astype(np.float16)
    dy = rng.standard_normal((B, S, H)).astype(np.float16)
    args = {"x": torch.from_numpy(x).to(device), "gradient_y": torch.from_numpy(dy).to(device),
            "y": torch.empty((B, S, H), dtype=torch.float16, device=device),
            "gradient_x": torch.empty((B, S, H), dtype=torch.float16, device=device)}
    for n in graphs.BERT_PARAM_NAMES:
        args[n] = torch.from_numpy(p[n].astype(np.float16)).to(device)
        args["gradient_" + n] = torch.empty(p[n].shape, dtype=torch.float32, device=device)
    return args, x, dy, p


def check_against_oracle(args, x, dy, p):
    """Untimed: the outputs of one step at the bench's own shape against the fp64 CPU oracle (checker only), at the
    tolerance the fp16 path is held to (rtol 2e-2 / atol 1e-2; an element of an fp32 master gradient, a sum over 4096 rows
    of products of tensors stored in fp16, is allowed 16 x 2^-11 x the root of the sum of squares of its exact terms on
    top of that)."""
    import numpy as np
    from oracle import bert_layer as OB
    x64 = x.astype(np.float64)
    p64 = {k: v.astype(np.float16).astype(np.float64) for k, v in p.items()}
    y, saved = OB.forward(x64, p64, HEADS, eps=1e-12, keep=True)
    g = OB.backward(x64, p64, HEADS, dy.astype(np.float64), saved, eps=1e-12, term_scales=True)
    del saved
    worst, ok, n_checked = {}, True, 0
    for name, want, scaled in [("y", y, False), ("gradient_x", g["x"], False)] + \
            [("gradient_" + n, g[n], True) for n in OB.PARAM_NAMES]:
        got = args[name].float().cpu().numpy().astype(np.float64)
        atol = 1e-2 + 16.0 * 2.0 ** -11 * g["terms:" + name[len("gradient_"):]] if scaled else 1e-2
        err = np.abs(got - want)
        excess = err - (atol + 2e-2 * np.abs(want))
        worst[name] = float(err.max())
        ok = ok and bool((excess <= 0).all()) and bool(np.isfinite(got).all())
        n_checked += got.size
    return {"checked": ok, "max_abs_error": {"y": worst["y"], "gradient_x": worst["gradient_x"],
                                             "parameter_gradients": max(v for k, v in worst.items()
                                                                        if k not in ("y", "gradient_x"))},
            "elements_checked": n_checked,
            "check": "y, gradient_x and all 16 parameter gradients of the first (untimed) step vs the fp64 oracle, "
                     "rtol 2e-2 / atol 1e-2 (parameter gradients: atol 1e-2 + 16 x 2^-11 x the root-sum-square of the "
                     "element's 4096 exact terms)"}


def kernel_breakdown(prog, reps=10):
    """HIP-event duration of every launch, averaged over `reps` passes: one event on the launch stream between
    consecutive launches, so a launch's time is the kernel plus its dispatch on the stream and the times of a pass
    add up to the pass."""
    acc = None
    for _ in range(reps):
        rows = prog.launch_timed()
        if acc is None:
            acc = [[l, 0.0] for l, _ in rows]
        for i, (_, ms) in enumerate(rows):
            acc[i][1] += ms
    return [(l, ms / reps) for l, ms in acc]


def cpu_baseline(x, dy, p, budget_s=25.0):
    """The CPU restatement of the pure expansions on the full workload in fp32, repeated within a time budget: the
    C++ / OpenMP loop nests (`value`; one parallel map or reduction per statement, blocked-loop contractions) and,
    beside it, the NumPy statements with BLAS contractions."""
    import numpy as np
    from oracle import bert_layer as OB
    from oracle import bert_layer_loops as OL
    x32 = x.astype(np.float32)
    dy32 = dy.astype(np.float32)
    p32 = {k: v.astype(np.float32) for k, v in p.items()}

    def repeat(fn, budget, most):
        times = []
        t_end = time.perf_counter() + budget
        while True:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
            if time.perf_counter() + times[-1] > t_end or len(times) >= most:
                return times

    def numpy_step():
        _, saved = OB.forward(x32, p32, HEADS, eps=1e-12, keep=True)
        OB.backward(x32, p32, HEADS, dy32, saved, eps=1e-12)

    loops = repeat(lambda: OL.forward_backward(x32, p32, HEADS, dy32, eps=1e-12), budget_s * 0.6, 4)
    blas = repeat(numpy_step, budget_s * 0.4, 3)
    try:
        from threadpoolctl import threadpool_info
        blas_threads = max([i.get("num_threads", 1) for i in threadpool_info() if i.get("user_api") == "blas"] or [1])
    except Exception:
        blas_threads = os.cpu_count() or 1
    return {"value": round(min(loops) * 1e3, 2), "unit": "ms/iter", "cores": OL.threads(), "kind": "port",
            "sample": "full workload (B=8, S=512), %d fwd+bwd repetitions in fp32 of the C++/OpenMP restatement of the "
                      "pure expansions (one parallel loop nest per statement, blocked-loop contractions), best of them"
                      % len(loops),
            "blas_variant": {"value": round(min(blas) * 1e3, 2), "unit": "ms/iter", "cores": int(blas_threads),
                             "sample": "%d repetitions of the NumPy statements; contractions through np.matmul (BLAS, "
                                       "`cores` threads), every other statement on one core" % len(blas)}}


SETTLE_MS = 40.0


def settle(step, ms=SETTLE_MS):
    """Untimed steps, ahead of the warm-up steps, until the GPU has been under this load for `ms` of wall time. After
    an idle stretch (the oracle check on the CPU, a fresh process) the GPU runs its first two or three steps at boost
    clocks, then about twenty of them 5 - 25 % slower while its power management finds the clock this load sustains; a
    short warm-up would put that stretch into the timed region (measured: steps 5 - 24 from a cold start average
    0.589 ms, steps 100 - 199 average 0.547 ms). Returns the number of steps run."""
    import torch
    n = 0
    torch.cuda.synchronize()
    t_end = time.perf_counter() + ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(5):
            step()
        n += 5
        torch.cuda.synchronize()
    return n


# ----------------------------------------------------------------------------- the other configurations
def _time_program(prog, steps, warmup, graph=False):
    """ms per step; with `graph` the step's launches are replayed from a HIP graph captured once."""
    import torch
    step = prog.capture().replay if graph else prog.launch
    settle(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def attention_trace(device):
    """Where the fused-attention workgroups' time goes on the benchmarked shape ([8, 16, 512, 64] as head-split views of
    [8, 512, 1024]): the library's per-workgroup clock readings (``dmlhip_debug_attention_trace``, 100 MHz wall clock),
    printed as microseconds after the first workgroup of each kernel started. A diagnostic, not a benchmark line."""
    import numpy as np
    import torch
    from daceml_amd import _lib, kernels as K
    lib = _lib.load()
    mk = lambda: torch.randn(B, S, HEADS, H // HEADS, device=device).half().permute(0, 2, 1, 3)  # noqa: E731
    q, k, v, do = mk(), mk(), mk(), mk()
    scale = 1.0 / float(np.sqrt(H // HEADS))
    out, lse = K.attention(q, k, v, scale)
    for _ in range(5):
        K.attention(q, k, v, scale, out=out)
        K.attention_backward(q, k, v, out, lse, do, scale)
    wgs = B * HEADS * S // 128
    readings = torch.zeros(2 * wgs * 16, dtype=torch.int64, device=device)

    def report(name, t):
        us = (t.astype(np.float64) - t[:, 0].min()) / 100.0
        per_tile = np.median(np.diff(us[:, 2:2 + S // 64], axis=1), axis=0)
        print("%-16s start %.2f (max %.2f) | first tile in LDS %.2f (max %.2f) | first tile done %.2f | further tiles %s | "
              "end %.2f (max %.2f); workgroups of the first / second launch round end at %.2f / %.2f"
              % (name, np.median(us[:, 0]), us[:, 0].max(), np.median(us[:, 1]), us[:, 1].max(), np.median(us[:, 2]),
                 " ".join("%.2f" % x for x in per_tile), np.median(us[:, 15]), us[:, 15].max(),
                 np.median(us[:256, 15]), np.median(us[256:, 15])))

    lib.dmlhip_debug_attention_trace(readings.data_ptr())
    try:
        K.attention(q, k, v, scale, out=out)
        torch.cuda.synchronize()
        report("forward", readings.cpu().numpy()[:wgs * 16].reshape(wgs, 16))
        readings.zero_()
        K.attention_backward(q, k, v, out, lse, do, scale)
        torch.cuda.synchronize()
    finally:
        lib.dmlhip_debug_attention_trace(None)
    t = readings.cpu().numpy().reshape(2 * wgs, 16)
    report("backward, dQ", t[:wgs])
    report("backward, dK/dV", t[wgs:])


def secondary_workload(name, device, steps, warmup, verbose, graph=False, fused_rolling="", reuse_transients=True):
    """BASELINE.json configs[0..3]: parity-test cases that are also worth a measured line. Same JSON keys as the
    headline; `roofline` is that of the launch that takes the most time."""
    import numpy as np
    import torch
    from daceml_amd import graphs
    from daceml_amd.runtime import CompiledSDFG
    from daceml_amd.transformation import fusion
    rng = np.random.default_rng(1234)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    if name == "bert_fwd":
        sdfg = graphs.bert_encoder_layer(B, S, H, HEADS, FFN, torch.float16, eps=1e-12)
        fusion.auto_optimize(sdfg)
        p = graphs.bert_init_params(H, FFN, 1234 + 2)
        args = {n: dev(p[n].astype(np.float16)) for n in graphs.BERT_PARAM_NAMES}
        args["x"] = dev(rng.standard_normal((B, S, H)).astype(np.float16))
        args["y"] = torch.empty((B, S, H), dtype=torch.float16, device=device)
        what, dtype = "BERT-large encoder layer forward, B=8 S=512, fp16 (BASELINE.json configs[2])", "f16"
    elif name == "nodes":
        g = graphs.GraphBuilder("memory_bound_nodes", torch.float16)
        sc = g.input("scores", (8, 16, 512, 512))
        pr = g.node("Softmax", {"input": sc}, {"output": (8, 16, 512, 512)}, label="softmax", axis=-1)["output"]
        g.output(pr, "probs")
        xin = g.input("x", (8, 512, 1024))
        g.input("gamma", (1024, ))
        g.input("beta", (1024, ))
        g.output(g.layer_norm(xin, "gamma", "beta", 1e-5, "ln"), "y")
        sdfg = g.sdfg
        fusion.auto_optimize(sdfg)
        args = {"scores": dev(rng.standard_normal((8, 16, 512, 512)).astype(np.float16)),
                "probs": torch.empty((8, 16, 512, 512), dtype=torch.float16, device=device),
                "x": dev(rng.standard_normal((8, 512, 1024)).astype(np.float16)),
                "gamma": dev(rng.uniform(0.5, 1.5, 1024).astype(np.float16)),
                "beta": dev((rng.standard_normal(1024) * 0.1).astype(np.float16)),
                "y": torch.empty((8, 512, 1024), dtype=torch.float16, device=device)}
        what, dtype = "Softmax [8,16,512,512] and LayerNorm chain [8,512,1024], fp16 (BASELINE.json configs[1])", "f16"
    elif name == "mbconv":
        sdfg = graphs.mbconv_block(96, 32, 112)
        fusion.auto_optimize(sdfg)
        shapes = {"expand": (192, 32, 1, 1), "dw": (192, 1, 3, 3), "se1": (8, 192, 1, 1), "se2": (192, 8, 1, 1),
                  "proj": (48, 192, 1, 1)}
        args = {"x": dev(rng.standard_normal((96, 32, 112, 112)).astype(np.float32)),
                "y": torch.empty((96, 48, 56, 56), dtype=torch.float32, device=device)}
        for n, shp in shapes.items():
            fan_in = shp[1] * shp[2] * shp[3]
            args[n + "_w"] = dev((rng.standard_normal(shp) * np.sqrt(2.0 / fan_in)).astype(np.float32))
            args[n + "_b"] = dev((rng.standard_normal(shp[0]) * 0.1).astype(np.float32))
        what, dtype = "EfficientNet-B0 MBConv block, batch 96, [96,32,112,112], fp32 (BASELINE.json configs[3])", "f32"
    elif name == "conv":
        g = graphs.GraphBuilder("conv_c1", torch.float32)
        xin = g.input("x", (5, 3, 10, 10))
        g.input("w", (16, 3, 3, 3))
        g.output(g.node("Conv", {"X": xin, "W": "w"}, {"Y": (5, 16, 4, 4)}, label="conv", kernel_shape=[3, 3],
                        strides=[2, 2])["Y"], "y")
        sdfg = g.sdfg
        args = {"x": dev(rng.uniform(0, 1, (5, 3, 10, 10)).astype(np.float32)),
                "w": dev(rng.uniform(0, 1, (16, 3, 3, 3)).astype(np.float32)),
                "y": torch.empty((5, 16, 4, 4), dtype=torch.float32, device=device)}
        what, dtype = "single Conv fp32 X[5,3,10,10] W[16,3,3,3] stride 2 (BASELINE.json configs[0]; launch latency)", "f32"
    elif name == "conv_dense_train":
        # not a BASELINE.json configuration: a ResNet-sized dense 3x3 convolution with its data and weight gradients,
        # the shape the implicit-GEMM kernels are quoted on
        from daceml_amd.autodiff import add_backward_pass
        g = graphs.GraphBuilder("conv_dense_train", torch.float32)
        xin = g.input("x", (32, 64, 56, 56))
        g.input("w", (64, 64, 3, 3))
        g.output(g.node("Conv", {"X": xin, "W": "w"}, {"Y": (32, 64, 56, 56)}, label="conv", kernel_shape=[3, 3],
                        pads=[1, 1, 1, 1])["Y"], "y")
        sdfg = g.sdfg
        add_backward_pass(sdfg, g.state, ["y"], ["x", "w"])
        args = {"x": dev(rng.standard_normal((32, 64, 56, 56)).astype(np.float32)),
                "w": dev((rng.standard_normal((64, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float32)),
                "y": torch.empty((32, 64, 56, 56), dtype=torch.float32, device=device),
                "gradient_y": dev(rng.standard_normal((32, 64, 56, 56)).astype(np.float32)),
                "gradient_x": torch.empty((32, 64, 56, 56), dtype=torch.float32, device=device),
                "gradient_w": torch.empty((64, 64, 3, 3), dtype=torch.float32, device=device)}
        what, dtype = "dense Conv 3x3 fp32 X[32,64,56,56] W[64,64,3,3] pad 1, forward + data and weight gradients", "f32"
    else:
        sys.exit("unknown workload %r" % name)
    prog = CompiledSDFG(sdfg, device=device, reuse_transients=reuse_transients)
    prog(**args)
    ms = _time_program(prog, steps, warmup, graph)
    rows = kernel_breakdown(prog)
    launches = []
    for l, t in rows:
        e = {"label": l.label, "kind": l.kind, "us": round(t * 1e3, 2)}
        if l.flops:
            e["TFLOP/s"] = round(l.flops / (t * 1e-3) / 1e12, 2)
        if l.bytes_moved:
            e["GB/s"] = round(l.bytes_moved / (t * 1e-3) / 1e9, 1)
        launches.append(e)
        if verbose:
            sys.stderr.write("%-28s %-40s %8.1f us %s\n" % (l.kind, l.label[:40], t * 1e3, {k: v for k, v in e.items()
                                                                                             if "/s" in k}))
    top, top_t = max(rows, key=lambda r: r[1])
    if top.kind in ("gemm", "attention") and dtype == "f16":
        roof = {"bound": "mfma", "achieved": round(top.flops / (top_t * 1e-3) / 1e12, 1), "peak": PEAK_FP16_TFLOPS,
                "unit": "TFLOP/s"}
    elif dtype == "f32" and top.flops and top.bytes_moved and \
            top.flops / top.bytes_moved > PEAK_FP32_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9):
        # more flops per byte than the fp32 matrix pipe can absorb at full HBM rate (the fused expand + depthwise node)
        roof = {"bound": "mfma", "achieved": round(top.flops / (top_t * 1e-3) / 1e12, 1), "peak": PEAK_FP32_TFLOPS,
                "unit": "TFLOP/s"}
    else:
        roof = {"bound": "hbm", "achieved": round(top.bytes_moved / (top_t * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s"}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["traffic"] = None
    roof["kernel"] = top.label
    line = {"metric": what + " ms/iter at 1 GPU", "value": round(ms, 4), "unit": "ms/iter", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
            "config": {"workload": what, "launches_per_step": len(prog.launches), "hip_graph": bool(graph),
                       **({"fused_rolling": fused_rolling} if fused_rolling else {})},
            "roofline": roof, "launches": launches}
    if name == "nodes":
        line["stream_timing"] = stream_timing(device, max(3, min(steps, 10)))
    print(json.dumps(line))


def stream_timing(device, rounds):
    """The two `nodes` kernels and a plain copy of the same bytes (the library's identity kernel: 128-bit loads and
    stores, the bandwidth a one-pass kernel of that size can be held against), each timed as a stream of 40 launches
    replayed from a HIP graph between one pair of events - no host call between the launches, so a kernel of a few
    microseconds is not timed waiting for its own submission, as it is with an event pair around a single launch. The
    figure per launch includes the gap to the next launch on the stream. `cached`: the launches rotate over few tensor
    pairs that stay in the 256 MB last-level cache; `cold`: over enough pairs (LayerNorm: 40 x 16.8 MB = 671 MB) that
    a pair has left it by the time it comes round again and the launch reads from HBM."""
    import numpy as np
    import torch
    from daceml_amd import graphs
    from daceml_amd.runtime import CompiledSDFG
    from daceml_amd.transformation import fusion
    launches = 40
    rng = np.random.default_rng(99)
    gamma = torch.from_numpy(rng.uniform(0.5, 1.5, 1024).astype(np.float16)).to(device)
    beta = torch.from_numpy((rng.standard_normal(1024) * 0.1).astype(np.float16)).to(device)

    def run(kind, shape, pairs):
        g = graphs.GraphBuilder("stream_" + kind, torch.float16)
        if kind == "layernorm":
            g.input("gamma", (1024, ))
            g.input("beta", (1024, ))
        for i in range(launches):
            xin = g.input("x%d" % i, shape)
            if kind == "layernorm":
                out = g.layer_norm(xin, "gamma", "beta", 1e-5, "ln%d" % i)
            elif kind == "softmax":
                out = g.node("Softmax", {"input": xin}, {"output": shape}, label="sm%d" % i, axis=-1)["output"]
            else:
                out = g.node("Identity", {"input": xin}, {"output": shape}, label="copy%d" % i)["output"]
            g.output(out, "y%d" % i)
        fusion.auto_optimize(g.sdfg)
        prog = CompiledSDFG(g.sdfg, device=device)
        assert len(prog.launches) == launches, [l.symbol for l in prog.launches]
        xs = [torch.randn(shape, dtype=torch.float16, device=device) for _ in range(pairs)]
        ys = [torch.empty(shape, dtype=torch.float16, device=device) for _ in range(pairs)]
        args = {"x%d" % i: xs[i % pairs] for i in range(launches)}
        args.update({"y%d" % i: ys[i % pairs] for i in range(launches)})
        if kind == "layernorm":
            args.update(gamma=gamma, beta=beta)
        prog(**args)
        cap = prog.capture()
        cap.replay()
        times = []
        for _ in range(rounds):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            cap.replay()
            e.record()
            torch.cuda.synchronize(device)
            times.append(s.elapsed_time(e) * 1e3 / launches)
        us = float(np.median(times))
        nbytes = 4 * int(np.prod(shape))
        gbs = nbytes / (us * 1e-6) / 1e9
        del cap, prog, xs, ys
        torch.cuda.empty_cache()
        return {"us": round(us, 2), "min_us": round(float(np.min(times)), 2), "bytes": nbytes, "GB/s": round(gbs, 1),
                "frac": round(gbs / PEAK_HBM_GBS, 4), "pairs": pairs}

    ln, sm = (8, 512, 1024), (8, 16, 512, 512)
    return {"launches_per_replay": launches, "replays": rounds,
            "layernorm": {"cached": run("layernorm", ln, 4), "cold": run("layernorm", ln, 40)},
            "copy_of_layernorm_bytes": {"cached": run("copy", ln, 4), "cold": run("copy", ln, 40)},
            "softmax": {"one_pair": run("softmax", sm, 1), "cold": run("softmax", sm, 5)},
            "copy_of_softmax_bytes": {"one_pair": run("copy", sm, 1), "cold": run("copy", sm, 5)}}


def module_workload(device, steps, warmup):
    """HuggingFace BertLayer (BERT-large sizes, fp16, no dropout) wrapped in DaceModule: forward + backward through
    torch.autograd, next to the same module run by PyTorch itself on the same GPU. Includes everything a user of
    the wrapper pays per call (autograd bookkeeping, output allocation, gradient casts)."""
    import copy
    import warnings
    import torch
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer
    from daceml_amd.torch import DaceModule

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            cfg = BertConfig(hidden_size=H, num_attention_heads=HEADS, intermediate_size=FFN, hidden_dropout_prob=0.0,
                             attention_probs_dropout_prob=0.0)
            cfg._attn_implementation = "eager"
            self.layer = BertLayer(cfg)

        def forward(self, x):
            out = self.layer(x)
            return out[0] if isinstance(out, (tuple, list)) else out

    torch.manual_seed(1234)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        eager = Layer().to(device).half().eval()
        wrapped = DaceModule(copy.deepcopy(eager), backward=True)
        x = torch.randn(B, S, H, device=device, dtype=torch.float16, requires_grad=True)
        dy = torch.randn(B, S, H, device=device, dtype=torch.float16)
        wrapped(x)   # traces, imports, fuses, binds

    def step(mod):
        x.grad = None
        for p_ in mod.parameters():
            p_.grad = None
        mod(x).backward(dy)

    def timed(mod):
        settle(lambda: step(mod))
        for _ in range(warmup):
            step(mod)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(mod)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    ms, ms_eager = timed(wrapped), timed(eager)
    what = "HuggingFace BertLayer (BERT-large sizes, B=8 S=512, fp16) forward + backward through DaceModule"
    print(json.dumps({"metric": what + " ms/iter at 1 GPU", "value": round(ms, 4), "unit": "ms/iter", "n_gpus": 1,
                      "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "higher_is_better": False,
                      "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
                      "config": {"workload": what, "launches_per_step": len(wrapped.compiled.launches)},
                      "pytorch_eager_ms": round(ms_eager, 4), "speedup_over_pytorch_eager": round(ms_eager / ms, 2),
                      "optimization_stats": wrapped.optimization_stats}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="bert_fwd_bwd", choices=["bert_fwd_bwd", "bert_fwd", "nodes", "mbconv", "conv", "conv_dense_train", "module_bert"],
                    help="bert_fwd_bwd is the headline (default); the others are BASELINE.json's remaining configs")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true", help="skip the untimed comparison with the CPU oracle")
    ap.add_argument("--verbose", action="store_true", help="per-launch table on stderr")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed region, launch a plain 128 MiB -> 128 MiB copy kernel three times: under "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE its counters give the scale of those counters")
    ap.add_argument("--graph", action="store_true",
                    help="replay the step from a HIP graph captured once instead of launching kernel by kernel (what a "
                         "step of a few short kernels is bound by); recorded in config.hip_graph, not the reported "
                         "configuration of the headline workload")
    ap.add_argument("--gemm-config", type=int, default=-1,
                    help="pin the tile configuration of the fp16 contraction kernel for the whole run (the library's "
                         "diagnostic switch; -1 = the library's own choice). For comparing configurations, not for the "
                         "reported figure: the JSON line carries the value in config.gemm_config")
    ap.add_argument("--gelu-epilogue", action="store_true",
                    help="fold the Gelu of the feed-forward block into the epilogue of the contraction before it (off in "
                         "the reported configuration: measured slower with one workgroup per compute unit); recorded in "
                         "config.gelu_epilogue")
    ap.add_argument("--fused-rolling", default="",
                    help="ROWS,WAVES: run the fused expand + depthwise convolution with its rolling-window kernel (the "
                         "library's diagnostic switch; ROWS -1 = as many as fit). For comparing kernels, not for the "
                         "reported figure: the JSON line carries the value in config.fused_rolling")
    ap.add_argument("--own-buffers", action="store_true",
                    help="give every transient a buffer of its own instead of letting dead ones hand their memory on "
                         "(for comparing)")
    ap.add_argument("--attention-trace", action="store_true",
                    help="print where the fused-attention workgroups' time goes on the benchmarked shape (the library's "
                         "per-workgroup clock trace) and exit: a diagnostic, no JSON line")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures the single-GPU path only: this build uses one GPU (no collectives, no sharding); "
                 "run with --gpus 1")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    if a.gemm_config >= 0:
        from daceml_amd import _lib
        _lib.load().dmlhip_debug_force_gemm_config(a.gemm_config)
    if a.fused_rolling:
        from daceml_amd import _lib
        rows, waves = (int(v) for v in a.fused_rolling.split(","))
        _lib.load().dmlhip_debug_fused_rolling(rows, waves)

    if a.attention_trace:
        return attention_trace(device)
    if a.workload == "module_bert":
        return module_workload(device, a.steps, a.warmup)
    if a.workload != "bert_fwd_bwd":
        return secondary_workload(a.workload, device, a.steps, a.warmup, a.verbose, a.graph, a.fused_rolling,
                                  reuse_transients=not a.own_buffers)

    prog = build_program(device, a.gelu_epilogue, reuse_transients=not a.own_buffers)
    args, x, dy, p = synthetic_inputs(device)
    prog(**args)  # binds pointers, first run
    torch.cuda.synchronize()
    checked = None if a.no_check else check_against_oracle(args, x, dy, p)
    # --graph: the step replayed from a HIP graph (for comparing; the reported configuration launches kernel by kernel)
    step = prog.capture().replay if a.graph else prog.launch
    settled = settle(step)
    for _ in range(a.warmup):
        step()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(a.steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        marks[i].record()
        step()
    marks[a.steps].record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / a.steps * 1e3
    # per-step statistics as the reference's profiler reports them (event_profiler.py:87-143): HIP events between
    # the steps of the timed region
    import statistics
    per_step = [marks[i].elapsed_time(marks[i + 1]) for i in range(a.steps)]
    step_stats = {"min": round(min(per_step), 4), "median": round(statistics.median(per_step), 4),
                  "mean": round(statistics.fmean(per_step), 4), "max": round(max(per_step), 4),
                  "stdev": round(statistics.pstdev(per_step), 4)}

    if a.calibrate_copy:
        from daceml_amd import _lib as L, kernels as K
        src = torch.zeros(64 << 20, dtype=torch.float16, device=device)   # 128 MiB
        dst = torch.empty_like(src)
        for _ in range(3):
            K.unary(L.IDENTITY, src, out=dst)
        torch.cuda.synchronize()

    rows = kernel_breakdown(prog)
    if a.verbose:
        for l, t in rows:
            rate = ("%7.1f TFLOP/s" % (l.flops / (t * 1e-3) / 1e12)) if l.flops else \
                   ("%7.1f GB/s" % (l.bytes_moved / (t * 1e-3) / 1e9)) if l.bytes_moved else ""
            sys.stderr.write("%-9s %-28s %-44s %8.1f us %s\n" % (l.state[-9:], l.kind, l.label[:44], t * 1e3, rate))
    gemm_ms = sum(t for l, t in rows if l.kind == "gemm")
    gemm_flops = sum(l.flops for l, _ in rows if l.kind == "gemm")
    n_gemm = sum(1 for l, _ in rows if l.kind == "gemm")
    gemm_bytes = sum(l.bytes_moved for l, _ in rows if l.kind == "gemm")
    tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12
    attn = {}
    for l, t in rows:
        if l.kind in ("attention", "attention_backward"):
            attn[l.kind] = {"ms": round(t, 4), "flops": l.flops, "TFLOP/s": round(l.flops / (t * 1e-3) / 1e12, 1)}
    hbm = {}
    for l, t in rows:
        if l.kind in ("gemm", "attention", "attention_backward") or l.bytes_moved == 0:
            continue
        e = hbm.setdefault(l.kind, {"ms": 0.0, "bytes": 0, "launches": 0})
        e["ms"] += t
        e["bytes"] += l.bytes_moved
        e["launches"] += 1
    for e in hbm.values():
        e["GB/s"] = round(e["bytes"] / (e["ms"] * 1e-3) / 1e9, 1)
        e["frac"] = round(e["GB/s"] / PEAK_HBM_GBS, 4)
        e["ms"] = round(e["ms"], 4)
    out = {
        "metric": METRIC, "value": round(ms, 4), "unit": "ms/iter", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (fp32 accumulate, fp32 master gradients)", "data": "synthetic",
        "config": {"workload": "BERT-large encoder layer forward + autodiff backward, B=8 S=512 hidden=1024 heads=16 "
                               "ffn=4096, fp16 (BASELINE.json configs[4])",
                   "launches_per_step": len(prog.launches),
                   **({"gemm_config": a.gemm_config} if a.gemm_config >= 0 else {}),
                   **({"gelu_epilogue": True} if a.gelu_epilogue else {}),
                   **({"hip_graph": True} if a.graph else {})},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_FP16_TFLOPS, 4),
                     "traffic": GEMM_TRAFFIC_BYTES_PER_STEP["fetched"] + GEMM_TRAFFIC_BYTES_PER_STEP["written"],
                     "traffic_note": "bytes per step over the same launches (rocprofv3 FETCH_SIZE + WRITE_SIZE, "
                                     "calibrated on a copy kernel; a constant measured with: %s%s); algorithmic bytes "
                                     "of those launches: %d" % (GEMM_TRAFFIC_BYTES_PER_STEP["measured_with"],
                                                                "; THIS RUN PINS ANOTHER CONFIGURATION" if a.gemm_config >= 0
                                                                else "", gemm_bytes),
                     "kernel": "gemm_f16_pipe_kernel (all %d contraction launches of a step)" % n_gemm,
                     "flops_per_step": gemm_flops, "ms_per_step": round(gemm_ms, 4)},
        "attention_nodes": attn,
        "hbm_nodes": hbm,
        "sum_of_kernel_ms": round(sum(t for _, t in rows), 4),
        "step_ms": step_stats,
        "untimed_steps_before_warmup": settled,
        "untimed_steps_note": "%g ms of untimed steps ahead of the warm-up steps: after an idle stretch the GPU needs "
                              "about twenty steps to settle on the clock this load sustains" % SETTLE_MS,
        "transient_arena": {"bytes": prog.arena_bytes, "reuse_transients": prog.reuse_transients},
    }
    if checked is not None:
        out.update(checked)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(x, dy, p)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
