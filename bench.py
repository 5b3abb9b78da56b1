#!/usr/bin/env python3
"""Benchmark of the group-quantized linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-graph] [--skip-extra] [--skip-cpu] [--prefill-only]

A "step" is one decode token's worth of q4f16_1 GEMVs at Llama-3-8B shapes, batch 1:
32 layers x (fused qkv 6144x4096, o_proj 4096x4096, fused gate_up 28672x4096, down 4096x14336)
plus lm_head 128256x4096 = 129 launches that stream 4.23 GB of distinct packed weights and
scales (every layer owns its own tensors, so nothing is re-read from cache between launches).
Inputs are resident in HBM before the timed region.  `value` is the algorithmic GB/s of the whole
step (weights + scales + activations + outputs, each counted once) measured with HIP events on the
launch stream; the step is replayed from a HIP graph unless --no-graph is given.

The JSON line also carries
  roofline      the dominant kernel (the gate_up GEMV, 52 % of a step's bytes) timed on its own
                over the 32 distinct gate_up weight sets;
  cpu_baseline  the C restatement of the reference's fused dequantize-matmul loop nest on the
                host cores (a reported baseline, not the target);
  extra         per-shape GEMV GB/s for batch 1/4/8/16 and prefill GEMM TFLOP/s at M = 2048.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mlc-llm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
BITS, G = 4, 32
LAYERS = 32
SHAPES = {  # name: (N, K)
    "qkv": (6144, 4096),
    "o_proj": (4096, 4096),
    "gate_up": (28672, 4096),
    "down": (4096, 14336),
}
LM_HEAD = (128256, 4096)


def gemv_bytes(n: int, k: int, b: int = 1) -> int:
    ng = -(-k // G)
    return n * 4 * ng * 4 + n * ng * 2 + b * k * 2 + b * n * 2


def run_only(args, dev, gq, ops, torch, make_weight) -> int:
    """One linear (or the Mixtral layer) over distinct weight copies: a short run for rocprofv3 counters."""
    parts = args.only.split(":")
    q3 = parts[0] == "q3"
    if q3:
        parts = parts[1:]
    gx = torch.Generator(device=dev).manual_seed(1)

    def timed_loop(fn, per_call):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (args.steps * per_call)

    if parts[0] == "moe":
        from mlc_llm_amd import QUANTIZATION
        from mlc_llm_amd.nn import MixtralMoE

        t = int(parts[1])
        moe = MixtralMoE(4096, 14336, 8, 2, QUANTIZATION["q4f16_1"], device=dev)
        for e in range(8):
            g = torch.Generator(device=dev).manual_seed(7000 + e)
            w13 = (torch.randn((28672, 4096), generator=g, device=dev) * 0.02).half()
            moe.e1_e3.q_weight.data[e], moe.e1_e3.q_scale.data[e] = ops.quantize(w13, BITS, G)
            w2 = (torch.randn((4096, 14336), generator=g, device=dev) * 0.02).half()
            moe.e2.q_weight.data[e], moe.e2.q_scale.data[e] = ops.quantize(w2, BITS, G)
            del w13, w2
        xt = torch.randn((1, t, 4096), generator=gx, device=dev).half()
        logits = torch.randn((t, 8), generator=torch.Generator(device=dev).manual_seed(2), device=dev).half()
        us = timed_loop(lambda: moe(xt, logits), 1)
        print(json.dumps({"only": args.only, "us_per_layer": round(us, 2), "steps": args.steps}))
        return 0

    name, rows = parts[0], int(parts[1])
    shapes = dict(SHAPES, lm_head=LM_HEAD)
    if q3:
        shapes = {"qkv": (12288, 4096), "o_proj": (4096, 4096), "gate_up": (22016, 4096), "down": (4096, 11008)}
    n, k = shapes[name]
    bits, gsz = (3, 40) if q3 else (BITS, G)
    ng = -(-k // gsz)
    copies = max(2, min(32, int(1.2e9 // (n * ng * 18))))
    ws = []
    for c in range(copies):
        g = torch.Generator(device=dev).manual_seed(100 + c)
        w = (torch.randn((n, k), generator=g, device=dev) * 0.02).half()
        ws.append(ops.quantize(w, bits, gsz))
        del w
    x = torch.randn((rows, k), generator=gx, device=dev).half()
    y = torch.empty((rows, n), dtype=torch.float16, device=dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def sweep():
        for qw, qs in ws:
            ops.linear(x, qw, qs, bits, gsz, None, torch.float16, y)
            if args.probe:
                gq._lib.call("mi355gq_testing_stream_read", qw.data_ptr(), qw.numel() * 4, qs.data_ptr(), qs.numel() * 2,
                             sink.data_ptr(), stream)

    us = timed_loop(sweep, copies)
    nbytes = n * 4 * ng * 4 + n * ng * 2 + rows * k * 2 + rows * n * 2
    print(json.dumps({"only": args.only, "kernel": gq._lib.last_kernel(), "copies": copies,
                      "us_per_launch" + ("_incl_probe" if args.probe else ""): round(us, 2),
                      "algorithmic_bytes": nbytes, "flop": 2 * rows * n * k, "steps": args.steps}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--skip-extra", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--prefill-only", action="store_true",
                    help="time only the prefill GEMM (gate_up 28672x4096, M = 2048): the run the MFMA counters "
                         "under profiles/ are collected on")
    ap.add_argument("--only", default=None, metavar="SHAPE:ROWS",
                    help="time only one linear, e.g. gate_up:1, o_proj:8, down:2048 (SHAPE in qkv, o_proj, gate_up, "
                         "down, lm_head; q3:SHAPE:ROWS for the q3f16_1 Llama-2-7B shapes; moe:T for the Mixtral layer) "
                         "over distinct weight copies, plus the read-only probe on the same tensors with --probe: the "
                         "runs the counter summaries under profiles/ are collected on")
    ap.add_argument("--probe", action="store_true", help="with --only: also launch the read-only probe on each copy")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device copy (known bytes) so that a rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE run of this command can scale its counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1\n")
        return 2

    import numpy as np
    import torch

    import mlc_llm_amd as gq
    from mlc_llm_amd import ops

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU\n")
        return 1
    if not os.path.exists(gq._lib.LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()
    gq._lib.call("mi355gq_check_device")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---------------------------------------------------------------- synthetic model, quantized on the GPU
    def make_weight(n, k, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        w = (torch.randn((n, k), generator=g, device=dev, dtype=torch.float32) * 0.02).half()
        return ops.quantize(w, BITS, G)

    if args.only:
        return run_only(args, dev, gq, ops, torch, make_weight)

    if args.prefill_only:
        n, k, m = *SHAPES["gate_up"], 2048
        qw, qs = make_weight(n, k, 2)
        xm = torch.randn((m, k), generator=torch.Generator(device=dev).manual_seed(1), device=dev).half()
        ym = torch.empty((m, n), dtype=torch.float16, device=dev)
        for _ in range(args.warmup):
            ops.linear(xm, qw, qs, BITS, G, None, torch.float16, ym)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            ops.linear(xm, qw, qs, BITS, G, None, torch.float16, ym)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.steps
        tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
        print(json.dumps({"metric": "q4f16_1 prefill GEMM, gate_up 28672x4096, M=2048", "value": round(tf, 1),
                          "unit": "TFLOP/s", "us_per_call": round(ms * 1e3, 1), "steps": args.steps,
                          "warmup": args.warmup, "frac_mfma": round(tf / MFMA_F16_PEAK_TFLOPS, 3),
                          "flop_per_call": 2 * m * n * k}))
        return 0

    layers = []
    for layer in range(LAYERS):
        layers.append({name: make_weight(n, k, 1000 * layer + i) for i, (name, (n, k)) in enumerate(SHAPES.items())})
    lm_head = make_weight(*LM_HEAD, 999_999)
    gx = torch.Generator(device=dev).manual_seed(1)
    x_in = {k: torch.randn((16, k), generator=gx, device=dev).half() for k in (4096, 14336)}
    outs = {name: torch.empty((16, n), dtype=torch.float16, device=dev) for name, (n, _) in SHAPES.items()}
    out_lm = torch.empty((16, LM_HEAD[0]), dtype=torch.float16, device=dev)
    torch.cuda.synchronize()

    def run_linear(name, qw, qs, b, out):
        n, k = qw.shape[0], (LM_HEAD[1] if name == "lm_head" else SHAPES[name][1])
        ops.linear(x_in[k][:b], qw, qs, BITS, G, None, torch.float16, out[:b])

    def decode_step(b=1):
        for lw in layers:
            for name in SHAPES:
                run_linear(name, lw[name][0], lw[name][1], b, outs[name])
        run_linear("lm_head", lm_head[0], lm_head[1], b, out_lm)

    step_bytes = LAYERS * sum(gemv_bytes(n, k) for n, k in SHAPES.values()) + gemv_bytes(*LM_HEAD)
    launches_per_step = LAYERS * len(SHAPES) + 1

    # ---------------------------------------------------------------- parity gate before timing
    from oracle import c_oracle
    from oracle import gq_oracle as o

    s4 = o.SCHEMES["q4f16_1"]
    x1_h = x_in[4096][:1].cpu().numpy()

    def sampled_parity(what, y, x, qw, qs, scheme, cols=384, rows=12):
        """y [M, N] against the oracle on sampled weight rows (first, last, tile edges, random) and sampled
        activation rows; the packed words and scales are copied from the tensors the kernel read."""
        rng = np.random.default_rng(len(what) + qw.shape[0])
        n, m = qw.shape[0], x.shape[0]
        ci = np.unique(np.concatenate([[0, 1, 127, 128, 255, 256, n // 2, n - 2, n - 1], rng.integers(0, n, cols)]))
        ri = np.arange(m) if m <= rows else np.unique(np.concatenate([[0, 1, 31, 32, 127, 128, 255, 256, m - 1],
                                                                      rng.integers(0, m, rows)]))
        ri = ri[ri < m]
        ct, rt = torch.from_numpy(ci).to(dev), torch.from_numpy(ri).to(dev)
        x_h = x[rt].cpu().numpy()
        ref = o.linear_fp32(x_h, qw[ct].cpu().numpy().view(np.uint32), qs[ct].cpu().numpy(), scheme)
        err, bound, rel = o.check_linear(y[rt][:, ct].float().cpu().numpy(), ref, x_h, x.shape[1])
        if not (err <= bound and rel <= 2e-3):
            raise SystemExit(f"parity check failed before timing ({what}): err {err} bound {bound} rel {rel}")

    # every shape the step runs, at every batch the extras time, before anything is timed
    for name, (n, k) in list(SHAPES.items()) + [("lm_head", LM_HEAD)]:
        qw_, qs_ = lm_head if name == "lm_head" else layers[0][name]
        out_ = out_lm if name == "lm_head" else outs[name]
        for b in (1, 4, 8, 16):
            run_linear(name, qw_, qs_, b, out_)
            sampled_parity(f"{name} B={b}", out_[:b], x_in[k][:b], qw_, qs_, s4)
    run_linear("gate_up", *layers[0]["gate_up"], 1, outs["gate_up"])
    dominant_kernel = gq._lib.last_kernel()  # the instantiation the dispatcher picked in this run

    # ---------------------------------------------------------------- timed region: K decode steps
    def timed(fn, iters, warmup, use_graph):
        """ms per call of fn, HIP events on the current (launch) stream."""
        if use_graph:
            fn()  # eager once: lazy init must not happen under capture
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn()
            call = graph.replay
        else:
            call = fn
        for _ in range(warmup):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            call()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    use_graph = not args.no_graph
    t_wall0 = time.perf_counter()
    ms_step = timed(decode_step, args.steps, args.warmup, use_graph)
    value = step_bytes / (ms_step * 1e-3) / 1e9

    # ---------------------------------------------------------------- roofline of the dominant kernel
    def gate_up_sweep():
        for lw in layers:
            run_linear("gate_up", lw["gate_up"][0], lw["gate_up"][1], 1, outs["gate_up"])

    ms_sweep = timed(gate_up_sweep, max(5, args.steps), 2, use_graph)
    us_gate_up = ms_sweep * 1e3 / LAYERS
    gu_bytes = gemv_bytes(*SHAPES["gate_up"])
    achieved = gu_bytes / (us_gate_up * 1e-6) / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "gemv_gate_up_traffic.json")
    if os.path.exists(tpath):
        with open(tpath, encoding="utf-8") as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")
    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(7)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    # the same tensors through the library's read-only probe (one launch per layer, 128-bit
    # loads, no arithmetic): what this device delivers for these bytes, measured in this run
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def read_sweep():
        for lw in layers:
            qw, qs = lw["gate_up"]
            gq._lib.call("mi355gq_testing_stream_read", qw.data_ptr(), qw.numel() * 4, qs.data_ptr(), qs.numel() * 2,
                      sink.data_ptr(), torch.cuda.current_stream().cuda_stream)

    us_read = timed(read_sweep, max(5, args.steps), 2, use_graph) * 1e3 / LAYERS
    read_bytes = layers[0]["gate_up"][0].numel() * 4 + layers[0]["gate_up"][1].numel() * 2

    # ... and the whole step through the probe: the same 129 launches in the same order, each only reading the weight
    # and scale tensors of its linear.  What separate launches over these tensors cost on this device when nothing is
    # computed: the floor for any implementation behind an operator-per-linear boundary.
    def probe_step():
        stream = torch.cuda.current_stream().cuda_stream
        for lw in layers:
            for name in SHAPES:
                qw, qs = lw[name]
                gq._lib.call("mi355gq_testing_stream_read", qw.data_ptr(), qw.numel() * 4, qs.data_ptr(), qs.numel() * 2,
                             sink.data_ptr(), stream)
        gq._lib.call("mi355gq_testing_stream_read", lm_head[0].data_ptr(), lm_head[0].numel() * 4, lm_head[1].data_ptr(),
                     lm_head[1].numel() * 2, sink.data_ptr(), stream)

    ms_probe_step = timed(probe_step, max(5, args.steps), 2, use_graph)
    roofline = {
        "bound": "hbm", "kernel": f"{dominant_kernel} (gate_up 28672x4096, batch 1)",
        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
        "traffic_source": "profiles/gemv_gate_up_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                          "command, scaled by a 256 MiB device copy in the same runs)",
        "bytes_per_launch": gu_bytes, "us_per_launch": round(us_gate_up, 3),
        "read_only_probe": {"what": "plain 128-bit streaming read of the same weight and scale tensors, one launch each",
                            "us_per_launch": round(us_read, 3),
                            "GB/s": round(read_bytes / (us_read * 1e-6) / 1e9, 1),
                            "gemv_time_over_probe_time": round(us_gate_up / us_read, 3),
                            "whole_step_ms": round(ms_probe_step, 4),
                            "whole_step_what": "the decode step's 129 launches with each linear replaced by the probe "
                                               "over its weight and scale tensors",
                            "step_time_over_probe_step_time": round(ms_step / ms_probe_step, 3)},
    }

    # ---------------------------------------------------------------- extra: per shape, batch 1/4/8/16, prefill GEMM
    extra = {}
    if not args.skip_extra:
        per_shape = {}
        for name, (n, k) in list(SHAPES.items()) + [("lm_head", LM_HEAD)]:
            for b in (1, 4, 8, 16):
                if name == "lm_head":
                    # 8 launches on the one lm_head (296 MB: larger than the 256 MB infinity cache)
                    def sweep(b=b):
                        for _ in range(8):
                            run_linear("lm_head", lm_head[0], lm_head[1], b, out_lm)
                    cnt = 8
                else:
                    def sweep(name=name, b=b):
                        for lw in layers:
                            run_linear(name, lw[name][0], lw[name][1], b, outs[name])
                    cnt = LAYERS
                us = timed(sweep, 5, 3, use_graph) * 1e3 / cnt  # (the first replays of a new graph run a few % slow)
                gbs = gemv_bytes(n, k, b) / (us * 1e-6) / 1e9
                per_shape[f"{name}_b{b}"] = {"us": round(us, 2), "GB/s": round(gbs, 1),
                                             "frac_hbm": round(gbs / HBM_PEAK_GBS, 3)}
        extra["gemv"] = per_shape
        gemm = {}
        m = 2048
        xm = {k: torch.randn((m, k), generator=gx, device=dev).half() for k in (4096, 14336)}
        for name, (n, k) in list(SHAPES.items()) + [("lm_head", LM_HEAD)]:
            qw, qs = lm_head if name == "lm_head" else layers[0][name]
            ym = torch.empty((m, n), dtype=torch.float16, device=dev)

            def call(qw=qw, qs=qs, k=k, ym=ym):
                ops.linear(xm[k], qw, qs, BITS, G, None, torch.float16, ym)
            call()
            sampled_parity(f"{name} M={m}", ym, xm[k], qw, qs, s4, cols=256, rows=16)
            # (the first ten to twenty launches of this kernel in a process run 5-30 % slow while the clocks settle)
            ms = timed(call, 30, 25 if name != "lm_head" else 10, False)
            tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
            gemm[f"{name}_m{m}"] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(tf, 1),
                                    "frac_mfma": round(tf / MFMA_F16_PEAK_TFLOPS, 3)}
            del ym
        extra["prefill_gemm"] = gemm
        for m2 in (256, 8192):  # the other two prefill sizes, on the largest per-layer shape
            n, k = SHAPES["gate_up"]
            xm2 = torch.randn((m2, k), generator=gx, device=dev).half()
            ym2 = torch.empty((m2, n), dtype=torch.float16, device=dev)
            qw, qs = layers[0]["gate_up"]
            ms = timed(lambda: ops.linear(xm2, qw, qs, BITS, G, None, torch.float16, ym2), 20 if m2 == 256 else 10,
                       20 if m2 == 256 else 6, False)
            tf = 2.0 * m2 * n * k / (ms * 1e-3) / 1e12
            gemm[f"gate_up_m{m2}"] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(tf, 1),
                                      "frac_mfma": round(tf / MFMA_F16_PEAK_TFLOPS, 3)}
            del xm2, ym2
        # context for the MFMA fractions: the vendor library's dense fp16 GEMM (torch's linear) on the
        # same shapes, weights already dequantised (4x the weight bytes, no unpacking in the loop)
        lib = {}
        for name in ("gate_up", "down"):
            n, k = SHAPES[name]
            wd = (torch.randn((n, k), generator=gx, device=dev) * 0.02).half()
            ms = timed(lambda: torch.nn.functional.linear(xm[k], wd), 20, 8, False)
            lib[f"{name}_m{m}"] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1)}
            del wd
        extra["library_dense_fp16_gemm_reference"] = lib
        # gate_up with silu(x1) * x2 folded into the matmul kernel, against the two calls it replaces
        fused = {}
        n, k = SHAPES["gate_up"]
        for mf in (1, 8, 2048):
            xf = xm[k][:mf].contiguous()
            sweep_layers = layers if mf <= 8 else layers[:1]  # one launch per layer's weights, as in the GEMV lines

            def run_fused():
                for lw in sweep_layers:
                    ops.linear_silu_mul(xf, lw["gate_up"][0], lw["gate_up"][1], BITS, G)

            def run_two():
                for lw in sweep_layers:
                    ops.silu_mul(ops.linear(xf, lw["gate_up"][0], lw["gate_up"][1], BITS, G))
            us_f = timed(run_fused, 5, 2, use_graph) * 1e3 / len(sweep_layers)
            us_2 = timed(run_two, 5, 2, use_graph) * 1e3 / len(sweep_layers)
            fused[f"m{mf}"] = {"fused_us": round(us_f, 1), "linear_then_silu_mul_us": round(us_2, 1)}
        extra["gate_up_silu_mul"] = fused
        del xm
        extra["decode_tokens_per_s_linear_only"] = round(1e3 / ms_step, 1)

        # what the runtime's own device-to-device copy reaches on this box (context for the HBM
        # fractions): 1 GiB copies between four distinct buffers, bytes = read + written
        bufs = [torch.ones(1024 * 1024 * 1024, dtype=torch.uint8, device=dev) for _ in range(4)]

        def copy_sweep():
            for i in range(4):
                bufs[(i + 1) % 4].copy_(bufs[i])
        ms = timed(copy_sweep, 3, 1, False) / 4
        extra["device_copy_reference"] = {"what": "1 GiB device-to-device copy, read + write bytes",
                                          "GB/s": round(2 * 2**30 / (ms * 1e-3) / 1e9, 1)}
        del bufs

        # q3f16_1 decode GEMV at Llama-2-7B shapes, batch 1 (the q3 configuration of the benchmark definition)
        q3 = {}
        for name, (n, k) in {"qkv": (12288, 4096), "o_proj": (4096, 4096), "gate_up": (22016, 4096),
                             "down": (4096, 11008)}.items():
            ng3 = -(-k // 40)
            copies = max(2, min(32, int(1.2e9 // (n * ng3 * 18))))
            ws = []
            for c in range(copies):
                g = torch.Generator(device=dev).manual_seed(5000 + c)
                w = (torch.randn((n, k), generator=g, device=dev) * 0.02).half()
                ws.append(ops.quantize(w, 3, 40))
                del w
            x3 = torch.randn((1, k), generator=gx, device=dev).half()
            y3 = torch.empty((1, n), dtype=torch.float16, device=dev)

            def sweep3():
                for qw, qs in ws:
                    ops.linear(x3, qw, qs, 3, 40, None, torch.float16, y3)
            us = timed(sweep3, 5, 1, use_graph) * 1e3 / copies
            nbytes = n * 4 * ng3 * 4 + n * ng3 * 2 + k * 2 + n * 2
            q3[name] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                        "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)}
            if name == "gate_up":  # the same matrix at batch 4 / 8 (quad-row kernel) and as a 2048-row prefill GEMM
                for m3 in (4, 8, 2048):
                    xm3 = torch.randn((m3, k), generator=gx, device=dev).half()
                    ym3 = torch.empty((m3, n), dtype=torch.float16, device=dev)

                    def sweep3m():
                        for qw, qs in ws[: (2 if m3 > 8 else len(ws))]:
                            ops.linear(xm3, qw, qs, 3, 40, None, torch.float16, ym3)
                    cnt3 = 2 if m3 > 8 else len(ws)
                    us = timed(sweep3m, 3, 1, use_graph and m3 <= 8) * 1e3 / cnt3
                    q3[f"gate_up_m{m3}"] = {"us": round(us, 2)}
                    if m3 > 8:
                        q3[f"gate_up_m{m3}"]["TFLOP/s"] = round(2.0 * m3 * n * k / us / 1e6, 1)
                    else:
                        q3[f"gate_up_m{m3}"]["GB/s"] = round(nbytes / us / 1e3, 1)
                    del xm3, ym3
            del ws
        extra["q3f16_1"] = q3

        # q4f16_1 Mixtral-8x7B MoE layer (the MoE configuration of the benchmark definition): 8 experts, top-2, T in {1, 16, 512}
        from mlc_llm_amd import QUANTIZATION
        from mlc_llm_amd.nn import MixtralMoE

        moe = MixtralMoE(4096, 14336, 8, 2, QUANTIZATION["q4f16_1"], device=dev)
        for e in range(8):
            g = torch.Generator(device=dev).manual_seed(7000 + e)
            w13 = (torch.randn((28672, 4096), generator=g, device=dev) * 0.02).half()
            moe.e1_e3.q_weight.data[e], moe.e1_e3.q_scale.data[e] = ops.quantize(w13, BITS, G)
            w2 = (torch.randn((4096, 14336), generator=g, device=dev) * 0.02).half()
            moe.e2.q_weight.data[e], moe.e2.q_scale.data[e] = ops.quantize(w2, BITS, G)
            del w13, w2
        g2 = torch.Generator(device=dev).manual_seed(2)
        moe_res = {}
        for t in (1, 16, 32, 64, 512):
            xt = torch.randn((1, t, 4096), generator=gx, device=dev).half()
            logits = torch.randn((t, 8), generator=g2, device=dev).half()
            ms = timed(lambda: moe(xt, logits), 10, 2, use_graph)
            ids = ops.gating_softmax_topk(logits, 2)[1]
            distinct = int(torch.unique(ids).numel())
            wbytes = distinct * 99_090_432
            flops = 2.0 * t * 2 * (28672 * 4096 + 4096 * 14336)
            moe_res[f"T{t}"] = {"us": round(ms * 1e3, 1), "experts_touched": distinct,
                                "weight_GB/s": round(wbytes / (ms * 1e-3) / 1e9, 1),
                                "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 2)}
        extra["mixtral_moe_layer"] = moe_res
        del moe

        # packing, unpacking and the embedding gather: HBM-bound byte work, algorithmic bytes =
        # fp16 matrix + packed words + scales (each once)
        pk = {}
        n, k = SHAPES["gate_up"]
        wq = (torch.randn((n, k), generator=gx, device=dev) * 0.02).half()
        for bits_, g_ in ((4, 32), (3, 40)):
            kq = k if bits_ == 4 else (k // 40) * 40
            wv = wq[:, :kq].contiguous()
            qwq, qsq = ops.quantize(wv, bits_, g_)
            nbytes = wv.numel() * 2 + qwq.numel() * 4 + qsq.numel() * 2
            ms = timed(lambda: ops.quantize(wv, bits_, g_), 5, 2, False)
            pk[f"quantize_q{bits_}_gate_up"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
            ms = timed(lambda: ops.dequantize(qwq, qsq, kq, bits_, g_), 5, 2, False)
            pk[f"dequantize_q{bits_}_gate_up"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
            del wv, qwq, qsq
        del wq
        ids = torch.randint(0, LM_HEAD[0], (8192,), generator=gx, device=dev, dtype=torch.int32)
        ms = timed(lambda: ops.embedding_take(ids, lm_head[0], lm_head[1], LM_HEAD[1], BITS, G), 5, 2, False)
        row_bytes = LM_HEAD[1] // G * 18 + LM_HEAD[1] * 2  # packed row + scales read, fp16 row written
        pk["embedding_take_8192_tokens"] = {"us": round(ms * 1e3, 1), "GB/s": round(8192 * row_bytes / ms / 1e6, 1)}
        extra["packing"] = pk

        # KN-layout tensors (q4f16_0: q_weight [nw, N], q_scale [ng, N]) through mi355gq_linear_kn: the GEMV that streams them
        # as stored, on rotating copies of the transposed gate_up / o_proj tensors of the first layers
        kn = {}
        for name in ("o_proj", "gate_up"):
            n, k = SHAPES[name]
            cnt = min(LAYERS, 16)
            kn_w = [ops.nk_to_kn(layers[i][name][0], layers[i][name][1], k, BITS, G) for i in range(cnt)]
            for b in (1, 4, 8):
                xb = torch.randn((b, k), generator=gx, device=dev).half()
                def sweep(xb=xb, kn_w=kn_w):
                    for qw_kn, qs_kn in kn_w:
                        ops.linear_kn(xb, qw_kn, qs_kn, BITS, G)
                us = timed(sweep, 5, 3, use_graph) * 1e3 / cnt
                kn[f"{name}_b{b}"] = {"us": round(us, 2), "GB/s": round(gemv_bytes(n, k, b) / (us * 1e-6) / 1e9, 1)}
            del kn_w
        extra["kn_layout_gemv"] = kn

        # the other model dtypes of the registry (q4bf16_1, q4f32_1) on the gate_up shape: packing,
        # batch-1 GEMV (weight bytes per second) and the M = 2048 GEMM
        other = {}
        n, k = SHAPES["gate_up"]
        for label, dt in (("q4bf16_1", torch.bfloat16), ("q4f32_1", torch.float32)):
            wd = (torch.randn((n, k), generator=gx, device=dev) * 0.02).to(dt)
            qwd, qsd = ops.quantize(wd, 4, 32)
            el = wd.element_size()
            nbytes = wd.numel() * el + qwd.numel() * 4 + qsd.numel() * el
            res = {}
            ms = timed(lambda: ops.quantize(wd, 4, 32), 5, 2, False)
            res["quantize"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
            ms = timed(lambda: ops.dequantize(qwd, qsd, k, 4, 32), 5, 2, False)
            res["dequantize"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
            del wd
            x1 = torch.randn((1, k), generator=gx, device=dev).to(dt)
            def sweep8(xs):  # eight launches per graph replay, so that replay overhead does not show
                for _ in range(8):
                    ops.linear(xs, qwd, qsd, 4, 32)
            ms = timed(lambda: sweep8(x1), 10, 3, use_graph) / 8
            res["gemv_b1"] = {"us": round(ms * 1e3, 1),
                              "GB/s": round((qwd.numel() * 4 + qsd.numel() * el + (k + n) * el) / ms / 1e6, 1)}
            x4 = torch.randn((4, k), generator=gx, device=dev).to(dt)
            ms = timed(lambda: sweep8(x4), 10, 3, use_graph) / 8
            res["gemv_b4"] = {"us": round(ms * 1e3, 1),
                              "GB/s": round((qwd.numel() * 4 + qsd.numel() * el + 4 * (k + n) * el) / ms / 1e6, 1)}
            xm_ = torch.randn((2048, k), generator=gx, device=dev).to(dt)
            ms = timed(lambda: ops.linear(xm_, qwd, qsd, 4, 32), 6 if dt == torch.bfloat16 else 3, 2, False)
            res["gemm_m2048"] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(2.0 * 2048 * n * k / ms / 1e9, 1),
                                 "matrix_instruction": "v_mfma_f32_32x32x16_bf16" if dt == torch.bfloat16
                                 else "v_mfma_f32_32x32x2_f32 (157 TFLOP/s peak)"}
            other[label] = res
            del qwd, qsd, x1, x4, xm_
        extra["other_model_dtypes"] = other

    # ---------------------------------------------------------------- CPU baseline (bounded sample)
    cpu = None
    if not args.skip_cpu:
        n, k = SHAPES["gate_up"]
        qw_h = layers[0]["gate_up"][0].cpu().numpy().view(np.uint32)
        qs_h = layers[0]["gate_up"][1].cpu().numpy()
        scratch = np.empty(k, np.float32)
        out_h = np.empty((1, n), np.float32)
        c_oracle.linear(x1_h, qw_h, qs_h, BITS, G, None, scratch, out_h)  # warm-up + parity
        run_linear("gate_up", *layers[0]["gate_up"], 1, outs["gate_up"])
        gpu_y = outs["gate_up"][:1].float().cpu().numpy()
        cerr = float(np.abs(gpu_y - out_h).max())
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0:
            c_oracle.linear(x1_h, qw_h, qs_h, BITS, G, None, scratch, out_h)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        cpu = {
            "value": round(gu_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": c_oracle.num_threads(),
            "kind": "port",
            "sample": f"gate_up 28672x4096 q4f16_1 GEMV, batch 1, {reps} calls in 10 s "
                      "(C restatement of the reference loop nest, OpenMP over N; TVM's llvm build "
                      "is not available offline)",
            "us_per_call": round(dt * 1e6, 1), "max_abs_diff_vs_gpu": cerr,
        }

    line = {
        "metric": "q4f16_1 dequant-GEMV GB/s (% of HBM peak), Llama-3-8B decode; prefill TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 in/out, f32 accumulate, u32 packed int4",
        "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B q4f16_1 decode linears, batch 1: 32 x (qkv 6144x4096, o 4096x4096, "
                        "gate_up 28672x4096, down 4096x14336) + lm_head 128256x4096 "
                        "(BASELINE configs[1], B=1)",
            "launches_per_step": launches_per_step, "bytes_per_step": step_bytes,
            "hip_graph": use_graph, "group_size": G, "bits": BITS,
        },
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
        "wall_s": round(time.perf_counter() - t_wall0, 1),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
