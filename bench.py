#!/usr/bin/env python3
"""Benchmark of the FP8 quantized-matmul path on one MI355X.

A step is one pass of the whole path over the Qwen2.5-7B MLP at 8192 tokens (configuration 4 of
BASELINE.json): for the fused gate+up linear (3584 -> 37888) and the down linear (18944 -> 3584),
forward + dgrad + wgrad, with every abs-max, quantize, transpose and quantize+transpose launch the
reference's forward_qmm / backward_qmm issue (src/models/llama_model.cpp:25-47, 309-339), plus the
per-step weight abs-max + quantize (src/models/llama_weights.cpp:207-223).  Inputs are synthetic and
already resident in HBM when the timed region starts.

One JSON line is printed:
  value           e4m3 GEMM TFLOP/s of the whole step: 2*M*N*K summed over the six GEMMs divided by the
                  step time (abs-max / quantize / transpose launches included in the time)
  roofline        the GEMM kernel alone: algorithmic FLOP / mean launch duration (HIP events around
                  each GEMM launch inside the timed steps) against the dense FP8 MFMA peak
  quantize        abs-max + quantize (+transpose) launches: algorithmic bytes / event-timed duration
                  against 8 TB/s, inside the step (events around these launches are recorded in a second pass over the
                  same steps, right after the timed ones, so that the timed steps carry events around the GEMMs only); quantize.cold_large_tensor holds the same kernels timed
                  on their own on 310 MB tensors that no cache holds (median of 20 launches)
  cpu_baseline    the multithreaded CPU port of the same path on a bounded sample (host cores of this box)
  gemm_error      max-abs and relative-Frobenius error of each of the six GEMMs against the exact product of the same
                  e4m3 operands (sampled outputs; computed with the CPU oracle beside the CPU baseline)
Extra fields: roofline.mfma_only_ceiling_TFLOPs (register-only matrix-instruction loops: what the chip sustains
under its power limit), roofline.sensors_under_step_load (the driver's package power and shader clock, sampled while the
steps run once more after the timed region), roofline.traffic (hardware-counter bytes per GEMM launch, from profiles/), hip_graph_replay
(the same step replayed from a HIP graph), fused_quantize_transpose_step (the step with the single-read
quantize + transposed-copy extension), direct_gradient_layout_step (the step with the backward matmuls reading
weights, activations and output gradients in their stored layouts, matmul modes NN / NT / TT, instead of transposed
copies), vendor_gemm (torch._scaled_mm, i.e. hipBLASLt, on the six GEMM shapes,
alternating with this library's GEMM: context for the roofline fraction, not part of the path).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0   # MI355X dense FP8 MFMA peak
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E

BT, C, FFN = 8192, 3584, 18944
UP = 2 * FFN  # fused gate+up output features


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # A step takes 4.4 ms.  The chip needs about 50 ms of this load before its clock settles (measured: the GEMM
    # launches of timed steps 1-10 after 3 warm-up steps run 2 % slower than those after 10 warm-up steps or the later
    # ones of 30 timed steps), so the defaults leave that transient to the warm-up and time a steady 0.2 s.
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the step")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB copy kernel (reference point for hardware traffic counters)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="rough budget of the CPU baseline sample")
    ap.add_argument("--hbm-kernels-only", action="store_true",
                    help="run only the cold-tensor section of the HBM-bound kernels (abs-max, quantize, quantize+transpose, "
                         "transpose, plain copy) and print its figures: the workload of the profiles named hbm_kernels__*")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); multi-GPU sharding is a design note, "
              "not a code path", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from llmq_amd import capi, kernels as K   # fails loudly if the HIP library is missing

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(4)

    def randn(shape, std):
        return (torch.randn(shape, device=dev, generator=gen, dtype=torch.float32) * std).to(torch.bfloat16)

    # ---- synthetic tensors (configuration 4) ----
    t = {
        "x": randn((BT, C), 1.0), "w_up": randn((UP, C), 0.015),
        "h": randn((BT, FFN), 1.0), "w_down": randn((C, FFN), 0.015),
        "dy_up": randn((BT, UP), 1e-4), "dy_down": randn((BT, C), 1e-4),
    }
    f8 = torch.float8_e4m3fn
    e = lambda *s: torch.empty(s, dtype=f8, device=dev)
    q = {"x": e(BT, C), "w_up": e(UP, C), "h": e(BT, FFN), "w_down": e(C, FFN), "dy_up": e(BT, UP), "dy_down": e(BT, C),
         "w_up_t": e(C, UP), "w_down_t": e(FFN, C), "x_t": e(C, BT), "h_t": e(FFN, BT), "dy_up_t": e(UP, BT),
         "dy_down_t": e(C, BT)}
    stats = {k: torch.zeros(2, device=dev) for k in t}   # [abs_max, scale] pairs, as Tensor::Stats in the reference
    out = {"y_up": torch.empty((BT, UP), dtype=torch.bfloat16, device=dev),
           "y_down": torch.empty((BT, C), dtype=torch.bfloat16, device=dev),
           "dh": torch.empty((BT, FFN), dtype=torch.bfloat16, device=dev),
           "dx": torch.empty((BT, C), dtype=torch.bfloat16, device=dev),
           "dw_up": torch.empty((UP, C), dtype=torch.bfloat16, device=dev),
           "dw_down": torch.empty((C, FFN), dtype=torch.bfloat16, device=dev)}

    ws = torch.empty(32 << 20, dtype=torch.uint8, device=dev)   # matmul workspace, sized as in the reference
    timers = {}   # name -> list of (start, end, work) ; work in bytes or flop
    # 0: no events; 1: events around the GEMM launches only (the timed steps); 2: events around every other launch
    # (a second, instrumented pass over the same steps: the figures of the quantize section come from there, so that
    # the timed steps carry 12 event records instead of 70)
    record = [0]

    def timed(name, work, fn):
        if (record[0] == 1) == (name == "gemm") and record[0] != 0:
            s, f = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            fn()
            f.record()
            timers.setdefault(name, []).append((s, f, work))
        else:
            fn()

    def absmax_and_quantize(name):
        n = t[name].numel()
        timed("abs_max", 2 * n, lambda: K.abs_max(stats[name][0:1], t[name]))
        timed("quantize", 3 * n, lambda: K.quantize_with_abs_max(q[name], stats[name][1:2], t[name], stats[name][0:1]))

    def gemm(c, a, b, sa, sb, M, N, Kd, b_kmajor=False, a_kmajor=False):
        timed("gemm", 2.0 * M * N * Kd, lambda: K.matmul(c, a, b, None, sa, sb, M, N, Kd, workspace=ws, b_kmajor=b_kmajor,
                                                         a_kmajor=a_kmajor))
        if record[0] == 1:
            timers["gemm"][-1] += ("M%d_N%d_K%d" % (M, N, Kd),)

    def tr(dst, src):
        timed("transpose", 2 * src.numel(), lambda: K.transpose(dst, src))

    def qtr(dst, name):
        timed("quantize_transpose", 3 * t[name].numel(),
              lambda: K.quantize_and_transpose_with_abs_max(dst, None, t[name], stats[name][0:1]))

    def step():
        # weights: abs-max + quantize once per step (they change every optimizer step)
        absmax_and_quantize("w_up")
        absmax_and_quantize("w_down")
        # forward gate+up, down
        absmax_and_quantize("x")
        gemm(out["y_up"], q["w_up"], q["x"], stats["w_up"][1:2], stats["x"][1:2], UP, BT, C)
        absmax_and_quantize("h")
        gemm(out["y_down"], q["w_down"], q["h"], stats["w_down"][1:2], stats["h"][1:2], C, BT, FFN)
        # backward down: dgrad dH = dY W, wgrad dW = dY^T H
        absmax_and_quantize("dy_down")
        tr(q["w_down_t"], q["w_down"])
        gemm(out["dh"], q["w_down_t"], q["dy_down"], stats["w_down"][1:2], stats["dy_down"][1:2], FFN, BT, C)
        qtr(q["h_t"], "h")
        tr(q["dy_down_t"], q["dy_down"])
        gemm(out["dw_down"], q["h_t"], q["dy_down_t"], stats["h"][1:2], stats["dy_down"][1:2], FFN, C, BT)
        # backward gate+up
        absmax_and_quantize("dy_up")
        tr(q["w_up_t"], q["w_up"])
        gemm(out["dx"], q["w_up_t"], q["dy_up"], stats["w_up"][1:2], stats["dy_up"][1:2], C, BT, UP)
        qtr(q["x_t"], "x")
        tr(q["dy_up_t"], q["dy_up"])
        gemm(out["dw_up"], q["x_t"], q["dy_up_t"], stats["x"][1:2], stats["dy_up"][1:2], C, UP, BT)

    def both(name, dst_t):
        n = t[name].numel()
        timed("quantize_both", 4 * n, lambda: K.quantize_with_abs_max_and_transpose(
            q[name], dst_t, stats[name][1:2], t[name], stats[name][0:1]))

    def step_fused():
        """Same results with the library's single-read "quantize + transposed copy" kernel wherever the
        reference sequence runs quantize_with_abs_max and transpose back to back on one tensor (weights, output
        gradients): 4 instead of 5 bytes per element and one launch less."""
        timed("abs_max", 0, lambda: K.abs_max(stats["w_up"][0:1], t["w_up"]))
        both("w_up", q["w_up_t"])
        timed("abs_max", 0, lambda: K.abs_max(stats["w_down"][0:1], t["w_down"]))
        both("w_down", q["w_down_t"])
        absmax_and_quantize("x")
        gemm(out["y_up"], q["w_up"], q["x"], stats["w_up"][1:2], stats["x"][1:2], UP, BT, C)
        absmax_and_quantize("h")
        gemm(out["y_down"], q["w_down"], q["h"], stats["w_down"][1:2], stats["h"][1:2], C, BT, FFN)
        timed("abs_max", 0, lambda: K.abs_max(stats["dy_down"][0:1], t["dy_down"]))
        both("dy_down", q["dy_down_t"])
        gemm(out["dh"], q["w_down_t"], q["dy_down"], stats["w_down"][1:2], stats["dy_down"][1:2], FFN, BT, C)
        qtr(q["h_t"], "h")
        gemm(out["dw_down"], q["h_t"], q["dy_down_t"], stats["h"][1:2], stats["dy_down"][1:2], FFN, C, BT)
        timed("abs_max", 0, lambda: K.abs_max(stats["dy_up"][0:1], t["dy_up"]))
        both("dy_up", q["dy_up_t"])
        gemm(out["dx"], q["w_up_t"], q["dy_up"], stats["w_up"][1:2], stats["dy_up"][1:2], C, BT, UP)
        qtr(q["x_t"], "x")
        gemm(out["dw_up"], q["x_t"], q["dy_up_t"], stats["x"][1:2], stats["dy_up"][1:2], C, UP, BT)

    def step_direct():
        """The step as backward_qmm issues it with DirectGradLayout: the matmuls read their operands where they lie
        (matmul modes NN / NT / TT) wherever that is cheaper than a transposed copy.  Weights: no transposed copies (both
        dgrads in mode NN).  Down projection: the weight gradient reads h and dY in place (mode NT; h is quantized
        again, as the reference's path without a retained quantized input does, but not transposed).  Gate+up: the weight
        gradient reads dY[8192, 37888] in place (mode TT) and keeps the quantize+transpose of the small x."""
        absmax_and_quantize("w_up")
        absmax_and_quantize("w_down")
        absmax_and_quantize("x")
        gemm(out["y_up"], q["w_up"], q["x"], stats["w_up"][1:2], stats["x"][1:2], UP, BT, C)
        absmax_and_quantize("h")
        gemm(out["y_down"], q["w_down"], q["h"], stats["w_down"][1:2], stats["h"][1:2], C, BT, FFN)
        absmax_and_quantize("dy_down")
        gemm(out["dh"], q["w_down"], q["dy_down"], stats["w_down"][1:2], stats["dy_down"][1:2], FFN, BT, C, a_kmajor=True)
        timed("quantize", 3 * t["h"].numel(), lambda: K.quantize_with_abs_max(q["h"], stats["h"][1:2], t["h"], stats["h"][0:1]))
        gemm(out["dw_down"], q["h"], q["dy_down"], stats["h"][1:2], stats["dy_down"][1:2], FFN, C, BT, a_kmajor=True, b_kmajor=True)
        absmax_and_quantize("dy_up")
        gemm(out["dx"], q["w_up"], q["dy_up"], stats["w_up"][1:2], stats["dy_up"][1:2], C, BT, UP, a_kmajor=True)
        qtr(q["x_t"], "x")
        gemm(out["dw_up"], q["x_t"], q["dy_up"], stats["x"][1:2], stats["dy_up"][1:2], C, UP, BT, b_kmajor=True)

    gemm_flop = 3 * (2.0 * UP * BT * C) + 3 * (2.0 * C * BT * FFN)

    # Part of the set-up, like the allocations above: from idle the chip takes about 50 ms of this load to bring its clock
    # up (see --warmup), so a caller that asks for fewer than 20 warm-up steps gets the difference here, before them.
    for _ in range(max(0, 20 - args.warmup)):
        step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.hbm_kernels_only:
        args.steps, args.no_graph, args.no_cpu_baseline = 1, True, True   # nothing but the cold section below
    record[0] = 1
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    record[0] = 2
    sensors = SensorSampler(enabled=not args.hbm_kernels_only and args.steps >= 20)   # package power and shader clock while the second pass runs (never during the timed one)
    for i_step in range(max(args.steps, 150 if sensors.available else 0)):   # 0.6 s of load: the sensors need it
        if i_step == args.steps:
            record[0] = 0       # events only around the first args.steps steps
        step()
    torch.cuda.synchronize()
    sensor_report = sensors.stop()
    record[0] = 0

    # Samples for the error report (gemm_error): operands, scales and sampled outputs of the six GEMMs are taken
    # now, while the buffers hold the step's values; the oracle evaluates them in the CPU leg at the end.
    error_samples = None
    if not args.no_cpu_baseline:
        gemms = [("gate_up fwd", out["y_up"], q["w_up"], q["x"], "w_up", "x"),
                 ("down fwd", out["y_down"], q["w_down"], q["h"], "w_down", "h"),
                 ("down dgrad", out["dh"], q["w_down_t"], q["dy_down"], "w_down", "dy_down"),
                 ("down wgrad", out["dw_down"], q["h_t"], q["dy_down_t"], "h", "dy_down"),
                 ("gate_up dgrad", out["dx"], q["w_up_t"], q["dy_up"], "w_up", "dy_up"),
                 ("gate_up wgrad", out["dw_up"], q["x_t"], q["dy_up_t"], "x", "dy_up")]
        error_samples = collect_gemm_samples(gemms, stats, np, torch)

    # The same step recorded once into a HIP graph and replayed (the reference replays its transformer
    # block from a graph as well, src/models/llama_model.cpp:49-71): removes the launch gaps.
    graph_ms = None
    if not args.no_graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        graph.replay()
        torch.cuda.synchronize()
        g0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - g0) * 1e3 / args.steps
    # The two extension sequences, timed in alternation (three rounds of args.steps steps each, median round), so that
    # clock and temperature drift over the run touches both alike.  The gate+up dW of the direct-layout sequence must
    # equal the materialised route's bit for bit.
    fused_ms, direct_ms, direct_identical = None, None, None
    if not args.no_graph:
        def ms_of(fn):
            torch.cuda.synchronize()
            f0 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - f0) * 1e3 / args.steps
        step_fused()
        want = [out[k].clone() for k in ("dh", "dw_down", "dx", "dw_up")]
        step_direct()
        torch.cuda.synchronize()
        # bit for bit, except where the materialised route cuts its last round of tiles into K segments (dw_down):
        # other partial sums, same tolerance
        direct_identical = {k: bool(torch.equal(out[k], w)) for k, w in zip(("dh", "dw_down", "dx", "dw_up"), want)}
        del want
        rounds = [(ms_of(step_fused), ms_of(step_direct)) for _ in range(3)]
        fused_ms = sorted(r[0] for r in rounds)[1]
        direct_ms = sorted(r[1] for r in rounds)[1]
    vendor = None
    if not args.no_graph and hasattr(torch, "_scaled_mm"):
        one = torch.ones(1, device=dev)
        shapes = [("gate_up fwd", q["w_up"], q["x"], out["y_up"]), ("down fwd", q["w_down"], q["h"], out["y_down"]),
                  ("down dgrad", q["w_down_t"], q["dy_down"], out["dh"]), ("down wgrad", q["h_t"], q["dy_down_t"], out["dw_down"]),
                  ("gate_up dgrad", q["w_up_t"], q["dy_up"], out["dx"]), ("gate_up wgrad", q["x_t"], q["dy_up_t"], out["dw_up"])]

        def us_of(fn, iters=5):
            fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters * 1e3

        try:
            per_shape, ours_total, theirs_total = {}, 0.0, 0.0
            for name, a_op, b_op, c_out in shapes:
                M_, Kd_ = a_op.shape
                N_ = b_op.shape[0]
                mine = lambda: K.matmul(c_out, a_op, b_op, None, one, one, M_, N_, Kd_, workspace=ws)
                theirs = lambda: torch._scaled_mm(b_op, a_op.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
                t_mine = min(us_of(mine), us_of(mine))
                t_theirs = min(us_of(theirs), us_of(theirs))
                t_mine = min(t_mine, us_of(mine))
                t_theirs = min(t_theirs, us_of(theirs))
                flop = 2.0 * M_ * N_ * Kd_
                per_shape[name] = {"this_library_TFLOPs": flop / t_mine / 1e6, "vendor_TFLOPs": flop / t_theirs / 1e6}
                ours_total += t_mine
                theirs_total += t_theirs
            vendor = {"what": "torch._scaled_mm (hipBLASLt) on the same e4m3 operands, bf16 output, best of 3 x 5 launches, "
                              "alternating with this library", "per_shape": per_shape,
                      "six_gemms_us": {"this_library": ours_total, "vendor": theirs_total},
                      "speed_vs_vendor": theirs_total / ours_total}
        except Exception as ex:   # the comparison is context only; a torch build without fp8 support skips it
            vendor = {"skipped": str(ex)[:200]}
    # The activation between the two projections and its gradient (the producers of `h` and `dy_up`), with
    # the abs-max of their outputs computed on the way: not part of the step above, which starts from given
    # tensors as BASELINE.json's configuration does; reported for the next stage of the path.
    swiglu = None
    if not args.no_graph:
        def gbs(fn, nbytes, iters=5):
            fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / iters * 1e3
            return {"GBps": nbytes / us / 1e3, "frac_hbm": nbytes / us / 1e3 / HBM_PEAK_GBS, "mean_us": us}

        y3, h3, dh3, dy3 = (v.view(1, BT, -1) for v in (out["y_up"], t["h"], out["dh"], t["dy_up"]))
        hq3 = q["h"].view(1, BT, -1)
        n_act = BT * FFN
        sw_am, sw_sc = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
        swiglu = {
            "what": "producers of the projections' inputs with the abs-max of their output computed on the way: "
                    "h = swiglu(y_up) [8192 x 18944], the same as e4m3 codes, its backward, the residual add + rmsnorm [8192 x 3584] "
                    "and the rmsnorm backward, the AdamW step of a weight; backward_bias on e4m3 gradients and the e5m2 "
                    "gradient dtype (quantize, matmul)",
            "swiglu_forward+abs_max (6 B/el)": gbs(lambda: K.swiglu_forward(h3, y3, sw_am), 6 * n_act),
            "swiglu_forward_quant (5 B/el)": gbs(lambda: K.swiglu_forward_quant(hq3, sw_sc, y3, sw_am), 5 * n_act),
            "swiglu_backward+abs_max (10 B/el)": gbs(lambda: K.swiglu_backward(dy3, dh3, y3, sw_am), 10 * n_act),
        }
        # x = rmsnorm(residual + attention output) [8192 x 3584], the producer of the gate+up projection's input
        x3 = t["x"].view(1, BT, C)
        r_in, r_att = torch.randn_like(x3), torch.randn_like(x3)
        r_out, r_norm, r_rms = torch.empty_like(x3), torch.empty_like(x3), torch.empty((1, BT), device=dev)
        r_w = torch.ones(C, dtype=torch.bfloat16, device=dev)
        # dy_down = rmsnorm_backward(...) [8192 x 3584], the producer of the down projection's gradient input
        r_scr = torch.empty(K.get_rmsnorm_backward_scratch_size(C), dtype=torch.float32, device=dev)
        r_dw = torch.zeros(C, dtype=torch.bfloat16, device=dev)
        r_rstd = torch.ones((1, BT), device=dev)
        swiglu["rmsnorm_backward+abs_max (8 B/el)"] = gbs(
            lambda: K.rmsnorm_backward(r_out, r_dw, r_scr, r_att, out["dx"].view(1, BT, C), r_in, r_w, r_rstd, sw_am),
            8 * BT * C, iters=10)
        # the optimizer step on W_up [37888 x 3584] with bf16 moments: its epilogue is the weight abs-max of the next step
        a_m, a_v = torch.zeros_like(t["w_up"]), torch.zeros_like(t["w_up"])
        a_p, a_g = t["w_up"].clone(), (1e-3 * torch.randn_like(t["w_up"]))
        a_gs = torch.ones(1, device=dev)
        swiglu["adamw_update+abs_max, bf16 moments (14 B/param)"] = gbs(
            lambda: K.adamw_update(a_p, a_g, a_m, a_v, 1e-4, 0.9, 0.95, 2, 1e-8, 0.1, a_gs, None, sw_am, 7), 14 * UP * C)
        del a_m, a_v, a_p, a_g
        # backward_bias on the quantized gradient of the attention's QKV projection (the 7B model's
        # [8192 x 4608], e4m3 codes with two scales): the other consumer of the quantized gradient bytes
        QKV = C + 2 * 512
        bb_dout = q["dy_up"].view(-1)[:BT * QKV].view(1, BT, QKV)
        bb_dbias = torch.zeros(QKV, dtype=torch.bfloat16, device=dev)
        bb_scr = torch.empty(K.get_bias_backward_scratch_size(f8, QKV, BT) // 4, dtype=torch.float32, device=dev)
        swiglu["backward_bias e4m3 [8192 x 4608] (1 B/el)"] = gbs(
            lambda: K.backward_bias(bb_dbias, bb_dout, sw_sc, sw_sc, bb_scr), BT * QKV, iters=10)
        # the e5m2 gradient dtype: quantize to e5m2 and the e4m3 x e5m2 matmul (gate+up dgrad shape)
        g5 = torch.empty((BT, UP), dtype=torch.float8_e5m2, device=dev)
        swiglu["quantize to e5m2 [8192 x 37888] (3 B/el)"] = gbs(
            lambda: K.quantize_with_abs_max(g5, sw_sc, t["dy_up"], stats["dy_up"][0:1]), 3 * BT * UP)
        e5_us = min(gbs(lambda: K.matmul(out["dx"], q["w_up_t"], g5, None, stats["w_up"][1:2], sw_sc, C, BT, UP, workspace=ws), 1)["mean_us"]
                    for _ in range(3))
        swiglu["matmul e4m3 x e5m2, gate_up dgrad shape"] = {"TFLOPs": 2.0 * C * BT * UP / e5_us / 1e6, "us": e5_us,
                                                             "timing": "best of 3 x 5 launches"}
        del g5
        swiglu["fused_residual_rmsnorm_forward+abs_max (8 B/el)"] = gbs(
            lambda: K.fused_residual_rmsnorm_forward(r_out, r_norm, r_rms, r_in, r_att, r_w, sw_am, 1e-6), 8 * BT * C, iters=10)
        # the fp32 overloads of the same producers (an fp32 model in front of FP8 matmuls): twice the bytes per element
        f_y = torch.randn((1, BT // 2, 2 * FFN), device=dev)
        f_h, f_dh, f_dy = torch.empty((1, BT // 2, FFN), device=dev), torch.randn((1, BT // 2, FFN), device=dev), torch.empty_like(f_y)
        n32 = (BT // 2) * FFN
        swiglu["fp32 swiglu_forward+abs_max [4096 x 18944] (12 B/el)"] = gbs(lambda: K.swiglu_forward(f_h, f_y, sw_am), 12 * n32)
        swiglu["fp32 swiglu_backward+abs_max [4096 x 18944] (20 B/el)"] = gbs(lambda: K.swiglu_backward(f_dy, f_dh, f_y, sw_am), 20 * n32)
        del f_y, f_h, f_dh, f_dy
        f_in, f_att = torch.randn((1, BT, C), device=dev), torch.randn((1, BT, C), device=dev)
        f_out, f_norm, f_w, f_dw = torch.empty_like(f_in), torch.empty_like(f_in), torch.ones(C, device=dev), torch.zeros(C, device=dev)
        swiglu["fp32 fused_residual_rmsnorm_forward+abs_max (16 B/el)"] = gbs(
            lambda: K.fused_residual_rmsnorm_forward(f_out, f_norm, r_rms, f_in, f_att, f_w, sw_am, 1e-6), 16 * BT * C, iters=10)
        swiglu["fp32 rmsnorm_backward+abs_max (16 B/el)"] = gbs(
            lambda: K.rmsnorm_backward(f_out, f_dw, r_scr, f_att, f_norm, f_in, f_w, r_rstd, sw_am), 16 * BT * C, iters=10)
        f_tab = K.precompute_freqs_cis(128, 2048, 1e6, dtype=torch.float32).to(dev)
        f_qkv = torch.randn((BT // 2048, 2048, 4608), device=dev)
        swiglu["fp32 rope_forward+abs_max in place [8192 x 4608] (q, k heads 8 B/el, v heads 4)"] = gbs(
            lambda: K.rope_forward(f_qkv, f_qkv, f_tab, sw_am, 28, 4), BT * 128 * (32 * 8 + 4 * 4), iters=10)
        del f_in, f_att, f_out, f_norm, f_qkv
    # The HBM-bound kernels on their own, cold: 5 warm-up and 20 timed launches each, one pair of events per
    # launch, rotating through three distinct 310 MB tensors (930 MB, well beyond the 256 MB last-level cache,
    # so every launch reads from HBM); median and best launch.  The in-step figures above include what the
    # previous kernel left in the cache and the launch gaps of tensors as small as 59 MB.
    def cold_section():
        n_h = BT * FFN
        srcs = [t["h"], out["dh"], out["y_up"].view(-1)[:n_h].view(BT, FFN)]
        q_srcs = [q["h"], q["dy_up"].view(-1)[:n_h].view(BT, FFN), q["dy_up"].view(-1)[n_h:].view(BT, FFN)]
        am3 = [torch.zeros(1, device=dev) for _ in srcs]
        for a, s_ in zip(am3, srcs):
            K.abs_max(a, s_)

        def cold_run(fn, nbytes, warm=5, timed=20):
            for i in range(warm):
                fn(i % 3)
            evs = []
            for i in range(timed):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn((warm + i) % 3)
                e1.record()
                evs.append((e0, e1))
            torch.cuda.synchronize()
            us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in evs)
            med = 0.5 * (us[len(us) // 2] + us[(len(us) - 1) // 2])
            return {"median_us": med, "min_us": us[0], "GBps": nbytes / med / 1e3, "frac_hbm": nbytes / med / 1e3 / HBM_PEAK_GBS,
                    "best_GBps": nbytes / us[0] / 1e3}

        q_dsts = q_srcs                                   # three distinct 155 MB outputs as well
        qt_dsts = [q["h_t"], q["dy_up_t"].view(-1)[:n_h].view(FFN, BT), q["dy_up_t"].view(-1)[n_h:].view(FFN, BT)]

        def pair(i):
            K.abs_max(am3[i], srcs[i])
            K.quantize_with_abs_max(q_dsts[i], stats["h"][1:2], srcs[i], am3[i])

        cold = {
            "what": "20 timed launches after 5 warm-ups, events around each launch, rotating through three 8192 x 18944 "
                    "source tensors (930 MB) and three destinations, so that no launch finds its data in a cache",
            "abs_max (2 B/el)": cold_run(lambda i: K.abs_max(am3[i], srcs[i]), 2 * n_h),
            "quantize (3 B/el)": cold_run(lambda i: K.quantize_with_abs_max(q_dsts[i], stats["h"][1:2], srcs[i], am3[i]), 3 * n_h),
            "abs_max + quantize of one tensor (5 B/el)": cold_run(pair, 5 * n_h),
            "quantize_and_transpose (3 B/el)": cold_run(
                lambda i: K.quantize_and_transpose_with_abs_max(qt_dsts[i], None, srcs[i], am3[i]), 3 * n_h),
            "transpose (2 B/el)": cold_run(lambda i: K.transpose(qt_dsts[i], q_srcs[(i + 1) % 3]), 2 * n_h),
            # what a plain streaming copy sustains under the same protocol: the practical ceiling of a
            # read + write stream on this chip, for reading the fractions above
            "plain copy kernel, same protocol (2 B/el)": cold_run(lambda i: capi.check(capi.testaid().llmq_debug_copy_u8(
                qt_dsts[i].data_ptr(), q_srcs[(i + 1) % 3].data_ptr(), n_h, torch.cuda.current_stream().cuda_stream)), 2 * n_h),
            # the same access pattern with the reads only (310 MB: what abs-max streams) and with the writes only
            "plain read-only kernel, same protocol (2 B/el)": cold_run(lambda i: capi.check(capi.testaid().llmq_debug_stream_u8(
                am3[i].data_ptr(), srcs[i].data_ptr(), 2 * n_h, 0, torch.cuda.current_stream().cuda_stream)), 2 * n_h),
            "plain write-only kernel, same protocol (1 B/el)": cold_run(lambda i: capi.check(capi.testaid().llmq_debug_stream_u8(
                qt_dsts[i].data_ptr(), None, n_h, 1, torch.cuda.current_stream().cuda_stream)), n_h),
        }
        # Independent of this repository's kernels: what the vendor's own routines sustain under the same protocol
        # (same tensors, same rotation, same event pairs) -- a device-to-device copy (torch's copy_, i.e. the HIP
        # runtime's copy path) and two full reductions over the bf16 tensor (torch's amax and its infinity norm, which
        # is an abs-max).  They bound what "a read stream" and "a 1:1 stream" reach on this chip from outside.
        v_am = [torch.zeros((), dtype=torch.bfloat16, device=dev) for _ in srcs]
        v_u8 = [x_.view(torch.uint8).view(-1) for x_ in q_srcs]
        v_t8 = [x_.view(torch.uint8).view(-1) for x_ in qt_dsts]
        v_bf = [x_.view(-1) for x_ in srcs]
        v_dst = [torch.empty(n_h, dtype=torch.bfloat16, device=dev) for _ in srcs]
        cold["vendor"] = {
            "what": "torch / HIP runtime routines under the same protocol: copy_ between two 155 MB byte tensors and between "
                    "two 310 MB bf16 tensors, torch.amax and torch.linalg.vector_norm(inf) over a 310 MB bf16 tensor",
            "copy_ 155 MB bytes (2 B/el)": cold_run(lambda i: v_t8[i].copy_(v_u8[(i + 1) % 3]), 2 * n_h),
            "copy_ 310 MB bf16 (4 B/el)": cold_run(lambda i: v_dst[i].copy_(v_bf[i]), 4 * n_h),
            "amax over bf16 (2 B/el)": cold_run(lambda i: torch.amax(v_bf[i], 0, out=v_am[i]), 2 * n_h),
            "vector_norm(inf) over bf16 = abs-max (2 B/el)": cold_run(
                lambda i: torch.linalg.vector_norm(v_bf[i], float("inf"), out=v_am[i]), 2 * n_h),
        }
        del v_dst
        K.abs_max(stats["h"][0:1], t["h"])   # restore what the step left in the buffers used above
        K.quantize_with_abs_max(q["h"], stats["h"][1:2], t["h"], stats["h"][0:1])
        qtr(q["h_t"], "h")
        K.quantize_with_abs_max(q["dy_up"], stats["dy_up"][1:2], t["dy_up"], stats["dy_up"][0:1])
        tr(q["dy_up_t"], q["dy_up"])
        return cold

    cold = cold_section() if (not args.no_graph or args.hbm_kernels_only) else None
    if args.hbm_kernels_only:
        print(json.dumps({"hbm_kernels_cold_large_tensor": cold, "peak_GBps": HBM_PEAK_GBS}))
        return
    if args.calibrate_copy:
        src = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        capi.check(capi.testaid().llmq_debug_copy_u8(dst.data_ptr(), src.data_ptr(), src.numel(),
                                               torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
    # Secondary: the matmul alone on the layer shapes of BASELINE.json's other configurations (Qwen2.5-0.5B block,
    # 8192 tokens; Qwen2.5-1.5B MLP, 16384 tokens), forward / dgrad / wgrad, bf16 output, best of 3 x 5 launches.
    secondary = None
    if not args.no_graph:
        secondary = {"what": "matmul only, e4m3 operands of the given shape (matmul M, N, K), bf16 output, best of 3 x 5 "
                             "launches; TFLOP/s and fraction of the dense FP8 peak"}
        layers = {"0.5B qkv": (8192, 896, 1152), "0.5B o_proj": (8192, 896, 896), "0.5B gate_up": (8192, 896, 9728),
                  "0.5B down": (8192, 4864, 896), "1.5B gate_up": (16384, 1536, 17920), "1.5B down": (16384, 8960, 1536)}
        one1 = torch.ones(1, device=dev)
        for lname, (bt, cin, oc) in layers.items():
            for kind, (M_, N_, K_) in (("fwd", (oc, bt, cin)), ("dgrad", (cin, bt, oc)), ("wgrad", (cin, oc, bt))):
                a_op = q["dy_up"].view(-1)[:M_ * K_].view(M_, K_)       # any resident codes of the right size
                b_op = q["dy_up_t"].view(-1)[:N_ * K_].view(N_, K_)
                c_op = out["y_up"].view(-1)[:N_ * M_].view(N_, M_)
                best = 1e30
                for _ in range(3):
                    K.matmul(c_op, a_op, b_op, None, one1, one1, M_, N_, K_, workspace=ws)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(5):
                        K.matmul(c_op, a_op, b_op, None, one1, one1, M_, N_, K_, workspace=ws)
                    e1.record()
                    torch.cuda.synchronize()
                    best = min(best, e0.elapsed_time(e1) / 5 * 1e3)
                tf = 2.0 * M_ * N_ * K_ / best / 1e6
                secondary["%s %s (%d, %d, %d)" % (lname, kind, M_, N_, K_)] = {
                    "us": best, "TFLOPs": tf, "frac_fp8_peak": tf / FP8_PEAK_TFLOPS}
    secondary_steps = None
    if not args.no_graph:
        secondary_steps = secondary_path_steps(K, torch, dev, ws)
    step_ms = (t1 - t0) * 1e3 / args.steps

    # What the matrix cores sustain with no memory traffic at all: a register-only MFMA loop on random
    # fp8 operands (the chip lowers its clock under that load), about 0.3 s of it.
    scratch = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    ceiling = {}
    for label, rnd in (("constant_operands", 0), ("random_operands", 1), ("random_operands_16x16x128", 2)):
        capi.check(capi.testaid().llmq_debug_mfma_ceiling(scratch.data_ptr(), 256, 20000, rnd, st))
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        reps, iters = 6, 50000
        for _ in range(reps):
            capi.check(capi.testaid().llmq_debug_mfma_ceiling(scratch.data_ptr(), 256, iters, rnd, st))
        ev1.record()
        torch.cuda.synchronize()
        ceiling[label] = 256.0 * 8 * iters * 8 * 131072.0 * reps / (ev0.elapsed_time(ev1) * 1e-3) / 1e12

    def summarize(name):
        evs = timers.get(name, [])
        ms = [e[0].elapsed_time(e[1]) for e in evs]
        work = sum(e[2] for e in evs)
        return {"launches": len(evs), "mean_ms": sum(ms) / max(len(ms), 1), "total_ms": sum(ms), "work": work}

    def median(v):
        v = sorted(v)
        return 0.5 * (v[len(v) // 2] + v[(len(v) - 1) // 2])

    # per GEMM shape of the step: median and best launch over the timed steps
    shape_ms = {}
    for ev in timers.get("gemm", []):
        shape_ms.setdefault(ev[3], []).append((ev[0].elapsed_time(ev[1]), ev[2]))
    per_shape = {n: {"median_us": median([m for m, _ in v]) * 1e3, "min_us": min(m for m, _ in v) * 1e3,
                     "TFLOPs_at_median": v[0][1] / (median([m for m, _ in v]) * 1e-3) / 1e12,
                     "frac_at_median": v[0][1] / (median([m for m, _ in v]) * 1e-3) / 1e12 / FP8_PEAK_TFLOPS}
                 for n, v in shape_ms.items()}
    gemm_flop_sum = sum(v[0][1] for v in shape_ms.values())
    tflops_median = gemm_flop_sum / (sum(p["median_us"] for p in per_shape.values()) * 1e-6) / 1e12
    tflops_best = gemm_flop_sum / (sum(p["min_us"] for p in per_shape.values()) * 1e-6) / 1e12

    ks = {n: summarize(n) for n in ("gemm", "abs_max", "quantize", "quantize_transpose", "transpose")}
    gemm_tflops_kernel = ks["gemm"]["work"] / (ks["gemm"]["total_ms"] * 1e-3) / 1e12
    qnames = ("abs_max", "quantize", "quantize_transpose", "transpose")
    per_kernel = {n: {"GBps": ks[n]["work"] / (ks[n]["total_ms"] * 1e-3) / 1e9,
                      "frac_hbm": ks[n]["work"] / (ks[n]["total_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                      "mean_us": ks[n]["mean_ms"] * 1e3} for n in qnames}
    aq_bytes = ks["abs_max"]["work"] + ks["quantize"]["work"]
    aq_ms = ks["abs_max"]["total_ms"] + ks["quantize"]["total_ms"]
    aq_gbs = aq_bytes / (aq_ms * 1e-3) / 1e9

    result = {
        "metric": "e4m3 GEMM TFLOP/s + % FP8 peak; quantize GB/s + % HBM (Qwen-7B MLP shape)",
        "value": gemm_flop / (step_ms * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "untimed_steps_before_warmup": max(0, 20 - args.warmup),
        "ms_per_step": step_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "e4m3 x e4m3 -> fp32 accumulate -> bf16", "data": "synthetic",
        "config": {"workload": "Qwen2.5-7B MLP (gate+up 3584->37888, down 18944->3584), 8192 tokens, fwd+dgrad+wgrad "
                               "with per-tensor abs-max/quantize/transpose (BASELINE.json configs[3])",
                   "tokens": BT, "gemm_flop_per_step": gemm_flop},
        "roofline": {"bound": "mfma", "kernel": "gemm_tn_e4m3_w4_kernel", "achieved": gemm_tflops_kernel,
                     "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": gemm_tflops_kernel / FP8_PEAK_TFLOPS,
                     "traffic": measured_traffic(), "sensors_under_step_load": sensor_report,
                     "mfma_only_ceiling_TFLOPs": ceiling,
                     "frac_of_mfma_only_ceiling": gemm_tflops_kernel / max(ceiling["random_operands"], ceiling["random_operands_16x16x128"]),
                     "mean_launch_ms": ks["gemm"]["mean_ms"], "launches": ks["gemm"]["launches"],
                     "achieved_at_median_launch": tflops_median, "achieved_at_best_launch": tflops_best,
                     "per_shape": per_shape},
        "quantize": {"bound": "hbm", "kernels": "abs_max + quantize_with_abs_max (5 bytes/element)",
                     "achieved": aq_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": aq_gbs / HBM_PEAK_GBS,
                     "per_kernel": per_kernel, "cold_large_tensor": cold},
        "hip_graph_replay": None if graph_ms is None else {"ms_per_step": graph_ms,
                                                           "value": gemm_flop / (graph_ms * 1e-3) / 1e12},
        "fused_quantize_transpose_step": None if fused_ms is None else {
            "ms_per_step": fused_ms, "value": gemm_flop / (fused_ms * 1e-3) / 1e12,
            "note": "extension: single-read quantize + transposed copy for weights and output gradients"},
        "direct_gradient_layout_step": None if direct_ms is None else {
            "ms_per_step": direct_ms, "value": gemm_flop / (direct_ms * 1e-3) / 1e12,
            "gradients_identical_to_materialised_route": direct_identical,
            "note": "extension: the backward matmuls read their operands in their stored layouts (modes NN for both dgrads, "
                    "NT for the down weight gradient, TT for the gate+up weight gradient): no transposed copies of the "
                    "weights, of h or of the output gradients"},
        "vendor_gemm": vendor,
        "secondary_gemm_shapes": secondary,
        "secondary_steps": secondary_steps,
        "producers": swiglu,
        "library": capi.version(),
    }

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(t, np, torch, args.cpu_seconds)
        # the six GEMMs of the step against the exact product of the same e4m3 operands (oracle as the checker,
        # part of this CPU leg, outside every timed region)
        result["gemm_error"] = gemm_error_report(error_samples, np)
    print(json.dumps(result))


def secondary_path_steps(K, torch, dev, ws, iters=20):
    """The whole path (not the matmul alone) on the layers of BASELINE.json's small configurations, where launches and
    the extra passes weigh most: the Qwen2.5-0.5B block (qkv, o_proj, gate+up, down; 8192 tokens; bf16 dX, fp32 dW as
    configuration 3 asks) and the Qwen2.5-1.5B MLP (gate+up, down; 16384 tokens).  Per linear and step, the reference's
    sequence (src/models/llama_model.cpp:25-47, 309-339 and the weight quantization of llama_weights.cpp:207-223):
    weight abs-max + quantize; forward: abs-max + quantize of x, matmul; backward: abs-max + quantize of dY, transpose
    of W, dgrad matmul, quantize+transpose of x, transpose of dY, wgrad matmul.  Timed eagerly and replayed from a HIP
    graph, next to the matmuls alone (the three matmul launches per linear and nothing else) and to the sequence with the single-read quantize + transposed copy for W and dY."""
    f8, bf = torch.float8_e4m3fn, torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(9)
    models = {
        "qwen2.5-0.5B block, 8192 tokens": (8192, [("qkv", 896, 1152), ("o_proj", 896, 896), ("gate_up", 896, 9728),
                                                    ("down", 4864, 896)], torch.float32),
        "qwen2.5-1.5B mlp, 16384 tokens": (16384, [("gate_up", 1536, 17920), ("down", 8960, 1536)], bf),
    }
    report = {"what": "full path steps (every abs-max / quantize / transpose launch and the three matmuls per linear, "
                      "per-step weight quantization included), %d steps each after 3 warm-ups: eager, replayed from a HIP "
                      "graph, the matmuls alone, and the sequence with the single-read quantize + transposed copy for "
                      "weights and output gradients; launches = stream operations per step" % iters}

    def ms_of(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        f0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - f0) * 1e3 / iters

    for mname, (bt, linears, dw_dtype) in models.items():
        L = []
        for lname, cin, oc in linears:
            d = {"cin": cin, "oc": oc}
            d["x"] = torch.randn((bt, cin), device=dev, generator=gen).to(bf)
            d["w"] = (torch.randn((oc, cin), device=dev, generator=gen) * 0.02).to(bf)
            d["dy"] = (torch.randn((bt, oc), device=dev, generator=gen) * 1e-3).to(bf)
            for k_, shp in (("xq", (bt, cin)), ("xq_t", (cin, bt)), ("wq", (oc, cin)), ("wq_t", (cin, oc)), ("dyq", (bt, oc)),
                            ("dyq_t", (oc, bt))):
                d[k_] = torch.empty(shp, dtype=f8, device=dev)
            d["st"] = {k_: torch.zeros(2, device=dev) for k_ in ("x", "w", "dy")}
            d["y"] = torch.empty((bt, oc), dtype=bf, device=dev)
            d["dx"] = torch.empty((bt, cin), dtype=bf, device=dev)
            d["dw"] = torch.empty((oc, cin), dtype=dw_dtype, device=dev)
            L.append(d)
        launches = [0]

        def aq(d, name, src, dst):
            K.abs_max(d["st"][name][0:1], src)
            K.quantize_with_abs_max(dst, d["st"][name][1:2], src, d["st"][name][0:1])
            launches[0] += 2

        def mm(c, a, b, sa, sb, M, N, Kd):
            K.matmul(c, a, b, None, sa, sb, M, N, Kd, workspace=ws)
            launches[0] += 1

        def matmuls(d, bt=bt):
            s_ = d["st"]
            mm(d["y"], d["wq"], d["xq"], s_["w"][1:2], s_["x"][1:2], d["oc"], bt, d["cin"])
            mm(d["dx"], d["wq_t"], d["dyq"], s_["w"][1:2], s_["dy"][1:2], d["cin"], bt, d["oc"])
            mm(d["dw"], d["xq_t"], d["dyq_t"], s_["x"][1:2], s_["dy"][1:2], d["cin"], d["oc"], bt)

        def step(fused):
            for d in L:
                s_ = d["st"]
                if fused:
                    K.abs_max(s_["w"][0:1], d["w"])
                    K.quantize_with_abs_max_and_transpose(d["wq"], d["wq_t"], s_["w"][1:2], d["w"], s_["w"][0:1])
                    launches[0] += 2
                else:
                    aq(d, "w", d["w"], d["wq"])
                aq(d, "x", d["x"], d["xq"])
                mm(d["y"], d["wq"], d["xq"], s_["w"][1:2], s_["x"][1:2], d["oc"], bt, d["cin"])
            for d in reversed(L):
                s_ = d["st"]
                if fused:
                    K.abs_max(s_["dy"][0:1], d["dy"])
                    K.quantize_with_abs_max_and_transpose(d["dyq"], d["dyq_t"], s_["dy"][1:2], d["dy"], s_["dy"][0:1])
                    launches[0] += 2
                else:
                    aq(d, "dy", d["dy"], d["dyq"])
                    K.transpose(d["wq_t"], d["wq"])
                    launches[0] += 1
                mm(d["dx"], d["wq_t"], d["dyq"], s_["w"][1:2], s_["dy"][1:2], d["cin"], bt, d["oc"])
                K.quantize_and_transpose_with_abs_max(d["xq_t"], None, d["x"], s_["x"][0:1])
                launches[0] += 1
                if not fused:
                    K.transpose(d["dyq_t"], d["dyq"])
                    launches[0] += 1
                mm(d["dw"], d["xq_t"], d["dyq_t"], s_["x"][1:2], s_["dy"][1:2], d["cin"], d["oc"], bt)

        def count(fn):
            launches[0] = 0
            fn()
            return launches[0]

        flop = sum(6.0 * bt * d["cin"] * d["oc"] for d in L)
        n_ref, n_fused = count(lambda: step(False)), count(lambda: step(True))
        eager = ms_of(lambda: step(False))
        fused = ms_of(lambda: step(True))
        only = ms_of(lambda: [matmuls(d) for d in L])
        graphs = {}
        for label, fz in (("reference sequence", False), ("single-read quantize + transposed copy", True)):
            g_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g_):
                step(fz)
            graphs[label] = ms_of(g_.replay)
            del g_
        report[mname] = {
            "gemm_flop_per_step": flop,
            "reference sequence": {"launches": n_ref, "eager_ms": eager, "hip_graph_ms": graphs["reference sequence"],
                                   "TFLOPs_eager": flop / eager / 1e9, "TFLOPs_hip_graph": flop / graphs["reference sequence"] / 1e9},
            "single-read quantize + transposed copy": {
                "launches": n_fused, "eager_ms": fused, "hip_graph_ms": graphs["single-read quantize + transposed copy"],
                "TFLOPs_hip_graph": flop / graphs["single-read quantize + transposed copy"] / 1e9},
            "matmuls_alone_ms": only, "TFLOPs_matmuls_alone": flop / only / 1e9,
            "non_matmul_share_of_eager_step": 1.0 - only / eager,
        }
        del L
    return report


class SensorSampler:
    """Reads the driver's package power and shader clock (hwmon power1_input / power1_cap, pp_dpm_sclk under
    /sys/class/drm/card*/device) every 10 ms from a thread until stop(); figures from the second half of the samples.
    Absent files (another driver, no permission) give {"available": False}."""

    def __init__(self, enabled=True):
        import glob
        import threading
        self.available = False
        if not enabled:
            return
        pw = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
        cap = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap")
        ck = glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
        self.files = (pw[0], ck[0]) if len(pw) == 1 and len(ck) == 1 else None
        self.cap = None
        self.samples, self.halt, self.thread = [], False, None
        if self.files is None:
            return
        try:
            self.cap = int(open(cap[0]).read()) / 1e6 if cap else None
            self.idle = self.read()
        except (OSError, ValueError):
            return
        self.available = True
        self.thread = threading.Thread(target=self.run, daemon=True)
        self.thread.start()

    def read(self):
        import re
        watts = int(open(self.files[0]).read()) / 1e6
        m = re.search(r"(\d+)Mhz \*", open(self.files[1]).read())
        return watts, (int(m.group(1)) if m else None)

    def run(self):
        while not self.halt:
            try:
                self.samples.append(self.read())
            except (OSError, ValueError):
                pass
            time.sleep(0.01)

    def stop(self):
        if not self.available:
            return {"available": False}
        self.halt = True
        self.thread.join()
        late = self.samples[len(self.samples) // 2:]
        watts = sorted(w for w, _ in late)
        mhz = sorted(c for _, c in late if c)
        if not watts or not mhz:
            return {"available": False}
        return {"available": True, "what": "hwmon power1_input and pp_dpm_sclk sampled every 10 ms while the steps of the "
                "second (untimed) pass run; second half of the samples",
                "samples": len(late), "power_W_median": watts[len(watts) // 2], "power_W_max": watts[-1],
                "power_cap_W": self.cap, "sclk_MHz_median": mhz[len(mhz) // 2], "sclk_MHz_min": mhz[0],
                "first_sample_right_after_the_timed_steps": {"power_W": self.idle[0], "sclk_MHz": self.idle[1]}}


def measured_traffic():
    """HBM-side bytes per GEMM launch (L2 fetch + write-back) from the hardware-counter summary kept
    under profiles/ for this same workload; None when that file is absent."""
    path = os.path.join(ROOT, "profiles", "gemm_tn_e4m3_w4_kernel__bench_qwen7b_mlp__traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch"):
                return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def collect_gemm_samples(gemms, stats, np, torch, samples=8192):
    """Host copies of what the error report needs: per GEMM the operand codes, the fp32 factor sa*sb and
    `samples` seeded output coordinates with the device results there."""
    taken = []
    for i, (name, c, a_op, b_op, sa_name, sb_name) in enumerate(gemms):
        N, M = c.shape
        rng = np.random.default_rng(100 + i)
        idx_n = rng.integers(0, N, samples).astype(np.int32)
        idx_m = rng.integers(0, M, samples).astype(np.int32)
        got = c[torch.from_numpy(idx_n).long().cuda(), torch.from_numpy(idx_m).long().cuda()].float().cpu().numpy()
        taken.append({"name": name, "M": M, "N": N, "a": a_op.view(torch.uint8).cpu().numpy(),
                      "b": b_op.view(torch.uint8).cpu().numpy(), "idx_n": idx_n, "idx_m": idx_m, "got": got.astype(np.float64),
                      "scale": float(np.float32(stats[sa_name][1].item()) * np.float32(stats[sb_name][1].item()))})
    return taken


def gemm_error_report(taken, np):
    """Per GEMM of the step: max-abs and relative-Frobenius error of the bf16 device result against the exact
    (fp64) product of the same e4m3 operands times the fp32 factor sa*sb, on seeded output coordinates (the
    reference's acceptance loop prints the same two figures, src/testing/test-gemm.cpp:114-148), and the worst
    ratio of an element's error to the stated bound 2^-8 |ref| + 2^-11 sa sb sum|a b|."""
    from oracle import pyoracle as O
    report = {"what": "bf16 result vs exact fp64 product of the same e4m3 operands x (sa*sb), %d sampled outputs per "
                      "GEMM; bound = 2^-8 |ref| + 2^-11 sa sb sum_k|a_k b_k|, relative Frobenius limit 2.5e-3"
                      % taken[0]["idx_n"].size}
    for s in taken:
        ex, sabs = O.gemm_exact_sampled(s["a"], s["b"], s["idx_n"], s["idx_m"])
        ref = ex * s["scale"]
        err = np.abs(s["got"] - ref)
        bound = 2.0 ** -8 * np.abs(ref) + 2.0 ** -11 * s["scale"] * sabs + 1e-300
        fro = float(np.sqrt((err ** 2).sum() / (ref ** 2).sum()))
        report[s["name"]] = {"M": s["M"], "N": s["N"], "K": int(s["a"].shape[1]), "max_abs": float(err.max()),
                             "rel_frobenius": fro, "max_abs_ref": float(np.abs(ref).max()),
                             "worst_err_over_bound": float((err / bound).max()),
                             "within_tolerance": bool((err <= bound).all() and fro <= 2.5e-3)}
    return report


def cpu_baseline(t, np, torch, budget_s):
    """The multithreaded CPU port (oracle/llmq_cpu_mt.c) on a bounded sample of the same workload:
    abs-max + quantize of X [8192x3584] and of a row-slice of W_up, then the gate+up forward GEMM for
    that slice of output features against all 8192 tokens."""
    import ctypes
    from oracle import pyoracle as O
    L = O.lib()
    cores = min(L.mt_num_threads(), 16)      # the GPU box grants 16 host cores to a one-GPU job
    L.mt_set_num_threads(cores)
    to_bits = lambda x: x.cpu().view(torch.int16).numpy().view(np.uint16)
    x = to_bits(t["x"])
    # calibrate the GEMM slice: 64 weight rows first, then scale to the budget
    w_all = t["w_up"]
    t0 = time.perf_counter()
    ax = float(L.mt_abs_max_bf16(x.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), x.size))
    xq, _ = O.quantize_e4m3(x, ax, mt=True)
    t_q = time.perf_counter() - t0
    q_gbs = 5 * x.size / t_q / 1e9

    def gemm_rows(m_rows):
        w = to_bits(w_all[:m_rows].contiguous())
        aw = O.abs_max_bf16(w)
        wq, _ = O.quantize_e4m3(w, aw, mt=True)
        s = time.perf_counter()
        O.gemm_tn(wq, xq, sa=1.0, sb=1.0, mt=True)
        return time.perf_counter() - s

    t64 = gemm_rows(64)
    rows = int(max(64, min(UP, (budget_s / max(t64, 1e-3)) * 64)) // 64 * 64)
    tg = gemm_rows(rows) if rows > 64 else t64
    flop = 2.0 * rows * BT * C
    return {"value": flop / tg / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "gate+up forward GEMM for %d of %d output features x 8192 tokens x K=3584 (%.1f GFLOP, %.1f s); "
                      "abs-max+quantize of X[8192x3584]: %.2f GB/s" % (rows, UP, flop / 1e9, tg, q_gbs),
            "quantize_GBps": q_gbs}


if __name__ == "__main__":
    main()
