#!/usr/bin/env python3
"""Benchmark of the SimNets Similarity / MEX hot path on one MI355X.

One "step" = one Similarity L2 forward over benchmark configuration 3 (input 256x64x32x32, 128
templates 64x3x3, stride 1, padding 1 -> 256x128x32x32; 19.33 G generalized MACs), inputs already
resident in HBM, called through the C ABI exactly as an op layer would (the self-packing entry
point: parameter packing included in every step).  The other configurations (1, 2, 3-L1, 4, and the
backward operators of configuration 5) and the alternative evaluation paths are timed in the same
run and reported under "others", each beside the CPU oracle timed on a bounded sample of the same
workload.  Prints ONE JSON line.

The CPU baseline legs time the CPU oracle (a restatement of the reference's CPU kernels); they are
the only places this file touches oracle/, and they run after the GPU timings.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_FP32_TFLOPS = 157.3   # MI355X published FP32 vector / FP32 matrix peak (256 CU x 128 FMA lanes x 2.4 GHz x 2)
PEAK_HBM_GBS = 8000.0
EXP_RATE_STATED = 9.83e12  # exponentials per second the work table of the baseline document prices MEX against
EXP_RATE_MEASURED = 19.66e12  # v_exp_f32 at a quarter of the 128 lanes/clk/CU VALU rate (17.6e12 measured on the box)

# HBM bytes per launch of the dominant kernel of the headline workload, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs
# scaled by a copy kernel of known size; not measured inside this run: "traffic_source" names the committed summary.
MEASURED_TRAFFIC = {
    "sqrtw": (231.8e6, "profiles/sim_direct_l2_config3.md"),
    "direct": (None, "no counter run of the current three-instruction kernel"),
    "mfma": (223.3e6, "profiles/sim_direct_l2_config3_other_forms.md"),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle", type=float, default=1.5,
                    help="seconds of untimed load before the warm-up steps (lets the clocks of an idle GPU settle)")
    ap.add_argument("--settle-others", type=float, default=0.25,
                    help="seconds of untimed load before every other timed workload")
    ap.add_argument("--algo", default=None, choices=[None, "direct", "sqrtw", "mfma"],
                    help="evaluation path of the headline Similarity kernel (default: the library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-others", action="store_true", help="time only the headline workload")
    ap.add_argument("--pmc-calib", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a plain copy kernel of known size, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--cpu-images", type=int, default=12,
                    help="images of configuration 3 the single-threaded CPU baseline times per function (12 ~ 3 s)")
    ap.add_argument("--shapes", action="store_true",
                    help="instead of the benchmark line: time Similarity forward, input gradient and parameter "
                         "gradients on network-like shapes away from the benchmark configurations (one JSON object)")
    ap.add_argument("--train", action="store_true",
                    help="instead of the benchmark line: time only the training step of the config-4 stack (the run "
                         "to put under a kernel trace; one JSON object)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path is data parallel over the batch; "
              "each GPU would take a share of the images); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from __graft_entry__ import load_package, build
    from util import config1, config2, config3, config4_stack, rel_err

    if not os.path.exists(os.path.join(ROOT, "simnets-tf_amd", "libsimnets_hip.so")):
        build()
    pkg = load_package()
    assert torch.cuda.is_available(), "bench.py needs a GPU: there is no CPU fallback"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    host_cpus = os.cpu_count() or 1
    threads = min(host_cpus, 16)

    def to_dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def timed(fn, steps, warmup):
        """(wall ms per step, HIP-event ms per step) for `steps` calls after `warmup` calls.
        The events are recorded on the stream the kernels are launched on (torch's current stream,
        whose handle the op layer passes through the C ABI).  Like the headline, every workload first runs
        untimed for a moment (--settle-others): the host-side set-up between two workloads leaves the chip idle
        long enough for its clocks to drop."""
        until = time.perf_counter() + args.settle_others
        while time.perf_counter() < until:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        start.record()
        for _ in range(steps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return wall, start.elapsed_time(stop) / steps

    def graph_of(fn, reps):
        """A HIP graph of `reps` back-to-back calls: per-call time without the host's share of a launch."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                fn()
        return g

    def config4_training_step(X4, T4, W4, kw4, layer_offsets, offl, nl, kwl):
        """A training step of the config-4 stack through the differentiable layer functions: forward with the
        unfused MEX calls (their gradients take the unpooled outputs), then every operator's gradient calls."""
        L = pkg.layers
        params = [T4.clone().requires_grad_(), W4.clone().requires_grad_()] + \
                 [off.clone().requires_grad_() for off, _, _ in layer_offsets] + [offl.clone().requires_grad_()]

        def train_step():
            for q in params:
                q.grad = None
            cur = L.similarity(X4, params[0], params[1], **kw4)
            for i, (_, n, kw) in enumerate(layer_offsets):
                cur = L.mex_sum_pool(cur, params[2 + i], n, (2, 2), normalize_offsets=True, **kw)
            out = L.mex(cur, params[-1], nl, normalize_offsets=True, **kwl)
            out.sum().backward()
        return train_step

    if args.train:
        x4, t4, w4, kw4, layers_np, (offl_np, nl, kwl) = config4_stack(512)
        step = config4_training_step(to_dev(x4), to_dev(t4), to_dev(w4), kw4,
                                     [(to_dev(o), n, kw) for o, n, kw in layers_np], to_dev(offl_np), nl, kwl)
        _, ms = timed(step, args.steps, args.warmup)
        print(json.dumps({"config4_train_step_ms": round(ms, 4), "batch": 512, "steps": args.steps,
                          "warmup": args.warmup, "dtype": "f32"}))
        return

    if args.shapes:
        # (name, input shape, templates, block, stride, padding): layers of a residual-network-like stack at batch 32
        shapes = [
            ("3x224x224->64 7x7 s2 p3", (32, 3, 224, 224), 64, 7, 2, 3),
            ("64x56x56->64 3x3 s1 p1", (32, 64, 56, 56), 64, 3, 1, 1),
            ("128x28x28->128 3x3 s1 p1", (32, 128, 28, 28), 128, 3, 1, 1),
            ("256x14x14->256 3x3 s1 p1", (32, 256, 14, 14), 256, 3, 1, 1),
            ("512x7x7->512 3x3 s1 p1", (32, 512, 7, 7), 512, 3, 1, 1),
            ("64x56x56->128 3x3 s2 p1", (32, 64, 56, 56), 128, 3, 2, 1),
            ("256x56x56->64 1x1", (32, 256, 56, 56), 64, 1, 1, 0),
            ("64x32x32->128 3x3 s1 p1 batch 256", (256, 64, 32, 32), 128, 3, 1, 1),
        ]
        table = {}
        torch.manual_seed(1234)
        for name, shp, n_templates, blk, stride, pad in shapes:
            xs = torch.randn(*shp, device=dev)
            ts = torch.randn(n_templates, shp[1], blk, blk, device=dev)
            ws = torch.rand_like(ts) + 0.1
            kws = dict(blocks=[blk, blk], strides=[stride, stride], padding=[pad, pad])
            outs = pkg.similarity(xs, ts, ws, **kws)
            gs = torch.randn_like(outs)
            gmac = outs.numel() * shp[1] * blk * blk
            row = {}
            for key, fn in (("forward", lambda: pkg.similarity(xs, ts, ws, out=outs, **kws)),
                            ("input_grad", lambda: pkg.similarity_input_grad(xs, ts, ws, gs, **kws)),
                            ("params_grad", lambda: pkg.similarity_parameters_grad(xs, ts, ws, gs, **kws))):
                reps = [timed(fn, args.steps, args.warmup)[1] for _ in range(3)]   # the fastest of three batches
                ms = min(reps)
                row[key] = {"ms": round(ms, 4), "T_gMAC_per_s": round(gmac / ms / 1e9, 2),
                            "slowest_batch_ms": round(max(reps), 4)}
            table[name] = row
        print(json.dumps({"similarity_shapes": table, "steps": args.steps, "warmup": args.warmup, "dtype": "f32"}))
        return

    if args.pmc_calib:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ headline: configuration 3, L2
    x3, t3, w3, kw3 = config3()
    X3, T3, W3 = to_dev(x3), to_dev(t3), to_dev(w3)
    out3 = torch.empty((256, 128, 32, 32), device=dev)
    gmac3 = 256 * 128 * 32 * 32 * 576
    bytes3 = 67108864 + 589824 + 134217728

    def sim3(func="L2", algo=None):
        return lambda: pkg.similarity(X3, T3, W3, similarity_function=func, algo=algo, out=out3, **kw3)

    # A GPU that has been idle (process start-up, host-side data generation) needs on the order of a second of load
    # before its clocks settle: the same 50 steps read 1.09 ms right after start-up and 0.86 ms on a busy chip.
    # Untimed load of the headline kernel first, then the W warm-up steps and the K timed ones.
    # The same K steps are first timed "cold": after the W warm-up steps only, on a chip that has idled through
    # process start-up and input generation (reported beside the headline, never as the headline).
    so = args.settle_others
    args.settle_others = 0.0
    cold_wall_ms, cold_ev_ms = timed(sim3("L2", args.algo), args.steps, args.warmup)
    args.settle_others = so
    settle_until = time.perf_counter() + args.settle
    while time.perf_counter() < settle_until:
        for _ in range(50):
            sim3("L2", args.algo)()
        torch.cuda.synchronize()
    wall_ms, ev_ms = timed(sim3("L2", args.algo), args.steps, args.warmup)
    gmacs = gmac3 / (ev_ms * 1e-3)
    flop_per_gmac = 4
    achieved_tflops = gmacs * flop_per_gmac / 1e12
    path = args.algo or "sqrtw"
    traffic, traffic_source = MEASURED_TRAFFIC[path]
    result = {
        "metric": "Similarity L2 fwd generalized-GMAC/s (config 3), 1 MI355X",
        "value": round(gmac3 / (wall_ms * 1e-3) / 1e9, 1),
        "unit": "GMAC/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config3: Similarity L2 fwd 256x64x32x32, 128 templates 64x3x3, s1 p1 "
                               "-> 256x128x32x32 (M=262144 N=128 K=576)",
                   "algo": args.algo or "auto (sqrt-weight form; waves with a partial sum near zero are recomputed "
                                        "term by term)",
                   "entry_point": "simnets_hip_similarity_fwd (packs the parameters in every step)",
                   "gmac_per_step": gmac3},
        # compute bound: the FP32 vector ALU ("valu") unless the matrix-core path is asked for; the two peaks are
        # the same 157.3 TFLOP/s
        "roofline": {"bound": "mfma" if args.algo == "mfma" else "valu",
                     "achieved": round(achieved_tflops, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved_tflops / PEAK_FP32_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel_ms": round(ev_ms, 4), "flop_per_gmac": flop_per_gmac,
                     "cold_start": {"kernel_ms": round(cold_ev_ms, 4), "ms_per_step": round(cold_wall_ms, 4),
                                    "frac": round(gmac3 * flop_per_gmac / (cold_ev_ms * 1e-3) / 1e12 / PEAK_FP32_TFLOPS, 4),
                                    "what": "the same %d steps timed right after the %d warm-up steps, before the "
                                            "%.1f s of untimed load that precede the headline's steps"
                                            % (args.steps, args.warmup, args.settle)},
                     "algorithmic_bytes": bytes3,
                     "hbm_frac": round(bytes3 / (ev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)},
    }

    # ------------------------------------------------------------------ the other configurations
    others = {}
    cpu_jobs = []   # (name, callable returning the cpu_baseline dict): run after all GPU timings, once `oracle` is imported
    oracle = None

    def entry(ms, gmac, nbytes, bound, flop=None, mex=False):
        """bound: which roofline prices this shape ("valu", "mfma", "hbm"); frac is taken against it.
        MEX rows (mex=True) are priced on HBM: the product form runs one exponential per patch element and one fused
        multiply-add per term on the matrix cores, so neither the exponential rate nor the vector ALU bounds them."""
        rate = gmac / (ms * 1e-3)
        e = {"kernel_ms": round(ms, 4), "gmac_per_s_G": round(rate / 1e9, 1), "bound": bound,
             "algorithmic_bytes": int(nbytes),
             "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        if flop and not mex:
            e["valu_frac"] = round(rate * flop / 1e12 / PEAK_FP32_TFLOPS, 4)
        if mex:
            e["reference_formulation_not_executed"] = {
                "what": "1 exp + 5 flop per term, as the reference evaluates MEX; this library's default kernels do "
                        "not execute that work, so these are side figures, not roofline fractions",
                "exp_frac": round(rate / EXP_RATE_STATED, 4),
                "exp_frac_measured_rate": round(rate / EXP_RATE_MEASURED, 4),
                "valu_frac": round(rate * (flop or 5) / 1e12 / PEAK_FP32_TFLOPS, 4)}
            e["matrix_pipe_frac"] = round(rate * 2 / 1e12 / PEAK_FP32_TFLOPS, 4)
        e["frac"] = {"valu": e.get("valu_frac"), "mfma": e.get("valu_frac"), "hbm": e["hbm_frac"]}[bound]
        return e

    def cpu_leg(sample, run_single, run_all, gmac_single, gmac_all, err):
        t0 = time.perf_counter()
        run_single()
        dt = time.perf_counter() - t0
        t0 = time.perf_counter()
        run_all()
        dta = time.perf_counter() - t0
        return {"value": round(gmac_single / dt / 1e9, 4), "unit": "GMAC/s", "cores": 1, "kind": "port",
                "sample": sample, "seconds": round(dt, 2),
                "all_cores": {"value": round(gmac_all / dta / 1e9, 4), "threads": threads,
                              "note": "batch loop spread over threads; not reference behaviour"},
                "host_cpus": host_cpus, "max_rel_err_gpu_vs_cpu": err}

    if not args.no_others:
        def mex_err(got, x, off, n, **kw):
            """MEX error under both metrics: relative to max(|cpu|, |m|) (m = the largest term, the shift every
            implementation subtracts: where m and log(sum) cancel the rounding noise scales with |m|), and under
            the plain max(|cpu|, 1e-6 max|cpu|) of the Similarity rows, plus the largest absolute deviation."""
            want = oracle.mex_fwd(x, off, n, threads=threads, **kw)
            shift = oracle.mex_fwd(x, off, n, threads=threads,
                                   **dict(kw, epsilon=math.copysign(math.inf, kw.get("epsilon", 1.0))))
            exact = oracle.mex_fwd(x.astype(np.float64), off.astype(np.float64), n, threads=threads, **kw)
            # (the largest term's magnitude, or the largest offset's where the terms of the maximum cancel: the rounding of
            # a normalised offset is of that size)
            floor = np.maximum(np.abs(shift), np.abs(off).max() if np.isfinite(off).all() else 0.0)
            return {"floor_max_term": rel_err(got, want, floor=floor), "plain_metric": rel_err(got, want),
                    "max_abs_dev": float(np.abs(got - want).max()), "max_abs_term": float(np.abs(shift).max()),
                    "plain_metric_gpu_vs_fp64_oracle": rel_err(got, exact),
                    "plain_metric_fp32_oracle_vs_fp64_oracle": rel_err(want, exact),
                    "what": "floor_max_term: |gpu - cpu| / max(|cpu|, |m|), m = the largest term; plain_metric: "
                            "|gpu - cpu| / max(|cpu|, 1e-6 max|cpu|), which is unbounded where the output crosses "
                            "zero (the fp32 CPU result is as far from the exact value under it, last figure)"}

        # ---- configuration 3, other functions and forms
        _, ms = timed(sim3("L1", None), args.steps, args.warmup)
        others["config3_L1_direct"] = entry(ms, gmac3, bytes3, "valu", flop=3)
        prep3 = pkg.similarity_prepare(x3.shape, T3, W3, similarity_function="L2", algo=args.algo, **kw3)
        _, ms = timed(lambda: prep3(X3, out=out3), args.steps, args.warmup)
        others["config3_L2_prepared"] = entry(ms, gmac3, bytes3, "mfma" if args.algo == "mfma" else "valu", flop=4)
        others["config3_L2_prepared"]["entry_point"] = "simnets_hip_similarity_fwd_prepared (parameters packed once)"
        del prep3
        for algo in ("direct", "sqrtw", "mfma"):
            if algo == path:
                continue
            try:
                _, ms = timed(sim3("L2", algo), args.steps, args.warmup)
                others["config3_L2_" + algo] = entry(ms, gmac3, bytes3, "mfma" if algo == "mfma" else "valu", flop=4)
            except pkg.SimnetsError as e:
                others["config3_L2_" + algo] = {"error": str(e)}
        # worst case of the sqrt-weight form's guard: every wave stops after the first channel chunk and is
        # recomputed term by term (inputs and templates 1000 +- 3: all outputs far below the thresholds)
        g = np.random.default_rng(77)
        XA = to_dev((g.normal(size=x3.shape) + 1000).astype(np.float32))
        TA = to_dev((g.normal(size=t3.shape) + 1000).astype(np.float32))
        _, ms_w = timed(lambda: pkg.similarity(XA, TA, W3, out=out3, **kw3), args.steps, args.warmup)
        got_w = out3.clone()
        _, ms_d = timed(lambda: pkg.similarity(XA, TA, W3, out=out3, algo="direct", **kw3), args.steps, args.warmup)
        others["config3_L2_guard_worst_case"] = {
            "kernel_ms": round(ms_w, 4), "direct_same_data_ms": round(ms_d, 4), "ratio": round(ms_w / ms_d, 3),
            "bit_identical_to_direct": bool(torch.equal(got_w, out3)),
            "data": "inputs and templates ~ N(1000, 1): every wave is flagged"}
        del XA, TA, got_w

        # the reference's other L2 modes at this scale (include/utils/similarity_utils.hpp:38-80): the normalisation
        # term (half the log-weight per element, and with NaN inputs ignored only for the elements present), 25 % of the
        # input missing, NaN beyond the border.  Priced at the functor's 6 flop per term (subtract, square, weight,
        # halve, add the log term, accumulate); the kernels spend 4 instructions on them.
        def sim3_mode(X, mode):
            return lambda: pkg.similarity(X, T3, W3, similarity_function="L2", out=out3, **dict(kw3, **mode))

        xn3 = x3.copy()
        xn3[np.random.default_rng(78).random(x3.shape) < 0.25] = np.nan
        XN3 = to_dev(xn3)
        modes3 = {
            "config3_L2_normalized": (x3, X3, dict(normalization_term=True)),
            "config3_L2_normalized_ignore_nan": (xn3, XN3, dict(normalization_term=True, ignore_nan_input=True,
                                                                out_of_bounds_value=float("nan"))),
        }
        for name, (_, Xm, mode) in modes3.items():
            _, ms = timed(sim3_mode(Xm, mode), args.steps, args.warmup)
            others[name] = entry(ms, gmac3, bytes3, "valu", flop=6)
            others[name]["flop_per_gmac"] = 6
            others[name]["attrs"] = {k: (str(v) if isinstance(v, float) else v) for k, v in mode.items()}
            if "ignore_nan_input" in mode:
                others[name]["data"] = "25 % of the input elements are NaN"

        def cpu3_mode(name):
            def job():
                xm, Xm, mode = modes3[name]
                n_img = 256 if threads >= 8 else 8 * threads
                want = oracle.similarity_fwd(xm[:n_img], t3, w3, similarity_function="L2", threads=threads,
                                             **dict(kw3, **mode))
                got = pkg.similarity(Xm[:n_img], T3, W3, similarity_function="L2", **dict(kw3, **mode)).cpu().numpy()
                return {"kind": "port", "sample": "%d of 256 images, %d threads: parity only, not timed" % (n_img, threads),
                        "max_rel_err_gpu_vs_cpu": rel_err(got, want),
                        "nan_positions_identical": bool(np.array_equal(np.isnan(got), np.isnan(want))),
                        "nan_outputs": int(np.isnan(want).sum())}
            return job
        for name in modes3:
            cpu_jobs.append((name, cpu3_mode(name)))

        def cpu3(func):
            def job():
                n_img = max(1, args.cpu_images)
                xm = x3[:min(256, threads * 4)]
                ref = [None]

                def single():
                    ref[0] = oracle.similarity_fwd(x3[:n_img], t3, w3, similarity_function=func, **kw3)
                got = pkg.similarity(X3[:n_img], T3, W3, similarity_function=func, algo=args.algo if func == "L2" else None,
                                     **kw3).cpu().numpy()
                leg = cpu_leg("%d of 256 images of config 3 (%s), single thread like the reference; -O2, no fast-math"
                              % (n_img, func), single,
                              lambda: oracle.similarity_fwd(xm, t3, w3, similarity_function=func, threads=threads, **kw3),
                              n_img * 128 * 1024 * 576, len(xm) * 128 * 1024 * 576, None)
                leg["max_rel_err_gpu_vs_cpu"] = rel_err(got, ref[0])
                return leg
            return job
        cpu_jobs.append(("config3_L1_direct", cpu3("L1")))

        # ---- configuration 1
        x1, t1, w1, kw1 = config1(batch=64, nan_frac=0.0)
        X1, T1, W1 = to_dev(x1), to_dev(t1), to_dev(w1)
        o1 = torch.empty((64, 32, 16, 16), device=dev)
        _, ms = timed(lambda: pkg.similarity(X1, T1, W1, out=o1, **kw1), args.steps, args.warmup)
        prep1 = pkg.similarity_prepare(x1.shape, T1, W1, **kw1)
        _, ms_p = timed(lambda: prep1(X1, out=o1), 4 * args.steps, args.warmup)
        _, ms_g = timed(graph_of(lambda: prep1(X1, out=o1), 20).replay, args.steps, args.warmup)
        _, ms_sg = timed(graph_of(lambda: pkg.similarity(X1, T1, W1, out=o1, **kw1), 20).replay, args.steps, args.warmup)
        others["config1_similarity"] = entry(ms_sg / 20, 2097152, 2298880, "hbm", flop=6)
        others["config1_similarity"].update({
            "eager_call_ms": round(ms, 4), "prepared_eager_call_ms": round(ms_p, 4),
            "prepared_kernel_ms": round(ms_g / 20, 4),
            "note": "latency bound: 256 single-wave workgroups.  kernel_ms (pack + main kernel of a self-packing "
                    "call) and prepared_kernel_ms (main kernel alone) are device times per call, from a HIP graph of "
                    "20 calls; the fractions are taken on kernel_ms.  The eager figures are calls through the Python "
                    "op layer, back to back: the host's share of a call (argument checks, two launches), not the "
                    "device, bounds them"})

        def cpu1():
            got = o1.cpu().numpy()
            return cpu_leg("all 64 images of config 1, single thread", lambda: oracle.similarity_fwd(x1, t1, w1, **kw1),
                           lambda: oracle.similarity_fwd(x1, t1, w1, threads=threads, **kw1), 2097152, 2097152,
                           rel_err(got, oracle.similarity_fwd(x1, t1, w1, **kw1)))
        cpu_jobs.append(("config1_similarity", cpu1))

        # ---- configuration 2
        x2, off2, n2, kw2 = config2()
        X2, O2 = to_dev(x2), to_dev(off2)
        o2 = torch.empty((64, 64, 16, 16), device=dev)
        _, ms = timed(lambda: pkg.mex(X2, O2, n2, normalize_offsets=True, out=o2, **kw2), args.steps, args.warmup)
        prep2 = pkg.mex_prepare(x2.shape, O2, n2, normalize_offsets=True, **kw2)
        _, ms_p = timed(lambda: prep2(X2, out=o2), 4 * args.steps, args.warmup)
        _, ms_g = timed(graph_of(lambda: prep2(X2, out=o2), 20).replay, args.steps, args.warmup)
        _, ms_sg = timed(graph_of(lambda: pkg.mex(X2, O2, n2, normalize_offsets=True, out=o2, **kw2), 20).replay,
                         args.steps, args.warmup)
        others["config2_mex"] = entry(ms_sg / 20, 33554432, 6324224, "hbm", flop=5, mex=True)
        others["config2_mex"].update({
            "eager_call_ms": round(ms, 4), "prepared_eager_call_ms": round(ms_p, 4),
            "prepared_kernel_ms": round(ms_g / 20, 4),
            "note": "latency bound at this size.  kernel_ms (offsets pack + main kernel of a self-packing call) and "
                    "prepared_kernel_ms (main kernel alone) are device times per call, from a HIP graph of 20 calls; "
                    "the fractions are taken on kernel_ms; the eager figures are back-to-back calls through the "
                    "Python op layer, bounded by the host's share of a call"})

        # ---- the same layer with offsets too far apart for the product form on their own (every row's scaled range far
        #      above 90): still the product form while every pixel's patch spans at most 90 (the largest term is then
        #      bounded through the patch instead), a max-tracked log-sum-exp on the VALU from the staged tiles when the
        #      patches are wide as well (input x 40); and an infinite epsilon (the maximum alone)
        OTHER_FORMS = {"wide_offsets": "rows beyond the product form's range, pixel patches within it: product form",
                       "wide_offsets_wide_pixels": "rows and pixel patches beyond it: max-tracked log-sum-exp on the VALU",
                       "eps_inf": "the maximum alone"}

        def other_forms(tag, X, off_np, n, kw, gmac, nbytes, shape_out):
            """device time per prepared call (HIP graph of 20) of the product form, wide offsets and eps = inf"""
            res = {}
            o = torch.empty(shape_out, device=dev)
            variants = (("product_form", off_np, kw, 1.0), ("wide_offsets", off_np * 1000.0, kw, 1.0),
                        ("wide_offsets_wide_pixels", off_np * 1000.0, kw, 40.0),
                        ("eps_inf", off_np, dict(kw, epsilon=math.inf), 1.0))
            for name, off_v, kw_v, xscale in variants:
                OV = to_dev(off_v.astype(np.float32))
                XV = X if xscale == 1.0 else X * xscale
                prep = pkg.mex_prepare(tuple(X.shape), OV, n, normalize_offsets=True, **kw_v)
                _, ms_v = timed(graph_of(lambda: prep(XV, out=o), 20).replay, args.steps, args.warmup)
                res[name] = (ms_v / 20, OV, kw_v, o.clone(), xscale)
            base = res["product_form"][0]
            out = {}
            for name, what in OTHER_FORMS.items():
                ms_v = res[name][0]
                e = entry(ms_v, gmac, nbytes, "hbm", flop=5, mex=True)
                e.update({"what": what, "product_form_kernel_ms": round(base, 4),
                          "ratio_to_product_form": round(ms_v / base, 2),
                          "entry_point": "simnets_hip_mex_fwd_prepared (device time per call, HIP graph of 20)"})
                out["%s_%s" % (tag, name)] = e
            return out, res

        forms2, keep2 = other_forms("config2_mex", X2, off2, n2, kw2, 33554432, 6324224, (64, 64, 16, 16))
        others.update(forms2)
        # one deep layer of the config-4 stack (128 x 4 x 4 -> 256 instances at batch 512: the panel kernel)
        xl3 = np.random.default_rng(1234).normal(size=(512, 128, 4, 4)).astype(np.float32)
        offl3 = (np.random.default_rng(4567).normal(size=(4, 256, 128, 1, 1)) * 0.1).astype(np.float32)
        kwl3 = dict(softmax_mode=True, blocks=[128, 1, 1], strides=[128, 1, 1], unshared_offset_region=[2])
        XL3 = to_dev(xl3)
        bytes_l3 = (xl3.size + offl3.size + 512 * 256 * 16) * 4
        forms3, keep3 = other_forms("config4_layer3_mex", XL3, offl3, 256, kwl3, 268435456, bytes_l3, (512, 256, 4, 4))
        others.update(forms3)

        def cpu_forms():
            """max error of the wide-offsets and infinite-epsilon results against the oracle (config-2 layer: all
            images; deep layer: 64 of the 512 images)"""
            out = {}
            for tag, keep, xs_np, off_np, n, nb in (("config2_mex", keep2, x2, off2, n2, 64),
                                                    ("config4_layer3_mex", keep3, xl3, offl3, 256, 64)):
                for name in OTHER_FORMS:
                    _, OV, kw_v, got, xscale = keep[name]
                    noff = oracle.normalize_offsets(OV.cpu().numpy())
                    xv = xs_np[:nb] if xscale == 1.0 else (xs_np[:nb] * np.float32(xscale))
                    out["%s_%s" % (tag, name)] = mex_err(got[:nb].cpu().numpy(), xv, noff, n, **kw_v)["floor_max_term"]
            return out
        cpu_jobs.append(("mex_other_forms_max_rel_err_gpu_vs_cpu", cpu_forms))

        def cpu2():
            got = o2.cpu().numpy()
            noff = oracle.normalize_offsets(off2)
            leg = cpu_leg("all 64 images of config 2, single thread", lambda: oracle.mex_fwd(x2, noff, n2, **kw2),
                          lambda: oracle.mex_fwd(x2, noff, n2, threads=threads, **kw2), 33554432, 33554432, None)
            errs = mex_err(got, x2, noff, n2, **kw2)
            leg["max_rel_err_gpu_vs_cpu"] = errs["floor_max_term"]
            leg["mex_errors"] = errs
            return leg
        cpu_jobs.append(("config2_mex", cpu2))

        # ---- configuration 4: Similarity -> 4 x (MEX + 2x2 sum pool) -> MEX(10), batch 512
        x4, t4, w4, kw4, layers_np, (offl_np, nl, kwl) = config4_stack(512)
        X4, T4, W4 = to_dev(x4), to_dev(t4), to_dev(w4)
        layers = [(to_dev(off), n, kw) for off, n, kw in layers_np]
        offl = to_dev(offl_np)

        def stack():
            cur = pkg.similarity(X4, T4, W4, **kw4)
            for off, n, kw in layers:
                cur = pkg.sum_pooling(pkg.mex(cur, off, n, normalize_offsets=True, **kw), (2, 2))
            return pkg.mex(cur, offl, nl, normalize_offsets=True, **kwl)

        _, ms = timed(stack, args.steps, args.warmup)
        # the same stack captured once into a HIP graph and replayed: 15 launches without per-launch host work
        graph = graph_of(stack, 1)
        _, ms_graph = timed(graph.replay, args.steps, args.warmup)
        gmac4 = 512 * 32 * 256 * 4 + 4 * 268435456 + 512 * 10 * 512
        bytes4 = 117e6   # compulsory traffic of the six operators (inputs, parameters, outputs once)
        e4 = entry(ms, gmac4, bytes4 + 79e6, "hbm", flop=5, mex=True)
        e4.update({"batch": 512, "kernels": "similarity + 4 x (offset pack + mex + sum pool) + offset pack + "
                                            "wave-per-pixel mex",
                   "hip_graph_replay_ms": round(ms_graph, 4)})
        others["config4_stack"] = e4
        # the same stack with every MEX + pooling pair as one call (a fused kernel for this geometry)
        def fused_stack():
            cur = pkg.similarity(X4, T4, W4, **kw4)
            for off, n, kw in layers:
                cur = pkg.mex_sum_pool(cur, off, n, (2, 2), normalize_offsets=True, **kw)
            return pkg.mex(cur, offl, nl, normalize_offsets=True, **kwl)

        _, ms_fused = timed(fused_stack, args.steps, args.warmup)
        e4["fused_pool_kernel_ms"] = round(ms_fused, 4)
        # ... with the Similarity layer evaluated inside the first of those kernels
        off0, n0, kwm0 = layers[0]

        def fused_stack3():
            cur = pkg.similarity_mex_sum_pool(X4, T4, W4, off0, n0, (2, 2), similarity=kw4,
                                              mex=dict(kwm0, normalize_offsets=True))
            for off, n, kw in layers[1:]:
                cur = pkg.mex_sum_pool(cur, off, n, (2, 2), normalize_offsets=True, **kw)
            return pkg.mex(cur, offl, nl, normalize_offsets=True, **kwl)

        _, ms_fused3 = timed(fused_stack3, args.steps, args.warmup)
        e4["fused_similarity_mex_pool_kernel_ms"] = round(ms_fused3, 4)
        # ... and with every layer prepared (parameters packed once): five launches per stack
        shapes, ch, size = [], 32, 16
        for _, n, _ in layers:
            shapes.append((512, ch, size, size))
            ch, size = n, size // 2
        pf = pkg.similarity_mex_sum_pool_prepare(x4.shape, T4, W4, off0, n0, (2, 2), similarity=kw4,
                                                 mex=dict(kwm0, normalize_offsets=True))
        pp = [pkg.mex_sum_pool_prepare(shapes[i], layers[i][0], layers[i][1], (2, 2), normalize_offsets=True,
                                       **layers[i][2]) for i in range(1, 4)]
        pl = pkg.mex_prepare((512, ch, 1, 1), offl, nl, normalize_offsets=True, **kwl)

        def prepared_stack():
            cur = pf(X4)
            for p in pp:
                cur = p(cur)
            return pl(cur)

        _, ms_prep = timed(prepared_stack, args.steps, args.warmup)
        e4.update({"fused_prepared_ms": round(ms_prep, 4),
                   "fused_prepared_hbm_frac": round((bytes4 / 1e9) / (ms_prep * 1e-3) / PEAK_HBM_GBS, 4),
                   "fused_prepared_bit_identical_to_fused": bool(torch.equal(prepared_stack(), fused_stack3()))})
        train_step = config4_training_step(X4, T4, W4, kw4, layers, offl, nl, kwl)
        _, ms_train = timed(train_step, args.steps, args.warmup)
        e4["train_step_ms"] = round(ms_train, 4)
        del train_step

        def cpu4():
            """The stack on the CPU oracle, layer by layer on 64 of the 512 images (single thread), all 512 with
            threads; the GPU's fused, prepared result against the oracle's on the 64 images."""
            def run(xb, th):
                cur = oracle.similarity_fwd(xb, t4, w4, threads=th, **kw4)
                for off, n, kw in layers_np:
                    y = oracle.mex_fwd(cur, oracle.normalize_offsets(off), n, threads=th, **kw)
                    B, Cc, H, W = y.shape
                    cur = y.reshape(B, Cc, H // 2, 2, W // 2, 2).sum(axis=(3, 5), dtype=np.float32)
                return oracle.mex_fwd(cur, oracle.normalize_offsets(offl_np), nl, threads=th, **kwl)
            nb = 64
            ref = [None]

            def single():
                ref[0] = run(x4[:nb], 1)
            got = prepared_stack()[:nb].cpu().numpy()
            leg = cpu_leg("%d of 512 images through the whole stack, single thread" % nb, single,
                          lambda: run(x4, threads), gmac4 * nb / 512, gmac4, None)
            leg["max_dev_of_scale_gpu_vs_cpu"] = float(np.abs(got - ref[0]).max() / np.abs(ref[0]).max())
            del leg["max_rel_err_gpu_vs_cpu"]
            return leg
        cpu_jobs.append(("config4_stack", cpu4))

        # ---- backward (configuration 5): gradients at the config-3 and config-2 shapes, upstream gradients ~N(0,1)
        G3 = to_dev(np.random.default_rng(6789).normal(size=(256, 128, 32, 32)).astype(np.float32))
        _, ms = timed(lambda: pkg.similarity_input_grad(X3, T3, W3, G3, similarity_function="L2", **kw3), args.steps,
                      args.warmup)
        others["config5_similarity_input_grad_L2"] = entry(ms, gmac3, 2 * 67108864 + 589824 + 134217728, "mfma", flop=4)
        _, ms = timed(lambda: pkg.similarity_parameters_grad(X3, T3, W3, G3, similarity_function="L2", **kw3),
                      args.steps, args.warmup)
        others["config5_similarity_params_grad_L2"] = entry(ms, gmac3, 67108864 + 3 * 589824 + 134217728, "mfma", flop=5)
        Y2 = pkg.mex(X2, O2, n2, normalize_offsets=True, **kw2)
        G2 = to_dev(np.random.default_rng(6789).normal(size=(64, 64, 16, 16)).astype(np.float32))
        _, ms = timed(lambda: pkg.mex_input_grad(X2, O2, Y2, G2, n2, normalize_offsets=True, **kw2), args.steps,
                      args.warmup)
        others["config5_mex_input_grad"] = entry(ms, 33554432, 2 * 2097152 + 2 * 4194304 + 32768, "hbm", flop=5, mex=True)
        _, ms = timed(lambda: pkg.mex_offsets_grad(X2, O2, Y2, G2, n2, normalize_offsets=True, **kw2), args.steps,
                      args.warmup)
        others["config5_mex_offsets_grad"] = entry(ms, 33554432, 2097152 + 2 * 4194304 + 2 * 32768, "hbm", flop=5,
                                                   mex=True)
        # ... and as a training step asks for them: both gradients from one call, without and with the offsets layout
        # that the forward call of the step kept (then nothing is packed)
        _, ms = timed(lambda: pkg.mex_grads(X2, O2, Y2, G2, n2, normalize_offsets=True, **kw2), args.steps, args.warmup)
        others["config5_mex_both_grads_one_call"] = entry(ms, 2 * 33554432, 2 * 2097152 + 2 * 4194304 + 2 * 32768, "hbm",
                                                          flop=5, mex=True)
        Y2s, saved2 = pkg.mex_saving(X2, O2, n2, normalize_offsets=True, **kw2)
        _, ms = timed(lambda: pkg.mex_grads(X2, O2, Y2s, G2, n2, normalize_offsets=True, saved=saved2, **kw2),
                      args.steps, args.warmup)
        others["config5_mex_both_grads_one_call_kept_offsets"] = entry(
            ms, 2 * 33554432, 2 * 2097152 + 2 * 4194304 + 2 * 32768, "hbm", flop=5, mex=True)

        def cpu5():
            """Achieved gradient errors against the fp64 oracle, beside the fp32 oracle's own: the error of an element
            relative to max(|want|, 1 % of the tensor's largest |want|); Similarity on 2 images of the config-3
            shape, MEX on 8 images of the config-2 shape."""
            def gerr(got, want):
                want = np.asarray(want)
                return rel_err(got, want, floor=np.full(want.shape, 1e-2 * float(np.abs(want).max())))
            f64 = lambda *a: [np.asarray(v, dtype=np.float64) for v in a]
            nb = 2
            xs, gs = x3[:nb], G3[:nb].cpu().numpy()
            XS, GS = to_dev(xs), to_dev(gs)
            out = {}
            for func in ("L2", "L1"):
                kw = dict(kw3, similarity_function=func)
                dx = pkg.similarity_input_grad(XS, T3, W3, GS, **kw).cpu().numpy()
                dt, dw = [v.cpu().numpy() for v in pkg.similarity_parameters_grad(XS, T3, W3, GS, **kw)]
                d = f64(xs, t3, w3, gs)
                tx = oracle.similarity_input_grad(*d, threads=threads, **kw)
                tt, tw = oracle.similarity_params_grad(*d, threads=threads, **kw)
                rx = oracle.similarity_input_grad(xs, t3, w3, gs, threads=threads, **kw)
                rt, rw = oracle.similarity_params_grad(xs, t3, w3, gs, threads=threads, **kw)
                out["similarity_" + func] = {"input": [gerr(dx, tx), gerr(rx, tx)], "templates": [gerr(dt, tt), gerr(rt, tt)],
                                             "weights": [gerr(dw, tw), gerr(rw, tw)]}
            nb = 8
            xm, gm = x2[:nb], G2[:nb].cpu().numpy()
            noff = oracle.normalize_offsets(off2)
            ym = oracle.mex_fwd(xm, noff, n2, **kw2)
            XM, GM, YM, NOFF = to_dev(xm), to_dev(gm), to_dev(ym), to_dev(noff)
            di = pkg.mex_input_grad(XM, NOFF, YM, GM, n2, **kw2).cpu().numpy()
            do = pkg.mex_offsets_grad(XM, NOFF, YM, GM, n2, **kw2).cpu().numpy()
            d = f64(xm, noff)
            y64 = oracle.mex_fwd(d[0], d[1], n2, **kw2)
            ti = oracle.mex_input_grad(d[0], d[1], y64, gm.astype(np.float64), n2, **kw2)
            to = oracle.mex_offsets_grad(d[0], d[1], y64, gm.astype(np.float64), n2, **kw2)
            ri = oracle.mex_input_grad(xm, noff, ym, gm, n2, **kw2)
            ro = oracle.mex_offsets_grad(xm, noff, ym, gm, n2, **kw2)
            out["mex"] = {"input": [gerr(di, ti), gerr(ri, ti)], "offsets": [gerr(do, to), gerr(ro, to)]}
            out["what"] = "[gpu, fp32 oracle] error against the fp64 oracle, relative to max(|want|, 1% of max|want|)"
            return out
        cpu_jobs.append(("config5_gradient_errors", cpu5))
    result["others"] = others

    # ------------------------------------------------------------------ CPU baselines (bounded samples)
    if not args.no_cpu:
        from oracle import oracle
        n_img = max(1, args.cpu_images)
        xs = x3[:n_img]
        t0 = time.perf_counter()
        ref = oracle.similarity_fwd(xs, t3, w3, similarity_function="L2", **kw3)
        dt = time.perf_counter() - t0
        xm = x3[:min(256, threads * 4)]
        t0 = time.perf_counter()
        oracle.similarity_fwd(xm, t3, w3, similarity_function="L2", threads=threads, **kw3)
        dtm = time.perf_counter() - t0
        gm = n_img * 128 * 1024 * 576
        gm_all = len(xm) * 128 * 1024 * 576
        got = pkg.similarity(X3[:n_img], T3, W3, similarity_function="L2", algo=args.algo, **kw3).cpu().numpy()
        err = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-6 * np.abs(ref).max())))
        # the reference's own ggemm_cpu (its header, compiled as it lies; include/utils/ggemm_cpu.hpp:462-511) on the
        # im2col matrices of a few of the same images: the loop the reference's CPU kernel spends its time in
        ref_ggemm = None
        if oracle.ref() is not None:
            A = np.ascontiguousarray(np.stack([t3.reshape(128, 576), w3.reshape(128, 576)], axis=-1))
            n_ref = min(n_img, 4)
            cols = []
            for i in range(n_ref):
                xp = np.pad(x3[i], ((0, 0), (1, 1), (1, 1)))
                cols.append(np.ascontiguousarray(np.stack([xp[:, dh:dh + 32, dw:dw + 32] for dh in range(3)
                                                           for dw in range(3)], axis=1).reshape(576, 1024)))
            t0 = time.perf_counter()
            outs = [oracle.ggemm_similarity(1, A, col, 128, 1024, 576, 0.001, "ref") for col in cols]
            dtr = time.perf_counter() - t0
            same = all(np.array_equal(o.reshape(128, 32, 32), ref[i]) for i, o in enumerate(outs))
            ref_ggemm = {"value": round(n_ref * 128 * 1024 * 576 / dtr / 1e9, 4), "unit": "GMAC/s", "images": n_ref,
                         "bit_identical_to_port": bool(same),
                         "what": "reference ggemm_cpu<sim_l2_forward> from its own header, im2col and interlace not timed"}
        result["cpu_baseline"] = {
            "value": round(gm / dt / 1e9, 4), "unit": "GMAC/s", "cores": 1, "kind": "port",
            "sample": "%d of 256 images of config 3 (L2), single thread like the reference; -O2, no fast-math" % n_img,
            "all_cores": {"value": round(gm_all / dtm / 1e9, 4), "threads": threads, "images": int(len(xm)),
                          "note": "batch loop spread over threads; not reference behaviour"},
            "host_cpus": host_cpus,
            "max_rel_err_gpu_vs_cpu": err,
        }
        if ref_ggemm is not None:
            result["cpu_baseline"]["reference_ggemm"] = ref_ggemm
        for name, job in cpu_jobs:
            leg = job()
            if name in others:
                others[name]["cpu_baseline"] = leg
            else:
                others[name] = leg
    print(json.dumps(result))


if __name__ == "__main__":
    main()
