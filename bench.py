#!/usr/bin/env python3
"""Benchmark of the SimNets Similarity / MEX hot path on one MI355X.

One "step" = one Similarity L2 forward over benchmark configuration 3 (input 256x64x32x32, 128
templates 64x3x3, stride 1, padding 1 -> 256x128x32x32; 19.33 G generalized MACs), inputs already
resident in HBM, called through the C ABI exactly as an op layer would.  The other configurations
(1, 2, 3-L1, 4, and the backward operators of configuration 5) and the alternative evaluation paths
are timed in the same run and reported under "others".  Prints ONE JSON line.

The CPU baseline leg times the CPU oracle (a restatement of the reference's CPU kernels) on a
bounded sample of the same workload; it is the only place this file touches oracle/.
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
EXP_RATE = 19.66e12        # v_exp_f32 at a quarter of the 128 lanes/clk/CU VALU rate (17.6e12 measured on the box)

# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this
# same workload scaled by a copy kernel of known size (profiles/sim_direct_l2_config3.md).
# Keyed by evaluation path; None where no counter run exists for the current kernel.
MEASURED_TRAFFIC_BYTES = {"sqrtw": 311.3e6, "direct": 287.0e6, "mfma": 223.3e6}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle", type=float, default=1.5,
                    help="seconds of untimed load before the warm-up steps (lets the clocks of an idle GPU settle)")
    ap.add_argument("--algo", default=None, choices=[None, "direct", "sqrtw", "mfma"],
                    help="evaluation path of the headline Similarity kernel (default: the library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="time only the headline workload")
    ap.add_argument("--pmc-calib", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a plain copy kernel of known size, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--cpu-images", type=int, default=24,
                    help="images of configuration 3 the single-threaded CPU baseline times (24 ~ 6 s)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path is data parallel over the batch; "
              "each GPU would take a share of the images); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from __graft_entry__ import load_package, build
    from util import config1, config2, config3

    if not os.path.exists(os.path.join(ROOT, "simnets-tf_amd", "libsimnets_hip.so")):
        build()
    pkg = load_package()
    assert torch.cuda.is_available(), "bench.py needs a GPU: there is no CPU fallback"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    def to_dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def timed(fn, steps, warmup):
        """(wall ms per step, HIP-event ms per step) for `steps` calls after `warmup` calls.
        The events are recorded on the stream the kernels are launched on (torch's current stream,
        whose handle the op layer passes through the C ABI)."""
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
    settle_until = time.perf_counter() + args.settle
    while time.perf_counter() < settle_until:
        for _ in range(50):
            sim3("L2", args.algo)()
        torch.cuda.synchronize()
    wall_ms, ev_ms = timed(sim3("L2", args.algo), args.steps, args.warmup)
    gmacs = gmac3 / (ev_ms * 1e-3)
    flop_per_gmac = 4
    achieved_tflops = gmacs * flop_per_gmac / 1e12
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
                   "algo": args.algo or "auto (sqrt-weight form + exact recomputation of near-zero outputs)",
                   "gmac_per_step": gmac3},
        # compute bound at the FP32 peak, which is the same figure for the vector ALU and the FP32 matrix
        # cores; "engine" says which of the two the kernel runs on
        "roofline": {"bound": "mfma", "engine": "mfma" if args.algo == "mfma" else "valu",
                     "achieved": round(achieved_tflops, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved_tflops / PEAK_FP32_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.algo or "sqrtw"),
                     "kernel_ms": round(ev_ms, 4), "flop_per_gmac": flop_per_gmac,
                     "algorithmic_bytes": bytes3,
                     "hbm_frac": round(bytes3 / (ev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)},
    }

    # ------------------------------------------------------------------ the other configurations
    others = {}
    if not args.no_others:
        def entry(ms, gmac, nbytes, flop=None, exp_bound=False):
            e = {"kernel_ms": round(ms, 4), "gmac_per_s_G": round(gmac / (ms * 1e-3) / 1e9, 1),
                 "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
            if flop:
                e["valu_frac"] = round(gmac / (ms * 1e-3) * flop / 1e12 / PEAK_FP32_TFLOPS, 4)
            if exp_bound:
                # MEX: 1 exp + 5 flop per gMAC
                e["exp_frac"] = round(gmac / (ms * 1e-3) / EXP_RATE, 4)
                e["valu_frac"] = round(gmac / (ms * 1e-3) * 5 / 1e12 / PEAK_FP32_TFLOPS, 4)
            return e

        _, ms = timed(sim3("L1", None), args.steps, args.warmup)
        others["config3_L1_direct"] = entry(ms, gmac3, bytes3, flop=3)
        for algo in ("direct", "sqrtw", "mfma"):
            if algo == (args.algo or "sqrtw"):
                continue
            try:
                _, ms = timed(sim3("L2", algo), args.steps, args.warmup)
                others["config3_L2_" + algo] = entry(ms, gmac3, bytes3, flop=4)
            except pkg.SimnetsError as e:
                others["config3_L2_" + algo] = {"error": str(e)}

        x1, t1, w1, kw1 = config1(batch=64, nan_frac=0.0)
        X1, T1, W1 = to_dev(x1), to_dev(t1), to_dev(w1)
        o1 = torch.empty((64, 32, 16, 16), device=dev)
        _, ms = timed(lambda: pkg.similarity(X1, T1, W1, out=o1, **kw1), args.steps, args.warmup)
        others["config1_similarity"] = entry(ms, 2097152, 2298880, flop=6)

        x2, off2, n2, kw2 = config2()
        X2, O2 = to_dev(x2), to_dev(off2)
        o2 = torch.empty((64, 64, 16, 16), device=dev)
        _, ms = timed(lambda: pkg.mex(X2, O2, n2, normalize_offsets=True, out=o2, **kw2), args.steps, args.warmup)
        others["config2_mex"] = entry(ms, 33554432, 6324224, exp_bound=True)

        # configuration 4: Similarity -> 4 x (MEX + 2x2 sum pool) -> MEX(10), batch 512
        x4, t4, w4, kw4 = config1(batch=512, nan_frac=0.25)
        X4, T4, W4 = to_dev(x4), to_dev(t4), to_dev(w4)
        g = np.random.default_rng(4567)
        layers, ch, size = [], 32, 16
        for _ in range(4):
            n = ch * 2
            off = to_dev((g.normal(size=(4 if size > 1 else 1, n, ch, 1, 1)) * 0.1).astype(np.float32))
            layers.append((off, n, dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1],
                                        unshared_offset_region=[2])))
            ch, size = n, size // 2
        offl = to_dev((g.normal(size=(1, 10, ch, 1, 1)) * 0.1).astype(np.float32))

        def stack():
            cur = pkg.similarity(X4, T4, W4, **kw4)
            for off, n, kw in layers:
                cur = pkg.sum_pooling(pkg.mex(cur, off, n, normalize_offsets=True, **kw), (2, 2))
            return pkg.mex(cur, offl, 10, normalize_offsets=True, softmax_mode=True, blocks=[ch, 1, 1],
                           strides=[ch, 1, 1], shared_offset_region=[1])

        _, ms = timed(stack, args.steps, args.warmup)
        # the same stack captured once into a HIP graph and replayed: 15 launches without per-launch host work
        stack()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            stack()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            graph_out = stack()
        _, ms_graph = timed(graph.replay, args.steps, args.warmup)
        graph_ok = bool(torch.equal(graph_out, stack()))
        gmac4 = 512 * 32 * 256 * 4 + 4 * 268435456 + 512 * 10 * 512
        others["config4_stack"] = {"kernel_ms": round(ms, 4), "gmac_per_s_G": round(gmac4 / (ms * 1e-3) / 1e9, 1),
                                   "exp_frac": round(gmac4 / (ms * 1e-3) / EXP_RATE, 4), "batch": 512,
                                   "kernels": "similarity + 4 x (offset pack + mex + sum pool) + wave-per-pixel mex",
                                   "hip_graph_replay_ms": round(ms_graph, 4), "hip_graph_matches_eager": graph_ok}
        # the same stack with every MEX + pooling pair as one call (a fused kernel for this geometry)
        def fused_stack():
            cur = pkg.similarity(X4, T4, W4, **kw4)
            for off, n, kw in layers:
                cur = pkg.mex_sum_pool(cur, off, n, (2, 2), normalize_offsets=True, **kw)
            return pkg.mex(cur, offl, 10, normalize_offsets=True, softmax_mode=True, blocks=[ch, 1, 1],
                           strides=[ch, 1, 1], shared_offset_region=[1])

        _, ms_fused = timed(fused_stack, args.steps, args.warmup)
        ref4 = stack()
        dev4 = float((fused_stack() - ref4).abs().max() / ref4.abs().max())
        others["config4_stack"].update({"fused_pool_kernel_ms": round(ms_fused, 4),
                                        "fused_pool_max_dev_of_scale": dev4})

        # ... and with the Similarity layer evaluated inside the first of those kernels
        off0, n0, kwm0 = layers[0]

        def fused_stack3():
            cur = pkg.similarity_mex_sum_pool(X4, T4, W4, off0, n0, (2, 2), similarity=kw4,
                                              mex=dict(kwm0, normalize_offsets=True))
            for off, n, kw in layers[1:]:
                cur = pkg.mex_sum_pool(cur, off, n, (2, 2), normalize_offsets=True, **kw)
            return pkg.mex(cur, offl, 10, normalize_offsets=True, softmax_mode=True, blocks=[ch, 1, 1],
                           strides=[ch, 1, 1], shared_offset_region=[1])

        _, ms_fused3 = timed(fused_stack3, args.steps, args.warmup)
        dev43 = float((fused_stack3() - ref4).abs().max() / ref4.abs().max())
        others["config4_stack"].update({"fused_similarity_mex_pool_kernel_ms": round(ms_fused3, 4),
                                        "fused_similarity_mex_pool_max_dev_of_scale": dev43})
        # a training step of the same stack through the differentiable layer functions: forward with the unfused
        # MEX calls (their gradients take the unpooled outputs), then every operator's gradient calls
        L = pkg.layers
        train_params = [T4.clone().requires_grad_(), W4.clone().requires_grad_()] + \
                       [off.clone().requires_grad_() for off, _, _ in layers] + [offl.clone().requires_grad_()]

        def train_step():
            for q in train_params:
                q.grad = None
            cur = L.similarity(X4, train_params[0], train_params[1], **kw4)
            for i, (_, n, kw) in enumerate(layers):
                cur = L.mex_sum_pool(cur, train_params[2 + i], n, (2, 2), normalize_offsets=True, **kw)
            out = L.mex(cur, train_params[-1], 10, normalize_offsets=True, softmax_mode=True, blocks=[ch, 1, 1],
                        strides=[ch, 1, 1], shared_offset_region=[1])
            out.sum().backward()

        _, ms_train = timed(train_step, args.steps, args.warmup)
        others["config4_stack"]["train_step_ms"] = round(ms_train, 4)
        del train_params
        # backward (configuration 5): gradients at the config-3 and config-2 shapes, upstream gradients ~N(0,1)
        G3 = to_dev(np.random.default_rng(6789).normal(size=(256, 128, 32, 32)).astype(np.float32))
        _, ms = timed(lambda: pkg.similarity_input_grad(X3, T3, W3, G3, similarity_function="L2", **kw3), args.steps,
                      args.warmup)
        others["config5_similarity_input_grad_L2"] = entry(ms, gmac3, 2 * 67108864 + 589824 + 134217728, flop=4)
        _, ms = timed(lambda: pkg.similarity_parameters_grad(X3, T3, W3, G3, similarity_function="L2", **kw3),
                      args.steps, args.warmup)
        others["config5_similarity_params_grad_L2"] = entry(ms, gmac3, 67108864 + 3 * 589824 + 134217728, flop=5)
        del G3
        Y2 = pkg.mex(X2, O2, n2, normalize_offsets=True, **kw2)
        G2 = to_dev(np.random.default_rng(6789).normal(size=(64, 64, 16, 16)).astype(np.float32))
        _, ms = timed(lambda: pkg.mex_input_grad(X2, O2, Y2, G2, n2, normalize_offsets=True, **kw2), args.steps,
                      args.warmup)
        others["config5_mex_input_grad"] = entry(ms, 33554432, 2 * 2097152 + 2 * 4194304 + 32768, exp_bound=True)
        _, ms = timed(lambda: pkg.mex_offsets_grad(X2, O2, Y2, G2, n2, normalize_offsets=True, **kw2), args.steps,
                      args.warmup)
        others["config5_mex_offsets_grad"] = entry(ms, 33554432, 2097152 + 2 * 4194304 + 2 * 32768, exp_bound=True)
    result["others"] = others

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    if not args.no_cpu:
        from oracle import oracle
        n_img = max(1, args.cpu_images)
        xs = x3[:n_img]
        t0 = time.perf_counter()
        ref = oracle.similarity_fwd(xs, t3, w3, similarity_function="L2", **kw3)
        dt = time.perf_counter() - t0
        cores = os.cpu_count() or 1
        threads = min(cores, 16)
        xm = x3[:min(256, threads * n_img)]
        t0 = time.perf_counter()
        oracle.similarity_fwd(xm, t3, w3, similarity_function="L2", threads=threads, **kw3)
        dtm = time.perf_counter() - t0
        gm = n_img * 128 * 1024 * 576
        gm_all = len(xm) * 128 * 1024 * 576
        got = out3.cpu().numpy() if False else pkg.similarity(X3[:n_img], T3, W3, similarity_function="L2",
                                                               algo=args.algo, **kw3).cpu().numpy()
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
            "host_cpus": cores,
            "max_rel_err_gpu_vs_cpu": err,
        }
        if ref_ggemm is not None:
            result["cpu_baseline"]["reference_ggemm"] = ref_ggemm
    print(json.dumps(result))


if __name__ == "__main__":
    main()
