#!/usr/bin/env python3
"""Writes tests/golden/ref_headers.npz: input/output vectors of the reference's own header-only CPU
building blocks, produced by oracle/_ref/libsimnets_ref.so (the reference's include/utils headers compiled
as they lie in the reference checkout; see oracle/ref_shim.cpp).  Run where that library has been built:

    make -C oracle && python tests/golden/make_golden.py

The fixture travels with the repository, so the oracle and the HIP library can be checked against the
reference's arithmetic on machines that have no reference checkout.  Contents (all fp32):
  ggemm_mode{0..3}_{A,B,C}   ggemm_cpu with sim_l1_forward / sim_l2_forward / sim_l2_normalized_forward
                             (plain and ignore-NaN): A [M,K,2] interlaced (template, weight), B [K,N] -> C [M,N]
  mex_{i}_{off,in,out,meta}  mex_forward (max pass + exp/sum/log pass): offsets [R,M,K], in [R,K,N] -> out [R,M,N];
                             meta = (softmax_mode, epsilon)
  split_{i}_{src,dst,meta}   split_patches_cpu forward: src [Dim,N] -> dst (untouched slots hold -7);
                             meta = (C,H,W, C_groups,H_groups,W_groups, C_step,H_step,W_step, use_unshared)
  bw_args / bw_weights{0..3} / bw_bottom{0..3} / bw_mex{0,1}
                             backward functors on a grid of scalar arguments (err, x, t, w, fudge, top)
"""
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402


def main():
    if orc.ref() is None:
        sys.exit("oracle/_ref/libsimnets_ref.so is missing: run `make -C oracle` next to a reference checkout")
    out = {}
    for mode in range(4):
        g = np.random.default_rng(500 + mode)
        M, N, K = 9, 70, 37
        A = np.empty((M, K, 2), np.float32)
        A[..., 0] = g.normal(size=(M, K))
        A[..., 1] = np.abs(g.normal(size=(M, K))) + 0.01
        B = g.normal(size=(K, N)).astype(np.float32)
        if mode == 3:
            B[g.random(size=B.shape) < 0.3] = np.nan
            B[:, 5] = np.nan
        out["ggemm_mode%d_A" % mode], out["ggemm_mode%d_B" % mode] = A, B
        out["ggemm_mode%d_C" % mode] = orc.ggemm_similarity(mode, A, B, M, N, K, 0.001, "ref")
    cases = [(s, e) for s in (False, True) for e in (1.0, -1.0, 2.5, -0.3, math.inf, -math.inf)]
    for i, (softmax, eps) in enumerate(cases):
        g = np.random.default_rng(600 + i)
        R, M, N, K = 4, 6, 36, 13
        off = g.normal(size=(R, M, K)).astype(np.float32)
        inp = (g.normal(size=(R, K, N)) * 3).astype(np.float32)
        out["mex_%d_off" % i], out["mex_%d_in" % i] = off, inp
        out["mex_%d_out" % i] = orc.mex_forward(off, inp, M, N, K, softmax, eps, R, "ref")
        out["mex_%d_meta" % i] = np.array([float(softmax), eps], np.float64)
    geoms = [((1, 16, 16), (1, 2, 2), (1, 8, 8)), ((3, 41, 40), (1, 14, 14), (3, 3, 3)), ((3, 9, 10), (2, 3, 4), (2, 3, 3))]
    i = 0
    for (Cc, H, W), (Cg, Hg, Wg), (Cs, Hs, Ws) in geoms:
        for unshared in (0, 1):
            g = np.random.default_rng(700 + i)
            N, Dim = Cc * H * W, 5
            src = g.normal(size=(Dim, N)).astype(np.float32)
            dst = np.full(Cg * Hg * Wg * Cs * Hs * Ws * Dim, -7.0, np.float32)
            orc.split_patches(False, src, dst, N, Dim, W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared, "ref")
            out["split_%d_src" % i], out["split_%d_dst" % i] = src, dst
            out["split_%d_meta" % i] = np.array([Cc, H, W, Cg, Hg, Wg, Cs, Hs, Ws, unshared], np.int32)
            i += 1
    g = np.random.default_rng(800)
    args = g.normal(size=(300, 6)).astype(np.float32)   # err, x, t, w, fudge, top
    args[:, 3] = np.abs(args[:, 3]) + 0.1
    args[:, 4] = np.abs(args[:, 4]) * 0.01
    args[::7, 1] = np.nan
    args[::11, 1] = args[::11, 2]
    out["bw_args"] = args
    for mode in range(4):
        out["bw_weights%d" % mode] = np.array(
            [orc.backward_functor("sim_backward_weights_fn", np.float32, mode, a[0], a[1], a[2], a[3], a[4], which="ref")
             for a in args], np.float32)
        out["bw_bottom%d" % mode] = np.array(
            [orc.backward_functor("sim_backward_bottom_fn", np.float32, mode, a[2], a[3], a[0], a[1], which="ref")
             for a in args], np.float32)
    fin = args[~np.isnan(args[:, 1])]
    out["bw_mex_args"] = fin
    for finite in (0, 1):
        rows = []
        for a in fin:
            top = a[1] + a[2] if (finite == 0 and a[5] > 0) else a[5]
            rows.append(orc.backward_functor("mex_backward_term_fn", np.float32, finite, a[2], top, a[0], a[1], a[3], a[4],
                                             which="ref"))
        out["bw_mex%d" % finite] = np.array(rows, np.float32)
    path = os.path.join(HERE, "ref_headers.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
