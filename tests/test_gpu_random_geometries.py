"""Seeded random sweep over the attribute space of both operators, forward and backward, against the oracle.
Every case prints nothing and is small; the point is breadth (block/stride/padding combinations, template
counts around the tile sizes, region specifications, epsilon signs) beyond the hand-picked cases."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import rel_err
from test_gpu_grads import assert_grad_close, f64

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def random_similarity_case(g):
    while True:
        C = int(g.choice([1, 2, 3, 5, 8, 9, 17, 33]))
        O = int(g.choice([1, 2, 7, 8, 9, 16, 31, 40, 65]))
        H, W = int(g.integers(3, 40)), int(g.integers(3, 70))
        bh, bw = int(g.integers(1, min(H, 6) + 1)), int(g.integers(1, min(W, 6) + 1))
        sh, sw = int(g.integers(1, 5)), int(g.integers(1, 5))
        ph, pw = int(g.integers(0, bh + 1)), int(g.integers(0, bw + 1))
        mode = int(g.integers(0, 4))
        kw = dict(similarity_function="L1" if mode == 0 else "L2", blocks=[bh, bw], strides=[sh, sw], padding=[ph, pw],
                  normalization_term=mode >= 2, ignore_nan_input=mode == 3,
                  out_of_bounds_value=float("nan") if mode == 3 else float(g.normal()))
        B = int(g.integers(1, 4))
        try:
            orc.similarity_out_dims(orc.similarity_args((B, C, H, W), O, **{k: v for k, v in kw.items()}))
        except ValueError:
            continue
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        if mode == 3:
            x[g.random(size=x.shape) < 0.2] = np.nan
        t = g.normal(size=(O, C, bh, bw)).astype(np.float32)
        w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
        return x, t, w, kw


@pytest.mark.parametrize("seed", range(60))
def test_similarity_random_geometry(pkg, seed):
    g = np.random.default_rng(1000 + seed)
    x, t, w, kw = random_similarity_case(g)
    want = orc.similarity_fwd(x, t, w, **kw)
    got = pkg.similarity(dev(x), dev(t), dev(w), **kw).cpu().numpy()
    assert rel_err(got, want) <= 1e-5, kw
    go = g.normal(size=want.shape).astype(np.float32)
    dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(go), **kw).cpu().numpy()
    dt, dw = [a.cpu().numpy() for a in pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(go), **kw)]
    d = f64(x, t, w, go)
    assert_grad_close(dx, orc.similarity_input_grad(x, t, w, go, **kw), orc.similarity_input_grad(*d, **kw), "dX %s" % kw)
    w32, w64 = orc.similarity_params_grad(x, t, w, go, **kw), orc.similarity_params_grad(*d, **kw)
    assert_grad_close(dt, w32[0], w64[0], "dT %s" % kw)
    assert_grad_close(dw, w32[1], w64[1], "dW %s" % kw)


def random_mex_case(g):
    while True:
        C, H, W = int(g.choice([1, 2, 3, 6, 16, 70])), int(g.integers(1, 14)), int(g.integers(1, 14))
        blocks = [int(g.integers(1, C + 1)), int(g.integers(1, min(H, 4) + 1)), int(g.integers(1, min(W, 4) + 1))]
        strides = [int(g.integers(1, blocks[0] + 2)), int(g.integers(1, 4)), int(g.integers(1, 4))]
        padding = [int(g.integers(0, blocks[0])), int(g.integers(0, blocks[1])), int(g.integers(0, blocks[2]))]
        unshared = bool(g.integers(0, 2))
        spec = [[-1], [1], [2], [3], [1, 2, 3], [2, 1, 2], [-1, 2, -1]][int(g.integers(0, 7))]
        eps = [1.0, -1.0, 0.5, 3.0, -2.5, math.inf, -math.inf][int(g.integers(0, 7))]
        kw = dict(blocks=blocks, strides=strides, padding=padding, epsilon=eps, softmax_mode=bool(g.integers(0, 2)),
                  blocks_round_down=bool(g.integers(0, 2)), blocks_out_of_bounds_value=float(g.normal()),
                  use_unshared_regions=unshared, shared_offset_region=spec, unshared_offset_region=spec)
        n = int(g.choice([1, 2, 5, 16, 17, 40]))
        B = int(g.integers(1, 5))
        try:
            d = orc.mex_dims(orc.mex_args((B, C, H, W), n, **kw))
        except ValueError:
            continue
        if d.num_regions * n * d.K > 200000:
            continue
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        off = g.normal(size=(d.num_regions, n) + tuple(blocks)).astype(np.float32)
        return x, off, n, kw


@pytest.mark.parametrize("seed", range(60))
def test_mex_random_geometry(pkg, seed):
    g = np.random.default_rng(2000 + seed)
    x, off, n, kw = random_mex_case(g)
    want = orc.mex_fwd(x, off, n, **kw)
    shift = orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, kw["epsilon"])))
    got = pkg.mex(dev(x), dev(off), n, **kw).cpu().numpy()
    # against the fp32 oracle, or - where a log-sum-exp lands near zero and the fp32 oracle's own rounding shows -
    # against the float64 oracle with twice the fp32 oracle's error as the bar
    e32 = rel_err(got, want, floor=shift)
    if e32 > 1e-4:
        x64, off64 = f64(x, off)
        true = orc.mex_fwd(x64, off64, n, **kw)
        assert rel_err(got, true, floor=np.abs(shift)) <= max(1e-4, 2.0 * rel_err(want, true, floor=np.abs(shift))), kw
    go = g.normal(size=want.shape).astype(np.float32)
    dx = pkg.mex_input_grad(dev(x), dev(off), dev(want), dev(go), n, **kw).cpu().numpy()
    doff = pkg.mex_offsets_grad(dev(x), dev(off), dev(want), dev(go), n, **kw).cpu().numpy()
    x64, off64, g64 = f64(x, off, go)
    out64 = orc.mex_fwd(x64, off64, n, **kw)
    if math.isinf(kw["epsilon"]):
        # the indicator (patch + offset == out) is evaluated on the fp32 data the op saw: compare with the fp32 oracle
        assert rel_err(dx, orc.mex_input_grad(x, off, want, go, n, **kw), floor=np.full(dx.shape, 1e-2 * np.abs(dx).max())) <= 1e-4, kw
        assert rel_err(doff, orc.mex_offsets_grad(x, off, want, go, n, **kw),
                       floor=np.full(doff.shape, 1e-2 * np.abs(doff).max())) <= 1e-4, kw
    else:
        assert_grad_close(dx, orc.mex_input_grad(x, off, want, go, n, **kw),
                          orc.mex_input_grad(x64, off64, out64, g64, n, **kw), "dX %s" % kw)
        assert_grad_close(doff, orc.mex_offsets_grad(x, off, want, go, n, **kw),
                          orc.mex_offsets_grad(x64, off64, out64, g64, n, **kw), "dOff %s" % kw)


def random_matrix_gradient_case(g):
    """Geometries the matrix-core gradient kernels take (L2 modes, at least 24 channels and 8 templates): small maps
    that share a workgroup tile, strides with two, four or more phases, contractions long enough to be split."""
    while True:
        C = int(g.choice([24, 25, 31, 33, 48, 64, 70]))
        O = int(g.choice([8, 9, 17, 30, 65, 100, 131]))
        small = bool(g.integers(0, 2))
        H, W = (int(g.integers(2, 12)), int(g.integers(2, 12))) if small else (int(g.integers(12, 34)), int(g.integers(12, 60)))
        bh, bw = int(g.integers(1, min(H, 5) + 1)), int(g.integers(1, min(W, 5) + 1))
        sh, sw = int(g.integers(1, min(bh, 3) + 1)), int(g.integers(1, min(bw, 3) + 1))
        ph, pw = int(g.integers(0, bh)), int(g.integers(0, bw))
        mode = int(g.integers(1, 4))
        B = int(g.integers(1, 10)) if small else int(g.integers(1, 4))
        kw = dict(similarity_function="L2", blocks=[bh, bw], strides=[sh, sw], padding=[ph, pw],
                  normalization_term=mode >= 2, ignore_nan_input=mode == 3,
                  out_of_bounds_value=float("nan") if mode == 3 else float(g.normal()))
        try:
            oh, ow = orc.similarity_out_dims(orc.similarity_args((B, C, H, W), O, **kw))
        except ValueError:
            continue
        if B * O * C * bh * bw * oh * ow > 40_000_000:
            continue
        x = (2.0 + g.normal(size=(B, C, H, W))).astype(np.float32)
        if mode == 3:
            x[g.random(size=x.shape) < 0.2] = np.nan
        t = (2.0 + g.normal(size=(O, C, bh, bw))).astype(np.float32)
        w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
        return x, t, w, kw


@pytest.mark.parametrize("seed", range(48))
def test_similarity_matrix_gradient_random_geometry(pkg, seed):
    g = np.random.default_rng(3000 + seed)
    x, t, w, kw = random_matrix_gradient_case(g)
    out = orc.similarity_fwd(x, t, w, **kw)
    go = g.normal(size=out.shape).astype(np.float32)
    dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(go), **kw).cpu().numpy()
    dt, dw = [a.cpu().numpy() for a in pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(go), **kw)]
    d = f64(x, t, w, go)
    want = orc.similarity_input_grad(x, t, w, go, **kw)
    assert np.array_equal(np.isnan(dx), np.isnan(want)), kw
    assert_grad_close(np.nan_to_num(dx), np.nan_to_num(want), np.nan_to_num(orc.similarity_input_grad(*d, **kw)),
                      "dX %s %s" % (x.shape, kw))
    w32, w64 = orc.similarity_params_grad(x, t, w, go, **kw), orc.similarity_params_grad(*d, **kw)
    assert_grad_close(dt, w32[0], w64[0], "dT %s" % kw)
    assert_grad_close(np.nan_to_num(dw), np.nan_to_num(w32[1]), np.nan_to_num(w64[1]), "dW %s" % kw)
