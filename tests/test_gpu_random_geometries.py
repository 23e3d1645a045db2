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


@pytest.mark.parametrize("seed", range(40))
def test_mex_whole_channel_layers_random_geometry(pkg, seed):
    # 2x2 unshared offsets over all channels of a pixel, channel counts and power-of-two maps around what the panel
    # kernel takes (and just outside: odd channel counts, widths that are no power of two), plain and with pooling
    g = np.random.default_rng(7000 + seed)
    C = int(g.choice([32, 64, 128, 256, 48, 96]))
    H = int(g.choice([2, 4, 8, 16, 6]))
    W = int(g.choice([2, 4, 8, 16, 32, 64, 12]))
    B = int(g.integers(1, 24))
    while B * C * H * W > 600_000:
        B = max(1, B // 2)
        if B == 1:
            break
    n = int(g.choice([1, 10, 16, 63, 64, 65, 130]))
    if B * C * H * W * n > 30_000_000:
        n = 10
    eps = float(g.choice([1.0, 0.25, 4.0, -1.5]))
    kw = dict(softmax_mode=bool(g.integers(0, 2)), blocks=[C, 1, 1], strides=[C, 1, 1], epsilon=eps,
              use_unshared_regions=True, unshared_offset_region=[1, 2, 2])
    x = (g.normal(size=(B, C, H, W)) * float(g.choice([0.5, 5.0, 40.0]))).astype(np.float32)
    off = (g.normal(size=(4, n, C, 1, 1)) * float(g.choice([0.1, 1.0, 30.0]))).astype(np.float32)
    if g.random() < 0.3:
        off[:, n // 2:] *= 20
    if g.random() < 0.3:
        x[g.random(size=x.shape) < 0.1] = -math.inf if eps > 0 else math.inf
    with np.errstate(invalid="ignore", over="ignore"):
        want = orc.mex_fwd(x, off, n, **kw)
        shift = np.abs(orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, eps))))
    got = pkg.mex(dev(x), dev(off), n, **kw).cpu().numpy()
    fused = pkg.mex_sum_pool(dev(x), dev(off), n, (2, 2), **kw).cpu().numpy()
    assert np.array_equal(np.isfinite(got), np.isfinite(want)), kw
    fin = np.isfinite(want)
    assert np.array_equal(got[~fin], want[~fin], equal_nan=True), kw
    bar = np.maximum(np.abs(want), shift)
    assert (np.abs(got[fin] - want[fin]) <= 1e-4 * np.maximum(bar[fin], 1e-30)).all(), kw

    def pool(y):
        return y.reshape(B, n, H // 2, 2, W // 2, 2).sum(axis=(3, 5))
    with np.errstate(invalid="ignore"):
        wantp, barp = pool(want), pool(bar)
    finp = np.isfinite(wantp)
    assert np.array_equal(np.isfinite(fused), finp), kw
    assert (np.abs(fused[finp] - wantp[finp]) <= 1e-4 * np.maximum(barp[finp], 1e-30)).all(), kw


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
