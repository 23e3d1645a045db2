"""Infinite and NaN inputs, switched-off elements, zero weights and overflowing squares on seeded random layers:
NaN positions and infinite values must be the reference's exactly (the oracle's), finite values within the operators'
tolerances.  Missing data reaches these operators as NaN (Similarity with ignore_nan_input) or as -inf log-probabilities
(MEX), so the special values are inputs of ordinary use, not only error paths."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def compare(got, want, floor, tol, what):
    """NaN positions and infinite values exactly; finite values relative to max(|want|, floor)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want)), "%s: NaN positions differ" % what
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]), "%s: infinite values differ" % what
    fin = np.isfinite(want)
    if fin.any():
        den = np.maximum(np.abs(want), floor)[fin]
        err = float((np.abs(got[fin] - want[fin]) / np.maximum(den, 1e-30)).max())
        assert err <= tol, "%s: %.3g" % (what, err)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_similarity_special_values_on_random_layers(pkg, seed):
    """All four modes; inputs with +inf, -inf or NaN entries, zero weights beside infinite inputs (0 * inf), squares that
    overflow; the default form (sqrt-weight arithmetic with its guard for plain L2) and algo='direct'.  Templates stay
    finite: with ignore_nan_input the kernels mask a skipped term by a multiplication, the reference skips it."""
    rng = np.random.default_rng(9000 + seed)
    ran = 0
    for case in range(40):
        func = "L1" if case % 4 == 0 else "L2"
        norm = func == "L2" and case % 4 >= 2
        ign = norm and case % 4 == 3
        C, H, W = int(rng.choice([1, 2, 3, 8, 24, 64])), int(rng.integers(3, 40)), int(rng.integers(3, 40))
        blocks = [int(rng.integers(1, min(5, H) + 1)), int(rng.integers(1, min(5, W) + 1))]
        strides = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        padding = [int(rng.integers(0, 3)), int(rng.integers(0, 3))]
        O = int(rng.choice([1, 7, 8, 9, 31, 32, 33, 64, 130]))
        B = int(rng.integers(1, max(2, min(20, 3000000 // (H * W * C * O * blocks[0] * blocks[1])) + 1)))
        g = np.random.default_rng(int(rng.integers(1 << 30)))
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        t = g.normal(size=(O, C) + tuple(blocks)).astype(np.float32)
        w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
        what = int(rng.integers(0, 5))
        if what == 0:
            x[g.random(size=x.shape) < 0.02] = np.inf
        elif what == 1:
            x[g.random(size=x.shape) < 0.02] = -np.inf
        elif what == 2:
            x[g.random(size=x.shape) < 0.02] = np.nan
        elif what == 3:
            w[g.random(size=w.shape) < 0.1] = 0.0
            x[g.random(size=x.shape) < 0.01] = np.inf
        else:
            x *= 1e18
            t *= 1e18
        oob = float("nan") if ign else float(rng.choice([0.0, 0.75, np.inf]))
        kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding, normalization_term=norm,
                  ignore_nan_input=ign, out_of_bounds_value=oob)
        try:
            with np.errstate(all="ignore"):
                want = orc.similarity_fwd(x, t, w, **kw)
        except ValueError:
            continue
        ran += 1
        tag = "case %d %s O=%d values %d %s" % (case, (B, C, H, W), O, what, kw)
        fin = np.isfinite(want)
        floor = 1e-6 * float(np.abs(want[fin]).max()) if fin.any() else 0.0
        compare(pkg.similarity(dev(x), dev(t), dev(w), **kw).cpu().numpy(), want, floor, 1e-5, tag)
        if func == "L2" and not norm:
            compare(pkg.similarity(dev(x), dev(t), dev(w), algo="direct", **kw).cpu().numpy(), want, floor, 1e-5,
                    "direct, " + tag)
    assert ran >= 30


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_mex_special_values_on_random_layers(pkg, seed):
    """Forward and both gradients; inputs with scattered or whole channels of -inf (+inf for a negative epsilon: the
    elements drop out), patches with nothing finite (NaN for finite epsilon, like the reference's exp(inf - inf)),
    the other infinity and NaN (which poison their patch), offsets that switch elements off, either sign of epsilon
    and +-inf.  Gradients against the fp64 oracle on the fp32 forward output."""
    rng = np.random.default_rng(9100 + seed)
    ran = 0
    for case in range(45):
        kind = case % 3
        if kind == 0:
            H, W = 1 << int(rng.integers(1, 4)), 1 << int(rng.integers(1, 5))
            C = int(rng.choice([3, 8, 32, 33, 64, 100]))
            blocks, strides = [C, 1, 1], [C, 1, 1]
        elif kind == 1:
            H, W = int(rng.integers(1, 8)), int(rng.integers(1, 8))
            C = int(rng.choice([3, 8, 32, 40, 64, 130]))
            blocks, strides = [C, 1, 1], [C, 1, 1]
        else:
            H, W, C = int(rng.integers(3, 8)), int(rng.integers(3, 8)), int(rng.integers(2, 6))
            blocks = [int(rng.integers(1, C + 1)), int(rng.integers(1, 3)), int(rng.integers(1, 3))]
            strides = [int(rng.integers(1, blocks[0] + 1)), int(rng.integers(1, 3)), int(rng.integers(1, 3))]
        n = int(rng.integers(1, 70))
        B = int(rng.integers(1, max(2, min(10, 30000 // max(1, H * W * C * n // 4)) + 1)))
        unshared = bool(rng.integers(0, 2))
        region = [1, 2, 2] if rng.integers(0, 2) else [int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        eps = float(rng.choice([1.0, -1.0, 2.5, -0.4, math.inf, -math.inf]))
        kw = dict(blocks=blocks, strides=strides, padding=[0, 0, 0], epsilon=eps, softmax_mode=bool(rng.integers(0, 2)),
                  use_unshared_regions=unshared)
        kw["unshared_offset_region" if unshared else "shared_offset_region"] = region
        try:
            d = orc.mex_dims(orc.mex_args((B, C, H, W), n, **kw))
        except ValueError:
            continue
        g = np.random.default_rng(int(rng.integers(1 << 30)))
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        lo = -math.inf if eps > 0 else math.inf
        mode = int(rng.integers(0, 5))
        if mode == 0:
            x[g.random(size=x.shape) < 0.05] = lo
        elif mode == 1:
            x[:, 0] = lo
        elif mode == 2:
            x[g.random(size=x.shape) < 0.3] = lo
        elif mode == 3:
            x[g.random(size=x.shape) < 0.03] = np.nan
        else:
            x[g.random(size=x.shape) < 0.03] = -lo
        off = (g.normal(size=(d.num_regions, n) + tuple(blocks)) * float(rng.choice([0.3, 2.0]))).astype(np.float32)
        if rng.integers(0, 2):
            off[g.random(size=off.shape) < 0.05] = lo
        tag = "case %d %s n=%d values %d %s" % (case, (B, C, H, W), n, mode, kw)
        with np.errstate(all="ignore"):
            out = orc.mex_fwd(x, off, n, **kw)
            shift = np.abs(orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, eps))))
            # the forward metric's floor: |m|, the extreme term every implementation subtracts first - and, where that
            # happens to be near zero, 2 % of the operands' size (rounding noise follows the terms, not their extreme)
            size = float(np.abs(x[np.isfinite(x)]).max()) + float(np.abs(off[np.isfinite(off)]).max())
            shift = np.maximum(np.where(np.isfinite(shift), shift, 0.0), 0.02 * size)
            X, O = dev(x), dev(off)
            got = pkg.mex(X, O, n, **kw)
            compare(got.cpu().numpy(), out, shift, 1e-4, "forward, " + tag)
            gy = g.normal(size=out.shape).astype(np.float32)
            x64, off64, g64 = [a.astype(np.float64) for a in (x, off, gy)]
            out64 = orc.mex_fwd(x64, off64, n, **kw)
            want_dx = orc.mex_input_grad(x64, off64, out64, g64, n, **kw)
            want_do = orc.mex_offsets_grad(x64, off64, out64, g64, n, **kw)
        # (infinite epsilon: the gradient goes to the elements that equal the output, so the output must be the
        # library's own; it is the oracle's bit for bit, as compare() has just shown where it is finite)
        dx, do = pkg.mex_grads(X, O, got if math.isinf(eps) else dev(out), dev(gy), n, **kw)
        for name, gotg, wantg in (("input gradient", dx, want_dx), ("offsets gradient", do, want_do)):
            fin = np.isfinite(wantg)
            floor = 1e-2 * float(np.abs(wantg[fin]).max()) if fin.any() else 0.0
            compare(gotg.cpu().numpy(), wantg, floor, 2e-4, "%s, %s" % (name, tag))
        ran += 1
    assert ran >= 30
