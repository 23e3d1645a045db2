"""GPU parity of the backward operators: the HIP library (through the C ABI via the op layer) against the
CPU oracle's restatement of the reference grad kernels on the same seeded inputs, to 1e-4.

Gradients are sums of many signed terms and cross zero, so
  * the error of an element is taken relative to max(|want|, 1e-2 * max|want|): element-wise for
    everything above a hundredth of the tensor's scale, relative to that hundredth below it (the
    rounding noise of an fp32 sum is proportional to the magnitude of its terms, not of its value);
  * it is measured against the oracle's fp64 instantiation (the exact value of the sum).  The bar is
    the plain 1e-4 at the benchmark shapes (configuration 5: the config-3, config-2 and config-1
    layer shapes, `strict=True`) and wherever the data are of order one.  Only the stress cases that
    put the data far off centre or make the sums cancel (named where they pass `strict=False`) may
    use 1e-4 or twice the error the reference's own fp32 arithmetic (the oracle's fp32
    instantiation) makes on the same inputs, whichever is larger: where the sum cancels, no fp32
    summation order is closer to another than both are to the exact value.
"""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import config1, config2, config3, rel_err

pytestmark = pytest.mark.gpu

GRAD_TOL = 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def grad_err(got, want):
    want = np.asarray(want)
    scale = float(np.abs(want[np.isfinite(want)]).max()) if np.isfinite(want).any() else 0.0
    return rel_err(got, want, floor=np.full(want.shape, 1e-2 * scale))


def assert_grad_close(got, want32, want64, what, strict=True):
    # The reference's fp32 arithmetic can overflow where the exact value is finite: the empty slots of a ragged
    # offsets region hold zeros, and with offsets near +-100 their terms are 0 * exp(250) = 0 * inf (NaN in fp32, 0 in
    # fp64; include/utils/mex_utils.hpp:33-41 on the zero padding of split_patches).  The library skips empty slots, so
    # its sums are finite there: such elements are judged against fp64 alone.
    overflow = np.isnan(want32) & ~np.isnan(want64)
    if overflow.any():
        print("%s: %d elements where the reference's fp32 arithmetic gives NaN and the exact value is finite"
              % (what, int(overflow.sum())))
        want32 = np.where(overflow, want64, want32).astype(want32.dtype)
    e_gpu, e_ref = grad_err(got, want64), grad_err(want32, want64)
    print("%s: gpu %.3g, fp32 reference %.3g (of max(|want|, 1%% of the scale), against fp64)" % (what, e_gpu, e_ref))
    bar = GRAD_TOL if strict else max(GRAD_TOL, 2.0 * e_ref)
    assert e_gpu <= bar, "%s: gpu %.3g, fp32 reference %.3g, bar %.3g" % (what, e_gpu, e_ref, bar)


def f64(*arrays):
    return [np.asarray(a, dtype=np.float64) for a in arrays]


def sim_grads_gpu(pkg, x, t, w, g, **kw):
    dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(g), **kw)
    dt, dw = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(g), **kw)
    torch.cuda.synchronize()
    return dx.cpu().numpy(), dt.cpu().numpy(), dw.cpu().numpy()


def check_sim_grads(pkg, x, t, w, seed=99, strict=True, **kw):
    out = orc.similarity_fwd(x, t, w, **kw)
    g = np.random.default_rng(seed).normal(size=out.shape).astype(np.float32)
    dx, dt, dw = sim_grads_gpu(pkg, x, t, w, g, **kw)
    want_dx = orc.similarity_input_grad(x, t, w, g, **kw)
    want_dt, want_dw = orc.similarity_params_grad(x, t, w, g, **kw)
    d = f64(x, t, w, g)
    true_dx = orc.similarity_input_grad(*d, **kw)
    true_dt, true_dw = orc.similarity_params_grad(*d, **kw)
    assert_grad_close(dx, want_dx, true_dx, "input grad", strict)
    assert_grad_close(dt, want_dt, true_dt, "templates grad", strict)
    assert_grad_close(dw, want_dw, true_dw, "weights grad", strict)


# ---- the reference's own gradient test matrix (python/simnets/test/__init__.py:55-103, :143-154) ------------
@pytest.mark.parametrize("strides", [[1, 1], [2, 2]])
@pytest.mark.parametrize("blocks", [[1, 1], [3, 3]])
@pytest.mark.parametrize("func,norm,ign", [("L2", True, False), ("L2", True, True), ("L1", False, False),
                                           ("L2", False, False)])
@pytest.mark.parametrize("O", [1, 5])
def test_similarity_grads_reference_matrix(pkg, strides, blocks, func, norm, ign, O):
    g = np.random.default_rng(167)
    x = (16.0 + g.normal(size=(1, 3, 10, 10))).astype(np.float32)
    w = (3.0 + np.abs(g.normal(size=(O, 3) + tuple(blocks)))).astype(np.float32)
    t = (3.0 + g.normal(size=w.shape)).astype(np.float32)
    kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=[0, 0], normalization_term=norm,
              ignore_nan_input=ign)
    check_sim_grads(pkg, x, t, w, **kw)


@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True)])
def test_similarity_params_grad_few_templates_short_patches(pkg, func, norm, ign):
    """Patches of 1 ... 9 elements with as many templates as the lanes-along-pixels kernel takes (4 * (32 // K)), one
    fewer and one more (the tiled kernel), seeded shapes, strides and padding; NaN inputs where they are ignored."""
    rng = np.random.default_rng(77)
    for blocks, C in (([1, 1], 1), ([1, 2], 1), ([1, 1], 3), ([2, 2], 1), ([1, 1], 5), ([2, 3], 1), ([1, 1], 7),
                      ([2, 2], 2), ([3, 3], 1)):
        K = C * blocks[0] * blocks[1]
        for O in (4 * (32 // K) - 1, 4 * (32 // K), 4 * (32 // K) + 1):
            B, H, W = int(rng.integers(1, 9)), int(rng.integers(4, 20)), int(rng.integers(4, 20))
            strides = [int(rng.integers(1, 3)), int(rng.integers(1, 3))]
            padding = [int(rng.integers(0, 3)), int(rng.integers(0, 3))]
            x, t, w = sim_inputs(int(rng.integers(1 << 30)), (B, C, H, W), O, blocks, nan_frac=0.2 if ign else 0.0)
            kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding, normalization_term=norm,
                      ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else 0.5)
            print("case", (B, C, H, W), O, blocks, strides, padding, flush=True)
            check_sim_grads(pkg, x, t, w, **kw)


def sim_inputs(seed, shape, O, blocks, nan_frac=0.0):
    g = np.random.default_rng(seed)
    x = g.normal(size=shape).astype(np.float32)
    t = g.normal(size=(O, shape[1]) + tuple(blocks)).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    if nan_frac:
        x[g.random(size=x.shape) < nan_frac] = np.nan
    return x, t, w


@pytest.mark.parametrize("func", ["L2", "L1"])
@pytest.mark.parametrize("case", [
    dict(shape=(2, 3, 20, 21), O=7, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),
    dict(shape=(2, 3, 20, 21), O=7, blocks=[3, 3], strides=[2, 2], padding=[1, 1]),       # phases with 1 and 2 taps
    dict(shape=(2, 3, 50, 31), O=7, blocks=[3, 2], strides=[1, 2], padding=[0, 1]),
    dict(shape=(1, 2, 9, 70), O=33, blocks=[5, 5], strides=[3, 3], padding=[2, 2]),
    dict(shape=(2, 2, 11, 13), O=3, blocks=[2, 2], strides=[3, 4], padding=[0, 1]),       # stride > block: uncovered pixels
    dict(shape=(2, 1, 28, 28), O=3, blocks=[28, 28], strides=[1, 1], padding=[0, 0]),     # one output pixel
    dict(shape=(3, 4, 12, 200), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),     # wide rows
    dict(shape=(1, 130, 6, 6), O=17, blocks=[2, 2], strides=[1, 1], padding=[1, 1]),      # many channels
    dict(shape=(2, 40, 34, 34), O=130, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),    # big lane tile, ragged O
    dict(shape=(2, 2, 5, 5), O=2, blocks=[2, 2], strides=[4, 5], padding=[3, 3]),         # padding beyond the block
    dict(shape=(1, 1, 7, 7), O=1, blocks=[2, 2], strides=[2, 2], padding=[0, 0]),         # last row/column never covered
    dict(shape=(1, 2, 6, 700), O=4, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),       # rows too wide for the LDS tile
])
def test_similarity_grads_geometries(pkg, case, func):
    x, t, w = sim_inputs(5, case["shape"], case["O"], case["blocks"])
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              out_of_bounds_value=0.25)
    check_sim_grads(pkg, x, t, w, **kw)


@pytest.mark.parametrize("nan_frac", [0.0, 0.25, 1.0])
@pytest.mark.parametrize("blocks,strides,padding", [([2, 2], [2, 2], [2, 2]), ([3, 3], [1, 1], [1, 1]),
                                                    ([3, 3], [2, 1], [1, 0])])
def test_similarity_grads_ignore_nan(pkg, nan_frac, blocks, strides, padding):
    x, t, w = sim_inputs(6, (3, 2, 14, 15), 6, blocks, nan_frac=nan_frac)
    kw = dict(similarity_function="L2", blocks=blocks, strides=strides, padding=padding, normalization_term=True,
              ignore_nan_input=True, out_of_bounds_value=float("nan"))
    check_sim_grads(pkg, x, t, w, **kw)


@pytest.mark.parametrize("algo", [None, "direct"])
@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True)])
@pytest.mark.parametrize("offset,spread", [(0.0, 1.0), (40.0, 1.0), (-7.0, 0.01), (3.0, 30.0)])
def test_similarity_params_grad_moment_and_term_by_term_forms(pkg, algo, func, norm, ign, offset, spread):
    """The L2 modes' parameter gradients by default combine moments about a centre near the templates; with
    algo='direct' they sum the reference's terms.  Both forms stay within the bar when the data sit far from zero
    (offset), when patches and templates nearly coincide (tiny spread) and when the templates lie far apart."""
    g = np.random.default_rng(31)
    x = (offset + g.normal(size=(3, 5, 14, 15))).astype(np.float32)
    t = (offset + spread * g.normal(size=(11, 5, 3, 3))).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    if ign:
        x[g.random(size=x.shape) < 0.2] = np.nan
    kw = dict(similarity_function=func, blocks=[3, 3], strides=[1, 1], padding=[1, 1], normalization_term=norm,
              ignore_nan_input=ign, out_of_bounds_value=offset)
    out = orc.similarity_fwd(x, t, w, **kw)
    og = g.normal(size=out.shape).astype(np.float32)
    dt, dw = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(og), algo=algo, **kw)
    want_dt, want_dw = orc.similarity_params_grad(x, t, w, og, **kw)
    true_dt, true_dw = orc.similarity_params_grad(*f64(x, t, w, og), **kw)
    assert_grad_close(dt.cpu().numpy(), want_dt, true_dt, "templates grad")
    assert_grad_close(dw.cpu().numpy(), want_dw, true_dw, "weights grad")


def test_similarity_params_grad_nan_template_stays_in_its_own_row(pkg):
    """A non-finite template poisons its own gradients only (the centre of the moment form ignores it)."""
    x, t, w = sim_inputs(8, (2, 3, 9, 9), 5, (2, 2))
    t[2, 1, 0, 1] = np.nan
    kw = dict(similarity_function="L2", blocks=[2, 2], strides=[1, 1], padding=[0, 0])
    out = orc.similarity_fwd(x, t, w, **kw)
    og = np.random.default_rng(3).normal(size=out.shape).astype(np.float32)
    dt, dw = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(og), **kw)
    want_dt, want_dw = orc.similarity_params_grad(x, t, w, og, **kw)
    for got, want in ((dt.cpu().numpy(), want_dt), (dw.cpu().numpy(), want_dw)):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert rel_err(got[ok], want[ok], floor=np.full(want[ok].shape, 1e-2 * np.abs(want[ok]).max())) <= GRAD_TOL


@pytest.mark.parametrize("algo", [None, "direct"])
def test_similarity_params_grad_infinite_input_like_the_reference(pkg, algo):
    """An infinite input element gives the parameter gradients of its patch element the reference's infinities and
    NaNs (g (x - t) = +-inf, sums of both signs = NaN), in both forms of the sums."""
    x, t, w = sim_inputs(9, (2, 2, 6, 6), 4, (2, 2))
    x[1, 0, 2, 3] = np.inf
    kw = dict(similarity_function="L2", blocks=[2, 2], strides=[2, 2], padding=[0, 0])
    out = orc.similarity_fwd(x, t, w, **kw)
    og = np.abs(np.random.default_rng(4).normal(size=out.shape)).astype(np.float32)   # one sign: the sums stay +-inf
    dt, dw = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(og), algo=algo, **kw)
    with np.errstate(invalid="ignore", over="ignore"):
        want_dt, want_dw = orc.similarity_params_grad(x, t, w, og, **kw)
    for got, want in ((dt.cpu().numpy(), want_dt), (dw.cpu().numpy(), want_dw)):
        assert np.isinf(want).any()
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[np.isinf(want)], want[np.isinf(want)])
        ok = np.isfinite(want)
        assert rel_err(got[ok], want[ok], floor=np.full(want[ok].shape, 1e-2 * np.abs(want[ok]).max())) <= GRAD_TOL


def test_similarity_grads_nan_input_without_ignore_propagates_like_the_reference(pkg):
    x, t, w = sim_inputs(7, (1, 2, 8, 8), 3, (3, 3))
    x[0, 1, 4, 4] = np.nan
    check_sim_grads(pkg, x, t, w, similarity_function="L2", blocks=[3, 3], strides=[1, 1], padding=[1, 1])


def test_similarity_grads_first_layer_of_the_missing_data_network(pkg):
    x, t, w, kw = config1(batch=8, nan_frac=0.25)
    check_sim_grads(pkg, x, t, w, strict=True, **kw)


@pytest.mark.parametrize("func", ["L2", "L1"])
def test_similarity_grads_conv_scale_shape_small_batch(pkg, func):
    x, t, w, kw = config3(batch=3)
    check_sim_grads(pkg, x, t, w, similarity_function=func, strict=True, **kw)


def oracle_params_grad_over_batch(x, t, w, g, kw, dtype, threads=8):
    """Parameter gradients of the oracle summed over a large batch.  fp32: one call, images accumulated one after
    the other like the reference's batch loop.  fp64 (the exact value, for which the order does not matter at the
    tolerances used here): the batch split over threads, partial sums added at the end."""
    from concurrent.futures import ThreadPoolExecutor
    if dtype == np.float32:
        return orc.similarity_params_grad(x, t, w, g, **kw)
    t64, w64 = f64(t, w)
    chunks = np.array_split(np.arange(len(x)), threads)
    with ThreadPoolExecutor(threads) as ex:
        parts = list(ex.map(lambda c: orc.similarity_params_grad(x[c].astype(np.float64), t64, w64,
                                                                 g[c].astype(np.float64), **kw), chunks))
    return sum(p[0] for p in parts), sum(p[1] for p in parts)


@pytest.mark.parametrize("func", ["L2", "L1"])
def test_similarity_grads_conv_scale_full_batch_against_the_oracle(pkg, func, record_property):
    """Full config-3 batch (256 images).  Input gradient: per-image oracle on a sample of images.  Parameter gradients:
    a template's gradient depends on that template's parameters and output-gradient channel only, so the oracle over
    all 256 images for a subset of the 128 templates pins those rows of the full call - for the default forms
    (moments on the matrix cores / scaled sign) and for algo='direct' (the reference's terms one by one), which must
    meet the plain 1e-4 bar.  Properties over everything: linearity in the output gradient (exact for a factor 2)."""
    x, t, w, kw = config3()
    kw = dict(kw, similarity_function=func)
    g = np.random.default_rng(6789).normal(size=(256, 128, 32, 32)).astype(np.float32)
    X, T, W, G = dev(x), dev(t), dev(w), dev(g)
    dx = pkg.similarity_input_grad(X, T, W, G, **kw)
    for b in (0, 131, 255):
        want = orc.similarity_input_grad(x[b:b + 1], t, w, g[b:b + 1], **kw)
        true = orc.similarity_input_grad(*f64(x[b:b + 1], t, w, g[b:b + 1]), **kw)
        assert_grad_close(dx[b:b + 1].cpu().numpy(), want, true, "input grad of image %d" % b, strict=True)
    idx = [0, 1, 37, 63, 64, 100, 126, 127]
    gs = np.ascontiguousarray(g[:, idx])
    ref_dt, ref_dw = oracle_params_grad_over_batch(x, t[idx], w[idx], gs, kw, np.float32)
    true_dt, true_dw = oracle_params_grad_over_batch(x, t[idx], w[idx], gs, kw, np.float64)
    e_ref = (grad_err(ref_dt, true_dt), grad_err(ref_dw, true_dw))
    for algo in (None, "direct"):
        dt, dw = pkg.similarity_parameters_grad(X, T, W, G, algo=algo, **kw)
        e = (grad_err(dt.cpu().numpy()[idx], true_dt), grad_err(dw.cpu().numpy()[idx], true_dw))
        print("config-3 %s parameter gradients, 256 images, algo=%s: templates %.3g, weights %.3g of the scale "
              "(fp32 oracle: %.3g, %.3g)" % (func, algo, e[0], e[1], e_ref[0], e_ref[1]))
        record_property("params_grad_err_%s_%s" % (func, algo), e)
        assert max(e) <= GRAD_TOL, (algo, e, e_ref)        # the plain bar, default forms included
        dt3, dw3 = pkg.similarity_parameters_grad(X, T, W, 2.0 * G, algo=algo, **kw)
        assert torch.equal(dt3, 2.0 * dt) and torch.equal(dw3, 2.0 * dw)      # scaling by 2 is exact in fp32


def test_similarity_params_grad_is_reproducible(pkg):
    x, t, w, kw = config3(batch=16)
    g = np.random.default_rng(1).normal(size=(16, 128, 32, 32)).astype(np.float32)
    a = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(g), **kw)
    b = pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(g), **kw)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_similarity_grads_empty_batch(pkg):
    x, t, w = sim_inputs(8, (0, 3, 9, 9), 4, (3, 3))
    g = np.zeros((0, 4, 7, 7), np.float32)
    dx, dt, dw = sim_grads_gpu(pkg, x, t, w, g, blocks=[3, 3], strides=[1, 1], padding=[0, 0])
    assert dx.shape == x.shape and not dt.any() and not dw.any()


def test_similarity_grads_reject_wrong_output_grad_shape(pkg):
    x, t, w = sim_inputs(9, (1, 3, 9, 9), 4, (3, 3))
    with pytest.raises(pkg.SimnetsError):
        pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(np.zeros((1, 4, 9, 9), np.float32)), blocks=[3, 3],
                                  strides=[1, 1], padding=[0, 0])


# ---- MEX ------------------------------------------------------------------------------------------
def mex_case(seed, im_dims, num_instances, **kw):
    g = np.random.default_rng(seed)
    d = orc.mex_dims(orc.mex_args(im_dims, num_instances, **kw))
    x = g.normal(size=im_dims).astype(np.float32)
    off = g.normal(size=(d.num_regions, num_instances) + tuple(kw["blocks"])).astype(np.float32)
    return x, off


def check_mex_grads(pkg, x, off, n, seed=77, strict=True, **kw):
    out = orc.mex_fwd(x, off, n, **kw)
    g = np.random.default_rng(seed).normal(size=out.shape).astype(np.float32)
    X, O, Y, G = dev(x), dev(off), dev(out), dev(g)
    dx = pkg.mex_input_grad(X, O, Y, G, n, **kw).cpu().numpy()
    doff = pkg.mex_offsets_grad(X, O, Y, G, n, **kw).cpu().numpy()
    x64, off64, g64 = f64(x, off, g)
    out64 = orc.mex_fwd(x64, off64, n, **kw)
    assert_grad_close(dx, orc.mex_input_grad(x, off, out, g, n, **kw), orc.mex_input_grad(x64, off64, out64, g64, n, **kw),
                      "input grad", strict)
    assert_grad_close(doff, orc.mex_offsets_grad(x, off, out, g, n, **kw),
                      orc.mex_offsets_grad(x64, off64, out64, g64, n, **kw), "offsets grad", strict)


# the reference's gradient tests (python/simnets/test/__init__.py:329-372)
@pytest.mark.parametrize("unshared", [True, False])
@pytest.mark.parametrize("shared_spec", [[1, 5, 4], [2], [-1]])
@pytest.mark.parametrize("unshared_spec", [[1, 5, 4], [2], [-1]])
def test_mex_grads_reference_matrix(pkg, unshared, shared_spec, unshared_spec):
    kw = dict(blocks=[3, 3, 1], strides=[1, 1, 2], padding=[0, 1, 0], softmax_mode=True, use_unshared_regions=unshared,
              shared_offset_region=shared_spec, unshared_offset_region=unshared_spec)
    x, off = mex_case(11, (2, 3, 12, 13), 2, **kw)
    check_mex_grads(pkg, x, off, 2, **kw)


def test_mex_grads_reference_blocks_bug_case(pkg):
    kw = dict(blocks=[3, 8, 8], strides=[1, 1, 2], padding=[0, 4, 4], softmax_mode=True, use_unshared_regions=True,
              shared_offset_region=[3, 3, 3], unshared_offset_region=[2])
    x, off = mex_case(12, (2, 3, 16, 16), 2, **kw)
    check_mex_grads(pkg, x, off, 2, **kw)


@pytest.mark.parametrize("eps", [1.0, -1.0, 2.5, -0.3, math.inf, -math.inf])
@pytest.mark.parametrize("softmax", [True, False])
def test_mex_grads_epsilon(pkg, eps, softmax):
    kw = dict(blocks=[2, 3, 3], strides=[1, 2, 2], padding=[0, 1, 1], epsilon=eps, softmax_mode=softmax,
              shared_offset_region=[1, 2, 3], use_unshared_regions=False)
    x, off = mex_case(13, (3, 5, 11, 10), 5, **kw)
    check_mex_grads(pkg, x, off, 5, **kw)


@pytest.mark.parametrize("case", [
    dict(im=(2, 6, 9, 9), n=20, kw=dict(blocks=[6, 1, 1], strides=[6, 1, 1], padding=[0, 0, 0], unshared_offset_region=[2])),
    dict(im=(3, 4, 7, 6), n=3, kw=dict(blocks=[2, 2, 2], strides=[2, 2, 2], padding=[0, 0, 0], use_unshared_regions=False,
                                      shared_offset_region=[-1])),                       # one region, ragged tiling
    dict(im=(2, 3, 6, 6), n=2, kw=dict(blocks=[2, 3, 2], strides=[1, 2, 2], padding=[1, 1, 0], blocks_round_down=False,
                                      blocks_out_of_bounds_value=-0.7, use_unshared_regions=False,
                                      shared_offset_region=[1, 2, 2])),                  # channel padding, round up
    dict(im=(2, 3, 5, 5), n=2, kw=dict(blocks=[3, 1, 1], strides=[3, 1, 1], padding=[0, 0, 0])),   # one region per pixel
    dict(im=(130, 70, 2, 2), n=9, kw=dict(blocks=[70, 1, 1], strides=[70, 1, 1], padding=[0, 0, 0],
                                        unshared_offset_region=[2])),                   # long K, many images
    dict(im=(2, 8, 8, 8), n=4, kw=dict(blocks=[1, 2, 2], strides=[1, 3, 3], padding=[0, 0, 0], use_unshared_regions=False,
                                      shared_offset_region=[2])),                        # stride > block: uncovered input
])
def test_mex_grads_geometries(pkg, case):
    x, off = mex_case(14, case["im"], case["n"], **case["kw"])
    check_mex_grads(pkg, x, off, case["n"], **case["kw"])


@pytest.mark.parametrize("spread", ["narrow", "wide", "mixed"])
@pytest.mark.parametrize("eps", [1.0, -2.0, 5.0, 12.0])
@pytest.mark.parametrize("geom", [
    dict(im=(5, 40, 6, 6), n=70, kw=dict(blocks=[40, 1, 1], strides=[40, 1, 1], padding=[0, 0, 0],
                                         unshared_offset_region=[2])),                  # several instance groups
    dict(im=(3, 6, 12, 12), n=10, kw=dict(blocks=[3, 3, 3], strides=[2, 1, 1], padding=[1, 1, 1],
                                          use_unshared_regions=False, shared_offset_region=[2])),   # overlapping patches
])
def test_mex_grads_offset_ranges_product_and_term_by_term_forms(pkg, geom, spread, eps):
    # finite epsilon: regions whose offsets span a small range run the product form on the matrix cores, wide ranges
    # the term-by-term waves; regions of one launch may differ
    g = np.random.default_rng(81)
    kw = dict(geom["kw"], epsilon=eps, softmax_mode=False)
    x, off = mex_case(15, geom["im"], geom["n"], **kw)
    x = x * 4
    off = off * 0.3
    if spread == "wide":
        off *= 300
    elif spread == "mixed":
        off[::2] *= 300
    # Stress case that needs the allowance (strict=False): inputs spanning +-16 and offsets spanning up to +-300,
    # times epsilon up to 12, put exponents of several hundred next to each other; the forward output the gradients
    # are formed from is then known to about 1e-5 of such an exponent, and the reference's own fp32 arithmetic is
    # 2e-4 ... 3e-3 away from the exact gradient here (the GPU's error equals it to two digits).
    check_mex_grads(pkg, x, off, geom["n"], strict=False, **kw)


@pytest.mark.parametrize("eps", [2.0, -math.inf])
def test_mex_input_grad_of_overlapping_patches_is_reproducible(pkg, eps):
    """Overlapping patches: the per-patch gradients are added per input element in a fixed order (no atomics), so
    two calls agree bit for bit; the sum over patches matches the oracle's col2im."""
    kw = dict(blocks=[3, 3, 3], strides=[1, 2, 1], padding=[1, 0, 2], epsilon=eps, softmax_mode=True,
              use_unshared_regions=False, shared_offset_region=[2, 3, 1], blocks_out_of_bounds_value=0.5)
    x, off = mex_case(23, (4, 7, 11, 9), 9, **kw)
    out = orc.mex_fwd(x, off, 9, **kw)
    go = np.random.default_rng(5).normal(size=out.shape).astype(np.float32)
    runs = [pkg.mex_input_grad(dev(x), dev(off), dev(out), dev(go), 9, **kw).cpu().numpy() for _ in range(3)]
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    want = orc.mex_input_grad(x, off, out, go, 9, **kw)
    assert rel_err(runs[0], want, floor=np.full(want.shape, 1e-2 * np.abs(want).max())) <= GRAD_TOL


def test_mex_grads_config2_shape(pkg):
    x, off, n, kw = config2(batch=64)
    off = orc.normalize_offsets(off)
    check_mex_grads(pkg, x, off, n, strict=True, **kw)


def test_mex_offsets_grad_through_the_offset_normalisation(pkg):
    """normalize_offsets=True returns d/d(raw offsets): G - softmax(raw) * sum_k G, with G the gradient the
    reference op would return for the normalised offsets."""
    x, off, n, kw = config2(batch=4, channels=16, size=6, instances=8)
    norm = orc.normalize_offsets(off)
    out = orc.mex_fwd(x, norm, n, **kw)
    g = np.random.default_rng(3).normal(size=out.shape).astype(np.float32)
    G = orc.mex_offsets_grad(x.astype(np.float64), norm.astype(np.float64), out.astype(np.float64),
                             g.astype(np.float64), n, **kw)
    want = G - np.exp(norm.astype(np.float64)) * G.sum(axis=(2, 3, 4), keepdims=True)
    got = pkg.mex_offsets_grad(dev(x), dev(off), dev(out), dev(g), n, normalize_offsets=True, **kw).cpu().numpy()
    assert grad_err(got, want) <= GRAD_TOL
    got_dx = pkg.mex_input_grad(dev(x), dev(off), dev(out), dev(g), n, normalize_offsets=True, **kw).cpu().numpy()
    assert grad_err(got_dx, orc.mex_input_grad(x, norm, out, g, n, **kw)) <= GRAD_TOL


@pytest.mark.parametrize("shape,blocks,n,shared", [
    ((3, 5, 16, 16), [5, 16, 16], 3, None),        # rows of 1280 elements: two launches
    ((6, 4, 16, 16), [4, 16, 16], 5, None),        # rows of 1024: one launch
    ((40, 3, 6, 6), [3, 2, 2], 7, [-1])])          # one region of 360 pixel slots: several pixel chunks
@pytest.mark.parametrize("normalize", [False, True])
def test_mex_offsets_grad_sum_over_pixel_chunks_and_chain_rule(pkg, shape, blocks, n, shared, normalize):
    """The offsets gradient's last step - partial sums of the pixel chunks added up, then the chain rule through
    the normalisation - runs as one launch for rows of at most 1024 elements and as two for longer ones."""
    g_ = np.random.default_rng(21)
    x = g_.normal(size=shape).astype(np.float32)
    kw = dict(blocks=blocks, strides=blocks, epsilon=1.0, softmax_mode=True)
    if shared is not None:
        kw.update(use_unshared_regions=False, shared_offset_region=shared)
    off = (0.3 * g_.normal(size=(1, n) + tuple(blocks))).astype(np.float32)
    used = orc.normalize_offsets(off) if normalize else off
    out = orc.mex_fwd(x, used, n, **kw)
    g = g_.normal(size=out.shape).astype(np.float32)
    G = orc.mex_offsets_grad(x.astype(np.float64), used.astype(np.float64), out.astype(np.float64),
                             g.astype(np.float64), n, **kw)
    want = G - np.exp(used.astype(np.float64)) * G.sum(axis=(2, 3, 4), keepdims=True) if normalize else G
    got = pkg.mex_offsets_grad(dev(x), dev(off), dev(out), dev(g), n, normalize_offsets=normalize, **kw)
    assert grad_err(got.cpu().numpy(), want) <= GRAD_TOL
    both = pkg.mex_grads(dev(x), dev(off), dev(out), dev(g), n, normalize_offsets=normalize, **kw)
    assert np.array_equal(both[1].cpu().numpy().view(np.uint32), got.cpu().numpy().view(np.uint32))


def test_mex_offsets_grad_is_reproducible_and_additive(pkg):
    x, off, n, kw = config2(batch=64)
    off = orc.normalize_offsets(off)
    X, O = dev(x), dev(off)
    Y = pkg.mex(X, O, n, **kw)
    G = dev(np.random.default_rng(4).normal(size=tuple(Y.shape)).astype(np.float32))
    a = pkg.mex_offsets_grad(X, O, Y, G, n, **kw)
    b = pkg.mex_offsets_grad(X, O, Y, G, n, **kw)
    assert torch.equal(a, b)
    halves = pkg.mex_offsets_grad(X[:32], O, Y[:32], G[:32], n, **kw) + pkg.mex_offsets_grad(X[32:], O, Y[32:], G[32:],
                                                                                          n, **kw)
    assert grad_err(halves.cpu().numpy(), a.cpu().numpy()) <= GRAD_TOL
    # softmax-mode, eps=1: the terms exp(x + off - out) of a pixel sum to 1 over k, so dX summed over the
    # patch equals the output gradient summed over the instances
    dx = pkg.mex_input_grad(X, O, Y, G, n, **kw)
    assert grad_err(dx.sum(dim=1).cpu().numpy(), G.sum(dim=1).cpu().numpy()) <= GRAD_TOL


def test_mex_grads_empty_batch(pkg):
    kw = dict(blocks=[3, 1, 1], strides=[3, 1, 1], padding=[0, 0, 0], use_unshared_regions=False)
    off = np.zeros((1, 2, 3, 1, 1), np.float32)
    x = np.zeros((0, 3, 4, 4), np.float32)
    y = np.zeros((0, 2, 4, 4), np.float32)
    assert pkg.mex_input_grad(dev(x), dev(off), dev(y), dev(y), 2, **kw).shape == x.shape
    assert not pkg.mex_offsets_grad(dev(x), dev(off), dev(y), dev(y), 2, **kw).cpu().numpy().any()


def test_similarity_l1_grads_at_ties_and_nan(pkg):
    """sign(0) = sign(NaN) = 0 in the reference's L1 functors (similarity_utils.hpp:82-84, :121-125): inputs that
    equal a template entry exactly, NaN inputs and zero weights."""
    x, t, w = sim_inputs(21, (2, 2, 9, 9), 3, (3, 3))
    t[0, 0, 1, 1] = x[0, 0, 4, 4]          # the centre tap of template 0 meets this pixel exactly
    x[1, 1, :, 3] = t[1, 1, 0, 0]          # a whole column equal to one template entry
    x[0, 1, 2, 2] = np.nan
    w[2, 0, 2, 2] = 0.0
    check_sim_grads(pkg, x, t, w, similarity_function="L1", blocks=[3, 3], strides=[1, 1], padding=[1, 1])


@pytest.mark.parametrize("nan", [False, True])
def test_similarity_l1_params_grad_scaled_sign_form_equals_the_term_by_term_form(pkg, nan):
    """L1 parameter gradients by default take sign and magnitude from 2^64 (x - t) (fma, med3); with algo='direct'
    they use compares and selects.  Same sums in the same order: bit-identical, ties and zero weights included;
    pixel chunks with a NaN input run the compare-and-select arithmetic in both."""
    x, t, w = sim_inputs(22, (3, 5, 17, 19), 37, (3, 3))
    t[0, 0, 1, 1] = x[0, 0, 4, 4]
    x[1, 1, :, 3] = t[1, 1, 0, 0]
    x[2, 3, 5:9, 2:11] = 0.0
    w[2, 0, 2, 2] = 0.0
    if nan:
        x[0, 1, 2, 2] = np.nan
        x[2, 4, 16, 18] = np.nan
    kw = dict(similarity_function="L1", blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    out = orc.similarity_fwd(x, t, w, **kw)
    og = np.random.default_rng(8).normal(size=out.shape).astype(np.float32)
    fast = [a.cpu().numpy() for a in pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(og), **kw)]
    exact = [a.cpu().numpy() for a in pkg.similarity_parameters_grad(dev(x), dev(t), dev(w), dev(og), algo="direct", **kw)]
    assert np.array_equal(fast[0], exact[0], equal_nan=True)
    assert np.array_equal(fast[1], exact[1], equal_nan=True)
    want_dt, want_dw = orc.similarity_params_grad(x, t, w, og, **kw)
    assert np.array_equal(np.isnan(fast[0]), np.isnan(want_dt)) and np.array_equal(np.isnan(fast[1]), np.isnan(want_dw))
    true_dt, true_dw = orc.similarity_params_grad(*f64(x, t, w, og), **kw)
    ok = ~np.isnan(want_dw)
    assert_grad_close(fast[0], want_dt, true_dt, "templates grad")
    assert_grad_close(np.where(ok, fast[1], 0), np.where(ok, want_dw, 0), np.where(ok, true_dw, 0), "weights grad")


@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True)])
@pytest.mark.parametrize("case", [
    dict(shape=(3, 5, 9, 32), O=70, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),     # ow = 32, ragged O and K
    dict(shape=(2, 3, 12, 64), O=9, blocks=[3, 3], strides=[2, 2], padding=[1, 1]),     # ow = 32 through stride 2
    dict(shape=(1, 16, 6, 66), O=130, blocks=[2, 3], strides=[1, 1], padding=[0, 0]),   # ow = 64, two chunks per row
    dict(shape=(2, 2, 5, 30), O=4, blocks=[1, 5], strides=[1, 1], padding=[0, 3]),      # ow = 32 with padding beyond the image
])
def test_similarity_params_grad_row_staged_matrix_form(pkg, case, func, norm, ign):
    """Output widths that are multiples of 32: the L2 parameter gradients stage g and the patch elements row by
    row for the matrix-core moments."""
    x, t, w = sim_inputs(41, case["shape"], case["O"], case["blocks"], nan_frac=0.15 if ign else 0.0)
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              normalization_term=norm, ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else -0.75)
    out = orc.similarity_fwd(x, t, w, **kw)
    assert out.shape[3] % 32 == 0
    check_sim_grads(pkg, x, t, w, **kw)


@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True)])
@pytest.mark.parametrize("case", [
    dict(shape=(2, 40, 13, 17), O=9, blocks=[3, 3], padding=[1, 1]),       # ragged channel tile, odd template count
    dict(shape=(1, 70, 9, 40), O=33, blocks=[2, 4], padding=[0, 3]),       # two channel tiles, asymmetric block
    dict(shape=(3, 24, 20, 20), O=16, blocks=[5, 5], padding=[4, 0]),      # padding = block - 1
    dict(shape=(2, 32, 6, 300), O=12, blocks=[1, 3], padding=[0, 1]),      # several pixel tiles per row
    dict(shape=(2, 24, 14, 15), O=10, blocks=[3, 3], padding=[1, 1], strides=[2, 2]),   # four phases: 4, 2, 2, 1 taps
    dict(shape=(1, 40, 23, 22), O=9, blocks=[7, 7], padding=[3, 3], strides=[2, 2]),    # 16, 12, 12, 9 taps
    dict(shape=(2, 26, 12, 17), O=8, blocks=[3, 2], padding=[2, 0], strides=[2, 1]),    # a phase starting past the padding
    dict(shape=(1, 30, 11, 20), O=11, blocks=[3, 4], padding=[0, 2], strides=[3, 2]),   # leftover rows no window covers
    dict(shape=(2, 24, 9, 9), O=8, blocks=[2, 2], padding=[0, 0], strides=[2, 2]),      # disjoint windows, one tap a phase
    dict(shape=(3, 64, 37, 41), O=19, blocks=[3, 3], padding=[1, 1], strides=[2, 2]),   # several position tiles, odd O
    dict(shape=(1, 25, 8, 70), O=12, blocks=[1, 4], padding=[0, 1], strides=[1, 2]),    # two phases along the width
    dict(shape=(1, 33, 19, 16), O=8, blocks=[3, 3], padding=[1, 1], strides=[3, 3]),    # nine phases, one launch grid each
    dict(shape=(7, 48, 7, 7), O=100, blocks=[3, 3], padding=[1, 1]),      # 5 + 2 images per workgroup, contraction split
    dict(shape=(3, 30, 5, 9), O=64, blocks=[2, 3], padding=[1, 2]),       # 45 pixels: one group of 3 images
    dict(shape=(1, 64, 20, 20), O=300, blocks=[3, 3], padding=[1, 1]),    # two pixel tiles, contraction split 11 ways
    dict(shape=(6, 24, 9, 10), O=90, blocks=[3, 3], padding=[1, 1], strides=[3, 3]),    # small phase grids, split
    dict(shape=(2, 24, 10, 11), O=300, blocks=[3, 3], padding=[1, 1], strides=[2, 2]),  # interleaved phases, split
    dict(shape=(1, 32, 12, 40), O=260, blocks=[2, 4], padding=[1, 0], strides=[1, 2]),  # two phases, split
])
def test_similarity_input_grad_matrix_form(pkg, case, func, norm, ign):
    """At least 24 channels, strides no larger than the window: the L2 modes' input gradient is A - (x - c) B with
    both products on the matrix cores.  Two or four stride phases share a workgroup's tile of the output gradient;
    other strides run one grid per phase.  Data sit away from zero (the centre c matters); algo='direct' takes the
    term-by-term kernel."""
    g = np.random.default_rng(52)
    x = (3.0 + g.normal(size=case["shape"])).astype(np.float32)
    t = (3.0 + g.normal(size=(case["O"], case["shape"][1]) + tuple(case["blocks"]))).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    if ign:
        x[g.random(size=x.shape) < 0.15] = np.nan
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case.get("strides", [1, 1]),
              padding=case["padding"], normalization_term=norm, ignore_nan_input=ign,
              out_of_bounds_value=float("nan") if ign else 1.5)
    out = orc.similarity_fwd(x, t, w, **kw)
    og = g.normal(size=out.shape).astype(np.float32)
    want = orc.similarity_input_grad(x, t, w, og, **kw)
    true = orc.similarity_input_grad(*f64(x, t, w, og), **kw)
    for algo in (None, "direct"):
        dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(og), algo=algo, **kw).cpu().numpy()
        assert np.array_equal(np.isnan(dx), np.isnan(want))
        assert_grad_close(np.nan_to_num(dx), np.nan_to_num(want), np.nan_to_num(true), "input grad (%s)" % algo)


@pytest.mark.parametrize("spread", ["narrow", "mixed"])
@pytest.mark.parametrize("eps", [1.0, -2.0])
def test_mex_grads_many_instances_and_patch_elements_on_a_small_map(pkg, eps, spread):
    """200 instances x 200 patch elements on 4x4 maps: the matrix kernels take the pixel factors and patch
    exponentials from the buffers of the factors kernel (formed once per pixel instead of once per tile of the other
    dimension), the input gradient splits the instance groups over workgroups; slot, instance and element counts are
    no multiples of the tile sizes.  'mixed': every other region has a wide offsets range and runs term by term."""
    kw = dict(blocks=[200, 1, 1], strides=[200, 1, 1], padding=[0, 0, 0], unshared_offset_region=[2], epsilon=eps,
              softmax_mode=True)
    x, off = mex_case(61, (6, 200, 4, 4), 200, **kw)
    off = off * 0.3
    if spread == "mixed":
        off[::2] *= 300
    # 'mixed' is a stress case that needs the allowance (offsets spanning +-300: the fp32 reference itself is more
    # than 1e-4 from the exact gradient); the narrow case meets the plain bar
    check_mex_grads(pkg, x, off, 200, strict=spread != "mixed", **kw)


@pytest.mark.parametrize("spread", ["narrow", "roomy", "mixed"])
@pytest.mark.parametrize("im,n", [
    ((3, 32, 16, 16), 64),     # a 256-pixel chunk is one image
    ((5, 40, 8, 8), 70),       # four images a chunk; ragged instance and channel blocks; the last chunk is part empty
    ((9, 16, 4, 4), 33),       # sixteen images a chunk
    ((3, 12, 2, 8), 5),        # two rows
    ((2, 8, 32, 64), 6),       # eight chunks an image, four rows each
    ((1, 5, 8, 128), 3),       # widest map the row-wise kernel takes: two rows a chunk
    ((6, 24, 4, 4), 140),      # few pixels, five instance groups: the input gradient splits them over workgroups
    ((2, 4, 4, 256), 3),       # wider: the gathering factors kernel
    ((70, 24, 2, 2), 40),      # width 2: below the row-wise kernels' widths (their 16-byte pieces would be one per image)
    ((5, 8, 8, 2), 6),
])
def test_mex_grads_row_wise_factors_on_power_of_two_maps(pkg, im, n, spread):
    """2 x 2 unshared offsets over whole-channel patches on maps with power-of-two sides: the pixel factors and patch
    exponentials are formed from whole rows (16-byte loads along the rows, regions interleaved through LDS) and both
    matrix kernels read them back.  'roomy': offsets ranges beyond the few-instances bound, 'mixed': every other
    region beyond the product form's range (term by term there).  Also through views that are not 16-byte aligned,
    which take the gathering kernel: same results to the same bar."""
    kw = dict(blocks=[im[1], 1, 1], strides=[im[1], 1, 1], padding=[0, 0, 0], unshared_offset_region=[2], epsilon=1.5,
              softmax_mode=False)
    x, off = mex_case(71, im, n, **kw)
    off = off * {"narrow": 0.5, "roomy": 4.0, "mixed": 0.3}[spread]
    if spread == "mixed":
        off[::2] *= 300
    check_mex_grads(pkg, x, off, n, strict=spread != "mixed", **kw)
    # unaligned views of the same tensors
    out = orc.mex_fwd(x, off, n, **kw)
    g = np.random.default_rng(3).normal(size=out.shape).astype(np.float32)

    def shifted(a):
        buf = torch.empty(a.size + 1, device="cuda", dtype=torch.float32)
        v = buf[1:].view(a.shape)
        v.copy_(torch.from_numpy(a))
        return v

    X, O, Y, G = dev(x), dev(off), dev(out), dev(g)
    dx, doff = pkg.mex_grads(X, O, Y, G, n, **kw)
    dx_u, doff_u = pkg.mex_grads(shifted(x), O, shifted(out), shifted(g), n, **kw)
    scale_x, scale_o = float(dx.abs().max()), float(doff.abs().max())
    assert float((dx - dx_u).abs().max()) <= 1e-4 * scale_x
    assert float((doff - doff_u).abs().max()) <= 1e-4 * scale_o


def test_mex_grads_row_wise_kernels_random_geometries(pkg):
    """Seeded sweep over the row-wise kernels' domain (power-of-two maps of width 4 ... 64, any batch, channel and
    instance counts): both gradients against the oracle, and from the pooled gradient bit for bit what the expanded
    gradient gives."""
    rng = np.random.default_rng(2024)
    for _ in range(24):
        H, W = 1 << int(rng.integers(1, 5)), 1 << int(rng.integers(2, 7))
        B = int(rng.integers(1, max(2, min(40, 4096 // (H * W)) + 1)))
        C, n = int(rng.integers(1, 72)), int(rng.integers(1, 80))
        eps = float(rng.choice([1.0, -1.5, 3.0]))
        kw = dict(blocks=[C, 1, 1], strides=[C, 1, 1], padding=[0, 0, 0], unshared_offset_region=[2], epsilon=eps,
                  softmax_mode=bool(rng.integers(0, 2)))
        x, off = mex_case(int(rng.integers(1 << 30)), (B, C, H, W), n, **kw)
        off = off * float(rng.choice([0.3, 1.0, 6.0]))
        print("case", (B, C, H, W), n, eps, flush=True)
        check_mex_grads(pkg, x, off, n, **kw)
        X, O = dev(x), dev(off)
        full, pooled = pkg.mex_sum_pool_both(X, O, n, (2, 2), **kw)
        gp = torch.randn_like(pooled)
        want = pkg.mex_grads(X, O, full, pkg.sum_pooling_input_grad(gp, full.shape, (2, 2)), n, **kw)
        got = pkg.mex_sum_pool_grads(X, O, full, gp, n, (2, 2), **kw)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_mex_grads_row_wise_kernels_on_a_large_batch(pkg):
    """512 chunks of 256 pixels and 64 channels: the input gradient takes 64 patch elements per workgroup."""
    im, n = (512, 64, 16, 16), 4
    kw = dict(blocks=[64, 1, 1], strides=[64, 1, 1], padding=[0, 0, 0], unshared_offset_region=[2], epsilon=1.0,
              softmax_mode=True)
    x, off = mex_case(72, im, n, **kw)
    check_mex_grads(pkg, x, off * 0.5, n, **kw)


@pytest.mark.parametrize("eps", [1.0, -2.5, math.inf, -math.inf])
@pytest.mark.parametrize("case", [
    dict(im=(37, 512, 1, 1), n=10, kw=dict(blocks=[512, 1, 1], strides=[512, 1, 1], padding=[0, 0, 0],
                                           use_unshared_regions=False, shared_offset_region=[-1])),   # classifier head
    dict(im=(9, 100, 2, 2), n=13, kw=dict(blocks=[100, 1, 1], strides=[100, 1, 1], padding=[0, 0, 0],
                                          unshared_offset_region=[2])),              # four regions, ragged K
    dict(im=(3, 20, 5, 4), n=6, kw=dict(blocks=[20, 2, 2], strides=[20, 1, 1], padding=[0, 1, 0],
                                        use_unshared_regions=False, shared_offset_region=[2])),   # overlapping patches, padding
    dict(im=(2, 1000, 1, 3), n=4, kw=dict(blocks=[1000, 1, 1], strides=[1000, 1, 1], padding=[0, 0, 0],
                                          use_unshared_regions=False, shared_offset_region=[1, 1, 2])),   # 16 elements a lane
])
def test_mex_grads_few_pixels_long_patches_few_instances(pkg, case, eps):
    """Few pixels, 64 <= K <= 1024, few instances (the classifier head of the reference's networks, where the forward
    pass runs its wave-per-pixel kernel): both gradients against the oracle for either epsilon; with the offsets
    normalisation one call for both equals the two separate calls bit for bit and every row of the offsets gradient
    sums to zero."""
    kw = dict(case["kw"], epsilon=eps, softmax_mode=True)
    x, off = mex_case(91, case["im"], case["n"], **kw)
    check_mex_grads(pkg, x, off * 0.5, case["n"], **kw)
    kwn = dict(kw, normalize_offsets=True)
    X, O = dev(x), dev(off)
    Y = pkg.mex(X, O, case["n"], **kwn)
    G = torch.randn_like(Y)
    dx, doff = pkg.mex_grads(X, O, Y, G, case["n"], **kwn)
    assert torch.equal(dx, pkg.mex_input_grad(X, O, Y, G, case["n"], **kwn))
    assert torch.equal(doff, pkg.mex_offsets_grad(X, O, Y, G, case["n"], **kwn))
    # the sum of an instance's offsets gradient vanishes under the normalisation (d/do of o - logsumexp(o))
    rows = doff.reshape(doff.shape[0], doff.shape[1], -1)
    assert float(rows.sum(-1).abs().max()) <= 1e-3 * max(1.0, float(rows.abs().max()))


@pytest.mark.parametrize("case", [
    dict(im=(5, 40, 6, 6), n=70, kw=dict(blocks=[40, 1, 1], strides=[40, 1, 1], padding=[0, 0, 0],
                                         unshared_offset_region=[2], epsilon=2.0, softmax_mode=True)),
    dict(im=(3, 6, 12, 12), n=10, kw=dict(blocks=[3, 3, 3], strides=[2, 1, 1], padding=[1, 1, 1], epsilon=-1.5,
                                          use_unshared_regions=False, shared_offset_region=[2])),   # overlapping patches
    dict(im=(4, 9, 7, 5), n=6, kw=dict(blocks=[3, 2, 2], strides=[3, 2, 2], padding=[0, 1, 0],
                                       epsilon=-math.inf, softmax_mode=False)),                     # infinite epsilon
    dict(im=(6, 200, 4, 4), n=200, kw=dict(blocks=[200, 1, 1], strides=[200, 1, 1], padding=[0, 0, 0],
                                           unshared_offset_region=[2], epsilon=1.0, softmax_mode=True)),  # factor buffers
])
@pytest.mark.parametrize("normalize", [False, True])
def test_mex_grads_in_one_call_equal_the_two_calls(pkg, case, normalize):
    """mex_grads = (mex_input_grad, mex_offsets_grad) bit for bit, with the shared preparation done once."""
    kw = dict(case["kw"], normalize_offsets=normalize)
    x, off = mex_case(33, case["im"], case["n"], **case["kw"])
    off = off * 0.5
    X, O = dev(x), dev(off)
    Y = pkg.mex(X, O, case["n"], **kw)
    G = torch.randn_like(Y)
    dx, doff = pkg.mex_grads(X, O, Y, G, case["n"], **kw)
    dx1 = pkg.mex_input_grad(X, O, Y, G, case["n"], **kw)
    do1 = pkg.mex_offsets_grad(X, O, Y, G, case["n"], **kw)
    assert torch.equal(do1, doff)
    assert torch.equal(dx1, dx)


@pytest.mark.parametrize("func,norm,ign", [("L1", False, False), ("L2", False, False), ("L2", True, True)])
@pytest.mark.parametrize("case", [
    dict(shape=(9, 12, 7, 7), O=20, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),     # 14 pixel groups: 4 images a wave
    dict(shape=(7, 5, 5, 6), O=33, blocks=[2, 3], strides=[1, 1], padding=[0, 2]),      # ragged image groups, odd sizes
    dict(shape=(11, 40, 9, 8), O=9, blocks=[3, 3], strides=[2, 2], padding=[1, 1]),     # stride phases of 5x4 pixels
    dict(shape=(70, 3, 3, 3), O=6, blocks=[3, 3], strides=[1, 1], padding=[0, 0]),      # 3 groups an image: 21 images a wave
])
def test_similarity_input_grad_small_maps_share_a_wave(pkg, case, func, norm, ign):
    """Phase grids of at most 32 pixel groups: a wave of the term-by-term input-gradient kernel covers several
    images (L1 always takes that kernel; the L2 modes with fewer than 24 channels, or with algo='direct')."""
    x, t, w = sim_inputs(77, case["shape"], case["O"], case["blocks"], nan_frac=0.15 if ign else 0.0)
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              normalization_term=norm, ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else 0.25)
    out = orc.similarity_fwd(x, t, w, **kw)
    og = np.random.default_rng(5).normal(size=out.shape).astype(np.float32)
    want = orc.similarity_input_grad(x, t, w, og, **kw)
    true = orc.similarity_input_grad(*f64(x, t, w, og), **kw)
    dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(og), algo="direct", **kw).cpu().numpy()
    assert np.array_equal(np.isnan(dx), np.isnan(want))
    assert_grad_close(np.nan_to_num(dx), np.nan_to_num(want), np.nan_to_num(true), "input grad")


@pytest.mark.parametrize("func,norm,ign", [("L1", False, False), ("L2", False, False), ("L2", True, True)])
@pytest.mark.parametrize("case", [
    dict(shape=(2, 3, 40, 50), O=9, blocks=[7, 7], strides=[2, 2], padding=[3, 3]),     # an image-like first layer
    dict(shape=(1, 4, 20, 33), O=17, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),    # four channels, ragged rows
    dict(shape=(3, 3, 9, 130), O=5, blocks=[2, 5], strides=[1, 3], padding=[0, 2]),     # wide rows: several pixel waves
])
def test_similarity_input_grad_of_few_channels(pkg, case, func, norm, ign):
    """Three or four input channels: the term-by-term input-gradient kernel runs 8 pixels x 4 channels per lane."""
    x, t, w = sim_inputs(78, case["shape"], case["O"], case["blocks"], nan_frac=0.15 if ign else 0.0)
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              normalization_term=norm, ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else -0.5)
    out = orc.similarity_fwd(x, t, w, **kw)
    og = np.random.default_rng(6).normal(size=out.shape).astype(np.float32)
    want = orc.similarity_input_grad(x, t, w, og, **kw)
    true = orc.similarity_input_grad(*f64(x, t, w, og), **kw)
    dx = pkg.similarity_input_grad(dev(x), dev(t), dev(w), dev(og), **kw).cpu().numpy()
    assert np.array_equal(np.isnan(dx), np.isnan(want))
    assert_grad_close(np.nan_to_num(dx), np.nan_to_num(want), np.nan_to_num(true), "input grad")


@pytest.mark.parametrize("case", [
    dict(shape=(32, 64, 56, 56), O=128, blocks=[3, 3], strides=[2, 2], padding=[1, 1]),   # interleaved stride phases
    dict(shape=(32, 512, 7, 7), O=512, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),    # images share a tile, split
    dict(shape=(32, 256, 14, 14), O=256, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),  # split contraction
    dict(shape=(8, 64, 57, 55), O=96, blocks=[3, 3], strides=[3, 2], padding=[1, 1]),     # six phase grids
])
def test_similarity_input_grad_forms_agree_at_network_sizes(pkg, case):
    """Sizes the oracle would take minutes for: the matrix-core form against the term-by-term kernel (which the small
    cases pin to the oracle), L2 with and without the normalization term."""
    g = torch.Generator(device="cuda").manual_seed(11)
    shape, O = case["shape"], case["O"]
    x = torch.randn(shape, device="cuda", generator=g) + 1.5
    t = torch.randn((O, shape[1]) + tuple(case["blocks"]), device="cuda", generator=g) + 1.5
    w = torch.rand(t.shape, device="cuda", generator=g) + 0.1
    for norm in (False, True):
        kw = dict(similarity_function="L2", blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
                  normalization_term=norm)
        og = torch.randn(pkg.similarity_output_shape(shape, t.shape, **kw), device="cuda", generator=g)
        fast = pkg.similarity_input_grad(x, t, w, og, **kw)
        exact = pkg.similarity_input_grad(x, t, w, og, algo="direct", **kw)
        scale = exact.abs().max().item()
        assert (fast - exact).abs().max().item() <= 1e-4 * scale, (case, norm)


@pytest.mark.parametrize("im,n,blocks", [((10, 1, 9, 7), 22, [1, 1, 1]), ((5, 3, 6, 5), 70, [3, 1, 1]),
                                         ((70, 4, 3, 3), 9, [2, 1, 1])])
@pytest.mark.parametrize("eps", [1.0, -2.0])
def test_mex_grads_regions_with_offsets_far_from_each_other(pkg, im, n, blocks, eps):
    # one region per pixel, a handful of pixel slots per region, the regions' offsets 300 apart: the empty slots of a
    # region's last group of 64 stand on a pixel of another region, whose output lies far from this region's offsets;
    # they must not reach the sums (zero times an overflowed exponential would be NaN).  Offsets this far from zero also
    # take the kernels' term-by-term form (exponents built from scaled values of size 150 |eps| log2(e) would carry
    # their last bit, 1.5e-5 ... 3e-5, into every term): the reference's arithmetic, to the usual bar
    g = np.random.default_rng(91)
    kw = dict(blocks=blocks, strides=blocks, padding=[0, 0, 0], epsilon=eps, softmax_mode=True,
              use_unshared_regions=False, shared_offset_region=[2, 1, 1])
    d = orc.mex_dims(orc.mex_args(im, n, **kw))
    x = g.normal(size=im).astype(np.float32)
    off = g.normal(size=(d.num_regions, n) + tuple(blocks)).astype(np.float32)
    off += (150.0 * np.where(np.arange(d.num_regions) % 2 == 0, -1.0, 1.0)).astype(np.float32)[:, None, None, None, None]
    # (with more than one patch element the reference's own x + o - out is rounded at this size: 2e-4 against fp64)
    check_mex_grads(pkg, x, off, n, strict=False, **kw)


@pytest.mark.parametrize("size,eps", [(30.0, 1.0), (50.0, 1.0), (30.0, -2.0)])
def test_mex_grads_single_element_patches_with_offsets_far_from_zero(pkg, size, eps):
    # K = 1: out = x + o, every term of the gradients is g exactly in the reference's arithmetic (it subtracts out from
    # x + o before scaling).  Offsets of a size whose scaled values reach 64 exponents of two are taken term by term for
    # that reason; just below, the product form's exponents carry the last bit of values of that size (4e-6)
    g = np.random.default_rng(92)
    im, n = (12, 1, 3, 8), 69
    kw = dict(blocks=[1, 1, 1], strides=[1, 1, 1], padding=[0, 0, 0], epsilon=eps, softmax_mode=True,
              use_unshared_regions=False, shared_offset_region=[1, 2, 2])
    d = orc.mex_dims(orc.mex_args(im, n, **kw))
    x = g.normal(size=im).astype(np.float32)
    off = (g.uniform(-1.0, 1.0, size=(d.num_regions, n, 1, 1, 1)) * size).astype(np.float32)
    check_mex_grads(pkg, x, off, n, **kw)


# ---- seeded sweeps over random layers -----------------------------------------------------------------------------
def test_mex_grads_random_geometries(pkg):
    """Both MEX gradients (the separate calls and the one call, which must agree bit for bit) on seeded random layers:
    whole-channel and small 3-D blocks, overlapping and strided patches, padding, shared and unshared regions, either
    sign of epsilon and +-inf, offsets of order one and of order thirty (beyond the product form)."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        whole = case % 3 != 2
        if whole:
            H, W = int(rng.integers(1, 10)), int(rng.integers(1, 10))
            C = int(rng.choice([1, 3, 8, 32, 40, 64, 130]))
            blocks, strides, padding = [C, 1, 1], [C, 1, 1], [0, 0, 0]
        else:
            H, W, C = int(rng.integers(3, 10)), int(rng.integers(3, 10)), int(rng.integers(1, 7))
            blocks = [int(rng.integers(1, C + 1)), int(rng.integers(1, 4)), int(rng.integers(1, 4))]
            strides = [int(rng.integers(1, blocks[0] + 1)), int(rng.integers(1, 3)), int(rng.integers(1, 3))]
            padding = [0, int(rng.integers(0, 2)), int(rng.integers(0, 2))]
        n = int(rng.integers(1, 70))
        B = int(rng.integers(1, max(2, min(12, 60000 // max(1, H * W * C * n // 4)) + 1)))
        unshared = bool(rng.integers(0, 2))
        region = [1, 2, 2] if rng.integers(0, 2) else [int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        eps = float(rng.choice([1.0, -1.0, 2.5, -0.4, math.inf, -math.inf]))
        kw = dict(blocks=blocks, strides=strides, padding=padding, epsilon=eps, softmax_mode=bool(rng.integers(0, 2)),
                  use_unshared_regions=unshared, blocks_out_of_bounds_value=float(rng.choice([0.0, -1.5])))
        kw["unshared_offset_region" if unshared else "shared_offset_region"] = region
        try:
            d = orc.mex_dims(orc.mex_args((B, C, H, W), n, **kw))
        except Exception:
            continue   # a geometry the reference rejects
        g = np.random.default_rng(int(rng.integers(1 << 30)))
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        scale = float(rng.choice([0.3, 1.0, 30.0]))
        off = (g.normal(size=(d.num_regions, n) + tuple(blocks)) * scale).astype(np.float32)
        print("case", case, (B, C, H, W), n, kw, scale, flush=True)
        # ties of the maximum (infinite epsilon) split the gradient differently in fp32 and fp64 only when two terms
        # are equal to the last bit: not with random data
        check_mex_grads(pkg, x, off, n, seed=case, strict=scale <= 1.0, **kw)
        out = orc.mex_fwd(x, off, n, **kw)
        gy = np.random.default_rng(case).normal(size=out.shape).astype(np.float32)
        X, O, Y, G = dev(x), dev(off), dev(out), dev(gy)
        both = pkg.mex_grads(X, O, Y, G, n, **kw)
        assert torch.equal(both[0], pkg.mex_input_grad(X, O, Y, G, n, **kw))
        assert torch.equal(both[1], pkg.mex_offsets_grad(X, O, Y, G, n, **kw))


def test_similarity_grads_random_geometries(pkg):
    """The Similarity gradients on seeded random layers: all four modes, blocks 1 ... 4, strides 1 ... 3, padding, NaN
    inputs where they are ignored, template counts around the kernels' tile sizes."""
    rng = np.random.default_rng(515)
    for case in range(60):
        func = "L1" if case % 4 == 0 else "L2"
        norm = func == "L2" and case % 4 >= 2
        ign = norm and case % 4 == 3
        C, H, W = int(rng.choice([1, 2, 3, 8, 24])), int(rng.integers(3, 24)), int(rng.integers(3, 24))
        blocks = [int(rng.integers(1, min(4, H) + 1)), int(rng.integers(1, min(4, W) + 1))]
        strides = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        padding = [int(rng.integers(0, 3)), int(rng.integers(0, 3))]
        O = int(rng.choice([1, 4, 7, 8, 9, 31, 32, 33, 70]))
        B = int(rng.integers(1, max(2, min(12, 600000 // (H * W * C * O * blocks[0] * blocks[1])) + 1)))
        g = np.random.default_rng(int(rng.integers(1 << 30)))
        x = g.normal(size=(B, C, H, W)).astype(np.float32)
        t = g.normal(size=(O, C) + tuple(blocks)).astype(np.float32)
        w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
        if ign:
            x[g.random(size=x.shape) < 0.2] = np.nan
        kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding, normalization_term=norm,
                  ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else float(rng.choice([0.0, 0.75])))
        try:
            orc.similarity_fwd(x, t, w, **kw)
        except Exception:
            continue
        print("case", case, (B, C, H, W), O, kw, flush=True)
        # L1: the gradient is a sum of signs, which an input equal to a template value would flip: not with random data
        check_sim_grads(pkg, x, t, w, seed=case, **kw)
