"""GPU parity: the HIP library (called through the C ABI via the op layer) against the CPU oracle
on the same seeded inputs.  Similarity must agree to 1e-5 relative with identical NaN positions,
MEX to 1e-4 relative (error metric: tests/util.py:rel_err)."""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import config1, config2, config3, rel_err

pytestmark = pytest.mark.gpu

SIM_TOL = 1e-5
MEX_TOL = 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_similarity(pkg, x, t, w, **kw):
    out = pkg.similarity(dev(x), dev(t), dev(w), **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_mex(pkg, x, off, n, **kw):
    out = pkg.mex(dev(x), dev(off), n, **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def sim_inputs(seed, shape, O, blocks, nan_frac=0.0):
    g = np.random.default_rng(seed)
    x = g.normal(size=shape).astype(np.float32)
    t = g.normal(size=(O, shape[1]) + tuple(blocks)).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    if nan_frac:
        x[g.random(size=x.shape) < nan_frac] = np.nan
    return x, t, w


# ---- the reference's own test matrices (python/simnets/test/__init__.py:106-141) -------------------
@pytest.mark.parametrize("strides", [[1, 1], [1, 2], [2, 1], [2, 2]])
@pytest.mark.parametrize("blocks", [[1, 1], [1, 3], [3, 1], [3, 3]])
@pytest.mark.parametrize("same", [True, False])
@pytest.mark.parametrize("shape", [(1, 1, 40, 40), (2, 3, 40, 40)])
def test_similarity_reference_dimensions(pkg, strides, blocks, same, shape):
    x, t, w = sim_inputs(1, shape, 1, blocks)
    kw = dict(blocks=blocks, strides=strides, padding=[b // 2 for b in blocks] if same else [0, 0])
    assert rel_err(run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL


@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True),
                                           ("L1", False, False)])
@pytest.mark.parametrize("O", [1, 5, 32])
def test_similarity_reference_params(pkg, func, norm, ign, O):
    x, t, w = sim_inputs(2, (3, 3, 30, 30), O, (3, 3), nan_frac=0.2 if ign else 0.0)
    kw = dict(similarity_function=func, blocks=[3, 3], strides=[2, 2], padding=[1, 1], normalization_term=norm,
              ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else 0.0)
    assert rel_err(run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL


def test_similarity_l1_on_a_single_pixel(pkg):
    x, t, w = sim_inputs(3, (1, 1, 1, 1), 1, (1, 1))
    kw = dict(similarity_function="L1", blocks=[1, 1], strides=[1, 1], padding=[0, 0])
    assert rel_err(run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL


# ---- geometry edge cases --------------------------------------------------------------------------
@pytest.mark.parametrize("case", [
    dict(shape=(2, 3, 50, 31), O=7, blocks=[3, 2], strides=[1, 2], padding=[0, 1]),
    dict(shape=(1, 2, 9, 70), O=33, blocks=[5, 5], strides=[3, 3], padding=[2, 2]),
    dict(shape=(2, 1, 28, 28), O=3, blocks=[28, 28], strides=[1, 1], padding=[0, 0]),   # one output pixel
    dict(shape=(3, 4, 12, 200), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),   # wide rows
    dict(shape=(1, 130, 6, 6), O=17, blocks=[2, 2], strides=[1, 1], padding=[1, 1]),    # many channels
    dict(shape=(2, 2, 5, 5), O=2, blocks=[2, 2], strides=[4, 5], padding=[3, 3]),       # padding beyond the block
    dict(shape=(1, 1, 3, 2100), O=9, blocks=[3, 5], strides=[1, 1], padding=[1, 2]),    # rows too long for the LDS tile
])
@pytest.mark.parametrize("func", ["L1", "L2"])
def test_similarity_geometries(pkg, case, func):
    x, t, w = sim_inputs(4, case["shape"], case["O"], case["blocks"])
    kw = dict(similarity_function=func, blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              out_of_bounds_value=-0.75)
    assert rel_err(run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL


def test_similarity_nan_positions_without_ignore_nan(pkg):
    # NaN padding and NaN pixels must poison exactly the outputs whose patch contains them
    x, t, w = sim_inputs(5, (2, 2, 12, 12), 6, (3, 3), nan_frac=0.03)
    for func, norm in (("L1", False), ("L2", False), ("L2", True)):
        kw = dict(similarity_function=func, blocks=[3, 3], strides=[1, 1], padding=[1, 1],
                  normalization_term=norm, out_of_bounds_value=float("nan"))
        got, want = run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)
        assert np.isnan(want).any() and not np.isnan(want).all()
        assert rel_err(got, want) <= SIM_TOL


def test_similarity_normalization_constant_modes(pkg):
    x, t, w = sim_inputs(6, (4, 2, 8, 8), 3, (3, 3))
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[0, 0], normalization_term=True)
    for every in (False, True):
        got = run_similarity(pkg, x, t, w, norm_const_every_iteration=every, **kw)
        want = orc.similarity_fwd(x, t, w, norm_const_every_iteration=every, **kw)
        assert rel_err(got, want) <= SIM_TOL


def test_similarity_empty_batch(pkg):
    x = torch.empty((0, 3, 8, 8), device="cuda")
    t = torch.zeros((2, 3, 3, 3), device="cuda")
    out = pkg.similarity(x, t, t.abs(), blocks=[3, 3], strides=[1, 1], padding=[0, 0])
    assert tuple(out.shape) == (0, 2, 6, 6)


def test_similarity_sqrtw_algorithm_matches_direct(pkg):
    x, t, w = sim_inputs(7, (2, 8, 20, 20), 16, (3, 3))
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    want = orc.similarity_fwd(x, t, w, **kw)
    assert rel_err(run_similarity(pkg, x, t, w, algo="sqrtw", **kw), want) <= SIM_TOL


# Plain L2 runs the sqrt-weight form by default: -(sqrt(w) t - sqrt(w) x)^2 rounds differently from the reference's
# -w (t - x)^2 where a patch (nearly) equals a template, so outputs near zero are recomputed with the reference's
# arithmetic.  These cases put outputs exactly at, and close to, zero.
@pytest.mark.parametrize("geom", [
    dict(shape=(3, 6, 40, 40), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),     # 16 x 8 lane tiles
    dict(shape=(2, 5, 17, 13), O=19, blocks=[3, 2], strides=[2, 1], padding=[0, 1]),     # 4 x 8 lane tiles, ragged
    dict(shape=(2, 3, 9, 50), O=9, blocks=[2, 2], strides=[1, 2], padding=[1, 0], out_of_bounds_value=0.75),
    dict(shape=(9, 6, 7, 7), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),       # small maps: images share a wave,
    dict(shape=(5, 8, 6, 9), O=19, blocks=[2, 3], strides=[1, 1], padding=[0, 1]),       # one guard flag per workgroup
])
@pytest.mark.parametrize("kind", ["exact", "near", "negative_weights", "nan_input", "all_zero"])
def test_similarity_l2_default_form_recomputes_outputs_near_zero(pkg, geom, kind):
    g = np.random.default_rng(41)
    shape, O, blocks = geom["shape"], geom["O"], geom["blocks"]
    kw = {k: v for k, v in geom.items() if k not in ("shape", "O")}
    x = (g.normal(size=shape) * 3 + 50).astype(np.float32)          # |t| >> |t - x|: the rounding of d matters
    t = (g.normal(size=(O, shape[1]) + tuple(blocks)) * 3 + 50).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    hits = []
    if kind in ("exact", "near"):
        # templates cut out of the (padded) input: their outputs at those positions are exactly 0
        ph, pw = geom["padding"]
        xp = np.full((shape[0], shape[1], shape[2] + 2 * ph, shape[3] + 2 * pw), geom.get("out_of_bounds_value", 0.0),
                     np.float32)
        xp[:, :, ph:ph + shape[2], pw:pw + shape[3]] = x
        oh = (shape[2] + 2 * ph - blocks[0]) // geom["strides"][0] + 1
        ow = (shape[3] + 2 * pw - blocks[1]) // geom["strides"][1] + 1
        for m in range(0, O, 2):
            b, i, j = int(g.integers(shape[0])), int(g.integers(oh)), int(g.integers(ow))
            i0, j0 = i * geom["strides"][0], j * geom["strides"][1]
            t[m] = xp[b, :, i0:i0 + blocks[0], j0:j0 + blocks[1]]
            hits.append((b, m, i, j))
        if kind == "near":
            t += (g.normal(size=t.shape) * 1e-4).astype(np.float32)
    elif kind == "negative_weights":
        w[1::3] *= -1.0
        w[2, 0, 0, 0] = -0.5
    elif kind == "nan_input":
        x[g.random(size=x.shape) < 0.02] = np.nan
    elif kind == "all_zero":
        x[:], t[:] = 0.0, 0.0
    want = orc.similarity_fwd(x, t, w, **kw)
    got = run_similarity(pkg, x, t, w, **kw)
    assert rel_err(got, want) <= SIM_TOL
    if kind == "exact":
        for b, m, i, j in hits:
            assert got[b, m, i, j] == 0.0
    # the recomputed outputs are the three-instruction form's, bit for bit; the others agree to rounding
    exact_form = run_similarity(pkg, x, t, w, algo="direct", **kw)
    assert rel_err(got, exact_form) <= SIM_TOL
    if kind == "negative_weights":   # every output of a template with a negative weight is recomputed
        assert np.array_equal(got[:, 1::3], exact_form[:, 1::3], equal_nan=True)
    if kind == "all_zero":
        assert np.array_equal(got[exact_form == 0.0], exact_form[exact_form == 0.0])


@pytest.mark.parametrize("case", [
    dict(shape=(2, 8, 20, 20), O=16, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),
    dict(shape=(3, 5, 17, 13), O=70, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),     # odd C, ragged pixel tiles
    dict(shape=(2, 4, 31, 29), O=130, blocks=[2, 3], strides=[2, 1], padding=[0, 2]),    # two template groups
    dict(shape=(1, 3, 40, 40), O=5, blocks=[5, 5], strides=[2, 2], padding=[2, 2]),
    dict(shape=(2, 1, 28, 28), O=32, blocks=[2, 2], strides=[2, 2], padding=[2, 2]),     # single channel
    dict(shape=(7, 20, 7, 7), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),      # 5 + 2 images per workgroup
    dict(shape=(3, 9, 12, 11), O=12, blocks=[3, 2], strides=[2, 1], padding=[0, 0]),     # 50 pixels: 3 images a group
    dict(shape=(12, 6, 4, 4), O=9, blocks=[2, 2], strides=[1, 1], padding=[1, 1]),       # 25 pixels: 10 + 2 images
])
def test_similarity_mfma_algorithm_matches_direct(pkg, case):
    x, t, w = sim_inputs(8, case["shape"], case["O"], case["blocks"])
    x += 3.0  # a common offset, which the per-channel shift of the MFMA path must absorb
    t += 3.0
    kw = dict(blocks=case["blocks"], strides=case["strides"], padding=case["padding"], out_of_bounds_value=2.5)
    want = orc.similarity_fwd(x, t, w, **kw)
    assert rel_err(run_similarity(pkg, x, t, w, algo="mfma", **kw), want) <= SIM_TOL


def test_config3_similarity_mfma_sampled(pkg):
    x, t, w, kw = config3()
    got = run_similarity(pkg, x, t, w, algo="mfma", **kw)
    idx = [0, 101, 255]
    assert rel_err(got[idx], orc.similarity_fwd(x[idx], t, w, **kw)) <= SIM_TOL
    direct = run_similarity(pkg, x, t, w, algo="direct", **kw)
    assert rel_err(got, direct) <= SIM_TOL


# ---- benchmark configurations ------------------------------------------------------------------------
def test_config1_similarity_missing_data_layer(pkg):
    x, t, w, kw = config1(batch=64, nan_frac=0.25)
    got, want = run_similarity(pkg, x, t, w, **kw), orc.similarity_fwd(x, t, w, **kw)
    assert got.shape == (64, 32, 16, 16) and not np.isnan(got).any()
    ring = np.ones((16, 16), bool)
    ring[1:-1, 1:-1] = False
    assert np.all(got[:, :, ring] == 0.0) and not np.signbit(got[:, :, ring]).any()
    assert rel_err(got, want) <= SIM_TOL


@pytest.mark.parametrize("func", ["L2", "L1"])
def test_config3_similarity_conv_scale_sampled(pkg, func):
    # full-size launch (256 x 64 x 32 x 32, 128 templates); the oracle checks 16 of the images: the first and last
    # ones of the batch and both sides of the places where a quarter, half or eighth of the grid ends
    x, t, w, kw = config3()
    got = run_similarity(pkg, x, t, w, similarity_function=func, **kw)
    assert got.shape == (256, 128, 32, 32)
    idx = [0, 1, 31, 32, 63, 64, 101, 127, 128, 159, 160, 191, 192, 223, 254, 255]
    want = orc.similarity_fwd(x[idx], t, w, similarity_function=func, threads=8, **kw)
    assert rel_err(got[idx], want) <= SIM_TOL
    # size-independent property over the whole batch: permuting the images permutes the outputs
    perm = np.random.default_rng(0).permutation(256)
    got2 = run_similarity(pkg, x[perm], t, w, similarity_function=func, **kw)
    assert np.array_equal(got2, got[perm])


@pytest.mark.parametrize("ignore_nan", [False, True])
def test_config3_similarity_normalized_modes_at_conv_scale(pkg, ignore_nan):
    # the reference's normalised L2 functors (include/utils/similarity_utils.hpp:38-80) at the full config-3 size;
    # with NaN inputs ignored a quarter of the input is missing and the border is NaN.  The oracle checks 16 images,
    # NaN positions included (rel_err asserts that they coincide); the whole batch through the permutation property.
    x, t, w, kw = config3()
    kw = dict(kw, normalization_term=True)
    if ignore_nan:
        x = x.copy()
        x[np.random.default_rng(5).random(x.shape) < 0.25] = np.nan
        kw.update(ignore_nan_input=True, out_of_bounds_value=float("nan"))
    got = run_similarity(pkg, x, t, w, **kw)
    assert got.shape == (256, 128, 32, 32)
    idx = [0, 1, 31, 32, 63, 64, 101, 127, 128, 159, 160, 191, 192, 223, 254, 255]
    want = orc.similarity_fwd(x[idx], t, w, threads=8, **kw)
    assert rel_err(got[idx], want) <= SIM_TOL
    perm = np.random.default_rng(1).permutation(256)
    got2 = run_similarity(pkg, x[perm], t, w, **kw)
    assert np.array_equal(got2, got[perm], equal_nan=True)


def test_config2_mex(pkg):
    x, off, n, kw = config2()
    offn = orc.normalize_offsets(off)
    assert mex_err(run_mex(pkg, x, off, n, normalize_offsets=True, **kw), x, offn, n, **kw) <= MEX_TOL
    got = run_mex(pkg, x, offn, n, **kw)
    assert mex_err(got, x, offn, n, **kw) <= MEX_TOL
    # under the plain metric the bar holds for every output that is not a near-cancellation of m and log(sum):
    # |out| >= |m| / 16 here (the rest are priced by the |m| floor above; their absolute deviation is bounded too)
    want = orc.mex_fwd(x, offn, n, **kw)
    shift = orc.mex_fwd(x, offn, n, **dict(kw, epsilon=math.inf))
    big = np.abs(want) >= np.abs(shift) / 16
    assert big.mean() > 0.9
    assert (np.abs(got - want)[big] / np.abs(want)[big]).max() <= MEX_TOL
    assert np.abs(got - want).max() <= 4e-6 * np.abs(shift).max()


# ---- MEX: the reference's region matrices (python/simnets/test/__init__.py:299-327) and more --------
MEX_ERRORS = []   # (|m|-floored error, error relative to max(|want|, 1e-6 max|want|), max |got - want|) per call


def mex_err(got, x, off, n, **kw):
    """MEX parity metric: relative to max(|want|, |m|), m = the max (min for eps < 0) term.

    The same comparison under the plain metric max(|want|, 1e-6 * max|want|) - which blows up wherever m and
    log(sum) cancel and the output passes through zero, with rounding noise of the size of ulp(m) - and the largest
    absolute deviation are kept in MEX_ERRORS; a fixture records them with the test's properties."""
    want = orc.mex_fwd(x, off, n, **kw)
    eps = kw.get("epsilon", 1.0)
    shift = orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, eps)))
    e = rel_err(got, want, floor=shift)
    fin = np.isfinite(want)
    MEX_ERRORS.append((e, rel_err(got, want), float(np.abs(got[fin] - want[fin]).max()) if fin.any() else 0.0))
    return e


def test_config2_mex_plain_metric_is_no_tighter_for_the_reference_arithmetic(pkg, record_property):
    """Under max(|want|, 1e-6 max|want|) the GPU's config-2 outputs are compared with the exact (fp64) values beside
    the fp32 CPU oracle's: where an output passes through zero both are ulp(m) away from it, which that metric turns
    into an arbitrarily large figure.  The GPU must not be further from the exact values than twice the reference's
    own fp32 arithmetic is, under either metric."""
    x, off, n, kw = config2()
    offn = orc.normalize_offsets(off)
    got = run_mex(pkg, x, offn, n, **kw)
    want32 = orc.mex_fwd(x, offn, n, **kw)
    exact = orc.mex_fwd(x.astype(np.float64), offn.astype(np.float64), n, **kw)
    shift = orc.mex_fwd(x, offn, n, **dict(kw, epsilon=math.inf))
    plain = (rel_err(got, exact), rel_err(want32, exact))
    floored = (rel_err(got, exact, floor=shift), rel_err(want32, exact, floor=shift))
    record_property("plain_metric_gpu_and_fp32_oracle_vs_fp64", plain)
    record_property("floor_m_metric_gpu_and_fp32_oracle_vs_fp64", floored)
    print("config 2 against fp64: plain metric gpu %.3g, fp32 oracle %.3g; |m|-floored gpu %.3g, fp32 oracle %.3g"
          % (plain + floored))
    assert floored[0] <= MEX_TOL and floored[0] <= 2 * floored[1] + 1e-6
    assert np.abs(got - exact).max() <= 2 * np.abs(want32 - exact).max() + 1e-7


@pytest.fixture(autouse=True)
def _record_mex_errors(record_property):
    del MEX_ERRORS[:]
    yield
    if MEX_ERRORS:
        record_property("mex_err_floor_m", max(e[0] for e in MEX_ERRORS))
        record_property("mex_err_plain_metric", max(e[1] for e in MEX_ERRORS))
        record_property("mex_max_abs_dev", max(e[2] for e in MEX_ERRORS))
        print("MEX error: %.3g relative to max(|want|, |m|); %.3g relative to max(|want|, 1e-6 max|want|); "
              "largest |got - want| %.3g" % tuple(max(e[i] for e in MEX_ERRORS) for i in range(3)))


def mex_inputs(seed, im_dims, num_instances, **kw):
    g = np.random.default_rng(seed)
    d = orc.mex_dims(orc.mex_args(im_dims, num_instances, **kw))
    x = g.normal(size=im_dims).astype(np.float32)
    off = g.normal(size=(d.num_regions, num_instances) + tuple(kw["blocks"])).astype(np.float32)
    return x, off


@pytest.mark.parametrize("unshared,spec", [(False, [2]), (False, [3]), (True, [1, 5, 4]), (True, [2])])
@pytest.mark.parametrize("strides", [[1, 1, 1], [1, 1, 4], [1, 4, 1], [1, 4, 4]])
@pytest.mark.parametrize("blocks", [[1, 1, 3], [1, 3, 3]])
@pytest.mark.parametrize("im_dims", [(1, 1, 41, 40), (2, 3, 40, 40), (2, 3, 41, 40)])
def test_mex_reference_region_matrix(pkg, unshared, spec, strides, blocks, im_dims):
    kw = dict(softmax_mode=True, padding=[0, 1, 0], strides=strides, blocks=blocks, use_unshared_regions=unshared,
              shared_offset_region=spec if not unshared else [2], unshared_offset_region=spec if unshared else [1])
    x, off = mex_inputs(11, im_dims, 2, **kw)
    assert mex_err(run_mex(pkg, x, off, 2, **kw), x, off, 2, **kw) <= MEX_TOL


@pytest.mark.parametrize("eps", [1.0, 2.0, -1.5, 0.25, math.inf, -math.inf])
@pytest.mark.parametrize("softmax", [True, False])
def test_mex_sanity_geometry_epsilons(pkg, eps, softmax):
    kw = dict(softmax_mode=softmax, blocks=[1, 3, 3], padding=[0, 1, 1], strides=[1, 2, 2], epsilon=eps)
    x, off = mex_inputs(12, (5, 1, 90, 90), 3, **kw)
    assert off.shape[0] == 2025
    assert mex_err(run_mex(pkg, x, off, 3, **kw), x, off, 3, **kw) <= MEX_TOL


@pytest.mark.parametrize("round_down", [True, False])
@pytest.mark.parametrize("unshared", [True, False])
def test_mex_3d_blocks_channel_padding_round_up(pkg, round_down, unshared):
    kw = dict(softmax_mode=False, blocks=[2, 2, 2], padding=[1, 1, 1], strides=[1, 3, 2], epsilon=0.7,
              blocks_out_of_bounds_value=-1.5, blocks_round_down=round_down, use_unshared_regions=unshared,
              shared_offset_region=[2, 2, 3], unshared_offset_region=[2, 3, 2])
    x, off = mex_inputs(13, (3, 3, 10, 13), 20, **kw)
    assert mex_err(run_mex(pkg, x, off, 20, **kw), x, off, 20, **kw) <= MEX_TOL


@pytest.mark.parametrize("case", [
    dict(im=(7, 64, 8, 8), n=128), dict(im=(9, 128, 4, 4), n=256), dict(im=(5, 256, 2, 2), n=512),
    dict(im=(6, 512, 1, 1), n=10, shared=True),
])
def test_mex_missing_data_stack_layers(pkg, case):
    Cc = case["im"][1]
    kw = dict(softmax_mode=True, blocks=[Cc, 1, 1], strides=[Cc, 1, 1])
    if case.get("shared"):
        kw.update(use_unshared_regions=True, shared_offset_region=[1])
    else:
        kw.update(use_unshared_regions=True, unshared_offset_region=[2])
    x, off = mex_inputs(14, case["im"], case["n"], **kw)
    got = run_mex(pkg, x, off, case["n"], normalize_offsets=True, **kw)
    assert mex_err(got, x, orc.normalize_offsets(off), case["n"], **kw) <= MEX_TOL


def test_mex_large_dynamic_range(pkg):
    # log-probability-like inputs spanning hundreds of units must not overflow or lose the max term
    g = np.random.default_rng(15)
    x = (g.normal(size=(4, 16, 6, 6)) * 150).astype(np.float32)
    off = np.log(g.dirichlet([1.0] * 16, size=(4, 8))).astype(np.float32).reshape(4, 8, 16, 1, 1)
    kw = dict(softmax_mode=True, blocks=[16, 1, 1], strides=[16, 1, 1], unshared_offset_region=[2])
    assert mex_err(run_mex(pkg, x, off, 8, **kw), x, off, 8, **kw) <= MEX_TOL


@pytest.mark.parametrize("geom", [
    dict(im=(6, 8, 40, 40), n=130, blocks=[8, 3, 3], strides=[8, 1, 1], padding=[0, 1, 1]),    # several pixels per lane, K = 72
    dict(im=(5, 200, 4, 4), n=70, blocks=[200, 1, 1], strides=[200, 1, 1], padding=[0, 0, 0]),  # K split over the waves
    dict(im=(40, 96, 2, 2), n=64, blocks=[96, 1, 1], strides=[96, 1, 1], padding=[0, 0, 0]),    # one pixel per image and region
])
@pytest.mark.parametrize("spread", ["narrow", "wide", "mixed", "masked"])
@pytest.mark.parametrize("eps", [1.0, -2.0, 30.0])
def test_mex_offset_ranges_product_and_two_sweep_forms(pkg, geom, spread, eps):
    # Finite epsilon: instances whose offsets span a small range take the product form
    # (sum_k exp(x_k - max x) * exp(o_k - max o)), wide or infinite ranges the two sweeps; groups of instances of
    # one launch may differ.  Patch values grow along k so that later chunks raise the running pixel maximum.
    g = np.random.default_rng(17)
    kw = dict(softmax_mode=False, blocks=geom["blocks"], strides=geom["strides"], padding=geom["padding"], epsilon=eps,
              unshared_offset_region=[2], blocks_out_of_bounds_value=-3.0)
    n = geom["n"]
    d = orc.mex_dims(orc.mex_args(geom["im"], n, **kw))
    x = (g.normal(size=geom["im"]) * 20).astype(np.float32)
    x += (np.arange(geom["im"][1], dtype=np.float32) * 0.5 * np.sign(eps))[None, :, None, None]
    off = (g.normal(size=(d.num_regions, n) + tuple(geom["blocks"])) * 0.3).astype(np.float32)
    if spread == "wide":
        off *= 400
    elif spread == "mixed":
        off[:, n // 2:] *= 400
        off[:, 3] *= 400
    elif spread == "masked":
        off[g.random(size=off.shape) < 0.2] = -math.inf if eps > 0 else math.inf
    got = run_mex(pkg, x, off, n, **kw)
    assert np.isfinite(got).all()
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL


@pytest.mark.parametrize("im,n,blocks", [
    ((9, 32, 16, 16), 64, None), ((21, 128, 4, 4), 70, None), ((45, 256, 2, 2), 40, None),   # panel and fused kernels
    ((7, 100, 4, 4), 70, None),                   # fused kernel, several chunks; tiled kernel with K split over the waves
    ((4, 8, 20, 20), 33, [8, 3, 3]),              # tiled kernel, spatial blocks with padding
    ((3, 40, 12, 12), 20, None),                  # tiled kernel, two chunks
])
@pytest.mark.parametrize("eps", [1.0, -2.0])
@pytest.mark.parametrize("span", [80.0, 100.0])
def test_mex_wide_offsets_with_patch_and_offsets_against_each_other(pkg, im, n, blocks, eps, span):
    """Offsets rows spanning far more than the product form's range.  The workgroup still takes the product form when
    every pixel's patch spans at most that range (span 80: below it, in units of the scaled exponent; 100: above it,
    the max-tracked log-sum-exp).  The case that stresses the bound: patch values and offsets run against each other,
    so the largest term is neither where the patch nor where the offsets peak, and the offsets of most terms lie
    hundreds of units below their row's maximum."""
    g = np.random.default_rng(61)
    Cc = im[1]
    blocks = blocks or [Cc, 1, 1]
    kw = dict(softmax_mode=True, blocks=blocks, strides=[Cc, 1, 1], padding=[0, blocks[1] // 2, blocks[2] // 2], epsilon=eps,
              use_unshared_regions=True, unshared_offset_region=[1, 2, 2], blocks_out_of_bounds_value=0.0)
    c1 = abs(eps) * math.log2(math.e)
    ramp = np.linspace(-0.5, 0.5, Cc, dtype=np.float32)
    x = (ramp[None, :, None, None] * (span / c1) * g.uniform(0.6, 0.97, size=(im[0], 1, im[2], im[3]))
         + g.normal(size=im) * 0.01).astype(np.float32)
    off = (-ramp[None, None, :, None, None] * g.uniform(0.5, 8.0, size=(4, n, 1, 1, 1)) * (span / c1)
           + g.normal(size=(4, n) + tuple(blocks)) * 0.3).astype(np.float32)
    got = run_mex(pkg, x, off, n, **kw)
    assert np.isfinite(got).all()
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL
    full, pooled_out = pkg.mex_sum_pool_both(dev(x), dev(off), n, (2, 2), **kw)
    assert mex_err(full.cpu().numpy(), x, off, n, **kw) <= MEX_TOL
    assert torch.equal(pooled_out, pkg.sum_pooling(full, (2, 2)))


@pytest.mark.parametrize("im,n", [((32, 512, 1, 1), 10), ((6, 200, 2, 2), 23)])
@pytest.mark.parametrize("eps", [1.0, -2.0])
@pytest.mark.parametrize("span", [80.0, 100.0])
def test_mex_wide_offsets_on_few_pixels_with_long_patches(pkg, im, n, eps, span):
    """The same two cases on the wave-per-pixel kernel (a network's head): every instance's offsets span far more than
    the product form's range; pixels whose patch spans less keep the product form, the others go term by term."""
    g = np.random.default_rng(62)
    Cc = im[1]
    kw = dict(softmax_mode=True, blocks=[Cc, 1, 1], strides=[Cc, 1, 1], epsilon=eps, use_unshared_regions=False,
              shared_offset_region=[-1])
    c1 = abs(eps) * math.log2(math.e)
    ramp = np.linspace(-0.5, 0.5, Cc, dtype=np.float32)
    x = (ramp[None, :, None, None] * (span / c1) * g.uniform(0.6, 0.97, size=(im[0], 1, im[2], im[3]))
         + g.normal(size=im) * 0.01).astype(np.float32)
    x[::3] *= 0.1          # some pixels far inside the range, next to ones at its edge
    off = (-ramp[None, None, :, None, None] * g.uniform(2.0, 8.0, size=(1, n, 1, 1, 1)) * (span / c1)
           + g.normal(size=(1, n, Cc, 1, 1)) * 0.3).astype(np.float32)
    got = run_mex(pkg, x, off, n, **kw)
    assert np.isfinite(got).all()
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL


def pooled(y, ph, pw):
    B, Cc, H, W = y.shape
    return y[:, :, :H // ph * ph, :W // pw * pw].reshape(B, Cc, H // ph, ph, W // pw, pw).sum(axis=(3, 5))


@pytest.mark.parametrize("case", [
    dict(im=(9, 32, 16, 16), n=64, pool=(2, 2)),                       # the missing-data stack's first MEX layer
    dict(im=(7, 100, 4, 4), n=70, pool=(2, 2)),                        # several K chunks, a partial instance group
    dict(im=(5, 40, 2, 2), n=130, pool=(2, 2)),                        # one window per image
    dict(im=(3, 6, 9, 11), n=20, pool=(2, 2)),                         # odd sizes: trailing row and column dropped
    dict(im=(4, 8, 6, 10), n=33, pool=(1, 2)),                         # two-pixel windows
    dict(im=(4, 8, 10, 6), n=33, pool=(2, 1)),
    dict(im=(3, 5, 12, 12), n=24, pool=(2, 2), blocks=[5, 3, 3], padding=[0, 1, 1]),   # spatial blocks, padding
    dict(im=(40, 16, 32, 32), n=20, pool=(2, 2)),                      # enough windows for the two-half workgroups
    dict(im=(36, 8, 16, 32), n=70, pool=(1, 2)),
    dict(im=(33, 7, 31, 33), n=20, pool=(2, 2), blocks=[7, 3, 3], padding=[0, 1, 1]),  # the same with ragged edges
    dict(im=(3, 6, 12, 12), n=24, pool=(2, 2), blocks=[2, 1, 1], strides=[2, 1, 1]),   # several output channels
    # whole-channel patches of 64 / 128 / 256 channels on power-of-two widths: the panel form of the kernel
    dict(im=(37, 64, 8, 8), n=70, pool=(2, 2)),                        # one image per workgroup, a partial instance group
    dict(im=(21, 128, 4, 4), n=64, pool=(2, 2)),                       # four images per workgroup, the last one part full
    dict(im=(45, 256, 2, 2), n=130, pool=(2, 2)),                      # one window per image, 16 images per workgroup
    dict(im=(5, 64, 16, 16), n=64, pool=(2, 2)),                       # four workgroups per image
    dict(im=(3, 64, 24, 16), n=16, pool=(2, 2)),                       # six workgroups per image
    dict(im=(3, 128, 4, 32), n=16, pool=(2, 2)),                       # wide and flat: two workgroups per image
    dict(im=(2, 64, 4, 64), n=16, pool=(2, 2)),                        # rows too wide for one-half workgroups: two halves
    dict(im=(2, 64, 4, 128), n=16, pool=(2, 2)),                       # rows too wide for it: the general kernel
    dict(im=(64, 64, 16, 16), n=256, pool=(2, 2)),                     # enough workgroups for its two-half form
])
@pytest.mark.parametrize("spread,eps", [("narrow", 1.0), ("narrow", -2.0), ("wide", 1.0), ("mixed", 3.0)])
def test_mex_sum_pool_fused_kernel(pkg, case, spread, eps):
    # unshared regions = the pooling window: one kernel computes a window's MEX values in one lane and adds them
    g = np.random.default_rng(18)
    Cc = case["im"][1]
    ph, pw = case["pool"]
    kw = dict(softmax_mode=False, blocks=case.get("blocks", [Cc, 1, 1]), strides=case.get("strides", [Cc, 1, 1]),
              padding=case.get("padding", [0, 0, 0]), epsilon=eps, use_unshared_regions=True,
              unshared_offset_region=[1, ph, pw], blocks_out_of_bounds_value=-2.0)
    n = case["n"]
    d = orc.mex_dims(orc.mex_args(case["im"], n, **kw))
    assert d.num_regions == ph * pw
    x = (g.normal(size=case["im"]) * 5).astype(np.float32)
    off = (g.normal(size=(d.num_regions, n) + tuple(kw["blocks"])) * 0.3).astype(np.float32)
    if spread == "wide":
        off *= 400
    elif spread == "mixed":
        off[:, n // 2:] *= 400
    got = pkg.mex_sum_pool(dev(x), dev(off), n, (ph, pw), **kw).cpu().numpy()
    want = pooled(orc.mex_fwd(x, off, n, **kw), ph, pw)
    shift = pooled(np.abs(orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, eps)))), ph, pw)
    assert got.shape == want.shape
    assert rel_err(got, want, floor=shift) <= MEX_TOL
    # and it is the two separate calls, up to the rounding of the MEX values
    two = pkg.sum_pooling(pkg.mex(dev(x), dev(off), n, **kw), (ph, pw)).cpu().numpy()
    assert rel_err(got, two, floor=shift) <= 1e-5


@pytest.mark.parametrize("im,n", [
    ((37, 64, 8, 8), 70), ((21, 128, 4, 4), 64), ((45, 256, 2, 2), 130), ((5, 64, 16, 16), 64), ((3, 64, 24, 16), 16),
    ((2, 64, 4, 64), 16), ((64, 64, 16, 16), 256), ((9, 32, 16, 16), 64), ((3, 32, 4, 8), 20),
])
@pytest.mark.parametrize("spread,eps", [("narrow", 1.0), ("narrow", -2.0), ("mixed", 3.0), ("wide", 1.0), ("wide", -2.0)])
def test_mex_panel_form_of_the_plain_call(pkg, im, n, spread, eps):
    # 2x2 unshared offsets over whole-channel patches of 32 / 64 / 128 / 256 channels: the plain MEX call runs the panel
    # kernel without its pooling; an input that is not 16-byte aligned takes the general tiled kernel on the same
    # packed offsets
    g = np.random.default_rng(46)
    kw = dict(softmax_mode=False, blocks=[im[1], 1, 1], strides=[im[1], 1, 1], epsilon=eps, use_unshared_regions=True,
              unshared_offset_region=[1, 2, 2])
    x = (g.normal(size=im) * 5).astype(np.float32)
    off = (g.normal(size=(4, n, im[1], 1, 1)) * 0.3).astype(np.float32)
    if spread == "mixed":
        off[:, n // 2:] *= 400
    elif spread == "wide":      # every workgroup runs the max-tracked log-sum-exp on the VALU from the staged tiles
        off *= 400
    got = run_mex(pkg, x, off, n, **kw)
    assert got.shape == (im[0], n, im[2], im[3])
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL
    flat = torch.empty(x.size + 1, device="cuda")
    shifted = flat[1:].view(*im)
    shifted.copy_(dev(x))
    assert shifted.data_ptr() % 16 == 4
    other = pkg.mex(shifted, dev(off), n, **kw).cpu().numpy()
    assert mex_err(other, x, off, n, **kw) <= MEX_TOL


@pytest.mark.parametrize("im,n", [
    ((37, 64, 8, 8), 70), ((21, 128, 4, 4), 64), ((45, 256, 2, 2), 130), ((5, 64, 16, 16), 64), ((3, 64, 24, 16), 16),
    ((2, 64, 4, 64), 16), ((64, 64, 16, 16), 256), ((9, 32, 16, 16), 64), ((3, 32, 4, 8), 20), ((300, 128, 4, 4), 200),
])
@pytest.mark.parametrize("eps", [math.inf, -math.inf])
@pytest.mark.parametrize("softmax", [True, False])
def test_mex_panel_form_with_infinite_epsilon(pkg, im, n, eps, softmax):
    # the same layers with epsilon = +-inf: the panel kernel takes the largest (smallest) patch + offset from its
    # tiles, an input that is not 16-byte aligned the tiled kernel; a term is one fp32 addition, so both give the
    # oracle's values bit for bit, pixels without a finite channel included
    g = np.random.default_rng(47)
    kw = dict(softmax_mode=softmax, blocks=[im[1], 1, 1], strides=[im[1], 1, 1], epsilon=eps, use_unshared_regions=True,
              unshared_offset_region=[1, 2, 2])
    x = (g.normal(size=im) * 5).astype(np.float32)
    lo = -math.inf if eps > 0 else math.inf
    x[g.random(size=im) < 0.05] = lo
    x[0, :, 0, 0] = lo
    off = g.normal(size=(4, n, im[1], 1, 1)).astype(np.float32)
    want = orc.mex_fwd(x, off, n, **kw)
    assert want[0, 0, 0, 0] == lo and np.isfinite(want).sum() > want.size // 2
    got = run_mex(pkg, x, off, n, **kw)
    assert np.array_equal(got, want)
    flat = torch.empty(x.size + 1, device="cuda")
    shifted = flat[1:].view(*im)
    shifted.copy_(dev(x))
    assert shifted.data_ptr() % 16 == 4
    assert np.array_equal(pkg.mex(shifted, dev(off), n, **kw).cpu().numpy(), want)
    two = pkg.mex_sum_pool(dev(x), dev(off), n, (2, 2), **kw).cpu().numpy()
    assert np.array_equal(two, pkg.sum_pooling(dev(got), (2, 2)).cpu().numpy())


@pytest.mark.parametrize("im,n", [((19, 64, 8, 8), 40), ((40, 256, 2, 2), 64), ((6, 128, 16, 16), 64)])
@pytest.mark.parametrize("eps", [1.0, -0.5])
def test_mex_sum_pool_panel_form_with_infinite_and_missing_inputs(pkg, im, n, eps):
    # pixels whose channels are all -inf (+inf for negative epsilon), single infinite or NaN channels, huge values:
    # the fused kernel gives what MEX followed by sum pooling gives, NaN for NaN
    g = np.random.default_rng(44)
    kw = dict(softmax_mode=True, blocks=[im[1], 1, 1], strides=[im[1], 1, 1], epsilon=eps, use_unshared_regions=True,
              unshared_offset_region=[1, 2, 2])
    x = (g.normal(size=im) * 30).astype(np.float32)
    lo = -math.inf if eps > 0 else math.inf
    x[g.random(size=im) < 0.05] = lo
    x[0, :, 0, 0] = lo                      # an empty column
    x[1, 3, 1, 1] = -lo                     # a column with an infinite maximum
    x[2, 5, 0, 1] = np.nan
    x[3] *= 1e4                             # maxima far from zero
    off = g.normal(size=(4, n, im[1], 1, 1)).astype(np.float32)
    got = pkg.mex_sum_pool(dev(x), dev(off), n, (2, 2), **kw).cpu().numpy()
    two = pkg.sum_pooling(pkg.mex(dev(x), dev(off), n, **kw), (2, 2)).cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(two))
    assert np.isnan(got[2]).any() and not np.isnan(got[4:]).any()
    with np.errstate(invalid="ignore"):
        want = pooled(orc.mex_fwd(x, off, n, **kw), 2, 2)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    fin = np.isfinite(want)
    assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
    assert np.abs(got[fin] - want[fin]).max() <= MEX_TOL * max(1.0, np.abs(want[fin]).max())


@pytest.mark.parametrize("im,n,kw", [
    ((6, 4, 7, 5), 55, dict(blocks=[1, 1, 2], strides=[1, 1, 1], use_unshared_regions=False, shared_offset_region=[1, 2, 2])),
    ((3, 2, 3, 4), 63, dict(blocks=[1, 2, 1], strides=[1, 1, 1], unshared_offset_region=[1, 3, 1])),
    ((40, 6, 2, 2), 130, dict(blocks=[6, 1, 1], strides=[6, 1, 1], unshared_offset_region=[2])),        # K-split waves
    ((20, 64, 1, 1), 10, dict(blocks=[64, 1, 1], strides=[64, 1, 1], shared_offset_region=[1])),        # wave per pixel
    ((7, 100, 2, 3), 5, dict(blocks=[100, 1, 1], strides=[100, 1, 1], unshared_offset_region=[2])),
])
@pytest.mark.parametrize("eps", [1.0, -2.0])
@pytest.mark.parametrize("offsets", ["wide", "switched_off"])
def test_mex_patches_without_a_finite_element_on_the_log_sum_exp_paths(pkg, im, n, kw, eps, offsets):
    # The reference's exp(eps (x + o - max)) is exp(inf - inf) = NaN when nothing of a patch is finite (inputs of -inf,
    # +inf for a negative epsilon: missing data), and so is its output; the product form reproduces that through its
    # pixel bound, the max-tracked log-sum-exp of the tiled and the wave-per-pixel kernels (offsets rows too wide for
    # the product form, or with entries that switch an element off) must as well - not -inf
    g = np.random.default_rng(48)
    kw = dict(kw, epsilon=eps, softmax_mode=True)
    d = orc.mex_dims(orc.mex_args(im, n, **kw))
    lo = -math.inf if eps > 0 else math.inf
    x = g.normal(size=im).astype(np.float32)
    x[g.random(size=im) < 0.3] = lo
    x[0] = lo                                   # nothing finite in the first image at all
    off = g.normal(size=(d.num_regions, n) + tuple(kw["blocks"])).astype(np.float32)
    if offsets == "wide":
        off *= 300.0
    else:
        off[g.random(size=off.shape) < 0.1] = lo
    with np.errstate(invalid="ignore", over="ignore"):
        want = orc.mex_fwd(x, off, n, **kw)
    got = run_mex(pkg, x, off, n, **kw)
    assert np.isnan(want[0]).all() and np.isfinite(want).any()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    fin = np.isfinite(want)
    assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
    assert np.abs(got[fin] - want[fin]).max() <= MEX_TOL * max(1.0, np.abs(want[fin]).max())


@pytest.mark.parametrize("kw,pool", [
    (dict(use_unshared_regions=True, unshared_offset_region=[1, 2, 2], epsilon=math.inf), (2, 2)),   # max: no product form
    (dict(use_unshared_regions=True, unshared_offset_region=[1, 2, 2]), (4, 4)),                     # window != regions
    (dict(use_unshared_regions=False, shared_offset_region=[2]), (2, 2)),                            # shared regions
    (dict(use_unshared_regions=True, unshared_offset_region=[2, 2, 2]), (2, 2)),                     # regions over channels
])
def test_mex_sum_pool_other_geometries_run_the_two_kernels(pkg, kw, pool):
    g = np.random.default_rng(19)
    kw = dict(dict(softmax_mode=True, blocks=[3, 1, 1], strides=[3, 1, 1]), **kw)
    im, n = (4, 12, 8, 8), 10
    d = orc.mex_dims(orc.mex_args(im, n, **kw))
    x = g.normal(size=im).astype(np.float32)
    off = g.normal(size=(d.num_regions, n, 3, 1, 1)).astype(np.float32)
    got = pkg.mex_sum_pool(dev(x), dev(off), n, pool, **kw).cpu().numpy()
    two = pkg.sum_pooling(pkg.mex(dev(x), dev(off), n, **kw), pool).cpu().numpy()
    assert np.array_equal(got, two)
    want = pooled(orc.mex_fwd(x, off, n, **kw), *pool)
    assert rel_err(got, want, floor=np.ones_like(want)) <= MEX_TOL


@pytest.mark.parametrize("sim", [
    dict(blocks=[2, 2], strides=[2, 2], padding=[2, 2], normalization_term=True, ignore_nan_input=True,
         out_of_bounds_value=float("nan")),                                                   # the missing-data layer
    dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1], normalization_term=True),             # normalized, 9 taps
    dict(blocks=[2, 2], strides=[1, 1], padding=[0, 0]),                                      # plain L2
    dict(blocks=[3, 2], strides=[2, 1], padding=[1, 0], similarity_function="L1", out_of_bounds_value=0.5),
])
@pytest.mark.parametrize("case", [
    dict(im=(9, 1, 28, 28), O=32, n=64), dict(im=(40, 1, 30, 34), O=40, n=70), dict(im=(3, 2, 13, 16), O=8, n=5),
])
@pytest.mark.parametrize("spread", ["narrow", "wide"])
def test_similarity_mex_sum_pool_one_kernel(pkg, sim, case, spread):
    # Similarity channels = the MEX patch of a pixel, offsets unshared over the pooling window: a single kernel
    # ("wide": offsets too far apart for the product form - the kernel's max-tracked log-sum-exp on the VALU)
    g = np.random.default_rng(23)
    im, O, n = case["im"], case["O"], case["n"]
    if im[1] * sim["blocks"][0] * sim["blocks"][1] > 16:
        pytest.skip("patch longer than the fused kernel takes (covered by the split path test)")
    x = g.uniform(-0.5, 0.5, size=im).astype(np.float32)
    if sim.get("ignore_nan_input"):
        x[g.random(size=x.shape) < 0.25] = np.nan
    t = (g.normal(size=(O, im[1]) + tuple(sim["blocks"])) * 0.3).astype(np.float32)
    w = g.uniform(0.5, 1.5, size=t.shape).astype(np.float32)
    s_ref = orc.similarity_fwd(x, t, w, **sim)
    mkw = dict(softmax_mode=True, blocks=[O, 1, 1], strides=[O, 1, 1], use_unshared_regions=True,
               unshared_offset_region=[1, 2, 2])
    d = orc.mex_dims(orc.mex_args(s_ref.shape, n, **mkw))
    off = (g.normal(size=(d.num_regions, n, O, 1, 1)) * (60.0 if spread == "wide" else 0.2)).astype(np.float32)
    got = pkg.similarity_mex_sum_pool(dev(x), dev(t), dev(w), dev(off), n, (2, 2), similarity=sim,
                                      mex=dict(mkw, normalize_offsets=True)).cpu().numpy()
    offn = orc.normalize_offsets(off)
    want = pooled(orc.mex_fwd(s_ref, offn, n, **mkw), 2, 2)
    shift = pooled(np.abs(orc.mex_fwd(s_ref, offn, n, **dict(mkw, epsilon=math.inf))), 2, 2)
    assert got.shape == want.shape
    assert rel_err(got, want, floor=shift) <= MEX_TOL
    # the Similarity values inside the kernel are the Similarity kernel's own (term-by-term form), so the result is
    # the separate calls' to the last bit
    s_dev = pkg.similarity(dev(x), dev(t), dev(w), algo="direct", **sim)
    two = pkg.mex_sum_pool(s_dev, dev(off), n, (2, 2), normalize_offsets=True, **mkw).cpu().numpy()
    assert np.array_equal(got, two, equal_nan=True)


def test_similarity_mex_sum_pool_other_geometries_run_the_separate_kernels(pkg):
    g = np.random.default_rng(24)
    x = g.normal(size=(3, 3, 12, 12)).astype(np.float32)
    t = g.normal(size=(6, 3, 3, 3)).astype(np.float32)          # 27 taps: too long for the fused kernel
    w = g.uniform(0.5, 1.5, size=t.shape).astype(np.float32)
    sim = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    mkw = dict(softmax_mode=True, blocks=[3, 1, 1], strides=[3, 1, 1], unshared_offset_region=[1, 2, 2])
    off = g.normal(size=(4, 5, 3, 1, 1)).astype(np.float32)
    got = pkg.similarity_mex_sum_pool(dev(x), dev(t), dev(w), dev(off), 5, (2, 2), similarity=sim, mex=mkw)
    two = pkg.mex_sum_pool(pkg.similarity(dev(x), dev(t), dev(w), **sim), dev(off), 5, (2, 2), **mkw)
    assert torch.equal(got, two)
    s_ref = orc.similarity_fwd(x, t, w, **sim)
    want = pooled(orc.mex_fwd(s_ref, off, 5, **mkw), 2, 2)
    assert rel_err(got.cpu().numpy(), want, floor=np.ones_like(want) * np.abs(s_ref).max()) <= MEX_TOL


def test_sum_pooling(pkg):
    g = np.random.default_rng(16)
    x = g.normal(size=(3, 5, 9, 8)).astype(np.float32)
    got = pkg.sum_pooling(dev(x), (2, 2)).cpu().numpy()
    want = x[:, :, :8].reshape(3, 5, 4, 2, 4, 2).sum(axis=(3, 5))
    assert got.shape == (3, 5, 4, 4)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(4, 6, 8, 16), (2, 3, 2, 4), (5, 7, 6, 28), (64, 64, 16, 16)])
def test_sum_pooling_2x2_vector_kernels(pkg, shape):
    # 2x2 windows on even heights and widths that are multiples of 4: the kernels that move 16 bytes per thread give
    # what the general kernels give (taken here on a copy that is not 16-byte aligned), bit for bit, forward and gradient
    g = np.random.default_rng(17)
    x = dev(g.normal(size=shape).astype(np.float32))
    B, Cc, H, W = shape
    got = pkg.sum_pooling(x, (2, 2))
    want = x.cpu().numpy().reshape(B, Cc, H // 2, 2, W // 2, 2).sum(axis=(3, 5))
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    flat = torch.empty(x.numel() + 1, device="cuda")
    shifted = flat[1:].view(*shape)
    shifted.copy_(x)
    assert shifted.data_ptr() % 16 == 4
    assert torch.equal(got, pkg.sum_pooling(shifted, (2, 2)))
    go = dev(g.normal(size=(B, Cc, H // 2, W // 2)).astype(np.float32))
    gi = pkg.sum_pooling_input_grad(go, shape, (2, 2))
    assert torch.equal(gi, go.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3))
    gflat = torch.empty(go.numel() + 1, device="cuda")
    gshift = gflat[1:].view(*go.shape)
    gshift.copy_(go)
    assert torch.equal(gi, pkg.sum_pooling_input_grad(gshift, shape, (2, 2)))


def test_missing_data_stack_end_to_end(pkg):
    # benchmark configuration 4 at a reduced batch: Similarity -> 4 x (MEX + 2x2 sum pool) -> MEX(10).
    # Each layer is checked on the GPU's own previous activations, so tolerances do not compound.
    B = 16
    x, t, w, kw = config1(batch=B, nan_frac=0.25)
    g = np.random.default_rng(4567)
    cur = pkg.similarity(dev(x), dev(t), dev(w), **kw)
    assert rel_err(cur.cpu().numpy(), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL
    ch = 32
    for layer in range(4):
        n, size = ch * 2, cur.shape[-1]
        mkw = dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1], unshared_offset_region=[2])
        off = (g.normal(size=(min(2, size) ** 2, n, ch, 1, 1)) * 0.1).astype(np.float32)
        inp = cur.cpu().numpy()
        m = pkg.mex(cur, dev(off), n, normalize_offsets=True, **mkw)
        assert mex_err(m.cpu().numpy(), inp, orc.normalize_offsets(off), n, **mkw) <= MEX_TOL
        cur = pkg.sum_pooling(m, (2, 2))
        pooled = m.cpu().numpy().reshape(B, n, size // 2, 2, size // 2, 2)
        want = (pooled[:, :, :, 0, :, 0] + pooled[:, :, :, 0, :, 1]) + pooled[:, :, :, 1, :, 0] + pooled[:, :, :, 1, :, 1]
        assert np.array_equal(cur.cpu().numpy(), want)
        ch = n
    off = (g.normal(size=(1, 10, ch, 1, 1)) * 0.1).astype(np.float32)
    mkw = dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1], shared_offset_region=[1])
    got = pkg.mex(cur, dev(off), 10, normalize_offsets=True, **mkw).cpu().numpy()
    assert got.shape == (B, 10, 1, 1)
    assert mex_err(got, cur.cpu().numpy(), orc.normalize_offsets(off), 10, **mkw) <= MEX_TOL


# ---- few pixels, long K: the wave-per-pixel kernel ---------------------------------------------------------------
@pytest.mark.parametrize("eps", [1.0, -2.0, math.inf, -math.inf])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("case", [
    dict(im=(20, 64, 1, 1), n=10, kw=dict(blocks=[64, 1, 1], strides=[64, 1, 1], shared_offset_region=[1])),
    dict(im=(7, 100, 2, 3), n=5, kw=dict(blocks=[100, 1, 1], strides=[100, 1, 1], unshared_offset_region=[2])),
    dict(im=(3, 300, 3, 2), n=17, kw=dict(blocks=[300, 1, 1], strides=[300, 1, 1], use_unshared_regions=False,
                                          shared_offset_region=[2])),                          # ragged regions
    dict(im=(2, 1024, 1, 1), n=3, kw=dict(blocks=[1024, 1, 1], strides=[1024, 1, 1])),
    dict(im=(2, 9, 6, 6), n=4, kw=dict(blocks=[9, 3, 3], strides=[9, 3, 3], padding=[0, 1, 1],
                                       blocks_out_of_bounds_value=-0.5, use_unshared_regions=False,
                                       shared_offset_region=[-1])),                           # K = 81 with padding
    dict(im=(2, 40, 3, 3), n=2, kw=dict(blocks=[20, 2, 2], strides=[10, 1, 1], padding=[5, 0, 0],
                                        unshared_offset_region=[1, 2, 2])),                    # 3-D blocks, channel padding
])
def test_mex_few_pixels_long_patches(pkg, case, normalize, eps):
    kw = dict(case["kw"], epsilon=eps, softmax_mode=normalize)
    x, off = mex_inputs(31, case["im"], case["n"], **kw)
    ref_off = orc.normalize_offsets(off) if normalize else off
    got = run_mex(pkg, x, off, case["n"], normalize_offsets=normalize, **kw)
    assert mex_err(got, x, ref_off, case["n"], **kw) <= MEX_TOL


# ---- one pixel per image and region, long K: the tiled kernel gathers with lanes along k ------------------------------
@pytest.mark.parametrize("eps", [1.0, -1.5, math.inf])
@pytest.mark.parametrize("case", [
    dict(im=(100, 256, 2, 2), n=64, kw=dict(blocks=[256, 1, 1], strides=[256, 1, 1], unshared_offset_region=[2])),
    dict(im=(130, 96, 1, 1), n=200, kw=dict(blocks=[96, 1, 1], strides=[96, 1, 1], shared_offset_region=[1],
                                           use_unshared_regions=False)),
    dict(im=(70, 40, 2, 2), n=48, kw=dict(blocks=[30, 2, 2], strides=[10, 1, 1], padding=[5, 1, 1],
                                         blocks_out_of_bounds_value=0.3)),                  # bounds checks, per-pixel regions
    dict(im=(65, 33, 3, 2), n=17, kw=dict(blocks=[33, 1, 1], strides=[33, 1, 1])),           # ragged K and M
])
def test_mex_one_pixel_per_region_long_patches(pkg, case, eps):
    kw = dict(case["kw"], epsilon=eps, softmax_mode=True)
    x, off = mex_inputs(41, case["im"], case["n"], **kw)
    got = run_mex(pkg, x, off, case["n"], **kw)
    assert mex_err(got, x, off, case["n"], **kw) <= MEX_TOL


# ---- larger, network-like geometries (oracle on one image; the batch must not matter) -----------------------------------
def test_similarity_stem_like_geometry(pkg):
    """7x7 templates, stride 2, padding 3 on 224x224 images: rows wider than the LDS tile of the big lane tile."""
    x, t, w = sim_inputs(51, (3, 3, 224, 224), 64, (7, 7))
    kw = dict(blocks=[7, 7], strides=[2, 2], padding=[3, 3])
    got = run_similarity(pkg, x, t, w, **kw)
    assert got.shape == (3, 64, 112, 112)
    for b in (0, 2):
        assert rel_err(got[b:b + 1], orc.similarity_fwd(x[b:b + 1], t, w, **kw)) <= SIM_TOL


def test_similarity_many_templates_small_images(pkg):
    x, t, w = sim_inputs(52, (64, 96, 8, 8), 384, (3, 3))
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1], similarity_function="L1")
    got = run_similarity(pkg, x, t, w, **kw)
    for b in (0, 63):
        assert rel_err(got[b:b + 1], orc.similarity_fwd(x[b:b + 1], t, w, **kw)) <= SIM_TOL


def test_mex_overlapping_3d_blocks_network_like(pkg):
    kw = dict(blocks=[64, 3, 3], strides=[64, 1, 1], padding=[0, 1, 1], softmax_mode=True, epsilon=1.0,
              use_unshared_regions=False, shared_offset_region=[4])
    x, off = mex_inputs(53, (6, 64, 28, 28), 32, **kw)
    got = run_mex(pkg, x, off, 32, **kw)
    assert got.shape == (6, 32, 28, 28)
    for b in (0, 5):
        assert mex_err(got[b:b + 1], x[b:b + 1], off, 32, **kw) <= MEX_TOL


@pytest.mark.parametrize("shape,O", [((128, 512, 7, 7), 512), ((32, 256, 14, 14), 256), ((64, 128, 8, 8), 128)])
def test_similarity_small_map_forms_agree_at_network_sizes(pkg, shape, O):
    """Deep, small maps at sizes the oracle would take minutes for: the default form (sqrt-weight arithmetic with its
    guard on the small-map kernel) against algo='direct' (the reference's arithmetic, pinned to the oracle by the
    small cases), to the forward tolerance."""
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn(shape, device="cuda", generator=g)
    t = torch.randn((O, shape[1], 3, 3), device="cuda", generator=g)
    w = torch.rand(t.shape, device="cuda", generator=g) + 0.1
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    fast = pkg.similarity(x, t, w, **kw).cpu().numpy()
    exact = pkg.similarity(x, t, w, algo="direct", **kw).cpu().numpy()
    assert rel_err(fast, exact) <= SIM_TOL


# ---- seeded sweeps: random geometries through whatever kernel the library picks -----------------------------------
def mex_close(got, x, off, n, **kw):
    """Within MEX_TOL of the fp32 oracle under mex_err's metric.  Where an output and its largest term both pass
    through zero (short patches), that metric divides rounding noise by almost nothing, for the reference's own fp32
    arithmetic as well: those elements must be within 1e-6 of the operands' size (max|x| + max|offsets|) of the exact
    (fp64) value instead, a few ulps of the terms they are made of."""
    if mex_err(got, x, off, n, **kw) <= MEX_TOL:
        return True
    want = orc.mex_fwd(x, off, n, **kw)
    exact = orc.mex_fwd(x.astype(np.float64), off.astype(np.float64), n, **kw)
    shift = orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, kw.get("epsilon", 1.0))))
    floor = np.maximum(np.abs(want), np.abs(shift))
    with np.errstate(invalid="ignore", divide="ignore"):
        bad = ~(np.abs(got - want) <= MEX_TOL * floor) & ~((got == want) | (np.isnan(got) & np.isnan(want)))
    size = float(np.abs(x).max() + np.abs(off[np.isfinite(off)]).max())
    worst = float(np.abs(got[bad] - exact[bad]).max())
    print("  %d of %d outputs beyond %g of the fp32 oracle, all with max(|want|, |m|) <= %.3g; against fp64 they are "
          "off by at most %.3g (operands up to %.3g; the fp32 oracle: %.3g)"
          % (bad.sum(), bad.size, MEX_TOL, floor[bad].max(), worst, size, np.abs(want[bad] - exact[bad]).max()))
    return bool(np.isfinite(got[bad]).all() and floor[bad].max() <= 1e-2 * size and worst <= 1e-6 * size)


def test_mex_forward_random_geometries(pkg):
    """MEX, MEX + pooling (with and without the unpooled output) on seeded random layers: whole-channel patches on
    power-of-two and ragged maps (the panel, fused, wave-per-pixel and tiled kernels), small 3-D blocks with padding,
    shared and unshared regions, either sign of epsilon and +-inf, narrow and wide offsets, with and without the
    offsets normalisation; every result against the oracle."""
    rng = np.random.default_rng(4242)
    for case in range(160):
        whole = case % 4 != 3
        if whole:
            pow2 = bool(rng.integers(0, 2))
            H = 1 << int(rng.integers(0, 5)) if pow2 else int(rng.integers(1, 13))
            W = 1 << int(rng.integers(0, 5)) if pow2 else int(rng.integers(1, 13))
            C = int(rng.choice([1, 3, 8, 32, 33, 64, 100, 128, 256, 300]))
            blocks, strides, padding = [C, 1, 1], [C, 1, 1], [0, 0, 0]
        else:
            H, W, C = int(rng.integers(3, 11)), int(rng.integers(3, 11)), int(rng.integers(1, 9))
            blocks = [int(rng.integers(1, C + 1)), int(rng.integers(1, 4)), int(rng.integers(1, 4))]
            strides = [int(rng.integers(1, blocks[0] + 1)), int(rng.integers(1, 3)), int(rng.integers(1, 3))]
            padding = [0, int(rng.integers(0, 2)), int(rng.integers(0, 2))]
        n = int(rng.integers(1, 140)) if C <= 128 else int(rng.integers(1, 24))
        B = int(rng.integers(1, max(2, min(24, 200000 // max(1, H * W * C * n // 8)) + 1)))
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
        off = (g.normal(size=(d.num_regions, n) + tuple(blocks)) * float(rng.choice([0.3, 2.0, 40.0]))).astype(np.float32)
        normalize = bool(rng.integers(0, 2))
        offn = orc.normalize_offsets(off) if normalize else off
        print("case", case, (B, C, H, W), n, kw, "normalize" if normalize else "", flush=True)
        got = run_mex(pkg, x, off, n, normalize_offsets=normalize, **kw)
        assert mex_close(got, x, offn, n, **kw)
        Ho, Wo = got.shape[2], got.shape[3]
        if Ho >= 2 and Wo >= 2:
            X, O = dev(x), dev(off)
            full, pooled = pkg.mex_sum_pool_both(X, O, n, (2, 2), normalize_offsets=normalize, **kw)
            assert mex_close(full.cpu().numpy(), x, offn, n, **kw)
            assert torch.equal(pooled, pkg.sum_pooling(full, (2, 2)))
            assert torch.equal(pooled, pkg.mex_sum_pool(X, O, n, (2, 2), normalize_offsets=normalize, **kw))


def test_similarity_forward_random_geometries(pkg):
    """Similarity on seeded random layers (all four modes, blocks 1 ... 5, strides 1 ... 3, padding, NaN inputs where
    they are ignored, template counts around the tile sizes) against the oracle."""
    rng = np.random.default_rng(777)
    for case in range(120):
        func = "L1" if case % 4 == 0 else "L2"
        norm = func == "L2" and case % 4 >= 2
        ign = norm and case % 4 == 3
        C, H, W = int(rng.choice([1, 2, 3, 8, 24, 64])), int(rng.integers(3, 40)), int(rng.integers(3, 40))
        blocks = [int(rng.integers(1, min(5, H) + 1)), int(rng.integers(1, min(5, W) + 1))]
        strides = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        padding = [int(rng.integers(0, 3)), int(rng.integers(0, 3))]
        O = int(rng.choice([1, 7, 8, 9, 31, 32, 33, 64, 130]))
        B = int(rng.integers(1, max(2, min(20, 3000000 // (H * W * C * O * blocks[0] * blocks[1])) + 1)))
        x, t, w = sim_inputs(int(rng.integers(1 << 30)), (B, C, H, W), O, blocks, nan_frac=0.2 if ign else 0.0)
        kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding, normalization_term=norm,
                  ignore_nan_input=ign, out_of_bounds_value=float("nan") if ign else float(rng.choice([0.0, 0.75])))
        try:
            want = orc.similarity_fwd(x, t, w, **kw)
        except Exception:
            continue
        print("case", case, (B, C, H, W), O, kw, flush=True)
        assert rel_err(run_similarity(pkg, x, t, w, **kw), want) <= SIM_TOL
