"""Prepared forward calls (parameters packed once, steady-state calls take the input only) through the C ABI:
bit-identical to the self-packing calls, within tolerance of the CPU oracle, and correct on repeated calls with
different inputs.  Also the wave-per-pixel MEX kernel with wide offset ranges, and the sqrt-weight Similarity form on
inputs that span several channel chunks (its guard looks at the partial sums after the first chunk)."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import config1, config2, config4_stack, rel_err

pytestmark = pytest.mark.gpu

SIM_TOL = 1e-5
MEX_TOL = 1e-4


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same_bits(a, b):
    return np.array_equal(a.cpu().numpy().view(np.uint32), b.cpu().numpy().view(np.uint32))


def mex_err(got, x, off, n, **kw):
    """MEX parity metric: relative to max(|want|, |m|), m = the max (min for eps < 0) term."""
    want = orc.mex_fwd(x, off, n, **kw)
    shift = orc.mex_fwd(x, off, n, **dict(kw, epsilon=math.copysign(math.inf, kw.get("epsilon", 1.0))))
    # the shift itself is a sum patch + offset that may cancel: its rounding scales with the offsets' size
    fin = np.abs(off[np.isfinite(off)])
    return rel_err(got, want, floor=np.maximum(np.abs(shift), fin.max() if fin.size else 0.0))


SIM_CASES = [
    dict(shape=(5, 1, 28, 28), O=32, kw=dict(similarity_function="L2", blocks=[2, 2], strides=[2, 2], padding=[2, 2],
                                            normalization_term=True, ignore_nan_input=True,
                                            out_of_bounds_value=float("nan")), nan=0.25),      # parameters through LDS
    dict(shape=(3, 3, 20, 31), O=21, kw=dict(similarity_function="L1", blocks=[3, 3], strides=[1, 2], padding=[1, 0]), nan=0),
    dict(shape=(2, 40, 34, 34), O=40, kw=dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1]), nan=0),  # several chunks
    dict(shape=(2, 40, 34, 34), O=40, kw=dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1], algo="direct"), nan=0),
    dict(shape=(2, 40, 34, 34), O=40, kw=dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1], algo="mfma"), nan=0),
    dict(shape=(2, 70, 12, 12), O=12, kw=dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1],
                                             normalization_term=True), nan=0),                 # 4x8 tile, several chunks
    dict(shape=(2, 2, 9, 9), O=3, kw=dict(blocks=[2, 3], strides=[1, 1], padding=[0, 2], out_of_bounds_value=1.5), nan=0),
]


@pytest.mark.parametrize("case", SIM_CASES)
def test_similarity_prepared_matches_plain_call_and_oracle(pkg, case):
    g = np.random.default_rng(7)
    shape, O, kw = case["shape"], case["O"], case["kw"]
    t = g.normal(size=(O, shape[1]) + tuple(kw["blocks"])).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    T, W = dev(t), dev(w)
    prep = pkg.similarity_prepare(shape, T, W, **kw)
    for rep in range(2):   # the second call reuses the buffer (and its per-call scratch) with another input
        x = g.normal(size=shape).astype(np.float32)
        if case["nan"]:
            x[g.random(size=shape) < case["nan"]] = np.nan
        X = dev(x)
        got = prep(X)
        assert same_bits(got, pkg.similarity(X, T, W, **kw))
        okw = {k: v for k, v in kw.items() if k != "algo"}
        assert rel_err(got.cpu().numpy(), orc.similarity_fwd(x, t, w, **okw)) <= SIM_TOL


SHORT_PATCH_MODES = [
    dict(similarity_function="L1"),
    dict(similarity_function="L2"),
    dict(similarity_function="L2", algo="direct"),
    dict(similarity_function="L2", normalization_term=True),
    dict(similarity_function="L2", normalization_term=True, ignore_nan_input=True, out_of_bounds_value=float("nan")),
]


@pytest.mark.parametrize("mode", SHORT_PATCH_MODES)
@pytest.mark.parametrize("geom", [((7, 3, 13, 17), 19, [2, 2], [2, 1], [1, 0]), ((4, 1, 9, 9), 8, [3, 3], [1, 1], [1, 1]),
                                  ((3, 12, 5, 6), 33, [1, 1], [1, 1], [0, 0]), ((2, 2, 6, 70), 5, [2, 3], [1, 2], [0, 2])])
def test_short_patches_self_packing_call_matches_prepared_and_oracle(pkg, mode, geom):
    """Patches of at most 12 elements: the self-packing call packs inside its one kernel, the prepared call reads
    parameters packed by the pack kernel; same bits, every mode, template counts off the tile size."""
    shape, O, blocks, strides, padding = geom
    kw = dict(mode, blocks=blocks, strides=strides, padding=padding)
    g = np.random.default_rng(11)
    t = g.normal(size=(O, shape[1]) + tuple(blocks)).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    w[0].flat[0] = 0.0
    x = g.normal(size=shape).astype(np.float32)
    if mode.get("ignore_nan_input"):
        x[g.random(size=shape) < 0.2] = np.nan
    X, T, W = dev(x), dev(t), dev(w)
    plain = pkg.similarity(X, T, W, **kw)
    assert same_bits(pkg.similarity_prepare(shape, T, W, **kw)(X), plain)
    okw = {k: v for k, v in kw.items() if k != "algo"}
    assert rel_err(plain.cpu().numpy(), orc.similarity_fwd(x, t, w, **okw)) <= SIM_TOL


def test_similarity_prepared_config1_full(pkg):
    x, t, w, kw = config1(batch=64, nan_frac=0.25)
    prep = pkg.similarity_prepare(x.shape, dev(t), dev(w), **kw)
    got = prep(dev(x)).cpu().numpy()
    assert rel_err(got, orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL


def test_prepared_rejects_other_shapes(pkg):
    x, t, w, kw = config1(batch=4)
    prep = pkg.similarity_prepare(x.shape, dev(t), dev(w), **kw)
    with pytest.raises(pkg.SimnetsError):
        prep(dev(x[:3]))


MEX_CASES = [
    dict(im=(64, 32, 16, 16), n=64, kw=dict(blocks=[32, 1, 1], strides=[32, 1, 1], unshared_offset_region=[2])),   # config 2
    dict(im=(6, 8, 40, 40), n=130, kw=dict(blocks=[8, 3, 3], strides=[8, 1, 1], padding=[0, 1, 1])),
    dict(im=(40, 96, 2, 2), n=64, kw=dict(blocks=[96, 1, 1], strides=[96, 1, 1], unshared_offset_region=[2])),
    dict(im=(20, 64, 1, 1), n=10, kw=dict(blocks=[64, 1, 1], strides=[64, 1, 1], shared_offset_region=[1])),     # wave per pixel
    dict(im=(3, 300, 3, 2), n=17, kw=dict(blocks=[300, 1, 1], strides=[300, 1, 1], use_unshared_regions=False,
                                          shared_offset_region=[2])),
]


@pytest.mark.parametrize("eps", [1.0, -2.0, math.inf])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("case", MEX_CASES)
def test_mex_prepared_matches_plain_call_and_oracle(pkg, case, normalize, eps):
    g = np.random.default_rng(9)
    kw = dict(case["kw"], epsilon=eps, softmax_mode=True)
    n = case["n"]
    d = orc.mex_dims(orc.mex_args(case["im"], n, **kw))
    off = (g.normal(size=(d.num_regions, n, d.block_c, d.block_h, d.block_w)) * 0.5).astype(np.float32)
    OFF = dev(off)
    prep = pkg.mex_prepare(case["im"], OFF, n, normalize_offsets=normalize, **kw)
    ref_off = orc.normalize_offsets(off) if normalize else off
    for rep in range(2):
        x = g.normal(size=case["im"]).astype(np.float32)
        X = dev(x)
        got = prep(X)
        assert same_bits(got, pkg.mex(X, OFF, n, normalize_offsets=normalize, **kw))
        assert mex_err(got.cpu().numpy(), x, ref_off, n, **kw) <= MEX_TOL


@pytest.mark.parametrize("spread", ["narrow", "wide", "mixed", "masked"])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("im,n", [((64, 32, 16, 16), 64), ((9, 32, 16, 16), 20), ((7, 32, 8, 16), 70), ((3, 32, 4, 8), 130)])
def test_mex_small_single_chunk_layer_packs_inside_its_kernel(pkg, im, n, normalize, spread):
    """A self-packing call of a layer with 2x2 unshared offsets over 32 channels on a small grid is one launch whose
    workgroups pack their offsets rows themselves: the same bits as the prepared call (pack kernel + forward kernel),
    with and without the logsumexp normalisation, for partial and several instance groups, and for rows too far apart
    for the product form (which both paths then evaluate as a max-tracked log-sum-exp)."""
    g = np.random.default_rng(31)
    eps = 1.5
    kw = dict(blocks=[32, 1, 1], strides=[32, 1, 1], unshared_offset_region=[2], epsilon=eps, softmax_mode=False)
    off = (g.normal(size=(4, n, 32, 1, 1)) * 0.5).astype(np.float32)
    if spread == "wide":
        off *= 300
    elif spread == "mixed":
        off[1:3, n // 3:] *= 300
    elif spread == "masked":
        off[g.random(size=off.shape) < 0.2] = -math.inf
    x = (g.normal(size=im) * 3).astype(np.float32)
    X, OFF = dev(x), dev(off)
    plain = pkg.mex(X, OFF, n, normalize_offsets=normalize, **kw)
    prep = pkg.mex_prepare(im, OFF, n, normalize_offsets=normalize, **kw)(X)
    assert same_bits(plain, prep)
    ref_off = orc.normalize_offsets(off) if normalize else off
    assert mex_err(plain.cpu().numpy(), x, ref_off, n, **kw) <= MEX_TOL
    # offsets that are not 16-byte aligned take the pack kernel: still the same bits
    flat = torch.empty(off.size + 1, device="cuda")
    shifted = flat[1:].view(*off.shape)
    shifted.copy_(OFF)
    assert shifted.data_ptr() % 16 == 4
    assert same_bits(pkg.mex(X, shifted, n, normalize_offsets=normalize, **kw), plain)


def test_mex_prepared_config2_full(pkg):
    x, off, n, kw = config2()
    prep = pkg.mex_prepare(x.shape, dev(off), n, normalize_offsets=True, **kw)
    got = prep(dev(x)).cpu().numpy()
    assert mex_err(got, x, orc.normalize_offsets(off), n, **kw) <= MEX_TOL


@pytest.mark.parametrize("spread", ["wide", "mixed", "masked", "all_masked_row"])
@pytest.mark.parametrize("eps", [1.0, -2.0, 30.0])
def test_mex_wave_per_pixel_offset_ranges(pkg, spread, eps):
    """The few-pixels kernel takes the product form per instance while the instance's offsets span a small range and
    sums term by term otherwise; groups of four instances may mix the two."""
    g = np.random.default_rng(23)
    im, n = (9, 200, 1, 1), 11
    kw = dict(softmax_mode=False, blocks=[200, 1, 1], strides=[200, 1, 1], epsilon=eps, shared_offset_region=[1])
    x = (g.normal(size=im) * 20).astype(np.float32)
    off = (g.normal(size=(1, n, 200, 1, 1)) * 0.3).astype(np.float32)
    if spread == "wide":
        off *= 400
    elif spread == "mixed":
        off[:, 5:] *= 400
        off[:, 2] *= 400
    elif spread == "masked":
        off[g.random(size=off.shape) < 0.2] = -math.inf if eps > 0 else math.inf
    else:
        off[:, 4] = -math.inf if eps > 0 else math.inf
    got = pkg.mex(dev(x), dev(off), n, **kw).cpu().numpy()
    if spread != "all_masked_row":
        assert np.isfinite(got).all()
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL
    x[3, 17] = math.inf if eps > 0 else -math.inf      # an infinite patch value: NaN like the reference's exp(inf - inf)
    x[5, 0] = np.nan
    got = pkg.mex(dev(x), dev(off), n, **kw).cpu().numpy()
    assert mex_err(got, x, off, n, **kw) <= MEX_TOL


def test_config4_stack_prepared_matches_plain_calls(pkg):
    """The missing-data stack with every layer prepared: separate calls, MEX + pooling pairs, and the Similarity layer
    inside the first pair - each bit-identical to the self-packing calls of the same layers, on two batches."""
    B = 64
    x, t, w, skw, layers, last = config4_stack(batch=B)
    T, W = dev(t), dev(w)
    offs = [dev(o) for o, _, _ in layers]
    offl, nl, kwl = last
    OFFL = dev(offl)
    shapes, ch, size = [], 32, 16
    for _, n, _ in layers:
        shapes.append((B, ch, size, size))
        ch, size = n, size // 2
    p_sim = pkg.similarity_prepare(x.shape, T, W, **skw)
    p_mex = [pkg.mex_prepare(s, o, n, normalize_offsets=True, **kw) for s, o, (_, n, kw) in zip(shapes, offs, layers)]
    p_pool = [pkg.mex_sum_pool_prepare(s, o, n, (2, 2), normalize_offsets=True, **kw)
              for s, o, (_, n, kw) in zip(shapes, offs, layers)]
    p_first = pkg.similarity_mex_sum_pool_prepare(x.shape, T, W, offs[0], layers[0][1], (2, 2), similarity=skw,
                                                  mex=dict(layers[0][2], normalize_offsets=True))
    p_last = pkg.mex_prepare((B, ch, 1, 1), OFFL, nl, normalize_offsets=True, **kwl)
    g = np.random.default_rng(3)
    for rep in range(2):
        xb = x if rep == 0 else np.where(g.random(size=x.shape) < 0.25, np.nan, g.uniform(-0.5, 0.5, size=x.shape)
                                          ).astype(np.float32)
        X = dev(xb)
        cur = pkg.similarity(X, T, W, **skw)
        assert same_bits(p_sim(X), cur)
        fused_first = pkg.similarity_mex_sum_pool(X, T, W, offs[0], layers[0][1], (2, 2), similarity=skw,
                                                  mex=dict(layers[0][2], normalize_offsets=True))
        assert same_bits(p_first(X), fused_first)
        for i, (_, n, kw) in enumerate(layers):
            y = pkg.mex(cur, offs[i], n, normalize_offsets=True, **kw)
            assert same_bits(p_mex[i](cur), y)
            pooled = pkg.mex_sum_pool(cur, offs[i], n, (2, 2), normalize_offsets=True, **kw)
            assert same_bits(p_pool[i](cur), pooled)
            cur = pkg.sum_pooling(y, (2, 2))
        head = pkg.mex(cur, OFFL, nl, normalize_offsets=True, **kwl)
        assert same_bits(p_last(cur), head)
        assert mex_err(head.cpu().numpy(), cur.cpu().numpy(), orc.normalize_offsets(offl), nl, **kwl) <= MEX_TOL


def test_unfused_pairs_prepared(pkg):
    """Geometries the fused kernels do not serve run the separate kernels through the prepared buffer's scratch."""
    g = np.random.default_rng(5)
    x = g.normal(size=(3, 6, 12, 12)).astype(np.float32)
    off = (g.normal(size=(1, 9, 6, 1, 1)) * 0.3).astype(np.float32)
    kw = dict(blocks=[6, 1, 1], strides=[6, 1, 1], use_unshared_regions=False, shared_offset_region=[-1],
              softmax_mode=True)
    X, OFF = dev(x), dev(off)
    p = pkg.mex_sum_pool_prepare(x.shape, OFF, 9, (3, 2), **kw)
    assert same_bits(p(X), pkg.mex_sum_pool(X, OFF, 9, (3, 2), **kw))
    xs = g.normal(size=(3, 2, 14, 14)).astype(np.float32)
    t = g.normal(size=(6, 2, 3, 3)).astype(np.float32)        # 18 taps: beyond what the fused kernel evaluates
    w = (np.abs(g.normal(size=t.shape)) + 0.1).astype(np.float32)
    skw = dict(blocks=[3, 3], strides=[1, 1], padding=[0, 0])
    mkw = dict(blocks=[6, 1, 1], strides=[6, 1, 1], unshared_offset_region=[2], softmax_mode=True)
    off2 = (g.normal(size=(4, 5, 6, 1, 1)) * 0.3).astype(np.float32)
    XS, T, W, OFF2 = dev(xs), dev(t), dev(w), dev(off2)
    p = pkg.similarity_mex_sum_pool_prepare(xs.shape, T, W, OFF2, 5, (2, 2), similarity=skw, mex=mkw)
    for _ in range(2):
        assert same_bits(p(XS), pkg.similarity_mex_sum_pool(XS, T, W, OFF2, 5, (2, 2), similarity=skw, mex=mkw))


# ---- sqrt-weight form over several channel chunks -----------------------------------------------------------------
CHUNKED = dict(shape=(2, 40, 34, 34), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1])   # 4x8 tile, 3 chunks
CHUNKED_SMALL = dict(shape=(2, 70, 20, 20), O=12, blocks=[3, 3], strides=[1, 1], padding=[1, 1])  # 4x8 tile, 2 tiles per image


@pytest.mark.parametrize("geom", [CHUNKED, CHUNKED_SMALL])
@pytest.mark.parametrize("kind", ["ordinary", "exact", "first_chunk_equal", "all_close", "negative_weights",
                                  "zero_weight_chunk", "late_nan"])
def test_similarity_sqrt_weight_form_over_channel_chunks(pkg, geom, kind):
    g = np.random.default_rng(43)
    shape, O, blocks = geom["shape"], geom["O"], geom["blocks"]
    kw = {k: v for k, v in geom.items() if k not in ("shape", "O")}
    x = (g.normal(size=shape) * 3 + 50).astype(np.float32)
    t = (g.normal(size=(O, shape[1]) + tuple(blocks)) * 3 + 50).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    hits = []
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    if kind in ("exact", "first_chunk_equal"):
        for m in range(0, O, 3):
            b, i, j = int(g.integers(shape[0])), int(g.integers(shape[2])), int(g.integers(shape[3]))
            patch = xp[b, :, i:i + 3, j:j + 3]
            if kind == "exact":
                t[m] = patch
                hits.append((b, m, i, j))
            else:
                t[m, :8] = patch[:8]    # equal over the first channels only: the partial sum is 0, the output is not
    elif kind == "all_close":
        # every patch within 3 of every template at offset 1000: all outputs are far below the threshold
        x = (g.normal(size=shape) + 1000).astype(np.float32)
        t = (g.normal(size=t.shape) + 1000).astype(np.float32)
    elif kind == "negative_weights":
        w[1::4] *= -1.0
    elif kind == "zero_weight_chunk":
        w[::2, :14] = 0.0
    elif kind == "late_nan":
        x[:, -3:][g.random(size=x[:, -3:].shape) < 0.05] = np.nan
    want = orc.similarity_fwd(x, t, w, **kw)
    got = pkg.similarity(dev(x), dev(t), dev(w), **kw).cpu().numpy()
    assert rel_err(got, want) <= SIM_TOL
    exact_form = pkg.similarity(dev(x), dev(t), dev(w), algo="direct", **kw).cpu().numpy()
    for b, m, i, j in hits:
        assert got[b, m, i, j] == 0.0
    if kind == "all_close":
        assert np.array_equal(got, exact_form)          # every wave is recomputed: the term-by-term result, bit for bit
    if kind == "negative_weights":
        assert np.array_equal(got[:, 1::4], exact_form[:, 1::4], equal_nan=True)
    if kind == "ordinary":
        assert not np.array_equal(got, exact_form)      # nothing is recomputed: the two forms round differently


# ---- the wide lane tile (16 pixels x 8 templates) needs a grid of 1536 waves: 96 images of 32 x 32 --------------------
def big_tile_case(C, seed):
    g = np.random.default_rng(seed)
    x = (g.normal(size=(96, C, 32, 32)) * 3 + 50).astype(np.float32)
    t = (g.normal(size=(128, C, 3, 3)) * 3 + 50).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    return x, t, w, dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])


@pytest.mark.parametrize("C", [5, 14, 27])      # one chunk; two chunks of 7 (odd number of rows); three chunks of 9
@pytest.mark.parametrize("func,algo", [("L2", None), ("L2", "direct"), ("L1", None)])
def test_similarity_wide_tile_row_loop(pkg, C, func, algo):
    """3 x 3 templates at stride 1 on the wide lane tile: the k loop walks (channel, dh) rows; sampled images
    against the oracle."""
    x, t, w, kw = big_tile_case(C, 51)
    got = pkg.similarity(dev(x), dev(t), dev(w), similarity_function=func, algo=algo, **kw).cpu().numpy()
    pick = [0, 37, 95]
    assert rel_err(got[pick], orc.similarity_fwd(x[pick], t, w, similarity_function=func, threads=8, **kw)) <= SIM_TOL


@pytest.mark.parametrize("kind", ["exact", "first_chunk_equal", "all_close", "negative_weights"])
def test_similarity_wide_tile_sqrt_weight_guard(pkg, kind):
    x, t, w, kw = big_tile_case(27, 52)
    g = np.random.default_rng(53)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    hits = []
    if kind in ("exact", "first_chunk_equal"):
        for m in range(0, 128, 5):
            b, i, j = int(g.integers(3)) * 47, int(g.integers(32)), int(g.integers(32))
            patch = xp[b, :, i:i + 3, j:j + 3]
            if kind == "exact":
                t[m] = patch
                hits.append((b, m, i, j))
            else:
                t[m, :9] = patch[:9]
    elif kind == "all_close":
        x = (g.normal(size=x.shape) + 1000).astype(np.float32)
        t = (g.normal(size=t.shape) + 1000).astype(np.float32)
    else:
        w[3::16] *= -1.0
    X, T, W = dev(x), dev(t), dev(w)
    got = pkg.similarity(X, T, W, **kw).cpu().numpy()
    exact_form = pkg.similarity(X, T, W, algo="direct", **kw).cpu().numpy()
    pick = [0, 47, 94]
    assert rel_err(got[pick], orc.similarity_fwd(x[pick], t, w, threads=8, **kw)) <= SIM_TOL
    assert rel_err(got, exact_form) <= SIM_TOL
    for b, m, i, j in hits:
        assert got[b, m, i, j] == 0.0
    if kind == "all_close":
        assert np.array_equal(got, exact_form)
    if kind == "negative_weights":
        assert np.array_equal(got[:, 3::16], exact_form[:, 3::16], equal_nan=True)


# ---- small maps: several images per wave, K split over the waves of a workgroup ---------------------------------------
SMALL_MAPS = [
    dict(shape=(9, 24, 7, 7), O=20, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),        # 4 images per wave, ragged batch
    dict(shape=(5, 10, 5, 6), O=9, blocks=[2, 3], strides=[1, 1], padding=[0, 1], out_of_bounds_value=0.5),
    dict(shape=(3, 37, 14, 14), O=40, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),      # one image per wave, K split only
    dict(shape=(2, 16, 13, 9), O=8, blocks=[3, 3], strides=[2, 2], padding=[1, 1]),        # stride 2
    dict(shape=(70, 6, 3, 3), O=5, blocks=[3, 3], strides=[1, 1], padding=[0, 0]),         # 1 x 1 outputs: 64 images per wave
    dict(shape=(64, 9, 7, 7), O=132, blocks=[3, 3], strides=[1, 1], padding=[1, 1]),       # 272 workgroups: four waves each
                                                                                           # (smaller grids above: eight)
]


@pytest.mark.parametrize("mode", [dict(similarity_function="L1"), dict(similarity_function="L2"),
                                  dict(similarity_function="L2", normalization_term=True),
                                  dict(similarity_function="L2", normalization_term=True, ignore_nan_input=True)])
@pytest.mark.parametrize("geom", SMALL_MAPS)
def test_similarity_small_maps(pkg, geom, mode):
    g = np.random.default_rng(61)
    shape, O = geom["shape"], geom["O"]
    kw = dict({k: v for k, v in geom.items() if k not in ("shape", "O")}, **mode)
    x = g.normal(size=shape).astype(np.float32)
    if mode.get("ignore_nan_input"):
        x[g.random(size=shape) < 0.1] = np.nan
        kw["out_of_bounds_value"] = float("nan")
    t = g.normal(size=(O, shape[1]) + tuple(geom["blocks"])).astype(np.float32)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(np.float32)
    X, T, W = dev(x), dev(t), dev(w)
    got = pkg.similarity(X, T, W, **kw)
    assert rel_err(got.cpu().numpy(), orc.similarity_fwd(x, t, w, **kw)) <= SIM_TOL
    assert same_bits(pkg.similarity_prepare(shape, T, W, **kw)(X), got)
    if not mode.get("normalization_term"):
        assert rel_err(pkg.similarity(X, T, W, algo="direct", **kw).cpu().numpy(), got.cpu().numpy()) <= SIM_TOL
