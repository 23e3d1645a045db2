"""Benchmark configuration 4 at its stated batch (512): the missing-data stack Similarity -> 4 x (MEX, 2x2 sum
pooling) -> MEX(10), run three ways (separate calls; MEX + pooling as one call; Similarity + MEX + pooling as one
call) and checked layer by layer against the CPU oracle on a sample of the 512 images.

The kernel variants the library picks depend on batch x region size, so only the full batch exercises the variants
the benchmark times.  Every layer is checked on the GPU's own previous activations (tolerances do not compound):
Similarity 1e-5, MEX 1e-4 (metric: tests/util.py:rel_err with the MEX shift as floor)."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import config4_stack, rel_err

pytestmark = pytest.mark.gpu

SIM_TOL = 1e-5
MEX_TOL = 1e-4
SAMPLE = [0, 1, 63, 64, 257, 300, 448, 511]      # first / last images, both sides of wave and workgroup boundaries
B = 512


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def pool2(y):
    b, c, h, w = y.shape
    p = y.reshape(b, c, h // 2, 2, w // 2, 2)
    return (p[:, :, :, 0, :, 0] + p[:, :, :, 0, :, 1]) + p[:, :, :, 1, :, 0] + p[:, :, :, 1, :, 1]


def mex_check(got, inp, off, n, kw, pooled=False):
    """`got` (sampled images) against the oracle on `inp` (the same images of the layer's input)."""
    offn = orc.normalize_offsets(off)
    want = orc.mex_fwd(inp, offn, n, **kw)
    shift = np.abs(orc.mex_fwd(inp, offn, n, **dict(kw, epsilon=math.inf)))
    if pooled:
        want, shift = pool2(want), pool2(shift)
    assert got.shape == want.shape
    err = rel_err(got, want, floor=shift)
    assert err <= MEX_TOL, err


@pytest.fixture(scope="module")
def stack():
    return config4_stack(B)


def test_config4_batch512_separate_calls(pkg, stack):
    x, t, w, skw, layers, (offl, nl, kwl) = stack
    cur = pkg.similarity(dev(x), dev(t), dev(w), **skw)
    got = cur.cpu().numpy()
    assert got.shape == (B, 32, 16, 16) and not np.isnan(got).any()
    assert rel_err(got[SAMPLE], orc.similarity_fwd(x[SAMPLE], t, w, **skw)) <= SIM_TOL
    for off, n, kw in layers:
        inp = cur.cpu().numpy()
        m = pkg.mex(cur, dev(off), n, normalize_offsets=True, **kw)
        mh = m.cpu().numpy()
        assert np.isfinite(mh).all()
        mex_check(mh[SAMPLE], inp[SAMPLE], off, n, kw)
        cur = pkg.sum_pooling(m, (2, 2))
        assert np.array_equal(cur.cpu().numpy(), pool2(mh))          # pooling: bit-exact, whole batch
    assert tuple(cur.shape) == (B, 512, 1, 1)
    out = pkg.mex(cur, dev(offl), nl, normalize_offsets=True, **kwl).cpu().numpy()
    assert out.shape == (B, 10, 1, 1)
    mex_check(out[SAMPLE], cur.cpu().numpy()[SAMPLE], offl, nl, kwl)
    # the classifier head is small enough for the oracle to see every image
    mex_check(out, cur.cpu().numpy(), offl, nl, kwl)


def test_config4_batch512_mex_sum_pool_calls(pkg, stack):
    x, t, w, skw, layers, (offl, nl, kwl) = stack
    cur = pkg.similarity(dev(x), dev(t), dev(w), **skw)
    for off, n, kw in layers:
        inp = cur.cpu().numpy()
        cur = pkg.mex_sum_pool(cur, dev(off), n, (2, 2), normalize_offsets=True, **kw)
        got = cur.cpu().numpy()
        assert np.isfinite(got).all()
        mex_check(got[SAMPLE], inp[SAMPLE], off, n, kw, pooled=True)
    out = pkg.mex(cur, dev(offl), nl, normalize_offsets=True, **kwl).cpu().numpy()
    mex_check(out, cur.cpu().numpy(), offl, nl, kwl)


def test_config4_batch512_similarity_mex_sum_pool_call(pkg, stack):
    x, t, w, skw, layers, (offl, nl, kwl) = stack
    off, n, kw = layers[0]
    cur = pkg.similarity_mex_sum_pool(dev(x), dev(t), dev(w), dev(off), n, (2, 2), similarity=skw,
                                      mex=dict(kw, normalize_offsets=True))
    got = cur.cpu().numpy()
    assert got.shape == (B, 64, 8, 8) and np.isfinite(got).all()
    # oracle: its own Similarity output feeds its MEX (the fused kernel's Similarity values are the term-by-term
    # kernel's, within 1e-5 of the oracle's; MEX is 1-Lipschitz in its input, so the MEX bar still applies with the
    # Similarity scale in the floor)
    s_ref = orc.similarity_fwd(x[SAMPLE], t, w, **skw)
    offn = orc.normalize_offsets(off)
    want = pool2(orc.mex_fwd(s_ref, offn, n, **kw))
    shift = pool2(np.abs(orc.mex_fwd(s_ref, offn, n, **dict(kw, epsilon=math.inf))))
    assert rel_err(got[SAMPLE], want, floor=shift) <= MEX_TOL
    # ... and bit for bit the separate calls with the term-by-term Similarity, over the whole batch
    s_dev = pkg.similarity(dev(x), dev(t), dev(w), algo="direct", **skw)
    two = pkg.mex_sum_pool(s_dev, dev(off), n, (2, 2), normalize_offsets=True, **kw)
    assert torch.equal(cur, two)
    for off, n, kw in layers[1:]:
        inp = cur.cpu().numpy()
        cur = pkg.mex_sum_pool(cur, dev(off), n, (2, 2), normalize_offsets=True, **kw)
        mex_check(cur.cpu().numpy()[SAMPLE], inp[SAMPLE], off, n, kw, pooled=True)
    out = pkg.mex(cur, dev(offl), nl, normalize_offsets=True, **kwl).cpu().numpy()
    mex_check(out, cur.cpu().numpy(), offl, nl, kwl)


def test_config4_batch_permutation_property(pkg, stack):
    """Size-independent property over all 512 images: permuting the images permutes the outputs, bit for bit
    (no result depends on an image's neighbours in the batch or on its place in a workgroup)."""
    x, t, w, skw, layers, (offl, nl, kwl) = stack

    def run(xx):
        cur = pkg.similarity(dev(xx), dev(t), dev(w), **skw)
        for off, n, kw in layers:
            cur = pkg.mex_sum_pool(cur, dev(off), n, (2, 2), normalize_offsets=True, **kw)
        return pkg.mex(cur, dev(offl), nl, normalize_offsets=True, **kwl).cpu().numpy()

    perm = np.random.default_rng(7).permutation(B)
    assert np.array_equal(run(x[perm]), run(x)[perm])
