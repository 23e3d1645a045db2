"""Bit-exact patch gathering on the GPU: operator calls whose output *is* the im2col matrix.

The library never materialises the reference's column matrix (src/utils/im2col.cpp:247-280); its kernels gather patch
elements while staging tiles.  These tests choose parameters that make an operator copy one patch element to each
output, so that the whole output tensor must equal the oracle's im2col_3d, bit for bit:

  * Similarity L1 with zero templates and a one-hot unit weight per template: out[b, k, h, w] = -|patch(b,h,w)[k]|
    (the other terms are -0 * |x| = -0, which leaves the sum unchanged).  With NaN as the out-of-bounds value the
    zero-weight terms of a padded patch are NaN, so the NaN positions of the output are exactly the patches that touch
    padding - the reference's NaN positions.
  * MEX with epsilon = +inf (max) / -inf (min) and offsets 0 at one patch element and -inf / +inf at the others:
    out[b, k*Cc + c, h, w] = patch(b,c,h,w)[k] + 0.

Input values are distinct per element (1 + index * 2^-20, exact in fp32), so any wrong index shows."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def distinct(shape, sign=False, seed=0):
    n = int(np.prod(shape))
    assert n <= 1 << 20
    v = (1.0 + np.arange(n, dtype=np.float64) / (1 << 20)).astype(np.float32)
    v = v[np.random.default_rng(seed).permutation(n)].reshape(shape)
    if sign:
        v = v * np.where(np.random.default_rng(seed + 1).random(size=shape) < 0.5, -1.0, 1.0).astype(np.float32)
    return v


SIM_CASES = [
    dict(shape=(2, 3, 11, 13), blocks=[3, 3], strides=[1, 1], padding=[1, 1]),
    dict(shape=(2, 3, 11, 13), blocks=[3, 2], strides=[2, 3], padding=[0, 1]),
    dict(shape=(3, 1, 28, 28), blocks=[2, 2], strides=[2, 2], padding=[2, 2]),          # padding beyond the block
    dict(shape=(2, 2, 5, 5), blocks=[2, 2], strides=[4, 5], padding=[3, 3]),            # patches entirely in padding
    dict(shape=(1, 5, 9, 70), blocks=[5, 5], strides=[3, 3], padding=[2, 2]),
    dict(shape=(16, 4, 48, 64), blocks=[3, 3], strides=[1, 1], padding=[1, 1]),         # 16 x 8 lane tile, 36 templates
    dict(shape=(2, 40, 6, 6), blocks=[2, 2], strides=[1, 1], padding=[1, 1]),           # several channel chunks
    dict(shape=(1, 2, 4, 700), blocks=[3, 3], strides=[1, 1], padding=[1, 1]),          # rows beyond the LDS tile: gather kernel
    dict(shape=(2, 1, 7, 7), blocks=[7, 7], strides=[1, 1], padding=[0, 0]),            # one output pixel
]


@pytest.mark.parametrize("oob", [0.75, float("nan")])
@pytest.mark.parametrize("case", SIM_CASES)
def test_similarity_output_is_the_im2col_matrix(pkg, case, oob):
    B, Cc, H, W = case["shape"]
    bh, bw = case["blocks"]
    K = Cc * bh * bw
    x = distinct(case["shape"], sign=True)
    t = np.zeros((K, Cc, bh, bw), np.float32)
    w = np.eye(K, dtype=np.float32).reshape(K, Cc, bh, bw)
    kw = dict(similarity_function="L1", blocks=case["blocks"], strides=case["strides"], padding=case["padding"],
              out_of_bounds_value=oob)
    got = pkg.similarity(dev(x), dev(t), dev(w), **kw).cpu().numpy()
    for b in range(B):
        col = orc.im2col_3d(x[b], [Cc, bh, bw], [0] + case["padding"], [Cc] + case["strides"], True, oob)[:, 0]
        want = -np.abs(col)
        if math.isnan(oob):
            want[:, np.isnan(col).any(axis=0)] = np.nan     # a padded patch: 0 * NaN in every template's sum
        assert got[b].shape == want.shape
        assert np.array_equal(np.isnan(got[b]), np.isnan(want)), "NaN positions differ (image %d)" % b
        ok = ~np.isnan(want)
        assert np.array_equal(got[b][ok].view(np.uint32), want[ok].view(np.uint32)), "gathered values differ (image %d)" % b


@pytest.mark.parametrize("case", SIM_CASES[:5])
def test_similarity_ignore_nan_marks_exactly_the_padded_elements(pkg, case):
    """Normalized L2 with ignore_nan_input and NaN padding: with zero templates, weights w_k = one-hot and fudge 1,
    template k's output is 0.5 * sum over the non-NaN patch elements j of (-w_kj x_j^2 - log(2 pi) + log(w_kj + 1)):
    the count of in-image elements and the one gathered value, both exactly determined by the im2col matrix."""
    B, Cc, H, W = case["shape"]
    bh, bw = case["blocks"]
    K = Cc * bh * bw
    x = distinct(case["shape"], sign=True)
    t = np.zeros((K, Cc, bh, bw), np.float32)
    w = np.eye(K, dtype=np.float32).reshape(K, Cc, bh, bw)
    kw = dict(blocks=case["blocks"], strides=case["strides"], padding=case["padding"], normalization_term=True,
              ignore_nan_input=True, out_of_bounds_value=float("nan"), normalization_term_fudge=1.0)
    got = pkg.similarity(dev(x), dev(t), dev(w), **kw).cpu().numpy()
    want = orc.similarity_fwd(x, t, w, **kw)
    assert not np.isnan(got).any()
    # patches entirely in padding give exactly +0.0
    for b in range(B):
        col = orc.im2col_3d(x[b], [Cc, bh, bw], [0] + case["padding"], [Cc] + case["strides"], True, float("nan"))[:, 0]
        empty = np.isnan(col).all(axis=0)
        assert np.all(got[b][:, empty] == 0.0) and not np.signbit(got[b][:, empty]).any()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)


MEX_CASES = [
    dict(im=(3, 3, 10, 13), kw=dict(blocks=[2, 2, 2], padding=[1, 1, 1], strides=[1, 3, 2], blocks_round_down=False)),
    dict(im=(3, 3, 10, 13), kw=dict(blocks=[2, 2, 2], padding=[1, 1, 1], strides=[1, 3, 2], blocks_round_down=True,
                                    use_unshared_regions=False, shared_offset_region=[2, 2, 3])),
    dict(im=(2, 1, 30, 31), kw=dict(blocks=[1, 3, 3], padding=[0, 1, 1], strides=[1, 2, 2])),
    dict(im=(2, 2, 9, 9), kw=dict(blocks=[1, 2, 2], padding=[0, 3, 3], strides=[1, 4, 5])),      # padding beyond the block
    dict(im=(6, 8, 40, 40), kw=dict(blocks=[8, 3, 3], strides=[8, 1, 1], padding=[0, 1, 1],
                                    unshared_offset_region=[2])),                            # several pixels per lane
    dict(im=(40, 96, 2, 2), kw=dict(blocks=[96, 1, 1], strides=[96, 1, 1], unshared_offset_region=[2])),   # lanes along k
    dict(im=(20, 64, 1, 1), kw=dict(blocks=[64, 1, 1], strides=[64, 1, 1], shared_offset_region=[1])),     # wave per pixel
    dict(im=(2, 40, 3, 3), kw=dict(blocks=[20, 2, 2], strides=[10, 1, 1], padding=[5, 0, 0],
                                   unshared_offset_region=[1, 2, 2])),                         # channel padding, 3-D blocks
    dict(im=(9, 32, 16, 16), kw=dict(blocks=[32, 1, 1], strides=[32, 1, 1], unshared_offset_region=[2])),  # 1x1 shortcut
]


@pytest.mark.parametrize("eps", [math.inf, -math.inf])
@pytest.mark.parametrize("case", MEX_CASES)
def test_mex_output_is_the_im2col_matrix(pkg, case, eps):
    kw = dict(case["kw"], epsilon=eps, blocks_out_of_bounds_value=0.75)
    im = case["im"]
    bc, bh, bw = kw["blocks"]
    K = bc * bh * bw
    d = orc.mex_dims(orc.mex_args(im, K, **kw))
    x = distinct(im, sign=True)
    off = np.full((d.num_regions, K, K), -eps, np.float32)
    off[:, np.arange(K), np.arange(K)] = 0.0
    got = pkg.mex(dev(x), dev(off.reshape((d.num_regions, K, bc, bh, bw))), K, **kw).cpu().numpy()
    assert got.shape == (im[0], K * d.channels_out, d.height_out, d.width_out)
    pad, strides = kw.get("padding", [0, 0, 0]), kw["strides"]
    for b in range(im[0]):
        col = orc.im2col_3d(x[b], [bc, bh, bw], pad, strides, kw.get("blocks_round_down", True), 0.75)
        assert np.array_equal(got[b].reshape(col.shape).view(np.uint32), col.view(np.uint32)), "image %d" % b
