"""Pins the CPU oracle (oracle/simnets_oracle.c) before anything is compared with it.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * the reference's own header-only templates compiled into oracle/_ref (bit-exact);
  * known-answer shapes held by the reference's Keras tests
    (python/simnets/test/keras/__init__.py:46-55, :110-119) and the 45*45-region sanity case
    (python/simnets/test/__init__.py:213);
  * library routines on special cases: torch unfold, cdist, logsumexp, scipy logsumexp;
  * fast path vs brute-force path, the comparison the reference's tests make
    (python/simnets/test/__init__.py:19-53, :226-258) but at fp64 and tight tolerance.
"""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F
from scipy.special import logsumexp

from oracle import oracle as orc

needs_ref = pytest.mark.skipif(orc.ref() is None, reason="oracle/_ref was not built (no reference checkout)")


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------------------------------------
# dimension arithmetic
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("num_instances,padding,strides,blocks,in_shape,out_shape", [
    (10, [0, 1], [1, 1], [2, 2], (3, 10, 13), (10, 9, 14)),
    (10, [1, 1], [3, 2], [2, 2], (3, 10, 13), (10, 4, 7)),
    (2, [1, 1], [3, 2], [2, 2], (1, 10, 13), (2, 4, 7)),
])
def test_similarity_known_answer_shapes(num_instances, padding, strides, blocks, in_shape, out_shape):
    a = orc.similarity_args((1,) + in_shape, num_instances, "L1", blocks, strides, padding)
    assert (num_instances,) + orc.similarity_out_dims(a) == out_shape


@pytest.mark.parametrize("num_instances,padding,strides,blocks,in_shape,out_shape", [
    (10, [1, 0, 1], [1, 1, 1], [1, 2, 2], (3, 10, 13), (50, 9, 14)),
    (10, [2, 1, 1], [1, 3, 2], [1, 2, 2], (3, 10, 13), (70, 5, 8)),
    (2, [1, 1, 1], [1, 3, 2], [1, 2, 2], (1, 10, 13), (6, 5, 8)),
])
def test_mex_known_answer_shapes(num_instances, padding, strides, blocks, in_shape, out_shape):
    a = orc.mex_args((1,) + in_shape, num_instances, True, padding, strides, blocks, 2.0, 1.0,
                     blocks_round_down=False, use_unshared_regions=False, shared_offset_region=[2])
    d = orc.mex_dims(a)
    assert (d.channels_out_total, d.height_out, d.width_out) == out_shape


def test_mex_regions_known_cases():
    # fully unshared default on the sanity geometry: every output pixel is its own region
    d = orc.mex_dims(orc.mex_args((5, 1, 90, 90), 3, blocks=[1, 3, 3], padding=[0, 1, 1], strides=[1, 2, 2]))
    assert (d.height_out, d.width_out, d.num_regions, d.region_size) == (45, 45, 2025, 1)
    # 16x16 map, unshared [2]: 2x2 interleaved regions of 8x8 pixels each
    d = orc.mex_dims(orc.mex_args((64, 32, 16, 16), 64, True, [0, 0, 0], [32, 1, 1], [32, 1, 1],
                                  unshared_offset_region=[2]))
    assert (d.offsets_c, d.offsets_h, d.offsets_w) == (1, 2, 2)
    assert (d.shared_region_c, d.shared_region_h, d.shared_region_w) == (1, 8, 8)
    assert (d.num_regions, d.region_size, d.M, d.K, d.N, d.is_1x1) == (4, 64, 64, 32, 256, 1)
    # shared [1] at 1x1 spatial: a single region
    d = orc.mex_dims(orc.mex_args((2, 512, 1, 1), 10, True, [0, 0, 0], [512, 1, 1], [512, 1, 1],
                                  use_unshared_regions=True, shared_offset_region=[1]))
    assert d.num_regions == 1


@pytest.mark.parametrize("unshared", [True, False])
@pytest.mark.parametrize("spec", [[2], [3], [1, 5, 4], [-1], [2, 7, 1]])
@pytest.mark.parametrize("hw", [(41, 40), (40, 40), (7, 5)])
def test_mex_region_tiling_invariants(unshared, spec, hw):
    a = orc.mex_args((1, 3, hw[0], hw[1]), 2, True, [0, 1, 0], [1, 1, 1], [1, 3, 3],
                     use_unshared_regions=unshared, shared_offset_region=spec, unshared_offset_region=spec)
    d = orc.mex_dims(a)
    assert d.num_regions == d.offsets_c * d.offsets_h * d.offsets_w
    assert d.region_size == d.shared_region_c * d.shared_region_h * d.shared_region_w
    assert d.num_regions * d.region_size >= d.N
    for full, n_off, reg in ((d.channels_out, d.offsets_c, d.shared_region_c),
                             (d.height_out, d.offsets_h, d.shared_region_h),
                             (d.width_out, d.offsets_w, d.shared_region_w)):
        assert n_off * reg >= full and (n_off - 1) * reg < full or unshared
        if full % n_off == 0 and full % reg == 0:
            assert n_off * reg == full


def test_round_up_uses_float_ceil():
    # (I + 2p - b) / s with ceil in float: 13/2 -> 7 (+1); exact multiples stay
    assert orc.dimension_out_size(13, 1, 2, 2, False) == 8
    assert orc.dimension_out_size(10, 1, 2, 3, False) == 5
    assert orc.dimension_out_size(10, 1, 2, 3, True) == 4
    assert orc.dimension_out_size(12, 0, 2, 2, False) == orc.dimension_out_size(12, 0, 2, 2, True) == 6


def test_invalid_arguments_are_rejected():
    with pytest.raises(ValueError):
        orc.similarity_out_dims(orc.similarity_args((1, 1, 4, 4), 1, "L1", normalization_term=True))
    with pytest.raises(ValueError):
        orc.similarity_out_dims(orc.similarity_args((1, 1, 4, 4), 1, "L2", ignore_nan_input=True))
    with pytest.raises(ValueError):
        orc.mex_dims(orc.mex_args((1, 2, 4, 4), 0))
    with pytest.raises(ValueError):
        orc.mex_dims(orc.mex_args((1, 2, 4, 4), 1, blocks=[3, 1, 1]))
    with pytest.raises(ValueError):
        orc.mex_dims(orc.mex_args((1, 2, 4, 4), 1, strides=[1, 1]))


# ---------------------------------------------------------------------------------------------
# building blocks against the reference's own compiled headers (bit-exact)
# ---------------------------------------------------------------------------------------------
@needs_ref
def test_padded_output_size_matches_reference():
    for M, N in [(32, 4), (1, 1), (16, 16), (17, 33), (128, 576)]:
        assert orc.lib().so_ggemm_padded_output_size(M, N) == orc.ref().ref_ggemm_padded_output_size(M, N)
    assert orc.lib().so_ggemm_padded_output_size(32, 4) == 384


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_ggemm_similarity_bit_exact_vs_reference(dtype, mode):
    g = rng(100 + mode)
    M, N, K = 7, 45, 29
    A = np.empty((M, K, 2), dtype=dtype)
    A[..., 0] = g.normal(size=(M, K))
    A[..., 1] = np.abs(g.normal(size=(M, K))) + 0.01
    Bm = g.normal(size=(K, N)).astype(dtype)
    if mode == 3:
        Bm[g.random(size=Bm.shape) < 0.3] = np.nan
        Bm[:, 5] = np.nan
    so = orc.ggemm_similarity(mode, A, Bm, M, N, K, 0.001, "oracle")
    rf = orc.ggemm_similarity(mode, A, Bm, M, N, K, 0.001, "ref")
    assert np.array_equal(so.view(np.uint8), rf.view(np.uint8))
    if mode == 3:
        assert np.all(so[:, 5] == 0) and not np.isnan(so).any()


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("softmax", [False, True])
@pytest.mark.parametrize("eps", [1.0, -1.0, 2.5, -0.3, math.inf, -math.inf])
def test_mex_forward_bit_exact_vs_reference(dtype, softmax, eps):
    g = rng(7)
    R, M, N, K = 3, 5, 19, 11
    off = g.normal(size=(R, M, K)).astype(dtype)
    inp = g.normal(size=(R, K, N)).astype(dtype) * 3
    so = orc.mex_forward(off, inp, M, N, K, softmax, eps, R, "oracle")
    rf = orc.mex_forward(off, inp, M, N, K, softmax, eps, R, "ref")
    assert np.array_equal(so.view(np.uint8), rf.view(np.uint8))


@needs_ref
@pytest.mark.parametrize("unshared", [False, True])
@pytest.mark.parametrize("geom", [  # (C,H,W) (groups c,h,w) (steps c,h,w)
    ((1, 16, 16), (1, 2, 2), (1, 8, 8)),
    ((3, 41, 40), (1, 14, 14), (3, 3, 3)),  # ragged rows: 14 * 3 = 42 > 41
    ((3, 9, 10), (2, 3, 4), (2, 3, 3)),     # ragged in every dimension
])
def test_split_patches_bit_exact_vs_reference(unshared, geom):
    (Cc, H, W), (Cg, Hg, Wg), (Cs, Hs, Ws) = geom
    N, Dim = Cc * H * W, 6
    g = rng(3)
    src = g.normal(size=(Dim, N)).astype(np.float32)
    size = Cg * Hg * Wg * Cs * Hs * Ws * Dim
    out_so = np.full(size, -7.0, np.float32)
    out_rf = out_so.copy()
    orc.split_patches(False, src, out_so, N, Dim, W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared, "oracle")
    orc.split_patches(False, src, out_rf, N, Dim, W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared, "ref")
    assert np.array_equal(out_so, out_rf)
    # every source element lands exactly once
    assert np.array_equal(np.sort(out_so[out_so != -7.0]), np.sort(src.ravel()))
    back_so = np.zeros_like(src)
    back_rf = np.zeros_like(src)
    orc.split_patches(True, back_so, out_so, N, Dim, W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared, "oracle")
    orc.split_patches(True, back_rf, out_rf, N, Dim, W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared, "ref")
    assert np.array_equal(back_so, back_rf) and np.array_equal(back_so, src)


# ---------------------------------------------------------------------------------------------
# im2col_3d against library unfold and against pad-then-slice
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("blocks,strides,padding", [
    ((3, 3), (1, 1), (1, 1)), ((2, 2), (2, 2), (2, 2)), ((3, 2), (1, 2), (0, 1)), ((1, 1), (1, 1), (0, 0)),
    ((5, 3), (2, 3), (2, 0)),
])
def test_im2col_matches_torch_unfold(blocks, strides, padding):
    g = rng(11)
    Cc, H, W = 3, 11, 9
    im = g.normal(size=(Cc, H, W)).astype(np.float32)
    col = orc.im2col_3d(im, (Cc,) + blocks, (0,) + padding, (Cc,) + strides, True, 0.0)
    unf = F.unfold(torch.from_numpy(im)[None], kernel_size=blocks, padding=padding, stride=strides)[0].numpy()
    assert col.shape[1] == 1
    assert np.array_equal(col.reshape(unf.shape), unf)


@pytest.mark.parametrize("round_down", [True, False])
@pytest.mark.parametrize("patch,pad,stride", [
    ((1, 3, 3), (0, 1, 1), (1, 2, 2)), ((2, 2, 3), (1, 0, 2), (1, 3, 2)), ((3, 1, 1), (0, 0, 0), (3, 1, 1)),
    ((1, 2, 2), (2, 1, 1), (1, 3, 2)),
])
def test_im2col_3d_matches_pad_then_slice(round_down, patch, pad, stride):
    g = rng(12)
    Cc, H, W = 3, 10, 13
    im = g.normal(size=(Cc, H, W))
    oob = np.nan
    col = orc.im2col_3d(im, patch, pad, stride, round_down, oob)
    _, cc, hc, wc = col.shape
    # pad generously on the high side: with round-up sizing the last patch may overhang
    hi = [p + s + b for p, s, b in zip(pad, stride, patch)]
    padded = np.pad(im, [(pad[0], hi[0]), (pad[1], hi[1]), (pad[2], hi[2])], constant_values=oob)
    exp = np.empty_like(col)
    for dc, dh, dw in itertools.product(range(patch[0]), range(patch[1]), range(patch[2])):
        p = (dc * patch[1] + dh) * patch[2] + dw
        exp[p] = padded[dc:dc + cc * stride[0]:stride[0], dh:dh + hc * stride[1]:stride[1],
                        dw:dw + wc * stride[2]:stride[2]]
    assert np.array_equal(np.isnan(col), np.isnan(exp))
    assert np.array_equal(np.nan_to_num(col), np.nan_to_num(exp))


def test_im2col_nan_border_count_of_the_28x28_geometry():
    # 28x28, block 2, stride 2, pad 2 -> 16x16 outputs; the outer ring of 60 outputs sees only padding
    im = np.zeros((1, 28, 28), np.float32)
    col = orc.im2col_3d(im, (1, 2, 2), (0, 2, 2), (1, 2, 2), True, np.nan)
    assert col.shape == (4, 1, 16, 16)
    assert int(np.isnan(col).sum()) == 240
    assert int(np.isnan(col).all(axis=0).sum()) == 60


# ---------------------------------------------------------------------------------------------
# Similarity: fast path vs brute force, and special cases that are library routines
# ---------------------------------------------------------------------------------------------
def _sim_inputs(g, shape, O, blocks, dtype):
    x = g.normal(size=shape).astype(dtype)
    t = g.normal(size=(O, shape[1]) + tuple(blocks)).astype(dtype)
    w = (np.abs(g.normal(size=t.shape)) + 0.05).astype(dtype)
    return x, t, w


@pytest.mark.parametrize("strides", [(1, 1), (2, 1), (2, 2)])
@pytest.mark.parametrize("blocks", [(1, 1), (3, 1), (3, 3)])
@pytest.mark.parametrize("same", [True, False])
@pytest.mark.parametrize("shape", [(1, 1, 14, 12), (2, 3, 14, 12)])
def test_similarity_fast_vs_bruteforce_dimensions(strides, blocks, same, shape):
    g = rng(21)
    x, t, w = _sim_inputs(g, shape, 2, blocks, np.float64)
    kw = dict(blocks=blocks, strides=strides, padding=[b // 2 for b in blocks] if same else [0, 0])
    np.testing.assert_allclose(orc.similarity_fwd(x, t, w, **kw), orc.similarity_ref(x, t, w, **kw),
                               rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 2e-5)])
@pytest.mark.parametrize("func,norm,ign", [("L2", False, False), ("L2", True, False), ("L2", True, True),
                                           ("L1", False, False)])
def test_similarity_fast_vs_bruteforce_params(dtype, tol, func, norm, ign):
    g = rng(22)
    x, t, w = _sim_inputs(g, (3, 3, 30, 30), 4, (3, 3), dtype)
    if ign:
        x[g.random(size=x.shape) < 0.2] = np.nan
    kw = dict(similarity_function=func, blocks=(3, 3), strides=(2, 2), padding=(1, 1), normalization_term=norm,
              ignore_nan_input=ign, out_of_bounds_value=np.nan if ign else 0.0)
    fast = orc.similarity_fwd(x, t, w, **kw)
    brute = orc.similarity_ref(x, t, w, **kw)
    assert not np.isnan(fast).any()
    np.testing.assert_allclose(fast, brute, rtol=tol, atol=tol * np.abs(brute).max())


def test_similarity_unit_weights_reduce_to_cdist():
    g = rng(23)
    x = g.normal(size=(2, 3, 9, 8))
    t = g.normal(size=(5, 3, 3, 2))
    w = np.ones_like(t)
    kw = dict(blocks=(3, 2), strides=(1, 2), padding=(1, 0))
    patches = F.unfold(torch.from_numpy(x), (3, 2), padding=(1, 0), stride=(1, 2)).transpose(1, 2)  # B,N,K
    tt = torch.from_numpy(t).reshape(5, -1)[None].expand(2, -1, -1).contiguous()
    for func, p in (("L2", 2), ("L1", 1)):
        d = torch.cdist(patches, tt, p=p)  # B,N,O
        exp = -(d ** 2 if p == 2 else d).transpose(1, 2).numpy()
        got = orc.similarity_fwd(x, t, w, similarity_function=func, **kw)
        np.testing.assert_allclose(got.reshape(exp.shape), exp, rtol=1e-10, atol=1e-10)


def test_similarity_weights_are_linear_in_the_output():
    # sum_k w_k phi_k is linear in w: f(w1 + w2) == f(w1) + f(w2); catches a dropped or squared weight
    g = rng(24)
    x, t, w1 = _sim_inputs(g, (1, 2, 7, 7), 3, (2, 2), np.float64)
    w2 = np.abs(g.normal(size=w1.shape))
    for func in ("L1", "L2"):
        kw = dict(similarity_function=func, blocks=(2, 2), strides=(1, 1), padding=(0, 0))
        np.testing.assert_allclose(orc.similarity_fwd(x, t, w1 + w2, **kw),
                                   orc.similarity_fwd(x, t, w1, **kw) + orc.similarity_fwd(x, t, w2, **kw),
                                   rtol=1e-12, atol=1e-12)


def test_similarity_normalized_is_a_gaussian_log_density():
    # with normalization the output is sum_k log N(x_k; t_k, 1/w_k) (up to the fudge inside the log)
    g = rng(25)
    x, t, w = _sim_inputs(g, (2, 2, 6, 6), 3, (3, 3), np.float64)
    fudge = 1e-3
    got = orc.similarity_fwd(x, t, w, blocks=(3, 3), strides=(1, 1), padding=(0, 0), normalization_term=True,
                             normalization_term_fudge=fudge)
    patches = F.unfold(torch.from_numpy(x), (3, 3)).numpy()  # B,K,N
    tt, ww = t.reshape(3, -1), w.reshape(3, -1)
    exp = np.zeros((2, 3, patches.shape[2]))
    for o in range(3):
        d = patches - tt[o][None, :, None]
        exp[:, o] = (-0.5 * ww[o][None, :, None] * d * d + 0.5 * np.log(np.float32(fudge) + ww[o])[None, :, None]
                     - 0.5 * math.log(2 * math.pi)).sum(axis=1)
    np.testing.assert_allclose(got.reshape(exp.shape), exp, rtol=1e-10, atol=1e-10)


def test_similarity_ignore_nan_marginalises_and_all_padding_patches_give_zero():
    g = rng(26)
    x = g.uniform(-0.5, 0.5, size=(3, 1, 28, 28)).astype(np.float32)
    t = (g.normal(size=(32, 1, 2, 2)) * 0.1).astype(np.float32)
    w = g.uniform(0.5, 1.5, size=t.shape).astype(np.float32)
    kw = dict(blocks=(2, 2), strides=(2, 2), padding=(2, 2), normalization_term=True, ignore_nan_input=True,
              out_of_bounds_value=np.nan)
    out = orc.similarity_fwd(x, t, w, **kw)
    assert out.shape == (3, 32, 16, 16) and not np.isnan(out).any()
    ring = np.ones((16, 16), bool)
    ring[1:-1, 1:-1] = False
    assert ring.sum() == 60
    assert np.all(out[:, :, ring] == 0.0) and not np.signbit(out[:, :, ring]).any()
    assert np.all(out[:, :, ~ring] != 0.0)
    # NaN pixels drop out term by term: NaN-ing one pixel removes exactly its summand
    x2 = x.copy()
    x2[0, 0, 6, 6] = np.nan  # belongs to output (4,4), patch position (0,0)
    out2 = orc.similarity_fwd(x2, t, w, **kw)
    changed = np.argwhere(out2 != out)
    assert {tuple(c[[0, 2, 3]]) for c in changed} == {(0, 4, 4)}
    term = 0.5 * (-w[:, 0, 0, 0].astype(np.float64) * (t[:, 0, 0, 0].astype(np.float64) - x[0, 0, 6, 6]) ** 2
                  - math.log(2 * math.pi) + np.log(w[:, 0, 0, 0].astype(np.float64) + 0.001))
    np.testing.assert_allclose(out[0, :, 4, 4] - out2[0, :, 4, 4], term, rtol=1e-4, atol=1e-5)


def test_similarity_normalization_constant_modes():
    g = rng(27)
    x, t, w = _sim_inputs(g, (3, 2, 6, 6), 2, (3, 3), np.float32)
    kw = dict(blocks=(3, 3), strides=(1, 1), padding=(0, 0), normalization_term=True)
    once = orc.similarity_fwd(x, t, w, **kw)
    every = orc.similarity_fwd(x, t, w, norm_const_every_iteration=True, **kw)
    brute = orc.similarity_ref(x, t, w, **kw)
    K = 2 * 3 * 3
    c = np.float32(-0.5 * K * math.log(2 * math.pi))
    np.testing.assert_allclose(once, brute, rtol=2e-5, atol=2e-5)
    assert np.array_equal(every[2], once[2])  # the last image gets it exactly once either way
    for n in range(3):
        np.testing.assert_allclose(every[n] - once[n], (3 - n - 1) * c, rtol=1e-5, atol=1e-4)


def test_similarity_threads_do_not_change_results():
    g = rng(28)
    x, t, w = _sim_inputs(g, (5, 2, 9, 9), 3, (3, 3), np.float32)
    kw = dict(blocks=(3, 3), strides=(1, 1), padding=(1, 1))
    assert np.array_equal(orc.similarity_fwd(x, t, w, **kw), orc.similarity_fwd(x, t, w, threads=3, **kw))


# ---------------------------------------------------------------------------------------------
# MEX: fast path vs brute force over the reference's test matrix, and library special cases
# ---------------------------------------------------------------------------------------------
def _mex_case(g, im_dims, num_instances, dtype, **kw):
    a = orc.mex_args(im_dims, num_instances, **kw)
    d = orc.mex_dims(a)
    x = g.normal(size=im_dims).astype(dtype)
    off = g.normal(size=(d.num_regions, num_instances) + tuple(kw["blocks"])).astype(dtype)
    return x, off, d


@pytest.mark.parametrize("unshared,spec", [(False, [2]), (False, [3]), (True, [1, 5, 4]), (True, [2])])
@pytest.mark.parametrize("strides", [[1, 1, 1], [1, 4, 1], [1, 4, 4]])
@pytest.mark.parametrize("blocks", [[1, 1, 3], [1, 3, 3]])
@pytest.mark.parametrize("im_dims", [(1, 1, 41, 40), (2, 3, 40, 40), (2, 3, 41, 40)])
def test_mex_fast_vs_bruteforce_region_matrix(unshared, spec, strides, blocks, im_dims):
    g = rng(31)
    kw = dict(softmax_mode=True, padding=[0, 1, 0], strides=strides, blocks=blocks, use_unshared_regions=unshared,
              shared_offset_region=spec if not unshared else [2], unshared_offset_region=spec if unshared else [1])
    x, off, d = _mex_case(g, im_dims, 2, np.float64, **kw)
    np.testing.assert_allclose(orc.mex_fwd(x, off, 2, **kw), orc.mex_ref(x, off, 2, **kw), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 1e-5)])
@pytest.mark.parametrize("eps", [1.0, 2.0, -1.5, math.inf, -math.inf])
@pytest.mark.parametrize("softmax", [True, False])
def test_mex_fast_vs_bruteforce_sanity_geometry(dtype, tol, eps, softmax):
    g = rng(32)
    kw = dict(softmax_mode=softmax, blocks=[1, 3, 3], padding=[0, 1, 1], strides=[1, 2, 2], epsilon=eps)
    x, off, d = _mex_case(g, (2, 1, 30, 30), 3, dtype, **kw)
    assert d.num_regions == 15 * 15
    np.testing.assert_allclose(orc.mex_fwd(x, off, 3, **kw), orc.mex_ref(x, off, 3, **kw), rtol=tol, atol=tol)


@pytest.mark.parametrize("round_down", [True, False])
def test_mex_fast_vs_bruteforce_3d_blocks_with_channel_padding(round_down):
    g = rng(33)
    kw = dict(softmax_mode=False, blocks=[2, 2, 2], padding=[1, 1, 1], strides=[1, 3, 2], epsilon=0.7,
              blocks_out_of_bounds_value=-1.5, blocks_round_down=round_down, use_unshared_regions=False,
              shared_offset_region=[2, 2, 3])
    x, off, d = _mex_case(g, (2, 3, 10, 13), 4, np.float64, **kw)
    np.testing.assert_allclose(orc.mex_fwd(x, off, 4, **kw), orc.mex_ref(x, off, 4, **kw), rtol=1e-12, atol=1e-12)


def test_mex_1x1_single_region_is_logsumexp():
    g = rng(34)
    B, Cc, H, W, M = 3, 8, 4, 5, 6
    x = g.normal(size=(B, Cc, H, W))
    off = g.normal(size=(1, M, Cc, 1, 1))
    kw = dict(blocks=[Cc, 1, 1], strides=[Cc, 1, 1], use_unshared_regions=False, shared_offset_region=[-1])
    v = torch.from_numpy(x)[:, None] + torch.from_numpy(off.reshape(M, Cc))[None, :, :, None, None]  # B,M,C,H,W
    for eps in (1.0, 3.0, -2.0):
        exp_soft = (torch.logsumexp(eps * v, dim=2) / eps).numpy()
        np.testing.assert_allclose(orc.mex_fwd(x, off, M, softmax_mode=True, epsilon=eps, **kw), exp_soft,
                                   rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(orc.mex_fwd(x, off, M, softmax_mode=False, epsilon=eps, **kw),
                                   exp_soft - math.log(Cc) / eps, rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(orc.mex_fwd(x, off, M, epsilon=math.inf, **kw), v.max(dim=2).values.numpy())
    np.testing.assert_array_equal(orc.mex_fwd(x, off, M, epsilon=-math.inf, **kw), v.min(dim=2).values.numpy())


def test_mex_unshared_regions_pick_offsets_by_pixel_parity():
    # unshared [2] on an even map: pixel (h, w) uses region (h % 2) * 2 + (w % 2)
    g = rng(35)
    B, Cc, H, W, M = 2, 4, 6, 6, 3
    x = g.normal(size=(B, Cc, H, W))
    off = g.normal(size=(4, M, Cc, 1, 1))
    got = orc.mex_fwd(x, off, M, softmax_mode=True, blocks=[Cc, 1, 1], strides=[Cc, 1, 1], unshared_offset_region=[2])
    hh, ww = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
    region = (hh % 2) * 2 + (ww % 2)
    o = off.reshape(4, M, Cc)[region]  # H,W,M,C
    exp = logsumexp(x[:, None].transpose(0, 1, 3, 4, 2) + o.transpose(2, 0, 1, 3)[None], axis=-1)
    np.testing.assert_allclose(got, exp, rtol=1e-12, atol=1e-12)


def test_mex_output_channel_order_is_instance_major():
    # output channel = instance * channels_out + c  (mex_kernel_cpu.cpp:113-115)
    g = rng(36)
    x = g.normal(size=(1, 4, 3, 3))
    off = np.zeros((1, 2, 1, 1, 1))
    off[0, 1] = 10.0
    got = orc.mex_fwd(x, off, 2, blocks=[1, 1, 1], strides=[1, 1, 1], softmax_mode=True, use_unshared_regions=False)
    assert got.shape == (1, 8, 3, 3)
    np.testing.assert_allclose(got[0, :4], x[0], atol=1e-12)
    np.testing.assert_allclose(got[0, 4:], x[0] + 10.0, atol=1e-12)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_normalize_offsets_is_logsumexp_normalisation(dtype):
    g = rng(37)
    off = (g.normal(size=(4, 6, 8, 2, 1)) * 3).astype(dtype)
    got = orc.normalize_offsets(off)
    flat = off.reshape(24, -1).astype(np.float64)
    exp = (flat - logsumexp(flat, axis=1, keepdims=True)).reshape(off.shape)
    tol = 1e-12 if dtype == np.float64 else 2e-6
    np.testing.assert_allclose(got, exp, rtol=tol, atol=tol)
    np.testing.assert_allclose(np.exp(got.reshape(24, -1).astype(np.float64)).sum(axis=1), 1.0, rtol=10 * tol)


# ---------------------------------------------------------------------------------------------
# backward operators.  The reference's own tests compare them with numeric differentiation of the
# forward op (python/simnets/test/__init__.py:60-100, :265-300); the same is done here against the
# fp64 forward oracle (element by element, central differences), plus torch.autograd on closed
# forms built from library routines, plus the combine functors bit for bit against oracle/_ref.
# ---------------------------------------------------------------------------------------------
def _numeric_grad(f, x, g_out, h=1e-6):
    """d <f(x), g_out> / dx by central differences; x is modified in place and restored."""
    grad = np.zeros_like(x)
    flat, gflat = x.reshape(-1), grad.reshape(-1)
    for i in range(flat.size):
        if np.isnan(flat[i]):
            continue
        keep = flat[i]
        flat[i] = keep + h
        up = f()
        flat[i] = keep - h
        dn = f()
        flat[i] = keep
        gflat[i] = np.nansum((up - dn) * g_out) / (2 * h)
    return grad


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_backward_functors_bit_exact_vs_reference(dtype):
    g = rng(60)
    vals = g.normal(size=(400, 6)).astype(dtype)
    vals[::7, 1] = np.nan                       # NaN data: the ignore-NaN variants must return zeros
    vals[::11, 1] = vals[::11, 2]               # x == t: sign(0) = 0 in the L1 functors
    for row in vals:
        err, x, t, w, fudge, extra = [dtype(v) for v in row]
        w, fudge = abs(w) + dtype(0.1), abs(fudge) * dtype(0.01)
        for mode in range(4):
            a = orc.backward_functor("sim_backward_weights_fn", dtype, mode, err, x, t, w, fudge)
            b = orc.backward_functor("sim_backward_weights_fn", dtype, mode, err, x, t, w, fudge, which="ref")
            assert a.tobytes() == b.tobytes(), (mode, row)
            a = orc.backward_functor("sim_backward_bottom_fn", dtype, mode, t, w, err, x)
            b = orc.backward_functor("sim_backward_bottom_fn", dtype, mode, t, w, err, x, which="ref")
            assert a.tobytes() == b.tobytes(), (mode, row)
        if np.isnan(x):
            continue
        for finite in (0, 1):
            top = x + t if (finite == 0 and extra > 0) else extra     # equality branch of the infinite form
            a = orc.backward_functor("mex_backward_term_fn", dtype, finite, t, top, err, x, w, fudge)
            b = orc.backward_functor("mex_backward_term_fn", dtype, finite, t, top, err, x, w, fudge, which="ref")
            assert a.tobytes() == b.tobytes(), (finite, row)


@pytest.mark.parametrize("patch,pad,stride", [((1, 3, 3), (0, 1, 1), (1, 1, 1)), ((2, 3, 2), (1, 0, 2), (1, 2, 1)),
                                              ((3, 1, 1), (0, 0, 0), (3, 1, 1)), ((2, 2, 2), (1, 1, 1), (2, 3, 2))])
@pytest.mark.parametrize("round_down", [True, False])
def test_col2im_3d_is_the_adjoint_of_im2col_3d(patch, pad, stride, round_down):
    g = rng(61)
    shape = (4, 7, 6)
    x = g.normal(size=shape)
    outs = [orc.dimension_out_size(shape[i], pad[i], patch[i], stride[i], round_down) for i in range(3)]
    col = orc.im2col_3d(x, patch, pad, stride, round_down=round_down, oob=0.0)
    c = g.normal(size=col.shape)
    assert col.size == np.prod(patch) * np.prod(outs)
    back = orc.col2im_3d(c, shape, patch, pad, stride, round_down=round_down)
    np.testing.assert_allclose(np.sum(col * c), np.sum(x * back), rtol=1e-12)
    # every basis image: <im2col(e_i), c> = col2im(c)[i]
    probe = np.zeros(shape)
    for idx in [(0, 0, 0), (3, 6, 5), (1, 3, 2), (2, 0, 5)]:
        probe[idx] = 1.0
        got = np.sum(orc.im2col_3d(probe, patch, pad, stride, round_down=round_down, oob=0.0) * c)
        probe[idx] = 0.0
        np.testing.assert_allclose(got, back[idx], rtol=1e-12, atol=1e-14)


def test_col2im_2d_matches_torch_fold():
    g = rng(62)
    C_, H, W = 3, 9, 8
    blocks, strides, padding = (3, 2), (2, 1), (1, 1)
    oh = orc.dimension_out_size(H, padding[0], blocks[0], strides[0])
    ow = orc.dimension_out_size(W, padding[1], blocks[1], strides[1])
    col = g.normal(size=(C_ * blocks[0] * blocks[1], oh * ow))
    want = F.fold(torch.from_numpy(col)[None], (H, W), blocks, padding=padding, stride=strides)[0].numpy()
    got = orc.col2im_3d(col, (C_, H, W), (C_,) + blocks, (0,) + padding, (C_,) + strides)
    np.testing.assert_allclose(got, want, rtol=1e-13, atol=1e-13)


SIM_GRAD_CASES = [  # func, norm, ignore_nan, blocks, strides, padding
    ("L2", False, False, (3, 3), (1, 1), (1, 1)),
    ("L2", False, False, (3, 1), (2, 1), (0, 0)),
    ("L1", False, False, (3, 3), (2, 2), (1, 1)),
    ("L1", False, False, (1, 1), (1, 1), (0, 0)),
    ("L2", True, False, (3, 3), (2, 1), (1, 0)),
    ("L2", True, True, (3, 3), (1, 1), (1, 1)),
    ("L2", True, True, (2, 3), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("func,norm,ign,blocks,strides,padding", SIM_GRAD_CASES)
def test_similarity_grads_match_numeric_differentiation(func, norm, ign, blocks, strides, padding):
    g = rng(63)
    x, t, w = _sim_inputs(g, (2, 3, 7, 6), 3, blocks, np.float64)
    if ign:
        x[g.random(size=x.shape) < 0.15] = np.nan
    kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding, normalization_term=norm,
              ignore_nan_input=ign, out_of_bounds_value=np.nan if ign else 0.3)
    out = orc.similarity_fwd(x, t, w, **kw)
    go = g.normal(size=out.shape)
    f = lambda: orc.similarity_fwd(x, t, w, **kw)
    gx = orc.similarity_input_grad(x, t, w, go, **kw)
    gt, gw = orc.similarity_params_grad(x, t, w, go, **kw)
    assert gx.shape == x.shape and gt.shape == t.shape and gw.shape == w.shape
    if ign:
        assert (gx[np.isnan(x)] == 0).all() and not np.isnan(gx).any()
    np.testing.assert_allclose(gx, _numeric_grad(f, x, go), rtol=2e-7, atol=2e-7)
    np.testing.assert_allclose(gt, _numeric_grad(f, t, go), rtol=2e-7, atol=2e-7)
    np.testing.assert_allclose(gw, _numeric_grad(f, w, go), rtol=2e-7, atol=2e-7)


@pytest.mark.parametrize("func", ["L1", "L2"])
def test_similarity_grads_match_torch_autograd_of_unfold_form(func):
    g = rng(64)
    blocks, strides, padding = (3, 2), (2, 1), (1, 1)
    x, t, w = _sim_inputs(g, (3, 4, 9, 8), 5, blocks, np.float64)
    kw = dict(similarity_function=func, blocks=blocks, strides=strides, padding=padding)
    tx, tt, tw = [torch.from_numpy(a).requires_grad_() for a in (x, t, w)]
    cols = F.unfold(tx, blocks, padding=padding, stride=strides)                    # [B, K, P]
    d = cols[:, None] - tt.reshape(5, -1)[None, :, :, None]                         # [B, O, K, P]
    d = d.abs() if func == "L1" else d * d
    out = -(tw.reshape(5, -1)[None, :, :, None] * d).sum(2)
    go = g.normal(size=tuple(out.shape))
    out.backward(torch.from_numpy(go))
    oshape = orc.similarity_fwd(x, t, w, **kw).shape
    go = go.reshape(oshape)
    np.testing.assert_allclose(orc.similarity_input_grad(x, t, w, go, **kw), tx.grad.numpy(), rtol=1e-11, atol=1e-12)
    gt, gw = orc.similarity_params_grad(x, t, w, go, **kw)
    np.testing.assert_allclose(gt, tt.grad.numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(gw, tw.grad.numpy(), rtol=1e-11, atol=1e-12)


def test_similarity_grads_fp32_follow_fp64():
    g = rng(65)
    x, t, w = _sim_inputs(g, (2, 5, 12, 11), 6, (3, 3), np.float32)
    kw = dict(similarity_function="L2", blocks=(3, 3), strides=(1, 2), padding=(1, 1), normalization_term=True)
    go = g.normal(size=orc.similarity_fwd(x, t, w, **kw).shape).astype(np.float32)
    a32 = (orc.similarity_input_grad(x, t, w, go, **kw),) + orc.similarity_params_grad(x, t, w, go, **kw)
    d = [a.astype(np.float64) for a in (x, t, w, go)]
    a64 = (orc.similarity_input_grad(*d, **kw),) + orc.similarity_params_grad(*d, **kw)
    for lo, hi in zip(a32, a64):
        assert lo.dtype == np.float32
        np.testing.assert_allclose(lo, hi, rtol=1e-4, atol=1e-4 * np.abs(hi).max())


MEX_GRAD_CASES = [  # im_dims, instances, kw
    ((2, 3, 6, 5), 2, dict(blocks=[1, 3, 3], strides=[1, 1, 1], padding=[0, 1, 1], shared_offset_region=[2])),
    ((2, 3, 6, 5), 2, dict(blocks=[1, 3, 3], strides=[1, 1, 1], padding=[0, 1, 1], shared_offset_region=[2],
                           use_unshared_regions=False)),
    ((1, 4, 7, 6), 3, dict(blocks=[2, 2, 2], strides=[2, 2, 1], padding=[0, 0, 0], shared_offset_region=[1, 2, 3])),
    ((2, 3, 5, 5), 2, dict(blocks=[3, 1, 1], strides=[3, 1, 1], padding=[0, 0, 0])),
    ((1, 3, 6, 6), 2, dict(blocks=[2, 3, 2], strides=[1, 2, 2], padding=[1, 1, 0], blocks_round_down=False,
                           blocks_out_of_bounds_value=-0.7, shared_offset_region=[1, 2, 2])),
]


@pytest.mark.parametrize("eps,softmax", [(1.0, False), (-2.0, False), (0.7, True), (math.inf, False),
                                         (-math.inf, False)])
@pytest.mark.parametrize("im_dims,inst,kw", MEX_GRAD_CASES)
def test_mex_grads_match_numeric_differentiation(im_dims, inst, kw, eps, softmax):
    g = rng(66)
    kw = dict(kw, epsilon=eps, softmax_mode=softmax)
    x, off, d = _mex_case(g, im_dims, inst, np.float64, **kw)
    out = orc.mex_fwd(x, off, inst, **kw)
    go = g.normal(size=out.shape)
    f = lambda: orc.mex_fwd(x, off, inst, **kw)
    gx = orc.mex_input_grad(x, off, out, go, inst, **kw)
    goff = orc.mex_offsets_grad(x, off, out, go, inst, **kw)
    assert gx.shape == x.shape and goff.shape == off.shape
    np.testing.assert_allclose(gx, _numeric_grad(f, x, go, h=1e-7), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(goff, _numeric_grad(f, off, go, h=1e-7), rtol=1e-6, atol=1e-6)


def test_mex_grads_1x1_single_region_match_torch_logsumexp():
    g = rng(67)
    B, C_, H, W, M = 2, 6, 4, 5, 3
    eps = 1.75                                  # exactly representable: the attribute is a C float
    kw = dict(blocks=[C_, 1, 1], strides=[C_, 1, 1], padding=[0, 0, 0], epsilon=eps, use_unshared_regions=False)
    x = g.normal(size=(B, C_, H, W))
    off = g.normal(size=(1, M, C_, 1, 1))
    tx, to = torch.from_numpy(x).requires_grad_(), torch.from_numpy(off).requires_grad_()
    z = tx[:, None] + to.reshape(M, C_)[None, :, :, None, None]                 # [B, M, C, H, W]
    out = (torch.logsumexp(eps * z, dim=2) - math.log(C_)) / eps
    go = g.normal(size=tuple(out.shape))
    out.backward(torch.from_numpy(go))
    fwd = orc.mex_fwd(x, off, M, **kw)
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(orc.mex_input_grad(x, off, fwd, go, M, **kw), tx.grad.numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(orc.mex_offsets_grad(x, off, fwd, go, M, **kw), to.grad.numpy(), rtol=1e-11,
                               atol=1e-13)


def test_mex_grads_fp32_follow_fp64():
    g = rng(68)
    kw = dict(blocks=[1, 3, 3], strides=[1, 2, 2], padding=[0, 1, 1], shared_offset_region=[3], epsilon=1.0)
    x, off, d = _mex_case(g, (2, 4, 11, 10), 4, np.float32, **kw)
    out = orc.mex_fwd(x, off, 4, **kw)
    go = g.normal(size=out.shape).astype(np.float32)
    lo = (orc.mex_input_grad(x, off, out, go, 4, **kw), orc.mex_offsets_grad(x, off, out, go, 4, **kw))
    d64 = [a.astype(np.float64) for a in (x, off)]
    out64 = orc.mex_fwd(*d64, 4, **kw)
    hi = (orc.mex_input_grad(*d64, out64, go.astype(np.float64), 4, **kw),
          orc.mex_offsets_grad(*d64, out64, go.astype(np.float64), 4, **kw))
    for a, b in zip(lo, hi):
        assert a.dtype == np.float32
        np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4 * np.abs(b).max())
