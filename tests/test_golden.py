"""The committed golden vectors (tests/golden/ref_headers.npz, written by tests/golden/make_golden.py from the
reference's own headers) against the CPU oracle, bit for bit.  Needs neither the reference checkout nor a GPU."""
import os

import numpy as np
import pytest

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_headers.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN, allow_pickle=False)


def same_bits(a, b):
    return a.shape == b.shape and a.tobytes() == b.tobytes()


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_oracle_ggemm_similarity_matches_golden(gold, mode):
    A, B, C = (gold["ggemm_mode%d_%s" % (mode, n)] for n in "ABC")
    M, K = A.shape[:2]
    assert same_bits(orc.ggemm_similarity(mode, A, B, M, B.shape[1], K, 0.001, "oracle"), C)


@pytest.mark.parametrize("i", range(12))
def test_oracle_mex_forward_matches_golden(gold, i):
    off, inp, want = gold["mex_%d_off" % i], gold["mex_%d_in" % i], gold["mex_%d_out" % i]
    softmax, eps = gold["mex_%d_meta" % i]
    R, M, K = off.shape
    assert same_bits(orc.mex_forward(off, inp, M, inp.shape[2], K, bool(softmax), float(eps), R, "oracle"), want)


@pytest.mark.parametrize("i", range(6))
def test_oracle_split_patches_matches_golden(gold, i):
    src, want = gold["split_%d_src" % i], gold["split_%d_dst" % i]
    Cc, H, W, Cg, Hg, Wg, Cs, Hs, Ws, unshared = [int(v) for v in gold["split_%d_meta" % i]]
    dst = np.full(want.shape, -7.0, np.float32)
    orc.split_patches(False, src.copy(), dst, Cc * H * W, src.shape[0], W, H, Cc, Wg, Hg, Cg, Ws, Hs, Cs, unshared,
                      "oracle")
    assert same_bits(dst, want)


def test_oracle_backward_functors_match_golden(gold):
    args = gold["bw_args"]
    for mode in range(4):
        got_w = np.array([orc.backward_functor("sim_backward_weights_fn", np.float32, mode, a[0], a[1], a[2], a[3], a[4])
                          for a in args], np.float32)
        got_b = np.array([orc.backward_functor("sim_backward_bottom_fn", np.float32, mode, a[2], a[3], a[0], a[1])
                          for a in args], np.float32)
        assert same_bits(got_w, gold["bw_weights%d" % mode]) and same_bits(got_b, gold["bw_bottom%d" % mode])
    fin = gold["bw_mex_args"]
    for finite in (0, 1):
        got = np.array([orc.backward_functor("mex_backward_term_fn", np.float32, finite, a[2],
                                             a[1] + a[2] if (finite == 0 and a[5] > 0) else a[5], a[0], a[1], a[3], a[4])
                        for a in fin], np.float32)
        assert same_bits(got, gold["bw_mex%d" % finite])
