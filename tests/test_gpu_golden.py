"""The HIP library against the committed golden vectors of the reference's own header-only kernels
(tests/golden/ref_headers.npz): a Similarity with 1x1 blocks is exactly one ggemm, a MEX with a [C,1,1] block and
one shared region is exactly one mex_forward.  Needs no reference checkout."""
import math
import os

import numpy as np
import pytest
import torch

from util import rel_err

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_headers.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN, allow_pickle=False)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_similarity_1x1_blocks_match_golden_ggemm(pkg, gold, mode):
    A, B, C = (gold["ggemm_mode%d_%s" % (mode, n)] for n in "ABC")
    M, K = A.shape[:2]
    N = B.shape[1]
    kw = dict(similarity_function="L1" if mode == 0 else "L2", blocks=[1, 1], strides=[1, 1], padding=[0, 0],
              normalization_term=mode >= 2, ignore_nan_input=mode == 3, normalization_term_fudge=0.001)
    t = np.ascontiguousarray(A[..., 0]).reshape(M, K, 1, 1)
    w = np.ascontiguousarray(A[..., 1]).reshape(M, K, 1, 1)
    got = pkg.similarity(dev(B.reshape(1, K, 1, N)), dev(t), dev(w), **kw).cpu().numpy().reshape(M, N)
    want = C
    if mode == 2:   # the op adds -0.5*K*log(2 pi) once per output on top of the ggemm (similarity_kernel_cpu.cpp:69)
        want = C + np.float32(np.float64(np.float32(-0.5) * np.float32(K)) * math.log(2.0 * math.pi))
    assert rel_err(got, want) <= 1e-5


@pytest.mark.parametrize("i", range(12))
def test_mex_channel_blocks_match_golden_mex_forward(pkg, gold, i):
    off, inp, want = gold["mex_%d_off" % i], gold["mex_%d_in" % i], gold["mex_%d_out" % i]
    softmax, eps = gold["mex_%d_meta" % i]
    R, M, K = off.shape
    N = inp.shape[2]
    kw = dict(blocks=[K, 1, 1], strides=[K, 1, 1], padding=[0, 0, 0], softmax_mode=bool(softmax), epsilon=float(eps),
              use_unshared_regions=False, shared_offset_region=[-1])
    for r in range(R):
        got = pkg.mex(dev(inp[r].reshape(1, K, 1, N)), dev(off[r].reshape(1, M, K, 1, 1)), M, **kw).cpu().numpy()
        m = (inp[r][None, :, :] + off[r][:, :, None])
        m = m.max(axis=1) if eps > 0 else m.min(axis=1)
        assert rel_err(got.reshape(M, N), want[r], floor=m) <= 1e-4
