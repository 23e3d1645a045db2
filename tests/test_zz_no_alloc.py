"""simnets_hip_similarity_fwd_static (the entry point that allocates nothing: its scratch is a fixed device array
inside the library) against simnets_hip_similarity_fwd (caller workspace), through the C ABI.

Both run the same kernels, so the outputs must be identical bit for bit; the oracle bounds them both (1e-5).
The second call of every pair uses a smaller input than the first: the static array still holds the first call's
packed parameters, thresholds and (small-map kernel only: the tiled kernels keep them in registers) guard flags, and
none of them may leak into the second result.  Every pair also checks that the static call leaves the device's free
memory and torch's allocator statistics untouched."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import config1, rel_err

pytestmark = pytest.mark.gpu

SIM_TOL = 1e-5


def _call_pair(pkg, x, t, w, **kw):
    """(static-scratch result, workspace result) of one problem, called through ctypes."""
    from simnets_tf_amd import _lib, ops
    l = _lib.lib()
    a = ops.similarity_attrs(**kw)
    I4 = C.c_int * 4
    xs, ts = I4(*x.shape), I4(*t.shape)
    oshape = I4()
    assert l.simnets_similarity_out_shape(C.byref(a), xs, ts, ts, oshape) == 0
    X, T, W = (torch.from_numpy(np.ascontiguousarray(v)).cuda() for v in (x, t, w))
    nbytes = C.c_size_t()
    assert l.simnets_hip_similarity_workspace_bytes(C.byref(a), xs, ts, C.byref(nbytes)) == 0
    assert nbytes.value <= _lib.STATIC_SCRATCH_BYTES
    ws = torch.empty(max(nbytes.value, 256), dtype=torch.uint8, device="cuda")
    want = torch.full(tuple(oshape), 7.0, dtype=torch.float32, device="cuda")
    got = torch.full(tuple(oshape), -7.0, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = l.simnets_hip_similarity_fwd(C.byref(a), xs, ts, ts, X.data_ptr(), T.data_ptr(), W.data_ptr(),
                                      want.data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, _lib.strerror(rc)
    rc = l.simnets_hip_similarity_fwd_static(C.byref(a), xs, ts, ts, X.data_ptr(), T.data_ptr(), W.data_ptr(),
                                             got.data_ptr(), stream)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    first = got.clone()
    # the call again, now that its kernels' code is resident: nothing may be allocated, by the library or through torch
    before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    rc = l.simnets_hip_similarity_fwd_static(C.byref(a), xs, ts, ts, X.data_ptr(), T.data_ptr(), W.data_ptr(),
                                             got.data_ptr(), stream)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert after == before, "the static-scratch call changed the device's memory state: %s -> %s" % (before, after)
    assert torch.equal(got, first)
    return got.cpu().numpy(), want.cpu().numpy()


def _inputs(seed, shape, O, blocks, spread=1.0):
    g = np.random.default_rng(seed)
    x = g.normal(size=shape).astype(np.float32)
    t = (g.normal(size=(O, shape[1]) + tuple(blocks)) * spread).astype(np.float32)
    w = g.uniform(0.1, 2.0, size=t.shape).astype(np.float32)
    return x, t, w


def _check(pkg, x, t, w, **kw):
    got, want = _call_pair(pkg, x, t, w, **kw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "static-scratch result differs from workspace result"
    assert rel_err(got, orc.similarity_fwd(x, t, w, **{k: v for k, v in kw.items() if k != "algo"})) <= SIM_TOL


@pytest.mark.parametrize("func", ["L2", "L1"])
def test_static_scratch_two_calls_second_smaller(pkg, func):
    kw = dict(similarity_function=func, blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    # first call: 16x8 lane tile, 40 templates of 24 channels; second: fewer, smaller everything (other tiling)
    _check(pkg, *_inputs(11, (6, 24, 32, 32), 40, (3, 3)), **kw)
    _check(pkg, *_inputs(12, (2, 5, 9, 13), 3, (3, 3)), **kw)


def test_static_scratch_guard_state_does_not_leak(pkg):
    """Plain L2 runs the sqrt-weight form with thresholds and per-wave flags in the scratch.  First call: a template
    equal to a patch and a negative-weight template (flags raised, an infinite threshold); second, smaller call on
    ordinary data must not see either."""
    kw = dict(blocks=[2, 2], strides=[1, 1], padding=[0, 0])
    x, t, w = _inputs(21, (3, 4, 20, 36), 9, (2, 2))
    t[2] = x[1, :, 5:7, 8:10]      # exact match at one pixel: that output is ~0 and gets recomputed
    w[4, 0, 0, 0] = -0.5           # sqrt undefined: every output of template 4 is recomputed
    _check(pkg, x, t, w, **kw)
    _check(pkg, *_inputs(22, (1, 4, 7, 9), 2, (2, 2)), **kw)


def test_static_scratch_small_map_guard_flags_do_not_leak(pkg):
    """The small-map kernel (several 7x7 images per wave) with the sqrt-weight form is the one path that keeps its
    guard flags - one per workgroup - in the scratch: the main launch writes them, the recomputing launch reads them.
    First call: an exact-match template and a negative-weight template raise flags; the second call (fewer images,
    ordinary data, same geometry) must recompute nothing it should not and miss nothing."""
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    x, t, w = _inputs(31, (32, 16, 7, 7), 24, (3, 3))
    t[3] = x[1, :, 2:5, 3:6]       # the patch of output pixel (3, 4) of image 1
    w[5, 0, 0, 0] = -0.5
    _check(pkg, x, t, w, **kw)
    _check(pkg, *_inputs(32, (16, 16, 7, 7), 24, (3, 3)), **kw)
    x, t, w = _inputs(33, (12, 16, 7, 7), 9, (3, 3))
    t[8] = x[11, :, 4:7, 0:3]
    _check(pkg, x, t, w, **kw)


def test_static_scratch_matrix_core_path(pkg):
    """algo='mfma' keeps its packed operand, bias and per-channel centre arrays in the scratch."""
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1], algo="mfma")
    _check(pkg, *_inputs(41, (4, 24, 20, 20), 70, (3, 3)), **kw)
    _check(pkg, *_inputs(42, (2, 5, 9, 13), 3, (3, 3)), **kw)


def test_static_scratch_normalized_ignore_nan(pkg):
    x, t, w, kw = config1(batch=8, nan_frac=0.25)
    _check(pkg, x, t, w, **kw)
    x, t, w, kw = config1(batch=2, nan_frac=0.25)
    _check(pkg, x[:, :, :13, :17].copy(), t[:5].copy(), w[:5].copy(), **kw)


def test_static_scratch_rejects_what_does_not_fit(pkg):
    """More packed parameters than the static array holds: refused with its own status, before any launch."""
    from simnets_tf_amd import _lib, ops
    l = _lib.lib()
    a = ops.similarity_attrs(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    I4 = C.c_int * 4
    xs, ts = I4(1, 64, 8, 8), I4(1024, 64, 3, 3)
    nbytes = C.c_size_t()
    assert l.simnets_hip_similarity_workspace_bytes(C.byref(a), xs, ts, C.byref(nbytes)) == 0
    assert nbytes.value > _lib.STATIC_SCRATCH_BYTES
    rc = l.simnets_hip_similarity_fwd_static(C.byref(a), xs, ts, ts, None, None, None, None, None)
    assert rc == -21 and "scratch" in _lib.strerror(rc)
