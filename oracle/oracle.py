"""ctypes bindings of the CPU oracle (oracle/libsimnets_oracle.so) and, when present, of the
reference's own TF-free headers (oracle/_ref/libsimnets_ref.so).

Test infrastructure: only the test-suite, the smoke check and the cpu_baseline leg of the
benchmark import this module.  The shipped library never does.
"""
import ctypes as C
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libsimnets_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libsimnets_ref.so")

SIM_L1, SIM_L2 = 0, 1


def build(reference="/root/reference"):
    """Compile the oracle (and the reference shim when the checkout is there)."""
    subprocess.run(["make", "-C", _HERE, "-B", "REFERENCE=" + reference, "all"], check=True,
                   stdout=subprocess.DEVNULL)


class SimilarityArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int), ("channels", C.c_int), ("height", C.c_int), ("width", C.c_int),
        ("num_instances", C.c_int),
        ("block_h", C.c_int), ("block_w", C.c_int),
        ("stride_h", C.c_int), ("stride_w", C.c_int),
        ("pad_h", C.c_int), ("pad_w", C.c_int),
        ("similarity_function", C.c_int),
        ("normalization_term", C.c_int),
        ("normalization_term_fudge", C.c_float),
        ("ignore_nan_input", C.c_int),
        ("out_of_bounds_value", C.c_float),
        ("norm_const_every_iteration", C.c_int),
        ("threads", C.c_int),
    ]


class MexArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int), ("channels", C.c_int), ("height", C.c_int), ("width", C.c_int),
        ("num_instances", C.c_int),
        ("softmax_mode", C.c_int),
        ("n_padding", C.c_int), ("padding", C.c_int * 3),
        ("n_strides", C.c_int), ("strides", C.c_int * 3),
        ("n_blocks", C.c_int), ("blocks", C.c_int * 3),
        ("epsilon", C.c_float),
        ("blocks_out_of_bounds_value", C.c_float),
        ("blocks_round_down", C.c_int),
        ("use_unshared_regions", C.c_int),
        ("n_shared", C.c_int), ("shared_offset_region", C.c_int * 3),
        ("n_unshared", C.c_int), ("unshared_offset_region", C.c_int * 3),
        ("threads", C.c_int),
    ]


class MexDims(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "pad_c", "pad_h", "pad_w", "stride_c", "stride_h", "stride_w", "block_c", "block_h", "block_w",
        "channels_out", "height_out", "width_out", "channels_out_total",
        "shared_region_c", "shared_region_h", "shared_region_w",
        "offsets_c", "offsets_h", "offsets_w",
        "num_regions", "region_size", "M", "K", "N", "is_1x1")]

    def asdict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build()
        _lib = C.CDLL(ORACLE_SO)
        _lib.so_dimension_out_size.restype = C.c_int
        _lib.so_ggemm_padded_output_size.restype = C.c_int
    return _lib


def ref():
    """The reference-header shim, or None when it was never built."""
    global _ref
    if _ref is None and os.path.exists(REF_SO):
        _ref = C.CDLL(REF_SO)
    return _ref


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32", C.c_float
    if dtype == np.float64:
        return "_f64", C.c_double
    raise TypeError(dtype)


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def dimension_out_size(image, pad, patch, stride, round_down=True):
    return lib().so_dimension_out_size(int(image), int(pad), int(patch), int(stride), int(bool(round_down)))


def _fill_list(dst, values):
    for i, v in enumerate(values):
        dst[i] = int(v)
    return len(values)


def similarity_args(x_shape, num_instances, similarity_function="L2", blocks=(3, 3), strides=(2, 2),
                    padding=(0, 0), normalization_term=False, normalization_term_fudge=0.001,
                    ignore_nan_input=False, out_of_bounds_value=0.0, norm_const_every_iteration=False,
                    threads=1):
    B, Cc, H, W = x_shape
    a = SimilarityArgs()
    a.batch, a.channels, a.height, a.width = B, Cc, H, W
    a.num_instances = num_instances
    a.block_h, a.block_w = blocks
    a.stride_h, a.stride_w = strides
    a.pad_h, a.pad_w = padding
    a.similarity_function = {"L1": SIM_L1, "L2": SIM_L2}[similarity_function]
    a.normalization_term = int(bool(normalization_term))
    a.normalization_term_fudge = normalization_term_fudge
    a.ignore_nan_input = int(bool(ignore_nan_input))
    a.out_of_bounds_value = out_of_bounds_value
    a.norm_const_every_iteration = int(bool(norm_const_every_iteration))
    a.threads = threads
    return a


def similarity_out_dims(a):
    oh, ow = C.c_int(), C.c_int()
    rc = lib().so_similarity_out_dims(C.byref(a), C.byref(oh), C.byref(ow))
    if rc:
        raise ValueError("similarity oracle: invalid arguments (%d)" % rc)
    return oh.value, ow.value


def _similarity(fn_base, x, templates, weights, **kw):
    x = np.ascontiguousarray(x)
    sfx, _ = _sfx(x.dtype)
    templates = np.ascontiguousarray(templates, dtype=x.dtype)
    weights = np.ascontiguousarray(weights, dtype=x.dtype)
    assert templates.shape == weights.shape and templates.shape[1] == x.shape[1]
    kw.setdefault("blocks", templates.shape[2:])
    assert tuple(kw["blocks"]) == tuple(templates.shape[2:])
    a = similarity_args(x.shape, templates.shape[0], **kw)
    oh, ow = similarity_out_dims(a)
    out = np.empty((x.shape[0], templates.shape[0], oh, ow), dtype=x.dtype)
    rc = getattr(lib(), fn_base + sfx)(C.byref(a), _ptr(x), _ptr(templates), _ptr(weights), _ptr(out))
    if rc:
        raise ValueError("similarity oracle failed (%d)" % rc)
    return out


def similarity_fwd(x, templates, weights, **kw):
    """Restatement of SimilarityKernelCPU::Compute (the fast CPU path)."""
    return _similarity("so_similarity_fwd", x, templates, weights, **kw)


def similarity_ref(x, templates, weights, **kw):
    """Restatement of the brute-force SimilarityRef op."""
    return _similarity("so_similarity_ref", x, templates, weights, **kw)


def mex_args(x_shape, num_instances, softmax_mode=False, padding=(0, 0, 0), strides=(1, 1, 1),
             blocks=(1, 1, 1), epsilon=1.0, blocks_out_of_bounds_value=0.0, blocks_round_down=True,
             use_unshared_regions=True, shared_offset_region=(-1,), unshared_offset_region=(-1,), threads=1):
    B, Cc, H, W = x_shape
    a = MexArgs()
    a.batch, a.channels, a.height, a.width = B, Cc, H, W
    a.num_instances = num_instances
    a.softmax_mode = int(bool(softmax_mode))
    a.n_padding = _fill_list(a.padding, padding)
    a.n_strides = _fill_list(a.strides, strides)
    a.n_blocks = _fill_list(a.blocks, blocks)
    a.epsilon = epsilon
    a.blocks_out_of_bounds_value = blocks_out_of_bounds_value
    a.blocks_round_down = int(bool(blocks_round_down))
    a.use_unshared_regions = int(bool(use_unshared_regions))
    a.n_shared = _fill_list(a.shared_offset_region, shared_offset_region)
    a.n_unshared = _fill_list(a.unshared_offset_region, unshared_offset_region)
    a.threads = threads
    return a


def mex_dims(a):
    d = MexDims()
    rc = lib().so_mex_calc_dims(C.byref(a), C.byref(d))
    if rc:
        raise ValueError("mex oracle: invalid arguments (%d)" % rc)
    return d


def _mex(fn_base, x, offsets, num_instances, **kw):
    x = np.ascontiguousarray(x)
    sfx, _ = _sfx(x.dtype)
    offsets = np.ascontiguousarray(offsets, dtype=x.dtype)
    a = mex_args(x.shape, num_instances, **kw)
    d = mex_dims(a)
    assert offsets.size == d.num_regions * d.M * d.K, (offsets.shape, d.asdict())
    out = np.empty((x.shape[0], d.channels_out_total, d.height_out, d.width_out), dtype=x.dtype)
    rc = getattr(lib(), fn_base + sfx)(C.byref(a), _ptr(x), _ptr(offsets), _ptr(out))
    if rc:
        raise ValueError("mex oracle failed (%d)" % rc)
    return out


def mex_fwd(x, offsets, num_instances, **kw):
    """Restatement of MEXKernelCPU::Compute (the fast CPU path)."""
    return _mex("so_mex_fwd", x, offsets, num_instances, **kw)


def mex_ref(x, offsets, num_instances, **kw):
    """Restatement of the brute-force MexRef op."""
    return _mex("so_mex_ref", x, offsets, num_instances, **kw)


def normalize_offsets(offsets):
    offsets = np.ascontiguousarray(offsets)
    sfx, _ = _sfx(offsets.dtype)
    K = int(np.prod(offsets.shape[2:]))
    rows = offsets.shape[0] * offsets.shape[1]
    out = np.empty_like(offsets)
    getattr(lib(), "so_normalize_offsets" + sfx)(rows, K, _ptr(offsets), _ptr(out))
    return out


def im2col_3d(im, patch, pad, stride, round_down=True, oob=0.0):
    im = np.ascontiguousarray(im)
    sfx, ct = _sfx(im.dtype)
    Cc, H, W = im.shape
    cc = dimension_out_size(Cc, pad[0], patch[0], stride[0], round_down)
    hc = dimension_out_size(H, pad[1], patch[1], stride[1], round_down)
    wc = dimension_out_size(W, pad[2], patch[2], stride[2], round_down)
    col = np.empty((patch[0] * patch[1] * patch[2], cc, hc, wc), dtype=im.dtype)
    getattr(lib(), "so_im2col_3d" + sfx)(_ptr(im), Cc, H, W, *[int(v) for v in patch], *[int(v) for v in pad],
                                         *[int(v) for v in stride], _ptr(col), int(bool(round_down)), ct(oob))
    return col


def _call_both(name, dtype, *args):
    sfx, _ = _sfx(dtype)
    return getattr(lib(), "so_" + name + sfx), (getattr(ref(), "ref_" + name + sfx) if ref() else None)


def ggemm_similarity(mode, A_interlaced, Bm, M, N, K, fudge=0.001, which="oracle"):
    A_interlaced = np.ascontiguousarray(A_interlaced)
    Bm = np.ascontiguousarray(Bm, dtype=A_interlaced.dtype)
    so, rf = _call_both("ggemm_similarity", A_interlaced.dtype)
    _, ct = _sfx(A_interlaced.dtype)
    fn = so if which == "oracle" else rf
    out = np.empty((M, N), dtype=A_interlaced.dtype)
    fn(int(mode), M, N, K, _ptr(A_interlaced), _ptr(Bm), _ptr(out), ct(fudge))
    return out


def mex_forward(offsets, inp, M, N, K, softmax_mode, epsilon, batch, which="oracle"):
    offsets = np.ascontiguousarray(offsets)
    inp = np.ascontiguousarray(inp, dtype=offsets.dtype)
    so, rf = _call_both("mex_forward", offsets.dtype)
    _, ct = _sfx(offsets.dtype)
    fn = so if which == "oracle" else rf
    out = np.zeros((batch, M, N), dtype=offsets.dtype)
    fn(M, N, K, int(bool(softmax_mode)), ct(epsilon), _ptr(offsets), _ptr(inp), _ptr(out), int(batch))
    return out


def split_patches(reverse, inp, out, N, Dim, W, H, Cc, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, use_unshared,
                  which="oracle"):
    """In-place like the reference: forward fills `out` from `inp`, reverse fills `inp` from `out`."""
    so, rf = _call_both("split_patches", inp.dtype)
    fn = so if which == "oracle" else rf
    fn(int(bool(reverse)), N, Dim, W, H, Cc, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, _ptr(inp), _ptr(out),
       int(bool(use_unshared)))


def _sim_grad_common(x, templates, weights, output_grad, kw):
    x = np.ascontiguousarray(x)
    templates = np.ascontiguousarray(templates, dtype=x.dtype)
    weights = np.ascontiguousarray(weights, dtype=x.dtype)
    output_grad = np.ascontiguousarray(output_grad, dtype=x.dtype)
    kw.setdefault("blocks", templates.shape[2:])
    a = similarity_args(x.shape, templates.shape[0], **kw)
    oh, ow = similarity_out_dims(a)
    assert output_grad.shape == (x.shape[0], templates.shape[0], oh, ow), output_grad.shape
    return a, x, templates, weights, output_grad


def similarity_input_grad(x, templates, weights, output_grad, **kw):
    """Restatement of SimilarityInputGradKernelCPU::Compute."""
    a, x, templates, weights, output_grad = _sim_grad_common(x, templates, weights, output_grad, kw)
    sfx, _ = _sfx(x.dtype)
    out = np.empty_like(x)
    rc = getattr(lib(), "so_similarity_input_grad" + sfx)(C.byref(a), _ptr(x), _ptr(templates), _ptr(weights),
                                                         _ptr(output_grad), _ptr(out))
    if rc:
        raise ValueError("similarity_input_grad oracle failed (%d)" % rc)
    return out


def similarity_params_grad(x, templates, weights, output_grad, **kw):
    """Restatement of SimilarityParametersGradKernelCPU::Compute -> (templates_grad, weights_grad)."""
    a, x, templates, weights, output_grad = _sim_grad_common(x, templates, weights, output_grad, kw)
    sfx, _ = _sfx(x.dtype)
    gt, gw = np.empty_like(templates), np.empty_like(weights)
    rc = getattr(lib(), "so_similarity_params_grad" + sfx)(C.byref(a), _ptr(x), _ptr(templates), _ptr(weights),
                                                          _ptr(output_grad), _ptr(gt), _ptr(gw))
    if rc:
        raise ValueError("similarity_params_grad oracle failed (%d)" % rc)
    return gt, gw


def _mex_grad(fn, x, offsets, output, output_grad, num_instances, kw):
    x = np.ascontiguousarray(x)
    sfx, _ = _sfx(x.dtype)
    offsets = np.ascontiguousarray(offsets, dtype=x.dtype)
    output = np.ascontiguousarray(output, dtype=x.dtype)
    output_grad = np.ascontiguousarray(output_grad, dtype=x.dtype)
    a = mex_args(x.shape, num_instances, **kw)
    d = mex_dims(a)
    assert output.shape == output_grad.shape == (x.shape[0], d.channels_out_total, d.height_out, d.width_out)
    assert offsets.size == d.num_regions * d.M * d.K
    res = np.empty_like(x if fn == "so_mex_input_grad" else offsets)
    rc = getattr(lib(), fn + sfx)(C.byref(a), _ptr(x), _ptr(offsets), _ptr(output), _ptr(output_grad), _ptr(res))
    if rc:
        raise ValueError("%s oracle failed (%d)" % (fn, rc))
    return res


def mex_input_grad(x, offsets, output, output_grad, num_instances, **kw):
    """Restatement of MEXGradInputKernelCPU::Compute."""
    return _mex_grad("so_mex_input_grad", x, offsets, output, output_grad, num_instances, kw)


def mex_offsets_grad(x, offsets, output, output_grad, num_instances, **kw):
    """Restatement of MEXGradOffsetsKernelCPU::Compute."""
    return _mex_grad("so_mex_offsets_grad", x, offsets, output, output_grad, num_instances, kw)


def col2im_3d(col, im_shape, patch, pad, stride, round_down=True):
    col = np.ascontiguousarray(col)
    sfx, _ = _sfx(col.dtype)
    Cc, H, W = im_shape
    im = np.empty(im_shape, dtype=col.dtype)
    getattr(lib(), "so_col2im_3d" + sfx)(_ptr(col), Cc, H, W, *[int(v) for v in patch], *[int(v) for v in pad],
                                         *[int(v) for v in stride], _ptr(im), int(bool(round_down)))
    return im


def backward_functor(name, dtype, *args, which="oracle"):
    """name in {'sim_backward_weights_fn', 'sim_backward_bottom_fn', 'mex_backward_term_fn'}; scalar in, scalar(s) out."""
    sfx, ct = _sfx(dtype)
    fn = getattr(lib() if which == "oracle" else ref(), ("so_" if which == "oracle" else "ref_") + name + sfx)
    cargs = [C.c_int(int(args[0]))] + [ct(float(v)) for v in args[1:]]
    if name == "sim_backward_weights_fn":
        out = (ct * 2)()
        fn(*cargs, out)
        return np.array([out[0], out[1]], dtype=dtype)
    fn.restype = ct
    return np.dtype(dtype).type(fn(*cargs))


LOG_2PI = math.log(2.0 * math.pi)
