"""Operator layer: the reference's Python op API (python/simnets/ops/similarity.py,
python/simnets/ops/mex.py) over the C ABI, with torch tensors as device memory.

Argument names, defaults (None = the registered op default, src/ops/similarity_op.cpp:67-74 and
src/ops/mex_op.cpp:62-73) and error conditions follow the reference; errors surface as
SimnetsError carrying the status code and the reference's message.
"""
import ctypes as C

import torch

from . import _lib
from ._lib import MexAttrs, MexDims, SimilarityAttrs


class SimnetsError(ValueError):
    def __init__(self, code):
        self.code = int(code)
        super().__init__("simnets_hip status %d: %s" % (self.code, _lib.strerror(self.code)))


def _check(code):
    if code != 0:
        raise SimnetsError(code)


def _fill(dst, values, cap):
    values = [int(v) for v in values]
    for i, v in enumerate(values[:cap]):
        dst[i] = v
    return len(values)


_workspaces = {}

# The current stream's handle without building a torch.cuda.Stream object (a few microseconds per call, as much as
# a small kernel runs); the public API where this build of torch lacks the direct accessor.
_raw_stream_of = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device):
    if _raw_stream_of is not None:
        return _raw_stream_of(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _workspace(device, nbytes, stream=None):
    """A scratch tensor per (device, current stream), grown on demand and reused across calls: the kernels that
    use it are ordered on that stream, and calls on different streams never share one."""
    # a buffer first allocated during stream capture lives in that graph's private pool: kept apart from the
    # eager calls' buffer, which a later replay of the graph must not share
    if stream is None:
        stream = _current_stream(device)
    key = (device.index, stream, torch.cuda.is_current_stream_capturing())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


_plans = {}


_PLAIN_KEY_TYPES = frozenset((int, str, bool, type(None), torch.Size))


def _freeze(v):
    if isinstance(v, (list, tuple)):
        return tuple(_freeze(e) for e in v)
    if isinstance(v, dict):
        return tuple(sorted((k, _freeze(e)) for k, e in v.items()))
    return repr(v) if isinstance(v, float) else v


def _key_part(v):
    t = type(v)
    if t in _PLAIN_KEY_TYPES:
        return v
    if t is float:
        return repr(v)
    if t is list or t is tuple:
        for e in v:
            if type(e) is not int:
                return _freeze(v)
        return tuple(v)
    return _freeze(v)


def _plan_key(*parts):
    """Hashable key of shapes and attribute values (floats by repr: NaN out-of-bounds values must compare equal).
    Called on every op call: values of the usual plain types and lists of ints take the short way."""
    return tuple([v if type(v) in _PLAIN_KEY_TYPES else _key_part(v) for v in parts])


def _cached_plan(key, make):
    """Attribute struct, shapes and workspace size of a call: the host-side queries are pure functions of the
    shapes and attributes, and repeated calls of a layer would otherwise spend more time in them than the GPU
    spends in a small kernel."""
    plan = _plans.get(key)
    if plan is None:
        if len(_plans) >= 512:
            _plans.clear()
        plan = _plans[key] = make()
    return plan


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device):
    """Context that makes `device` current for a launch; free when it already is (the usual case)."""
    return _NO_SWITCH if torch.cuda.current_device() == device.index else torch.cuda.device(device)


def _require_cuda_f32(name, t):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if t.dtype != torch.float32:
        raise TypeError("%s must be float32 (the HIP path computes in fp32), got %s" % (name, t.dtype))
    if not t.is_cuda:
        raise RuntimeError("%s must live on a HIP device: simnets_tf_amd has no CPU fallback" % name)
    return t.contiguous()


def similarity_attrs(templates_shape=None, similarity_function=None, blocks=None, strides=None, padding=None,
                     normalization_term=None, normalization_term_fudge=None, ignore_nan_input=None,
                     out_of_bounds_value=None, algo=None, norm_const_every_iteration=False):
    a = SimilarityAttrs()
    _lib.lib().simnets_similarity_attrs_default(C.byref(a))
    if similarity_function is not None:
        if isinstance(similarity_function, bytes):
            similarity_function = similarity_function.decode()
        a.similarity_function = {"L1": _lib.SIM_L1, "L2": _lib.SIM_L2}.get(similarity_function, -1)
    if blocks is not None:
        a.n_blocks = _fill(a.blocks, blocks, 2)
    if strides is not None:
        a.n_strides = _fill(a.strides, strides, 2)
    if padding is not None:
        a.n_padding = _fill(a.padding, padding, 2)
    if normalization_term is not None:
        a.normalization_term = int(bool(normalization_term))
    if normalization_term_fudge is not None:
        a.normalization_term_fudge = float(normalization_term_fudge)
    if ignore_nan_input is not None:
        a.ignore_nan_input = int(bool(ignore_nan_input))
    if out_of_bounds_value is not None:
        a.out_of_bounds_value = float(out_of_bounds_value)
    a.algo = _lib.ALGOS[algo]
    a.norm_const_every_iteration = int(bool(norm_const_every_iteration))
    return a


def similarity_output_shape(input_shape, templates_shape, weights_shape=None, **attrs):
    """Shape function of the op (SimilarityShape); runs every attribute check, needs no GPU."""
    a = similarity_attrs(**attrs)
    I4 = C.c_int * 4
    out = I4()
    weights_shape = templates_shape if weights_shape is None else weights_shape
    _check(_lib.lib().simnets_similarity_out_shape(C.byref(a), I4(*input_shape), I4(*templates_shape),
                                                   I4(*weights_shape), out))
    return tuple(out)


def similarity(input, templates, weights, similarity_function=None, blocks=None, strides=None, padding=None,
               normalization_term=None, normalization_term_fudge=None, ignore_nan_input=None,
               out_of_bounds_value=None, name=None, algo=None, norm_const_every_iteration=False, out=None):
    """Similarity forward; arguments as python/simnets/ops/similarity.py:48-121.

    input [B,C,H,W], templates/weights [O,C,bh,bw] (weights non-negative) -> [B,O,oh,ow].
    Extensions: `algo` in {None,'direct','sqrtw','mfma'} (None: 'sqrtw' for plain L2, else 'direct'), `norm_const_every_iteration`, `out`.
    """
    x = _require_cuda_f32("input", input)
    t = _require_cuda_f32("templates", templates)
    w = _require_cuda_f32("weights", weights)
    if x.dim() != 4 or t.dim() != 4 or w.dim() != 4:
        raise SimnetsError(-15)
    l = _lib.lib()

    def make():
        a = similarity_attrs(similarity_function=similarity_function, blocks=blocks, strides=strides, padding=padding,
                             normalization_term=normalization_term, normalization_term_fudge=normalization_term_fudge,
                             ignore_nan_input=ignore_nan_input, out_of_bounds_value=out_of_bounds_value, algo=algo,
                             norm_const_every_iteration=norm_const_every_iteration)
        I4 = C.c_int * 4
        xs, ts, wsh = I4(*x.shape), I4(*t.shape), I4(*w.shape)
        oshape = I4()
        _check(l.simnets_similarity_out_shape(C.byref(a), xs, ts, wsh, oshape))
        nbytes = C.c_size_t()
        _check(l.simnets_hip_similarity_workspace_bytes(C.byref(a), xs, ts, C.byref(nbytes)))
        return a, xs, ts, wsh, tuple(oshape), nbytes.value

    a, xs, ts, wsh, oshape, nbytes = _cached_plan(
        _plan_key("similarity", x.shape, t.shape, w.shape, similarity_function, blocks, strides, padding,
                  normalization_term, normalization_term_fudge, ignore_nan_input, out_of_bounds_value, algo,
                  norm_const_every_iteration), make)
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes, stream)
    if out is None:
        out = torch.empty(oshape, dtype=torch.float32, device=x.device)
    else:
        assert out.is_contiguous() and tuple(out.shape) == oshape and out.dtype == torch.float32
    with _on_device(x.device):
        _check(l.simnets_hip_similarity_fwd(C.byref(a), xs, ts, wsh, x.data_ptr(), t.data_ptr(), w.data_ptr(),
                                            out.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return out


def _similarity_grad_setup(input, templates, weights, output_grad, kw):
    x = _require_cuda_f32("input", input)
    t = _require_cuda_f32("templates", templates)
    w = _require_cuda_f32("weights", weights)
    g = _require_cuda_f32("output_grad", output_grad)
    if x.dim() != 4 or t.dim() != 4 or w.dim() != 4:
        raise SimnetsError(-15)
    l = _lib.lib()

    def make():
        a = similarity_attrs(**kw)
        I4 = C.c_int * 4
        xs, ts, wsh = I4(*x.shape), I4(*t.shape), I4(*w.shape)
        oshape = I4()
        _check(l.simnets_similarity_out_shape(C.byref(a), xs, ts, wsh, oshape))
        return a, xs, ts, wsh, tuple(oshape)

    a, xs, ts, wsh, oshape = _cached_plan(_plan_key("similarity_grad", x.shape, t.shape, w.shape, *kw.values()), make)
    if tuple(g.shape) != oshape:
        raise SimnetsError(-15)
    return l, a, x, t, w, g, xs, ts, wsh


def similarity_input_grad(input, templates, weights, output_grad, similarity_function=None, blocks=None, strides=None,
                          padding=None, normalization_term=None, normalization_term_fudge=None,
                          ignore_nan_input=None, out_of_bounds_value=None, name=None, algo=None):
    """Gradient of `similarity` w.r.t. its input: the SimilarityInputGrad op
    (python/simnets/ops/similarity.py:33-37, src/ops/similarity_op.cpp:141-156)."""
    l, a, x, t, w, g, xs, ts, wsh = _similarity_grad_setup(input, templates, weights, output_grad, dict(
        similarity_function=similarity_function, blocks=blocks, strides=strides, padding=padding,
        normalization_term=normalization_term, normalization_term_fudge=normalization_term_fudge,
        ignore_nan_input=ignore_nan_input, out_of_bounds_value=out_of_bounds_value, algo=algo))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_similarity_grad_workspace_bytes(C.byref(a), xs, ts, C.byref(nbytes), None))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    dx = torch.empty_like(x)
    with _on_device(x.device):
        _check(l.simnets_hip_similarity_input_grad(C.byref(a), xs, ts, wsh, x.data_ptr(), t.data_ptr(), w.data_ptr(),
                                                   g.data_ptr(), dx.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return dx


def similarity_parameters_grad(input, templates, weights, output_grad, similarity_function=None, blocks=None,
                               strides=None, padding=None, normalization_term=None, normalization_term_fudge=None,
                               ignore_nan_input=None, out_of_bounds_value=None, name=None, algo=None):
    """Gradients of `similarity` w.r.t. templates and weights: the SimilarityParametersGrad op
    (python/simnets/ops/similarity.py:38-44, src/ops/similarity_op.cpp:158-174).

    Extension: `algo='direct'` sums the reference's terms one by one; by default the L2 modes accumulate the
    moments sum g xc, sum g xc^2, sum g about a centre near the templates and combine them at the end."""
    l, a, x, t, w, g, xs, ts, wsh = _similarity_grad_setup(input, templates, weights, output_grad, dict(
        similarity_function=similarity_function, blocks=blocks, strides=strides, padding=padding,
        normalization_term=normalization_term, normalization_term_fudge=normalization_term_fudge,
        ignore_nan_input=ignore_nan_input, out_of_bounds_value=out_of_bounds_value, algo=algo))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_similarity_grad_workspace_bytes(C.byref(a), xs, ts, None, C.byref(nbytes)))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    dt, dw = torch.empty_like(t), torch.empty_like(w)
    with _on_device(x.device):
        _check(l.simnets_hip_similarity_params_grad(C.byref(a), xs, ts, wsh, x.data_ptr(), t.data_ptr(),
                                                    w.data_ptr(), g.data_ptr(), dt.data_ptr(), dw.data_ptr(),
                                                    ws.data_ptr(), ws.numel(), stream))
    return dt, dw


def mex_attrs(num_instances, softmax_mode=None, padding=None, strides=None, blocks=None, epsilon=None,
              blocks_out_of_bounds_value=None, blocks_round_down=None, use_unshared_regions=None,
              shared_offset_region=None, unshared_offset_region=None, normalize_offsets=False):
    a = MexAttrs()
    _lib.lib().simnets_mex_attrs_default(C.byref(a))
    a.num_instances = int(num_instances)
    if softmax_mode is not None:
        a.softmax_mode = int(bool(softmax_mode))
    if padding is not None:
        a.n_padding = _fill(a.padding, padding, 3)
    if strides is not None:
        a.n_strides = _fill(a.strides, strides, 3)
    if blocks is not None:
        a.n_blocks = _fill(a.blocks, blocks, 3)
    if epsilon is not None:
        a.epsilon = float(epsilon)
    if blocks_out_of_bounds_value is not None:
        a.blocks_out_of_bounds_value = float(blocks_out_of_bounds_value)
    if blocks_round_down is not None:
        a.blocks_round_down = int(bool(blocks_round_down))
    if use_unshared_regions is not None:
        a.use_unshared_regions = int(bool(use_unshared_regions))
    if shared_offset_region is not None:
        a.n_shared = _fill(a.shared_offset_region, shared_offset_region, 3)
    if unshared_offset_region is not None:
        a.n_unshared = _fill(a.unshared_offset_region, unshared_offset_region, 3)
    a.normalize_offsets = int(bool(normalize_offsets))
    return a


def mex_dims(image_chw, num_instances, **attrs):
    """MexDimensionsData::CalculateDimensions as a dict; needs no GPU."""
    a = mex_attrs(num_instances, **attrs)
    d = MexDims()
    _check(_lib.lib().simnets_mex_calc_dims(C.byref(a), (C.c_int * 3)(*image_chw), C.byref(d)))
    return d.asdict()


def mex_output_shape(input_shape, num_instances, **attrs):
    """(output_shape, offsets_shape) of the op (MexShape + the offsets variable of the Keras layer)."""
    a = mex_attrs(num_instances, **attrs)
    o, f = (C.c_int * 4)(), (C.c_int * 5)()
    _check(_lib.lib().simnets_mex_out_shape(C.byref(a), (C.c_int * 4)(*input_shape), C.byref(o), C.byref(f)))
    return tuple(o), tuple(f)


def _mex_dims_helper(input_dim, num_instances, blocks, padding=[0], strides=[1], blocks_round_down=True,
                     use_unshared_regions=True, shared_offset_region=[-1], unshared_offset_region=[-1]):
    """Number of offset regions of a MEX layer over an image of `input_dim` = (C, H, W).

    Same name, argument meaning and C call (`get_mex_offsets_nregions`, every list passed as a length followed by
    an int array) as the reference's helper, python/simnets/ops/mex.py:17-38.
    """
    def counted(values):
        ints = [int(v) for v in values]
        return C.c_int(len(ints)), (C.c_int * len(ints))(*ints)

    flags = (C.c_int(int(num_instances)), C.c_int(int(bool(blocks_round_down))),
             C.c_int(int(bool(use_unshared_regions))))
    call = counted(input_dim) + counted(padding) + counted(strides) + flags + counted(blocks) + \
        counted(shared_offset_region) + counted(unshared_offset_region)
    return _lib.lib().get_mex_offsets_nregions(*call)


def _expand_dim_specification(image_shape, dim_spec):
    """A (channels, rows, columns) triple from a 2- or 3-entry specification: a 2-entry one covers all channels,
    and an entry of -1 stands for the whole extent of the image (NCHW, or CHW without the batch) along that axis.
    Behaviour of python/simnets/ops/mex.py:84-111.
    """
    spec = list(dim_spec)
    if len(spec) not in (2, 3):
        raise ValueError('Bad dimensions specifications, should be a list of two or three, got %s' % dim_spec)
    chw = list(image_shape)[-3:]
    if len(spec) == 2:
        spec.insert(0, -1)
    return [extent if want == -1 else want for want, extent in zip(spec, chw)]


def mex(input, offsets, num_instances, softmax_mode=None, padding=None, strides=None, blocks=None, epsilon=None,
        blocks_out_of_bounds_value=None, blocks_round_down=None, use_unshared_regions=None,
        shared_offset_region=None, unshared_offset_region=None, name=None, normalize_offsets=False, out=None):
    """MEX forward; arguments as python/simnets/ops/mex.py:114-195.

    input [B,C,H,W], offsets [num_regions, num_instances, bc, bh, bw] -> [B, channels_out*num_instances, oh, ow].
    Extension: `normalize_offsets` applies the Keras layer's logsumexp normalisation on the device.
    """
    x = _require_cuda_f32("input", input)
    off = _require_cuda_f32("offsets", offsets)
    if x.dim() != 4:
        raise SimnetsError(-15)
    l = _lib.lib()

    def make():
        a = mex_attrs(num_instances, softmax_mode=softmax_mode, padding=padding, strides=strides, blocks=blocks,
                      epsilon=epsilon, blocks_out_of_bounds_value=blocks_out_of_bounds_value,
                      blocks_round_down=blocks_round_down, use_unshared_regions=use_unshared_regions,
                      shared_offset_region=shared_offset_region, unshared_offset_region=unshared_offset_region,
                      normalize_offsets=normalize_offsets)
        xs = (C.c_int * 4)(*x.shape)
        oshape = (C.c_int * 4)()
        _check(l.simnets_mex_out_shape(C.byref(a), xs, C.byref(oshape), None))
        nbytes = C.c_size_t()
        _check(l.simnets_hip_mex_workspace_bytes(C.byref(a), xs, C.byref(nbytes)))
        return a, xs, tuple(oshape), nbytes.value

    a, xs, oshape, nbytes = _cached_plan(
        _plan_key("mex", x.shape, num_instances, softmax_mode, padding, strides, blocks, epsilon,
                  blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                  unshared_offset_region, normalize_offsets), make)
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes, stream)
    if out is None:
        out = torch.empty(oshape, dtype=torch.float32, device=x.device)
    else:
        assert out.is_contiguous() and tuple(out.shape) == oshape and out.dtype == torch.float32
    with _on_device(x.device):
        _check(l.simnets_hip_mex_fwd(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), out.data_ptr(),
                                     ws.data_ptr(), ws.numel(), stream))
    return out


def _mex_grad_setup(input, offsets, output, output_grad, num_instances, kw):
    x = _require_cuda_f32("input", input)
    off = _require_cuda_f32("offsets", offsets)
    y = _require_cuda_f32("output", output)
    g = _require_cuda_f32("output_grad", output_grad)
    if x.dim() != 4:
        raise SimnetsError(-15)
    l = _lib.lib()

    def make():
        a = mex_attrs(num_instances, **kw)
        xs = (C.c_int * 4)(*x.shape)
        oshape = (C.c_int * 4)()
        _check(l.simnets_mex_out_shape(C.byref(a), xs, C.byref(oshape), None))
        return a, xs, tuple(oshape)

    a, xs, oshape = _cached_plan(_plan_key("mex_grad", x.shape, num_instances, *kw.values()), make)
    if tuple(y.shape) != oshape or tuple(g.shape) != oshape:
        raise SimnetsError(-15)
    return l, a, x, off, y, g, xs


def mex_input_grad(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None, strides=None,
                   blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                   use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                   normalize_offsets=False):
    """Gradient of `mex` w.r.t. its input: the MexInputGrad op (python/simnets/ops/mex.py:63-71,
    src/ops/mex_op.cpp:134-151).  `output` is the forward result."""
    l, a, x, off, y, g, xs = _mex_grad_setup(input, offsets, output, output_grad, num_instances, dict(
        softmax_mode=softmax_mode, padding=padding, strides=strides, blocks=blocks, epsilon=epsilon,
        blocks_out_of_bounds_value=blocks_out_of_bounds_value, blocks_round_down=blocks_round_down,
        use_unshared_regions=use_unshared_regions, shared_offset_region=shared_offset_region,
        unshared_offset_region=unshared_offset_region, normalize_offsets=normalize_offsets))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_mex_grad_workspace_bytes(C.byref(a), xs, C.byref(nbytes), None))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    dx = torch.empty_like(x)
    with _on_device(x.device):
        _check(l.simnets_hip_mex_input_grad(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), y.data_ptr(),
                                            g.data_ptr(), dx.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return dx


def mex_offsets_grad(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None,
                     strides=None, blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                     use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                     normalize_offsets=False):
    """Gradient of `mex` w.r.t. its offsets: the MexOffsetsGrad op (python/simnets/ops/mex.py:73-80,
    src/ops/mex_op.cpp:153-170).  With `normalize_offsets` the gradient is w.r.t. the raw offsets."""
    l, a, x, off, y, g, xs = _mex_grad_setup(input, offsets, output, output_grad, num_instances, dict(
        softmax_mode=softmax_mode, padding=padding, strides=strides, blocks=blocks, epsilon=epsilon,
        blocks_out_of_bounds_value=blocks_out_of_bounds_value, blocks_round_down=blocks_round_down,
        use_unshared_regions=use_unshared_regions, shared_offset_region=shared_offset_region,
        unshared_offset_region=unshared_offset_region, normalize_offsets=normalize_offsets))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_mex_grad_workspace_bytes(C.byref(a), xs, None, C.byref(nbytes)))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    doff = torch.empty_like(off)
    with _on_device(x.device):
        _check(l.simnets_hip_mex_offsets_grad(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), y.data_ptr(),
                                              g.data_ptr(), doff.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return doff


def mex_grads(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None, strides=None,
              blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
              use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
              normalize_offsets=False):
    """`(mex_input_grad(...), mex_offsets_grad(...))` as one call of the library: the same results bit for bit, with
    the work both share (offsets normalisation and packing, per-pixel factors) done once.  What the gradient
    registered for the Mex op (python/simnets/ops/mex.py:47-81) computes."""
    l, a, x, off, y, g, xs = _mex_grad_setup(input, offsets, output, output_grad, num_instances, dict(
        softmax_mode=softmax_mode, padding=padding, strides=strides, blocks=blocks, epsilon=epsilon,
        blocks_out_of_bounds_value=blocks_out_of_bounds_value, blocks_round_down=blocks_round_down,
        use_unshared_regions=use_unshared_regions, shared_offset_region=shared_offset_region,
        unshared_offset_region=unshared_offset_region, normalize_offsets=normalize_offsets))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_mex_grads_workspace_bytes(C.byref(a), xs, C.byref(nbytes)))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    dx, doff = torch.empty_like(x), torch.empty_like(off)
    with _on_device(x.device):
        _check(l.simnets_hip_mex_grads(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), y.data_ptr(),
                                       g.data_ptr(), dx.data_ptr(), doff.data_ptr(), ws.data_ptr(), ws.numel(),
                                       stream))
    return dx, doff


def mex_sum_pool(input, offsets, num_instances, pool_size=(2, 2), softmax_mode=None, padding=None, strides=None,
                 blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                 use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                 normalize_offsets=False, out=None):
    """`sum_pooling(mex(...), pool_size)` as one call (forward only): the MEX layer + pooling pair of the reference's
    networks (README.md:108-129).  With unshared offset regions equal to the pooling window and a finite epsilon a
    single kernel writes only the pooled tensor; other geometries run the two kernels through scratch memory."""
    x = _require_cuda_f32("input", input)
    off = _require_cuda_f32("offsets", offsets)
    if x.dim() != 4:
        raise SimnetsError(-15)
    ph, pw = int(pool_size[0]), int(pool_size[1])
    l = _lib.lib()

    def make():
        a = mex_attrs(num_instances, softmax_mode=softmax_mode, padding=padding, strides=strides, blocks=blocks,
                      epsilon=epsilon, blocks_out_of_bounds_value=blocks_out_of_bounds_value,
                      blocks_round_down=blocks_round_down, use_unshared_regions=use_unshared_regions,
                      shared_offset_region=shared_offset_region, unshared_offset_region=unshared_offset_region,
                      normalize_offsets=normalize_offsets)
        xs = (C.c_int * 4)(*x.shape)
        oshape = (C.c_int * 4)()
        _check(l.simnets_mex_out_shape(C.byref(a), xs, C.byref(oshape), None))
        nbytes = C.c_size_t()
        _check(l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(a), xs, ph, pw, C.byref(nbytes)))
        return a, xs, (oshape[0], oshape[1], oshape[2] // ph, oshape[3] // pw), nbytes.value

    a, xs, pshape, nbytes = _cached_plan(
        _plan_key("mex_sum_pool", x.shape, num_instances, ph, pw, softmax_mode, padding, strides, blocks, epsilon,
                  blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                  unshared_offset_region, normalize_offsets), make)
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes, stream)
    if out is None:
        out = torch.empty(pshape, dtype=torch.float32, device=x.device)
    else:
        assert out.is_contiguous() and tuple(out.shape) == pshape and out.dtype == torch.float32
    with _on_device(x.device):
        _check(l.simnets_hip_mex_sum_pool_fwd(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), ph, pw,
                                              out.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return out


def similarity_mex_sum_pool(input, templates, weights, offsets, num_instances, pool_size=(2, 2), similarity=None,
                            mex=None, out=None):
    """`sum_pooling(mex(similarity(input, templates, weights, **similarity), offsets, num_instances, **mex), pool_size)`
    as one call (forward only): the first layers of the reference's networks (README.md:108-129).  `similarity` and
    `mex` are dicts of the keyword arguments of those two functions.  One kernel when the MEX blocks are
    [templates, 1, 1], the offsets are unshared over exactly the pooling window and a Similarity patch has at most 16
    elements; the separate kernels through scratch memory otherwise."""
    x = _require_cuda_f32("input", input)
    t = _require_cuda_f32("templates", templates)
    w = _require_cuda_f32("weights", weights)
    off = _require_cuda_f32("offsets", offsets)
    if x.dim() != 4 or t.dim() != 4 or tuple(w.shape) != tuple(t.shape):
        raise SimnetsError(-15)
    sa = similarity_attrs(**(similarity or {}))
    ma = mex_attrs(num_instances, **(mex or {}))
    ph, pw = int(pool_size[0]), int(pool_size[1])
    l = _lib.lib()
    I4 = C.c_int * 4
    xs, ts = I4(*x.shape), I4(*t.shape)
    mid, oshape = I4(), I4()
    _check(l.simnets_similarity_out_shape(C.byref(sa), xs, ts, ts, mid))
    _check(l.simnets_mex_out_shape(C.byref(ma), mid, C.byref(oshape), None))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_similarity_mex_sum_pool_workspace_bytes(C.byref(sa), xs, ts, C.byref(ma), ph, pw,
                                                                 C.byref(nbytes)))
    stream = _current_stream(x.device)
    ws = _workspace(x.device, nbytes.value, stream)
    pshape = (oshape[0], oshape[1], oshape[2] // ph, oshape[3] // pw)
    if out is None:
        out = torch.empty(pshape, dtype=torch.float32, device=x.device)
    else:
        assert out.is_contiguous() and tuple(out.shape) == pshape and out.dtype == torch.float32
    with _on_device(x.device):
        _check(l.simnets_hip_similarity_mex_sum_pool_fwd(C.byref(sa), xs, ts, x.data_ptr(), t.data_ptr(), w.data_ptr(),
                                                         C.byref(ma), off.data_ptr(), off.numel(), ph, pw,
                                                         out.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return out


def sum_pooling(input, pool_size=(2, 2), out=None):
    """Non-overlapping 'valid' sum pooling: the AveragePooling2D * area glue of the reference's
    missing-data example (README.md:108-111)."""
    x = _require_cuda_f32("input", input)
    if x.dim() != 4:
        raise SimnetsError(-15)
    ph, pw = int(pool_size[0]), int(pool_size[1])
    B, Cc, H, W = x.shape
    oshape = (B, Cc, H // max(ph, 1), W // max(pw, 1))
    if out is None:
        out = torch.empty(oshape, dtype=torch.float32, device=x.device)
    else:
        assert out.is_contiguous() and tuple(out.shape) == oshape and out.dtype == torch.float32 \
            and out.device == x.device
    with _on_device(x.device):
        stream = _current_stream(x.device)
        _check(_lib.lib().simnets_hip_sum_pool_fwd((C.c_int * 4)(*x.shape), ph, pw, x.data_ptr(), out.data_ptr(),
                                                   stream))
    return out


def sum_pooling_input_grad(output_grad, input_shape, pool_size=(2, 2)):
    """Gradient of `sum_pooling` w.r.t. its input: each element receives its window's gradient, elements of a
    dropped trailing row or column receive 0."""
    g = _require_cuda_f32("output_grad", output_grad)
    ph, pw = int(pool_size[0]), int(pool_size[1])
    B, Cc, H, W = [int(v) for v in input_shape]
    if tuple(g.shape) != (B, Cc, H // max(ph, 1), W // max(pw, 1)):
        raise SimnetsError(-15)
    dx = torch.empty((B, Cc, H, W), dtype=torch.float32, device=g.device)
    with _on_device(g.device):
        stream = _current_stream(g.device)
        _check(_lib.lib().simnets_hip_sum_pool_input_grad((C.c_int * 4)(B, Cc, H, W), ph, pw, g.data_ptr(),
                                                          dx.data_ptr(), stream))
    return dx


# ---------------------------------------------------------------------------------------------------------------
# Prepared forward calls: the work that depends on the parameters alone (packing the templates / weights / offsets
# for the kernels) done once, for callers whose parameters stay fixed across calls (inference).  The reference
# redoes its counterpart on every call (interlace, src/kernels/similarity_kernel_gpu.cu:70; offsets copy,
# src/kernels/mex_kernel_gpu.cu:98-112).
# ---------------------------------------------------------------------------------------------------------------
class Prepared:
    """A forward operator bound to packed parameters and one input shape; call it with the input.

    Made by `similarity_prepare`, `mex_prepare`, `mex_sum_pool_prepare` or `similarity_mex_sum_pool_prepare`.  The
    results are those of the plain call, bit for bit.  The buffer also serves as the per-call scratch of the kernels,
    so calls of one object must not overlap (keep them on one stream).  Later changes of the parameter tensors are
    not seen: prepare again.
    """

    def __init__(self, input_shape, output_shape, buffer, run):
        self.input_shape = torch.Size(int(v) for v in input_shape)
        self.output_shape = tuple(int(v) for v in output_shape)
        self.buffer = buffer
        self._run = run
        self._device = buffer.device
        self._index = buffer.device.index

    def __call__(self, input, out=None):
        # (kept short: for the small layers this host code, not the kernel, bounds the call rate)
        x = input
        if x.shape != self.input_shape or x.device != self._device or x.dtype is not torch.float32:
            _require_cuda_f32("input", x)
            raise SimnetsError(-15)
        if not x.is_contiguous():
            x = x.contiguous()
        if out is None:
            out = torch.empty(self.output_shape, dtype=torch.float32, device=self._device)
        elif not (out.is_contiguous() and tuple(out.shape) == self.output_shape and out.dtype is torch.float32
                  and out.device == self._device):
            raise ValueError("out must be a contiguous float32 tensor of shape %s on %s"
                             % (self.output_shape, self._device))
        if torch.cuda.current_device() == self._index:
            code = self._run(x.data_ptr(), out.data_ptr(), _current_stream(self._device))
        else:
            with torch.cuda.device(self._device):
                code = self._run(x.data_ptr(), out.data_ptr(), _current_stream(self._device))
        if code != 0:
            raise SimnetsError(code)
        return out


def _prepared_buffer(device, nbytes):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def similarity_prepare(input_shape, templates, weights, similarity_function=None, blocks=None, strides=None,
                       padding=None, normalization_term=None, normalization_term_fudge=None, ignore_nan_input=None,
                       out_of_bounds_value=None, algo=None, norm_const_every_iteration=False):
    """`similarity(input, templates, weights, ...)` with the parameter packing done here, once: returns a `Prepared`
    whose call takes the input (of exactly `input_shape`, batch size included) and runs only the forward kernels."""
    t = _require_cuda_f32("templates", templates)
    w = _require_cuda_f32("weights", weights)
    if len(input_shape) != 4 or t.dim() != 4 or w.dim() != 4:
        raise SimnetsError(-15)
    l = _lib.lib()
    a = similarity_attrs(similarity_function=similarity_function, blocks=blocks, strides=strides, padding=padding,
                         normalization_term=normalization_term, normalization_term_fudge=normalization_term_fudge,
                         ignore_nan_input=ignore_nan_input, out_of_bounds_value=out_of_bounds_value, algo=algo,
                         norm_const_every_iteration=norm_const_every_iteration)
    I4 = C.c_int * 4
    xs, ts, wsh = I4(*[int(v) for v in input_shape]), I4(*t.shape), I4(*w.shape)
    oshape = I4()
    _check(l.simnets_similarity_out_shape(C.byref(a), xs, ts, wsh, oshape))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_similarity_workspace_bytes(C.byref(a), xs, ts, C.byref(nbytes)))
    buf = _prepared_buffer(t.device, nbytes.value)
    with _on_device(t.device):
        stream = _current_stream(t.device)
        _check(l.simnets_hip_similarity_prepare(C.byref(a), xs, ts, wsh, t.data_ptr(), w.data_ptr(), buf.data_ptr(),
                                                buf.numel(), stream))

    fn, ar, bp, bn = l.simnets_hip_similarity_fwd_prepared, C.byref(a), buf.data_ptr(), buf.numel()

    def run(x_ptr, out_ptr, stream):
        return fn(ar, xs, ts, x_ptr, bp, bn, out_ptr, stream)
    return Prepared(input_shape, tuple(oshape), buf, run)


def mex_prepare(input_shape, offsets, num_instances, normalize_offsets=False, **attrs):
    """`mex(input, offsets, num_instances, ...)` with the offsets packed here, once (keyword arguments as `mex`)."""
    off = _require_cuda_f32("offsets", offsets)
    if len(input_shape) != 4:
        raise SimnetsError(-15)
    l = _lib.lib()
    a = mex_attrs(num_instances, normalize_offsets=normalize_offsets, **attrs)
    xs = (C.c_int * 4)(*[int(v) for v in input_shape])
    oshape = (C.c_int * 4)()
    _check(l.simnets_mex_out_shape(C.byref(a), xs, C.byref(oshape), None))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_mex_workspace_bytes(C.byref(a), xs, C.byref(nbytes)))
    buf = _prepared_buffer(off.device, nbytes.value)
    with _on_device(off.device):
        stream = _current_stream(off.device)
        _check(l.simnets_hip_mex_prepare(C.byref(a), xs, off.data_ptr(), off.numel(), buf.data_ptr(), buf.numel(),
                                         stream))

    fn, ar, bp, bn = l.simnets_hip_mex_fwd_prepared, C.byref(a), buf.data_ptr(), buf.numel()

    def run(x_ptr, out_ptr, stream):
        return fn(ar, xs, x_ptr, bp, bn, out_ptr, stream)
    return Prepared(input_shape, tuple(oshape), buf, run)


def mex_sum_pool_prepare(input_shape, offsets, num_instances, pool_size=(2, 2), normalize_offsets=False, **attrs):
    """`mex_sum_pool(input, offsets, num_instances, pool_size, ...)` with the offsets packed here, once."""
    off = _require_cuda_f32("offsets", offsets)
    if len(input_shape) != 4:
        raise SimnetsError(-15)
    l = _lib.lib()
    a = mex_attrs(num_instances, normalize_offsets=normalize_offsets, **attrs)
    ph, pw = int(pool_size[0]), int(pool_size[1])
    xs = (C.c_int * 4)(*[int(v) for v in input_shape])
    oshape = (C.c_int * 4)()
    _check(l.simnets_mex_out_shape(C.byref(a), xs, C.byref(oshape), None))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(a), xs, ph, pw, C.byref(nbytes)))
    buf = _prepared_buffer(off.device, nbytes.value)
    with _on_device(off.device):
        stream = _current_stream(off.device)
        _check(l.simnets_hip_mex_sum_pool_prepare(C.byref(a), xs, off.data_ptr(), off.numel(), ph, pw, buf.data_ptr(),
                                                  buf.numel(), stream))

    fn, ar, bp, bn = l.simnets_hip_mex_sum_pool_fwd_prepared, C.byref(a), buf.data_ptr(), buf.numel()

    def run(x_ptr, out_ptr, stream):
        return fn(ar, xs, x_ptr, ph, pw, bp, bn, out_ptr, stream)
    return Prepared(input_shape, (oshape[0], oshape[1], oshape[2] // ph, oshape[3] // pw), buf, run)


def similarity_mex_sum_pool_prepare(input_shape, templates, weights, offsets, num_instances, pool_size=(2, 2),
                                    similarity=None, mex=None):
    """`similarity_mex_sum_pool(input, templates, weights, offsets, ...)` with all parameters packed here, once."""
    t = _require_cuda_f32("templates", templates)
    w = _require_cuda_f32("weights", weights)
    off = _require_cuda_f32("offsets", offsets)
    if len(input_shape) != 4 or t.dim() != 4 or tuple(w.shape) != tuple(t.shape):
        raise SimnetsError(-15)
    sa = similarity_attrs(**(similarity or {}))
    ma = mex_attrs(num_instances, **(mex or {}))
    ph, pw = int(pool_size[0]), int(pool_size[1])
    l = _lib.lib()
    I4 = C.c_int * 4
    xs, ts = I4(*[int(v) for v in input_shape]), I4(*t.shape)
    mid, oshape = I4(), I4()
    _check(l.simnets_similarity_out_shape(C.byref(sa), xs, ts, ts, mid))
    _check(l.simnets_mex_out_shape(C.byref(ma), mid, C.byref(oshape), None))
    nbytes = C.c_size_t()
    _check(l.simnets_hip_similarity_mex_sum_pool_workspace_bytes(C.byref(sa), xs, ts, C.byref(ma), ph, pw,
                                                                 C.byref(nbytes)))
    buf = _prepared_buffer(t.device, nbytes.value)
    with _on_device(t.device):
        stream = _current_stream(t.device)
        _check(l.simnets_hip_similarity_mex_sum_pool_prepare(C.byref(sa), xs, ts, t.data_ptr(), w.data_ptr(),
                                                             C.byref(ma), off.data_ptr(), off.numel(), ph, pw,
                                                             buf.data_ptr(), buf.numel(), stream))

    fn, sr, mr, bp, bn = (l.simnets_hip_similarity_mex_sum_pool_fwd_prepared, C.byref(sa), C.byref(ma), buf.data_ptr(),
                          buf.numel())

    def run(x_ptr, out_ptr, stream):
        return fn(sr, xs, ts, x_ptr, mr, ph, pw, bp, bn, out_ptr, stream)
    return Prepared(input_shape, (oshape[0], oshape[1], oshape[2] // ph, oshape[3] // pw), buf, run)
