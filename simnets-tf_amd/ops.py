"""Operator layer: the reference's Python op API (python/simnets/ops/similarity.py,
python/simnets/ops/mex.py) with torch tensors as device memory.

Argument names, defaults (None = the registered op default, src/ops/similarity_op.cpp:67-74 and
src/ops/mex_op.cpp:62-73) and error conditions follow the reference; errors surface as
SimnetsError carrying the status code and the reference's message.

Every call that launches work is a thin front of the compiled operator layer (csrc/op_layer.cpp, the module
`_simnets_native`), which checks the tensors, fills the attribute structs, allocates outputs and scratch and calls the
C ABI of libsimnets_hip.so.  The host-only queries (shapes, dimensions, attribute structs) go to the C ABI through
ctypes.
"""
import ctypes as C

import torch

from . import _lib
from . import _native
from ._lib import MexAttrs, MexDims, SimilarityAttrs

_n = _native.module()


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


# The current stream's handle without building a torch.cuda.Stream object (a few microseconds per call, as much as
# a small kernel runs); the public API where this build of torch lacks the direct accessor.
_raw_stream_of = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device):
    if _raw_stream_of is not None:
        return _raw_stream_of(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _freeze(v):
    """Hashable form of an attribute value (floats by repr: NaN out-of-bounds values must compare equal)."""
    if isinstance(v, (list, tuple)):
        return tuple(_freeze(e) for e in v)
    if isinstance(v, dict):
        return tuple(sorted((k, _freeze(e)) for k, e in v.items()))
    return repr(v) if isinstance(v, float) else v


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
    return _n.similarity(input, templates, weights, similarity_function, blocks, strides, padding, normalization_term,
                         normalization_term_fudge, ignore_nan_input, out_of_bounds_value, algo,
                         bool(norm_const_every_iteration), out)


def similarity_input_grad(input, templates, weights, output_grad, similarity_function=None, blocks=None, strides=None,
                          padding=None, normalization_term=None, normalization_term_fudge=None,
                          ignore_nan_input=None, out_of_bounds_value=None, name=None, algo=None):
    """Gradient of `similarity` w.r.t. its input: the SimilarityInputGrad op
    (python/simnets/ops/similarity.py:33-37, src/ops/similarity_op.cpp:141-156)."""
    return _n.similarity_input_grad(input, templates, weights, output_grad, similarity_function, blocks, strides, padding,
                                    normalization_term, normalization_term_fudge, ignore_nan_input, out_of_bounds_value,
                                    algo)


def similarity_parameters_grad(input, templates, weights, output_grad, similarity_function=None, blocks=None,
                               strides=None, padding=None, normalization_term=None, normalization_term_fudge=None,
                               ignore_nan_input=None, out_of_bounds_value=None, name=None, algo=None):
    """Gradients of `similarity` w.r.t. templates and weights: the SimilarityParametersGrad op
    (python/simnets/ops/similarity.py:38-44, src/ops/similarity_op.cpp:158-174).

    Extension: `algo='direct'` sums the reference's terms one by one; by default the L2 modes accumulate the
    moments sum g xc, sum g xc^2, sum g about a centre near the templates and combine them at the end."""
    return _n.similarity_parameters_grad(input, templates, weights, output_grad, similarity_function, blocks, strides,
                                         padding, normalization_term, normalization_term_fudge, ignore_nan_input,
                                         out_of_bounds_value, algo)


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
    return _n.mex(input, offsets, int(num_instances), softmax_mode, padding, strides, blocks, epsilon,
                  blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                  unshared_offset_region, bool(normalize_offsets), out)


def mex_input_grad(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None, strides=None,
                   blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                   use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                   normalize_offsets=False):
    """Gradient of `mex` w.r.t. its input: the MexInputGrad op (python/simnets/ops/mex.py:63-71,
    src/ops/mex_op.cpp:134-151).  `output` is the forward result."""
    return _n.mex_input_grad(input, offsets, output, output_grad, int(num_instances), softmax_mode, padding, strides, blocks, epsilon,
                          blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                          unshared_offset_region, bool(normalize_offsets))


def mex_offsets_grad(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None, strides=None,
                     blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                     use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                     normalize_offsets=False):
    """Gradient of `mex` w.r.t. its offsets: the MexOffsetsGrad op (python/simnets/ops/mex.py:73-80,
    src/ops/mex_op.cpp:153-170).  With `normalize_offsets` the gradient is w.r.t. the raw offsets."""
    return _n.mex_offsets_grad(input, offsets, output, output_grad, int(num_instances), softmax_mode, padding, strides, blocks, epsilon,
                            blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                            unshared_offset_region, bool(normalize_offsets))


def mex_grads(input, offsets, output, output_grad, num_instances, softmax_mode=None, padding=None, strides=None,
              blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
              use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
              normalize_offsets=False, saved=None):
    """`(mex_input_grad(...), mex_offsets_grad(...))` as one call of the library: the same results bit for bit, with
    the work both share (offsets normalisation and packing, per-pixel factors) done once.  What the gradient
    registered for the Mex op (python/simnets/ops/mex.py:47-81) computes.  `saved`: what `mex_saving` returned for
    the same input shape, attributes and offsets values; the call then packs no offsets."""
    return _n.mex_grads(input, offsets, output, output_grad, int(num_instances), softmax_mode, padding, strides, blocks, epsilon,
                     blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                     unshared_offset_region, bool(normalize_offsets), saved)


def mex_saving(input, offsets, num_instances, softmax_mode=None, padding=None, strides=None, blocks=None, epsilon=None,
               blocks_out_of_bounds_value=None, blocks_round_down=None, use_unshared_regions=None,
               shared_offset_region=None, unshared_offset_region=None, name=None, normalize_offsets=False):
    """`mex(...)` for a training step: `(output, saved)`, where `saved` (a byte tensor, empty when the layer's
    gradient kernels have no use for one) holds the offsets as the gradient kernels read them, written by the launch
    that re-orders them for the forward kernel; `mex_grads(..., saved=saved)` then packs nothing.  The registered
    gradient of the Mex op runs on the forward op's inputs (python/simnets/ops/mex.py:47-81)."""
    return _n.mex_saving(input, offsets, int(num_instances), softmax_mode, padding, strides, blocks, epsilon,
                         blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions, shared_offset_region,
                         unshared_offset_region, bool(normalize_offsets))


def mex_sum_pool(input, offsets, num_instances, pool_size=(2, 2), softmax_mode=None, padding=None, strides=None,
                 blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                 use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                 normalize_offsets=False, out=None):
    """`sum_pooling(mex(...), pool_size)` as one call (forward only): the MEX layer + pooling pair of the reference's
    networks (README.md:108-129).  With unshared offset regions equal to the pooling window and a finite epsilon a
    single kernel writes only the pooled tensor; other geometries run the two kernels through scratch memory."""
    return _n.mex_sum_pool(input, offsets, int(num_instances), int(pool_size[0]), int(pool_size[1]), softmax_mode, padding,
                           strides, blocks, epsilon, blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions,
                           shared_offset_region, unshared_offset_region, bool(normalize_offsets), out)


def mex_sum_pool_both(input, offsets, num_instances, pool_size=(2, 2), softmax_mode=None, padding=None, strides=None,
                      blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                      use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                      normalize_offsets=False):
    """`(mex(...), sum_pooling(mex(...), pool_size))` from the one call `mex_sum_pool` makes: the form a training step
    uses, since the MEX gradient operators take the output before pooling (src/ops/mex_op.cpp:134-170)."""
    return _n.mex_sum_pool_both(input, offsets, int(num_instances), int(pool_size[0]), int(pool_size[1]), softmax_mode,
                                padding, strides, blocks, epsilon, blocks_out_of_bounds_value, blocks_round_down,
                                use_unshared_regions, shared_offset_region, unshared_offset_region,
                                bool(normalize_offsets))


def mex_sum_pool_saving(input, offsets, num_instances, pool_size=(2, 2), softmax_mode=None, padding=None, strides=None,
                        blocks=None, epsilon=None, blocks_out_of_bounds_value=None, blocks_round_down=None,
                        use_unshared_regions=None, shared_offset_region=None, unshared_offset_region=None, name=None,
                        normalize_offsets=False):
    """`mex_sum_pool_both(...)` + `saved` as `mex_saving` returns it: `(mex_output, pooled, saved)`, for
    `mex_sum_pool_grads(..., saved=saved)`."""
    return _n.mex_sum_pool_saving(input, offsets, int(num_instances), int(pool_size[0]), int(pool_size[1]), softmax_mode,
                                  padding, strides, blocks, epsilon, blocks_out_of_bounds_value, blocks_round_down,
                                  use_unshared_regions, shared_offset_region, unshared_offset_region,
                                  bool(normalize_offsets))


def mex_sum_pool_grads(input, offsets, mex_output, pooled_output_grad, num_instances, pool_size=(2, 2), want_input=True,
                       want_offsets=True, softmax_mode=None, padding=None, strides=None, blocks=None, epsilon=None,
                       blocks_out_of_bounds_value=None, blocks_round_down=None, use_unshared_regions=None,
                       shared_offset_region=None, unshared_offset_region=None, name=None, normalize_offsets=False,
                       saved=None):
    """The gradients of `mex_sum_pool` w.r.t. (input, offsets) from the gradient of the POOLED output and the MEX
    output before pooling (`mex_sum_pool_both`'s first result): `mex_grads(input, offsets, mex_output,
    sum_pooling_input_grad(pooled_output_grad, ...))` in one call, without the expanded gradient tensor where every
    output pixel has a window (2 x 2 pooling of an even-sized map, one output channel per instance).  A gradient that is not wanted comes back as None."""
    gi, go = _n.mex_sum_pool_grads(input, offsets, mex_output, pooled_output_grad, int(num_instances), int(pool_size[0]),
                                   int(pool_size[1]), bool(want_input), bool(want_offsets), softmax_mode, padding, strides,
                                   blocks, epsilon, blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions,
                                   shared_offset_region, unshared_offset_region, bool(normalize_offsets), saved)
    return (gi if want_input else None), (go if want_offsets else None)


def similarity_mex_sum_pool(input, templates, weights, offsets, num_instances, pool_size=(2, 2), similarity=None,
                            mex=None, out=None):
    """`sum_pooling(mex(similarity(input, templates, weights, **similarity), offsets, num_instances, **mex), pool_size)`
    as one call (forward only): the first layers of the reference's networks (README.md:108-129).  `similarity` and
    `mex` are dicts of the keyword arguments of those two functions.  One kernel when the MEX blocks are
    [templates, 1, 1], the offsets are unshared over exactly the pooling window and a Similarity patch has at most 16
    elements; the separate kernels through scratch memory otherwise."""
    return _n.similarity_mex_sum_pool(input, templates, weights, offsets, int(num_instances), int(pool_size[0]),
                                      int(pool_size[1]), _sim_dict(similarity), _mex_dict(mex), out)


def sum_pooling(input, pool_size=(2, 2), out=None):
    """Non-overlapping 'valid' sum pooling: the AveragePooling2D * area glue of the reference's
    missing-data example (README.md:108-111)."""
    return _n.sum_pooling(input, int(pool_size[0]), int(pool_size[1]), out)


def sum_pooling_input_grad(output_grad, input_shape, pool_size=(2, 2)):
    """Gradient of `sum_pooling` w.r.t. its input: each element receives its window's gradient, elements of a
    dropped trailing row or column receive 0."""
    return _n.sum_pooling_input_grad(output_grad, [int(v) for v in input_shape], int(pool_size[0]), int(pool_size[1]))


# ---------------------------------------------------------------------------------------------------------------
# Prepared forward calls: the work that depends on the parameters alone (packing the templates / weights / offsets
# for the kernels) done once, for callers whose parameters stay fixed across calls (inference).  The reference
# redoes its counterpart on every call (interlace, src/kernels/similarity_kernel_gpu.cu:70; offsets copy,
# src/kernels/mex_kernel_gpu.cu:98-112).
# ---------------------------------------------------------------------------------------------------------------
Prepared = _n.Prepared


_SIM_KEYS = ("similarity_function", "blocks", "strides", "padding", "normalization_term", "normalization_term_fudge",
             "ignore_nan_input", "out_of_bounds_value", "algo", "norm_const_every_iteration")
_MEX_KEYS = ("softmax_mode", "padding", "strides", "blocks", "epsilon", "blocks_out_of_bounds_value",
             "blocks_round_down", "use_unshared_regions", "shared_offset_region", "unshared_offset_region",
             "normalize_offsets")


def _sim_dict(attrs):
    attrs = dict(attrs or {})
    attrs.pop("name", None)
    unknown = set(attrs) - set(_SIM_KEYS)
    if unknown:
        raise TypeError("unknown Similarity attributes: %s" % sorted(unknown))
    return attrs


def _mex_dict(attrs):
    attrs = dict(attrs or {})
    attrs.pop("name", None)
    unknown = set(attrs) - set(_MEX_KEYS)
    if unknown:
        raise TypeError("unknown Mex attributes: %s" % sorted(unknown))
    return attrs


def similarity_prepare(input_shape, templates, weights, similarity_function=None, blocks=None, strides=None,
                       padding=None, normalization_term=None, normalization_term_fudge=None, ignore_nan_input=None,
                       out_of_bounds_value=None, algo=None, norm_const_every_iteration=False):
    """`similarity(input, templates, weights, ...)` with the parameter packing done here, once: returns a `Prepared`
    whose call takes the input (of exactly `input_shape`, batch size included) and runs only the forward kernels."""
    return _n.similarity_prepare([int(v) for v in input_shape], templates, weights, dict(
        similarity_function=similarity_function, blocks=blocks, strides=strides, padding=padding,
        normalization_term=normalization_term, normalization_term_fudge=normalization_term_fudge,
        ignore_nan_input=ignore_nan_input, out_of_bounds_value=out_of_bounds_value, algo=algo,
        norm_const_every_iteration=norm_const_every_iteration))


def mex_prepare(input_shape, offsets, num_instances, normalize_offsets=False, **attrs):
    """`mex(input, offsets, num_instances, ...)` with the offsets packed here, once (keyword arguments as `mex`)."""
    return _n.mex_prepare([int(v) for v in input_shape], offsets, int(num_instances),
                          _mex_dict(dict(attrs, normalize_offsets=normalize_offsets)))


def mex_sum_pool_prepare(input_shape, offsets, num_instances, pool_size=(2, 2), normalize_offsets=False, **attrs):
    """`mex_sum_pool(input, offsets, num_instances, pool_size, ...)` with the offsets packed here, once."""
    return _n.mex_sum_pool_prepare([int(v) for v in input_shape], offsets, int(num_instances), int(pool_size[0]),
                                   int(pool_size[1]), _mex_dict(dict(attrs, normalize_offsets=normalize_offsets)))


def similarity_mex_sum_pool_prepare(input_shape, templates, weights, offsets, num_instances, pool_size=(2, 2),
                                    similarity=None, mex=None):
    """`similarity_mex_sum_pool(input, templates, weights, offsets, ...)` with all parameters packed here, once."""
    return _n.similarity_mex_sum_pool_prepare([int(v) for v in input_shape], templates, weights, offsets,
                                              int(num_instances), int(pool_size[0]), int(pool_size[1]),
                                              _sim_dict(similarity), _mex_dict(mex))


_n.set_error_class(SimnetsError)
