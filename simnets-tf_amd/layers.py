"""Differentiable ops and layer classes on top of the C ABI: the caller-side layer of the reference.

  * `SimilarityFunction` / `MexFunction` wire the backward entry points to torch.autograd the way
    `_similarity_grad` / `_mex_grad` register them with TensorFlow
    (python/simnets/ops/similarity.py:18-45, python/simnets/ops/mex.py:47-81).
  * `Similarity` / `Mex` are torch modules with the constructor arguments, parameter shapes and
    defaults of the Keras layers in python/simnets/keras.py:19-88 and :113-197, built lazily from
    the first input like Keras' `build(input_shape)`.
Everything computes in fp32 on a HIP device through libsimnets_hip.so; there is no CPU path.
"""
import math
import weakref

import numpy as np
import torch

from . import ops

_SIM_KEYS = ("similarity_function", "blocks", "strides", "padding", "normalization_term",
             "normalization_term_fudge", "ignore_nan_input", "out_of_bounds_value")
_MEX_KEYS = ("softmax_mode", "padding", "strides", "blocks", "epsilon", "blocks_out_of_bounds_value",
             "blocks_round_down", "use_unshared_regions", "shared_offset_region", "unshared_offset_region",
             "normalize_offsets")


class SimilarityFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, templates, weights, attrs):
        ctx.attrs = attrs
        ctx.save_for_backward(input, templates, weights)
        return ops.similarity(input, templates, weights, **attrs)

    @staticmethod
    def backward(ctx, grad):
        input, templates, weights = ctx.saved_tensors
        grad = grad.contiguous()
        gi = gt = gw = None
        if ctx.needs_input_grad[0]:
            gi = ops.similarity_input_grad(input, templates, weights, grad, **ctx.attrs)
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            gt, gw = ops.similarity_parameters_grad(input, templates, weights, grad, **ctx.attrs)
        return gi, gt, gw, None


class MexFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, offsets, num_instances, attrs):
        ctx.attrs, ctx.num_instances = attrs, num_instances
        # (the call also keeps the offsets as the gradient kernels read them)
        out, packed = ops.mex_saving(input, offsets, num_instances, **attrs)
        ctx.save_for_backward(input, offsets, out, packed)
        return out

    @staticmethod
    def backward(ctx, grad):
        input, offsets, out, packed = ctx.saved_tensors
        grad = grad.contiguous()
        gi = go = None
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[1]:
            gi, go = ops.mex_grads(input, offsets, out, grad, ctx.num_instances, saved=packed, **ctx.attrs)
        elif ctx.needs_input_grad[0]:
            gi = ops.mex_input_grad(input, offsets, out, grad, ctx.num_instances, **ctx.attrs)
        elif ctx.needs_input_grad[1]:
            go = ops.mex_offsets_grad(input, offsets, out, grad, ctx.num_instances, **ctx.attrs)
        return gi, go, None, None


class MexSumPoolFunction(torch.autograd.Function):
    """`mex` followed by non-overlapping sum pooling as one forward call that also keeps the MEX output before pooling
    (what the MEX gradient operators take) and the offsets as the gradient kernels read them
    (`ops.mex_sum_pool_saving`)."""

    @staticmethod
    def forward(ctx, input, offsets, num_instances, ph, pw, attrs):
        ctx.attrs, ctx.num_instances, ctx.pool = attrs, num_instances, (ph, pw)
        full, pooled, packed = ops.mex_sum_pool_saving(input, offsets, num_instances, (ph, pw), **attrs)
        ctx.save_for_backward(input, offsets, full, packed)
        return pooled

    @staticmethod
    def backward(ctx, grad):
        input, offsets, full, packed = ctx.saved_tensors
        gi, go = ops.mex_sum_pool_grads(input, offsets, full, grad.contiguous(), ctx.num_instances, ctx.pool,
                                        want_input=ctx.needs_input_grad[0], want_offsets=ctx.needs_input_grad[1],
                                        saved=packed, **ctx.attrs)
        return gi, go, None, None, None, None


class SumPoolFunction(torch.autograd.Function):
    """Non-overlapping 'valid' sum pooling (`ops.sum_pooling`) with its gradient."""

    @staticmethod
    def forward(ctx, input, ph, pw):
        ctx.shape, ctx.pool = tuple(input.shape), (ph, pw)
        return ops.sum_pooling(input.contiguous(), (ph, pw))

    @staticmethod
    def backward(ctx, grad):
        return ops.sum_pooling_input_grad(grad.contiguous(), ctx.shape, ctx.pool), None, None


def sum_pooling(input, pool_size=(2, 2)):
    """Differentiable `ops.sum_pooling`."""
    return SumPoolFunction.apply(input, int(pool_size[0]), int(pool_size[1]))


def similarity(input, templates, weights, **attrs):
    """Differentiable `ops.similarity` (same keyword arguments)."""
    unknown = set(attrs) - set(_SIM_KEYS)
    if unknown:
        raise TypeError("unknown Similarity attributes: %s" % sorted(unknown))
    return SimilarityFunction.apply(input, templates, weights, attrs)


def mex(input, offsets, num_instances, **attrs):
    """Differentiable `ops.mex` (same keyword arguments)."""
    unknown = set(attrs) - set(_MEX_KEYS)
    if unknown:
        raise TypeError("unknown Mex attributes: %s" % sorted(unknown))
    return MexFunction.apply(input, offsets, num_instances, attrs)


def mex_sum_pool(input, offsets, num_instances, pool_size=(2, 2), **attrs):
    """`mex` followed by non-overlapping sum pooling (the MEX layer + pooling pair of the reference's networks,
    README.md:108-129), one call of the library either way (a fused kernel when the offsets are unshared over exactly
    the pooling window).  When a gradient is needed the call also stores the MEX output before pooling, which the MEX
    gradient operators take."""
    unknown = set(attrs) - set(_MEX_KEYS)
    if unknown:
        raise TypeError("unknown Mex attributes: %s" % sorted(unknown))
    ph, pw = int(pool_size[0]), int(pool_size[1])
    if torch.is_grad_enabled() and (input.requires_grad or offsets.requires_grad):
        return MexSumPoolFunction.apply(input, offsets, num_instances, ph, pw, attrs)
    return ops.mex_sum_pool(input, offsets, num_instances, (ph, pw), **attrs)


def dirichlet_init(shape, alpha=1.0, generator=None):
    """log of Dirichlet(alpha) samples over the block volume, one per (region, instance):
    DirichletInit of python/simnets/keras.py:91-109."""
    num_regions, num_instances, bc, bh, bw = shape
    rng = generator if generator is not None else np.random
    sample = rng.dirichlet([alpha] * (bc * bh * bw), size=(num_regions, num_instances))
    return torch.from_numpy(np.log(sample).astype(np.float32).reshape(shape))


class _PreparedCache:
    """The packed-parameter buffers of a module's inference calls, one per stream (a buffer also holds the per-call
    scratch of its kernels, so calls on different streams must not share one).

    A buffer is reused while the parameters are the same tensor objects (held by weak reference: the address of a
    freed parameter may be handed to its replacement) at the same storage address and version counter, and the
    rest of the key (input shape, device, layer attributes) is unchanged.  In-place operations on a parameter bump
    its version; rebinding the attribute or `load_state_dict(assign=True)` changes the object.  Writes through
    `.data` touch none of these: the modules' `invalidate_prepared()` is for them."""

    def __init__(self):
        self._slots = {}

    @staticmethod
    def _same(refs, marks, params):
        for r, m, p in zip(refs, marks, params):
            if r() is not p or m != (p.data_ptr(), p._version):
                return False
        return True

    def get(self, stream, params, key, make):
        slot = self._slots.get(stream)
        if slot is None or slot[0] != key or not self._same(slot[1], slot[2], params):
            if len(self._slots) >= 8:
                self._slots.clear()
            slot = self._slots[stream] = (key, [weakref.ref(p) for p in params],
                                          [(p.data_ptr(), p._version) for p in params], make())
        return slot[3]

    def last(self, stream=None):
        """The Prepared object last made for `stream` (default: for any stream), or None."""
        if stream is None:
            slot = next(reversed(self._slots.values())) if self._slots else None
        else:
            slot = self._slots.get(stream)
        return None if slot is None else slot[3]

    def clear(self):
        self._slots.clear()

    # copies and pickles of a module start with an empty cache (the buffers belong to the original's calls)
    def __deepcopy__(self, memo):
        return _PreparedCache()

    def __reduce__(self):
        return (_PreparedCache, ())


def _resolve_padding(padding, blocks):
    if isinstance(padding, str):
        if padding.upper() not in ("SAME", "VALID"):
            raise ValueError("Padding must be one of SAME, VALID (or a list of ints)")
        return [0] * len(blocks) if padding.upper() == "VALID" else [e // 2 for e in blocks]
    return list(padding)


class Similarity(torch.nn.Module):
    """python/simnets/keras.py:19-88.  Parameters: `templates`, `sweights` [num_instances, C, bh, bw];
    the op sees abs(sweights) (keras.py:65)."""

    def __init__(self, num_instances=None, similarity_function="L2", strides=[1, 1], blocks=[3, 3], padding="SAME",
                 normalization_term=False, normalization_term_fudge=0.001, ignore_nan_input=False,
                 out_of_bounds_value=0, templates_initializer="random_normal", weights_initializer="ones",
                 channels_last=False):
        super().__init__()
        assert num_instances is not None
        self.num_instances = num_instances
        self.similarity_function = similarity_function
        self.strides, self.blocks = list(strides), list(blocks)
        self.padding = _resolve_padding(padding, self.blocks)
        self.normalization_term = normalization_term
        self.normalization_term_fudge = normalization_term_fudge
        self.ignore_nan_input = ignore_nan_input
        self.out_of_bounds_value = out_of_bounds_value
        self.templates_initializer, self.weights_initializer = templates_initializer, weights_initializer
        self.channels_last = channels_last
        self.templates = torch.nn.UninitializedParameter()
        self.sweights = torch.nn.UninitializedParameter()
        self._prepared = _PreparedCache()

    @staticmethod
    def _init(param, how):
        if callable(how):
            how(param)
        elif how == "ones":
            torch.nn.init.ones_(param)
        elif how == "zeros":
            torch.nn.init.zeros_(param)
        elif how == "random_normal":
            torch.nn.init.normal_(param, 0.0, 0.05)   # Keras' RandomNormal default
        else:
            raise ValueError("unknown initializer %r" % (how,))

    def build(self, input_shape):
        channels = input_shape[3] if self.channels_last else input_shape[1]
        shape = (self.num_instances, channels, self.blocks[0], self.blocks[1])
        for p, how in ((self.sweights, self.weights_initializer), (self.templates, self.templates_initializer)):
            p.materialize(shape, dtype=torch.float32)
            with torch.no_grad():
                self._init(p, how)

    def attrs(self):
        return dict(similarity_function=self.similarity_function, blocks=self.blocks, strides=self.strides,
                    padding=self.padding, normalization_term=self.normalization_term,
                    normalization_term_fudge=self.normalization_term_fudge, ignore_nan_input=self.ignore_nan_input,
                    out_of_bounds_value=self.out_of_bounds_value)

    def forward(self, x):
        if isinstance(self.templates, torch.nn.UninitializedParameter):
            self.build(x.shape)
            self.to(x.device)
        if self.channels_last:
            x = x.permute(0, 3, 1, 2).contiguous()
        if not torch.is_grad_enabled() and x.is_cuda:
            # inference: the parameters are packed once per (input shape, parameter identity and version, layer
            # attributes, stream); calls run the forward kernels on the prepared buffer
            attrs = self.attrs()
            key = (tuple(x.shape), x.device, ops._freeze(attrs))
            out = self._prepared.get(
                ops._current_stream(x.device), (self.templates, self.sweights), key, lambda: ops.similarity_prepare(
                    x.shape, self.templates.detach(), self.sweights.detach().abs(), **attrs))(x)
        else:
            out = similarity(x, self.templates, self.sweights.abs(), **self.attrs())
        return out.permute(0, 2, 3, 1) if self.channels_last else out

    def invalidate_prepared(self):
        """Drop the packed-parameter buffers of the inference path.  Needed only after the parameters were written
        through `.data` (or any other way that bypasses torch's version counter): in-place operations on the
        parameters, rebinding them and changes of the layer's attributes are noticed without it."""
        self._prepared.clear()

    def compute_output_shape(self, input_shape):
        shape = list(input_shape)
        if self.channels_last:
            shape = [shape[0], shape[3], shape[1], shape[2]]
        out = ops.similarity_output_shape(shape, (self.num_instances, shape[1], self.blocks[0], self.blocks[1]),
                                          **self.attrs())
        return (out[0], out[2], out[3], out[1]) if self.channels_last else tuple(out)

    def get_config(self):
        names = ["num_instances", "similarity_function", "strides", "blocks", "padding", "normalization_term",
                 "normalization_term_fudge", "ignore_nan_input", "out_of_bounds_value", "templates_initializer",
                 "weights_initializer", "channels_last"]
        return {k: getattr(self, k) for k in names}


class Mex(torch.nn.Module):
    """python/simnets/keras.py:113-197.  Parameter: `offsets` [num_regions, num_instances, bc, bh, bw].
    `normalize_offsets` is applied on the device inside the op (forward and backward)."""

    def __init__(self, num_instances=None, padding=[0, 0, 0], strides=[1, 1, 1], blocks=[1, 1, 1], epsilon=1.0,
                 use_unshared_regions=True, shared_offset_region=[-1], unshared_offset_region=[-1], softmax_mode=False,
                 blocks_out_of_bounds_value=0.0, blocks_round_down=True, normalize_offsets=False,
                 offsets_initializer="dirichlet", channels_last=False):
        super().__init__()
        assert num_instances is not None
        self.num_instances = num_instances
        self.padding, self.strides, self.blocks = padding, list(strides), list(blocks)
        self.epsilon = epsilon
        self.use_unshared_regions = use_unshared_regions
        self.shared_offset_region = list(shared_offset_region)
        self.unshared_offset_region = list(unshared_offset_region)
        self.softmax_mode = softmax_mode
        self.blocks_out_of_bounds_value = blocks_out_of_bounds_value
        self.blocks_round_down = blocks_round_down
        self.normalize_offsets = normalize_offsets
        self.offsets_initializer = offsets_initializer
        self.channels_last = channels_last
        self.offsets = torch.nn.UninitializedParameter()
        self._prepared = _PreparedCache()

    def build(self, input_shape):
        shape = list(input_shape)
        if self.channels_last:
            shape = [shape[0], shape[3], shape[1], shape[2]]
        self.blocks = ops._expand_dim_specification(shape, self.blocks)
        self.padding = _resolve_padding(self.padding, self.blocks)
        nregions = ops._mex_dims_helper(shape[1:], self.num_instances, blocks=self.blocks, padding=self.padding,
                                        strides=self.strides, use_unshared_regions=self.use_unshared_regions,
                                        shared_offset_region=self.shared_offset_region,
                                        blocks_round_down=self.blocks_round_down,
                                        unshared_offset_region=self.unshared_offset_region)
        oshape = (nregions, self.num_instances) + tuple(self.blocks)
        self.offsets.materialize(oshape, dtype=torch.float32)
        with torch.no_grad():
            how = self.offsets_initializer
            if callable(how):
                how(self.offsets)
            elif how == "dirichlet":
                self.offsets.copy_(dirichlet_init(oshape))
            elif how == "zeros":
                self.offsets.zero_()
            else:
                raise ValueError("unknown initializer %r" % (how,))

    def attrs(self):
        return dict(softmax_mode=self.softmax_mode, padding=self.padding, strides=self.strides, blocks=self.blocks,
                    epsilon=self.epsilon, blocks_out_of_bounds_value=self.blocks_out_of_bounds_value,
                    blocks_round_down=self.blocks_round_down, use_unshared_regions=self.use_unshared_regions,
                    shared_offset_region=self.shared_offset_region,
                    unshared_offset_region=self.unshared_offset_region, normalize_offsets=self.normalize_offsets)

    def forward(self, x):
        if isinstance(self.offsets, torch.nn.UninitializedParameter):
            self.build(x.shape)
            self.to(x.device)
        if self.channels_last:
            x = x.permute(0, 3, 1, 2).contiguous()
        if not torch.is_grad_enabled() and x.is_cuda:
            # inference: the offsets are packed once per (input shape, parameter identity and version, layer
            # attributes, stream)
            attrs = self.attrs()
            key = (tuple(x.shape), x.device, self.num_instances, ops._freeze(attrs))
            out = self._prepared.get(ops._current_stream(x.device), (self.offsets,), key, lambda: ops.mex_prepare(
                x.shape, self.offsets.detach(), self.num_instances, **attrs))(x)
        else:
            out = mex(x, self.offsets, self.num_instances, **self.attrs())
        return out.permute(0, 2, 3, 1) if self.channels_last else out

    def invalidate_prepared(self):
        """Drop the packed-parameter buffers of the inference path.  Needed only after the parameters were written
        through `.data` (or any other way that bypasses torch's version counter): in-place operations on the
        parameters, rebinding them and changes of the layer's attributes are noticed without it."""
        self._prepared.clear()

    def compute_output_shape(self, input_shape):
        shape = list(input_shape)
        if self.channels_last:
            shape = [shape[0], shape[3], shape[1], shape[2]]
        blocks = ops._expand_dim_specification(shape, self.blocks)
        attrs = dict(self.attrs(), blocks=blocks, padding=_resolve_padding(self.padding, blocks))
        out, _ = ops.mex_output_shape(shape, self.num_instances, **attrs)
        return (out[0], out[2], out[3], out[1]) if self.channels_last else tuple(out)

    def get_config(self):
        names = ["num_instances", "padding", "strides", "blocks", "epsilon", "use_unshared_regions",
                 "shared_offset_region", "unshared_offset_region", "softmax_mode", "blocks_out_of_bounds_value",
                 "blocks_round_down", "normalize_offsets", "offsets_initializer", "channels_last"]
        return {k: getattr(self, k) for k in names}
