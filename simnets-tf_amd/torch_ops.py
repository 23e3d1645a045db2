"""`torch.ops.simnets.similarity`, `torch.ops.simnets.mex` and their gradient ops: the counterpart of the reference's
REGISTER_OP / @RegisterGradient pairs (src/ops/similarity_op.cpp:61-174, src/ops/mex_op.cpp:58-170,
python/simnets/ops/similarity.py:18-45, python/simnets/ops/mex.py:47-81).

The operators and their HIP implementations are registered by the compiled operator layer (TORCH_LIBRARY in
csrc/op_layer.cpp, loaded through ops.py).  This module attaches what a graph tracer and autograd need on top of
that: fake (meta) implementations for shape inference, so that graphs containing the ops can be traced by
torch.compile / torch.export, and the autograd formulas, which call the gradient operators.
"""
import torch

from . import ops  # noqa: F401  (loads the compiled layer, which defines the operators)


def _sim_kw(similarity_function, blocks, strides, padding, normalization_term, normalization_term_fudge,
            ignore_nan_input, out_of_bounds_value):
    return dict(similarity_function=similarity_function, blocks=list(blocks), strides=list(strides),
                padding=list(padding), normalization_term=normalization_term,
                normalization_term_fudge=normalization_term_fudge, ignore_nan_input=ignore_nan_input,
                out_of_bounds_value=out_of_bounds_value)


def _mex_kw(softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value, blocks_round_down,
            use_unshared_regions, shared_offset_region, unshared_offset_region, normalize_offsets):
    return dict(softmax_mode=softmax_mode, padding=list(padding), strides=list(strides), blocks=list(blocks),
                epsilon=epsilon, blocks_out_of_bounds_value=blocks_out_of_bounds_value,
                blocks_round_down=blocks_round_down, use_unshared_regions=use_unshared_regions,
                shared_offset_region=list(shared_offset_region), unshared_offset_region=list(unshared_offset_region),
                normalize_offsets=normalize_offsets)


@torch.library.register_fake("simnets::similarity")
def _(input, templates, weights, similarity_function, blocks, strides, padding, normalization_term,
      normalization_term_fudge, ignore_nan_input, out_of_bounds_value):
    shape = ops.similarity_output_shape(tuple(input.shape), tuple(templates.shape), tuple(weights.shape),
                                        **_sim_kw(similarity_function, blocks, strides, padding, normalization_term,
                                                  normalization_term_fudge, ignore_nan_input, out_of_bounds_value))
    return input.new_empty(shape)


@torch.library.register_fake("simnets::similarity_input_grad")
def _(input, templates, weights, output_grad, *attrs):
    return torch.empty_like(input)


@torch.library.register_fake("simnets::similarity_parameters_grad")
def _(input, templates, weights, output_grad, *attrs):
    return torch.empty_like(templates), torch.empty_like(weights)


def _similarity_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs[:3])
    ctx.attrs = inputs[3:]


def _similarity_backward(ctx, grad):
    input, templates, weights = ctx.saved_tensors
    gi = gt = gw = None
    if ctx.needs_input_grad[0]:
        gi = torch.ops.simnets.similarity_input_grad(input, templates, weights, grad.contiguous(), *ctx.attrs)
    if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
        gt, gw = torch.ops.simnets.similarity_parameters_grad(input, templates, weights, grad.contiguous(), *ctx.attrs)
    return (gi, gt, gw) + (None,) * len(ctx.attrs)


torch.library.register_autograd("simnets::similarity", _similarity_backward, setup_context=_similarity_setup)


@torch.library.register_fake("simnets::mex")
def _(input, offsets, num_instances, softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value,
      blocks_round_down, use_unshared_regions, shared_offset_region, unshared_offset_region, normalize_offsets):
    shape, _ = ops.mex_output_shape(tuple(input.shape), num_instances,
                                    **_mex_kw(softmax_mode, padding, strides, blocks, epsilon,
                                              blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions,
                                              shared_offset_region, unshared_offset_region, normalize_offsets))
    return input.new_empty(shape)


@torch.library.register_fake("simnets::mex_input_grad")
def _(input, offsets, orig_output, output_grad, *attrs):
    return torch.empty_like(input)


@torch.library.register_fake("simnets::mex_offsets_grad")
def _(input, offsets, orig_output, output_grad, *attrs):
    return torch.empty_like(offsets)


def _mex_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0], inputs[1], output)
    ctx.attrs = inputs[2:]


def _mex_backward(ctx, grad):
    input, offsets, out = ctx.saved_tensors
    gi = go = None
    if ctx.needs_input_grad[0]:
        gi = torch.ops.simnets.mex_input_grad(input, offsets, out, grad.contiguous(), *ctx.attrs)
    if ctx.needs_input_grad[1]:
        go = torch.ops.simnets.mex_offsets_grad(input, offsets, out, grad.contiguous(), *ctx.attrs)
    return (gi, go) + (None,) * len(ctx.attrs)


torch.library.register_autograd("simnets::mex", _mex_backward, setup_context=_mex_setup)
