"""`torch.library` registration of the operators: `torch.ops.simnets.similarity`, `torch.ops.simnets.mex` and
their gradient ops, the counterpart of the reference's REGISTER_OP / @RegisterGradient pairs
(src/ops/similarity_op.cpp:61-174, src/ops/mex_op.cpp:58-170, python/simnets/ops/similarity.py:18-45,
python/simnets/ops/mex.py:47-81).  With fake (meta) implementations for shape inference, so that graphs
containing the ops can be traced by torch.compile / torch.export; the real implementations call the C ABI
through ops.py and exist for HIP devices only.
"""
from typing import List, Tuple

import torch

from . import ops

_lib_defined = False


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


@torch.library.custom_op("simnets::similarity", mutates_args=(), device_types="cuda")
def similarity(input: torch.Tensor, templates: torch.Tensor, weights: torch.Tensor, similarity_function: str,
               blocks: List[int], strides: List[int], padding: List[int], normalization_term: bool,
               normalization_term_fudge: float, ignore_nan_input: bool, out_of_bounds_value: float) -> torch.Tensor:
    return ops.similarity(input, templates, weights, **_sim_kw(similarity_function, blocks, strides, padding,
                                                               normalization_term, normalization_term_fudge,
                                                               ignore_nan_input, out_of_bounds_value))


@similarity.register_fake
def _(input, templates, weights, similarity_function, blocks, strides, padding, normalization_term,
      normalization_term_fudge, ignore_nan_input, out_of_bounds_value):
    shape = ops.similarity_output_shape(tuple(input.shape), tuple(templates.shape), tuple(weights.shape),
                                        **_sim_kw(similarity_function, blocks, strides, padding, normalization_term,
                                                  normalization_term_fudge, ignore_nan_input, out_of_bounds_value))
    return input.new_empty(shape)


@torch.library.custom_op("simnets::similarity_input_grad", mutates_args=(), device_types="cuda")
def similarity_input_grad(input: torch.Tensor, templates: torch.Tensor, weights: torch.Tensor,
                          output_grad: torch.Tensor, similarity_function: str, blocks: List[int], strides: List[int],
                          padding: List[int], normalization_term: bool, normalization_term_fudge: float,
                          ignore_nan_input: bool, out_of_bounds_value: float) -> torch.Tensor:
    return ops.similarity_input_grad(input, templates, weights, output_grad.contiguous(),
                                     **_sim_kw(similarity_function, blocks, strides, padding, normalization_term,
                                               normalization_term_fudge, ignore_nan_input, out_of_bounds_value))


@similarity_input_grad.register_fake
def _(input, templates, weights, output_grad, *attrs):
    return torch.empty_like(input)


@torch.library.custom_op("simnets::similarity_parameters_grad", mutates_args=(), device_types="cuda")
def similarity_parameters_grad(input: torch.Tensor, templates: torch.Tensor, weights: torch.Tensor,
                               output_grad: torch.Tensor, similarity_function: str, blocks: List[int],
                               strides: List[int], padding: List[int], normalization_term: bool,
                               normalization_term_fudge: float, ignore_nan_input: bool,
                               out_of_bounds_value: float) -> Tuple[torch.Tensor, torch.Tensor]:
    return ops.similarity_parameters_grad(input, templates, weights, output_grad.contiguous(),
                                          **_sim_kw(similarity_function, blocks, strides, padding, normalization_term,
                                                    normalization_term_fudge, ignore_nan_input, out_of_bounds_value))


@similarity_parameters_grad.register_fake
def _(input, templates, weights, output_grad, *attrs):
    return torch.empty_like(templates), torch.empty_like(weights)


def _similarity_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs[:3])
    ctx.attrs = inputs[3:]


def _similarity_backward(ctx, grad):
    input, templates, weights = ctx.saved_tensors
    gi = gt = gw = None
    if ctx.needs_input_grad[0]:
        gi = similarity_input_grad(input, templates, weights, grad, *ctx.attrs)
    if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
        gt, gw = similarity_parameters_grad(input, templates, weights, grad, *ctx.attrs)
    return (gi, gt, gw) + (None,) * len(ctx.attrs)


similarity.register_autograd(_similarity_backward, setup_context=_similarity_setup)


@torch.library.custom_op("simnets::mex", mutates_args=(), device_types="cuda")
def mex(input: torch.Tensor, offsets: torch.Tensor, num_instances: int, softmax_mode: bool, padding: List[int],
        strides: List[int], blocks: List[int], epsilon: float, blocks_out_of_bounds_value: float,
        blocks_round_down: bool, use_unshared_regions: bool, shared_offset_region: List[int],
        unshared_offset_region: List[int], normalize_offsets: bool) -> torch.Tensor:
    return ops.mex(input, offsets, num_instances,
                   **_mex_kw(softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value,
                             blocks_round_down, use_unshared_regions, shared_offset_region, unshared_offset_region,
                             normalize_offsets))


@mex.register_fake
def _(input, offsets, num_instances, softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value,
      blocks_round_down, use_unshared_regions, shared_offset_region, unshared_offset_region, normalize_offsets):
    shape, _ = ops.mex_output_shape(tuple(input.shape), num_instances,
                                    **_mex_kw(softmax_mode, padding, strides, blocks, epsilon,
                                              blocks_out_of_bounds_value, blocks_round_down, use_unshared_regions,
                                              shared_offset_region, unshared_offset_region, normalize_offsets))
    return input.new_empty(shape)


@torch.library.custom_op("simnets::mex_input_grad", mutates_args=(), device_types="cuda")
def mex_input_grad(input: torch.Tensor, offsets: torch.Tensor, orig_output: torch.Tensor, output_grad: torch.Tensor,
                   num_instances: int, softmax_mode: bool, padding: List[int], strides: List[int], blocks: List[int],
                   epsilon: float, blocks_out_of_bounds_value: float, blocks_round_down: bool,
                   use_unshared_regions: bool, shared_offset_region: List[int], unshared_offset_region: List[int],
                   normalize_offsets: bool) -> torch.Tensor:
    return ops.mex_input_grad(input, offsets, orig_output, output_grad.contiguous(), num_instances,
                              **_mex_kw(softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value,
                                        blocks_round_down, use_unshared_regions, shared_offset_region,
                                        unshared_offset_region, normalize_offsets))


@mex_input_grad.register_fake
def _(input, offsets, orig_output, output_grad, *attrs):
    return torch.empty_like(input)


@torch.library.custom_op("simnets::mex_offsets_grad", mutates_args=(), device_types="cuda")
def mex_offsets_grad(input: torch.Tensor, offsets: torch.Tensor, orig_output: torch.Tensor, output_grad: torch.Tensor,
                     num_instances: int, softmax_mode: bool, padding: List[int], strides: List[int],
                     blocks: List[int], epsilon: float, blocks_out_of_bounds_value: float, blocks_round_down: bool,
                     use_unshared_regions: bool, shared_offset_region: List[int], unshared_offset_region: List[int],
                     normalize_offsets: bool) -> torch.Tensor:
    return ops.mex_offsets_grad(input, offsets, orig_output, output_grad.contiguous(), num_instances,
                                **_mex_kw(softmax_mode, padding, strides, blocks, epsilon, blocks_out_of_bounds_value,
                                          blocks_round_down, use_unshared_regions, shared_offset_region,
                                          unshared_offset_region, normalize_offsets))


@mex_offsets_grad.register_fake
def _(input, offsets, orig_output, output_grad, *attrs):
    return torch.empty_like(offsets)


def _mex_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0], inputs[1], output)
    ctx.attrs = inputs[2:]


def _mex_backward(ctx, grad):
    input, offsets, out = ctx.saved_tensors
    gi = go = None
    if ctx.needs_input_grad[0]:
        gi = mex_input_grad(input, offsets, out, grad, *ctx.attrs)
    if ctx.needs_input_grad[1]:
        go = mex_offsets_grad(input, offsets, out, grad, *ctx.attrs)
    return (gi, go) + (None,) * len(ctx.attrs)


mex.register_autograd(_mex_backward, setup_context=_mex_setup)
