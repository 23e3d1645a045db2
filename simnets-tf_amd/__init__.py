"""MI355X-native SimNets operators (Similarity, MEX: forward and gradients) behind the reference's op API.

`similarity(...)` and `mex(...)` take the same arguments as python/simnets/ops/similarity.py:48
and python/simnets/ops/mex.py:114 of HUJI-Deep/simnets-tf, operate on CUDA(=HIP) torch tensors
and run hand-written gfx950 kernels through the C ABI of libsimnets_hip.so.  There is no CPU
fallback: without the compiled library, or without a GPU, the calls raise.
"""
from . import _lib  # noqa: F401
from .ops import (  # noqa: F401
    SimnetsError,
    similarity,
    similarity_output_shape,
    mex,
    mex_output_shape,
    sum_pooling,
    sum_pooling_input_grad,
    mex_sum_pool,
    mex_sum_pool_both,
    mex_sum_pool_grads,
    mex_saving,
    mex_sum_pool_saving,
    similarity_mex_sum_pool,
    similarity_input_grad,
    similarity_parameters_grad,
    mex_input_grad,
    mex_offsets_grad,
    mex_grads,
    Prepared,
    similarity_prepare,
    mex_prepare,
    mex_sum_pool_prepare,
    similarity_mex_sum_pool_prepare,
    _mex_dims_helper,
    _expand_dim_specification,
)

from . import layers  # noqa: F401,E402
from . import unsupervised  # noqa: F401,E402
from . import torch_ops  # noqa: F401,E402  (registers torch.ops.simnets.*)
from .layers import Similarity, Mex, dirichlet_init  # noqa: F401,E402

__all__ = ["layers", "unsupervised", "torch_ops", "Similarity", "Mex", "dirichlet_init", "similarity", "mex", "sum_pooling", "mex_sum_pool", "similarity_mex_sum_pool", "similarity_output_shape", "mex_output_shape", "SimnetsError",
           "similarity_input_grad", "similarity_parameters_grad", "mex_input_grad", "mex_offsets_grad",
           "sum_pooling_input_grad", "mex_grads", "mex_sum_pool_both", "mex_sum_pool_grads", "mex_saving", "mex_sum_pool_saving", "Prepared", "similarity_prepare", "mex_prepare", "mex_sum_pool_prepare",
           "similarity_mex_sum_pool_prepare"]
