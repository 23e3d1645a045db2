"""ctypes view of libsimnets_hip.so: structures and prototypes of include/simnets_hip.h."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsimnets_hip.so")

# every symbol include/simnets_hip.h declares
EXPORTS = [
    "simnets_hip_strerror", "simnets_hip_abi_version",
    "simnets_similarity_attrs_default", "simnets_similarity_out_shape",
    "simnets_hip_similarity_workspace_bytes", "simnets_hip_similarity_fwd", "simnets_hip_similarity_fwd_static",
    "simnets_mex_attrs_default", "simnets_mex_calc_dims", "simnets_mex_out_shape", "get_mex_offsets_nregions",
    "simnets_hip_mex_workspace_bytes", "simnets_hip_mex_fwd", "simnets_hip_sum_pool_fwd",
    "simnets_hip_sum_pool_input_grad",
    "simnets_hip_similarity_grad_workspace_bytes", "simnets_hip_similarity_input_grad",
    "simnets_hip_similarity_params_grad", "simnets_hip_mex_grad_workspace_bytes", "simnets_hip_mex_input_grad",
    "simnets_hip_mex_offsets_grad", "simnets_hip_mex_grads_workspace_bytes", "simnets_hip_mex_grads",
    "simnets_hip_mex_sum_pool_workspace_bytes", "simnets_hip_mex_sum_pool_fwd", "simnets_hip_mex_sum_pool_fwd_both",
    "simnets_hip_mex_sum_pool_grads_workspace_bytes", "simnets_hip_mex_sum_pool_grads",
    "simnets_hip_mex_saved_bytes", "simnets_hip_mex_fwd_saving", "simnets_hip_mex_sum_pool_fwd_saving",
    "simnets_hip_mex_grads_saved", "simnets_hip_mex_sum_pool_grads_saved",
    "simnets_hip_similarity_mex_sum_pool_workspace_bytes", "simnets_hip_similarity_mex_sum_pool_fwd",
    "simnets_hip_similarity_prepare", "simnets_hip_similarity_fwd_prepared",
    "simnets_hip_mex_prepare", "simnets_hip_mex_fwd_prepared",
    "simnets_hip_mex_sum_pool_prepare", "simnets_hip_mex_sum_pool_fwd_prepared",
    "simnets_hip_similarity_mex_sum_pool_prepare", "simnets_hip_similarity_mex_sum_pool_fwd_prepared",
]

SIM_L1, SIM_L2 = 0, 1
STATIC_SCRATCH_BYTES = 4 << 20  # SIMNETS_HIP_STATIC_SCRATCH_BYTES
ALGO_AUTO, ALGO_DIRECT, ALGO_SQRTW, ALGO_MFMA = 0, 1, 2, 3
ALGOS = {None: ALGO_AUTO, "auto": ALGO_AUTO, "direct": ALGO_DIRECT, "sqrtw": ALGO_SQRTW, "mfma": ALGO_MFMA}


class SimilarityAttrs(C.Structure):
    _fields_ = [
        ("similarity_function", C.c_int),
        ("n_blocks", C.c_int), ("blocks", C.c_int * 2),
        ("n_strides", C.c_int), ("strides", C.c_int * 2),
        ("n_padding", C.c_int), ("padding", C.c_int * 2),
        ("normalization_term", C.c_int),
        ("normalization_term_fudge", C.c_float),
        ("ignore_nan_input", C.c_int),
        ("out_of_bounds_value", C.c_float),
        ("algo", C.c_int),
        ("norm_const_every_iteration", C.c_int),
    ]


class MexAttrs(C.Structure):
    _fields_ = [
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
        ("normalize_offsets", C.c_int),
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


def lib():
    """The loaded library.  Raises if it has not been built: there is nothing to fall back to."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libsimnets_hip.so is missing (%s): build it with `python simnets-tf_amd/build.py`; "
                "this package has no CPU fallback" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        I4, I3, I5 = C.c_int * 4, C.c_int * 3, C.c_int * 5
        P = C.c_void_p
        l.simnets_hip_strerror.restype = C.c_char_p
        l.simnets_hip_strerror.argtypes = [C.c_int]
        l.simnets_hip_abi_version.restype = C.c_int
        l.simnets_similarity_attrs_default.argtypes = [C.POINTER(SimilarityAttrs)]
        l.simnets_similarity_attrs_default.restype = None
        l.simnets_similarity_out_shape.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, I4, I4]
        l.simnets_hip_similarity_workspace_bytes.argtypes = [C.POINTER(SimilarityAttrs), I4, I4,
                                                             C.POINTER(C.c_size_t)]
        l.simnets_hip_similarity_fwd.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, I4, P, P, P, P, P, C.c_size_t, P]
        l.simnets_hip_similarity_fwd_static.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, I4, P, P, P, P, P]
        l.simnets_hip_similarity_fwd_static.restype = C.c_int
        l.simnets_mex_attrs_default.argtypes = [C.POINTER(MexAttrs)]
        l.simnets_mex_attrs_default.restype = None
        l.simnets_mex_calc_dims.argtypes = [C.POINTER(MexAttrs), I3, C.POINTER(MexDims)]
        l.simnets_mex_out_shape.argtypes = [C.POINTER(MexAttrs), I4, C.POINTER(I4), C.POINTER(I5)]
        l.simnets_hip_mex_workspace_bytes.argtypes = [C.POINTER(MexAttrs), I4, C.POINTER(C.c_size_t)]
        l.simnets_hip_mex_fwd.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, C.c_size_t, P]
        l.simnets_hip_sum_pool_fwd.argtypes = [I4, C.c_int, C.c_int, P, P, P]
        l.simnets_hip_sum_pool_input_grad.argtypes = [I4, C.c_int, C.c_int, P, P, P]
        l.simnets_hip_mex_sum_pool_workspace_bytes.argtypes = [C.POINTER(MexAttrs), I4, C.c_int, C.c_int,
                                                               C.POINTER(C.c_size_t)]
        l.simnets_hip_mex_sum_pool_fwd.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, C.c_int, C.c_int, P, P,
                                                   C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_fwd_both.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, C.c_int, C.c_int, P,
                                                        P, P, C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_fwd_both.restype = C.c_int
        l.simnets_hip_mex_sum_pool_grads_workspace_bytes.argtypes = [C.POINTER(MexAttrs), I4, C.c_int, C.c_int,
                                                                     C.POINTER(C.c_size_t)]
        l.simnets_hip_mex_sum_pool_grads_workspace_bytes.restype = C.c_int
        l.simnets_hip_mex_sum_pool_grads.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, C.c_int, C.c_int, P, P, P, P,
                                                     P, C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_grads.restype = C.c_int
        l.simnets_hip_mex_saved_bytes.argtypes = [C.POINTER(MexAttrs), I4, C.POINTER(C.c_size_t)]
        l.simnets_hip_mex_fwd_saving.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, C.c_size_t, P,
                                                 C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_fwd_saving.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, C.c_int, C.c_int,
                                                          P, P, P, C.c_size_t, P, C.c_size_t, P]
        l.simnets_hip_mex_grads_saved.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, P, C.c_size_t, P, P,
                                                  P, C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_grads_saved.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, C.c_int, C.c_int,
                                                           P, P, P, C.c_size_t, P, P, P, C.c_size_t, P]
        for f in (l.simnets_hip_mex_saved_bytes, l.simnets_hip_mex_fwd_saving, l.simnets_hip_mex_sum_pool_fwd_saving,
                  l.simnets_hip_mex_grads_saved, l.simnets_hip_mex_sum_pool_grads_saved):
            f.restype = C.c_int
        SZ = C.POINTER(C.c_size_t)
        l.simnets_hip_similarity_mex_sum_pool_workspace_bytes.argtypes = [C.POINTER(SimilarityAttrs), I4, I4,
                                                                          C.POINTER(MexAttrs), C.c_int, C.c_int, SZ]
        l.simnets_hip_similarity_mex_sum_pool_fwd.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, P, P, P,
                                                              C.POINTER(MexAttrs), P, C.c_size_t, C.c_int, C.c_int, P,
                                                              P, C.c_size_t, P]
        l.simnets_hip_similarity_grad_workspace_bytes.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, SZ, SZ]
        l.simnets_hip_similarity_input_grad.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, I4, P, P, P, P, P, P,
                                                        C.c_size_t, P]
        l.simnets_hip_similarity_params_grad.argtypes = [C.POINTER(SimilarityAttrs), I4, I4, I4, P, P, P, P, P, P, P,
                                                         C.c_size_t, P]
        l.simnets_hip_mex_grad_workspace_bytes.argtypes = [C.POINTER(MexAttrs), I4, SZ, SZ]
        l.simnets_hip_mex_input_grad.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, P, P, C.c_size_t, P]
        l.simnets_hip_mex_offsets_grad.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, P, P, C.c_size_t,
                                                   P]
        l.simnets_hip_mex_grads_workspace_bytes.argtypes = [C.POINTER(MexAttrs), I4, C.POINTER(C.c_size_t)]
        l.simnets_hip_mex_grads.argtypes = [C.POINTER(MexAttrs), I4, P, P, C.c_size_t, P, P, P, P, P, C.c_size_t, P]
        SA, MA = C.POINTER(SimilarityAttrs), C.POINTER(MexAttrs)
        l.simnets_hip_similarity_prepare.argtypes = [SA, I4, I4, I4, P, P, P, C.c_size_t, P]
        l.simnets_hip_similarity_fwd_prepared.argtypes = [SA, I4, I4, P, P, C.c_size_t, P, P]
        l.simnets_hip_mex_prepare.argtypes = [MA, I4, P, C.c_size_t, P, C.c_size_t, P]
        l.simnets_hip_mex_fwd_prepared.argtypes = [MA, I4, P, P, C.c_size_t, P, P]
        l.simnets_hip_mex_sum_pool_prepare.argtypes = [MA, I4, P, C.c_size_t, C.c_int, C.c_int, P, C.c_size_t, P]
        l.simnets_hip_mex_sum_pool_fwd_prepared.argtypes = [MA, I4, P, C.c_int, C.c_int, P, C.c_size_t, P, P]
        l.simnets_hip_similarity_mex_sum_pool_prepare.argtypes = [SA, I4, I4, P, P, MA, P, C.c_size_t, C.c_int, C.c_int,
                                                                  P, C.c_size_t, P]
        l.simnets_hip_similarity_mex_sum_pool_fwd_prepared.argtypes = [SA, I4, I4, P, MA, C.c_int, C.c_int, P,
                                                                       C.c_size_t, P, P]
        for name in ("simnets_hip_similarity_prepare", "simnets_hip_similarity_fwd_prepared",
                     "simnets_hip_mex_prepare", "simnets_hip_mex_fwd_prepared", "simnets_hip_mex_sum_pool_prepare",
                     "simnets_hip_mex_sum_pool_fwd_prepared", "simnets_hip_similarity_mex_sum_pool_prepare",
                     "simnets_hip_similarity_mex_sum_pool_fwd_prepared"):
            getattr(l, name).restype = C.c_int
        for name in ("simnets_similarity_out_shape", "simnets_hip_similarity_workspace_bytes",
                     "simnets_hip_similarity_fwd", "simnets_mex_calc_dims", "simnets_mex_out_shape",
                     "simnets_hip_mex_workspace_bytes", "simnets_hip_mex_fwd", "simnets_hip_sum_pool_fwd",
                     "simnets_hip_sum_pool_input_grad",
    "simnets_hip_similarity_grad_workspace_bytes", "simnets_hip_similarity_input_grad",
    "simnets_hip_similarity_params_grad", "simnets_hip_mex_grad_workspace_bytes", "simnets_hip_mex_input_grad",
    "simnets_hip_mex_offsets_grad",
                     "get_mex_offsets_nregions", "simnets_hip_similarity_grad_workspace_bytes",
                     "simnets_hip_similarity_input_grad", "simnets_hip_similarity_params_grad",
                     "simnets_hip_mex_grad_workspace_bytes", "simnets_hip_mex_input_grad",
                     "simnets_hip_mex_offsets_grad", "simnets_hip_mex_grads_workspace_bytes",
                     "simnets_hip_mex_grads", "simnets_hip_mex_sum_pool_workspace_bytes",
                     "simnets_hip_mex_sum_pool_fwd", "simnets_hip_similarity_mex_sum_pool_workspace_bytes",
                     "simnets_hip_similarity_mex_sum_pool_fwd"):
            getattr(l, name).restype = C.c_int
        _lib = l
    return _lib


def strerror(code):
    return lib().simnets_hip_strerror(int(code)).decode()
