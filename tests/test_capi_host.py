"""CPU-only checks of the C ABI: the library loads, exports every declared symbol, and its host-side
validation / dimension logic agrees with the oracle and with the reference's known answers.  No
compute entry point is called with data here (that needs a GPU)."""
import ctypes as C
import itertools
import os
import re
import subprocess

import pytest

from oracle import oracle as orc
from conftest import ROOT


def test_library_exports_every_declared_symbol(pkg):
    l = pkg._lib.lib()
    header = open(os.path.join(ROOT, "include", "simnets_hip.h")).read()
    declared = set(re.findall(r"\b((?:simnets_[a-z_0-9]+|get_mex_offsets_nregions))\s*\(", header))
    declared -= {"simnets_status"}
    assert declared == set(pkg._lib.EXPORTS)
    for name in declared:
        assert hasattr(l, name), name
    assert l.simnets_hip_abi_version() == 1
    assert pkg._lib.strerror(0) == "ok"


def test_struct_layouts_match_the_header(pkg, tmp_path):
    # sizes as a C compiler sees the header vs the ctypes mirrors
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include "simnets_hip.h"\nint main(void){printf("%zu %zu %zu\\n",'
                   'sizeof(simnets_similarity_attrs),sizeof(simnets_mex_attrs),sizeof(simnets_mex_dims));return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    sizes = [int(v) for v in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert sizes == [C.sizeof(pkg._lib.SimilarityAttrs), C.sizeof(pkg._lib.MexAttrs), C.sizeof(pkg._lib.MexDims)]


def test_similarity_defaults_are_the_registered_op_defaults(pkg):
    a = pkg._lib.SimilarityAttrs()
    pkg._lib.lib().simnets_similarity_attrs_default(C.byref(a))
    assert (a.similarity_function, list(a.blocks), list(a.strides), list(a.padding)) == (1, [3, 3], [2, 2], [0, 0])
    assert (a.normalization_term, a.ignore_nan_input, a.out_of_bounds_value) == (0, 0, 0.0)
    assert abs(a.normalization_term_fudge - 0.001) < 1e-9
    m = pkg._lib.MexAttrs()
    pkg._lib.lib().simnets_mex_attrs_default(C.byref(m))
    assert (list(m.padding), list(m.strides), list(m.blocks)) == ([0, 0, 0], [1, 1, 1], [1, 1, 1])
    assert (m.epsilon, m.softmax_mode, m.blocks_round_down, m.use_unshared_regions) == (1.0, 0, 1, 1)
    assert (m.n_shared, m.shared_offset_region[0], m.n_unshared, m.unshared_offset_region[0]) == (1, -1, 1, -1)


@pytest.mark.parametrize("num_instances,padding,strides,blocks,in_shape,out_shape", [
    (10, [0, 1], [1, 1], [2, 2], (3, 10, 13), (10, 9, 14)),
    (10, [1, 1], [3, 2], [2, 2], (3, 10, 13), (10, 4, 7)),
    (2, [1, 1], [3, 2], [2, 2], (1, 10, 13), (2, 4, 7)),
])
def test_similarity_known_answer_shapes(pkg, num_instances, padding, strides, blocks, in_shape, out_shape):
    # python/simnets/test/keras/__init__.py:110-119
    got = pkg.similarity_output_shape((5,) + in_shape, (num_instances, in_shape[0]) + tuple(blocks),
                                      similarity_function="L1", blocks=blocks, strides=strides, padding=padding)
    assert got == (5,) + out_shape


@pytest.mark.parametrize("num_instances,padding,strides,blocks,in_shape,out_shape", [
    (10, [1, 0, 1], [1, 1, 1], [1, 2, 2], (3, 10, 13), (50, 9, 14)),
    (10, [2, 1, 1], [1, 3, 2], [1, 2, 2], (3, 10, 13), (70, 5, 8)),
    (2, [1, 1, 1], [1, 3, 2], [1, 2, 2], (1, 10, 13), (6, 5, 8)),
])
def test_mex_known_answer_shapes(pkg, num_instances, padding, strides, blocks, in_shape, out_shape):
    # python/simnets/test/keras/__init__.py:46-55
    o, f = pkg.mex_output_shape((4,) + in_shape, num_instances, padding=padding, strides=strides, blocks=blocks,
                                blocks_round_down=False, use_unshared_regions=False, shared_offset_region=[2],
                                softmax_mode=True, epsilon=2.0)
    assert o == (4,) + out_shape
    assert f[1:] == (num_instances,) + tuple(blocks)


def test_dims_helper_twin_of_the_reference_symbol(pkg):
    # python/simnets/test/__init__.py:213
    assert pkg._mex_dims_helper([1, 90, 90], 3, blocks=[1, 3, 3], padding=[0, 1, 1], strides=[1, 2, 2]) == 2025
    assert pkg._mex_dims_helper([3, 8, 8], 3, blocks=[1, 3]) == -1
    assert pkg._expand_dim_specification([5, 3, 10, 12], [2, 2]) == [3, 2, 2]
    assert pkg._expand_dim_specification([3, 10, 12], [1, -1, 4]) == [1, 10, 4]
    with pytest.raises(ValueError):
        pkg._expand_dim_specification([3, 10, 12], [1])


@pytest.mark.parametrize("unshared", [True, False])
@pytest.mark.parametrize("spec", [[2], [3], [1, 5, 4], [-1], [2, 7, 1]])
@pytest.mark.parametrize("geom", [((3, 41, 40), [1, 3, 3], [0, 1, 0], [1, 4, 1], True),
                                  ((3, 10, 13), [2, 2, 2], [1, 1, 1], [1, 3, 2], False),
                                  ((32, 16, 16), [32, 1, 1], [0, 0, 0], [32, 1, 1], True),
                                  ((4, 9, 9), [4, 3, 3], [0, 0], [-1, 2, 2], True)])
def test_mex_dims_agree_with_the_oracle(pkg, unshared, spec, geom):
    image, blocks, padding, strides, rd = geom
    kw = dict(blocks=blocks, padding=padding, strides=strides, blocks_round_down=rd, use_unshared_regions=unshared,
              shared_offset_region=spec, unshared_offset_region=spec)
    got = pkg.ops.mex_dims(image, 5, **kw)
    want = orc.mex_dims(orc.mex_args((1,) + tuple(image), 5, **kw)).asdict()
    assert got == want


def test_similarity_validation_mirrors_the_reference(pkg):
    E = pkg.SimnetsError
    shp = ((2, 3, 10, 10), (4, 3, 3, 3))

    def code(**kw):
        kw.setdefault("blocks", [3, 3])
        tshape = kw.pop("tshape", shp[1])
        wshape = kw.pop("wshape", None)
        try:
            pkg.similarity_output_shape(shp[0], tshape, wshape, **kw)
        except E as e:
            return e.code
        return 0

    assert code() == 0
    assert code(padding=[0]) == -2
    assert code(blocks=[3]) == -3
    assert code(strides=[1, 1, 1]) == -4
    assert code(similarity_function="cosine") == -5
    assert code(similarity_function="L1", normalization_term=True) == -6
    assert code(ignore_nan_input=True) == -7
    assert code(tshape=(4, 2, 3, 3)) == -8
    assert code(wshape=(4, 2, 3, 3)) == -9
    assert code(strides=[0, 1]) == -10
    assert code(blocks=[2, 2]) == -15            # blocks attribute disagrees with the template tensor
    assert code(blocks=[3, 3], tshape=(4, 3, 3, 3), wshape=(5, 3, 3, 3)) == -15
    assert code(algo="mfma", normalization_term=True) == -18
    assert "ignore_nan is relevant only if normalization_term is true" in pkg._lib.strerror(-7)
    assert "normalization_term is relevant only if similarity_function is L2" in pkg._lib.strerror(-6)


def test_mex_validation_mirrors_the_reference(pkg):
    E = pkg.SimnetsError

    def code(n=2, shape=(1, 3, 8, 8), **kw):
        try:
            pkg.mex_output_shape(shape, n, **kw)
        except E as e:
            return e.code
        return 0

    assert code() == 0
    assert code(n=0) == -11
    assert code(strides=[1, 1]) == -4
    assert code(blocks=[1, 1]) == -3
    assert code(padding=[1]) == -2
    assert code(unshared_offset_region=[1, 2]) == -12
    assert code(shared_offset_region=[1, 2]) == -13
    assert code(blocks=[4, 1, 1]) == -14
    assert code(strides=[1, 0, 1]) == -10
    assert code(padding=[0, 0]) == 0              # two entries: -1 (the channel count) is prepended
    assert "block depth must be smaller than input depth" in pkg._lib.strerror(-14)
    # a block larger than the padded image, a region extent of zero: the reference divides by zero in
    # CalculateDimensions (src/kernels/mex_kernel_common.cpp:86-139); the library and the oracle report it
    for bad in (dict(blocks=[1, 1, 9]), dict(blocks=[1, 9, 1], padding=[0, 0, 0]), dict(unshared_offset_region=[0]),
                dict(use_unshared_regions=False, shared_offset_region=[1, 0, 2])):
        assert code(**bad) < 0
        with pytest.raises(ValueError):
            orc.mex_dims(orc.mex_args((1, 3, 8, 8), 2, **bad))


def test_compute_entry_points_reject_bad_arguments_without_touching_the_device(pkg):
    l = pkg._lib.lib()
    a = pkg.ops.similarity_attrs(blocks=[3, 3], ignore_nan_input=True)
    I4 = C.c_int * 4
    rc = l.simnets_hip_similarity_fwd(C.byref(a), I4(1, 3, 8, 8), I4(2, 3, 3, 3), I4(2, 3, 3, 3), None, None, None,
                                      None, None, 0, None)
    assert rc == -7
    a = pkg.ops.similarity_attrs(blocks=[3, 3])
    rc = l.simnets_hip_similarity_fwd(C.byref(a), I4(1, 3, 8, 8), I4(2, 3, 3, 3), I4(2, 3, 3, 3), None, None, None,
                                      None, None, 0, None)
    assert rc == -1
    rc = l.simnets_hip_similarity_fwd(C.byref(a), I4(1, 3, 8, 8), I4(2, 3, 3, 3), I4(2, 3, 3, 3), 256, 256, 256, 256,
                                      None, 0, None)
    assert rc == -17
    m = pkg.ops.mex_attrs(2, blocks=[3, 1, 1])
    rc = l.simnets_hip_mex_fwd(C.byref(m), I4(1, 3, 8, 8), 256, 256, 5, 256, None, 0, None)
    assert rc == -15                               # offsets buffer shorter than R*M*K
    nbytes = C.c_size_t()
    assert l.simnets_hip_mex_workspace_bytes(C.byref(m), I4(1, 3, 8, 8), C.byref(nbytes)) == 0
    assert nbytes.value >= 64 * 2 * 3 * 4
    assert l.simnets_hip_sum_pool_fwd(I4(1, 1, 4, 4), 0, 2, None, None, None) == -15


def test_fused_mex_sum_pool_entry_validates_without_touching_the_device(pkg):
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    m = pkg.ops.mex_attrs(8, blocks=[3, 1, 1], unshared_offset_region=[2])
    fused, plain, split = C.c_size_t(), C.c_size_t(), C.c_size_t()
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), 2, 2, C.byref(fused)) == 0
    assert l.simnets_hip_mex_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), C.byref(plain)) == 0
    # a 3x3 window is not one pixel of each 2x2 region: MEX into scratch (the full output) + pooling
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), 3, 3, C.byref(split)) == 0
    assert split.value >= plain.value + 2 * 8 * 8 * 8 * 4 > fused.value > 0
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), 0, 2, C.byref(fused)) == -15
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), 9, 2, C.byref(fused)) == -16
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), I4(2, 3, 8, 8), 2, 2, None) == -1
    assert l.simnets_hip_mex_sum_pool_fwd(C.byref(m), I4(2, 3, 8, 8), 256, 256, 5, 2, 2, 256, None, 0, None) == -15
    assert l.simnets_hip_mex_sum_pool_fwd(C.byref(m), I4(2, 3, 8, 8), None, 256, 4 * 8 * 3, 2, 2, 256, None, 0,
                                          None) == -1
    assert l.simnets_hip_mex_sum_pool_fwd(C.byref(m), I4(2, 3, 8, 8), 256, 256, 4 * 8 * 3, 2, 2, 256, None, 0,
                                          None) == -17
    assert l.simnets_hip_mex_sum_pool_fwd(C.byref(m), I4(0, 3, 8, 8), None, None, 4 * 8 * 3, 2, 2, None, None, 0,
                                          None) == 0


def test_similarity_mex_sum_pool_entry_validates_without_touching_the_device(pkg):
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    sa = pkg.ops.similarity_attrs(blocks=[2, 2], strides=[2, 2], padding=[2, 2])
    ma = pkg.ops.mex_attrs(8, blocks=[4, 1, 1], strides=[4, 1, 1], unshared_offset_region=[2])
    x, t = I4(2, 1, 28, 28), I4(4, 1, 2, 2)
    one, split = C.c_size_t(), C.c_size_t()
    f = l.simnets_hip_similarity_mex_sum_pool_workspace_bytes
    assert f(C.byref(sa), x, t, C.byref(ma), 2, 2, C.byref(one)) == 0 and one.value > 0
    # a 4x4 window is not the 2x2 region grid: the Similarity output (2 x 4 x 16 x 16 floats) lives in scratch memory
    assert f(C.byref(sa), x, t, C.byref(ma), 4, 4, C.byref(split)) == 0
    assert split.value >= 2 * 4 * 16 * 16 * 4 + one.value - 4 * 4 * 3 * 4
    assert f(C.byref(sa), x, t, C.byref(ma), 0, 2, C.byref(one)) == -15
    assert f(C.byref(sa), x, t, C.byref(ma), 2, 2, None) == -1
    assert f(C.byref(sa), x, I4(4, 2, 2, 2), C.byref(ma), 2, 2, C.byref(one)) != 0      # template channels != input's
    g = l.simnets_hip_similarity_mex_sum_pool_fwd
    assert g(C.byref(sa), x, t, 256, 256, 256, C.byref(ma), 256, 5, 2, 2, 256, None, 0, None) == -15
    assert g(C.byref(sa), x, t, None, 256, 256, C.byref(ma), 256, 4 * 8 * 4, 2, 2, 256, None, 0, None) == -1
    assert g(C.byref(sa), x, t, 256, 256, 256, C.byref(ma), 256, 4 * 8 * 4, 2, 2, 256, None, 0, None) == -17
    assert g(C.byref(sa), I4(0, 1, 28, 28), t, None, None, None, C.byref(ma), None, 4 * 8 * 4, 2, 2, None, None, 0,
             None) == 0


def test_op_layer_refuses_cpu_tensors(pkg):
    import torch
    x = torch.zeros(1, 1, 4, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.similarity(x, x, x, blocks=[4, 4])
    with pytest.raises(TypeError):
        pkg.similarity(x.double(), x, x, blocks=[4, 4])


def test_gradient_entry_points_reject_bad_arguments_without_touching_the_device(pkg):
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    shapes = (I4(2, 3, 8, 8), I4(4, 3, 3, 3), I4(4, 3, 3, 3))
    a = pkg.ops.similarity_attrs(blocks=[3, 3], ignore_nan_input=True)     # ignore_nan_input needs normalization_term
    assert l.simnets_hip_similarity_input_grad(C.byref(a), *shapes, 256, 256, 256, 256, 256, None, 0, None) == -7
    a = pkg.ops.similarity_attrs(blocks=[3, 3])
    assert l.simnets_hip_similarity_input_grad(C.byref(a), *shapes, None, 256, 256, 256, 256, None, 0, None) == -1
    assert l.simnets_hip_similarity_params_grad(C.byref(a), *shapes, 256, 256, 256, None, 256, 256, None, 0, None) == -1
    wx, wp = C.c_size_t(), C.c_size_t()
    assert l.simnets_hip_similarity_grad_workspace_bytes(C.byref(a), shapes[0], shapes[1], C.byref(wx), C.byref(wp)) == 0
    assert wx.value > 0 and wp.value >= 2 * 4 * 27 * 4          # packed parameters; partial sums for both gradients
    assert l.simnets_hip_similarity_input_grad(C.byref(a), *shapes, 256, 256, 256, 256, 256, None, 0, None) == -17
    assert l.simnets_hip_similarity_params_grad(C.byref(a), *shapes, 256, 256, 256, 256, 256, 256, 256, 16, None) == -17
    assert l.simnets_hip_similarity_input_grad(C.byref(a), *shapes, 256, 256, 256, 256, 256, 257, 1 << 30, None) == -17  # misaligned

    m = pkg.ops.mex_attrs(2, blocks=[3, 1, 1], normalize_offsets=True)
    xs = I4(2, 3, 8, 8)
    assert l.simnets_hip_mex_input_grad(C.byref(m), xs, 256, 256, 5, 256, 256, 256, None, 0, None) == -15   # short offsets
    n_off = 64 * 2 * 3
    assert l.simnets_hip_mex_input_grad(C.byref(m), xs, 256, 256, n_off, None, 256, 256, None, 0, None) == -1
    assert l.simnets_hip_mex_offsets_grad(C.byref(m), xs, 256, 256, n_off, 256, 256, None, None, 0, None) == -1
    wi, wo = C.c_size_t(), C.c_size_t()
    assert l.simnets_hip_mex_grad_workspace_bytes(C.byref(m), xs, C.byref(wi), C.byref(wo)) == 0
    assert wi.value >= n_off * 4 and wo.value >= 2 * n_off * 4    # normalised copy; + partial sums
    assert l.simnets_hip_mex_input_grad(C.byref(m), xs, 256, 256, n_off, 256, 256, 256, None, 0, None) == -17
    bad = pkg.ops.mex_attrs(2, blocks=[4, 1, 1])                  # block deeper than the image
    assert l.simnets_hip_mex_offsets_grad(C.byref(bad), xs, 256, 256, n_off, 256, 256, 256, None, 0, None) < 0


def test_launch_time_division_constants_divide_exactly(tmp_path):
    # csrc/fast_div.h (the pixel enumeration of the MEX kernels divides by region sizes fixed per launch):
    # host restatement checked against `/` around multiples of d, at the ends of the range and on random values
    src = tmp_path / "fd.cpp"
    src.write_text(r"""
#include <cstdio>
#include <cstdlib>
#include "fast_div.h"
using namespace simnets;
int main() {
    const unsigned ds[] = {1, 2, 3, 4, 5, 6, 7, 9, 10, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 255, 256, 257, 1000, 4096,
                           65535, 65536, 65537, 1000003, 1u << 30, (1u << 31) - 1, 1u << 31, 0xffffffffu};
    long bad = 0;
    srand(1);
    for (unsigned d : ds) {
        const FastDiv f = make_fast_div(d);
        for (long i = 0; i < 300000; ++i) {
            const unsigned n = i < 1000 ? (unsigned)i : i < 2000 ? 0xffffffffu - (unsigned)(i - 1000)
                                                                 : ((unsigned)rand() << 16) ^ ((unsigned)rand() * 2654435761u);
            for (int dd = -1; dd <= 1; ++dd) {
                const unsigned nn = n - n % d + dd;
                bad += fast_div(nn, f) != nn / d;
            }
        }
    }
    for (unsigned d = 1; d < 2000; ++d) {
        const FastDiv f = make_fast_div(d);
        for (unsigned n = 0; n < 100000; ++n)
            bad += fast_div(n, f) != n / d;
    }
    printf("%ld\n", bad);
    return 0;
}
""")
    exe = tmp_path / "fd"
    subprocess.run(["g++", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "simnets-tf_amd", "csrc"), str(src), "-o",
                    str(exe)], check=True)
    assert subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.strip() == "0"


def test_sum_pool_input_grad_validates_like_the_forward_call(pkg):
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    assert l.simnets_hip_sum_pool_input_grad(I4(2, 3, 8, 8), 0, 2, None, None, None) < 0      # pool size
    assert l.simnets_hip_sum_pool_input_grad(I4(2, 3, 1, 8), 2, 2, None, None, None) < 0      # empty output
    assert l.simnets_hip_sum_pool_input_grad(I4(0, 3, 8, 8), 2, 2, None, None, None) == 0     # empty batch: nothing to do
    assert l.simnets_hip_sum_pool_input_grad(I4(2, 3, 8, 8), 2, 2, None, None, None) < 0      # null pointers


def test_parameter_gradient_tiling_with_many_tiles_and_few_pixels(pkg):
    # dense-layer-like Similarity (1x1 output): more than 512 template x patch-element tiles, fewer than 256 output
    # pixels, and the empty batch: the pixel-split arithmetic must not divide by zero (host only, no launch)
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    a = pkg.ops.similarity_attrs(blocks=[8, 8], strides=[1, 1], padding=[0, 0])
    for batch in (4, 1, 0):
        wp = C.c_size_t()
        assert l.simnets_hip_similarity_grad_workspace_bytes(C.byref(a), I4(batch, 64, 8, 8), I4(1100, 64, 8, 8), None,
                                                             C.byref(wp)) == 0
        assert wp.value >= 2 * 1100 * 64 * 8 * 8 * 4
    a = pkg.ops.similarity_attrs(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    wp = C.c_size_t()
    assert l.simnets_hip_similarity_grad_workspace_bytes(C.byref(a), I4(0, 64, 32, 32), I4(128, 64, 3, 3), None,
                                                         C.byref(wp)) == 0


def test_static_scratch_entry_point_validates_and_bounds_its_scratch(pkg):
    # simnets_hip_similarity_fwd_static: same validation as the workspace entry point, plus the size limit of the
    # library's fixed device array; all decided on the host before anything touches a device
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    a = pkg.ops.similarity_attrs(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    f = l.simnets_hip_similarity_fwd_static
    big = I4(1024, 64, 3, 3)
    need = C.c_size_t()
    assert l.simnets_hip_similarity_workspace_bytes(C.byref(a), I4(1, 64, 8, 8), big, C.byref(need)) == 0
    assert need.value > pkg._lib.STATIC_SCRATCH_BYTES
    assert f(C.byref(a), I4(1, 64, 8, 8), big, big, 256, 256, 256, 256, None) == -21
    assert "scratch" in pkg._lib.strerror(-21)
    small = I4(8, 64, 3, 3)
    assert f(C.byref(a), I4(0, 64, 8, 8), small, small, None, None, None, None, None) == 0     # empty batch
    assert f(C.byref(a), I4(1, 64, 8, 8), small, small, None, 256, 256, 256, None) == -1       # null input
    assert f(C.byref(a), I4(1, 63, 8, 8), small, small, 256, 256, 256, 256, None) == -8        # channel mismatch
    bad = pkg.ops.similarity_attrs(blocks=[3, 3], ignore_nan_input=True)
    assert f(C.byref(bad), I4(1, 64, 8, 8), small, small, 256, 256, 256, 256, None) == -7


def test_prepared_entry_points_validate_on_the_host(pkg):
    # the *_prepare / *_fwd_prepared pairs run the same checks as the self-packing calls before anything is launched
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    a = pkg.ops.similarity_attrs(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    xs, ts = I4(2, 8, 12, 12), I4(5, 8, 3, 3)
    need = C.c_size_t()
    assert l.simnets_hip_similarity_workspace_bytes(C.byref(a), xs, ts, C.byref(need)) == 0 and need.value > 0
    prep, run = l.simnets_hip_similarity_prepare, l.simnets_hip_similarity_fwd_prepared
    assert prep(C.byref(a), xs, ts, ts, None, 256, 256, need.value, None) == -1              # null templates
    assert prep(C.byref(a), xs, ts, ts, 256, 256, None, need.value, None) == -17             # no buffer
    assert prep(C.byref(a), xs, ts, ts, 256, 256, 256, need.value - 1, None) == -17          # buffer too small
    assert prep(C.byref(a), xs, ts, ts, 256, 256, 257, need.value, None) == -17              # misaligned buffer
    assert prep(C.byref(a), xs, I4(5, 7, 3, 3), I4(5, 7, 3, 3), 256, 256, 256, need.value, None) == -8
    assert run(C.byref(a), xs, ts, None, 256, need.value, 256, None) == -1                   # null input
    assert run(C.byref(a), xs, ts, 256, 256, need.value - 1, 256, None) == -17
    assert run(C.byref(a), I4(0, 8, 12, 12), ts, None, None, 0, None, None) == 0             # empty batch: nothing to do
    m = pkg.ops.mex_attrs(4, blocks=[8, 1, 1], strides=[8, 1, 1], unshared_offset_region=[2])
    ms = I4(2, 8, 6, 6)
    assert l.simnets_hip_mex_workspace_bytes(C.byref(m), ms, C.byref(need)) == 0 and need.value > 0
    n_off = 4 * 4 * 8
    assert l.simnets_hip_mex_prepare(C.byref(m), ms, 256, n_off - 1, 256, need.value, None) == -15   # too few offsets
    assert l.simnets_hip_mex_prepare(C.byref(m), ms, None, n_off, 256, need.value, None) == -1
    assert l.simnets_hip_mex_prepare(C.byref(m), ms, 256, n_off, 256, need.value - 1, None) == -17
    assert l.simnets_hip_mex_fwd_prepared(C.byref(m), ms, None, 256, need.value, 256, None) == -1
    assert l.simnets_hip_mex_fwd_prepared(C.byref(m), ms, 256, 256, need.value - 1, 256, None) == -17
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(m), ms, 2, 2, C.byref(need)) == 0
    assert l.simnets_hip_mex_sum_pool_prepare(C.byref(m), ms, 256, n_off, 0, 2, 256, need.value, None) == -15   # pool size
    assert l.simnets_hip_mex_sum_pool_prepare(C.byref(m), ms, 256, n_off, 2, 2, None, need.value, None) == -17
    assert l.simnets_hip_mex_sum_pool_fwd_prepared(C.byref(m), ms, 256, 8, 8, 256, need.value, 256, None) == -16  # empty output
    sa = pkg.ops.similarity_attrs(blocks=[2, 2], strides=[2, 2], padding=[0, 0])
    sx, st = I4(2, 1, 12, 12), I4(8, 1, 2, 2)
    assert l.simnets_hip_similarity_mex_sum_pool_workspace_bytes(C.byref(sa), sx, st, C.byref(m), 2, 2,
                                                                 C.byref(need)) == 0
    f = l.simnets_hip_similarity_mex_sum_pool_prepare
    assert f(C.byref(sa), sx, st, 256, None, C.byref(m), 256, n_off, 2, 2, 256, need.value, None) == -1         # null weights
    assert f(C.byref(sa), sx, st, 256, 256, C.byref(m), 256, n_off - 1, 2, 2, 256, need.value, None) == -15
    g = l.simnets_hip_similarity_mex_sum_pool_fwd_prepared
    assert g(C.byref(sa), sx, st, None, C.byref(m), 2, 2, 256, need.value, 256, None) == -1
    assert g(C.byref(sa), sx, st, 256, C.byref(m), 2, 2, 256, need.value - 1, 256, None) == -17


def test_saving_and_saved_entry_points_validate_on_the_host(pkg):
    """simnets_hip_mex_saved_bytes sizes the buffer a training forward fills for the gradient call; the *_saving and
    *_saved calls check it (size, 256-byte alignment, presence) before anything is launched."""
    l = pkg._lib.lib()
    I4 = C.c_int * 4
    xs = I4(2, 32, 8, 8)
    n_off = 4 * 6 * 32
    m = pkg.ops.mex_attrs(6, blocks=[32, 1, 1], strides=[32, 1, 1], unshared_offset_region=[1, 2, 2], normalize_offsets=True)
    kept = C.c_size_t()
    assert l.simnets_hip_mex_saved_bytes(C.byref(m), xs, C.byref(kept)) == 0
    # exponentials, scaled values and two row tables in groups of 32 instances, the element table, the normalised copy
    assert kept.value >= (2 * 4 * 32 * 32 + 4 * 6 * 32) * 4 and kept.value % 256 == 0
    assert l.simnets_hip_mex_saved_bytes(C.byref(m), xs, None) == -1
    inf = pkg.ops.mex_attrs(6, blocks=[32, 1, 1], strides=[32, 1, 1], unshared_offset_region=[1, 2, 2], epsilon=float("inf"))
    assert l.simnets_hip_mex_saved_bytes(C.byref(inf), xs, C.byref(kept)) == 0 and kept.value == 0
    # few instances over long patches: only the normalised copy (nothing without normalisation)
    head = pkg.ops.mex_attrs(10, blocks=[512, 1, 1], strides=[512, 1, 1], use_unshared_regions=False,
                             shared_offset_region=[-1], normalize_offsets=True)
    hs = I4(64, 512, 1, 1)
    assert l.simnets_hip_mex_saved_bytes(C.byref(head), hs, C.byref(kept)) == 0 and kept.value == 10 * 512 * 4
    head.normalize_offsets = 0
    assert l.simnets_hip_mex_saved_bytes(C.byref(head), hs, C.byref(kept)) == 0 and kept.value == 0

    assert l.simnets_hip_mex_saved_bytes(C.byref(m), xs, C.byref(kept)) == 0
    ws = C.c_size_t()
    assert l.simnets_hip_mex_workspace_bytes(C.byref(m), xs, C.byref(ws)) == 0
    big = 1 << 30
    # forward: no buffer, a short one, a misaligned one
    assert l.simnets_hip_mex_fwd_saving(C.byref(m), xs, 256, 256, n_off, 256, None, 0, 256, big, None) == -17
    assert l.simnets_hip_mex_fwd_saving(C.byref(m), xs, 256, 256, n_off, 256, 256, kept.value - 1, 256, big, None) == -17
    assert l.simnets_hip_mex_fwd_saving(C.byref(m), xs, 256, 256, n_off, 256, 257, big, 256, big, None) == -17
    assert l.simnets_hip_mex_fwd_saving(C.byref(m), xs, 256, 256, 5, 256, 256, big, 256, big, None) == -15     # short offsets
    assert l.simnets_hip_mex_sum_pool_fwd_saving(C.byref(m), xs, 256, 256, n_off, 2, 2, 256, 256, 256, 16, 256, big,
                                                 None) == -17
    assert l.simnets_hip_mex_sum_pool_fwd_saving(C.byref(m), xs, 256, 256, n_off, 2, 2, None, 256, 256, big, 256, big,
                                                 None) == -1                                                     # no MEX output
    assert l.simnets_hip_mex_sum_pool_fwd_saving(C.byref(m), xs, 256, 256, n_off, 0, 2, 256, 256, 256, big, 256, big,
                                                 None) == -15                                                    # window
    # gradients: a buffer that is given must be whole and aligned (none at all = the plain call)
    assert l.simnets_hip_mex_grads_saved(C.byref(m), xs, 256, 256, n_off, 256, 256, 256, 16, 256, 256, 256, big, None) == -17
    assert l.simnets_hip_mex_grads_saved(C.byref(m), xs, 256, 256, n_off, 256, 256, 257, big, 256, 256, 256, big, None) == -17
    assert l.simnets_hip_mex_grads_saved(C.byref(m), xs, 256, 256, n_off, 256, 256, 256, big, 256, None, 256, big, None) == -1
    assert l.simnets_hip_mex_sum_pool_grads_saved(C.byref(m), xs, 256, 256, n_off, 2, 2, 256, 256, 256, 16, 256, 256,
                                                  256, big, None) == -17
    assert l.simnets_hip_mex_sum_pool_grads_saved(C.byref(m), xs, 256, 256, n_off, 2, 2, 256, 256, 256, big, None, None,
                                                  256, big, None) == -1                                          # no gradient wanted
