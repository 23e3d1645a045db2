"""torch.library registration (simnets-tf_amd/torch_ops.py): shape inference without a GPU, execution,
autograd and tracing on one."""
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

from conftest import load_package

pkg = load_package()
SIM = ("L2", [2, 2], [3, 2], [1, 1], False, 0.001, False, 0.0)


def test_fake_kernels_infer_the_reference_known_answer_shapes():
    # python/simnets/test/keras/__init__.py:46-55
    with FakeTensorMode():
        x = torch.empty(5, 3, 10, 13, device="cuda")
        t = torch.empty(10, 3, 2, 2, device="cuda")
        y = torch.ops.simnets.similarity(x, t, t, *SIM)
        assert tuple(y.shape) == (5, 10, 4, 7)
        off = torch.empty(4, 6, 10, 1, 1, device="cuda")
        z = torch.ops.simnets.mex(y, off, 6, True, [0, 0, 0], [10, 1, 1], [10, 1, 1], 1.0, 0.0, True, True, [-1], [2], True)
        assert tuple(z.shape) == (5, 6, 4, 7)
        assert tuple(torch.ops.simnets.similarity_input_grad(x, t, t, y, *SIM).shape) == tuple(x.shape)
        assert tuple(torch.ops.simnets.mex_offsets_grad(y, off, z, z, 6, True, [0, 0, 0], [10, 1, 1], [10, 1, 1], 1.0, 0.0,
                                                        True, True, [-1], [2], True).shape) == tuple(off.shape)


def test_fake_kernels_reject_invalid_attributes():
    with FakeTensorMode():
        x = torch.empty(1, 3, 10, 13, device="cuda")
        t = torch.empty(4, 3, 2, 2, device="cuda")
        with pytest.raises(Exception):
            torch.ops.simnets.similarity(x, t, t, "L3", [2, 2], [1, 1], [0, 0], False, 0.001, False, 0.0)


@pytest.mark.gpu
def test_registered_ops_execute_differentiate_and_trace():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 10, 13, generator=g).cuda().requires_grad_()
    t = torch.randn(10, 3, 2, 2, generator=g).cuda().requires_grad_()
    w = (torch.rand(10, 3, 2, 2, generator=g) + 0.1).cuda().requires_grad_()
    off = torch.randn(4, 6, 10, 1, 1, generator=g).cuda().requires_grad_()
    mex_attrs = (6, True, [0, 0, 0], [10, 1, 1], [10, 1, 1], 1.0, 0.0, True, True, [-1], [2], True)

    def net(x, t, w, off):
        return torch.ops.simnets.mex(torch.ops.simnets.similarity(x, t, w, *SIM), off, *mex_attrs)

    y = net(x, t, w, off)
    ref_leaves = [a.detach().clone().requires_grad_() for a in (x, t, w, off)]
    ref = pkg.layers.mex(pkg.layers.similarity(*ref_leaves[:3], similarity_function="L2", blocks=[2, 2], strides=[3, 2],
                                               padding=[1, 1]),
                         ref_leaves[3], 6, softmax_mode=True, blocks=[10, 1, 1], strides=[10, 1, 1],
                         unshared_offset_region=[2], normalize_offsets=True)
    assert torch.equal(y, ref)
    go = torch.randn(y.shape, generator=g).cuda()
    y.backward(go)
    ref.backward(go)
    for a, b in zip((x, t, w, off), ref_leaves):
        assert torch.equal(a.grad, b.grad)
    traced = torch.compile(net, backend="aot_eager", fullgraph=True)
    assert torch.equal(traced(x.detach(), t.detach(), w.detach(), off.detach()), y.detach())
    torch.library.opcheck(torch.ops.simnets.similarity.default, (x.detach(), t.detach(), w.detach()) + SIM,
                          test_utils=("test_schema", "test_faketensor"))
