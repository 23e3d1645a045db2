"""The differentiable op layer and the module classes (python/simnets/keras.py of the reference) on the GPU."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from util import rel_err

pytestmark = pytest.mark.gpu


def test_autograd_routes_to_the_grad_entry_points(pkg):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 3, 9, 8, generator=g).cuda().requires_grad_()
    t = torch.randn(4, 3, 3, 3, generator=g).cuda().requires_grad_()
    w = (torch.rand(4, 3, 3, 3, generator=g) + 0.1).cuda().requires_grad_()
    kw = dict(blocks=[3, 3], strides=[2, 1], padding=[1, 1])
    out = pkg.layers.similarity(x, t, w, **kw)
    go = torch.randn(out.shape, generator=g).cuda()
    out.backward(go)
    assert torch.equal(x.grad, pkg.similarity_input_grad(x.detach(), t.detach(), w.detach(), go, **kw))
    dt, dw = pkg.similarity_parameters_grad(x.detach(), t.detach(), w.detach(), go, **kw)
    assert torch.equal(t.grad, dt) and torch.equal(w.grad, dw)

    off = torch.randn(4, 5, 3, 1, 1, generator=g).cuda().requires_grad_()
    x2 = x.detach().clone().requires_grad_()
    mkw = dict(blocks=[3, 1, 1], strides=[3, 1, 1], unshared_offset_region=[2], softmax_mode=True)
    y = pkg.layers.mex(x2, off, 5, **mkw)
    gy = torch.randn(y.shape, generator=g).cuda()
    y.backward(gy)
    assert torch.equal(x2.grad, pkg.mex_input_grad(x2.detach(), off.detach(), y.detach(), gy, 5, **mkw))
    assert torch.equal(off.grad, pkg.mex_offsets_grad(x2.detach(), off.detach(), y.detach(), gy, 5, **mkw))


def test_autograd_matches_torch_autograd_of_the_closed_form(pkg):
    """Similarity L2 written with unfold, MEX 1x1 written with logsumexp: torch's own autograd is the check."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 3, 10, 9, generator=g).cuda()
    t = torch.randn(6, 3, 3, 2, generator=g).cuda()
    w = (torch.rand(6, 3, 3, 2, generator=g) + 0.1).cuda()
    leaves = [a.clone().requires_grad_() for a in (x, t, w)]
    out = pkg.layers.similarity(*leaves, blocks=[3, 2], strides=[1, 2], padding=[1, 0])
    ref_leaves = [a.double().requires_grad_() for a in (x, t, w)]
    cols = F.unfold(ref_leaves[0], (3, 2), padding=(1, 0), stride=(1, 2))
    d = cols[:, None] - ref_leaves[1].reshape(6, -1)[None, :, :, None]
    ref = -(ref_leaves[2].reshape(6, -1)[None, :, :, None] * d * d).sum(2).reshape(out.shape)
    go = torch.randn(out.shape, generator=g).cuda()
    out.backward(go)
    ref.backward(go.double())
    assert rel_err(out.detach().cpu().numpy(), ref.detach().cpu().numpy()) <= 1e-5
    for a, b in zip(leaves, ref_leaves):
        scale = b.grad.abs().max().item()
        assert rel_err(a.grad.cpu().numpy(), b.grad.cpu().numpy(), floor=np.full(tuple(b.shape), 1e-2 * scale)) <= 1e-4


def test_layers_build_lazily_with_the_reference_shapes(pkg):
    # python/simnets/test/keras/__init__.py:46-55, :110-119
    for num, padding, strides, blocks, in_shape, out_shape in [
            (10, [0, 1], [1, 1], [2, 2], (3, 10, 13), (10, 9, 14)),
            (10, [1, 1], [3, 2], [2, 2], (3, 10, 13), (10, 4, 7)),
            (2, [1, 1], [3, 2], [2, 2], (1, 10, 13), (2, 4, 7))]:
        layer = pkg.Similarity(num, padding=padding, strides=strides, blocks=blocks)
        assert layer.compute_output_shape((5,) + in_shape) == (5,) + out_shape
        y = layer(torch.zeros((5,) + in_shape).cuda())
        assert tuple(y.shape) == (5,) + out_shape
        assert tuple(layer.templates.shape) == (num, in_shape[0]) + tuple(blocks) == tuple(layer.sweights.shape)
    layer = pkg.Mex(4, blocks=[-1, 2, 2], strides=[3, 2, 2], unshared_offset_region=[2], softmax_mode=True,
                    normalize_offsets=True)
    y = layer(torch.randn(2, 3, 8, 8).cuda())
    assert tuple(y.shape) == (2, 4, 4, 4) == layer.compute_output_shape((2, 3, 8, 8))
    assert tuple(layer.offsets.shape) == (4, 4, 3, 2, 2)
    # dirichlet initialisation: rows are log-probabilities
    np.testing.assert_allclose(layer.offsets.detach().exp().sum(dim=(2, 3, 4)).cpu().numpy(), 1.0, rtol=1e-5)


def test_channels_last_is_a_transposition(pkg):
    torch.manual_seed(3)
    a = pkg.Similarity(5, blocks=[3, 3], padding="SAME")
    b = pkg.Similarity(5, blocks=[3, 3], padding="SAME", channels_last=True)
    x = torch.randn(2, 3, 7, 6).cuda()
    ya = a(x)
    b.build((2, 7, 6, 3))
    b.cuda()
    with torch.no_grad():
        b.templates.copy_(a.templates)
        b.sweights.copy_(a.sweights)
    yb = b(x.permute(0, 2, 3, 1).contiguous())
    assert torch.equal(yb.permute(0, 3, 1, 2), ya)


def test_a_small_network_trains(pkg):
    """Similarity -> Mex -> Mex (to 1x1) as in the reference's example network; a few SGD steps on a fixed batch
    must lower the cross-entropy, with all parameters receiving finite gradients."""
    torch.manual_seed(4)
    net = torch.nn.Sequential(
        pkg.Similarity(8, blocks=[2, 2], strides=[2, 2], padding=[0, 0], normalization_term=True, ignore_nan_input=True,
                       out_of_bounds_value=float("nan")),
        pkg.Mex(6, blocks=[-1, 2, 2], strides=[8, 2, 2], softmax_mode=True, normalize_offsets=True,
                unshared_offset_region=[2]),
        pkg.Mex(3, blocks=[-1, -1, -1], softmax_mode=True, normalize_offsets=True, use_unshared_regions=False,
                shared_offset_region=[-1]),
    )
    x = torch.rand(16, 1, 8, 8).cuda() - 0.5
    x[torch.rand(x.shape, device="cuda") < 0.2] = float("nan")
    labels = (torch.arange(16) % 3).cuda()
    logits = net(x)
    assert tuple(logits.shape) == (16, 3, 1, 1)
    opt = torch.optim.SGD(net.parameters(), lr=0.05)
    losses = []
    for _ in range(12):
        opt.zero_grad()
        loss = torch.nn.functional.cross_entropy(net(x).flatten(1), labels)
        loss.backward()
        for p in net.parameters():
            assert torch.isfinite(p.grad).all()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0]


def test_layerwise_unsupervised_initialisation(pkg):
    """perform_unsupervised_init walks the network like python/simnets/keras.py:199-243: each Similarity layer is
    initialised from what the already initialised layers before it produce."""
    torch.manual_seed(5)
    net = torch.nn.Sequential(
        pkg.Similarity(6, blocks=[2, 2], strides=[2, 2], padding=[0, 0]),
        pkg.Mex(4, blocks=[-1, 1, 1], strides=[6, 1, 1], softmax_mode=True, normalize_offsets=True),
        pkg.Similarity(3, blocks=[2, 2], strides=[1, 1], padding=[0, 0]),
    )
    data = torch.randn(32, 2, 8, 8).cuda()
    net(data[:2])    # builds the lazily shaped parameters
    before = [net[0].templates.detach().clone(), net[2].templates.detach().clone()]
    pkg.unsupervised.perform_unsupervised_init(net, "kmeans", data=data, batch_size=8)
    assert not torch.equal(net[0].templates, before[0]) and not torch.equal(net[2].templates, before[1])
    assert torch.equal(net[0].sweights, torch.ones_like(net[0].sweights))
    # the first layer's templates are means of input patches: inside the data's range
    assert net[0].templates.abs().max() <= data.abs().max()
    assert torch.isfinite(net(data)).all()


def test_missing_data_stack_replays_from_a_hip_graph(pkg):
    """The whole stack (Similarity -> 4 x (MEX + sum pool) -> MEX) is kernel launches on the caller's stream and
    nothing else (no allocation, no memset, no host synchronisation once the workspace exists), so it can be
    captured once and replayed.  Every replay, with new input contents and eager work in between, must reproduce the
    eager result bit for bit."""
    from util import config1
    x, t, w, kw = config1(batch=32, nan_frac=0.25)
    T, W = torch.from_numpy(t).cuda(), torch.from_numpy(w).cuda()
    g = np.random.default_rng(4567)
    layers, ch, size = [], 32, 16
    for _ in range(4):
        n = ch * 2
        off = torch.from_numpy((g.normal(size=(4 if size > 1 else 1, n, ch, 1, 1)) * 0.1).astype(np.float32)).cuda()
        layers.append((off, n, dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1], unshared_offset_region=[2])))
        ch, size = n, size // 2
    offl = torch.from_numpy((g.normal(size=(1, 10, ch, 1, 1)) * 0.1).astype(np.float32)).cuda()

    def stack(inp):
        cur = pkg.similarity(inp, T, W, **kw)
        for off, n, lkw in layers:
            cur = pkg.sum_pooling(pkg.mex(cur, off, n, normalize_offsets=True, **lkw), (2, 2))
        return pkg.mex(cur, offl, 10, normalize_offsets=True, softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1],
                       shared_offset_region=[1])

    static_in = torch.from_numpy(x).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):          # warm-up on the capture stream: workspace and allocator pools exist afterwards
            stack(static_in)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = stack(static_in)
    for trial in range(4):
        fresh, _, _, _ = config1(batch=32, seed=100 + trial, nan_frac=0.25)
        static_in.copy_(torch.from_numpy(fresh))
        graph.replay()
        torch.cuda.synchronize()
        got = static_out.clone()
        want = stack(torch.from_numpy(fresh).cuda())     # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), "replay %d" % trial


def test_mex_sum_pool_functional_fused_without_gradients_split_with(pkg):
    g = np.random.default_rng(31)
    x = torch.from_numpy(g.normal(size=(3, 16, 8, 8)).astype(np.float32)).cuda()
    off = torch.from_numpy((g.normal(size=(4, 12, 16, 1, 1)) * 0.2).astype(np.float32)).cuda()
    kw = dict(blocks=[16, 1, 1], strides=[16, 1, 1], unshared_offset_region=[1, 2, 2], softmax_mode=True)
    with torch.no_grad():
        fused = pkg.layers.mex_sum_pool(x, off, 12, (2, 2), **kw)
    off.requires_grad_()
    split = pkg.layers.mex_sum_pool(x, off, 12, (2, 2), **kw)
    assert split.requires_grad and fused.shape == split.shape == (3, 12, 4, 4)
    assert float((fused - split.detach()).abs().max()) <= 1e-5 * float(split.detach().abs().max())
    split.sum().backward()
    y = pkg.mex(x, off.detach(), 12, **kw)
    want = pkg.mex_offsets_grad(x, off.detach(), y, torch.ones_like(y), 12, **kw)
    assert torch.allclose(off.grad, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("case", [
    dict(im=(9, 32, 16, 16), n=64, pool=(2, 2)),                        # fused kernel (first MEX layer of the stack)
    dict(im=(7, 64, 8, 8), n=70, pool=(2, 2)),                          # panel form, a partial instance group
    dict(im=(5, 256, 2, 2), n=130, pool=(2, 2)),                        # panel form, one window per image
    dict(im=(3, 6, 9, 11), n=20, pool=(2, 2)),                          # odd sizes: pixels no window takes still get a MEX value
    dict(im=(4, 8, 6, 10), n=33, pool=(1, 2)),                          # two-pixel windows
    dict(im=(4, 12, 8, 8), n=10, pool=(2, 2), kw=dict(blocks=[3, 1, 1], strides=[3, 1, 1], shared_offset_region=[2],
                                                      use_unshared_regions=False)),   # not fusable: two kernels
])
@pytest.mark.parametrize("spread", ["narrow", "wide"])
def test_mex_sum_pool_for_training_keeps_the_mex_output(pkg, case, spread):
    """`mex_sum_pool_both` (what `layers.mex_sum_pool` runs when a gradient is needed) returns the MEX output before
    pooling and the pooled output from one call: the pooled tensor has the bits `mex_sum_pool` gives (the same kernel
    with one more store), the MEX output the values of `mex` up to rounding (another kernel may serve the plain call),
    and gradients through it agree with those of the two separate differentiable calls."""
    g = torch.Generator(device="cuda").manual_seed(12)
    im, n, pool = case["im"], case["n"], case["pool"]
    kw = dict(dict(softmax_mode=True, blocks=[im[1], 1, 1], strides=[im[1], 1, 1],
                   unshared_offset_region=[1, pool[0], pool[1]], epsilon=1.5), **case.get("kw", {}))
    x = torch.randn(im, device="cuda", generator=g)
    _, oshape = pkg.mex_output_shape(im, n, **kw)
    off = torch.randn(oshape, device="cuda", generator=g) * (150.0 if spread == "wide" else 0.3)
    full, pooled = pkg.mex_sum_pool_both(x, off, n, pool, normalize_offsets=True, **kw)
    plain = pkg.mex(x, off, n, normalize_offsets=True, **kw)
    scale = float(plain.abs().max())
    assert full.shape == plain.shape and float((full - plain).abs().max()) <= 1e-5 * scale
    assert torch.equal(pooled, pkg.mex_sum_pool(x, off, n, pool, normalize_offsets=True, **kw))
    assert torch.equal(pooled, pkg.sum_pooling(full, pool))
    # gradients: fused forward against the two separate differentiable calls
    L = pkg.layers
    leaves = [t.clone().requires_grad_() for t in (x, off, x, off)]
    y1 = L.mex_sum_pool(leaves[0], leaves[1], n, pool, normalize_offsets=True, **kw)
    y2 = L.sum_pooling(L.mex(leaves[2], leaves[3], n, normalize_offsets=True, **kw), pool)
    assert float((y1 - y2).detach().abs().max()) <= 1e-5 * float(y2.detach().abs().max())
    go = torch.randn(y1.shape, device="cuda", generator=g)
    y1.backward(go)
    y2.backward(go)
    for a, b in ((leaves[0].grad, leaves[2].grad), (leaves[1].grad, leaves[3].grad)):
        assert float((a - b).abs().max()) <= 1e-4 * float(b.abs().max())


@pytest.mark.parametrize("spread", ["narrow", "mixed"])
@pytest.mark.parametrize("im,n,pool,kw", [
    ((5, 32, 16, 16), 64, (2, 2), {}),                      # row-wise kernels read the window gradients themselves
    ((9, 40, 8, 8), 70, (2, 2), {}),                        # ... ragged blocks, part-empty last chunk
    ((17, 16, 4, 4), 33, (2, 2), {}),                       # ... sixteen images a chunk
    ((3, 8, 4, 32), 6, (2, 2), {}),
    ((70, 16, 2, 2), 20, (2, 2), {}),                       # width 2: expanded gradient, gathering kernels
    ((6, 8, 8, 2), 5, (2, 2), {}),
    ((3, 12, 6, 10), 5, (2, 2), {}),                        # map sides no powers of two: expanded gradient
    ((2, 6, 9, 8), 4, (3, 2), {}),                          # 3 x 2 windows, a row left over
    ((4, 6, 8, 8), 5, (2, 2), dict(unshared_offset_region=[1, 4, 4])),   # window is not the region grid
    ((3, 16, 8, 8), 7, (2, 2), dict(epsilon=float("inf"))),
    ((5, 96, 4, 4), 6, (2, 2), {}),                                       # few instances over long patches: one kernel for both
    ((40, 256, 2, 2), 48, (2, 2), {}),                                    # 2x2 maps: the gathering kernels
])
def test_mex_sum_pool_grads_from_the_pooled_gradient(pkg, im, n, pool, kw, spread):
    """`mex_sum_pool_grads` = `mex_grads` on the expanded pooling gradient, bit for bit - whether the gradient kernels
    read the window gradients themselves or the call expands them first -, for both gradients, either alone, and
    through unaligned views."""
    g = torch.Generator(device="cuda").manual_seed(21)
    kw = dict(dict(softmax_mode=True, blocks=[im[1], 1, 1], strides=[im[1], 1, 1],
                   unshared_offset_region=[1, pool[0], pool[1]], epsilon=1.5, normalize_offsets=True), **kw)
    x = torch.randn(im, device="cuda", generator=g)
    _, oshape = pkg.mex_output_shape(im, n, **{k: v for k, v in kw.items() if k != "normalize_offsets"})
    off = torch.randn(oshape, device="cuda", generator=g) * 0.3
    if spread == "mixed":
        off[::2] *= 300
    full, pooled = pkg.mex_sum_pool_both(x, off, n, pool, **kw)
    gp = torch.randn(pooled.shape, device="cuda", generator=g)
    want_dx, want_doff = pkg.mex_grads(x, off, full, pkg.sum_pooling_input_grad(gp, full.shape, pool), n, **kw)
    dx, doff = pkg.mex_sum_pool_grads(x, off, full, gp, n, pool, **kw)
    assert torch.equal(dx, want_dx) and torch.equal(doff, want_doff)
    only_dx, none = pkg.mex_sum_pool_grads(x, off, full, gp, n, pool, want_offsets=False, **kw)
    assert none is None and torch.equal(only_dx, want_dx)
    none, only_doff = pkg.mex_sum_pool_grads(x, off, full, gp, n, pool, want_input=False, **kw)
    assert none is None and torch.equal(only_doff, want_doff)

    def shifted(t):
        buf = torch.empty(t.numel() + 1, device="cuda")
        v = buf[1:].view(t.shape)
        v.copy_(t)
        return v

    dx_u, doff_u = pkg.mex_sum_pool_grads(shifted(x), off, shifted(full), shifted(gp), n, pool, **kw)
    assert float((dx_u - want_dx).abs().max()) <= 1e-4 * float(want_dx.abs().max())
    assert float((doff_u - want_doff).abs().max()) <= 1e-4 * float(want_doff.abs().max())
    with pytest.raises(pkg.SimnetsError):
        pkg.mex_sum_pool_grads(x, off, full, gp[:, :, :-1], n, pool, **kw)


@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("im,n,kw", [
    ((64, 32, 16, 16), 64, {}),                            # one-launch forward that packs inside its kernel
    ((8, 32, 16, 16), 70, {}),                             # instance count that pads both layouts differently (128 / 96)
    ((16, 64, 8, 8), 128, {}),                             # panel kernel, row-wise gradient kernels
    ((16, 256, 2, 2), 40, {}),                             # 2x2 maps: gathering gradient kernels
    ((32, 100, 1, 1), 10, dict(unshared_offset_region=[1, 1, 1])),   # head: wave-per-pixel forward (groups of one)
    ((3, 6, 9, 7), 21, dict(blocks=[3, 2, 2], strides=[2, 1, 1], padding=[1, 1, 0], unshared_offset_region=[2, 3, 2])),
    ((4, 16, 8, 8), 33, dict(use_unshared_regions=False, shared_offset_region=[2])),
    ((4, 16, 8, 8), 9, dict(epsilon=float("-inf"))),       # nothing to keep: the gradient kernels read the offsets
    ((4, 600, 4, 4), 12, {}),                              # rows of more than 256 elements
    ((0, 16, 8, 8), 5, {}),
])
def test_mex_forward_keeps_the_offsets_for_the_gradient_call(pkg, im, n, kw, normalize):
    """`mex_saving` / `mex_sum_pool_saving` = the plain forward calls, and the gradient calls given what they kept =
    the plain gradient calls, all bit for bit; the kept buffer stays valid while other layers run on the stream (it is
    no part of the calls' scratch)."""
    g = torch.Generator(device="cuda").manual_seed(5)
    kw = dict(dict(softmax_mode=True, blocks=[im[1], 1, 1], strides=[im[1], 1, 1], unshared_offset_region=[1, 2, 2],
                   epsilon=1.5, normalize_offsets=normalize), **kw)
    x = torch.randn(im, device="cuda", generator=g)
    _, oshape = pkg.mex_output_shape(im, n, **{k: v for k, v in kw.items() if k != "normalize_offsets"})
    off = torch.randn(oshape, device="cuda", generator=g)
    off[:, ::3] *= 40           # some instances beyond the product form
    y = pkg.mex(x, off, n, **kw)
    ys, kept = pkg.mex_saving(x, off, n, **kw)
    assert torch.equal(y, ys) and kept.dtype == torch.uint8
    # nothing to keep where the gradient kernels read the offsets as they are: an infinite epsilon, and the kernel for
    # few instances over long patches (which only wants the normalised copy)
    if not math.isfinite(kw["epsilon"]) or (im[1] == 100 and not normalize):
        assert kept.numel() == 0
    # another layer in between: its calls reuse the scratch of this one's
    other = pkg.mex(torch.randn(5, 8, 6, 6, device="cuda"), torch.randn(1, 3, 8, 1, 1, device="cuda"), 3,
                    blocks=[8, 1, 1], strides=[8, 1, 1], use_unshared_regions=False, shared_offset_region=[-1])
    gy = torch.randn(y.shape, device="cuda", generator=g)
    want = pkg.mex_grads(x, off, y, gy, n, **kw)
    got = pkg.mex_grads(x, off, y, gy, n, saved=kept, **kw)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    assert other.shape == (5, 3, 6, 6)
    if y.shape[2] >= 2 and y.shape[3] >= 2:
        full, pooled = pkg.mex_sum_pool_both(x, off, n, (2, 2), **kw)
        fulls, pooleds, kept2 = pkg.mex_sum_pool_saving(x, off, n, (2, 2), **kw)
        assert torch.equal(full, fulls) and torch.equal(pooled, pooleds)
        gp = torch.randn(pooled.shape, device="cuda", generator=g)
        want = pkg.mex_sum_pool_grads(x, off, full, gp, n, (2, 2), **kw)
        got = pkg.mex_sum_pool_grads(x, off, full, gp, n, (2, 2), saved=kept2, **kw)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        only = pkg.mex_sum_pool_grads(x, off, full, gp, n, (2, 2), want_input=False, saved=kept2, **kw)
        assert only[0] is None and torch.equal(only[1], want[1])
    if kept.numel() > 256:
        with pytest.raises(pkg.SimnetsError):   # a buffer that is too small
            pkg.mex_grads(x, off, y, gy, n, saved=kept[:256], **kw)


@pytest.mark.parametrize("shape,pool", [((3, 5, 8, 10), (2, 2)), ((2, 3, 7, 9), (2, 3)), ((1, 4, 5, 5), (5, 1))])
def test_sum_pooling_gradient(pkg, shape, pool):
    """layers.sum_pooling: forward = avg_pool2d * area ('valid': trailing rows/columns dropped), the gradient spreads
    each window's gradient over its elements and gives the dropped ones 0 - checked against torch's own autograd."""
    x = torch.randn(*shape, device="cuda", requires_grad=True)
    y = pkg.layers.sum_pooling(x, pool)
    g = torch.randn_like(y)
    y.backward(g)
    xr = x.detach().clone().requires_grad_()
    yr = torch.nn.functional.avg_pool2d(xr, pool) * float(pool[0] * pool[1])
    yr.backward(g)
    assert torch.allclose(y, yr, rtol=1e-6, atol=1e-6)
    assert torch.equal(x.grad, xr.grad * 0 + x.grad) and torch.allclose(x.grad, xr.grad, rtol=1e-6, atol=1e-7)
    with pytest.raises(pkg.SimnetsError):
        pkg.sum_pooling_input_grad(g[:, :, :-1] if g.shape[2] > 1 else g[:, :-1], shape, pool)


def test_gradient_calls_replay_from_a_hip_graph(pkg):
    """The gradient calls, too, are kernel launches on the caller's stream and nothing else: their scratch (partial
    sums, centres, packed parameters, flags, the patch-gradient buffer of overlapping MEX patches) is rewritten by
    every call.  Captured once, every replay on new data - with eager calls in between - reproduces the eager
    results bit for bit (the sums run in a fixed order)."""
    g = np.random.default_rng(77)
    skw = dict(similarity_function="L2", blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    mkw = dict(blocks=[3, 2, 2], strides=[2, 1, 1], padding=[1, 0, 0], epsilon=2.0, softmax_mode=True,
               use_unshared_regions=False, shared_offset_region=[2])
    T = torch.from_numpy(g.normal(size=(12, 32, 3, 3)).astype(np.float32)).cuda()
    W = torch.from_numpy((np.abs(g.normal(size=(12, 32, 3, 3))) + 0.05).astype(np.float32)).cuda()

    def fresh(seed):
        q = np.random.default_rng(seed)
        x = torch.from_numpy(q.normal(size=(3, 32, 12, 32)).astype(np.float32)).cuda()
        gs = torch.from_numpy(q.normal(size=(3, 12, 12, 32)).astype(np.float32)).cuda()
        return x, gs

    sx, sg = fresh(0)
    n_inst = 5
    y0 = pkg.similarity(sx, T, W, **skw)
    dshape, oshape = pkg.mex_output_shape(tuple(y0.shape), n_inst, **mkw)
    off = torch.from_numpy((g.normal(size=oshape) * 0.3).astype(np.float32)).cuda()
    gm = torch.from_numpy(g.normal(size=dshape).astype(np.float32)).cuda()

    def work(x, gs):
        y = pkg.similarity(x, T, W, **skw)
        dx = pkg.similarity_input_grad(x, T, W, gs, **skw)
        dt, dw = pkg.similarity_parameters_grad(x, T, W, gs, **skw)
        z = pkg.mex(y, off, n_inst, **mkw)
        dy = pkg.mex_input_grad(y, off, z, gm, n_inst, **mkw)
        do = pkg.mex_offsets_grad(y, off, z, gm, n_inst, **mkw)
        return dx, dt, dw, dy, do

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            work(sx, sg)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = work(sx, sg)
    for trial in range(3):
        x, gs = fresh(10 + trial)
        sx.copy_(x)
        sg.copy_(gs)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in static_out]
        want = work(x, gs)
        torch.cuda.synchronize()
        for a, b, name in zip(got, want, ("dX", "dT", "dW", "mex dX", "mex dOff")):
            assert torch.equal(a, b), "replay %d: %s" % (trial, name)


def test_modules_pack_parameters_once_for_inference(pkg):
    """Under no_grad the Similarity / Mex modules run the prepared calls: same bits as the training-mode forward, one
    buffer per (input shape, parameter version), a fresh one after the parameters change."""
    g = torch.Generator(device="cuda").manual_seed(5)
    sim = pkg.Similarity(12, blocks=[3, 3], strides=[1, 1], padding=[1, 1]).cuda()
    mexl = pkg.Mex(7, blocks=[-1, 1, 1], strides=[12, 1, 1], softmax_mode=True, normalize_offsets=True,
                   unshared_offset_region=[2]).cuda()
    x = torch.randn((3, 5, 10, 10), device="cuda", generator=g)
    y_train = mexl(sim(x))
    with torch.no_grad():
        y1 = mexl(sim(x))
        first = (sim._prepared.last(), mexl._prepared.last())
        y2 = mexl(sim(x))
        assert sim._prepared.last() is first[0] and mexl._prepared.last() is first[1]      # reused
        assert torch.equal(y1, y_train.detach()) and torch.equal(y2, y1)
        sim.templates.add_(0.25)
        mexl.offsets.mul_(0.5)
        y3 = mexl(sim(x))
        assert sim._prepared.last() is not first[0] and mexl._prepared.last() is not first[1]
    assert torch.equal(y3, mexl(sim(x)).detach()) and not torch.equal(y3, y1)
    with torch.no_grad():
        assert mexl(sim(x[:2])).shape[0] == 2                                      # another input shape: prepared anew


def test_modules_notice_rebound_parameters_changed_attributes_and_other_streams(pkg):
    """The inference cache must never serve a stale packed buffer: rebinding a parameter (a new tensor object whose
    version counter starts at 0 again), `load_state_dict(assign=True)`, and a changed layer attribute each prepare
    anew; a write through `.data` (invisible to torch's version counter) needs `invalidate_prepared()`; every stream
    gets a buffer of its own.  Each result equals the grad-mode forward, which packs on every call."""
    g = torch.Generator(device="cuda").manual_seed(11)
    sim = pkg.Similarity(9, blocks=[3, 3], strides=[1, 1], padding=[1, 1]).cuda()
    mexl = pkg.Mex(5, blocks=[-1, 1, 1], strides=[9, 1, 1], softmax_mode=True, normalize_offsets=True,
                   unshared_offset_region=[2]).cuda()
    x = torch.randn((2, 4, 8, 8), device="cuda", generator=g)

    def both():
        with torch.no_grad():
            fast = mexl(sim(x))
        slow = mexl(sim(x)).detach()
        assert torch.equal(fast, slow)
        return fast

    y0 = both()
    # rebinding: fresh Parameter objects (version 0, like the ones they replace)
    sim.templates = torch.nn.Parameter(torch.randn(sim.templates.shape, device="cuda", generator=g))
    mexl.offsets = torch.nn.Parameter(torch.randn(mexl.offsets.shape, device="cuda", generator=g))
    y1 = both()
    assert not torch.equal(y1, y0)
    # load_state_dict(assign=True) swaps the tensors as well
    state = {k: torch.randn(v.shape, device="cuda", generator=g) for k, v in sim.state_dict().items()}
    sim.load_state_dict(state, assign=True)
    y2 = both()
    assert not torch.equal(y2, y1)
    # a layer attribute changed after the first call
    sim.out_of_bounds_value = 3.0
    mexl.epsilon = 2.0
    y3 = both()
    assert not torch.equal(y3, y2)
    # .data writes are invisible to the version counter: the documented way is invalidate_prepared()
    sim.sweights.data.mul_(1.5)
    mexl.offsets.data.add_(0.5 * torch.randn(mexl.offsets.shape, device="cuda", generator=g))
    sim.invalidate_prepared()
    mexl.invalidate_prepared()
    y4 = both()
    assert not torch.equal(y4, y3)
    # another stream: its own buffer, the first stream's one kept
    main = sim._prepared.last()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        y5 = mexl(sim(x))
        assert sim._prepared.last() is not main
    side.synchronize()
    assert torch.equal(y5, y4)
    with torch.no_grad():
        mexl(sim(x))
    assert sim._prepared.last(pkg.ops._current_stream(x.device)) is main


@pytest.mark.parametrize("im,n", [((64, 32, 16, 16), 64),      # panel form, one chunk
                                  ((16, 64, 8, 8), 128),       # panel form, two halves
                                  ((40, 16, 8, 8), 20)])       # fused kernel
def test_mex_outputs_that_are_only_4_byte_aligned(pkg, im, n):
    """The kernels store the two pixels of a window row as one 8-byte piece where the output tensor allows it: outputs
    (the MEX output, the pooled output, the unpooled output of the fused call) a float off that alignment, passed
    through the C ABI, hold the same values."""
    import ctypes as C
    from simnets_tf_amd import _lib, ops
    l = _lib.lib()
    kw = dict(softmax_mode=True, blocks=[im[1], 1, 1], strides=[im[1], 1, 1], unshared_offset_region=[1, 2, 2], epsilon=1.5)
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(im, device="cuda", generator=g)
    _, oshape = pkg.mex_output_shape(im, n, **kw)
    off = torch.randn(oshape, device="cuda", generator=g)
    want = pkg.mex(x, off, n, **kw)
    want_full, want_pooled = pkg.mex_sum_pool_both(x, off, n, (2, 2), **kw)
    a = ops.mex_attrs(n, **kw)
    xs = (C.c_int * 4)(*im)
    stream = torch.cuda.current_stream().cuda_stream

    def off_by_one(shape):
        buf = torch.zeros(int(np.prod(shape)) + 1, device="cuda")
        v = buf[1:].view(tuple(shape))
        assert v.data_ptr() % 8 == 4
        return v

    nbytes = C.c_size_t()
    assert l.simnets_hip_mex_workspace_bytes(C.byref(a), xs, C.byref(nbytes)) == 0
    ws = torch.empty(max(nbytes.value, 256), dtype=torch.uint8, device="cuda")
    y = off_by_one(want.shape)
    rc = l.simnets_hip_mex_fwd(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), y.data_ptr(), ws.data_ptr(),
                               ws.numel(), stream)
    assert rc == 0, _lib.strerror(rc)
    assert torch.equal(y, want)
    assert l.simnets_hip_mex_sum_pool_workspace_bytes(C.byref(a), xs, 2, 2, C.byref(nbytes)) == 0
    ws = torch.empty(max(nbytes.value, 256), dtype=torch.uint8, device="cuda")
    full, pooled = off_by_one(want_full.shape), off_by_one(want_pooled.shape)
    rc = l.simnets_hip_mex_sum_pool_fwd_both(C.byref(a), xs, x.data_ptr(), off.data_ptr(), off.numel(), 2, 2,
                                             full.data_ptr(), pooled.data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, _lib.strerror(rc)
    assert torch.equal(full, want_full) and torch.equal(pooled, want_pooled)
