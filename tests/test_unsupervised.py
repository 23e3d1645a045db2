"""Unsupervised initialisers (simnets-tf_amd/unsupervised.py): plain torch code, checked on the CPU against
numpy / scikit-learn on data whose answer is known.  The reference delegates the clustering itself to
tf.contrib (absent here), so agreement with it bit for bit is not claimed: parity unpinned for the
clustering trajectories; what the reference defines itself (patch layout, which statistic becomes which
parameter) is what these tests pin."""
import numpy as np
import pytest
import torch
from sklearn.cluster import KMeans

from conftest import load_package

pkg = load_package()
uns = pkg.unsupervised


def test_patch_layout_is_the_template_layout():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 7, 8, generator=g)
    p = uns.extract_patches(x, (3, 2), (2, 1))
    oh, ow = (7 - 3) // 2 + 1, (8 - 2) // 1 + 1
    assert p.shape == (2 * oh * ow, 3 * 3 * 2)
    b, yo, xo = 1, 1, 4
    want = x[b, :, yo * 2:yo * 2 + 3, xo:xo + 2].reshape(-1)
    assert torch.equal(p[(b * oh + yo) * ow + xo], want)


def _blob_images(n_img, protos, noise, seed):
    """Images tiled with 2x2 prototypes (+ noise): every non-overlapping 2x2 patch is a noisy prototype."""
    g = np.random.default_rng(seed)
    k, c = protos.shape[0], protos.shape[1]
    lab = g.integers(0, k, size=(n_img, 4, 4))
    img = np.zeros((n_img, c, 8, 8), np.float32)
    for i in range(4):
        for j in range(4):
            img[:, :, 2 * i:2 * i + 2, 2 * j:2 * j + 2] = protos[lab[:, i, j]]
    return torch.from_numpy(img + noise * g.normal(size=img.shape).astype(np.float32))


def _match(got, want):
    """rows of `got` reordered to best match the rows of `want`"""
    d = ((got[:, None] - want[None]) ** 2).sum(-1)
    return got[d.argmin(0)]


def test_kmeans_init_recovers_prototypes_and_sets_unit_weights():
    protos = np.random.default_rng(1).normal(size=(4, 2, 2, 2)).astype(np.float32) * 3
    data = _blob_images(64, protos, 0.05, 2)
    layer = pkg.Similarity(4, blocks=[2, 2], strides=[2, 2], padding=[0, 0])
    uns.similarity_unsupervised_init("kmeans", layer, data, batch_size=16, generator=torch.Generator().manual_seed(3))
    got = layer.templates.detach().numpy().reshape(4, -1)
    want = protos.reshape(4, -1)
    np.testing.assert_allclose(_match(got, want), want, atol=0.05)
    assert torch.equal(layer.sweights.detach(), torch.ones_like(layer.sweights))
    # the same clusters scikit-learn finds on the same patches
    patches = uns.extract_patches(data, (2, 2), (2, 2)).numpy()
    sk = KMeans(4, n_init=4, random_state=0).fit(patches).cluster_centers_
    np.testing.assert_allclose(_match(got, sk), sk, atol=0.05)


def test_gmm_em_recovers_means_and_standard_deviations():
    protos = np.random.default_rng(4).normal(size=(3, 1, 2, 2)).astype(np.float32) * 4
    data = _blob_images(200, protos, 0.3, 5)
    patches = uns.extract_patches(data, (2, 2), (2, 2))
    gmm = uns.DiagonalGMM(3)
    # EM converges to a local optimum that depends on the seeding; seeded with one sample near each blob it
    # must find the blobs
    d = ((patches[:, None] - torch.from_numpy(protos.reshape(3, -1))[None]) ** 2).sum(-1)
    gmm.means = patches[d.argmin(0)].clone()
    gmm.covs = patches.var(dim=0, unbiased=False).repeat(3, 1)
    for _ in range(10):
        gmm.partial_fit(patches)
    np.testing.assert_allclose(_match(gmm.means.numpy(), protos.reshape(3, -1)), protos.reshape(3, -1), atol=0.05)
    np.testing.assert_allclose(gmm.covs.sqrt().numpy(), 0.3, atol=0.03)


def test_gmm_init_assigns_means_and_root_covariances():
    protos = np.random.default_rng(4).normal(size=(3, 1, 2, 2)).astype(np.float32) * 4
    data = _blob_images(50, protos, 0.3, 5)
    layer = pkg.Similarity(3, blocks=[2, 2], strides=[2, 2], padding=[0, 0])
    model = uns.similarity_unsupervised_init("gmm", layer, data, batch_size=10,
                                             generator=torch.Generator().manual_seed(1))
    assert torch.equal(layer.templates.detach(), model.means.reshape(3, 1, 2, 2))
    assert torch.equal(layer.sweights.detach(), model.covs.sqrt().reshape(3, 1, 2, 2))
    assert (model.covs > 0).all()


def test_pca_init_matches_the_eigenvectors_of_the_patch_covariance():
    g = torch.Generator().manual_seed(6)
    mix = torch.randn(12, 12, generator=g)
    data = (torch.randn(40, 12, 5 * 5, generator=g).transpose(1, 2) @ mix).transpose(1, 2).reshape(40, 12, 5, 5)
    data = data[:, :3] + 2.0        # 3 channels, non-zero mean
    conv = torch.nn.Conv2d(3, 5, kernel_size=2, stride=1, bias=False)
    uns.pca_unsupervised_init(conv, data, batch_size=8)
    patches = uns.extract_patches(data, (2, 2), (1, 1)).double().numpy()
    cov = np.cov(patches.T, bias=True)
    w, v = np.linalg.eigh(cov)
    top = v[:, np.argsort(w)[::-1][:5]].T
    got = conv.weight.detach().double().numpy().reshape(5, -1)
    for a, b in zip(got, top):
        assert min(np.abs(a - b).max(), np.abs(a + b).max()) < 1e-4


def test_nan_patches_are_skipped_and_bad_kind_is_rejected():
    data = _blob_images(8, np.ones((2, 1, 2, 2), np.float32), 0.1, 7)
    data[0, 0, 0, 0] = float("nan")
    layer = pkg.Similarity(2, blocks=[2, 2], strides=[2, 2], padding=[0, 0])
    uns.similarity_unsupervised_init("kmeans", layer, data, batch_size=8, generator=torch.Generator().manual_seed(0))
    assert torch.isfinite(layer.templates).all()
    with pytest.raises(ValueError):
        uns.similarity_unsupervised_init("svm", layer, data, batch_size=8)


# ---- single steps against what the mathematics fixes ------------------------------------------------------------
def test_one_kmeans_step_from_a_fixed_start_is_assignment_plus_mean():
    """With zero counts, one mini-batch step moves every centre that received points to the plain mean of its points
    (brute-force nearest-centre assignment in float64) and leaves the others alone: one Lloyd step."""
    g = np.random.default_rng(21)
    pts = g.normal(size=(300, 6)).astype(np.float32)
    start = np.concatenate([pts[[3, 50, 120, 200]], np.full((1, 6), 40.0, np.float32)])   # the last centre gets nothing
    km = uns.MiniBatchKMeans(5)
    km.centers = torch.from_numpy(start.copy())
    km.counts = torch.zeros(5)
    km.partial_fit(torch.from_numpy(pts))
    d = ((pts[:, None].astype(np.float64) - start[None].astype(np.float64)) ** 2).sum(-1)
    assign = d.argmin(1)
    assert set(assign) == {0, 1, 2, 3}
    for c in range(4):
        np.testing.assert_allclose(km.centers[c].numpy(), pts[assign == c].astype(np.float64).mean(0), rtol=0, atol=1e-5)
    assert np.array_equal(km.centers[4].numpy(), start[4])
    assert np.array_equal(km.counts.numpy(), np.bincount(assign, minlength=5).astype(np.float32))
    # a second batch: the centre is the mean of everything it has been given (the 1/count step rule, summed)
    more = g.normal(size=(100, 6)).astype(np.float32) + km.centers[0].numpy()
    before, n0 = km.centers.clone().double().numpy(), km.counts.clone().numpy()
    km.partial_fit(torch.from_numpy(more))
    d2 = ((more[:, None].astype(np.float64) - before[None]) ** 2).sum(-1).argmin(1)
    for c in range(5):
        sel = more[d2 == c].astype(np.float64)
        want = before[c] if len(sel) == 0 else (before[c] * n0[c] + sel.sum(0)) / (n0[c] + len(sel))
        np.testing.assert_allclose(km.centers[c].numpy(), want, rtol=0, atol=1e-5)


def _diag_gmm_loglik(pts, means, covs):
    """Mean log-likelihood of a uniform mixture of diagonal Gaussians, float64, straight from the definition."""
    pts, means, covs = (np.asarray(a, dtype=np.float64) for a in (pts, means, covs))
    diff = pts[:, None, :] - means[None]
    logp = -0.5 * ((diff ** 2) / covs[None] + np.log(2 * np.pi * covs)[None]).sum(-1) - np.log(len(means))
    m = logp.max(1, keepdims=True)
    return float((m[:, 0] + np.log(np.exp(logp - m).sum(1))).mean())


def test_em_steps_never_decrease_the_likelihood_and_follow_the_textbook_update():
    g = np.random.default_rng(22)
    centres = g.normal(size=(3, 5)) * 3
    pts = np.concatenate([c + g.normal(size=(150, 5)) * s for c, s in zip(centres, (0.5, 1.0, 1.5))]).astype(np.float32)
    gmm = uns.DiagonalGMM(3, generator=torch.Generator().manual_seed(2), min_var=1e-6)
    T = torch.from_numpy(pts)
    gmm.partial_fit(T)                       # seeds, then one step
    ll = [_diag_gmm_loglik(pts, gmm.means, gmm.covs)]
    for _ in range(8):
        means0, covs0 = gmm.means.double().numpy(), gmm.covs.double().numpy()
        gmm.partial_fit(T)
        ll.append(_diag_gmm_loglik(pts, gmm.means, gmm.covs))
        # the textbook EM update from (means0, covs0), in float64: responsibilities sum to 1 per point
        diff = pts[:, None, :].astype(np.float64) - means0[None]
        logp = -0.5 * ((diff ** 2) / covs0[None] + np.log(covs0)[None]).sum(-1)
        resp = np.exp(logp - logp.max(1, keepdims=True))
        resp /= resp.sum(1, keepdims=True)
        np.testing.assert_allclose(resp.sum(1), 1.0, atol=1e-12)
        mass = resp.sum(0)
        means1 = resp.T @ pts.astype(np.float64) / mass[:, None]
        covs1 = (resp[:, :, None] * (pts[:, None, :] - means1[None]) ** 2).sum(0) / mass[:, None]
        np.testing.assert_allclose(gmm.means.numpy(), means1, rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(gmm.covs.numpy(), np.maximum(covs1, 1e-6), rtol=2e-3, atol=2e-4)
    assert all(b >= a - 1e-6 for a, b in zip(ll, ll[1:])), ll


def test_pca_components_are_the_eigenvectors_torch_eigh_finds():
    g = torch.Generator().manual_seed(23)
    data = torch.randn(30, 2, 6, 6, generator=g) * torch.tensor([1.0, 3.0]).view(1, 2, 1, 1) + 0.7
    pca = uns.RunningPCA()
    for i in range(0, 30, 7):                                   # ragged batches: the running moments must not care
        pca.partial_fit(uns.extract_patches(data[i:i + 7], (2, 3), (1, 2)))
    patches = uns.extract_patches(data, (2, 3), (1, 2)).double()
    mu = patches.mean(0)
    cov = (patches - mu).t() @ (patches - mu) / patches.shape[0]
    w, v = torch.linalg.eigh(cov)
    order = torch.argsort(w, descending=True)
    comps = pca.components(4)
    for a, b in zip(comps, v[:, order[:4]].t()):
        assert min(float((a - b).abs().max()), float((a + b).abs().max())) < 1e-8
