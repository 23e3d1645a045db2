"""Unsupervised initialisation of Similarity layers (k-means, diagonal GMM) and of convolutions (PCA):
the torch counterpart of python/simnets/unsupervised/ and of `perform_unsupervised_init`
(python/simnets/keras.py:199-243).

What the reference defines itself is kept: which patches are used (the layer's blocks and strides, VALID
padding whatever the layer's own padding is: unsupervised/kmeans.py:38-45), how clusters become parameters
(templates = cluster centres; weights = ones for k-means, kmeans.py:50-57; weights = sqrt of the diagonal
covariances for GMM, gmm.py:63-70; PCA filters = leading right singular vectors of the patch covariance,
pca.py:83-91) and the batch-wise driver.  The clustering algorithms themselves live in TensorFlow's contrib
package (`tf.contrib.factorization.KMeans` with use_mini_batch=True and kmeans++ seeding; `gmm` with
covariance_type='diag', params='mc', random seeding), which is not part of the reference checkout: they are
restated here from their published descriptions (mini-batch k-means with per-centre counts; EM for a diagonal
Gaussian mixture with fixed uniform mixing weights), so results agree in distribution, not bit for bit.
Plain torch code: runs on whatever device the data lives on.
"""
import torch
import torch.nn.functional as F


def extract_patches(x, blocks, strides):
    """[B,C,H,W] -> [B*oh*ow, C*bh*bw] (element order c, dh, dw: the layout of a template), VALID padding."""
    cols = F.unfold(x, kernel_size=tuple(blocks), stride=tuple(strides))
    return cols.transpose(1, 2).reshape(-1, cols.shape[1])


def _drop_nan_rows(p):
    return p[~torch.isnan(p).any(dim=1)]


class MiniBatchKMeans:
    """Mini-batch k-means: kmeans++ seeding on the first batch, then per batch every point moves its nearest
    centre by 1/count of that centre."""

    def __init__(self, num_clusters, generator=None):
        self.k = num_clusters
        self.centers = None
        self.counts = None
        self.generator = generator

    def _seed(self, pts):
        n = pts.shape[0]
        idx = torch.randint(n, (1,), generator=self.generator, device="cpu").item()
        centers = [pts[idx]]
        d2 = ((pts - centers[0]) ** 2).sum(1)
        for _ in range(1, self.k):
            prob = d2 / d2.sum() if float(d2.sum()) > 0 else torch.full_like(d2, 1.0 / n)
            idx = torch.multinomial(prob.cpu(), 1, generator=self.generator).item()
            centers.append(pts[idx])
            d2 = torch.minimum(d2, ((pts - centers[-1]) ** 2).sum(1))
        self.centers = torch.stack(centers).clone()
        self.counts = torch.zeros(self.k, device=pts.device, dtype=pts.dtype)

    def partial_fit(self, pts):
        pts = _drop_nan_rows(pts)
        if pts.shape[0] == 0:
            return self
        if self.centers is None:
            self._seed(pts)
        assign = torch.cdist(pts, self.centers).argmin(dim=1)
        ones = torch.ones(pts.shape[0], device=pts.device, dtype=pts.dtype)
        batch_counts = torch.zeros_like(self.counts).index_add_(0, assign, ones)
        sums = torch.zeros_like(self.centers).index_add_(0, assign, pts)
        self.counts += batch_counts
        hit = batch_counts > 0
        # equivalent to applying the per-point update c += (x - c)/count in one step for the batch
        self.centers[hit] += (sums[hit] - batch_counts[hit, None] * self.centers[hit]) / self.counts[hit, None]
        return self


class DiagonalGMM:
    """EM for a mixture of diagonal Gaussians with fixed uniform mixing weights (only means and covariances are
    learned); one EM step per batch."""

    def __init__(self, num_clusters, generator=None, min_var=1e-3):
        self.k = num_clusters
        self.means = None
        self.covs = None
        self.generator = generator
        self.min_var = min_var

    def partial_fit(self, pts):
        pts = _drop_nan_rows(pts)
        if pts.shape[0] == 0:
            return self
        if self.means is None:
            idx = torch.randperm(pts.shape[0], generator=self.generator)[:self.k].to(pts.device)
            if idx.numel() < self.k:
                idx = torch.randint(pts.shape[0], (self.k,), generator=self.generator).to(pts.device)
            self.means = pts[idx].clone()
            self.covs = pts.var(dim=0, unbiased=False).clamp_min(self.min_var).repeat(self.k, 1)
        # E step: responsibilities under uniform mixing weights
        diff = pts[:, None, :] - self.means[None]
        logp = -0.5 * ((diff * diff) / self.covs[None] + torch.log(self.covs)[None]).sum(-1)
        resp = torch.softmax(logp, dim=1)
        # M step
        mass = resp.sum(0).clamp_min(1e-12)
        self.means = (resp.t() @ pts) / mass[:, None]
        diff = pts[:, None, :] - self.means[None]
        self.covs = ((resp[:, :, None] * diff * diff).sum(0) / mass[:, None]).clamp_min(self.min_var)
        return self


class RunningPCA:
    """Running mean of the patches and of their outer products; filters = leading singular vectors of
    E[p p^T] - E[p] E[p]^T (pca.py:70-91)."""

    def __init__(self):
        self.n = 0
        self.mu = None
        self.second = None

    def partial_fit(self, pts):
        pts = _drop_nan_rows(pts).double()
        if pts.shape[0] == 0:
            return self
        n = pts.shape[0]
        mu, second = pts.mean(0), pts.t() @ pts / n
        if self.n == 0:
            self.mu, self.second = mu, second
        else:
            total = self.n + n
            self.mu += (mu - self.mu) * (n / total)
            self.second += (second - self.second) * (n / total)
        self.n += n
        return self

    def components(self, k):
        cov = self.second - torch.outer(self.mu, self.mu)
        _, _, vh = torch.linalg.svd(cov)
        return vh[:k]   # rows = components


def _batches(data, batch_size):
    if isinstance(data, torch.Tensor):
        if batch_size is None:
            raise ValueError("data is a tensor, so batch size must be given")
        return (data[i:i + batch_size] for i in range(0, data.shape[0], batch_size))
    return iter(data() if callable(data) else data)


def similarity_unsupervised_init(kind, layer, data, batch_size=None, generator=None):
    """Initialise `layer` (a layers.Similarity) from batches of ITS INPUT: templates <- cluster centres;
    weights <- ones (kmeans) or sqrt of the diagonal covariances (gmm).  Returns the fitted model."""
    if kind not in ("kmeans", "gmm"):
        raise ValueError('kind must be one of "kmeans" or "gmm"')
    model = (MiniBatchKMeans if kind == "kmeans" else DiagonalGMM)(layer.num_instances, generator=generator)
    first = None
    for batch in _batches(data, batch_size):
        if layer.channels_last:
            batch = batch.permute(0, 3, 1, 2)
        first = batch if first is None else first
        model.partial_fit(extract_patches(batch.float(), layer.blocks, layer.strides))
    if first is None:
        raise ValueError("no data")
    if isinstance(layer.templates, torch.nn.UninitializedParameter):
        layer.build(first.shape if not layer.channels_last else first.permute(0, 2, 3, 1).shape)
        layer.to(first.device)
    shape = layer.templates.shape
    with torch.no_grad():
        if kind == "kmeans":
            layer.templates.copy_(model.centers.reshape(shape))
            layer.sweights.fill_(1.0)
        else:
            layer.templates.copy_(model.means.reshape(shape))
            layer.sweights.copy_(model.covs.sqrt().reshape(shape))
    return model


def pca_unsupervised_init(conv, data, batch_size=None):
    """Initialise a torch.nn.Conv2d's filters with the leading principal directions of its input patches."""
    pca = RunningPCA()
    for batch in _batches(data, batch_size):
        pca.partial_fit(extract_patches(batch.float(), conv.kernel_size, conv.stride))
    comps = pca.components(conv.out_channels)
    with torch.no_grad():
        conv.weight.copy_(comps.reshape(conv.weight.shape).to(conv.weight.dtype))
    return pca


def perform_unsupervised_init(model, kind="gmm", layers=(), data=None, batch_size=None):
    """Layer by layer like python/simnets/keras.py:199-243: every Similarity (k-means / GMM) or Conv2d (PCA) layer
    of a torch.nn.Sequential is initialised from the activations the already initialised layers before it produce
    for `data` (a tensor + batch_size, an iterable of batches, or a callable returning one)."""
    from .layers import Similarity
    mods = list(model.children())
    targets = list(layers) or [m for m in mods if isinstance(m, (Similarity, torch.nn.Conv2d))]
    for layer in targets:
        pos = next(i for i, m in enumerate(mods) if m is layer)
        prefix = torch.nn.Sequential(*mods[:pos])

        def inputs(prefix=prefix):
            for batch in _batches(data, batch_size):
                with torch.no_grad():
                    yield prefix(batch)

        if isinstance(layer, Similarity):
            similarity_unsupervised_init(kind, layer, inputs)
        else:
            pca_unsupervised_init(layer, inputs)
    return model
