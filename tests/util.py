"""Helpers shared by the parity tests: seeded inputs and the error metric."""
import numpy as np


def rel_err(got, want, floor=None):
    """max |got - want| / max(|want|, floor, 1e-6 * max|want|) over finite entries of `want`.

    Outputs may cross zero, so the denominator has an absolute floor tied to the tensor's scale.
    `floor` (array like `want`, optional) raises it per element: MEX passes |m|, the shift
    m = max_k(patch_k + offset_k) that every implementation subtracts before exponentiating.
    The MEX output is m + log(sum exp(eps (v - m))) / eps, so its rounding noise is proportional
    to |m| even where the two terms cancel and the output itself is near zero.
    NaN / Inf positions must coincide and are excluded from the ratio.
    """
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.array_equal(np.isnan(got), np.isnan(want)), "NaN positions differ"
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]), "Inf entries differ"
    fin = np.isfinite(want)
    if not fin.any():
        return 0.0
    scale = np.abs(want[fin]).max()
    den = np.maximum(np.abs(want[fin]), 1e-6 * scale)
    if floor is not None:
        den = np.maximum(den, np.abs(np.asarray(floor, dtype=np.float64))[fin])
    den = np.maximum(den, np.finfo(np.float64).tiny)
    return float((np.abs(got[fin] - want[fin]) / den).max())


def config1(batch=64, seed=1234, nan_frac=0.0):
    g = np.random.default_rng(seed)
    x = g.uniform(-0.5, 0.5, size=(batch, 1, 28, 28)).astype(np.float32)
    if nan_frac > 0:
        x[np.random.default_rng(5678).random(size=x.shape) < nan_frac] = np.nan
    t = (np.random.default_rng(2345).normal(size=(32, 1, 2, 2)) * 0.1).astype(np.float32)
    w = np.random.default_rng(3456).uniform(0.5, 1.5, size=t.shape).astype(np.float32)
    kw = dict(similarity_function="L2", blocks=[2, 2], strides=[2, 2], padding=[2, 2], normalization_term=True,
              ignore_nan_input=True, out_of_bounds_value=float("nan"))
    return x, t, w, kw


def config2(batch=64, channels=32, size=16, instances=64, seed=1234):
    x = np.random.default_rng(seed).normal(size=(batch, channels, size, size)).astype(np.float32)
    r = min(2, size) ** 2
    off = (np.random.default_rng(4567).normal(size=(r, instances, channels, 1, 1)) * 0.1).astype(np.float32)
    kw = dict(softmax_mode=True, blocks=[channels, 1, 1], strides=[channels, 1, 1], padding=[0, 0, 0], epsilon=1.0,
              use_unshared_regions=True, unshared_offset_region=[2])
    return x, off, instances, kw


def config3(batch=256, seed=1234, channels=64, size=32, templates=128):
    x = np.random.default_rng(seed).normal(size=(batch, channels, size, size)).astype(np.float32)
    t = np.random.default_rng(2345).normal(size=(templates, channels, 3, 3)).astype(np.float32)
    w = np.random.default_rng(3456).uniform(0.1, 2.0, size=t.shape).astype(np.float32)
    kw = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])
    return x, t, w, kw


def config4_stack(batch=512):
    """The missing-data network (examples/mnist_ght_model_missing_data.py:81-112 of the reference): Similarity on
    1x28x28 images with 25 % NaN pixels, four MEX layers (64, 128, 256, 512 instances over all channels of a pixel,
    offsets unshared over 2x2) each followed by 2x2 sum pooling, and a MEX layer to 10 classes.
    Returns (x, templates, weights, similarity kwargs, [(offsets, num_instances, mex kwargs)] x 4, (offsets, 10, kwargs))."""
    x, t, w, skw = config1(batch=batch, nan_frac=0.25)
    g = np.random.default_rng(4567)
    layers, ch, size = [], 32, 16
    for _ in range(4):
        n = ch * 2
        off = (g.normal(size=(4 if size > 1 else 1, n, ch, 1, 1)) * 0.1).astype(np.float32)
        layers.append((off, n, dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1],
                                    unshared_offset_region=[2])))
        ch, size = n, size // 2
    offl = (g.normal(size=(1, 10, ch, 1, 1)) * 0.1).astype(np.float32)
    last = (offl, 10, dict(softmax_mode=True, blocks=[ch, 1, 1], strides=[ch, 1, 1], shared_offset_region=[1]))
    return x, t, w, skw, layers, last
