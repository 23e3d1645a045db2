"""The standalone C++ bench harness (simnets-tf_amd/simnets_bench, linked against libsimnets_hip.so only) run as a
child process for every benchmark configuration: exit status 0, every printed line one JSON object, and the checksum
it prints for each output tensor equal to the checksum of what the Python op layer computes, through the same C ABI,
from the inputs the harness dumped.  (The harness fills its inputs with its own counter-based generator; they are
read back from its --dump files rather than regenerated, so that libm differences cannot enter.)"""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "simnets-tf_amd", "simnets_bench")


def checksum(t):
    """sum_i (bits(t[i]) + 1) * (2 i + 1) mod 2^64 over the fp32 bit patterns: the harness's formula."""
    bits = t.detach().contiguous().cpu().numpy().reshape(-1).view(np.uint32).astype(np.uint64)
    with np.errstate(over="ignore"):
        acc = ((bits + np.uint64(1)) * (np.uint64(2) * np.arange(bits.size, dtype=np.uint64) + np.uint64(1))).sum(
            dtype=np.uint64)
    return "%016x" % int(acc)


def run_harness(config, tmp_path, *extra):
    assert os.path.exists(BENCH), "simnets_bench is not built (python simnets-tf_amd/build.py)"
    r = subprocess.run([BENCH, "--config", str(config), "--steps", "2", "--warmup", "1", "--dump", str(tmp_path),
                        *extra], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.strip()]      # every line parses
    assert lines and all(isinstance(ln, dict) for ln in lines)
    sums = {ln["checksum"]: (ln["value"], ln["elements"]) for ln in lines if "checksum" in ln}
    timings = [ln for ln in lines if "config" in ln]
    assert timings and all(ln["ms"] > 0 for ln in timings)
    return sums, timings


def load(tmp_path, name, shape):
    a = np.fromfile(os.path.join(str(tmp_path), name + ".bin"), dtype=np.float32)
    return torch.from_numpy(a.reshape(shape)).cuda()


SIM1 = dict(blocks=[2, 2], strides=[2, 2], padding=[2, 2], normalization_term=True, ignore_nan_input=True,
            out_of_bounds_value=float("nan"))
SIM3 = dict(blocks=[3, 3], strides=[1, 1], padding=[1, 1])


def mex_kw(channels, shared1=False):
    kw = dict(softmax_mode=True, blocks=[channels, 1, 1], strides=[channels, 1, 1], normalize_offsets=True)
    kw.update(dict(shared_offset_region=[1]) if shared1 else dict(unshared_offset_region=[2]))
    return kw


def expect(sums, name, tensor):
    assert name in sums, (name, sorted(sums))
    value, n = sums[name]
    assert n == tensor.numel()
    assert value == checksum(tensor), "%s: harness %s, op layer %s" % (name, value, checksum(tensor))


def test_harness_config1(pkg, tmp_path):
    sums, _ = run_harness(1, tmp_path)
    x, t, w = load(tmp_path, "c1_x", (64, 1, 28, 28)), load(tmp_path, "c1_t", (32, 1, 2, 2)), load(tmp_path, "c1_w", (32, 1, 2, 2))
    y = pkg.similarity(x, t, w, **SIM1)
    expect(sums, "config1", y)
    expect(sums, "config1 prepared", pkg.similarity_prepare(x.shape, t, w, **SIM1)(x))


def test_harness_config2(pkg, tmp_path):
    sums, _ = run_harness(2, tmp_path)
    x, off = load(tmp_path, "c2_x", (64, 32, 16, 16)), load(tmp_path, "c2_off", (4, 64, 32, 1, 1))
    expect(sums, "config2", pkg.mex(x, off, 64, **mex_kw(32)))
    expect(sums, "config2 prepared", pkg.mex_prepare(x.shape, off, 64, **mex_kw(32))(x))


def test_harness_config3(pkg, tmp_path):
    sums, timings = run_harness(3, tmp_path)
    assert len(timings) == 4
    x, t, w = load(tmp_path, "c3_x", (256, 64, 32, 32)), load(tmp_path, "c3_t", (128, 64, 3, 3)), load(tmp_path, "c3_w", (128, 64, 3, 3))
    for func in ("L2", "L1"):
        expect(sums, "config3 " + func, pkg.similarity(x, t, w, similarity_function=func, **SIM3))


def test_harness_config4(pkg, tmp_path):
    sums, _ = run_harness(4, tmp_path)
    B = 512
    x, t, w = load(tmp_path, "c4_x", (B, 1, 28, 28)), load(tmp_path, "c4_t", (32, 1, 2, 2)), load(tmp_path, "c4_w", (32, 1, 2, 2))
    offs, ch = [], 32
    for l in range(4):
        offs.append((load(tmp_path, "c4_mex%d_off" % l, (4, 2 * ch, ch, 1, 1)), 2 * ch, mex_kw(ch)))
        ch *= 2
    head = (load(tmp_path, "c4_mex4_off", (1, 10, ch, 1, 1)), 10, mex_kw(ch, shared1=True))

    cur = pkg.similarity(x, t, w, **SIM1)
    for off, n, kw in offs:
        cur = pkg.sum_pooling(pkg.mex(cur, off, n, **kw), (2, 2))
    expect(sums, "config4 separate calls", pkg.mex(cur, head[0], head[1], **head[2]))

    cur = pkg.similarity(x, t, w, **SIM1)
    for off, n, kw in offs:
        cur = pkg.mex_sum_pool(cur, off, n, (2, 2), **kw)
    expect(sums, "config4 fused pooling", pkg.mex(cur, head[0], head[1], **head[2]))

    cur = pkg.similarity_mex_sum_pool(x, t, w, offs[0][0], offs[0][1], (2, 2), similarity=SIM1, mex=offs[0][2])
    for off, n, kw in offs[1:]:
        cur = pkg.mex_sum_pool(cur, off, n, (2, 2), **kw)
    final = pkg.mex(cur, head[0], head[1], **head[2])
    expect(sums, "config4 fused similarity and pooling", final)
    expect(sums, "config4 fused prepared", final)      # the prepared calls run the same kernels on the same packing
    expect(sums, "config4 fused prepared graph", final)   # ... and so does their replay from a HIP graph


def test_harness_config5(pkg, tmp_path):
    sums, timings = run_harness(5, tmp_path)
    assert len(timings) == 6
    x, t, w = load(tmp_path, "c5_x", (256, 64, 32, 32)), load(tmp_path, "c5_t", (128, 64, 3, 3)), load(tmp_path, "c5_w", (128, 64, 3, 3))
    g = load(tmp_path, "c5_g", (256, 128, 32, 32))
    for func in ("L2", "L1"):
        kw = dict(SIM3, similarity_function=func)
        expect(sums, "config5 %s input grad" % func, pkg.similarity_input_grad(x, t, w, g, **kw))
        dt, dw = pkg.similarity_parameters_grad(x, t, w, g, **kw)
        expect(sums, "config5 %s templates grad" % func, dt)
        expect(sums, "config5 %s weights grad" % func, dw)
    del x, g
    xm, off = load(tmp_path, "c5_mex_x", (64, 32, 16, 16)), load(tmp_path, "c5_mex_off", (4, 64, 32, 1, 1))
    gm = load(tmp_path, "c5_mex_g", (64, 64, 16, 16))
    y = pkg.mex(xm, off, 64, **mex_kw(32))
    expect(sums, "config5 mex input grad", pkg.mex_input_grad(xm, off, y, gm, 64, **mex_kw(32)))
    expect(sums, "config5 mex offsets grad", pkg.mex_offsets_grad(xm, off, y, gm, 64, **mex_kw(32)))


def test_harness_machine_probes_run(tmp_path):
    """--peaks: the machine micro-benchmarks and the hand-written co-issue probe kernels run to completion and every
    line parses (their figures are quoted in the kernel notes; nothing else exercises those kernels)."""
    r = subprocess.run([BENCH, "--peaks"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.strip()]
    assert sum("peak" in ln for ln in lines) == 4 and sum("probe" in ln for ln in lines) == 7
