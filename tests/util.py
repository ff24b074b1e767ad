"""Shared helpers for the GPU parity tests."""
import numpy as np
import torch

REL = 1e-5   # float-mode tolerance of the hot path: relative error <= 1e-5


def seed_of(*key):
    """Deterministic seed from a test's parameters (python's hash() is salted per process)."""
    import zlib
    return zlib.crc32(repr(key).encode()) & 0x7fffffff


def dev():
    return torch.device('cuda:0')


def sparse_input(gen, shape, p=0.05, amp=1.0):
    """Bernoulli(p) events times Normal(0, amp) weights (the workload family of the benchmark)."""
    return (torch.rand(shape, generator=gen) < p).float() * torch.randn(shape, generator=gen) * amp


def assert_exact(gpu, ref, what=''):
    g = gpu.detach().cpu()
    assert g.shape == ref.shape, (what, g.shape, ref.shape)
    if not torch.equal(g, ref):
        bad = (g != ref)
        idx = bad.nonzero()[0].tolist()
        raise AssertionError(f'{what}: {int(bad.sum())} of {bad.numel()} elements differ; '
                             f'first at {idx}: gpu={g[tuple(idx)].item()!r} ref={ref[tuple(idx)].item()!r}')


def assert_rel(gpu, ref, what='', rel=REL):
    """max |gpu - ref| <= rel * max |ref| and elementwise |gpu - ref| <= rel * (|ref| + max|ref| * 1e-2)."""
    g = gpu.detach().cpu().double()
    r = ref.detach().double()
    assert g.shape == r.shape, (what, g.shape, r.shape)
    scale = float(r.abs().max()) if r.numel() else 0.0
    err = (g - r).abs()
    if r.numel() and float(err.max()) > rel * scale:
        raise AssertionError(f'{what}: max abs err {float(err.max()):.3e} > {rel} * {scale:.3e}')
    tol = rel * (r.abs() + 1e-2 * scale)
    if r.numel() and bool((err > tol).any()):
        i = int(torch.argmax(err - tol))
        raise AssertionError(f'{what}: elementwise tolerance exceeded at flat index {i}: '
                             f'gpu={g.flatten()[i].item()!r} ref={r.flatten()[i].item()!r}')


SCAN_MIN = 1 << 20   # float backward recurrences run as wave scans from this many elements on (csrc/scan.hip)


def assert_scale(gpu, ref, what='', rel=REL):
    """max |gpu - ref| <= rel * max |ref|: the bar for float gradients that went through a scan (its rounding
    differs from a step-by-step evaluation by a few ulp of the largest terms, not of each result)."""
    g = gpu.detach().cpu().double()
    r = ref.detach().cpu().double()
    assert g.shape == r.shape, (what, g.shape, r.shape)
    if r.numel() == 0:
        return
    scale = float(r.abs().max())
    err = float((g - r).abs().max())
    if err > rel * scale:
        raise AssertionError(f'{what}: max abs err {err:.3e} > {rel} * {scale:.3e}')


def assert_same_gradient(a, b, what=''):
    """Two evaluations of the same float gradient on the GPU: bit-identical while both are step-by-step
    (small tensors), within 1e-5 of the scale once the scan kernels take over."""
    if a.numel() < SCAN_MIN:
        assert torch.equal(a, b), what
    else:
        assert_scale(a, b, what)
