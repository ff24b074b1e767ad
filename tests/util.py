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


def assert_sum(gpu, ref, magnitude, what='', rel=REL):
    """A parameter gradient is a sum of very many terms of both signs: |gpu - ref| <= rel * (sum of the terms'
    magnitudes), per parameter.  ``ref`` is the sum and ``magnitude`` the sum of absolute values, both in float64.
    (Relative to the result itself no summation order, the reference's included, can promise anything once the
    terms cancel.)"""
    g = gpu.detach().cpu().double().reshape(-1)
    r = ref.detach().cpu().double().reshape(-1)
    m = magnitude.detach().cpu().double().reshape(-1)
    assert g.shape == r.shape == m.shape, (what, g.shape, r.shape, m.shape)
    err = (g - r).abs()
    bad = err > rel * m
    if bool(bad.any()):
        i = int(torch.argmax(err / m.clamp_min(1e-300)))
        raise AssertionError(f'{what}: |{g[i].item()!r} - {r[i].item()!r}| = {err[i].item():.3e} > {rel} * '
                             f'{m[i].item():.3e} (parameter {i})')


def li_bwd_f64(grad_out, a):
    """g[t] = a g[t+1] + grad_out[t] on rows [R, T] in float64 (neuron/dynamics/leaky_integrator.py:234-259 in the
    reference, a = 1 - decay / 4096 per row), and next to it the same recurrence on magnitudes,
    B[t] = |a| B[t+1] + |grad_out[t]|: the sum of the magnitudes of the terms a^k grad_out[t+k] that make up g[t].
    A float32 evaluation in any order is off by a few ulp of B[t], not of g[t]: where the terms cancel, the bar for
    an element is rel * B[t] (``assert_sum``), which is rel * |g[t]| wherever they do not."""
    go = grad_out.detach().cpu().double()
    a = a.detach().cpu().double().reshape(-1, 1)
    g, bound = torch.zeros_like(go), torch.zeros_like(go)
    acc = torch.zeros(go.shape[0], 1, dtype=torch.float64)
    mag = torch.zeros_like(acc)
    for t in range(go.shape[1] - 1, -1, -1):
        acc = a * acc + go[:, t:t + 1]
        mag = a.abs() * mag + go[:, t:t + 1].abs()
        g[:, t:t + 1], bound[:, t:t + 1] = acc, mag
    return g, bound


def param_sum_f64(terms, num_params):
    """(sum, sum of magnitudes) in float64 of ``terms`` [N, C, ..., T'] per parameter, addressed as the kernels
    address decays: one shared value, one per channel, or one per neuron of a batch element."""
    t = terms.detach().cpu().double()
    n = t.shape[0]
    if num_params == 1:
        return t.sum().reshape(1), t.abs().sum().reshape(1)
    per_batch = 1
    for d in t.shape[1:-1]:
        per_batch *= d
    r = t.reshape(n, num_params, (per_batch // num_params) * t.shape[-1])
    return r.sum(dim=(0, 2)), r.abs().sum(dim=(0, 2))


def li_decay_grad_f64(grad_in, out, num_decays):
    """Decay gradient of the leaky integrator from its input gradient and saved output
    (neuron/dynamics/leaky_integrator.py:250-257 in the reference): sum of grad_in[t+1] * out[t], with the sum of the
    terms' magnitudes, both in float64, for ``assert_sum``."""
    return param_sum_f64(grad_in.detach().cpu().double()[..., 1:] * out.detach().cpu().double()[..., :-1], num_decays)


def res_decay_grads_f64(g_re_in, g_im_in, re, im, num_decays):
    """(sin sum, sin magnitudes, cos sum, cos magnitudes) of the resonator's decay gradients
    (neuron/dynamics/resonator.py:440-467 in the reference) in float64."""
    gr, gi = g_re_in.detach().cpu().double()[..., 1:], g_im_in.detach().cpu().double()[..., 1:]
    r, i = re.detach().cpu().double()[..., :-1], im.detach().cpu().double()[..., :-1]
    s_sum, _ = param_sum_f64(-gr * i + gi * r, num_decays)
    c_sum, _ = param_sum_f64(gr * r + gi * i, num_decays)
    _, mag = param_sum_f64((gr * i).abs() + (gi * r).abs(), num_decays)
    _, mag_c = param_sum_f64((gr * r).abs() + (gi * i).abs(), num_decays)
    return s_sum, mag, c_sum, mag_c


def assert_same_gradient(a, b, what=''):
    """Two evaluations of the same float gradient on the GPU: bit-identical while both are step-by-step
    (small tensors), within 1e-5 of the scale once the scan kernels take over."""
    if a.numel() < SCAN_MIN:
        assert torch.equal(a, b), what
    else:
        assert_scale(a, b, what)
