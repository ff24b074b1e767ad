"""GPU parity of the spike functions, time shift and temporal filter against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import seed_of, dev, sparse_input, assert_exact, assert_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


SHAPES = [(4, 128, 200), (2, 3, 5, 7, 37), (3, 70, 129), (1, 5, 3), (2, 64, 1)]


@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('graded', [False, True])
@pytest.mark.parametrize('tensor_th', [False, True])
def test_spike_fwd_bwd(slayer, shape, graded, tensor_th):
    gen = torch.Generator().manual_seed(seed_of(shape, graded, tensor_th))
    v = torch.randn(shape, generator=gen) * 2
    v[..., 0] = 0.7                                            # exact hits of the scalar threshold
    th = (torch.randn(shape, generator=gen) if tensor_th else 0.7)
    g = torch.randn(shape, generator=gen)
    tau, rho, scale = 1.3, 0.9, 4
    vg = v.to(dev()).requires_grad_()
    thg = th.to(dev()) if tensor_th else th
    s = slayer.spike.Spike.apply(vg, thg, tau, rho, graded, 0, scale)
    assert_exact(s, O.spike_fwd(v, th, graded, scale), f'spike fwd {shape}')
    s.backward(g.to(dev()))
    assert_rel(vg.grad, O.spike_bwd(g, v, th, tau, rho, graded), f'spike bwd {shape}')


@pytest.mark.parametrize('shape', SHAPES)
@pytest.mark.parametrize('graded', [False, True])
def test_cspike_fwd_bwd(slayer, shape, graded):
    gen = torch.Generator().manual_seed(seed_of(shape, graded, 'c'))
    re = torch.randn(shape, generator=gen) * 2
    im = torch.randn(shape, generator=gen) * 2
    im[..., -1] = 0.0                                          # imag == 0 counts as "not negative"
    g = torch.randn(shape, generator=gen)
    last = torch.randn(shape[:-1], generator=gen)
    th, tau, rho, scale = 0.4, 0.5, 10.0, 8
    rg, ig = re.to(dev()).requires_grad_(), im.to(dev()).requires_grad_()
    s = slayer.spike.complex.Spike.apply(rg, ig, th, tau, rho, graded, last.to(dev()), scale)
    assert_exact(s, O.cspike_fwd(re, im, th, last, graded, scale), f'cspike fwd {shape}')
    s.backward(g.to(dev()))
    ref_re, ref_im = O.cspike_bwd(g, re, im, th, tau, rho, graded)
    assert_rel(rg.grad, ref_re, f'cspike bwd real {shape}')
    assert_rel(ig.grad, ref_im, f'cspike bwd imag {shape}')
    # scalar imag_last
    s0 = slayer.spike.complex.Spike.apply(rg, ig, th, tau, rho, graded, -1.0, scale)
    assert_exact(s0, O.cspike_fwd(re, im, th, -1.0, graded, scale), 'cspike scalar last')


def test_shift_scalar_and_lut(slayer):
    """The reference's own check (tests/.../utils/time/test_shift.py): +-10 scalar and a per-channel
    ramp against plain slicing, here on [10, 200, 1000] plus odd shapes."""
    gen = torch.Generator().manual_seed(50)
    x = torch.rand((10, 200, 1000), generator=gen)
    xg = x.to(dev())
    for k in (10, -10, 0, 4, -8, 999, 1000, -1500, 2.7, -2.7):
        assert_exact(slayer.utils.time.shift(xg, k), O.shift(x, k), f'shift scalar {k}')
    assert_exact(slayer.utils.time.shift(xg, torch.tensor(7.0)), O.shift(x, 7), 'shift one-element tensor')
    assert_exact(slayer.utils.time.shift(xg, 6, 2), O.shift(x, 3), 'shift sampling time')
    lut = torch.arange(200, dtype=torch.float32) - 100
    assert_exact(slayer.utils.time.shift(xg, lut.to(dev())), O.shift(x, lut), 'shift per-channel ramp')
    lut = torch.rand(200, generator=gen) * 64 - 32          # fractional values are truncated toward zero
    assert_exact(slayer.utils.time.shift(xg, lut.to(dev())), O.shift(x, lut), 'shift fractional lut')
    for shape in [(2, 3, 5, 7, 37), (3, 70, 129), (1, 5, 3), (2, 64, 1)]:
        x = torch.rand(shape, generator=gen)
        lut = torch.randint(-5, 6, shape[1:-1], generator=gen).float()
        assert_exact(slayer.utils.time.shift(x.to(dev()), lut.to(dev())), O.shift(x, lut), f'shift lut {shape}')
        assert_exact(slayer.utils.time.shift(x.to(dev()), 2), O.shift(x, 2), f'shift scalar {shape}')
    with pytest.raises(Exception):
        slayer.utils.time.shift(xg, torch.zeros(7, device=dev()))
    with pytest.raises(AssertionError):
        slayer.utils.time.shift(torch.zeros(5, device=dev()), 1)


@pytest.mark.parametrize('shape,K', [((200, 1000), 50), ((4, 32, 300), 64), ((2, 3, 5, 37), 7), ((3, 1500), 1),
                                     ((2, 5, 20), 64), ((1000,), 50)])
def test_conv_corr(slayer, shape, K):
    """The reference's own check (tests/.../utils/filter/test_conv_filter.py) uses [200, 1000], K=50."""
    gen = torch.Generator().manual_seed(seed_of(shape, K))
    x = torch.rand(shape, generator=gen)
    f = torch.rand(K, generator=gen)
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    for ts in (1, 0.5):
        assert_rel(slayer.utils.filter.conv(x.to(dev()), f.to(dev()), ts), O.conv_fwd(x2, f, ts), f'conv {shape}')
        assert_rel(slayer.utils.filter.corr(x.to(dev()), f.to(dev()), ts), O.conv_bwd(x2, f, ts), f'corr {shape}')
    # float64 numpy.convolve on one row
    row = x2.reshape(-1, x2.shape[-1])[0].double().numpy()
    y = slayer.utils.filter.conv(x.to(dev()), f.to(dev())).reshape(-1, x2.shape[-1])[0].cpu().double().numpy()
    assert np.allclose(y, np.convolve(row, f.double().numpy())[:row.size], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('shape,K', [((6, 300), 5000), ((3, 40), 4097), ((2, 3, 9000), 6000), ((4, 100), 100000),
                                     ((2, 5000), 12288), ((5, 129), 129), ((3, 12), 13)])
def test_filters_longer_than_the_rows_or_than_4096_taps(slayer, shape, K):
    """The reference takes filters of any length (utils/filter/conv.cu:42-46 skips the taps that meet no sample one
    by one).  Only the first min(K, T) taps can meet a sample: results equal those of the truncated filter bit for
    bit and scipy.signal.lfilter with the whole filter in float64; a non-finite tap beyond the row length changes
    nothing, as in the reference."""
    from scipy.signal import lfilter
    gen = torch.Generator().manual_seed(seed_of('long filter', shape, K))
    x = torch.randn(shape, generator=gen)
    f = torch.randn(K, generator=gen) / K ** 0.5
    T = shape[-1]
    rows = x.reshape(-1, T).double().numpy()
    fd = f.double().numpy()
    conv_ref = lfilter(fd, [1.0], rows, axis=-1)
    corr_ref = lfilter(fd, [1.0], rows[:, ::-1], axis=-1)[:, ::-1]
    y = slayer.utils.filter.conv(x.to(dev()), f.to(dev()), 0.5)
    z = slayer.utils.filter.corr(x.to(dev()), f.to(dev()), 0.5)
    scale = 0.5 * np.abs(fd[:T]).sum() * np.abs(rows).max()
    assert np.abs(y.reshape(-1, T).cpu().double().numpy() - 0.5 * conv_ref).max() <= 1e-5 * scale
    assert np.abs(z.reshape(-1, T).cpu().double().numpy() - 0.5 * corr_ref).max() <= 1e-5 * scale
    if K > T:
        short = f[:T].contiguous().to(dev())
        assert torch.equal(y, slayer.utils.filter.conv(x.to(dev()), short, 0.5))
        assert torch.equal(z, slayer.utils.filter.corr(x.to(dev()), short, 0.5))
        wild = f.clone()
        wild[T:] = float('inf')
        assert torch.equal(y, slayer.utils.filter.conv(x.to(dev()), wild.to(dev()), 0.5))


def test_rows_and_filters_both_beyond_the_window_are_refused(slayer):
    x = torch.zeros(1, 12292, device=dev())
    with pytest.raises(RuntimeError, match='-3'):
        slayer.utils.filter.conv(x, torch.ones(12289, device=dev()))
    slayer.utils.filter.conv(x, torch.ones(12288, device=dev()))


@pytest.mark.parametrize('shape,K', [((16, 64), 9), ((5, 3, 16), 16), ((37, 132), 17), ((3, 700, 48), 32), ((2, 9, 1000), 33),
                                     ((64, 256, 100), 64), ((1, 20, 2048), 64), ((130, 4), 64), ((50, 260), 65),
                                     ((7, 11, 300), 100), ((33, 520), 128), ((33, 520), 129), ((4, 12), 40),
                                     ((50, 16), 64), ((40, 20), 17), ((700, 36), 128), ((33, 148), 100),
                                     ((4000, 300), 64), ((3, 5, 1500), 64), ((5, 2, 4096), 9), ((1, 1, 16), 16),
                                     ((2, 1021, 256), 33), ((300, 1028), 16),
                                     # rows that are not whole quads (the tensor as a whole still is)
                                     ((4, 37, 350), 64), ((8, 301), 64), ((12, 1003), 33), ((64, 250), 16),
                                     ((4, 5, 18), 9), ((20, 17), 12), ((2, 6, 1450), 100), ((4000, 302), 64),
                                     ((4, 999, 19), 64), ((2, 2, 4099), 128)])
def test_conv_corr_matrix_core_path(slayer, shape, K):
    """The matrix-core kernel walks the tensor as one stream of 256-sample tiles.  Tap counts either side of every
    padded size (16, 32, 64, 128) and of the kernel's limits (8 < K <= 128, T >= 16); rows shorter than a block, a
    tile or the filter (several rows in one window), rows that end inside a 16-sample block (T % 16 != 0: the
    two-view tiles) and on one, tensors of one tile and of thousands (several waves, each starting mid-row), rows
    that begin and end inside a quad (T % 4 != 0), a signed filter.  Every row against scipy.signal.lfilter in float64."""
    from scipy.signal import lfilter
    gen = torch.Generator().manual_seed(seed_of('mfma conv', shape, K))
    x = torch.randn(shape, generator=gen)
    f = torch.randn(K, generator=gen)
    T = shape[-1]
    rows = x.reshape(-1, T).double().numpy()
    fd = f.double().numpy()
    conv_ref = lfilter(fd, [1.0], rows, axis=-1)
    corr_ref = lfilter(fd, [1.0], rows[:, ::-1], axis=-1)[:, ::-1]
    assert np.allclose(conv_ref[0], np.convolve(rows[0], fd)[:T]) and \
        np.allclose(corr_ref[-1], np.convolve(rows[-1][::-1], fd)[:T][::-1])
    for ts in (1, 0.25):
        y = slayer.utils.filter.conv(x.to(dev()), f.to(dev()), ts).reshape(-1, T).cpu().double().numpy()
        z = slayer.utils.filter.corr(x.to(dev()), f.to(dev()), ts).reshape(-1, T).cpu().double().numpy()
        scale = ts * np.abs(fd).sum() * np.abs(rows).max()
        assert np.abs(y - ts * conv_ref).max() <= 1e-5 * scale, (shape, K, 'conv')
        assert np.abs(z - ts * corr_ref).max() <= 1e-5 * scale, (shape, K, 'corr')
    # non-negative data (no cancellation): the elementwise tolerance against the oracle holds as well
    xp, fp = x.abs(), f.abs()
    assert_rel(slayer.utils.filter.conv(xp.to(dev()), fp.to(dev()), 1), O.conv_fwd(xp, fp, 1), f'conv {shape} K={K}')
    assert_rel(slayer.utils.filter.corr(xp.to(dev()), fp.to(dev()), 1), O.conv_bwd(xp, fp, 1), f'corr {shape} K={K}')


@pytest.mark.parametrize('K', [16, 64, 128])
@pytest.mark.parametrize('x_scale,f_scale', [(1e-25, 1.0), (1e25, 1e-3), (1.0, 1e-30), (1e-12, 1e-12)])
def test_conv_corr_small_and_large_magnitudes(slayer, K, x_scale, f_scale):
    """The bar holds relative to the data's own scale from 1e-30 to 1e25 (beyond 32 taps the operands are split into
    bfloat16 parts, which keeps full precision while the parts stay normal float32 numbers: down to about 3e-33)."""
    from scipy.signal import lfilter
    gen = torch.Generator().manual_seed(seed_of('magnitudes', K, x_scale, f_scale))
    x = torch.randn(64, 300, generator=gen) * x_scale
    f = torch.randn(K, generator=gen) * f_scale
    rows, fd = x.double().numpy(), f.double().numpy()
    scale = np.abs(fd).sum() * np.abs(rows).max()
    y = slayer.utils.filter.conv(x.to(dev()), f.to(dev()), 1).cpu().double().numpy()
    z = slayer.utils.filter.corr(x.to(dev()), f.to(dev()), 1).cpu().double().numpy()
    assert np.abs(y - lfilter(fd, [1.0], rows, axis=-1)).max() <= 1e-5 * scale
    assert np.abs(z - lfilter(fd, [1.0], rows[:, ::-1], axis=-1)[:, ::-1]).max() <= 1e-5 * scale


@pytest.mark.parametrize('K', [16, 64, 128])
def test_conv_corr_at_the_top_of_the_float32_range(slayer, K):
    """Sparse samples of the largest float32 magnitudes (3.3895e38 is the largest bfloat16, 3.4028e38 the largest
    float32: in between a sample has no nearest bfloat16) and taps of the same magnitudes against unit samples:
    the results stay finite and meet the bar, as the reference's float32 multiply-adds do
    (utils/filter/conv.cu:25-78)."""
    from scipy.signal import lfilter
    gen = torch.Generator().manual_seed(seed_of('top of range', K))
    big = torch.tensor([3.3895e38, 3.39e38, 3.40e38, 3.4028234e38, -3.395e38, -3.4028234e38, 1.7e38, 3.38e38])
    x = torch.zeros(64, 300)
    pos = torch.randperm(64 * 300, generator=gen)[:400]
    x.view(-1)[pos] = big[torch.randint(0, len(big), (400,), generator=gen)]
    f = torch.randn(K, generator=gen) * (0.5 / K)            # sums of overlapping windows stay below the maximum
    for xs, fs in ((x, f), ((x != 0).float() * 0.125, torch.cat([big, torch.zeros(K - len(big))])[torch.randperm(K, generator=gen)])):
        rows, fd = xs.double().numpy(), fs.double().numpy()
        scale = np.abs(fd).sum() * np.abs(rows).max()
        y = slayer.utils.filter.conv(xs.to(dev()), fs.to(dev()), 1).cpu().double().numpy()
        z = slayer.utils.filter.corr(xs.to(dev()), fs.to(dev()), 1).cpu().double().numpy()
        assert np.isfinite(y).all() and np.isfinite(z).all()
        assert np.abs(y - lfilter(fd, [1.0], rows, axis=-1)).max() <= 1e-5 * scale
        assert np.abs(z - lfilter(fd, [1.0], rows[:, ::-1], axis=-1)[:, ::-1]).max() <= 1e-5 * scale


@pytest.mark.parametrize('K', [16, 24, 64, 100])
@pytest.mark.parametrize('shape', [(8192, 3200), (40000, 302)])
def test_conv_corr_many_tiles_per_wave(slayer, shape, K):
    """Tensors of tens of millions of samples, where a wave takes 8 (up to 16 taps) or 32 consecutive tiles: every
    row against scipy.signal.lfilter in float64."""
    from scipy.signal import lfilter
    gen = torch.Generator().manual_seed(seed_of('many tiles', shape, K))
    M, T = shape
    x = torch.randn(shape, generator=gen)
    f = torch.randn(K, generator=gen)
    rows, fd = x.double().numpy(), f.double().numpy()
    scale = np.abs(fd).sum() * np.abs(rows).max()
    y = slayer.utils.filter.conv(x.to(dev()), f.to(dev()), 1).cpu().double().numpy()
    assert np.abs(y - lfilter(fd, [1.0], rows, axis=-1)).max() <= 1e-5 * scale
    del y
    z = slayer.utils.filter.corr(x.to(dev()), f.to(dev()), 1).cpu().double().numpy()
    assert np.abs(z - lfilter(fd, [1.0], rows[:, ::-1], axis=-1)[:, ::-1]).max() <= 1e-5 * scale


@pytest.mark.parametrize('T,K', [(300, 64), (304, 16), (20, 100), (1500, 33), (301, 64), (350, 16), (19, 100), (1003, 33)])
def test_conv_rows_do_not_see_each_other(slayer, T, K):
    """A row's window is cut at the row: an Inf at the end (start) of one row leaves every other row finite and
    unchanged in conv (corr); inside its own row it arrives where the filter carries it."""
    gen = torch.Generator().manual_seed(seed_of('rows', T, K))
    M = 97 if T % 4 == 0 else 100          # the matrix kernel wants the tensor as a whole in whole quads
    x = torch.randn(M, T, generator=gen)
    f = torch.randn(K, generator=gen)
    base_c = slayer.utils.filter.conv(x.to(dev()), f.to(dev()), 1).cpu()
    base_r = slayer.utils.filter.corr(x.to(dev()), f.to(dev()), 1).cpu()
    for r in (0, 41, M - 1):
        bad = x.clone()
        bad[r, T - 1] = float('inf')
        y = slayer.utils.filter.conv(bad.to(dev()), f.to(dev()), 1).cpu()
        others = [i for i in range(M) if i != r]
        assert torch.equal(y[others], base_c[others]), f'conv: row {r} leaked'
        assert not torch.isfinite(y[r, T - 1])
        bad = x.clone()
        bad[r, 0] = float('inf')
        z = slayer.utils.filter.corr(bad.to(dev()), f.to(dev()), 1).cpu()
        assert torch.equal(z[others], base_r[others]), f'corr: row {r} leaked'
        assert not torch.isfinite(z[r, 0])


def test_conv_autograd_is_corr(slayer):
    gen = torch.Generator().manual_seed(61)
    x = torch.rand((3, 6, 90), generator=gen)
    f = torch.rand(11, generator=gen)
    g = torch.randn((3, 6, 90), generator=gen)
    xg = x.to(dev()).requires_grad_()
    slayer.utils.filter.conv(xg, f.to(dev()), 2).backward(g.to(dev()))
    assert_rel(xg.grad, O.conv_bwd(g, f, 2), 'conv backward')
    xg.grad = None
    slayer.utils.filter.corr(xg, f.to(dev()), 2).backward(g.to(dev()))
    assert_rel(xg.grad, O.conv_fwd(g, f, 2), 'corr backward')


def test_delay_module(slayer):
    gen = torch.Generator().manual_seed(70)
    x = torch.rand((2, 5, 3, 40), generator=gen)
    g = torch.randn((2, 5, 3, 40), generator=gen)
    d = torch.tensor([0.0, 3.2, 7.9, 1.0, 12.5])
    mod = slayer.axon.Delay(grad_scale=2.0)
    mod.delay.data = d.to(dev())
    mod.init = True
    xg = x.to(dev()).requires_grad_()
    y = mod(xg)
    per_neuron = d.reshape(-1, 1).repeat(1, 3)
    assert_exact(y, O.delay_fwd(x, per_neuron), 'delay forward')
    y.backward(g.to(dev()))
    ref_gi, ref_gd = O.delay_bwd(g, O.delay_fwd(x, per_neuron), per_neuron, grad_scale=2.0)
    assert_exact(xg.grad, ref_gi, 'delay grad_input')
    assert_rel(mod.delay.grad, ref_gd.sum(dim=1), 'delay grad_delay')
    # functional form, default one step
    assert_exact(slayer.axon.delay(x.to(dev())), O.shift(x, 1), 'delay()')


@pytest.mark.parametrize('shape,ts', [((2, 5, 3, 40), 1), ((3, 7, 37), 1), ((2, 6, 1000), 1), ((4, 9, 4, 4, 300), 2),
                                      ((1, 3, 3), 1), ((2, 64, 1), 1), ((5, 130, 516), 0.5)])
def test_delay_backward_kernel(slayer, shape, ts):
    """slayer_delay_bwd against the reference's four-step backward (filter, product, sum, shift): rows longer
    than one pass of a wave, T % 4 != 0, sampling times other than 1, shifts that empty a row, fractional and
    negative delays."""
    import importlib
    D = importlib.import_module('lava_dl_amd.slayer.axon.delay')      # the package attribute is the function
    gen = torch.Generator().manual_seed(seed_of('delay bwd', shape, ts))
    spatial = shape[1:-1]
    y = torch.rand(shape, generator=gen)
    g = torch.randn(shape, generator=gen)
    d = torch.rand(spatial, generator=gen) * 24 * ts - 2 * ts          # a few negative ones
    d.view(-1)[0] = 0.0
    d.view(-1)[-1] = (shape[-1] + 5) * ts                               # shifts the whole row out
    if d.numel() > 3:
        d.view(-1)[1] = 4 * ts                                          # aligned shift
    ref_gi, ref_gd = O.delay_bwd(g, y, d, grad_scale=1.0, sampling_time=ts)
    gi, gsum = D._delay_bwd(g.to(dev()), y.to(dev()), d.to(dev()), ts)
    assert_exact(gi, ref_gi, f'delay grad_input {shape}')
    assert_rel(gsum * ts, ref_gd, f'delay grad_delay {shape}')
    # misaligned views take the dword path and must agree with the aligned run
    if shape[-1] % 4 == 0:
        flat = torch.zeros(g.numel() + 1, device=dev())
        flat[1:] = g.to(dev()).flatten()
        gi2, gsum2 = D._delay_bwd(flat[1:].reshape(shape), y.to(dev()), d.to(dev()), ts)
        assert torch.equal(gi2, gi) and torch.equal(gsum2, gsum)


def test_delay_backward_entry_point_scalar_shift_and_no_sum(slayer):
    """C ABI directly: lut == NULL moves every row by scalar_steps; grad_sum == NULL skips the sums."""
    from lava_dl_amd.slayer import _native as N
    gen = torch.Generator().manual_seed(71)
    g = torch.randn(3, 10, 64, generator=gen)
    y = torch.rand(3, 10, 64, generator=gen)
    gg, yg = g.to(dev()), y.to(dev())
    for steps in (0, 5, -3, 64, 1000):
        out = torch.full_like(gg, float('nan'))
        N.check(N.lib().slayer_delay_bwd(N.ptr(out), None, N.ptr(gg), N.ptr(yg), None, steps, 1.0, None,
                                         30, 10, 64, N.stream_handle()))
        assert_exact(out, O.shift(g, -steps), f'delay_bwd scalar shift {steps}')
    assert N.lib().slayer_delay_bwd(N.ptr(out), N.ptr(out), N.ptr(gg), N.ptr(yg), None, 0, 1.0, None,
                                    30, 10, 64, N.stream_handle()) != 0           # sums wanted, no workspace
    assert N.lib().slayer_delay_bwd(N.ptr(out), None, N.ptr(gg), N.ptr(yg), None, 0, 0.0, None,
                                    30, 10, 64, N.stream_handle()) != 0           # sampling time 0


# --------------------------------------------------------------------------------- sigma-delta
@pytest.mark.parametrize('shape', [(3, 6, 200), (2, 3, 5, 7, 37), (4, 70, 129), (1, 5, 3), (4, 9000, 64)])
@pytest.mark.parametrize('cum', [False, True])
def test_delta_unit_and_sigma(slayer, shape, cum):
    from lava_dl_amd.slayer.axon import delta as D
    from lava_dl_amd.slayer.dendrite import sigma as SG
    gen = torch.Generator().manual_seed(seed_of(shape, cum, 'delta'))
    x = torch.cumsum(torch.randn(shape, generator=gen) * 0.3, dim=-1)
    C = shape[1]
    st = lambda: torch.randn(shape[:-1], generator=gen) * 0.2
    pre, res, err = st(), st(), st() * 0
    for thr in (torch.tensor([0.5]), (0.3 + torch.rand(C, generator=gen)).reshape([C] + [1] * (len(shape) - 3))):
        r_out, r_din, r_res, r_err = O.delta_fwd(x, thr, pre, res, err, cum)
        out, din, res_o, err_o = D._fwd(x.to(dev()), thr.to(dev()), pre.to(dev()), res.to(dev()), err.to(dev()), cum)
        assert_exact(out, r_out, f'delta events {shape}')
        assert_exact(din, r_din, f'delta input {shape}')
        assert_exact(res_o, r_res, 'delta residual')
        assert_exact(err_o, r_err, 'delta error')
        outq = D._fwd(x.to(dev()), thr.to(dev()), pre.to(dev()), res.to(dev()), err.to(dev()), cum, 1 / 64)[0]
        assert_exact(outq, O.quantize_floor(r_out, 1 / 64), 'delta quantised events')
        g = torch.randn(shape, generator=gen)
        w_in, w_thr = O.delta_bwd(g, r_din, thr, 0.8, 1.5)
        g_in, g_thr = D._bwd(g.to(dev()), din, thr.to(dev()), 0.8, 1.5)
        assert_exact(g_in, w_in, 'delta grad_input')
        assert_rel(g_thr.reshape(w_thr.shape), w_thr, 'delta grad_threshold')
    # running sum: float-mode against torch's cumsum, exact against strictly sequential float32 adds,
    # and exact against torch's cumsum on quantised events (multiples of 1/64 add without rounding)
    assert_rel(SG._cumsum(out), O.sigma_fwd(r_out), 'sigma running sum')
    assert_exact(SG._cumsum(out), _seq_cumsum(r_out, torch.zeros(shape[:-1])), 'sigma sequential sum')
    assert_exact(SG._cumsum(out, pre.to(dev())), _seq_cumsum(r_out, pre), 'sigma with carried state')
    rq = O.quantize_floor(r_out, 1 / 64)
    assert_exact(SG._cumsum(outq), O.sigma_fwd(rq), 'sigma on quantised events')
    assert_exact(SG._cumsum(outq, None, reverse=True), torch.flip(O.sigma_fwd(torch.flip(rq, [-1])), [-1]),
                 'sigma reverse sum')


def _seq_cumsum(x, start):
    """Sequential float32 running sum that starts from ``start`` (the kernel adds the state first)."""
    out = torch.zeros_like(x)
    y = start.clone()
    for t in range(x.shape[-1]):
        y = y + x[..., t]
        out[..., t] = y
    return out


def test_delta_sigma_modules(slayer):
    gen = torch.Generator().manual_seed(90)
    x = torch.cumsum(torch.randn((2, 4, 3, 150), generator=gen) * 0.3, dim=-1)
    for shared, cum in ((True, False), (False, True)):
        enc = slayer.axon.Delta(threshold=0.5, cum_error=cum, shared_param=shared, requires_grad=True).to(dev())
        dec = slayer.dendrite.Sigma().to(dev())
        xg = x.to(dev()).requires_grad_()
        ev = enc(xg)
        thr = enc.threshold.detach().cpu()
        zero = torch.zeros(x.shape[:-1])
        r_out, r_din, _, _ = O.delta_fwd(x, thr, zero, zero, zero, cum)
        assert_exact(ev, O.quantize_floor(r_out, 1 / 64), 'Delta module events')
        y = dec(ev)
        assert_exact(y, O.sigma_fwd(O.quantize_floor(r_out, 1 / 64)), 'Sigma module output')
        g = torch.randn(x.shape, generator=gen)
        y.backward(g.to(dev()))
        # gradient of the running sum = running sum from the last step backwards (sequential float32 adds;
        # a differently grouped sum would differ by an ulp of the partial sums, which the time difference
        # in the delta backward then magnifies)
        g_ev = torch.flip(_seq_cumsum(torch.flip(g, [-1]), torch.zeros(x.shape[:-1])), [-1])
        w_in, w_thr = O.delta_bwd(g_ev, r_din, thr, 1, 1)
        assert_exact(xg.grad, w_in, 'Delta module grad_input')
        assert enc.threshold.grad.shape == enc.threshold.shape
        assert_rel(enc.threshold.grad.reshape(w_thr.shape), w_thr, 'Delta module grad_threshold')
    # persistent state: two halves equal one pass
    enc_full = slayer.axon.Delta(0.5).to(dev())
    enc_split = slayer.axon.Delta(0.5, persistent_state=True).to(dev())
    dec_split = slayer.dendrite.Sigma(persistent_state=True).to(dev())
    xg = x.to(dev())
    full = enc_full(xg)
    a, b = enc_split(xg[..., :70].contiguous()), enc_split(xg[..., 70:].contiguous())
    assert torch.equal(torch.cat([a, b], -1), full)
    ya, yb = dec_split(a), dec_split(b)
    assert torch.equal(torch.cat([ya, yb], -1), slayer.dendrite.Sigma().to(dev())(full))
