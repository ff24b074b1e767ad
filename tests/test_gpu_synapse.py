"""The convolution synapse on time-innermost tensors (csrc/synapse.hip, slayer.synapse.Conv) against the oracle's
float64 evaluation of the reference's call (synapse/layer.py:297-323: F.conv3d with a (kh, kw, 1) kernel on NCHWT),
every output element to 1e-5 of the sum of the magnitudes of its terms; the gradients of the input and of the
weights (slayer_conv_synapse_wgrad) against float64 autograd to the same bar;
shapes the kernel does not take go to the library call and give the same result."""
import pytest
import torch
import torch.nn.functional as F

from oracle import slayer_oracle as O
from tests.util import assert_sum, dev, seed_of

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _check(slayer, shape, co, kernel, stride, padding, dilation, what, backward=True):
    n, ci, h, w, t = shape
    gen = torch.Generator().manual_seed(seed_of('conv-synapse', shape, co, kernel, stride, padding, dilation))
    x = (torch.rand(shape, generator=gen) < 0.3).float() * torch.randn(shape, generator=gen)
    wt = torch.randn(co, ci, kernel[0], kernel[1], 1, generator=gen)
    xg = x.to(dev()).requires_grad_(backward)
    wg = wt.to(dev()).requires_grad_(backward)
    got = slayer.synapse.conv_synapse(xg, wg, stride, padding, dilation)
    want = O.conv_synapse(x, wt, stride, padding, dilation)
    mag = O.conv_synapse(x.abs(), wt.abs(), stride, padding, dilation)
    assert got.shape == want.shape and got.is_contiguous()
    assert_sum(got, want.double(), mag.double(), what + ' forward')
    if backward:
        g = torch.randn(want.shape, generator=gen)
        got.backward(g.to(dev()))
        xd, wd = x.double().requires_grad_(), wt.double().requires_grad_()
        ref = F.conv3d(xd, wd, None, tuple(stride) + (1,), tuple(padding) + (0,), tuple(dilation) + (1,))
        ref.backward(g.double())
        # magnitudes of the terms of both gradients: the same sums over absolute values
        xa, wa = x.abs().double().requires_grad_(), wt.abs().double().requires_grad_()
        F.conv3d(xa, wa, None, tuple(stride) + (1,), tuple(padding) + (0,), tuple(dilation) + (1,)).backward(g.abs().double())
        assert_sum(xg.grad, xd.grad, xa.grad, what + ' grad input')
        assert_sum(wg.grad, wd.grad, wa.grad, what + ' grad weight')


@pytest.mark.parametrize('shape,co,kernel,stride,padding,dilation', [
    ((2, 3, 6, 7, 8), 5, (3, 3), (1, 1), (1, 1), (1, 1)),          # fewer than 16 output channels, one short tile
    ((2, 8, 9, 9, 64), 16, (3, 3), (1, 1), (1, 1), (1, 1)),         # exactly one tile of 64 steps
    ((1, 2, 34, 34, 300), 16, (5, 5), (2, 2), (2, 2), (1, 1)),      # stride 2, T = 4 tiles + 44 steps
    ((2, 4, 12, 10, 100), 40, (3, 2), (1, 2), (0, 1), (2, 1)),      # three blocks of output channels, mixed geometry
    ((3, 16, 8, 8, 36), 32, (1, 1), (1, 1), (0, 0), (1, 1)),        # 1x1: a dense synapse per pixel
    ((1, 5, 10, 12, 260), 7, (3, 3), (1, 1), (0, 0), (2, 2)),       # no padding, dilation 2
    ((2, 16, 7, 9, 72), 8, (3, 3), (1, 1), (1, 1), (1, 1)),         # 144 taps: two passes of the weight gradient
    ((3, 1, 9, 8, 132), 4, (3, 3), (1, 1), (1, 1), (1, 1)),         # 9 taps: one tile of taps
    ((1, 20, 5, 5, 1032), 3, (3, 3), (1, 1), (2, 2), (1, 1)),       # 180 taps, long rows: several shares of time
    ((2, 3, 9, 9, 40), 6, (5, 5), (1, 1), (2, 2), (1, 1)),          # five taps per row, one tile of pairs
    # rows that are not whole quads of steps (T % 4 = 1, 2, 3), whole tiles of 64 steps and a few steps more
    ((2, 8, 9, 9, 65), 16, (3, 3), (1, 1), (1, 1), (1, 1)),
    ((1, 3, 6, 7, 350), 5, (3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 4, 5, 6, 131), 20, (3, 3), (2, 1), (1, 1), (1, 1)),
    ((1, 2, 12, 10, 7), 3, (5, 5), (2, 2), (2, 2), (1, 1)),
    ((3, 5, 4, 4, 4), 2, (1, 1), (1, 1), (0, 0), (1, 1)),
    ((1, 7, 8, 8, 36), 20, (5, 3), (1, 1), (2, 1), (1, 1)),         # 35 pairs: two tiles and a second pass; kw = 3, kh = 5
    ((1, 7, 8, 8, 36), 20, (3, 5), (1, 1), (1, 2), (1, 1)),         # kw = 5, kh = 3
    # strides whose residue classes differ in their taps (the input gradient is one convolution per class): a common
    # factor of stride and dilation, a stride beyond the kernel, a stride of 3 under 5 taps, strides of 16
    ((2, 3, 11, 11, 20), 4, (3, 3), (2, 2), (1, 1), (2, 2)),
    ((1, 4, 17, 12, 24), 6, (3, 2), (4, 4), (2, 0), (6, 2)),
    ((2, 2, 14, 17, 12), 3, (2, 2), (3, 5), (0, 1), (1, 1)),
    ((1, 5, 16, 16, 44), 16, (5, 5), (3, 3), (2, 2), (1, 1)),
    ((1, 2, 40, 36, 8), 3, (3, 3), (16, 16), (1, 1), (1, 1)),
    ((2, 1, 13, 12, 30), 1, (3, 3), (2, 2), (1, 1), (1, 1)),        # one channel in and out: the vector-unit kernel
    ((1, 1, 9, 9, 21), 1, (2, 3), (1, 2), (1, 0), (2, 1)),
])
def test_conv_synapse_against_the_oracle(slayer, shape, co, kernel, stride, padding, dilation):
    _check(slayer, shape, co, kernel, stride, padding, dilation, f'{shape} -> {co}')


def test_conv_module_mirrors_the_reference_layer(slayer):
    """slayer.synapse.Conv: same constructor and weight shape as the reference layer, pre_hook_fx applied to the
    weight, gradients reach weight and input."""
    gen = torch.Generator().manual_seed(3)
    syn = slayer.synapse.Conv(3, 6, 3, padding=1, weight_scale=2, pre_hook_fx=lambda w: (w * 8).round() / 8).to(dev())
    assert tuple(syn.weight.shape) == (6, 3, 3, 3, 1) and syn.bias is None
    x = (torch.rand(2, 3, 8, 8, 40, generator=gen) < 0.2).float().to(dev()).requires_grad_()
    y = syn(x)
    want = O.conv_synapse(x.detach().cpu(), ((syn.weight * 8).round() / 8).detach().cpu(), (1, 1), (1, 1), (1, 1))
    assert float((y.detach().cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    y.sum().backward()
    assert syn.weight.grad is not None and x.grad is not None and x.grad.shape == x.shape


def test_shapes_the_kernel_does_not_take_go_to_the_library_call(slayer):
    gen = torch.Generator().manual_seed(4)
    x = torch.randn(2, 4, 6, 6, 3, generator=gen).to(dev())                  # fewer than four steps
    w = torch.randn(6, 4, 3, 3, 1, generator=gen).to(dev())
    assert torch.equal(slayer.synapse.conv_synapse(x, w, 1, 1, 1), F.conv3d(x, w, None, (1, 1, 1), (1, 1, 0)))
    w2 = torch.randn(6, 2, 3, 3, 1, generator=gen).to(dev())                 # two groups
    x2 = torch.randn(2, 4, 6, 6, 12, generator=gen).to(dev())
    assert torch.equal(slayer.synapse.conv_synapse(x2, w2, 1, 1, 1, groups=2),
                       F.conv3d(x2, w2, None, (1, 1, 1), (1, 1, 0), (1, 1, 1), 2))


def test_conv_synapse_at_the_size_of_the_benchmark_tensor(slayer):
    """The synapse that produces config[1]'s tensor: spikes [32, 8, 32, 32, 300] -> [32, 16, 32, 32, 300], 3x3,
    padding 1.  Slabs against the oracle, the whole tensor against the library call within 1e-5 of the terms'
    magnitudes, and the fused CUBA neuron reads the result where the kernel left it."""
    gen = torch.Generator(device=dev()).manual_seed(9)
    shape = (32, 8, 32, 32, 300)
    x = (torch.rand(shape, device=dev(), generator=gen) < 0.05).float()
    w = torch.randn(16, 8, 3, 3, 1, device=dev(), generator=gen) * 0.3
    z = slayer.synapse.conv_synapse(x, w, 1, 1, 1)
    assert z.shape == (32, 16, 32, 32, 300) and z.is_contiguous()
    lib = F.conv3d(x, w, None, (1, 1, 1), (1, 1, 0))
    mag = F.conv3d(x, w.abs(), None, (1, 1, 1), (1, 1, 0))
    assert bool(((z - lib).abs() <= 1e-5 * mag + 1e-30).all())
    for n in (0, 31):
        want = O.conv_synapse(x[n:n + 1].cpu(), w.cpu(), (1, 1), (1, 1), (1, 1))
        mg = O.conv_synapse(x[n:n + 1].cpu(), w.abs().cpu(), (1, 1), (1, 1), (1, 1))
        assert_sum(z[n:n + 1], want.double(), mg.double() + 1e-30, f'batch entry {n}')
    neuron = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03).to(dev())
    spikes = neuron(z)
    assert spikes.shape == z.shape and 0 < float(spikes.sum()) < spikes.numel()


def test_weight_gradient_at_the_size_of_the_benchmark_tensor(slayer):
    """grad_weight of the synapse above at full size against nine float64 matrix products over the shifted views
    (the defining sum), 1e-5 of the sum of the terms' magnitudes."""
    gen = torch.Generator(device=dev()).manual_seed(10)
    shape = (32, 8, 32, 32, 300)
    x = (torch.rand(shape, device=dev(), generator=gen) < 0.05).float()
    g = torch.randn((32, 16, 32, 32, 300), device=dev(), generator=gen)
    w = (torch.randn(16, 8, 3, 3, 1, device=dev(), generator=gen) * 0.3).requires_grad_()
    slayer.synapse.conv_synapse(x, w, 1, 1, 1).backward(g)
    want = torch.empty(16, 8, 3, 3, dtype=torch.float64, device=dev())
    mag = torch.empty_like(want)
    xp = F.pad(x, (0, 0, 1, 1, 1, 1))
    for n0 in range(0, 32, 8):                                     # float64 copies of a quarter of the batch at a time
        gf = g[n0:n0 + 8].permute(1, 0, 2, 3, 4).reshape(16, -1).double()
        for y in range(3):
            for xx in range(3):
                v = xp[n0:n0 + 8, :, y:y + 32, xx:xx + 32, :].permute(1, 0, 2, 3, 4).reshape(8, -1).double()
                if n0 == 0:
                    want[:, :, y, xx] = 0
                    mag[:, :, y, xx] = 0
                want[:, :, y, xx] += gf @ v.t()
                mag[:, :, y, xx] += gf.abs() @ v.t()
    assert_sum(w.grad[..., 0], want, mag, 'grad weight at [32,8,32,32,300]')


def test_tensors_at_dword_aligned_addresses(slayer):
    """Input and gradient that start one float into their allocations (contiguous views): same results as the
    aligned copies, bit for bit."""
    gen = torch.Generator().manual_seed(21)
    shape, co = (2, 4, 6, 7, 70), 6
    x = (torch.rand(shape, generator=gen) < 0.3).float() * torch.randn(shape, generator=gen)
    w = torch.randn(co, 4, 3, 3, 1, generator=gen).to(dev())
    g = torch.randn((2, co, 6, 7, 70), generator=gen)

    def off_by_one(t):
        buf = torch.empty(t.numel() + 1, device=dev())
        view = buf[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 4 and view.is_contiguous()
        return view

    results = []
    for shifted in (False, True):
        xs = (off_by_one(x) if shifted else x.to(dev())).requires_grad_()
        ws = w.clone().requires_grad_()
        y = slayer.synapse.conv_synapse(xs, ws, 1, 1, 1)
        y.backward(off_by_one(g) if shifted else g.to(dev()))
        results.append((y.detach(), xs.grad, ws.grad))
    for a, b, what in zip(results[0], results[1], ('forward', 'grad input', 'grad weight')):
        assert torch.equal(a, b), what


@pytest.mark.parametrize('shape,kernel,stride,scale', [((2, 3, 8, 6, 20), 2, None, 1.0), ((1, 4, 7, 9, 64), 2, None, 0.5),
                                                        ((2, 2, 9, 8, 33), (3, 2), None, 2.0), ((1, 16, 32, 32, 100), 2, None, 1.0),
                                                        ((2, 3, 9, 8, 12), 3, 3, 1.0), ((1, 2, 12, 10, 18), (4, 2), (4, 2), 1.0)])
def test_pool_layer(slayer, shape, kernel, stride, scale):
    """slayer.synapse.Pool (synapse/layer.py:326-510 in the reference) through the convolution kernels: the sums
    over the windows as the reference forms them (channels folded into the height, zero rows behind an image that
    is not a whole number of windows), and the gradient of the input through the transposed kernel, against
    float64 autograd of the same expression."""
    gen = torch.Generator().manual_seed(seed_of('pool', shape, kernel, stride))
    pool = slayer.synapse.Pool(kernel, stride, weight_scale=scale).to(dev())
    x = (torch.rand(shape, generator=gen) < 0.3).float() * torch.randn(shape, generator=gen)
    xg = x.to(dev()).requires_grad_()
    y = pool(xg)

    def reference(v):
        kh, kw = pool.weight.shape[2], pool.weight.shape[3]
        if v.shape[2] % kh:
            v = torch.cat((v, v.new_zeros(v.shape[0], v.shape[1], v.shape[2] % kh, v.shape[3], v.shape[4])), 2)
        if v.shape[3] % kw:
            v = torch.cat((v, v.new_zeros(v.shape[0], v.shape[1], v.shape[2], v.shape[3] % kw, v.shape[4])), 3)
        n, c, h, w, t = v.shape
        r = F.conv3d(v.reshape(n, 1, c * h, w, t), pool.weight.detach().cpu().to(v.dtype), None, pool.stride)
        return r.reshape(n, c, -1, r.shape[3], t)

    xd, xa = x.double().requires_grad_(), x.abs().double().requires_grad_()
    want, mag = reference(xd), reference(xa)
    assert y.shape == want.shape
    assert_sum(y, want.detach(), mag.detach() + 1e-30, 'pooled spikes')
    g = torch.randn(want.shape, generator=gen)
    y.backward(g.to(dev()))
    want.backward(g.double())
    mag.backward(g.abs().double())
    assert_sum(xg.grad, xd.grad, xa.grad + 1e-30, 'gradient of the input')


@pytest.mark.parametrize('shape,co,kernel,stride,padding,dilation', [
    ((2, 5, 6, 7, 8), 3, (3, 3), (1, 1), (1, 1), (1, 1)),
    ((1, 16, 17, 17, 300), 2, (5, 5), (2, 2), (2, 2), (1, 1)),      # what a decoder holds: few maps out of many
    ((2, 8, 9, 9, 64), 16, (2, 2), (2, 2), (0, 0), (1, 1)),          # kernel = stride: every output has one term
    ((2, 4, 6, 5, 101), 20, (3, 2), (1, 2), (0, 1), (2, 1)),
    ((1, 3, 5, 6, 37), 7, (4, 4), (3, 3), (1, 1), (1, 1)),           # T % 4 = 1, stride 3
    ((3, 6, 4, 4, 4), 5, (1, 1), (1, 1), (0, 0), (1, 1)),
    # residue classes of the output pixels that differ in their taps: stride and dilation with a common factor
    # (every other class meets no tap at all), a stride beyond the kernel (classes without taps, rows of zeros),
    # a stride of 3 under 5 taps (classes of two taps and of one)
    ((2, 3, 5, 5, 20), 4, (3, 3), (2, 2), (1, 1), (2, 2)),
    ((1, 4, 4, 5, 24), 6, (3, 2), (4, 4), (2, 0), (6, 2)),
    ((2, 2, 6, 4, 12), 3, (2, 2), (3, 5), (0, 1), (1, 1)),
    ((1, 5, 6, 6, 44), 16, (5, 5), (3, 3), (2, 2), (1, 1)),
    ((2, 1, 7, 6, 30), 1, (3, 3), (2, 2), (1, 1), (1, 1)),          # one channel in and out: the vector-unit kernel
])
def test_conv_transpose_synapse(slayer, shape, co, kernel, stride, padding, dilation):
    """slayer.synapse.conv_transpose_synapse (the reference's F.conv_transpose3d call, synapse/layer.py:630-658)
    on the convolution kernels with their roles exchanged: output and both gradients against float64 evaluation of
    that call, every element to 1e-5 of the sum of the magnitudes of its terms."""
    n, ci, h, w, t = shape
    gen = torch.Generator().manual_seed(seed_of('conv-transpose', shape, co, kernel, stride, padding, dilation))
    x = (torch.rand(shape, generator=gen) < 0.3).float() * torch.randn(shape, generator=gen)
    wt = torch.randn(ci, co, kernel[0], kernel[1], 1, generator=gen)
    xg, wg = x.to(dev()).requires_grad_(), wt.to(dev()).requires_grad_()
    calls = []
    plain = slayer.synapse.layer._launch_input_grad
    slayer.synapse.layer._launch_input_grad = lambda *a: calls.append(1) or plain(*a)
    try:
        got = slayer.synapse.conv_transpose_synapse(xg, wg, stride, padding, dilation)
    finally:
        slayer.synapse.layer._launch_input_grad = plain
    assert calls, 'the library call ran instead of the kernel'

    def reference(a, b):
        return F.conv_transpose3d(a, b, None, tuple(stride) + (1,), tuple(padding) + (0,), 0, 1, tuple(dilation) + (1,))

    xd, wd = x.double().requires_grad_(), wt.double().requires_grad_()
    xa, wa = x.abs().double().requires_grad_(), wt.abs().double().requires_grad_()
    want, mag = reference(xd, wd), reference(xa, wa)
    assert got.shape == want.shape and got.is_contiguous()
    assert_sum(got, want.detach(), mag.detach() + 1e-30, 'forward')
    g = torch.randn(want.shape, generator=gen)
    got.backward(g.to(dev()))
    want.backward(g.double())
    mag.backward(g.abs().double())
    assert_sum(xg.grad, xd.grad, xa.grad + 1e-30, 'grad input')
    assert_sum(wg.grad, wd.grad, wa.grad + 1e-30, 'grad weight')


def test_transposed_layers_mirror_the_reference_layers(slayer):
    """ConvTranspose and Unpool (synapse/layer.py:511-838): module attributes, the weight pre-hook, the channels of
    the unpooling layer folded into the height; what the kernels do not take goes to the library call."""
    gen = torch.Generator().manual_seed(77)
    quant = lambda v: (v * 8).round() / 8
    up = slayer.synapse.ConvTranspose(6, 4, 3, stride=2, padding=1, weight_scale=2, pre_hook_fx=quant).to(dev())
    assert tuple(up.shape) == (6, 4, 3, 3, 1) and up.bias is None and up.complex is False
    x = torch.randn(2, 6, 5, 7, 24, generator=gen)
    y = up(x.to(dev()))
    want = F.conv_transpose3d(x.double(), quant(up.weight.detach().cpu()).double(), None, (2, 2, 1), (1, 1, 0))
    assert y.shape == want.shape == (2, 4, 9, 13, 24)
    assert float((y.cpu().double() - want).abs().max()) < 1e-4
    grouped = slayer.synapse.ConvTranspose(6, 4, 3, groups=2).to(dev())         # groups: the library call
    assert grouped(x.to(dev())).shape == (2, 4, 7, 9, 24)
    assert slayer.synapse.ConvTranspose(6, 4, 3).to(dev())(x[..., :3].to(dev())).shape == (2, 4, 7, 9, 3)   # T < 4

    unpool = slayer.synapse.Unpool(2, weight_scale=0.5).to(dev())
    assert tuple(unpool.weight.shape) == (1, 1, 2, 2, 1) and not unpool.weight.requires_grad
    xg = x.to(dev()).requires_grad_()
    z = unpool(xg)
    assert z.shape == (2, 6, 10, 14, 24)
    # every sample spread over its own window of its own channel
    assert torch.equal(z.detach().cpu(), 0.5 * x.repeat_interleave(2, 2).repeat_interleave(2, 3))
    g = torch.randn(z.shape, generator=gen)
    z.backward(g.to(dev()))
    want = 0.5 * g.reshape(2, 6, 5, 2, 7, 2, 24).double().sum(dim=(3, 5))
    assert float((xg.grad.cpu().double() - want).abs().max()) < 1e-5
    pair = slayer.synapse.complex.ConvTranspose(6, 4, 3, stride=2).to(dev())
    re, im = pair(x.to(dev()))
    assert re.shape == im.shape == (2, 4, 11, 15, 24) and not torch.equal(re, im)


def test_synapse_kernels_under_graph_capture_replays(slayer):
    """The synapse entry points enqueue kernels only (the weight gradient clears nothing with a memset, its
    workspace comes from the caller), so a training step of a convolution and a pooling layer can be captured in a
    graph; every replay, with eager work in between, must equal the eager result bit for bit."""
    L = slayer.synapse.layer
    gen = torch.Generator().manual_seed(seed_of('synapse graph'))
    x = torch.zeros(2, 3, 8, 8, 40, device=dev())
    g = torch.zeros(2, 5, 4, 4, 40, device=dev())
    w = torch.randn(5, 3, 3, 3, 1, generator=gen).to(dev())
    pool_w = torch.ones(1, 1, 2, 2, device=dev())

    def fill():
        x.copy_(((torch.rand(x.shape, generator=gen) < 0.3).float() * torch.randn(x.shape, generator=gen)).to(dev()))
        g.copy_(torch.randn(g.shape, generator=gen).to(dev()))

    def step():
        w4 = w[..., 0].contiguous()
        z = L._launch(x, w4, (2, 2), (1, 1), (1, 1))                               # strided convolution
        g_x = L._launch_input_grad(g, w4.transpose(0, 1).contiguous(), x.shape, (2, 2), (1, 1), (1, 1))
        g_w = L._weight_gradient(x, w.shape, g, (2, 2), (1, 1), (1, 1))
        n, c, h, wd, t = z.shape
        pooled = L._launch(z.view(n, 1, c * h, wd, t), pool_w, (2, 2), (0, 0), (1, 1))
        spread = L._launch_input_grad(pooled, pool_w, (n, 1, c * h, wd, t), (2, 2), (0, 0), (1, 1))
        return z, g_x, g_w, pooled, spread

    fill()
    step()                                      # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    torch.cuda.synchronize()
    for k in range(3):
        fill()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()                           # eager work between the replays
        torch.cuda.synchronize()
        assert float(want[0].abs().sum()) > 0 and float(want[2].abs().sum()) > 0
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f'replay {k}: output {i} differs from the eager result'
