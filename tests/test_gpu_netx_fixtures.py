"""The fused neuron kernels, as `cuba.Neuron.forward` / `rf.Neuron.forward` run them, on the known answers the
reference's own tests hold (tests/lava/lib/dl/netx/test_blocks.py:180-228 dense LIF block, :282-332 complex dense RF
block; fixtures re-encoded by tests/golden/make_fixtures.py): every form of the forward pass (spikes only, without the
current trace, with every trace) and the one-step block delay folded into the kernel, which is the latency the
lava-side blocks of those fixtures have."""
import numpy as np
import pytest
import torch

from tests.golden import fixtures as G
from tests.util import dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _cuba(slayer, fx, trainable):
    n = slayer.neuron.cuba.Neuron(threshold=6 / 64, current_decay=1.0, voltage_decay=0.1,
                                  requires_grad=trainable).to(dev())
    assert n.s_scale == G.W_SCALE and abs(n.threshold + n.threshold_eps - fx['threshold']) < 1e-9
    n.current_decay.data = torch.tensor([fx['current_decay']], device=dev())
    n.voltage_decay.data = torch.tensor([fx['voltage_decay']], device=dev())
    return n


@pytest.mark.parametrize('form', ['inference', 'lean', 'full', 'debug'])
def test_cuba_neuron_forward_on_the_dense_lif_fixture(slayer, form):
    fx = G.dense_lif()
    n = _cuba(slayer, fx, trainable=(form == 'full'))
    x = fx['x'].to(dev())
    if form == 'inference':
        with torch.no_grad():
            spk = n(x)
    else:
        n.debug = form == 'debug'                       # debug: the separate, cross-checked operators
        spk = n(x.requires_grad_())
        spk.sum().backward()
        assert torch.isfinite(x.grad).all() and float(x.grad.abs().sum()) > 0
    got = spk[0].detach().cpu().numpy().astype(np.int64)[:, :fx['expected'].shape[1]]
    assert int((got != fx['expected']).sum()) == 0
    assert got.sum() == 1826


@pytest.mark.parametrize('form', ['inference', 'lean'])
def test_cuba_block_tail_with_the_step_delay_folded_on_the_dense_lif_fixture(slayer, form):
    """neuron -> step_delay in one kernel: the spike of step t leaves at t + 1, which is where the lava-side
    block of the fixture has it (expected[:, t] = out.npy[:, t + 1])."""
    fx = G.dense_lif()

    class Block:
        delay_shift, delay = True, None
    blk = Block()
    blk.neuron = _cuba(slayer, fx, trainable=False)
    x = fx['x'].to(dev())
    if form == 'inference':
        with torch.no_grad():
            out = slayer.block.neuron_delay(blk, x)
    else:
        out = slayer.block.neuron_delay(blk, x.requires_grad_())
    got = out[0].detach().cpu().numpy().astype(np.int64)
    assert int(got[:, 0].sum()) == 0
    assert int((got[:, 1:] != fx['expected']).sum()) == 0 and got.sum() >= 1826 - 256


@pytest.mark.parametrize('form', ['inference', 'grad', 'trainable', 'debug'])
def test_rf_neuron_forward_on_the_complex_dense_fixture(slayer, form):
    fx = G.complex_dense_rf()
    n = slayer.neuron.rf.Neuron(threshold=25 / 64, period=11, decay=0.05, requires_grad=(form == 'trainable')).to(dev())
    assert n.s_scale == G.W_SCALE and abs(n.threshold - fx['threshold']) < 1e-9
    n.sin_decay.data = torch.tensor([fx['sin_decay']], device=dev())
    n.cos_decay.data = torch.tensor([fx['cos_decay']], device=dev())
    xr, xi = fx['xr'].to(dev()), fx['xi'].to(dev())
    if form == 'inference':
        with torch.no_grad():
            spk = n((xr, xi))
    else:
        n.debug = form == 'debug'
        spk = n((xr.requires_grad_(), xi.requires_grad_()))
        spk.sum().backward()
        assert torch.isfinite(xr.grad).all() and torch.isfinite(xi.grad).all()
    got = spk[0].detach().cpu().numpy().astype(np.int64)[:, :fx['expected'].shape[1]]
    assert int((got != fx['expected']).sum()) == 0 and got.sum() > 40000


def test_dense_synapse_output_feeds_the_fused_neuron_without_a_layout_pass(slayer):
    """The reference's Dense synapse is a 1x1x1 `conv3d` over [N, C_in, 1, 1, T] (synapse/layer.py:144-175), i.e. the
    batched GEMM weight @ x over [N, C_in, T].  Its output [N, C_out, T] is contiguous with time innermost, which is
    the layout the kernels take: the fused neuron kernel receives the GEMM's own buffer (no transpose, no copy in
    between).  Checked on the dense LIF block of the netx fixture, synapse included, for both ways of writing it."""
    import torch.nn.functional as F
    from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
    fx = G.dense_lif_block()
    s, w = fx['spikes'].to(dev()), fx['weight'].to(dev())
    z_conv = F.conv3d(s.reshape(1, s.shape[1], 1, 1, -1), w.reshape(w.shape[0], w.shape[1], 1, 1, 1))
    z_mm = torch.matmul(w, s)
    assert z_conv.is_contiguous() and z_conv.shape == (1, 256, 1, 1, s.shape[-1])
    assert z_mm.is_contiguous() and z_mm.shape == (1, 256, s.shape[-1])
    assert torch.equal(z_mm.cpu(), fx['x']), 'synaptic input differs from weight @ spikes'
    assert torch.equal(z_conv.reshape(z_mm.shape), z_mm)
    library = cuba_fused.N.lib()
    seen = []

    class Spy:
        def __getattr__(self, name):
            fn = getattr(library, name)
            if name != 'slayer_cuba_fwd':
                return fn
            return lambda *a: (seen.append(a[5]), fn(*a))[1]         # a[5]: the input pointer handed to the kernel
    real_lib = cuba_fused.N.lib
    cuba_fused.N.lib = lambda: Spy()
    try:
        for z in (z_mm, z_conv):
            n = _cuba(slayer, fx, trainable=False)
            with torch.no_grad():
                spk = n(z)
            got = spk.reshape(256, -1).cpu().numpy().astype(np.int64)[:, :fx['expected'].shape[1]]
            assert int((got != fx['expected']).sum()) == 0 and got.sum() == 1826
    finally:
        cuba_fused.N.lib = real_lib
    assert seen == [z_mm.data_ptr(), z_conv.data_ptr()], 'the kernel did not read the GEMM output in place'
