"""Axonal delays folded into the fused CUBA / ALIF / RF kernels (the shift before a neuron, step_delay and
the learnable Delay after it: block/base.py:15-39,549-553, axon/delay.py:132-221, utils/time/shift.py:94-143
in the reference) against the chain of separate operators on the GPU, bit for bit, and against the
oracle's chain on the CPU."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import assert_exact, assert_rel, assert_scale, assert_sum, dev, seed_of, sparse_input, SCAN_MIN

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _delays(slayer, gen, shape, in_kind, out_kind, steps, head, ts=1.0, train_delay=False):
    """A Delays and its description for the oracle: (input shift tensor|number|None, output delay tensor|None)."""
    neurons = shape[1:-1]
    T = shape[-1]
    in_shift = out_delay = head_t = None
    if in_kind == 'table':
        in_shift = (torch.rand(neurons, generator=gen) * min(40, T + 3) * ts)
        in_shift.view(-1)[0] = 0.0                      # no shift at all
        if in_shift.numel() > 2:
            in_shift.view(-1)[1] = (T + 2) * ts         # empties the row
            in_shift.view(-1)[2] = -3.0 * ts            # advances
    elif in_kind == 'scalar':
        in_shift = 5.5 * ts
    if out_kind == 'table':
        out_delay = (torch.rand(neurons, generator=gen) * min(33, T + 3) * ts)
        out_delay.view(-1)[0] = 0.0
        if out_delay.numel() > 1:
            out_delay.view(-1)[-1] = (T - 1) * ts       # only the first spike sample survives
    if head:
        head_t = (torch.rand(shape[:-1], generator=gen) < 0.5).float()
    D = slayer.neuron.dynamics.delays.Delays
    od = None if out_delay is None else out_delay.to(dev()).requires_grad_(train_delay)
    d = D(input_shift=None if in_shift is None else (in_shift.to(dev()) if torch.is_tensor(in_shift) else in_shift),
          output_delay=od, output_steps=steps, output_head=None if head_t is None else head_t.to(dev()),
          sampling_time=ts, grad_scale=0.5)
    return d, (in_shift, out_delay, head_t)


def _oracle_in(x, in_shift, ts):
    return x if in_shift is None else O.shift(x, in_shift, ts)


def _oracle_out(spk, out_delay, steps, head, ts):
    if steps:
        spk = O.shift(spk, steps, 1)
        if head is not None:
            spk[..., 0] = head
    if out_delay is not None:
        spk = O.shift(spk, out_delay, ts)
    return spk


GEOMS = [((2, 5, 64), 'table', 'table', 1, True),
         ((3, 7, 100), 'table', 'table', 1, False),        # T % 32 != 0: shared lines
         ((2, 3, 4, 5, 76), 'table', 'table', 0, False),   # NCHWT, per-neuron tables
         ((2, 70, 37), 'table', 'table', 1, True),         # T % 4 != 0: dword kernel; more rows than one wave
         ((1, 130, 300), 'scalar', 'table', 1, False),
         ((2, 9, 40), None, None, 1, True),                # step_delay alone
         ((2, 9, 40), 'table', None, 0, False),            # input shift alone
         ((4, 33, 20), 'table', 'table', 2, False),        # rows shorter than a line
         ((2, 70, 301), 'table', 'table', 1, True),        # T % 4 != 0, long rows: multi-wave kernels, every tensor
         ((1, 130, 258), 'scalar', 'table', 1, False)]     # on the careful path next to the really shifted ones


# Tensors of 2^20 elements and more: the backward passes run as wave scans, with the delays folded into the scans'
# loads and stores (csrc/scan.hip); the chain's backward pass is the same scan without delays plus separate shifts,
# so the input gradients must agree bit for bit.
GEOMS_SCAN = [((4, 300, 900), 'table', 'table', 1, True),          # T % 32 != 0
              ((2, 16, 6, 7, 800), 'table', 'table', 0, False),    # NCHWT, per-neuron tables
              ((8, 450, 300), 'scalar', 'table', 1, False),        # short rows: spans of 8 rows
              ((2, 260, 2048), 'table', None, 2, False),           # rows a power of two long
              ((4, 300, 901), 'table', 'table', 1, True),          # rows that are not whole quads
              ((8, 450, 302), 'scalar', 'table', 1, False)]


def _same_gradient(a, b, what):
    """Folded against chain: bit-identical (both step by step below the scan threshold, both scans above it)."""
    assert torch.equal(a, b), what


@pytest.mark.parametrize('geom', GEOMS + GEOMS_SCAN)
@pytest.mark.parametrize('form', ['full', 'lean', 'inference'])
@pytest.mark.parametrize('graded', [False, True])
def test_cuba_fused_with_delays(slayer, geom, form, graded):
    shape, in_kind, out_kind, steps, head = geom
    gen = torch.Generator().manual_seed(seed_of('cuba-delays', geom, form, graded))
    F = slayer.neuron.dynamics.cuba_fused
    x = sparse_input(gen, shape, p=0.3, amp=1.5)
    g = torch.randn(shape, generator=gen)
    C = shape[1]
    # decays of at least 1/16: with near-integrators the reverse recurrences cancel over hundreds of steps and
    # the last-bit differences between the GPU's and the CPU's exp show up above 1e-5 of the result
    cd = torch.randint(256, 4096, (C,), generator=gen).float()
    vd = torch.randint(256, 4096, (C,), generator=gen).float()
    cs = torch.randn(shape[:-1], generator=gen)
    vs = torch.randn(shape[:-1], generator=gen) * 0.5
    w, thr, tau, rho = 64, 1.0, 1.0, 1.0
    train = form == 'full'
    d, (in_shift, out_delay, head_t) = _delays(slayer, gen, shape, in_kind, out_kind, steps, head,
                                               train_delay=(form != 'inference' and out_kind == 'table'))
    to = lambda t: t.to(dev())
    # ---- folded
    xg = to(x).requires_grad_(form != 'inference')
    cdg, vdg = to(cd).requires_grad_(train), to(vd).requires_grad_(train)
    if form == 'inference':
        cur_f, vol_f, spk_f, last_f = F.spikes(xg, cdg, vdg, to(cs), to(vs), w, thr, graded, 2, delays=d)
    else:
        cur_f, vol_f, spk_f, last_f = F.dynamics(xg, cdg, vdg, to(cs), to(vs), w, thr, tau, rho, graded, 2,
                                                 keep_current=train, delays=d)
        spk_f.backward(to(g))
    # ---- chain of separate operators on the GPU (the fused kernel without delays in the middle)
    D = slayer.neuron.dynamics.delays
    xc = to(x).requires_grad_(form != 'inference')
    cdc, vdc = to(cd).requires_grad_(train), to(vd).requires_grad_(train)
    odc = None if d.output_delay is None else d.output_delay.detach().clone().requires_grad_(d.output_delay.requires_grad)
    dc = D.Delays(d.input_shift, odc, d.output_steps, d.output_head, d.sampling_time, d.grad_scale)
    xin = D.chain_input(dc, xc)
    if form == 'inference':
        cur_c, vol_c, spk_u = F.spikes(xin, cdc, vdc, to(cs), to(vs), w, thr, graded, 2)
    else:
        cur_c, vol_c, spk_u = F.dynamics(xin, cdc, vdc, to(cs), to(vs), w, thr, tau, rho, graded, 2, keep_current=train)
    spk_c = D.chain_output(dc, spk_u)
    assert torch.equal(spk_f, spk_c), 'delayed spikes differ from the chain'
    assert torch.equal(cur_f, cur_c) and torch.equal(vol_f, vol_c)
    assert torch.equal(last_f, spk_u[..., -1]), 'last undelayed spike'
    if form != 'inference':
        spk_c.backward(to(g))
        _same_gradient(xg.grad, xc.grad, 'grad_input differs from the chain')
        if train:
            assert_rel(cdg.grad, cdc.grad.cpu(), 'grad current decay')
            assert_rel(vdg.grad, vdc.grad.cpu(), 'grad voltage decay')
        if d.output_delay is not None and d.output_delay.requires_grad:
            assert_rel(d.output_delay.grad, odc.grad.cpu(), 'grad delay')
    # ---- oracle chain
    r_in = _oracle_in(x, in_shift, 1.0)
    r_cur = O.li_fwd(r_in, cd, cs, w)
    r_vol = O.li_fwd(r_cur, vd, vs, w, thr)
    r_spk_u = O.spike_fwd(r_vol, thr, graded, 2)
    r_spk = _oracle_out(r_spk_u.clone(), out_delay, steps, head_t, 1.0)
    assert_exact(spk_f, r_spk, 'delayed spikes vs oracle')
    assert_exact(last_f, r_spk_u[..., -1], 'last spike vs oracle')
    if form == 'inference':
        assert_exact(cur_f, r_cur[..., -1], 'last current')
        assert_exact(vol_f, r_vol[..., -1], 'last voltage')
        return
    assert_exact(vol_f, r_vol, 'voltage vs oracle')
    # backward: undo the output delays, surrogate, two reverse recurrences, undo the input shift
    r_g = g
    if out_delay is not None:
        r_g, r_gd = O.delay_bwd(r_g, r_spk, out_delay, 0.5, 1.0)
    if steps:
        r_g = O.shift(r_g, -steps, 1)
    r_gv = O.spike_bwd(r_g, r_vol, thr, tau, rho, graded)
    r_gc, _ = O.li_bwd(r_gv, r_vol, vd)
    r_gx, _ = O.li_bwd(r_gc, r_cur, cd)
    if in_shift is not None:
        r_gx = O.shift(r_gx, -in_shift if torch.is_tensor(in_shift) else -in_shift, 1.0)
    (assert_scale if x.numel() >= SCAN_MIN else assert_rel)(xg.grad, r_gx, 'grad_input vs oracle')
    if d.output_delay is not None and d.output_delay.requires_grad:
        assert_rel(d.output_delay.grad, r_gd, 'grad delay vs oracle')


@pytest.mark.parametrize('geom', GEOMS[:5] + GEOMS_SCAN)
@pytest.mark.parametrize('form', ['full', 'lean', 'inference'])
def test_alif_fused_with_delays(slayer, geom, form):
    shape, in_kind, out_kind, steps, head = geom
    gen = torch.Generator().manual_seed(seed_of('alif-delays', geom, form))
    F = slayer.neuron.dynamics.alif_fused
    D = slayer.neuron.dynamics.delays
    x = sparse_input(gen, shape, p=0.4, amp=2.0)
    g = torch.randn(shape, generator=gen)
    C = shape[1]
    decays = [torch.randint(0, 4096, (C,), generator=gen).float() for _ in range(4)]
    states = [torch.randn(shape[:-1], generator=gen) * 0.3 for _ in range(2)] + \
             [torch.ones(shape[:-1]), torch.zeros(shape[:-1])]
    w, th_step, th0, tau, rho = 64, 0.5, 1.0, 1.0, 1.0
    train = form == 'full'
    d, (in_shift, out_delay, head_t) = _delays(slayer, gen, shape, in_kind, out_kind, steps, head,
                                               train_delay=(form != 'inference' and out_kind == 'table'))
    to = lambda t: t.to(dev())

    def run(delays, inp):
        ds = [to(t).requires_grad_(train and i < 2) for i, t in enumerate(decays)]
        if form == 'inference':
            return F.spikes(inp, *ds, *[to(s) for s in states], th_step, th0, w, False, 1, delays=delays), ds
        return F.dynamics(inp, *ds, *[to(s) for s in states], th_step, th0, w, tau, rho, False, 1,
                          keep_current=train, delays=delays), ds

    xg = to(x).requires_grad_(form != 'inference')
    res_f, ds_f = run(d, xg)
    xc = to(x).requires_grad_(form != 'inference')
    odc = None if d.output_delay is None else d.output_delay.detach().clone().requires_grad_(d.output_delay.requires_grad)
    dc = D.Delays(d.input_shift, odc, d.output_steps, d.output_head, d.sampling_time, d.grad_scale)
    res_c, ds_c = run(None, D.chain_input(dc, xc))
    spk_c = D.chain_output(dc, res_c[3])
    assert torch.equal(res_f[3], spk_c), 'delayed spikes differ from the chain'
    assert torch.equal(res_f[6], res_c[3][..., -1]), 'last undelayed spike'
    for i in (0, 1, 4, 5):
        assert torch.equal(res_f[i], res_c[i]), f'result {i}'
    assert float(res_c[3].detach().sum()) > 0
    if form != 'inference':
        res_f[3].backward(to(g))
        spk_c.backward(to(g))
        _same_gradient(xg.grad, xc.grad, 'grad_input differs from the chain')
        if train:
            for a, b in zip(ds_f[:2], ds_c[:2]):
                assert_rel(a.grad, b.grad.cpu(), 'decay gradient')
        if d.output_delay is not None and d.output_delay.requires_grad:
            assert_rel(d.output_delay.grad, odc.grad.cpu(), 'grad delay')
    # oracle chain, forward
    r_in = _oracle_in(x, in_shift, 1.0)
    r_cur = O.li_fwd(r_in, decays[0], states[0], w)
    r_vol = O.li_fwd(r_cur, decays[1], states[1], w)
    r_th, r_ref = O.ath_fwd(r_vol, states[3], decays[3], states[2], decays[2], th_step, th0, w)
    r_spk_u = O.spike_fwd(r_vol, r_th + r_ref)
    assert_exact(res_f[3], _oracle_out(r_spk_u.clone(), out_delay, steps, head_t, 1.0), 'delayed spikes vs oracle')
    assert_exact(res_f[6], r_spk_u[..., -1], 'last spike vs oracle')


@pytest.mark.parametrize('geom', GEOMS[:5] + GEOMS_SCAN)
@pytest.mark.parametrize('form', ['train', 'plain', 'inference'])
def test_rf_fused_with_delays(slayer, geom, form):
    shape, in_kind, out_kind, steps, head = geom
    gen = torch.Generator().manual_seed(seed_of('rf-delays', geom, form))
    F = slayer.neuron.dynamics.rf_fused
    D = slayer.neuron.dynamics.delays
    xr = sparse_input(gen, shape, p=0.3, amp=0.6)
    xi = sparse_input(gen, shape, p=0.3, amp=0.6)
    g = torch.randn(shape, generator=gen)
    C = shape[1]
    decay = torch.randint(100, 600, (C,), generator=gen).float()
    phi = 2 * 3.141592653589793 / (5 + 15 * torch.rand(C, generator=gen))
    sin_d = torch.round((4096 - decay) * torch.sin(phi)).clamp(min=1)
    cos_d = torch.round((4096 - decay) * torch.cos(phi)).clamp(min=0)
    rs = torch.randn(shape[:-1], generator=gen) * 0.2
    is_ = torch.randn(shape[:-1], generator=gen) * 0.2
    w, thr, tau, rho = 64, 0.3, 0.5, 10.0
    train = form == 'train'
    d, (in_shift, out_delay, head_t) = _delays(slayer, gen, shape, in_kind, out_kind, steps, head,
                                               train_delay=(form != 'inference' and out_kind == 'table'))
    to = lambda t: t.to(dev())

    def run(delays, a, b):
        sd, cdd = to(sin_d).requires_grad_(train), to(cos_d).requires_grad_(train)
        if form == 'inference':
            return F.spikes(a, b, sd, cdd, to(rs), to(is_), to(is_), w, thr, False, 1, delays=delays), (sd, cdd)
        return F.dynamics(a, b, sd, cdd, to(rs), to(is_), to(is_), w, thr, tau, rho, False, 1, delays=delays), (sd, cdd)

    ag, bg = to(xr).requires_grad_(form != 'inference'), to(xi).requires_grad_(form != 'inference')
    res_f, p_f = run(d, ag, bg)
    ac, bc = to(xr).requires_grad_(form != 'inference'), to(xi).requires_grad_(form != 'inference')
    odc = None if d.output_delay is None else d.output_delay.detach().clone().requires_grad_(d.output_delay.requires_grad)
    dc = D.Delays(d.input_shift, odc, d.output_steps, d.output_head, d.sampling_time, d.grad_scale)
    res_c, p_c = run(None, D.chain_input(dc, ac), D.chain_input(dc, bc))
    spk_c = D.chain_output(dc, res_c[2])
    assert torch.equal(res_f[2], spk_c), 'delayed spikes differ from the chain'
    assert torch.equal(res_f[3], res_c[2][..., -1]), 'last undelayed spike'
    assert torch.equal(res_f[0], res_c[0]) and torch.equal(res_f[1], res_c[1])
    assert float(res_c[2].detach().sum()) > 0
    if form != 'inference':
        res_f[2].backward(to(g))
        spk_c.backward(to(g))
        assert torch.equal(ag.grad, ac.grad) and torch.equal(bg.grad, bc.grad), 'input gradients differ from the chain'
        if train:
            for a, b in zip(p_f, p_c):
                assert_rel(a.grad, b.grad.cpu(), 'decay gradient')
        if d.output_delay is not None and d.output_delay.requires_grad:
            assert_rel(d.output_delay.grad, odc.grad.cpu(), 'grad delay')
    r_re, r_im = O.res_fwd(_oracle_in(xr, in_shift, 1.0), _oracle_in(xi, in_shift, 1.0), sin_d, cos_d, rs, is_, w)
    r_spk_u = O.cspike_fwd(r_re, r_im, thr, is_)
    assert_exact(res_f[2], _oracle_out(r_spk_u.clone(), out_delay, steps, head_t, 1.0), 'delayed spikes vs oracle')
    assert_exact(res_f[3], r_spk_u[..., -1], 'last spike vs oracle')


# More workgroups than the chip holds at once (131 072 rows): the multi-wave kernels then run in several rounds, held
# to a few workgroups per compute unit, with the delays folded in.
GEOM_ROUNDS = ((32, 4096, 128), 'table', 'table', 1, True)


@pytest.mark.parametrize('form', ['full', 'lean'])
def test_cuba_fused_with_delays_in_several_rounds(slayer, form):
    test_cuba_fused_with_delays(slayer, GEOM_ROUNDS, form, False)


def test_alif_fused_with_delays_in_several_rounds(slayer):
    test_alif_fused_with_delays(slayer, GEOM_ROUNDS, 'full')


def test_rf_fused_with_delays_in_several_rounds(slayer):
    test_rf_fused_with_delays(slayer, GEOM_ROUNDS, 'train')


class _Block:
    """What block.neuron_delay needs of a block: neuron, delay_shift, delay (and its own delay_buffer)."""

    def __init__(self, neuron, delay_shift, delay):
        self.neuron, self.delay_shift, self.delay = neuron, delay_shift, delay


@pytest.mark.parametrize('kind', ['cuba', 'alif', 'rf'])
@pytest.mark.parametrize('persistent', [False, True])
@pytest.mark.parametrize('with_delay', [False, True])
def test_block_tail_fused_equals_unfused_over_several_calls(slayer, kind, persistent, with_delay):
    """neuron -> step_delay -> Delay as a block runs it, fused and with the separate operators: same spikes
    call after call (carried neuron state and step_delay buffer), same input and delay gradients."""
    gen = torch.Generator().manual_seed(seed_of('block-tail', kind, persistent, with_delay))
    shape = (3, 8, 6, 90) if kind != 'rf' else (3, 8, 90)
    torch.manual_seed(11)

    def make():
        if kind == 'cuba':
            n = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03, persistent_state=persistent)
        elif kind == 'alif':
            n = slayer.neuron.alif.Neuron(1.0, 0.5, 0.25, 0.1, 0.05, 0.2, persistent_state=persistent)
        else:
            n = slayer.neuron.rf.Neuron(1.0, 11, 0.05, persistent_state=persistent)
        dl = slayer.axon.Delay(max_delay=40) if with_delay else None
        return _Block(n.to(dev()), True, None if dl is None else dl.to(dev()))

    fused_b, plain_b = make(), make()
    calls = []
    for i in range(3):
        if kind == 'rf':
            z = tuple(sparse_input(gen, shape, p=0.3, amp=2.0).to(dev()) for _ in range(2))
        else:
            z = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
        calls.append(z)
    g = torch.randn(shape, generator=gen).to(dev())
    for i, z in enumerate(calls):
        zf = tuple(t.clone().requires_grad_() for t in z) if kind == 'rf' else z.clone().requires_grad_()
        zp = tuple(t.clone().requires_grad_() for t in z) if kind == 'rf' else z.clone().requires_grad_()
        if with_delay and i == 0:
            like = z[0] if kind == 'rf' else z
            plain_b.delay.per_neuron(like)
            plain_b.delay.delay.data = torch.rand(shape[1], generator=gen).to(dev()) * 30
            fused_b.delay.per_neuron(like)
            fused_b.delay.delay.data = plain_b.delay.delay.data.clone()
        xf = slayer.block.neuron_delay(fused_b, zf, fused=True)
        xp = slayer.block.neuron_delay(plain_b, zp, fused=False)
        assert torch.equal(xf, xp), f'{kind}: call {i} differs'
        assert float(xp.detach().sum()) > 0
        xf.backward(g)
        xp.backward(g)
        for a, b in zip(zf if kind == 'rf' else (zf,), zp if kind == 'rf' else (zp,)):
            assert torch.equal(a.grad, b.grad), f'{kind}: input gradient of call {i} differs'
        if with_delay:
            assert_rel(fused_b.delay.delay.grad, plain_b.delay.delay.grad.cpu(), 'delay gradient')
            fused_b.delay.delay.grad = None
            plain_b.delay.delay.grad = None
        if persistent:
            assert torch.equal(fused_b.delay_buffer, plain_b.delay_buffer)
            # step_delay keeps a slice of the previous output, graph and all (as the reference does); cut it
            # loose, or the next call's backward pass would walk into this call's freed graph
            plain_b.delay_buffer = plain_b.delay_buffer.detach()


def test_debug_neuron_takes_the_cross_checked_operators(slayer):
    """debug=True routes forward through dynamics() + spike(), whose kernels are cross-checked."""
    gen = torch.Generator().manual_seed(5)
    x = sparse_input(gen, (2, 6, 60), p=0.3).to(dev())
    n = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03).to(dev())
    ref = n(x)
    n.debug = True
    assert torch.equal(n(x), ref)


def test_fused_cuba_with_delays_at_synapse_workload_size(slayer):
    """[32, 256, 1500] with per-channel shifts U[0, 32): folded kernels vs the chain on the whole tensor, and
    slabs of rows against the oracle."""
    gen = torch.Generator().manual_seed(1004)
    shape = (32, 256, 1500)
    F = slayer.neuron.dynamics.cuba_fused
    D = slayer.neuron.dynamics.delays
    x = sparse_input(gen, shape, p=0.03, amp=4.0)
    g = torch.randn(shape, generator=gen)
    in_shift = torch.rand(256, generator=gen) * 32
    out_delay = torch.rand(256, generator=gen) * 32
    cd, vd, zero = torch.tensor([1024.0]), torch.tensor([128.0]), torch.tensor([0.0])
    w, thr = 64, 1.25
    to = lambda t: t.to(dev())
    d = D.Delays(to(in_shift), to(out_delay).requires_grad_(), 1, None, 1, 1)
    xg = to(x).requires_grad_()
    cur, vol, spk, last = F.dynamics(xg, to(cd), to(vd), to(zero), to(zero), w, thr, 1.0, 1.0, False, 1,
                                     keep_current=False, delays=d)
    spk.backward(to(g))
    dc = D.Delays(to(in_shift), to(out_delay).requires_grad_(), 1, None, 1, 1)
    xc = to(x).requires_grad_()
    _, vol_c, spk_u = F.dynamics(D.chain_input(dc, xc), to(cd), to(vd), to(zero), to(zero), w, thr, 1.0, 1.0, False, 1,
                                 keep_current=False)
    spk_c = D.chain_output(dc, spk_u)
    spk_c.backward(to(g))
    assert torch.equal(spk, spk_c) and torch.equal(vol, vol_c)
    assert torch.equal(xg.grad, xc.grad), 'grad_input'
    assert_rel(d.output_delay.grad, dc.output_delay.grad.cpu(), 'grad delay')
    assert float(spk_u.detach().sum()) > 1000
    for b in (0, 17, 31):
        sl = slice(96, 128)
        xs = x[b:b + 1, sl]
        r_in = O.shift(xs, in_shift[sl], 1)
        r_cur = O.li_fwd(r_in, cd, zero, w)
        r_vol = O.li_fwd(r_cur, vd, zero, w, thr)
        r_spk = O.shift(O.shift(O.spike_fwd(r_vol, thr), 1, 1), out_delay[sl], 1)
        assert_exact(spk[b:b + 1, sl], r_spk, f'slab {b} spikes')
        assert_exact(vol[b:b + 1, sl], r_vol, f'slab {b} voltage')
        r_g = O.shift(O.shift(g[b:b + 1, sl], -out_delay[sl], 1), -1, 1)
        r_gv = O.spike_bwd(r_g, r_vol, thr, 1.0, 1.0)
        r_gc, _ = O.li_bwd(r_gv, r_vol, vd)
        r_gx, _ = O.li_bwd(r_gc, r_cur, cd)
        assert_rel(xg.grad[b:b + 1, sl], O.shift(r_gx, -in_shift[sl], 1), f'slab {b} grad_input')


def test_delay_parts_of_opposite_sign_move_the_spikes_by_their_sum(slayer):
    """``output_steps`` and a negative ``output_delay`` add up to one shift in the fused kernels; the separate
    operators (debug, dropout or norm) must not drop the samples that two shifts in a row would push off the
    row in between: the same ``Neuron.forward(delays=...)`` gives the same spikes either way."""
    D = slayer.neuron.dynamics.delays
    gen = torch.Generator().manual_seed(11)
    x = sparse_input(gen, (2, 6, 64), p=0.4).to(dev())
    table = torch.tensor([-1.0, 0.0, -2.0, 1.0, -1.0, 3.0])
    n = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03).to(dev())
    plain = n(x)
    assert float(plain[..., -1].abs().sum()) > 0 or float(plain[..., -2].abs().sum()) > 0
    fused = n(x, delays=D.Delays(output_delay=table, output_steps=1))
    n.debug = True
    chain = n(x, delays=D.Delays(output_delay=table, output_steps=1))
    assert torch.equal(fused, chain)
    # rows whose parts cancel are the undelayed spikes, last sample included
    assert torch.equal(fused[:, 0], plain[:, 0]) and torch.equal(fused[:, 4], plain[:, 4])
    assert torch.equal(fused[:, 2, :-1], plain[:, 2, 1:])
    with pytest.raises(RuntimeError):
        D.Delays(output_steps=-1)
    with pytest.raises(RuntimeError):
        D.chain_output(D.Delays(output_delay=table.to(dev()).requires_grad_(), output_steps=1), plain)


@pytest.mark.parametrize('shape,ts,steps', [((4, 300, 900), 1.0, 1), ((8, 450, 300), 0.5, 0), ((2, 16, 6, 7, 800), 1.0, 2),
                                            ((4, 300, 901), 1.0, 1), ((2, 260, 2048), 2.0, 0)])
@pytest.mark.parametrize('kind', ['cuba', 'alif', 'rf'])
def test_delay_gradient_from_the_backward_scan(slayer, shape, ts, steps, kind):
    """The gradient of a learnable spike delay (axon/delay.py:201-221 in the reference: sum over batch and time of
    grad[t] * (out[t-1] - out[t]) / Ts on the delayed spikes) comes out of the fused backward scan, which reads the
    gradient through the delay anyway.  Against float64 sums of the same terms (1e-5 of the sum of their
    magnitudes) and against the stand-alone kernel, for delays of either sign, zero, beyond the row length, with and
    without the sample a step delay carries over."""
    from lava_dl_amd.slayer import _native as N
    D = slayer.neuron.dynamics.delays
    gen = torch.Generator().manual_seed(seed_of('delay-grad-scan', shape, ts, steps, kind))
    T = shape[-1]
    npb = 1
    for s in shape[1:-1]:
        npb *= s
    table = (torch.rand(npb, generator=gen) * 40 - 8) * ts            # mostly delays, some advances
    table[0], table[1], table[2], table[3] = 0.0, (T + 5) * ts, -(T + 2) * ts, (T - 1) * ts
    table[4] = -0.4 * ts                                              # truncates to zero
    total = steps + torch.trunc(table / ts)                           # steps of every neuron
    spikes = (torch.rand(shape, generator=gen) < 0.2).float() * (1 + torch.rand(shape, generator=gen))
    delayed = slayer.utils.time.shift(spikes.to(dev()), total.to(dev()), 1)
    if steps == 1:                                                    # the sample before the first one
        head = torch.rand(shape[:-1], generator=gen)
        rows = delayed.reshape(-1, T)
        k = total.repeat(shape[0]).long()
        at = (k - 1).clamp(0, T - 1)
        ok = ((k >= 1) & (k - 1 < T)).to(dev())
        rows[torch.arange(rows.shape[0], device=dev())[ok], at.to(dev())[ok]] = head.reshape(-1).to(dev())[ok]
    g = torch.randn(shape, generator=gen).to(dev())
    vol = (torch.randn(shape, generator=gen) * 1.5).to(dev())
    aux = torch.randn(shape, generator=gen).to(dev())
    C = shape[1]
    d1 = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    d2 = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    delays = D.Delays(output_delay=table.to(dev()).requires_grad_(), output_steps=steps, sampling_time=ts)
    folded = D.fold(delays, g, forward=False, delayed_spikes=delayed)
    F = slayer.neuron.dynamics
    # the gradient as the neuron sees it, by a separate shift (delays of either sign): the folded pass gives the
    # same input gradient bit for bit
    g_back = slayer.utils.time.shift(g, -total.to(dev()), 1)
    if kind == 'cuba':
        res = F.cuba_fused._bwd(g, vol, aux, d1, d2, 1.0, 0.7, 1.3, False, True, folded)
        ref_in = F.cuba_fused._bwd(g_back, vol, aux, d1, d2, 1.0, 0.7, 1.3, False, True)
    elif kind == 'alif':
        res = F.alif_fused._bwd(g, vol, 1 + aux.abs(), aux, d1, d2, 0.7, 1.3, False, True, folded)
        ref_in = F.alif_fused._bwd(g_back, vol, 1 + aux.abs(), aux, d1, d2, 0.7, 1.3, False, True)
    else:
        sin, cos = ((4096 - d1.clamp(40, 4095)) * 0.6).round(), ((4096 - d1.clamp(40, 4095)) * 0.8).round()
        res = F.rf_fused._bwd(g, vol, aux, sin, cos, 1.0, 0.7, 1.3, False, True, folded)
        ref_in = F.rf_fused._bwd(g_back, vol, aux, sin, cos, 1.0, 0.7, 1.3, False, True)
        assert torch.equal(res[1], ref_in[1]), 'imaginary input gradient with the delay folded in'
    assert torch.equal(res[0], ref_in[0]), 'input gradient with the delay folded in'
    got = folded.grad_sum
    # float64 sums of the same terms
    gd, od = g.double().cpu(), delayed.double().cpu()
    prev = torch.cat([torch.zeros_like(od[..., :1]), od[..., :-1]], -1)
    terms = (gd * (prev - od) / ts).reshape(shape[0], npb, T)
    assert_sum(got, terms.sum(dim=(0, 2)), terms.abs().sum(dim=(0, 2)), f'{kind} delay gradient from the scan')
    # the stand-alone kernel on the same tensors
    M = shape[0] * npb
    ref = torch.empty(npb, device=dev())
    ws = torch.empty(M + 64 * npb, device=dev())
    N.check(N.lib().slayer_delay_bwd(None, N.ptr(ref), N.ptr(g), N.ptr(delayed), None, 0, float(ts), N.ptr(ws), M, npb, T,
                                     N.stream_handle()))
    assert_sum(ref, terms.sum(dim=(0, 2)), terms.abs().sum(dim=(0, 2)), 'stand-alone kernel')
