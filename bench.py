"""Benchmark of the SLAYER neuron-dynamics hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cuba|cuba_fused|cuba_fused_lean|cuba_inference|cuba_fwd_small|alif|alif_fused|alif_fused_lean|rf|rf_fused|rf_fused_lean|rf_inference|synapse|synapse_fused|synapse_folded|synapse_delay_grad|dense_synapse]

A step is one pass of the workload's op sequence over one batch of synthetic input that is already
resident in HBM (outputs come from torch's caching allocator inside the timed region).  The default
workload is the CUBA conv-layer neuron tensor [32,16,32,32,300], forward + backward
(LI, LI+threshold, Spike; Spike bwd, LI bwd, LI bwd) -- the configuration the headline metric is
quoted on.  The other workloads are the remaining benchmark configurations; they exist for
profiling and parity at full size, the default run prints ONE JSON line for `cuba`:
whole-job neuron-timesteps/s, per-kernel roofline and the CPU baseline (the torch-CPU oracle
timed on this box's host cores).
"""
import argparse
import gc
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

def _events(gen, shape, p, amp=1.0):
    return (torch.rand(shape, generator=gen) < p).float() * torch.randn(shape, generator=gen) * amp


class _Null:
    def __enter__(self):
        return self

    def __exit__(self, *a):
        return False


class _Section:
    def __init__(self, timers, name):
        self.timers, self.name = timers, name

    def __enter__(self):
        self.a = torch.cuda.Event(enable_timing=True)
        self.b = torch.cuda.Event(enable_timing=True)
        self.a.record()
        return self

    def __exit__(self, *exc):
        self.b.record()
        self.timers.events.setdefault(self.name, []).append((self.a, self.b))
        return False


class Timers:
    """Per-op device time from events recorded on the stream the kernels are launched on
    (torch's current stream)."""

    def __init__(self):
        self.events = {}

    def section(self, name):
        return _Section(self, name)

    def median_ms(self):
        """Median over the passes: an interval between two events also contains whatever kept the host from
        launching in time (an allocator or interpreter pause shows up as tens of milliseconds in one pass)."""
        out = {}
        for k, v in self.events.items():
            times = sorted(a.elapsed_time(b) for a, b in v)
            n = len(times)
            out[k] = times[n // 2] if n % 2 else 0.5 * (times[n // 2 - 1] + times[n // 2])
        return out


class Workload:
    """ops: (name, kernel, algorithmic bytes per neuron-timestep = 4 B x tensors read + written)."""
    name = ''
    shape = ()
    ops = []

    def __init__(self, dev, seed):
        from lava_dl_amd.slayer.neuron.dynamics import leaky_integrator, adaptive_threshold, resonator
        from lava_dl_amd.slayer.spike import spike, complex
        import importlib
        from lava_dl_amd.slayer.utils.time import shift
        self.L, self.A, self.R, self.S, self.CS = leaky_integrator, adaptive_threshold, resonator, spike, complex
        self.shift = shift
        self.conv = importlib.import_module('lava_dl_amd.slayer.utils.filter.conv')   # module with fwd / bwd
        self.dev = dev
        self.gen = torch.Generator().manual_seed(seed)
        self.cpu = {}
        self.zero = torch.zeros(1, device=dev)
        self.one = torch.ones(1, device=dev)

    def put(self, **tensors):
        for k, v in tensors.items():
            self.cpu[k] = v
            setattr(self, k, v.to(self.dev))

    @property
    def nt(self):
        return math.prod(self.shape)

    def bytes_per_nt(self):
        return sum(b for _, _, b in self.ops)


class Cuba(Workload):
    name = 'CUBA conv-layer neuron tensor fwd+bwd'
    shape = (32, 16, 32, 32, 300)
    ops = [('li_fwd_current', 'stream_kernel_duo<LiFwd>', 8), ('li_fwd_voltage', 'stream_kernel_duo<LiFwd>', 8),
           ('spike_fwd', 'spike_fwd_kernel', 8), ('spike_bwd', 'spike_bwd_kernel', 12),
           ('li_bwd_voltage', 'li_bwd_scan_kernel', 12), ('li_bwd_current', 'li_bwd_scan_kernel', 12)]
    w, thr = 64, 1.0
    note = 'w_scale=64, per-channel decays uniform over [0,4096), threshold 1.0, input Bernoulli(0.02) x N(0,0.5)'

    def __init__(self, dev):
        super().__init__(dev, 1001)
        g = self.gen
        self.put(x=_events(g, self.shape, 0.02, 0.5),
                 d_i=torch.randint(0, 4096, (self.shape[1],), generator=g).float(),
                 d_v=torch.randint(0, 4096, (self.shape[1],), generator=g).float(),
                 g=torch.randn(self.shape, generator=g))

    def step(self, t):
        L, S = self.L, self.S
        with t('li_fwd_current'):
            cur = L._fwd(self.x, self.d_i, self.zero, -1, self.w)
        with t('li_fwd_voltage'):
            vol = L._fwd(cur, self.d_v, self.zero, self.thr, self.w)
        with t('spike_fwd'):
            spk = S._fwd(vol, None, self.thr, False, 1)
        with t('spike_bwd'):
            g_vol = S._bwd(self.g, vol, None, self.thr, 1.0, 1.0, False)
        with t('li_bwd_voltage'):
            g_cur, gd_v = L._bwd(g_vol, vol, self.d_v)
        with t('li_bwd_current'):
            g_x, gd_i = L._bwd(g_cur, cur, self.d_i)
        return spk, g_x, gd_v, gd_i

    def kernel_only(self, op):
        """A launch of the op's main kernel alone (the leaky-integrator backward op is that kernel plus two small
        reduction launches for the decay gradient), for the roofline entry."""
        if op not in ('li_bwd_voltage', 'li_bwd_current'):
            return None
        L = self.L
        cur = L._fwd(self.x, self.d_i, self.zero, -1, self.w)
        if op == 'li_bwd_current':
            return lambda: L._bwd(self.g, cur, self.d_i, False, True)
        vol = L._fwd(cur, self.d_v, self.zero, self.thr, self.w)
        return lambda: L._bwd(self.g, vol, self.d_v, False, True)

    def cpu_step(self, n, sl=None):
        """The oracle on batch[:n] (channels `sl` when given); returns (spikes, grad of the input)."""
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        x, g, d_i, d_v = c['x'][:n], c['g'][:n], c['d_i'], c['d_v']
        if sl is not None:
            x, g, d_i, d_v = x[:, sl], g[:, sl], d_i[sl], d_v[sl]
        cur = O.li_fwd(x, d_i, zero, self.w)
        vol = O.li_fwd(cur, d_v, zero, self.w, self.thr)
        spk = O.spike_fwd(vol, self.thr)
        g_vol = O.spike_bwd(g, vol, self.thr, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, d_v)
        g_x, _ = O.li_bwd(g_cur, cur, d_i)
        return spk, g_x

    parity_slab = (1, slice(3, 5))      # batch[:1], two channels


class CubaFused(Cuba):
    """Same tensor and parameters as `cuba`, run through the fused kernels: the intermediates are written
    (autograd needs them) but never re-read by a separate operator.  Reported against its own byte count."""
    name = 'CUBA conv-layer neuron tensor fwd+bwd, fused kernels'
    ops = [('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 16), ('cuba_bwd', 'cuba_bwd_scan_kernel', 16)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
        self.F = cuba_fused

    def step(self, t):
        with t('cuba_fwd'):
            cur, vol, spk = self.F._fwd(self.x, self.d_i, self.d_v, self.zero, self.zero, self.w, self.thr, False, 1)
        with t('cuba_bwd'):
            g_x, gd_i, gd_v = self.F._bwd(self.g, vol, cur, self.d_i, self.d_v, self.thr, 1.0, 1.0, False)
        return spk, g_x, gd_v, gd_i


class CubaFusedLean(Cuba):
    name = 'CUBA neuron fwd+bwd, fused kernels without the current trace (no decay gradients)'
    ops = [('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 12), ('cuba_bwd', 'cuba_bwd_scan_kernel', 12)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
        self.F = cuba_fused

    def step(self, t):
        with t('cuba_fwd'):
            _, vol, spk = self.F._fwd(self.x, self.d_i, self.d_v, self.zero, self.zero, self.w, self.thr, False, 1, True)
        with t('cuba_bwd'):
            g_x, _, _ = self.F._bwd(self.g, vol, None, self.d_i, self.d_v, self.thr, 1.0, 1.0, False, False)
        return spk, g_x


class CubaInference(Cuba):
    name = 'CUBA neuron forward, spikes only (inference)'
    ops = [('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 8)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
        self.F = cuba_fused

    def step(self, t):
        with t('cuba_fwd'):
            out = self.F._fwd(self.x, self.d_i, self.d_v, self.zero, self.zero, self.w, self.thr, False, 1, True, True)
        return out


class CubaFwdSmall(Workload):
    name = 'CUBA LIF dynamics forward only (latency-bound: 512 neurons)'
    shape = (4, 128, 200)
    ops = [('li_fwd_current', 'stream_kernel_duo<LiFwd>', 8), ('li_fwd_voltage', 'stream_kernel_duo<LiFwd>', 8)]
    note = 'w_scale=64, scalar decays 1024 / 128, threshold 1.25, input Bernoulli(0.05) x N(0,1)'

    def __init__(self, dev):
        super().__init__(dev, 1000)
        self.put(x=_events(self.gen, self.shape, 0.05), d_i=torch.tensor([1024.0]), d_v=torch.tensor([128.0]))

    def step(self, t):
        with t('li_fwd_current'):
            cur = self.L._fwd(self.x, self.d_i, self.zero, -1, 64)
        with t('li_fwd_voltage'):
            vol = self.L._fwd(cur, self.d_v, self.zero, 1.25, 64)
        return vol

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        x = c['x'][:n] if sl is None else c['x'][:n, sl]
        return O.li_fwd(O.li_fwd(x, c['d_i'], zero, 64), c['d_v'], zero, 64, 1.25), None

    parity_slab = (4, slice(0, 128))    # the whole tensor


class Alif(Workload):
    name = 'ALIF adaptive-threshold dynamics fwd+bwd'
    shape = (64, 512, 1000)
    ops = [('li_fwd_current', 'stream_kernel_duo<LiFwd>', 8), ('li_fwd_voltage', 'stream_kernel_duo<LiFwd>', 8),
           ('ath_fwd', 'stream_kernel_duo<AthFwd>', 12), ('threshold_add', 'torch add (outside the API)', 12),
           ('spike_fwd', 'spike_fwd_kernel', 12), ('spike_bwd', 'spike_bwd_kernel', 16),
           ('li_bwd_voltage', 'li_bwd_scan_kernel', 12), ('li_bwd_current', 'li_bwd_scan_kernel', 12)]
    note = 'w_scale=64, four per-channel decay vectors uniform over [0,4096), th0 1.0, step 0.5'

    def __init__(self, dev):
        super().__init__(dev, 1002)
        g = self.gen
        C = self.shape[1]
        self.put(x=_events(g, self.shape, 0.05), g=torch.randn(self.shape, generator=g),
                 **{k: torch.randint(0, 4096, (C,), generator=g).float() for k in ('d_i', 'd_v', 'd_th', 'd_ref')})

    def step(self, t):
        L, A, S = self.L, self.A, self.S
        with t('li_fwd_current'):
            cur = L._fwd(self.x, self.d_i, self.zero, -1, 64)
        with t('li_fwd_voltage'):
            vol = L._fwd(cur, self.d_v, self.zero, -1, 64)
        with t('ath_fwd'):
            th, ref = A._fwd(vol, self.zero, self.d_ref, self.one, self.d_th, 0.5, 1.0, 64)
        with t('threshold_add'):
            theta = th + ref
        with t('spike_fwd'):
            spk = S._fwd(vol, theta, 0.0, False, 1)
        with t('spike_bwd'):
            g_vol = S._bwd(self.g, vol, theta, 0.0, 1.0, 1.0, False)
        with t('li_bwd_voltage'):
            g_cur, _ = L._bwd(g_vol, vol, self.d_v)
        with t('li_bwd_current'):
            g_x, _ = L._bwd(g_cur, cur, self.d_i)
        return spk, g_x

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero, one = self.cpu, torch.tensor([0.0]), torch.tensor([1.0])
        x, g = c['x'][:n], c['g'][:n]
        d_i, d_v, d_ref, d_th = c['d_i'], c['d_v'], c['d_ref'], c['d_th']
        if sl is not None:
            x, g, d_i, d_v, d_ref, d_th = x[:, sl], g[:, sl], d_i[sl], d_v[sl], d_ref[sl], d_th[sl]
        cur = O.li_fwd(x, d_i, zero, 64)
        vol = O.li_fwd(cur, d_v, zero, 64)
        th, ref = O.ath_fwd(vol, zero, d_ref, one, d_th, 0.5, 1.0, 64)
        theta = th + ref
        spk = O.spike_fwd(vol, theta)
        g_vol = O.spike_bwd(g, vol, theta, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, d_v)
        g_x, _ = O.li_bwd(g_cur, cur, d_i)
        return spk, g_x

    parity_slab = (1, slice(100, 132))


class AlifFused(Alif):
    name = 'ALIF adaptive-threshold dynamics fwd+bwd, fused kernels'
    ops = [('alif_fwd', 'stream_kernel_duo<AlifFwd>', 20), ('alif_bwd', 'cuba_bwd_scan_kernel<THETA>', 20)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import alif_fused
        self.F = alif_fused

    def step(self, t):
        with t('alif_fwd'):
            cur, vol, theta, spk, _, _ = self.F._fwd(
                self.x, (self.d_i, self.d_v, self.d_th, self.d_ref), (self.zero, self.zero, self.one, self.zero),
                0.5, 1.0, 64, False, 1)
        with t('alif_bwd'):
            g_x = self.F._bwd(self.g, vol, theta, cur, self.d_i, self.d_v, 1.0, 1.0, False)
        return spk, g_x


class AlifFusedLean(Alif):
    name = 'ALIF fwd+bwd, fused kernels without the current trace (no decay gradients)'
    ops = [('alif_fwd', 'stream_kernel_duo<AlifFwd>', 16), ('alif_bwd', 'cuba_bwd_scan_kernel<THETA>', 16)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import alif_fused
        self.F = alif_fused

    def step(self, t):
        with t('alif_fwd'):
            _, vol, theta, spk, _, _ = self.F._fwd(
                self.x, (self.d_i, self.d_v, self.d_th, self.d_ref), (self.zero, self.zero, self.one, self.zero),
                0.5, 1.0, 64, False, 1, True, True)
        with t('alif_bwd'):
            g_x = self.F._bwd(self.g, vol, theta, None, self.d_i, self.d_v, 1.0, 1.0, False, False)
        return spk, g_x


class Rf(Workload):
    name = 'Resonator (RF) dynamics fwd+bwd'
    shape = (64, 1024, 2000)
    ops = [('res_fwd', 'stream_kernel_duo<ResFwd>', 16), ('cspike_fwd', 'cspike_fwd_kernel', 12),
           ('cspike_bwd', 'cspike_bwd_kernel', 20), ('res_bwd', 'res_bwd_scan_kernel', 24)]
    note = 'w_scale=64, per-channel decay uniform over [0,4096), frequency uniform over [5,50] Hz at 1 ms'

    def __init__(self, dev):
        super().__init__(dev, 1003)
        g = self.gen
        C = self.shape[1]
        decay = torch.randint(0, 4096, (C,), generator=g).float()
        phi = 2 * math.pi * (5 + 45 * torch.rand(C, generator=g)) * 1e-3
        sin, cos = ((4096 - decay) * torch.sin(phi)).round(), ((4096 - decay) * torch.cos(phi)).round()
        gain = torch.sqrt(sin ** 2 + cos ** 2)                       # the RF neuron's parameter clamp
        ratio = gain.clamp(0, 4095) / gain.clamp_min(1e-9)
        sin, cos = (sin * ratio).round().clamp_min(1), (cos * ratio).round().clamp_min(0)
        self.put(xr=_events(g, self.shape, 0.1, 0.3), xi=_events(g, self.shape, 0.1, 0.3), sin=sin, cos=cos,
                 g=torch.randn(self.shape, generator=g))

    def step(self, t):
        R, CS = self.R, self.CS
        with t('res_fwd'):
            re, im = R._fwd(self.xr, self.xi, self.sin, self.cos, self.zero, self.zero, -1, 64)
        with t('cspike_fwd'):
            spk = CS._fwd(re, im, None, 1.0, None, 0.0, False, 1)
        with t('cspike_bwd'):
            g_re, g_im = CS._bwd(self.g, re, im, None, 1.0, 0.5, 10.0, False)
        with t('res_bwd'):
            out = R._bwd(g_re, g_im, re, im, self.sin, self.cos)
        return spk, out

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        xr, xi, g, sin, cos = c['xr'][:n], c['xi'][:n], c['g'][:n], c['sin'], c['cos']
        if sl is not None:
            xr, xi, g, sin, cos = xr[:, sl], xi[:, sl], g[:, sl], sin[sl], cos[sl]
        re, im = O.res_fwd(xr, xi, sin, cos, zero, zero, 64)
        spk = O.cspike_fwd(re, im, 1.0, 0.0)
        g_re, g_im = O.cspike_bwd(g, re, im, 1.0, 0.5, 10.0)
        out = O.res_bwd(g_re, g_im, re, im, sin, cos)
        return spk, out[0]

    parity_slab = (1, slice(500, 516))


class RfFused(Rf):
    name = 'Resonator (RF) dynamics fwd+bwd, fused kernels'
    ops = [('rf_fwd', 'stream_kernel_duo<RfFwd>', 20), ('rf_bwd', 'res_bwd_scan_kernel<SURR>', 20)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import rf_fused
        self.F = rf_fused

    def step(self, t):
        with t('rf_fwd'):
            re, im, spk = self.F._fwd(self.xr, self.xi, self.sin, self.cos, self.zero, self.zero, self.zero, 64,
                                      1.0, False, 1)
        with t('rf_bwd'):
            out = self.F._bwd(self.g, re, im, self.sin, self.cos, 1.0, 0.5, 10.0, False)
        return spk, out


class RfFusedLean(RfFused):
    name = 'Resonator (RF) dynamics fwd+bwd, fused kernels, no decay gradients'

    def step(self, t):
        with t('rf_fwd'):
            re, im, spk = self.F._fwd(self.xr, self.xi, self.sin, self.cos, self.zero, self.zero, self.zero, 64,
                                      1.0, False, 1)
        with t('rf_bwd'):
            out = self.F._bwd(self.g, re, im, self.sin, self.cos, 1.0, 0.5, 10.0, False, False)
        return spk, out


class RfInference(Rf):
    name = 'Resonator (RF) neuron forward, spikes only (inference)'
    ops = [('rf_fwd', 'stream_kernel_duo<RfFwd>', 12)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import rf_fused
        self.F = rf_fused

    def step(self, t):
        with t('rf_fwd'):
            out = self.F._fwd(self.xr, self.xi, self.sin, self.cos, self.zero, self.zero, self.zero, 64, 1.0, False, 1,
                              True)
        return out


class Synapse(Workload):
    name = 'SLAYER synapse stack (conv K=64 -> per-channel shift -> CUBA) fwd+bwd'
    shape = (32, 256, 1500)
    ops = [('conv', 'conv_mfma_split_kernel<64,conv>', 8), ('shift', 'shift_kernel', 8),
           ('li_fwd_current', 'stream_kernel_duo<LiFwd>', 8), ('li_fwd_voltage', 'stream_kernel_duo<LiFwd>', 8),
           ('spike_fwd', 'spike_fwd_kernel', 8), ('spike_bwd', 'spike_bwd_kernel', 12),
           ('li_bwd_voltage', 'li_bwd_scan_kernel', 12), ('li_bwd_current', 'li_bwd_scan_kernel', 12),
           ('shift_back', 'shift_kernel', 8), ('corr', 'conv_mfma_split_kernel<64,corr>', 8)]
    note = 'alpha kernel tau 4, K=64, delays uniform over [0,32), CUBA scalar decays 1024/128, threshold 1.25'

    def __init__(self, dev):
        super().__init__(dev, 1004)
        g = self.gen
        i = torch.arange(64, dtype=torch.float32)
        self.put(x=(torch.rand(self.shape, generator=g) < 0.03).float(), filt=(i / 4) * torch.exp(1 - i / 4),
                 delay=torch.rand(self.shape[1], generator=g) * 32, g=torch.randn(self.shape, generator=g),
                 d_i=torch.tensor([1024.0]), d_v=torch.tensor([128.0]))
        self.neg_delay = -self.delay

    def step(self, t):
        L, S = self.L, self.S
        with t('conv'):
            y = self.conv.fwd(self.x, self.filt, 1)
        with t('shift'):
            z = self.shift(y, self.delay, 1)
        with t('li_fwd_current'):
            cur = L._fwd(z, self.d_i, self.zero, -1, 64)
        with t('li_fwd_voltage'):
            vol = L._fwd(cur, self.d_v, self.zero, 1.25, 64)
        with t('spike_fwd'):
            spk = S._fwd(vol, None, 1.25, False, 1)
        with t('spike_bwd'):
            g_vol = S._bwd(self.g, vol, None, 1.25, 1.0, 1.0, False)
        with t('li_bwd_voltage'):
            g_cur, _ = L._bwd(g_vol, vol, self.d_v)
        with t('li_bwd_current'):
            g_z, _ = L._bwd(g_cur, cur, self.d_i)
        with t('shift_back'):
            g_y = self.shift(g_z, self.neg_delay, 1)
        with t('corr'):
            g_x = self.conv.bwd(g_y, self.filt, 1)
        return spk, g_x

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        x, g, delay = c['x'][:n], c['g'][:n], c['delay']
        if sl is not None:
            x, g, delay = x[:, sl], g[:, sl], delay[sl]
        y = O.conv_fwd(x, c['filt'], 1)
        z = O.shift(y, delay, 1)
        cur = O.li_fwd(z, c['d_i'], zero, 64)
        vol = O.li_fwd(cur, c['d_v'], zero, 64, 1.25)
        spk = O.spike_fwd(vol, 1.25)
        g_vol = O.spike_bwd(g, vol, 1.25, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, c['d_v'])
        g_z, _ = O.li_bwd(g_cur, cur, c['d_i'])
        return spk, O.conv_bwd(O.shift(g_z, -delay, 1), c['filt'], 1)

    parity_slab = (1, slice(64, 96))


class SynapseFused(Synapse):
    name = 'SLAYER synapse stack (conv K=64 -> per-channel shift -> CUBA) fwd+bwd, fused CUBA kernels without the current trace'
    ops = [('conv', 'conv_mfma_split_kernel<64,conv>', 8), ('shift', 'shift_kernel', 8), ('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 12),
           ('cuba_bwd', 'cuba_bwd_scan_kernel', 12), ('shift_back', 'shift_kernel', 8), ('corr', 'conv_mfma_split_kernel<64,corr>', 8)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
        self.F = cuba_fused

    def step(self, t):
        with t('conv'):
            y = self.conv.fwd(self.x, self.filt, 1)
        with t('shift'):
            z = self.shift(y, self.delay, 1)
        with t('cuba_fwd'):
            _, vol, spk = self.F._fwd(z, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True)
        with t('cuba_bwd'):
            g_z, _, _ = self.F._bwd(self.g, vol, None, self.d_i, self.d_v, 1.25, 1.0, 1.0, False, False)
        with t('shift_back'):
            g_y = self.shift(g_z, self.neg_delay, 1)
        with t('corr'):
            g_x = self.conv.bwd(g_y, self.filt, 1)
        return spk, g_x


class SynapseFolded(SynapseFused):
    name = ('SLAYER synapse stack (conv K=64 -> per-channel shift -> CUBA) fwd+bwd, the shift folded into the fused '
            'CUBA kernels (read of the input, store of its gradient)')
    ops = [('conv', 'conv_mfma_split_kernel<64,conv>', 8), ('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 12),
           ('cuba_bwd', 'cuba_bwd_scan_kernel', 12), ('corr', 'conv_mfma_split_kernel<64,corr>', 8)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import delays
        self.D = delays
        self.delays = delays.Delays(input_shift=self.delay)

    def step(self, t):
        with t('conv'):
            y = self.conv.fwd(self.x, self.filt, 1)
        with t('cuba_fwd'):
            _, vol, spk = self.F._fwd(y, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True,
                                      folded=self.D.fold(self.delays, y))
        with t('cuba_bwd'):
            g_y, _, _ = self.F._bwd(self.g, vol, None, self.d_i, self.d_v, 1.25, 1.0, 1.0, False, False,
                                    folded=self.D.fold(self.delays, self.g, forward=False))
        with t('corr'):
            g_x = self.conv.bwd(g_y, self.filt, 1)
        return spk, g_x


class SynapseDelayGrad(SynapseFused):
    """Synaptic filter -> CUBA neuron -> learnable per-channel Delay, the order of a SLAYER block (block/base.py:549-553
    in the reference: the Delay follows the neuron), forward and backward including the delay's gradient
    (axon/delay.py:201-221).  The Delay is folded into the neuron's two kernels: the forward kernel stores its spikes
    through the delay, the backward scan reads the gradient back through it and sums grad * (out[t-1] - out[t]) / Ts
    per row on the way.  `block_tail` is the neuron + Delay part of this stack with separate kernels."""
    name = ('SLAYER synapse stack with a learnable delay (conv K=64 -> fused CUBA -> Delay, the Delay folded into the '
            'neuron kernels) fwd+bwd incl. the delay gradient')
    ops = [('conv', 'conv_mfma_split_kernel<64,conv>', 8), ('cuba_fwd', 'stream_kernel_staged<CubaFwd,SHIFT>', 12),
           ('cuba_bwd', 'cuba_bwd_scan_kernel<SHIFT,DELAY>', 16), ('corr', 'conv_mfma_split_kernel<64,corr>', 8)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import delays
        self.D = delays
        self.delays = delays.Delays(output_delay=self.delay)

    def step(self, t):
        with t('conv'):
            y = self.conv.fwd(self.x, self.filt, 1)
        with t('cuba_fwd'):
            _, vol, out = self.F._fwd(y, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True,
                                      folded=self.D.fold(self.delays, y))
        with t('cuba_bwd'):
            folded = self.D.fold(self.delays, self.g, forward=False, delayed_spikes=out)
            g_y, _, _ = self.F._bwd(self.g, vol, None, self.d_i, self.d_v, 1.25, 1.0, 1.0, False, False, folded=folded)
            g_delay = folded.grad_sum
        with t('corr'):
            g_x = self.conv.bwd(g_y, self.filt, 1)
        return out, g_x, g_delay

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        x, g, delay = c['x'][:n], c['g'][:n], c['delay']
        if sl is not None:
            x, g, delay = x[:, sl], g[:, sl], delay[sl]
        y = O.conv_fwd(x, c['filt'], 1)
        cur = O.li_fwd(y, c['d_i'], zero, 64)
        vol = O.li_fwd(cur, c['d_v'], zero, 64, 1.25)
        out = O.shift(O.spike_fwd(vol, 1.25), delay, 1)
        g_vol = O.spike_bwd(O.shift(g, -delay, 1), vol, 1.25, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, c['d_v'])
        g_y, _ = O.li_bwd(g_cur, cur, c['d_i'])
        return out, O.conv_bwd(g_y, c['filt'], 1)


class BlockTail(SynapseFused):
    """The tail of a SLAYER block with a trained axonal delay (block/base.py:549-553, axon/delay.py:178-221 in the
    reference): fused CUBA neuron -> learnable per-channel Delay, forward and backward including the delay's
    gradient, by separate operators: the Delay is a shift after the neuron, its backward pass one kernel that
    shifts the gradient back and sums grad * (out[t-1] - out[t]) / Ts per channel."""
    name = 'Block tail: fused CUBA -> learnable Delay (separate kernels), fwd+bwd incl. the delay gradient'
    ops = [('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 8), ('delay', 'shift_kernel', 8),
           ('delay_bwd', 'delay_bwd_kernel', 12), ('cuba_bwd', 'cuba_bwd_scan_kernel', 12)]

    def __init__(self, dev):
        super().__init__(dev)
        import importlib
        self.AX = importlib.import_module('lava_dl_amd.slayer.axon.delay')

    def step(self, t):
        with t('cuba_fwd'):
            _, vol, spk = self.F._fwd(self.x, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True)
        with t('delay'):
            out = self.shift(spk, self.delay, 1)
        with t('delay_bwd'):
            g_spk, g_delay = self.AX._delay_bwd(self.g, out, self.delay, 1)
        with t('cuba_bwd'):
            g_x, _, _ = self.F._bwd(g_spk, vol, None, self.d_i, self.d_v, 1.25, 1.0, 1.0, False, False)
        return out, g_x, g_delay

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        x, g, delay = c['x'][:n], c['g'][:n], c['delay']
        if sl is not None:
            x, g, delay = x[:, sl], g[:, sl], delay[sl]
        cur = O.li_fwd(x, c['d_i'], zero, 64)
        vol = O.li_fwd(cur, c['d_v'], zero, 64, 1.25)
        out = O.shift(O.spike_fwd(vol, 1.25), delay, 1)
        g_vol = O.spike_bwd(O.shift(g, -delay, 1), vol, 1.25, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, c['d_v'])
        return out, O.li_bwd(g_cur, cur, c['d_i'])[0]


class BlockTailFolded(BlockTail):
    """The same block tail with the Delay folded into the neuron's two kernels: the forward kernel stores its spikes
    through the delay, the backward scan reads the gradient back through it and, with the delayed spikes as one more
    input, leaves the delay gradient's per-row sums on the way.  Same results (spikes and input gradient bit for
    bit)."""
    name = 'Block tail: fused CUBA with the learnable Delay folded into its kernels, fwd+bwd incl. the delay gradient'
    ops = [('cuba_fwd', 'stream_kernel_staged<CubaFwd,SHIFT>', 8), ('cuba_bwd', 'cuba_bwd_scan_kernel<SHIFT,DELAY>', 16)]

    def __init__(self, dev):
        super().__init__(dev)
        from lava_dl_amd.slayer.neuron.dynamics import delays
        self.D = delays
        self.delays = delays.Delays(output_delay=self.delay)

    def step(self, t):
        with t('cuba_fwd'):
            _, vol, out = self.F._fwd(self.x, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True,
                                      folded=self.D.fold(self.delays, self.x))
        with t('cuba_bwd'):
            folded = self.D.fold(self.delays, self.g, forward=False, delayed_spikes=out)
            g_x, _, _ = self.F._bwd(self.g, vol, None, self.d_i, self.d_v, 1.25, 1.0, 1.0, False, False, folded=folded)
            g_delay = folded.grad_sum
        return out, g_x, g_delay


class ConvSynapse(Cuba):
    """The convolution synapse that produces config[1]'s tensor (synapse/layer.py:297-323 in the reference: F.conv3d
    with a 3x3x1 kernel on NCHWT spikes), feeding the fused CUBA neuron, forward and backward down to the gradient of
    the input spikes.  The synapse kernel works on the time-innermost layout as it is; the neuron reads its output in
    place.  Weights are multiples of 1/64 (quantised, as a SLAYER synapse's are), so the weighted spikes are exact
    and the forward parity check stays bit for bit.  Bytes per neuron-timestep of the output tensor."""
    name = 'Conv synapse (3x3, 8 -> 16 channels) -> fused CUBA neuron, fwd+bwd (input and weight gradients)'
    ops = [('conv_synapse', 'synapse_conv_row_kernel', 6), ('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 16),
           ('cuba_bwd', 'cuba_bwd_scan_kernel', 16), ('conv_synapse_bwd', 'synapse_conv_row_kernel', 6),
           ('conv_synapse_wgrad', 'synapse_wgrad_kernel', 6)]
    weight_gradient = True
    note = Cuba.note + '; input spikes Bernoulli(0.05) on 8 channels, weights round(N(0, 0.3) * 64) / 64'
    in_channels = 8

    def __init__(self, dev):
        super().__init__(dev)
        import importlib
        g = self.gen
        self.put(s=(torch.rand((self.shape[0], self.in_channels) + self.shape[2:], generator=g) < 0.05).float(),
                 wgt=(torch.randn(self.shape[1], self.in_channels, 3, 3, 1, generator=g) * 0.3 * 64).round() / 64)
        self.syn = importlib.import_module('lava_dl_amd.slayer.synapse.layer')
        self.F = importlib.import_module('lava_dl_amd.slayer.neuron.dynamics.cuba_fused')
        self.w4 = self.wgt[..., 0].contiguous()
        self.w4_back = self.wgt[..., 0].flip(2, 3).transpose(0, 1).contiguous()

    def synapse(self, s):
        return self.syn._launch(s, self.w4, (1, 1), (1, 1), (1, 1))

    def synapse_back(self, g):
        return self.syn._launch(g, self.w4_back, (1, 1), (1, 1), (1, 1))

    def step(self, t):
        with t('conv_synapse'):
            z = self.synapse(self.s)
        with t('cuba_fwd'):
            cur, vol, spk = self.F._fwd(z, self.d_i, self.d_v, self.zero, self.zero, self.w, self.thr, False, 1)
        with t('cuba_bwd'):
            g_z, _, _ = self.F._bwd(self.g, vol, cur, self.d_i, self.d_v, self.thr, 1.0, 1.0, False)
        with t('conv_synapse_bwd'):
            g_s = self.synapse_back(g_z)
        if self.weight_gradient:
            with t('conv_synapse_wgrad'):
                self.g_w = self.syn._weight_gradient(self.s, self.wgt.shape, g_z, (1, 1), (1, 1), (1, 1))
        return spk, g_s

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        s, g, wgt, d_i, d_v = c['s'][:n], c['g'][:n], c['wgt'], c['d_i'], c['d_v']
        z = O.conv_synapse(s, wgt, (1, 1), (1, 1), (1, 1))
        cur = O.li_fwd(z, d_i, zero, self.w)
        vol = O.li_fwd(cur, d_v, zero, self.w, self.thr)
        spk = O.spike_fwd(vol, self.thr)
        g_vol = O.spike_bwd(g, vol, self.thr, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, d_v)
        g_z, _ = O.li_bwd(g_cur, cur, d_i)
        g_s = torch.nn.grad.conv3d_input(s.shape, wgt.double(), g_z.double(), (1, 1, 1), (1, 1, 0)).float()
        return (spk if sl is None else spk[:, sl]), None if sl is not None else g_s

    parity_slab = (1, slice(0, 16))


class ConvSynapseLibrary(ConvSynapse):
    """The same stack with the reference's own call for the synapse: the library convolution transposes the tensor to
    channels-last and back around its kernel (three extra passes each way).  Without the weight gradient:
    torch.nn.grad.conv3d_weight takes 1.3 s per call on this tensor on this platform."""
    name = 'Conv synapse by F.conv3d (library kernel + layout transposes) -> fused CUBA neuron, fwd+bwd (input gradient only)'
    ops = [('conv_synapse', 'F.conv3d: library conv + batched_transpose x3', 6), ('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 16),
           ('cuba_bwd', 'cuba_bwd_scan_kernel', 16), ('conv_synapse_bwd', 'conv3d_input: library conv + transposes', 6)]
    weight_gradient = False

    def synapse(self, s):
        return torch.nn.functional.conv3d(s, self.wgt, None, (1, 1, 1), (1, 1, 0))

    def synapse_back(self, g):
        return torch.nn.grad.conv3d_input(self.s.shape, self.wgt, g, (1, 1, 1), (1, 1, 0))


class PoolSynapse(Workload):
    """The pooling synapse behind config[1]'s spikes (synapse/layer.py:326-510 in the reference: the channels folded
    into the image height, a one-channel F.conv3d with a constant 2x2 kernel and stride 2), forward and the gradient
    of its input.  Nothing to contract: one thread per quad of steps on the vector units.  Bytes per sample of the
    layer's input tensor: the forward pass reads it and writes a quarter of it, the backward pass the reverse."""
    name = 'Pool synapse 2x2 on the spikes of the conv-layer tensor, fwd + input gradient'
    shape = (32, 16, 32, 32, 300)
    ops = [('pool_synapse', 'synapse_plane_kernel<false>', 5), ('pool_synapse_bwd', 'synapse_plane_kernel<true>', 5)]
    note = 'input spikes Bernoulli(0.05), weight 1.0, upstream gradient N(0, 1)'

    def __init__(self, dev):
        super().__init__(dev, 1007)
        import importlib
        g = self.gen
        n, c, h, w, t = self.shape
        self.put(s=(torch.rand(self.shape, generator=g) < 0.05).float(),
                 g=torch.randn(n, c, h // 2, w // 2, t, generator=g), wgt=torch.ones(1, 1, 2, 2))
        self.syn = importlib.import_module('lava_dl_amd.slayer.synapse.layer')
        self.folded = (n, 1, c * h, w, t)

    def step(self, t):
        n, c, h, w, steps = self.shape
        with t('pool_synapse'):
            y = self.syn._launch(self.s.view(self.folded), self.wgt, (2, 2), (0, 0), (1, 1))
        with t('pool_synapse_bwd'):
            g_s = self.syn._launch_input_grad(self.g.view(n, 1, c * h // 2, w // 2, steps), self.wgt, self.folded,
                                              (2, 2), (0, 0), (1, 1))
        return y.view(n, c, h // 2, w // 2, steps), g_s.view(self.shape)

    def cpu_step(self, n, sl=None):
        c = self.cpu
        s, g = c['s'][:n].double(), c['g'][:n].double()
        y = s[:, :, 0::2, 0::2] + s[:, :, 0::2, 1::2] + s[:, :, 1::2, 0::2] + s[:, :, 1::2, 1::2]
        g_s = g.repeat_interleave(2, 2).repeat_interleave(2, 3)
        sl = slice(None) if sl is None else sl
        return y[:, sl].float(), g_s[:, sl].float()

    parity_slab = (2, slice(0, 16))


class ConvTransposeSynapse(Workload):
    """A decoder stage (synapse/layer.py:511-658 in the reference: F.conv_transpose3d with a 4x4x1 kernel, stride 2,
    padding 1 on NCHWT spikes): 16 maps of 16x16 to 8 maps of 32x32, forward and both gradients.  One plain
    convolution per residue class of the output pixels (four launches forward), the strided convolution kernel for
    the input gradient, the weight-gradient kernels with input and output exchanged.  Weights are multiples of 1/64,
    so the forward result is exact.  Bytes per sample of the layer's output tensor (4 written + 8 read forward, 4
    read + 8 written for the input gradient, 12 read for the weight gradient: output 8 channels, input 16 at a
    quarter of the pixels)."""
    name = 'ConvTranspose synapse 4x4 stride 2, 16 -> 8 channels, 16x16 -> 32x32, fwd + input and weight gradients'
    shape = (32, 8, 32, 32, 300)
    ops = [('conv_transpose', 'synapse_conv_row_kernel<2> x 4 residue classes', 6), ('conv_transpose_bwd', 'synapse_conv_kernel (stride 2)', 6),
           ('conv_transpose_wgrad', 'synapse_wgrad_kernel', 6)]
    note = 'input spikes Bernoulli(0.05) on 16 channels of 16x16, weights round(N(0, 0.3) * 64) / 64, upstream gradient N(0, 1)'

    def __init__(self, dev):
        super().__init__(dev, 1008)
        import importlib
        g = self.gen
        n, co, h, w, t = self.shape
        self.put(s=(torch.rand(n, 16, h // 2, w // 2, t, generator=g) < 0.05).float(),
                 wgt=(torch.randn(16, co, 4, 4, 1, generator=g) * 0.3 * 64).round() / 64,
                 g=torch.randn(self.shape, generator=g))
        self.syn = importlib.import_module('lava_dl_amd.slayer.synapse.layer')
        self.w4 = self.wgt[..., 0].contiguous()                      # [Ci, Co, kh, kw]: the backward convolution's weights
        self.w4_t = self.wgt[..., 0].transpose(0, 1).contiguous()    # channel axes exchanged for the class launches

    def step(self, t):
        cfg = ((2, 2), (1, 1), (1, 1))
        with t('conv_transpose'):
            y = self.syn._launch_input_grad(self.s, self.w4_t, self.shape, *cfg)
        with t('conv_transpose_bwd'):
            g_s = self.syn._launch(self.g, self.w4, *cfg)
        with t('conv_transpose_wgrad'):
            self.g_w = self.syn._weight_gradient(self.g, self.wgt.shape, self.s, *cfg)
        return y, g_s

    def cpu_step(self, n, sl=None):
        c = self.cpu
        F = torch.nn.functional
        y = F.conv_transpose3d(c['s'][:n].double(), c['wgt'].double(), None, (2, 2, 1), (1, 1, 0))
        g_s = F.conv3d(c['g'][:n].double(), c['wgt'].double(), None, (2, 2, 1), (1, 1, 0))
        sl = slice(None) if sl is None else sl
        return y[:, sl].float(), g_s[:, sl].float()

    parity_slab = (1, slice(0, 8))


class DenseSynapse(Workload):
    """Dense synapse (the reference's 1x1x1 conv3d over [N, C, 1, 1, T], synapse/layer.py:144-175, written as the
    batched GEMM it is) feeding the fused CUBA kernel, forward only: the kernel list of this workload shows what runs
    between the GEMM and the neuron.  (`F.conv3d` itself goes through MIOpen here, which transposes to channels-last
    and back around its kernel; `torch.matmul` does not.)"""
    name = 'Dense synapse (batched GEMM) -> fused CUBA neuron, forward'
    shape = (32, 256, 1500)
    ops = [('dense_gemm', 'torch.matmul (GEMM, outside this library)', 8), ('cuba_fwd', 'stream_kernel_staged<CubaFwd>', 8)]
    note = '256 -> 256 neurons, input Bernoulli(0.03), weights N(0, 0.3) on the 2/64 grid, CUBA decays 1024/128, threshold 1.25'

    def __init__(self, dev):
        super().__init__(dev, 1005)
        from lava_dl_amd.slayer.neuron.dynamics import cuba_fused
        self.F = cuba_fused
        g = self.gen
        self.put(s=(torch.rand(self.shape, generator=g) < 0.03).float(),
                 wgt=(torch.randn(256, 256, generator=g) * 0.3 * 32).round() / 32,
                 d_i=torch.tensor([1024.0]), d_v=torch.tensor([128.0]))

    def step(self, t):
        with t('dense_gemm'):
            z = torch.matmul(self.wgt, self.s)           # [256, C] @ [N, C, T] -> [N, 256, T], time innermost
        with t('cuba_fwd'):
            out = self.F._fwd(z, self.d_i, self.d_v, self.zero, self.zero, 64, 1.25, False, 1, True, True)
        return out[2]

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c, zero = self.cpu, torch.tensor([0.0])
        z = torch.matmul(c['wgt'], c['s'][:n])
        if sl is not None:
            z = z[:, sl]
        cur = O.li_fwd(z, c['d_i'], zero, 64)
        vol = O.li_fwd(cur, c['d_v'], zero, 64, 1.25)
        return O.spike_fwd(vol, 1.25), None

    parity_slab = (1, slice(32, 64))


class Recurrent(Workload):
    """A recurrent CUBA layer (utils/recurrent.py:45-112 in the reference: s[t] = neuron(z[t] + R s[t-1]), one neuron
    call per time step in a Python loop), forward and backward with the gradient of the recurrent weights, through
    the module interface (custom_recurrent).  2048 neurons take the launch-per-step kernels: a step reads the
    [C x C] matrix once for the whole batch, so the algorithmic bytes per neuron-timestep are those of the tensors
    (z, spikes, voltage; gradient, voltage, gradient of z) plus 4 C / N for the matrix."""
    name = 'Recurrent CUBA layer, 2048 neurons, fwd+bwd (module interface)'
    shape = (32, 2048, 300)
    ops = [('recurrent_fwd', 'recurrent_step_fwd_kernel, one launch per time step', 12 + 4 * 2048 // 32),
           ('recurrent_bwd', 'recurrent_step_bwd_kernel, one launch per time step, + weight-gradient GEMM', 12 + 4 * 2048 // 32)]
    note = ('CUBA decays 0.25 / 0.25, threshold 1.25, z ~ 1.5 N(0,1), weights N(0, 0.6) * 6 / sqrt(C) quantised to '
            '8 bits (the synapse pre-hook), about 40 % of the neurons spike per step')
    generic_loop = False

    def __init__(self, dev):
        super().__init__(dev, 1011)
        import importlib
        slayer = importlib.import_module('lava_dl_amd.slayer')
        self.Rm = slayer.utils.recurrent
        g = self.gen
        n, c, t = self.shape
        self.neuron = slayer.neuron.cuba.Neuron(threshold=1.25, current_decay=0.25, voltage_decay=0.25,
                                                persistent_state=True).to(dev)
        self.put(z=torch.randn(self.shape, generator=g) * 1.5, g=torch.rand(self.shape, generator=g),
                 wgt=torch.randn(c, c, generator=g) * 0.6 * 6.0 / c ** 0.5)
        self.z.requires_grad_()

        class _Synapse:
            pass
        self.syn = _Synapse()
        self.syn.weight = self.wgt.reshape(c, c, 1, 1, 1).requires_grad_()
        self.syn.pre_hook_fx = self.neuron.quantize_8bit

    def step(self, t):
        R, neuron = self.Rm, self.neuron
        for k in ('current_state', 'voltage_state'):          # every step starts from the initial state
            neuron._buffers[k] = self.zero
        self.z.grad = None
        self.syn.weight.grad = None
        with t('recurrent_fwd'):
            if self.generic_loop:
                out = R.CustomRecurrent.apply(self.z, neuron, R._recurrent_matrix(self.syn))
            else:
                out = R.custom_recurrent(self.z, neuron, self.syn)
        with t('recurrent_bwd'):
            out.backward(self.g)
        return out.detach(), self.z.grad

    def cpu_step(self, n, sl=None):
        from oracle import slayer_oracle as O
        c = self.cpu
        neuron = self.neuron
        rec = neuron.quantize_8bit(c['wgt'])
        d_i, d_v = neuron.current_decay.detach().round().cpu(), neuron.voltage_decay.detach().round().cpu()
        thr = neuron.threshold + neuron.threshold_eps
        zero = torch.tensor([0.0])
        spk, vol, _, _ = O.recurrent_cuba_fwd(c['z'][:n], rec, d_i, d_v, zero, zero, int(neuron.s_scale), thr)
        g_z, _ = O.recurrent_cuba_bwd(c['g'][:n], spk, vol, rec, thr, neuron.tau_rho * 100, neuron.scale_rho * 0.1)
        return spk[:, sl], g_z[:, sl]

    parity_slab = (1, slice(0, 2048))


class RecurrentLoop(Recurrent):
    """The same layer through the reference's loop of one-step neuron calls (CustomRecurrent, the path layers take
    that the kernels do not cover)."""
    name = 'Recurrent CUBA layer, 2048 neurons, fwd+bwd: loop of one-step neuron calls'
    ops = [('recurrent_fwd', 'a dozen launches per time step (one-step neuron calls + torch.matmul)', 12 + 4 * 2048 // 32),
           ('recurrent_bwd', 'autograd of every step + torch.matmul', 12 + 4 * 2048 // 32)]
    generic_loop = True


WORKLOADS = {'cuba': Cuba, 'cuba_fused': CubaFused, 'cuba_fused_lean': CubaFusedLean, 'cuba_inference': CubaInference, 'cuba_fwd_small': CubaFwdSmall, 'alif': Alif, 'alif_fused': AlifFused, 'alif_fused_lean': AlifFusedLean, 'rf': Rf, 'rf_fused': RfFused, 'rf_fused_lean': RfFusedLean, 'rf_inference': RfInference, 'synapse': Synapse, 'synapse_fused': SynapseFused, 'synapse_folded': SynapseFolded, 'synapse_delay_grad': SynapseDelayGrad, 'block_tail': BlockTail, 'block_tail_folded': BlockTailFolded,
             'conv_synapse': ConvSynapse, 'conv_synapse_library': ConvSynapseLibrary, 'pool_synapse': PoolSynapse, 'conv_transpose_synapse': ConvTransposeSynapse,
             'dense_synapse': DenseSynapse, 'recurrent': Recurrent, 'recurrent_loop': RecurrentLoop}


def cpu_baseline(job, budget_s=20.0):
    """The torch-CPU oracle (the reference's per-timestep loops restated, same op sequence) on this
    box's host cores: repeated runs on (a batch prefix of) the same workload for about budget_s seconds."""
    N = job.shape[0]

    def run(n):
        t0 = time.perf_counter()
        job.cpu_step(n)
        return time.perf_counter() - t0

    dt = run(1)
    n_sub = max(1, min(N, int(budget_s / 4 / max(dt, 1e-9))))      # one run = at most a quarter of the budget
    times, t_start = [], time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        times.append(run(n_sub))
    times.sort()
    med = times[len(times) // 2]
    nt = n_sub * math.prod(job.shape[1:])
    return dict(value=nt / med, unit='neuron-timesteps/s', cores=torch.get_num_threads(), kind='port',
                sample=f'oracle (torch CPU per-timestep loop, same op sequence) on batch[:{n_sub}] of '
                       f'{list(job.shape)}: median of {len(times)} runs, {med:.2f} s each, '
                       f'{sum(times):.1f} s total; torch threads={torch.get_num_threads()}, '
                       f'os.cpu_count()={os.cpu_count()}')


def _first_two(out):
    """(spikes or final trace, input gradient or None) of a workload's step() result."""
    if torch.is_tensor(out):
        return out, None
    spk, grad = out[0], (out[1] if len(out) > 1 else None)
    if isinstance(grad, (tuple, list)):
        grad = grad[0]
    return spk, grad


def parity(job):
    """One step on the GPU against the oracle on a slab of the same tensors (outside every timed region):
    forward results bit for bit, the input gradient within 1e-5 of its largest magnitude."""
    n, sl = job.parity_slab
    spk, grad = _first_two(job.step(lambda name: _Null()))
    torch.cuda.synchronize()
    r_spk, r_grad = job.cpu_step(n, sl)
    got = spk[:n, sl].cpu()
    if got.shape != r_spk.shape or not torch.equal(got, r_spk):
        bad = int((got != r_spk).sum()) if got.shape == r_spk.shape else -1
        raise SystemExit(f'parity FAILED for {job.name}: {bad} forward samples differ from the oracle')
    info = {'forward': f'bit-exact on batch[:{n}], channels {sl.start}:{sl.stop} ({r_spk.numel()} samples, '
                       f'{int((r_spk != 0).sum())} non-zero)'}
    if grad is not None and r_grad is not None:
        g = grad[:n, sl].cpu().double()
        err = float((g - r_grad.double()).abs().max())
        scale = float(r_grad.abs().max())
        if not err <= 1e-5 * scale:
            raise SystemExit(f'parity FAILED for {job.name}: input gradient off by {err:.3e} (scale {scale:.3e})')
        info['grad_input'] = f'max abs err {err:.2e} of scale {scale:.2e}'
    return info


def timed_median(job, iters, warmup):
    """Median over `iters` whole steps, each between two events on the launch stream."""
    null = lambda name: _Null()
    for _ in range(warmup):
        job.step(null)
    torch.cuda.synchronize()
    pairs = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        job.step(null)
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in pairs)
    return times[len(times) // 2]


# The other benchmark configurations, reported next to the headline in `other_configs` (unfused = the op
# sequence of the configuration, then the fused forms with their own smaller byte counts).
OTHER = ['cuba_fwd_small', 'cuba_fused', 'cuba_fused_lean', 'alif', 'alif_fused', 'alif_fused_lean', 'rf', 'rf_fused',
         'synapse', 'synapse_fused', 'synapse_folded', 'synapse_delay_grad', 'block_tail', 'block_tail_folded',
         'conv_synapse', 'conv_synapse_library', 'pool_synapse', 'conv_transpose_synapse', 'recurrent', 'recurrent_loop']


def other_configs(dev, iters):
    rows = []
    for name in OTHER:
        job = WORKLOADS[name](dev)
        ok = parity(job)
        ms = timed_median(job, iters, 20)
        # the same steps back to back between two synchronisations, as the headline is timed: the event records
        # between steps cost the device about 10 us a step, which shows on the steps of a fraction of a millisecond
        null = lambda name: _Null()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            job.step(null)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / iters
        bpn = job.bytes_per_nt()
        rows.append({'workload': name, 'shape': list(job.shape), 'bytes_per_nt': bpn, 'ms_per_step': round(ms, 4),
                     'neuron_timesteps_per_s': job.nt / (ms * 1e-3),
                     'frac': round(job.nt * bpn / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     'wall_ms_per_step': round(wall_ms, 4),
                     'wall_frac': round(job.nt * bpn / (wall_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     'timing': f'ms_per_step, frac: median of {iters} event-timed steps after 20 warm-up steps; '
                               f'wall_ms_per_step, wall_frac: {iters} steps back to back between two synchronisations',
                     'parity': 'ok', 'parity_detail': ok})
        if job.nt < (1 << 20):
            # latency-bound: host time per call matters as much as the kernels; wall clock over many steps
            null = lambda name: _Null()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(2000):
                job.step(null)
            torch.cuda.synchronize()
            rows[-1]['us_per_step_event_timed'] = round(ms * 1e3, 2)
            rows[-1]['us_per_step_wall_clock'] = round((time.perf_counter() - t0) / 2000 * 1e6, 2)
        del job
        gc.collect()
        torch.cuda.empty_cache()
    return rows


def traffic_factor(kernel):
    """HBM bytes per launch / algorithmic bytes for `kernel` from profiles/traffic_factors.txt (rocprofv3 --pmc
    FETCH_SIZE and WRITE_SIZE runs of this script, scaled by a plain copy of known size), or None when the file
    was measured on other sources of those kernels (the files it lists) than the ones in the tree."""
    import hashlib
    path = os.path.join(ROOT, 'profiles', 'traffic_factors.txt')
    if not os.path.exists(path):
        return None, 'no profiles/traffic_factors.txt'
    rec = json.load(open(path))
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, 'lava-dl_amd', 'csrc')
    for f in rec.get('sources', []):                 # the sources the measured kernels are built from
        h.update(open(os.path.join(csrc, f), 'rb').read())
    if h.hexdigest()[:16] != rec.get('csrc_sha16'):
        return None, f"stale: measured at csrc {rec.get('csrc_sha16')} ({rec.get('commit')}), tree is {h.hexdigest()[:16]}"
    return rec['factors'].get(kernel), f"measured at commit {rec.get('commit')} (csrc {rec.get('csrc_sha16')})"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='cuba', choices=sorted(WORKLOADS))
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-other-configs', action='store_true')
    ap.add_argument('--iters', type=int, default=100, help='event-timed iterations behind every median')
    ap.add_argument('--calibration-copies', type=int, default=0,
                    help='also run N plain device copies of one input tensor (a kernel of known traffic, '
                         'used to scale hardware byte counters when profiling)')
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit('bench.py measures one GPU: this hot path has no multi-GPU component '
                         '(neurons are independent, so it would shard along the batch axis with one small all-reduce of the '
                         'parameter gradients). Use --gpus 1.')
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    import lava_dl_amd.slayer  # noqa: F401  (fails loudly if the HIP library is missing)

    job = WORKLOADS[a.workload](dev)
    for _ in range(a.calibration_copies):
        first = next(v for v in vars(job).values() if torch.is_tensor(v) and v.numel() == job.nt)
        torch.empty_like(first).copy_(first)
    nt = job.nt
    null = lambda name: _Null()
    parity_info = parity(job)        # before any timing; raises when the GPU path and the oracle disagree

    for _ in range(a.warmup):
        job.step(null)
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()                 # a collection of the interpreter's cyclic garbage would stall the launches for milliseconds
    t0 = time.perf_counter()
    for _ in range(a.steps):
        job.step(null)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps
    median_ms = timed_median(job, a.iters, 20)
    gc.enable()

    # per-kernel device time (separate pass so the event records do not perturb the headline number)
    timers = Timers()
    for _ in range(a.iters):
        job.step(timers.section)
    torch.cuda.synchronize()
    op_ms = timers.median_ms()
    per_op = []
    for name, kernel, bpn in job.ops:
        gbs = nt * bpn / (op_ms[name] * 1e-3) / 1e9
        per_op.append(dict(op=name, kernel=kernel, ms=round(op_ms[name], 4), bytes_per_nt=bpn,
                           achieved_GBps=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4)))
    dom = dict(max(per_op, key=lambda r: r['ms']))
    launch = job.kernel_only(dom['op']) if hasattr(job, 'kernel_only') else None
    if launch is not None:      # the op is more than one launch: time its main kernel by itself
        n = a.iters
        launch()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()                      # on the stream the kernel is launched on (torch's current stream)
        for _ in range(n):
            launch()
        end.record()
        torch.cuda.synchronize()
        dom['ms'] = round(begin.elapsed_time(end) / n, 4)
        gbs = nt * dom['bytes_per_nt'] / (dom['ms'] * 1e-3) / 1e9
        dom['achieved_GBps'], dom['frac'] = round(gbs, 1), round(gbs / HBM_PEAK_GBS, 4)
    total_bpn = job.bytes_per_nt()
    value = nt / (ms_per_step * 1e-3)
    factor, factor_note = traffic_factor(dom['kernel'])

    out = {
        'metric': 'neuron-timesteps/sec fwd+bwd (CUBA) + % of MI355X HBM peak, 1 GPU',
        'value': value, 'unit': 'neuron-timesteps/s', 'n_gpus': 1, 'steps': a.steps, 'warmup': a.warmup,
        'ms_per_step': ms_per_step, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'int32 fixed-point state (fwd) / f32 (bwd), f32 tensors', 'data': 'synthetic',
        'config': {'workload': f'{job.name} {list(job.shape)}; {job.note}', 'bytes_per_nt': total_bpn},
        'hbm_frac_whole_step': value * total_bpn / 1e9 / HBM_PEAK_GBS,
        'median_ms_per_step': round(median_ms, 4),
        'median_note': f'median of {a.iters} event-timed steps after 20 warm-up steps',
        'parity': 'ok', 'parity_detail': parity_info,
        'roofline': {'bound': 'hbm', 'kernel': dom['kernel'], 'op': dom['op'],
                     'achieved': dom['achieved_GBps'], 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': dom['frac'], 'kernel_ms': dom['ms'],
                     'traffic': nt * dom['bytes_per_nt'] * factor if factor else None,
                     'traffic_unit': 'bytes per launch (rocprofv3 FETCH_SIZE x2 + WRITE_SIZE, see profiles/)',
                     'traffic_note': factor_note},
        'per_op': per_op,
    }
    if not a.no_other_configs and a.workload == 'cuba':
        del job
        gc.collect()
        torch.cuda.empty_cache()
        out['other_configs'] = other_configs(dev, a.iters)
        job = WORKLOADS[a.workload](dev) if not a.no_cpu_baseline else None
    if not a.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(job)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
