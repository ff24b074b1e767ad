"""Benchmark of the SLAYER neuron-dynamics hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cuba|alif|rf|synapse|cuba_small]

A step is one pass of the op sequence of the workload over one batch of synthetic input that is
already resident in HBM.  The default workload is the CUBA conv-layer neuron tensor
[32,16,32,32,300], forward + backward (LI, LI+threshold, Spike; Spike bwd, LI bwd, LI bwd).
Prints ONE JSON line: whole-job neuron-timesteps/s, per-kernel roofline and the CPU baseline
(the torch-CPU oracle timed on this box's host cores on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch divided by algorithmic bytes, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script scaled by a plain copy of known size (profiles/cuba_fwd_bwd_32x16x32x32x300.md).
MEASURED_TRAFFIC_FACTOR = {'stream_kernel<LiFwd>': 1.038, 'stream_kernel<LiBwd>': 1.057,
                           'spike_fwd_kernel': 1.000, 'spike_bwd_kernel': 1.000}


def make_inputs(workload, dev):
    """Synthetic inputs generated on the CPU with a fixed seed, then copied to the GPU."""
    gen = torch.Generator().manual_seed(1001)
    if workload in ('cuba', 'cuba_small'):
        shape = (32, 16, 32, 32, 300) if workload == 'cuba' else (4, 16, 32, 32, 300)
        x = (torch.rand(shape, generator=gen) < 0.02).float() * torch.randn(shape, generator=gen) * 0.5
        d_i = torch.randint(0, 4096, (16,), generator=gen).float()
        d_v = torch.randint(0, 4096, (16,), generator=gen).float()
        g = torch.randn(shape, generator=gen)
        return dict(shape=shape, x=x.to(dev), g=g.to(dev), d_i=d_i.to(dev), d_v=d_v.to(dev),
                    cpu=dict(x=x, g=g, d_i=d_i, d_v=d_v))
    raise SystemExit(f'unknown workload {workload}')


class Cuba:
    """CUBA fwd+bwd op sequence; bytes per neuron-timestep of each API-level op = every input
    tensor read once + every output written once, 4 B per element."""
    name = 'CUBA conv-layer neuron tensor fwd+bwd'
    ops = [('li_fwd_current', 8), ('li_fwd_voltage', 8), ('spike_fwd', 8),
           ('spike_bwd', 12), ('li_bwd_voltage', 12), ('li_bwd_current', 12)]
    kernel_of = {'li_fwd_current': 'stream_kernel<LiFwd>', 'li_fwd_voltage': 'stream_kernel<LiFwd>',
                 'spike_fwd': 'spike_fwd_kernel', 'spike_bwd': 'spike_bwd_kernel',
                 'li_bwd_voltage': 'stream_kernel<LiBwd>', 'li_bwd_current': 'stream_kernel<LiBwd>'}

    def __init__(self, inp):
        from lava_dl_amd.slayer.neuron.dynamics import leaky_integrator as L
        from lava_dl_amd.slayer.spike import spike as S
        self.L, self.S, self.i = L, S, inp
        self.zero = torch.zeros(1, device=inp['x'].device)
        self.w, self.thr = 64, 1.0

    def step(self, timers=None):
        i, L, S = self.i, self.L, self.S
        t = timers.section if timers else (lambda name: _Null())
        with t('li_fwd_current'):
            cur = L._fwd(i['x'], i['d_i'], self.zero, -1, self.w)
        with t('li_fwd_voltage'):
            vol = L._fwd(cur, i['d_v'], self.zero, self.thr, self.w)
        with t('spike_fwd'):
            spk = S._fwd(vol, None, self.thr, False, 1)
        with t('spike_bwd'):
            g_vol = S._bwd(i['g'], vol, None, self.thr, 1.0, 1.0, False)
        with t('li_bwd_voltage'):
            g_cur, gd_v = L._bwd(g_vol, vol, i['d_v'])
        with t('li_bwd_current'):
            g_x, gd_i = L._bwd(g_cur, cur, i['d_i'])
        return spk, g_x, gd_v, gd_i


class _Null:
    def __enter__(self):
        return self

    def __exit__(self, *a):
        return False


class Timers:
    """Per-op device time from events recorded on the stream the kernels are launched on."""

    def __init__(self):
        self.events = {}

    def section(self, name):
        timers = self

        class _S:
            def __enter__(self):
                self.a = torch.cuda.Event(enable_timing=True)
                self.b = torch.cuda.Event(enable_timing=True)
                self.a.record()
                return self

            def __exit__(self, *a):
                self.b.record()
                timers.events.setdefault(name, []).append((self.a, self.b))
                return False
        return _S()

    def mean_ms(self):
        return {k: sum(a.elapsed_time(b) for a, b in v) / len(v) for k, v in self.events.items()}


def cpu_baseline(workload, inp, budget_s=20.0):
    """The torch-CPU oracle (the reference's per-timestep loop restated) on a batch subsample of the
    same workload; returns nt/s, threads used and a description of the sample."""
    from oracle import slayer_oracle as O
    c = inp['cpu']
    N = inp['shape'][0]
    n_sub = 1
    zero = torch.tensor([0.0])

    def run(n):
        x, g = c['x'][:n], c['g'][:n]
        t0 = time.perf_counter()
        cur = O.li_fwd(x, c['d_i'], zero, 64)
        vol = O.li_fwd(cur, c['d_v'], zero, 64, 1.0)
        O.spike_fwd(vol, 1.0)
        g_vol = O.spike_bwd(g, vol, 1.0, 1.0, 1.0)
        g_cur, _ = O.li_bwd(g_vol, vol, c['d_v'])
        O.li_bwd(g_cur, cur, c['d_i'])
        return time.perf_counter() - t0

    dt = run(n_sub)
    n_sub = max(1, min(N, int(budget_s / 4 / max(dt, 1e-9))))      # one run = at most a quarter of the budget
    times, t_start = [], time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        times.append(run(n_sub))
    times.sort()
    med = times[len(times) // 2]
    nt = n_sub * int(torch.tensor(inp['shape'][1:]).prod())
    return dict(value=nt / med, unit='neuron-timesteps/s', cores=torch.get_num_threads(), kind='port',
                sample=f'oracle (torch CPU per-timestep loop, same op sequence) on batch[:{n_sub}] of '
                       f'{list(inp["shape"])}: median of {len(times)} runs, {med:.2f} s each, '
                       f'{sum(times):.1f} s total; torch threads={torch.get_num_threads()}, '
                       f'os.cpu_count()={os.cpu_count()}')


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='cuba')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--calibration-copies', type=int, default=0,
                    help='also run N plain device copies of one input tensor (a kernel of known traffic, '
                         'used to scale hardware byte counters when profiling)')
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit('bench.py measures one GPU: this hot path has no multi-GPU component '
                         '(neurons are independent; see DESIGN.md for how it would shard). Use --gpus 1.')
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    import lava_dl_amd.slayer  # noqa: F401  (fails loudly if the HIP library is missing)

    inp = make_inputs(a.workload, dev)
    job = Cuba(inp)
    for _ in range(a.calibration_copies):
        torch.empty_like(inp['x']).copy_(inp['x'])
    nt = int(torch.tensor(inp['shape']).prod())

    for _ in range(a.warmup):
        job.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        job.step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps

    # per-kernel device time (separate pass so the event records do not perturb the headline number)
    timers = Timers()
    for _ in range(max(3, a.steps // 2)):
        job.step(timers)
    torch.cuda.synchronize()
    op_ms = timers.mean_ms()
    per_op = []
    for name, bpn in job.ops:
        gbs = nt * bpn / (op_ms[name] * 1e-3) / 1e9
        per_op.append(dict(op=name, kernel=job.kernel_of[name], ms=round(op_ms[name], 4),
                           bytes_per_nt=bpn, achieved_GBps=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4)))
    dom = max(per_op, key=lambda r: r['ms'])
    total_bpn = sum(b for _, b in job.ops)
    value = nt / (ms_per_step * 1e-3)

    out = {
        'metric': 'neuron-timesteps/sec fwd+bwd (CUBA) + % of MI355X HBM peak, 1 GPU',
        'value': value, 'unit': 'neuron-timesteps/s', 'n_gpus': 1, 'steps': a.steps, 'warmup': a.warmup,
        'ms_per_step': ms_per_step, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'int32 fixed-point state (fwd) / f32 (bwd), f32 tensors', 'data': 'synthetic',
        'config': {'workload': f'{job.name} {list(inp["shape"])} w_scale=64 per-channel decays',
                   'bytes_per_nt': total_bpn},
        'hbm_frac_whole_step': value * total_bpn / 1e9 / HBM_PEAK_GBS,
        'roofline': {'bound': 'hbm', 'kernel': dom['kernel'], 'op': dom['op'],
                     'achieved': dom['achieved_GBps'], 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': dom['frac'],
                     'traffic': (nt * dom['bytes_per_nt'] * MEASURED_TRAFFIC_FACTOR[dom['kernel']]
                                 if a.workload == 'cuba' else None),
                     'traffic_unit': 'bytes per launch (rocprofv3 FETCH_SIZE x2 + WRITE_SIZE, see profiles/)'},
        'per_op': per_op,
    }
    if not a.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(a.workload, inp)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
