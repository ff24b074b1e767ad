"""Input/output vectors of the reference's axonal delay (`axon/delay.py`: the `Delay` module, forward, gradient
of the input and gradient of the delays) and of its per-neuron `utils/time/shift.py` at sampling times other than
1 (where its CPU branch divides the shift by the sampling time twice and its CUDA kernel once).  No fixture that is
present in the reference pins either (the only network with axonal delays, netx/gts/ntidigits, is a git-lfs pointer).

Run in the build container only (it reads /root/reference, which never travels):

    python tests/golden/make_reference_delay_vectors.py

What is imported: `axon/delay.py`, `utils/time/shift.py`, `utils/filter/conv.py` of the reference and what they
import, under empty stand-in packages for `slayer`, `slayer.utils` and `slayer.axon` (the package `__init__` files
that pull in h5py / matplotlib / lava do not run).  Only the CPU branch is exercised.  No bytecode is written.
"""
import importlib
import os
import sys
import types

import numpy as np
import torch

SRC = '/root/reference/src/lava/lib/dl/slayer'
DST = os.path.dirname(os.path.abspath(__file__))


def _stand_in(name, path):
    pkg = types.ModuleType(name)
    pkg.__path__ = [path]
    sys.modules[name] = pkg
    return pkg


def load():
    sys.dont_write_bytecode = True
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.dirname(SRC))))
    for name, path in (('lava', root + '/lava'), ('lava.lib', root + '/lava/lib'), ('lava.lib.dl', root + '/lava/lib/dl'),
                       ('lava.lib.dl.slayer', SRC), ('lava.lib.dl.slayer.axon', SRC + '/axon'),
                       ('lava.lib.dl.slayer.utils', SRC + '/utils')):
        _stand_in(name, path)
    delay = importlib.import_module('lava.lib.dl.slayer.axon.delay')
    shift = importlib.import_module('lava.lib.dl.slayer.utils.time.shift')
    return delay, shift


def main():
    delay_mod, shift_mod = load()
    out = {}
    gen = torch.Generator().manual_seed(6100)
    # ---- Delay module: forward, grad_input, grad_delay
    for name, shape, ts, max_delay, grad_scale in (('delay_nct', (3, 5, 40), 1, 12, 1.0),
                                                   ('delay_nchwt', (2, 4, 3, 2, 36), 1, 10, 0.25),
                                                   ('delay_ts2', (3, 6, 44), 2, 16, 1.0)):
        x = (torch.rand(shape, generator=gen) < 0.3).float() * torch.randn(shape, generator=gen)
        g = torch.randn(shape, generator=gen)
        d = torch.rand(shape[1], generator=gen) * max_delay
        mod = delay_mod.Delay(sampling_time=ts, max_delay=max_delay, grad_scale=grad_scale)
        mod.delay.data = d.clone()
        mod.init = True
        xin = x.clone().requires_grad_()
        y = mod(xin)
        y.backward(g)
        out[f'{name}/in'], out[f'{name}/grad_out'], out[f'{name}/delay'] = x.numpy(), g.numpy(), d.numpy()
        out[f'{name}/cfg'] = np.array([ts, max_delay, grad_scale], dtype=np.float64)
        out[f'{name}/out'] = y.detach().numpy()
        out[f'{name}/grad_in'] = xin.grad.numpy()
        out[f'{name}/grad_delay'] = mod.delay.grad.numpy()
        print(name, 'moved', float((y.detach() != x).float().mean()), 'grad_delay', mod.delay.grad[:3].tolist())
    # ---- per-neuron shift at sampling times other than 1 (CPU branch)
    for name, shape, ts in (('shift_ts2', (2, 6, 40), 2.0), ('shift_ts_half', (2, 3, 2, 32), 0.5)):
        x = torch.randn(shape, generator=gen)
        neurons = shape[1:-1]
        sv = (torch.rand(neurons, generator=gen) * 24 - 6)
        y = shift_mod.shift(x, sv, ts)
        out[f'{name}/in'], out[f'{name}/shift'], out[f'{name}/ts'] = x.numpy(), sv.numpy(), np.array(ts)
        out[f'{name}/out'] = y.numpy()
        # which whole-step shift each row actually received
        steps = []
        rows_in, rows_out = x.reshape(shape[0], -1, shape[-1])[0], y.reshape(shape[0], -1, shape[-1])[0]
        for r in range(rows_in.shape[0]):
            found = [k for k in range(-shape[-1], shape[-1] + 1)
                     if torch.equal(torch.roll(rows_in[r], k)[max(k, 0):shape[-1] + min(k, 0)],
                                    rows_out[r][max(k, 0):shape[-1] + min(k, 0)])
                     and float(rows_out[r][:max(k, 0)].abs().sum() + rows_out[r][shape[-1] + min(k, 0):].abs().sum()) == 0]
            steps.append(found[0] if found else 10 ** 6)
        out[f'{name}/steps'] = np.array(steps)
        print(name, 'shift/ts', (sv.flatten() / ts)[:6].tolist(), 'steps taken', steps[:6])
    path = os.path.join(DST, 'reference_delay_vectors.npz')
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
