"""Input/output vectors of the reference's CPU branch for the two float32-promotion corners that
nothing else pins.

Run in the build container only (it reads /root/reference, which never travels):

    python tests/golden/make_reference_vectors.py

What is imported: `neuron/dynamics/leaky_integrator.py` and `neuron/dynamics/resonator.py` of the
reference (plus the two helper modules they import, `utils/int_utils.py`, `utils/utils.py`, and
`jitconfig.py`), as sub-modules of empty stand-in packages so that no package `__init__` of the
reference runs.  Only the CPU branch is exercised (CPU tensors).  No bytecode is written.

Corners (states of magnitude beyond 2**24 at w_scale = 4096, where int64 -> float32 conversion rounds):
  * leaky integrator with a threshold: the reset decision compares float32(state) with
    float32(threshold * w_scale) (leaky_integrator.py:210-231);
  * resonator with a threshold: decision as above, and the imaginary reset value goes through a
    mixed int64 / float32 expression before it is cast back to int64 (resonator.py:333-376).

Outputs are stored as the integer state (output * w_scale is exact: w_scale is a power of two), inputs as
float32, in `reference_big_state_vectors.npz` (about 100 KB).
"""
import importlib
import os
import sys
import types

import numpy as np
import torch

SRC = '/root/reference/src/lava/lib/dl/slayer'
DST = os.path.dirname(os.path.abspath(__file__))
W = 4096


def _stand_in(name, path):
    pkg = types.ModuleType(name)
    pkg.__path__ = [path]
    sys.modules[name] = pkg
    return pkg


def load_reference_dynamics():
    sys.dont_write_bytecode = True
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.dirname(SRC))))
    for name, path in (('lava', root + '/lava'), ('lava.lib', root + '/lava/lib'), ('lava.lib.dl', root + '/lava/lib/dl'),
                       ('lava.lib.dl.slayer', SRC), ('lava.lib.dl.slayer.utils', SRC + '/utils'),
                       ('lava.lib.dl.slayer.neuron', SRC + '/neuron'),
                       ('lava.lib.dl.slayer.neuron.dynamics', SRC + '/neuron/dynamics')):
        _stand_in(name, path)
    li = importlib.import_module('lava.lib.dl.slayer.neuron.dynamics.leaky_integrator')
    res = importlib.import_module('lava.lib.dl.slayer.neuron.dynamics.resonator')
    return li, res


def li_case(gen, thr, shape=(1, 32, 200)):
    """No decay; now and then a jump to just below threshold * w >= 2**24, then steps of a few LSB."""
    jump = (torch.rand(shape, generator=gen) < 0.1).float()
    x = jump * (thr - torch.randint(0, 6, shape, generator=gen).float() / W) \
        + (1 - jump) * torch.randint(-2, 4, shape, generator=gen).float() / W
    return x


def res_case(gen, thr, shape=(1, 32, 200)):
    """Per-channel rotation from none (sin 0, cos 4096) to a few degrees per step; the imaginary input
    jumps to just below the threshold now and then, the real input wanders by a few LSB, and a large
    negative kick sends some rows far below -2**24 as well."""
    C = shape[1]
    sin = torch.zeros(C)
    cos = torch.full((C,), 4096.0)
    ang = torch.linspace(0, 0.08, C - C // 2)
    sin[C // 2:] = torch.round(4090 * torch.sin(ang))
    cos[C // 2:] = torch.round(4090 * torch.cos(ang))
    jump = (torch.rand(shape, generator=gen) < 0.08).float()
    kick = (torch.rand(shape, generator=gen) < 0.01).float()
    xi = jump * (thr - torch.randint(0, 6, shape, generator=gen).float() / W) \
        + (1 - jump) * torch.randint(-2, 4, shape, generator=gen).float() / W - kick * 1.5 * thr
    xr = torch.randint(-3, 4, shape, generator=gen).float() / W \
        + (torch.rand(shape, generator=gen) < 0.02).float() * thr * 0.7
    return xr, xi, sin, cos


def exact_int(t):
    v = (t.double() * W)
    assert torch.equal(v, v.round()) and float(v.abs().max()) < 2 ** 31
    return v.to(torch.int32).numpy()


def main():
    li, res = load_reference_dynamics()
    out = {}
    zero = torch.tensor([0.0])
    for k, thr in enumerate([4100.0, 4096.0 + 1.0 / 4096, 7000.3, 16384.0]):
        gen = torch.Generator().manual_seed(4200 + k)
        x = li_case(gen, thr)
        y = li.dynamics(x, zero, zero, W, thr)
        out[f'li{k}_thr'] = np.float64(thr)
        out[f'li{k}_x'] = x.numpy()
        out[f'li{k}_out'] = exact_int(y)
        print('li', thr, 'fired', float((y * W >= thr * W).float().mean()), 'max', float(y.abs().max()) * W)
    for k, thr in enumerate([4100.0, 4096.0 + 1.0 / 4096, 7000.3]):
        gen = torch.Generator().manual_seed(4300 + k)
        xr, xi, sin, cos = res_case(gen, thr)
        re, im = res.dynamics(xr, xi, sin, cos, zero, zero, W, thr)
        out[f'res{k}_thr'] = np.float64(thr)
        out[f'res{k}_xr'] = xr.numpy()
        out[f'res{k}_xi'] = xi.numpy()
        out[f'res{k}_sin'] = sin.numpy()
        out[f'res{k}_cos'] = cos.numpy()
        out[f'res{k}_re'] = exact_int(re)
        out[f'res{k}_im'] = exact_int(im)
        print('res', thr, 'fired', float((im * W >= thr * W).float().mean()), 'max |im|', float(im.abs().max()) * W,
              'min im', float(im.min()) * W)
    path = os.path.join(DST, 'reference_big_state_vectors.npz')
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
