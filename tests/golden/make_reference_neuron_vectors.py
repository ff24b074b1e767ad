"""Input/output vectors of the reference's neuron classes: alif, adrf, adrf_iz and sigma_delta, which no fixture
of the reference pins, and cuba, rf and rf_iz, whose dynamics the netx fixtures pin but whose class-level behaviour
(surrogate constants, carried states over two calls, graded spikes, per-channel parameters) they do not.

Run in the build container only (it reads /root/reference, which never travels):

    python tests/golden/make_reference_neuron_vectors.py

What is imported: `neuron/{base,cuba,alif,rf,rf_iz,adrf,adrf_iz,sigma_delta}.py` of the reference and what they import
(`neuron/dynamics/*.py`, `spike/`, `axon/`, `dendrite/`, `utils/{quantize,int_utils,utils}.py`, `utils/time/`,
`utils/filter/`, `jitconfig.py`), under empty stand-in packages for `slayer`, `slayer.utils`, `slayer.neuron` and
`slayer.neuron.dynamics`, so that the package `__init__` files that pull in h5py / matplotlib / lava do not run.
Only the CPU branch is exercised.  No bytecode is written.

Every case: a neuron with persistent state is built from the recorded keyword arguments, called on two
consecutive inputs (the second call starts from the carried state), and its outputs and carried states are stored.
Per-channel parameters are drawn at random by the neuron on its first call and are stored as well.  A second
neuron with the same parameters and no carried state runs the first input again with autograd on, and the
gradient of sum(output * g) with respect to the input(s) is stored together with g.
"""
import importlib
import json
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


def load_reference_neurons():
    sys.dont_write_bytecode = True
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.dirname(SRC))))
    for name, path in (('lava', root + '/lava'), ('lava.lib', root + '/lava/lib'), ('lava.lib.dl', root + '/lava/lib/dl'),
                       ('lava.lib.dl.slayer', SRC), ('lava.lib.dl.slayer.neuron', SRC + '/neuron'),
                       ('lava.lib.dl.slayer.neuron.dynamics', SRC + '/neuron/dynamics')):
        _stand_in(name, path)
    utils = _stand_in('lava.lib.dl.slayer.utils', SRC + '/utils')
    quantize = importlib.import_module('lava.lib.dl.slayer.utils.quantize')
    utils.quantize, utils.QUANTIZE_MODE = quantize.quantize, quantize.MODE       # what utils/__init__.py re-exports
    return {name: importlib.import_module('lava.lib.dl.slayer.neuron.' + name)
            for name in ('alif', 'adrf', 'adrf_iz', 'sigma_delta', 'cuba', 'rf', 'rf_iz')}


def events(gen, shape, p, amp):
    return (torch.rand(shape, generator=gen) < p).float() * torch.randn(shape, generator=gen) * amp


CASES = [
    # name, module, constructor arguments, complex input?, input (p, amplitude)
    ('alif_shared', 'alif', dict(threshold=0.5, threshold_step=0.25, current_decay=0.25, voltage_decay=0.1,
                                 threshold_decay=0.05, refractory_decay=0.2), False, (0.3, 1.0)),
    ('alif_graded_channel', 'alif', dict(threshold=0.6, threshold_step=0.3, current_decay=[0.1, 0.4],
                                         voltage_decay=[0.05, 0.2], threshold_decay=[0.02, 0.1],
                                         refractory_decay=[0.1, 0.3], shared_param=False, graded_spike=True,
                                         scale=32), False, (0.4, 1.5)),
    ('adrf_shared', 'adrf', dict(threshold=0.4, threshold_step=0.2, period=8, decay=0.08, threshold_decay=0.05,
                                 refractory_decay=0.2), True, (0.4, 1.0)),
    ('adrf_channel', 'adrf', dict(threshold=0.5, threshold_step=0.25, period=[5, 20], decay=[0.02, 0.2],
                                  threshold_decay=0.05, refractory_decay=0.3, shared_param=False), True, (0.4, 1.0)),
    ('adrf_iz_shared', 'adrf_iz', dict(threshold=0.4, threshold_step=0.2, period=8, decay=0.08,
                                       threshold_decay=0.05, refractory_decay=0.2), True, (0.4, 1.0)),
    ('adrf_iz_graded', 'adrf_iz', dict(threshold=0.5, threshold_step=0.1, period=12, decay=0.05,
                                       threshold_decay=0.1, refractory_decay=0.4, graded_spike=True), True, (0.5, 1.2)),
    ('sigma_delta_relu', 'sigma_delta', dict(threshold=0.1, activation='relu'), False, (0.5, 0.3)),
    # cum_error=True is left out: that branch of the reference (axon/delta.py:39, `1 - (bool tensor)`) raises
    # under the installed torch
    ('cuba_shared', 'cuba', dict(threshold=0.5, current_decay=0.25, voltage_decay=0.1), False, (0.3, 1.0)),
    ('cuba_graded_channel', 'cuba', dict(threshold=0.6, current_decay=[0.1, 0.4], voltage_decay=[0.05, 0.2],
                                         shared_param=False, graded_spike=True, scale=32), False, (0.4, 1.5)),
    ('rf_shared', 'rf', dict(threshold=0.4, period=8, decay=0.08), True, (0.4, 1.0)),
    ('rf_channel', 'rf', dict(threshold=0.5, period=[5, 20], decay=[0.02, 0.2], shared_param=False), True, (0.4, 1.0)),
    ('rf_iz_shared', 'rf_iz', dict(threshold=0.4, period=8, decay=0.08), True, (0.4, 1.0)),
    ('rf_iz_graded', 'rf_iz', dict(threshold=0.5, period=12, decay=0.05, graded_spike=True), True, (0.5, 1.2)),
]
ACTIVATIONS = {'relu': torch.relu}
SHAPE = (3, 6, 48)


def main():
    mods = load_reference_neurons()
    out = {}
    for k, (name, module, kwargs, is_complex, (p, amp)) in enumerate(CASES):
        gen = torch.Generator().manual_seed(5100 + k)
        torch.manual_seed(5200 + k)                      # per-channel parameters are drawn with the global generator
        build = dict(kwargs, persistent_state=True)
        if 'activation' in build:
            build['activation'] = ACTIVATIONS[build['activation']]
        neuron = mods[module].Neuron(**build)
        out[f'{name}/kwargs'] = np.array(json.dumps(kwargs))
        out[f'{name}/module'] = np.array(module)
        for call in (0, 1):
            if is_complex:
                x = (events(gen, SHAPE, p, amp), events(gen, SHAPE, p, amp))
                out[f'{name}/in{call}_real'], out[f'{name}/in{call}_imag'] = x[0].numpy(), x[1].numpy()
            else:
                x = events(gen, SHAPE, p, amp)
                out[f'{name}/in{call}'] = x.numpy()
            with torch.no_grad():
                if module == 'adrf_iz':                  # its forward() passes spike() one argument too few
                    y = neuron.spike(*neuron.dynamics(x))
                else:
                    y = neuron(x)
            out[f'{name}/out{call}'] = y.numpy()
            for sname, state in neuron.named_buffers(recurse=True):
                out[f'{name}/state{call}/{sname}'] = state.detach().numpy().copy()
        for pname, prm in neuron.named_parameters(recurse=True):
            out[f'{name}/param/{pname}'] = prm.detach().numpy().copy()
        # gradients: a fresh neuron without carried state and with the same parameters, first input again
        torch.manual_seed(5200 + k)
        fresh = mods[module].Neuron(**dict(build, persistent_state=False))
        g = torch.randn(SHAPE, generator=gen)
        if is_complex:
            leaves = [torch.tensor(out[f'{name}/in0_real']).requires_grad_(),
                      torch.tensor(out[f'{name}/in0_imag']).requires_grad_()]
            y = fresh.spike(*fresh.dynamics(tuple(leaves))) if module == 'adrf_iz' else fresh(tuple(leaves))
        else:
            leaves = [torch.tensor(out[f'{name}/in0']).requires_grad_()]
            y = fresh(leaves[0])
        for pname, prm in fresh.named_parameters(recurse=True):
            assert np.array_equal(prm.detach().numpy(), out[f'{name}/param/{pname}']), pname
        assert np.array_equal(y.detach().numpy(), out[f'{name}/out0'])
        y.backward(g)
        out[f'{name}/grad_out'] = g.numpy()
        for i, leaf in enumerate(leaves):
            out[f'{name}/grad_in{i}'] = leaf.grad.numpy()
        print(name, 'events per call', [float((out[f'{name}/out{c}'] != 0).mean()) for c in (0, 1)])
    path = os.path.join(DST, 'reference_neuron_vectors.npz')
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
