"""Loaders for the committed known-answer fixtures (see make_fixtures.py).

Each loader returns float32 tensors shaped [1, neurons, T] ready for the
dynamics API at w_scale = 4096 (the neuron classes' s_scale = 64 * 64), plus
the expected output spike raster.  The reference's lava-side blocks emit a
spike one step after the slayer-side tensor does, so ``expected`` is already
aligned: expected[:, t] is the spike the dynamics must produce at step t,
for t in [0, T-1).
"""
import os
import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
W_SCALE = 4096


def _unpack(b, T):
    return np.unpackbits(b, axis=-1)[..., :T].astype(np.int64)


def dense_lif():
    """LIF dense block: vth=6, du=4095 (full current decay), dv=415.

    Returns dict(x=[1,256,T] synaptic input, current_decay, voltage_decay,
    threshold, expected=[256,T-1]).
    """
    z = np.load(os.path.join(HERE, 'netx_dense_lif.npz'))
    T = int(z['num_steps'])
    a = z['weight'].astype(np.int64) @ _unpack(z['in_bits'], T)      # [256, T]
    x = torch.tensor(a * 64 / W_SCALE, dtype=torch.float32).reshape(1, 256, T)
    return dict(x=x, current_decay=4096.0, voltage_decay=415.0,
                threshold=6 / 64 + 0.01 / W_SCALE,
                expected=_unpack(z['out_bits'], T)[:, 1:])


def dense_lif_block():
    """The same dense LIF block before its synapse: dict(spikes=[1,200,T] 0/1 input, weight=[256,200] synaptic
    weights in units of the state scale (integer weight * 64 / 4096), then as dense_lif())."""
    z = np.load(os.path.join(HERE, 'netx_dense_lif.npz'))
    T = int(z['num_steps'])
    fx = dense_lif()
    fx['spikes'] = torch.tensor(_unpack(z['in_bits'], T), dtype=torch.float32).reshape(1, -1, T)
    fx['weight'] = torch.tensor(z['weight'].astype(np.float64) * 64 / W_SCALE, dtype=torch.float32)
    return fx


def complex_dense_rf():
    """RF dense block: vth=25, period=11, alpha=0.05 (no reset, phase spike)."""
    z = np.load(os.path.join(HERE, 'netx_complex_dense_rf.npz'))
    T = int(z['num_steps'])
    s = _unpack(z['in_bits'], T)
    ar = z['weight_real'].astype(np.int64) @ s
    ai = z['weight_imag'].astype(np.int64) @ s
    f = lambda a: torch.tensor(a * 64 / W_SCALE, dtype=torch.float32).reshape(1, 256, T)
    return dict(xr=f(ar), xi=f(ai),
                sin_decay=float(int(0.95 * np.sin(2 * np.pi / 11) * 4096)),
                cos_decay=float(int(0.95 * np.cos(2 * np.pi / 11) * 4096)),
                threshold=25 * 64 / W_SCALE,
                expected=_unpack(z['out_bits'], T)[:, 1:])


def complex_input_rf_iz():
    """RF_IZ input block: vth=1.1, period=7, alpha=0.05; the same 0/1 input
    drives the real and the imaginary port; spike = imag >= vth with reset
    (real -> 0, imag -> vth - 1).  Here the lava block has no extra latency,
    so expected[:, t] is the spike at step t for all t.
    """
    z = np.load(os.path.join(HERE, 'netx_complex_dense_rf.npz'))
    T = int(z['num_steps'])
    s = _unpack(z['in_bits'], T)
    x = torch.tensor(s * 64 / W_SCALE, dtype=torch.float32).reshape(1, 200, T)
    return dict(x=x,
                sin_decay=float(int(0.95 * np.sin(2 * np.pi / 7) * 4096)),
                cos_decay=float(int(0.95 * np.cos(2 * np.pi / 7) * 4096)),
                threshold=1.1 * 64 / W_SCALE,
                expected=_unpack(z['iz_out_bits'], T))


def reference_big_state_vectors():
    """Vectors written by make_reference_vectors.py from the reference's CPU branch: states beyond 2**24 at
    w_scale = 4096 next to a threshold.  Returns (li_cases, res_cases); each case is a dict of float32
    tensors, expected outputs already divided by w_scale (exact: integers below 2**31 times 2**-12)."""
    z = np.load(os.path.join(HERE, 'reference_big_state_vectors.npz'))

    def state(a):
        return (torch.tensor(a.astype(np.float64)) / W_SCALE).float()

    li, res = [], []
    k = 0
    while f'li{k}_thr' in z:
        li.append(dict(threshold=float(z[f'li{k}_thr']), x=torch.tensor(z[f'li{k}_x']), out=state(z[f'li{k}_out'])))
        k += 1
    k = 0
    while f'res{k}_thr' in z:
        res.append(dict(threshold=float(z[f'res{k}_thr']), xr=torch.tensor(z[f'res{k}_xr']),
                        xi=torch.tensor(z[f'res{k}_xi']), sin=torch.tensor(z[f'res{k}_sin']),
                        cos=torch.tensor(z[f'res{k}_cos']), re=state(z[f'res{k}_re']), im=state(z[f'res{k}_im'])))
        k += 1
    return li, res


def reference_neuron_vectors():
    """Vectors written by make_reference_neuron_vectors.py from the reference's own neuron classes (alif, adrf,
    adrf_iz, sigma_delta; CPU branch, persistent state, two consecutive calls).  Returns a list of dicts:
    name, module, kwargs, inputs [call] (tensor or (real, imag)), outputs [call], states [call] {name: tensor},
    params {name: tensor}, grad_out and grad_in (list: one entry per input tensor of the first call)."""
    import json
    z = np.load(os.path.join(HERE, 'reference_neuron_vectors.npz'))
    names = sorted({k.split('/')[0] for k in z.files})
    cases = []
    for name in names:
        pick = {k[len(name) + 1:]: z[k] for k in z.files if k.startswith(name + '/')}
        case = dict(name=name, module=str(pick['module']), kwargs=json.loads(str(pick['kwargs'])),
                    inputs=[], outputs=[], states=[], params={})
        for call in (0, 1):
            if f'in{call}' in pick:
                case['inputs'].append(torch.tensor(pick[f'in{call}']))
            else:
                case['inputs'].append((torch.tensor(pick[f'in{call}_real']), torch.tensor(pick[f'in{call}_imag'])))
            case['outputs'].append(torch.tensor(pick[f'out{call}']))
            case['states'].append({k.split('/', 1)[1]: torch.tensor(v) for k, v in pick.items()
                                   if k.startswith(f'state{call}/')})
        case['params'] = {k.split('/', 1)[1]: torch.tensor(v) for k, v in pick.items() if k.startswith('param/')}
        # gradient of sum(output * grad_out) with respect to the first input (no carried state)
        case['grad_out'] = torch.tensor(pick['grad_out'])
        case['grad_in'] = [torch.tensor(pick[f'grad_in{i}']) for i in (0, 1) if f'grad_in{i}' in pick]
        cases.append(case)
    return cases


def reference_delay_vectors():
    """Vectors written by make_reference_delay_vectors.py from the reference's own `axon.Delay` module (forward,
    gradient of the input, gradient of the delays) and per-neuron `shift` at sampling times other than 1 (CPU branch).
    Returns {case name: {key: tensor}}."""
    z = np.load(os.path.join(HERE, 'reference_delay_vectors.npz'))
    cases = {}
    for k in z.files:
        name, key = k.split('/', 1)
        cases.setdefault(name, {})[key] = torch.tensor(z[k])
    return cases
