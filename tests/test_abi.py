"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares (and nothing the binding does not know), argument validation rejects bad sizes before any
launch, and the python operators refuse CPU tensors."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'slayer_hip.h')


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(slayer_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    from lava_dl_amd.slayer import _native
    names = declared_symbols()
    assert len(names) >= 14
    handle = ctypes.CDLL(_native.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f'{n} declared in slayer_hip.h but not exported'
    assert sorted(_native.EXPORTS) == names, 'python binding and header disagree'
    assert _native.lib().slayer_abi_version() == _native.ABI_VERSION == 4
    assert b'success' in _native.lib().slayer_error_string(0)
    assert b'inconsistent' in _native.lib().slayer_error_string(-1)


def test_argument_validation_happens_before_any_launch():
    """Invalid sizes return SLAYER_E* without touching the device (safe without a GPU)."""
    from lava_dl_amd.slayer import _native
    L = _native.lib()
    one = ctypes.c_void_p(16)          # non-null dummy pointers; never dereferenced on these paths
    EINVAL, ENULL, ERANGE = -1, -2, -3
    # M not a multiple of neurons_per_batch
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 64, 10, 3, 1, 1, 8, None) == EINVAL
    # 3 decays do not divide 4 neurons per batch
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 64, 8, 4, 3, 1, 8, None) == EINVAL
    # state count neither 1 nor M
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 64, 8, 4, 1, 5, 8, None) == EINVAL
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 0, 8, 4, 1, 1, 8, None) == EINVAL      # w_scale 0
    assert L.slayer_li_fwd(None, one, one, one, 1.0, 64, 8, 4, 1, 1, 8, None) == ENULL
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 64, 8, 4, 1, 1, 1 << 31, None) == ERANGE
    assert L.slayer_li_fwd(one, one, one, one, 1.0, 64, 0, 4, 1, 1, 8, None) == 0          # empty is fine
    assert L.slayer_li_bwd(one, one, one, one, one, None, 8, 4, 1, 8, None) == ENULL       # grad wanted, no workspace
    # delays folded into a fused block: a table needs a sampling time
    bad = _native.Delays(16, None, None, None, 0, 0, 0.0)
    assert L.slayer_cuba_fwd(None, one, one, None, None, one, one, one, one, one, 1.0, 1.0, 0, 1.0, 64,
                             8, 4, 1, 1, 1, 1, 8, ctypes.byref(bad), None) == EINVAL
    # the allocation-free form refuses what its built-in scratch cannot hold
    assert L.slayer_li_bwd_static(one, one, one, one, one, (1 << 20) + 64, 64, 1, 8, None) == -4
    assert L.slayer_li_bwd_static(one, one, one, one, one, 8192, 8192, 8192, 8, None) == -4
    assert b'scratch' in L.slayer_error_string(-4)
    assert L.slayer_res_bwd(one, one, one, None, one, one, one, one, one, one, one, 8, 4, 1, 8, None) == ENULL
    assert L.slayer_conv(one, one, one, 0, 1.0, 8, 8, None) == EINVAL
    # which float backward passes are wave scans: tensors of 2^20 elements and more, whole quads or rows of 64+ steps
    assert L.slayer_bwd_takes_scan(4096, 64, 300) == 1 and L.slayer_bwd_takes_scan(4096, 64, 301) == 1
    assert L.slayer_bwd_takes_scan(512, 64, 300) == 0 and L.slayer_bwd_takes_scan(1 << 20, 64, 3) == 0
    # the range flag needs a device to map its word for; without one the call says so instead of failing
    raised = ctypes.c_int(7)
    code = L.slayer_range_status(ctypes.byref(raised), 0)
    assert code == (0 if torch.cuda.is_available() else -5)
    assert b'range flag' in L.slayer_error_string(-5)
    assert L.slayer_conv(one, one, one, 13000, 1.0, 8, 13000, None) == ERANGE      # rows and filter beyond the window
    assert L.slayer_shift(one, one, None, 1, 1.0, 8, 3, 8, None) == EINVAL
    assert L.slayer_spike_fwd(one, one, one, 3, 0.0, 0, 1.0, 8, None) == EINVAL             # 3 thresholds for 8 samples
    assert L.slayer_ath_fwd(one, one, one, one, one, one, one, 1 << 40, 0, 64, 8, 4, 1, 1, 1, 1, 8, None) == ERANGE
    # delay backward: sampling time 0, rows not a multiple of the neurons per batch, sums wanted without workspace
    assert L.slayer_delay_bwd(one, None, one, one, None, 1, 0.0, None, 8, 4, 8, None) == EINVAL
    assert L.slayer_delay_bwd(one, None, one, one, None, 1, 1.0, None, 10, 4, 8, None) == EINVAL
    assert L.slayer_delay_bwd(one, one, one, one, one, 0, 1.0, None, 8, 4, 8, None) == ENULL
    # fused resonate-and-fire forward: the integer spike decision needs a positive scale
    rf_tail = (1.0, 0, 1.0)
    assert L.slayer_rf_fwd(one, one, one, None, None, one, one, one, one, one, one, one, *rf_tail, 0,
                           8, 4, 1, 1, 1, 1, 8, None, None) == EINVAL
    assert L.slayer_rf_fwd(one, one, one, None, None, one, one, one, one, one, one, one, *rf_tail, -64,
                           8, 4, 1, 1, 1, 1, 8, None, None) == EINVAL
    assert L.slayer_rf_fwd(one, None, one, None, None, one, one, one, one, one, one, one, *rf_tail, 64,
                           8, 4, 1, 1, 1, 1, 8, None, None) == ENULL                               # real without imag trace


def test_operators_refuse_cpu_tensors():
    import lava_dl_amd.slayer as slayer
    x = torch.zeros(2, 4, 16)
    d = torch.tensor([100.0])
    z = torch.tensor([0.0])
    with pytest.raises(RuntimeError, match='no CPU implementation'):
        slayer.neuron.dynamics.leaky_integrator.dynamics(x, d, z, 64)
    with pytest.raises(RuntimeError):
        slayer.neuron.dynamics.adaptive_threshold.dynamics(x, z, d, z, d, 0.5, 1.0, 64)
    with pytest.raises(RuntimeError):
        slayer.neuron.dynamics.resonator.dynamics(x, x, d, d, z, z, 64)
    with pytest.raises(RuntimeError):
        slayer.spike.Spike.apply(x, 1.0, 1.0, 1.0, False, 0, 1)
    with pytest.raises(RuntimeError):
        slayer.spike.complex.Spike.apply(x, x, 1.0, 1.0, 1.0, False, 0, 1)
    with pytest.raises(RuntimeError):
        slayer.utils.time.shift(x, 2)
    with pytest.raises(RuntimeError):
        slayer.utils.filter.conv(x, torch.ones(3))


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, 'lava-dl_amd')
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(('.py', '.hip', '.h')):
                text = open(os.path.join(d, f)).read()
                assert 'oracle' not in text, f'{f} mentions the oracle'


def test_right_shift_to_zero():
    import lava_dl_amd.slayer as slayer
    x = torch.tensor([-8193, -4097, -4096, -4095, -1, 0, 1, 4095, 4096, 8191], dtype=torch.int64)
    assert slayer.utils.int_utils.right_shift_to_zero(x, 12).tolist() == [-2, -1, -1, 0, 0, 0, 0, 0, 1, 1]
    with pytest.raises(Exception):
        slayer.utils.right_shift_to_zero(torch.zeros(2), 12)


def test_missing_library_fails_loudly(tmp_path):
    """Without the built library there is nothing to fall back to: the first use raises and says how to build it
    (checked in a fresh interpreter so that the loaded library of this process is not disturbed)."""
    import subprocess
    import sys
    code = (
        'import sys, torch\n'
        f'sys.path.insert(0, {ROOT!r})\n'
        'import lava_dl_amd.slayer as slayer\n'
        'from lava_dl_amd.slayer import _native\n'
        'try:\n'
        '    _native.lib()\n'
        'except RuntimeError as e:\n'
        '    print("RAISED", e)\n'
        'else:\n'
        '    print("LOADED")\n')
    env = dict(os.environ, SLAYER_HIP_LIB=str(tmp_path / 'libslayer_hip.so'))
    run = subprocess.run([sys.executable, '-c', code], env=env, capture_output=True, text=True, timeout=300)
    assert 'RAISED' in run.stdout and 'is missing' in run.stdout and 'no fallback' in run.stdout.lower(), \
        run.stdout + run.stderr
