"""ctypes binding of libslayer_hip.so (C ABI declared in include/slayer_hip.h).

The shared library is the only implementation: there is no CPU or eager
fallback.  Loading fails loudly when the library has not been built, and every
operator raises when handed a tensor that is not float32 on a GPU.
"""
import contextlib
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# SLAYER_HIP_LIB points at an alternative build of the same library (e.g. a tuning build)
LIB_PATH = os.environ.get('SLAYER_HIP_LIB') or os.path.join(_HERE, 'libslayer_hip.so')
ABI_VERSION = 4

_lib = None
_lib_lock = threading.Lock()       # forward runs on the user thread, backward on an autograd thread

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_INT = ctypes.c_int
_F = ctypes.c_float
_D = ctypes.c_double



class Delays(ctypes.Structure):
    """struct slayer_delays of include/slayer_hip.h (device pointers as integers)."""
    _fields_ = [('in_shift', _P), ('out_delay', _P), ('out_head', _P), ('spike_last', _P),
                ('in_steps', _I64), ('out_steps', _I64), ('sampling_time', _F),
                ('delayed_spikes', _P), ('grad_out_delay', _P), ('grad_workspace', _P)]


_DP = ctypes.POINTER(Delays)

_SIGNATURES = {
    'slayer_abi_version': (_INT, []),
    'slayer_error_string': (ctypes.c_char_p, [_INT]),
    'slayer_range_status': (_INT, [ctypes.POINTER(_INT), _INT]),
    'slayer_range_word': (_P, []),
    'slayer_bwd_takes_scan': (_INT, [_I64, _I64, _I64]),
    'slayer_li_fwd': (_INT, [_P, _P, _P, _P, _D, _INT, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_li_bwd': (_INT, [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    'slayer_li_bwd_static': (_INT, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    'slayer_ath_fwd': (_INT, [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _INT,
                              _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_res_fwd': (_INT, [_P, _P, _P, _P, _P, _P, _P, _P, _D, _INT,
                              _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_res_bwd': (_INT, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    'slayer_spike_fwd': (_INT, [_P, _P, _P, _I64, _F, _INT, _F, _I64, _P]),
    'slayer_spike_bwd': (_INT, [_P, _P, _P, _P, _I64, _F, _F, _F, _INT, _I64, _P]),
    'slayer_cspike_fwd': (_INT, [_P, _P, _P, _P, _I64, _F, _P, _I64, _F, _INT, _F, _I64, _I64, _P]),
    'slayer_cspike_bwd': (_INT, [_P, _P, _P, _P, _P, _P, _I64, _F, _F, _F, _INT, _I64, _P]),
    'slayer_shift': (_INT, [_P, _P, _P, _I64, _F, _I64, _I64, _I64, _P]),
    'slayer_delay_bwd': (_INT, [_P, _P, _P, _P, _P, _I64, _F, _P, _I64, _I64, _I64, _P]),
    'slayer_conv_synapse': (_INT, [_P, _P, _P] + [_I64] * 14 + [_P]),
    'slayer_conv_synapse_input_grad': (_INT, [_P, _P, _P] + [_I64] * 14 + [_P]),
    'slayer_conv_synapse_wgrad_workspace': (_I64, [_I64] * 11),
    'slayer_conv_synapse_wgrad': (_INT, [_P, _P, _P] + [_I64] * 14 + [_P, _I64, _P]),
    'slayer_conv': (_INT, [_P, _P, _P, _I64, _F, _I64, _I64, _P]),
    'slayer_corr': (_INT, [_P, _P, _P, _I64, _F, _I64, _I64, _P]),
    'slayer_apth_fwd': (_INT, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _INT,
                               _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_adres_fwd': (_INT, [_P] * 14 + [_I64, _I64, _INT] + [_I64] * 10 + [_P]),
    'slayer_delta_fwd': (_INT, [_P] * 9 + [_INT, _F] + [_I64] * 7 + [_P]),
    'slayer_delta_bwd': (_INT, [_P] * 6 + [_F, _F] + [_I64] * 4 + [_P]),
    'slayer_cumsum': (_INT, [_P, _P, _P, _I64, _INT, _I64, _I64, _P]),
    'slayer_cuba_fwd': (_INT, [_P] * 10 + [_D, _F, _INT, _F, _INT] + [_I64] * 7 + [_DP, _P]),
    'slayer_cuba_bwd': (_INT, [_P] * 8 + [_F, _F, _F, _INT, _P] + [_I64] * 5 + [_DP, _P]),
    'slayer_rf_fwd': (_INT, [_P] * 12 + [_F, _INT, _F, _INT] + [_I64] * 7 + [_DP, _P]),
    'slayer_rf_bwd': (_INT, [_P] * 9 + [_F, _F, _F, _INT, _P] + [_I64] * 4 + [_DP, _P]),
    'slayer_alif_fwd': (_INT, [_P] * 17 + [_I64, _I64, _INT, _F, _INT] + [_I64] * 11 + [_DP, _P]),
    'slayer_alif_bwd': (_INT, [_P] * 9 + [_F, _F, _INT, _P] + [_I64] * 5 + [_DP, _P]),
    'slayer_cuba_recurrent_fwd': (_INT, [_P] * 10 + [_F, _INT, _F, _INT] + [_I64] * 7 + [_P]),
    'slayer_alif_recurrent_fwd': (_INT, [_P] * 17 + [_F, _I64, _INT, _F, _INT] + [_I64] * 11 + [_P]),
    'slayer_recurrent_bwd': (_INT, [_P] * 5 + [_F, _F, _F, _INT] + [_I64] * 3 + [_P]),
    'slayer_recurrent_steps_workspace': (_I64, [_I64, _I64, _I64, _INT]),
    'slayer_cuba_recurrent_steps_fwd': (_INT, [_P] * 10 + [_F, _INT, _F, _INT] + [_I64] * 7 + [_P, _I64, _P]),
    'slayer_alif_recurrent_steps_fwd': (_INT, [_P] * 17 + [_F, _I64, _INT, _F, _INT] + [_I64] * 11 + [_P, _I64, _P]),
    'slayer_recurrent_steps_bwd': (_INT, [_P] * 5 + [_F, _F, _F, _INT] + [_I64] * 3 + [_P, _I64, _P]),
    'slayer_li_fwd_naive': (_INT, [_P, _P, _P, _P, _D, _INT, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_li_bwd_naive': (_INT, [_P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    'slayer_ath_fwd_naive': (_INT, [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _INT,
                                    _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_res_fwd_naive': (_INT, [_P, _P, _P, _P, _P, _P, _P, _P, _D, _INT,
                                    _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    'slayer_res_bwd_naive': (_INT, [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
}

EXPORTS = tuple(_SIGNATURES)


def lib():
    """The loaded library (torch is imported first so that its HIP runtime,
    which has the same soname as the one the library was linked against, is the
    single runtime in the process)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f'{LIB_PATH} is missing: build it with `make -C lava-dl_amd/csrc` '
                    '(hipcc, gfx950). There is no fallback implementation.')
            handle = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = res
                fn.argtypes = args
            if handle.slayer_abi_version() != ABI_VERSION:
                raise RuntimeError('libslayer_hip.so ABI version mismatch; rebuild the library')
            _lib = handle
    return _lib


def check(code):
    if code != 0:
        msg = lib().slayer_error_string(code).decode()
        raise RuntimeError(f'libslayer_hip call failed ({code}): {msg}')
    if (_range_word or _find_range_word()).value:
        _range_raised()


# ---- range of the 32-bit fixed-point states -------------------------------------------------------------------
# The forward kernels raise a flag (one word of pinned host memory, slayer_range_status in include/slayer_hip.h)
# when a state comes within a factor of two of the int32 limit, where the reference's int64 CPU branch
# (neuron/dynamics/leaky_integrator.py:213) would simply go on.  Every operator call looks at the word after its
# launch -- a plain memory read -- so an overflow of a launch that has completed is reported by the next call, and
# range_check() reports it on demand.
_range_word = None
_range_policy = 'raise'


def _find_range_word():
    global _range_word
    addr = lib().slayer_range_word()
    if not addr:                      # no device to map the word for: nothing can be launched either
        return ctypes.c_uint(0)
    _range_word = ctypes.c_uint.from_address(addr)
    return _range_word


def _range_raised():
    if _range_policy == 'ignore':           # nobody is looking: the flag stays up until someone lowers it
        return
    clear_range_flag()
    msg = ('a fixed-point state of a slayer kernel came within a factor of two of the 32-bit range (or a decay '
           'multiplier lies beyond +-8191): results since the last check may differ from a 64-bit evaluation. '
           'Lower w_scale or the input magnitude, or run with debug=True to compare against the 64-bit kernels.')
    if _range_policy == 'raise':
        raise OverflowError(msg)
    if _range_policy == 'warn':
        import warnings
        warnings.warn(msg, RuntimeWarning, stacklevel=3)


def range_policy(mode=None):
    """What a raised range flag does when an operator call or ``range_check`` sees it: ``'raise'`` (default,
    OverflowError), ``'warn'`` (RuntimeWarning) or ``'ignore'`` (nothing happens and the flag stays up until
    ``clear_range_flag``).  Reporting lowers the flag.  Returns the mode that was set before."""
    global _range_policy
    before = _range_policy
    if mode is not None:
        if mode not in ('raise', 'warn', 'ignore'):
            raise ValueError(f'unknown range policy {mode!r}')
        _range_policy = mode
    return before


def range_flag():
    """True when a launch that has completed raised the range flag since it was last cleared."""
    return bool((_range_word or _find_range_word()).value)


def clear_range_flag():
    """Lowers the flag; returns whether it was up."""
    raised = ctypes.c_int(0)
    lib().slayer_range_status(ctypes.byref(raised), 1)
    return bool(raised.value)


def range_check(sync=True):
    """Waits for the device (unless ``sync`` is false) and applies the policy to the flag: the definite answer for
    everything launched so far."""
    if sync and torch.cuda.is_available():
        torch.cuda.synchronize()
    if range_flag():
        _range_raised()


def require_gpu(*tensors):
    """Same conditions the reference kernels assert (CHECK_INPUT / CHECK_DEVICE,
    neuron/dynamics/leaky_integrator.cu:14-17,120-124), raised as RuntimeError."""
    dev = None
    for t in tensors:
        if not torch.is_tensor(t):
            raise RuntimeError(f'expected a tensor, got {type(t)}')
        if not t.is_cuda:
            raise RuntimeError('slayer HIP kernels need tensors on an MI355X device; '
                               'there is no CPU implementation in this package')
        if t.dtype != torch.float32:
            raise RuntimeError(f'slayer HIP kernels are float32 only, got {t.dtype}')
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f'tensors on different devices: {dev} and {t.device}')
    return dev


def scan_tolerance(grad):
    """Tolerance of the debug cross-check of a float backward pass on ``grad``: 1e-5 of the largest magnitude when
    the library evaluates a tensor of this shape as a wave scan (whose rounding differs from a step-by-step
    evaluation by a few ulp of the largest terms), None -- every bit must agree -- when it walks it step by step."""
    M, T = rows_and_steps(grad)
    scan = lib().slayer_bwd_takes_scan(M, neurons_per_batch(grad), T) and grad.data_ptr() % 16 == 0
    return 1e-5 if scan else None


def raise_on_mismatch(what, fast, check, rel=None):
    """debug mode: the streaming kernel and the one-thread-per-neuron kernel must agree, bit for bit for the
    fixed-point forward passes and for float gradients that both kernels walk step by step; float gradients that
    went through a scan (``rel`` given, see ``scan_tolerance``) within ``rel`` of their largest magnitude."""
    if rel is not None:
        scale = float(check.abs().max()) if check.numel() else 0.0
        err = float((fast - check).abs().max()) if check.numel() else 0.0
        if not err <= rel * scale:
            raise Exception(f'{what}: the two GPU implementations differ by {err:.3e}, more than {rel} of the '
                            f'largest magnitude {scale:.3e}')
        return
    if not torch.equal(fast, check):
        bad = fast != check
        first = bad.nonzero()[0].tolist()
        raise Exception(f'{what}: the two GPU implementations differ in {int(bad.sum())} of {bad.numel()} '
                        f'elements, first at {first}: {fast[tuple(first)].item()!r} vs '
                        f'{check[tuple(first)].item()!r} (a 32-bit state overflow shows up like this)')


def wants_grad(*tensors):
    """True when a backward pass could reach one of the tensors: otherwise the operators call their
    kernels directly and skip the autograd node (a few microseconds per call, which is most of a
    call on a tensor of one time step)."""
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


_no_guard = contextlib.nullcontext()


def device_guard(dev):
    """Context in which ``dev`` is the current device.  ``torch.cuda.device`` switches the device twice even when
    it already is the current one (~3 us of host time, a quarter of a call on a tensor of one time step), so that
    case gets an empty context."""
    return _no_guard if dev.index == torch._C._cuda_getDevice() else torch.cuda.device(dev)


def ptr(t):
    return None if t is None else t.data_ptr()


def stream_handle():
    """Raw handle of torch's current stream on the current device (the direct binding: the public
    accessor costs ~150 us of host time per call once the launch queue is busy)."""
    try:
        return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())
    except AttributeError:
        return torch.cuda.current_stream().cuda_stream


def rows_and_steps(t):
    T = t.shape[-1]
    return (t.numel() // T if T > 0 else 0), T


def neurons_per_batch(t):
    n = 1
    for s in t.shape[1:-1]:
        n *= s
    return n
