"""CPU oracle for the SLAYER neuron-dynamics / temporal-op hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, and
only as the checker (or as the timed CPU baseline), never as the product path.

Every function restates, in torch CPU ops and the same per-timestep op order,
what the reference's CPU branch computes.  Citations are relative to
/root/reference/src/lava/lib/dl/slayer/ (abbreviated S/, and DYN/ for
S/neuron/dynamics/).

Pin status (see tests/test_oracle_*.py):
  li_fwd, spike_fwd (binary)      reference-held fixture gts/dense + scalar spec + closed forms
  res_fwd (no threshold), cspike  reference-held fixture gts/complex_dense + scalar spec
  res_fwd (threshold mode)        reference-held fixture gts/complex_dense (RF_IZ input block) + scalar spec;
                                  beyond 2**24, where the reset expression rounds through float32:
                                  vectors computed by the reference's CPU branch
                                  (tests/golden/make_reference_vectors.py)
  li_fwd beyond 2**24             the same vectors (float32 reset compare)
  ath_fwd                         vectors of the reference's alif.Neuron (tests/golden/make_reference_neuron_vectors.py)
                                  + scalar spec + closed forms + leak invariants
  apth_fwd, adres_fwd             vectors of the reference's adrf.Neuron / adrf_iz.Neuron (same script) + scalar spec;
                                  identity with the pinned pieces they are made of
                                  (ath recurrences + complex spike condition; res_fwd + ath_fwd on imag)
  li_bwd, res_bwd                 torch autograd through a float IIR + scipy.signal.lfilter (float64)
  spike_bwd, cspike_bwd           closed forms evaluated in float64
  shift                           numpy slicing (the reference's own test_shift.py check)
  conv_fwd / conv_bwd             numpy.convolve (the reference's own test_conv_filter.py check)
  delay_bwd                       finite-difference identity on the conv([-1,1]) form
  delta_fwd / delta_bwd, sigma    hand-computed sequences, reconstruction invariant |x - sigma(delta(x))| < threshold,
                                  float64 closed forms of the threshold gradient, numpy.cumsum
  recurrent_cuba_fwd/_bwd,        no reference fixture; without feedback = the pinned operators over the whole sequence,
  recurrent_alif_fwd              hand-computed cases (delay and orientation of R, graded value, threshold / refractory
                                  jump), backward = float64 autograd through an independently written unrolled graph
"""

import numpy as np
import torch

I64 = torch.int64
SHIFT = 12
ONE = 1 << SHIFT


# --------------------------------------------------------------------------
# integer helpers
# --------------------------------------------------------------------------
def rs0(x, bits=SHIFT):
    """Right shift that rounds toward zero.  S/utils/int_utils.py:9-31.

    The sign factor is +1 for x > 0 and -1 otherwise (x == 0 uses -1, which is
    harmless because -(-0 >> bits) == 0).
    """
    if x.dtype not in (torch.int32, torch.int64):
        raise TypeError(f'rs0 needs an integer tensor, got {x.dtype}')
    sgn = 2 * (x > 0) - 1
    return (sgn * ((sgn * x) >> bits)).to(x.dtype)


def neuron_shaped(param, shape):
    """View a decay/parameter vector so it broadcasts over ``shape[:-1]``.

    The reference CPU loops rely on plain broadcasting (DYN/leaky_integrator.py:221),
    which only works for [N, C, T] tensors.  For tensors with spatial axes the
    accelerated kernels define the rule instead (DYN/leaky_integrator.cu:46-52,
    145-147): one value -> shared; C values -> per channel; prod(shape[1:-1])
    values -> per neuron.  This helper applies that rule for any rank.
    """
    n = param.numel()
    spatial = tuple(shape[1:-1])
    if n == 1:
        return param.reshape(())
    if n == int(np.prod(spatial)):
        return param.reshape(spatial)
    if len(spatial) >= 1 and n == spatial[0]:
        return param.reshape((n,) + (1,) * (len(spatial) - 1))
    raise ValueError(f'cannot map {n} parameters onto neurons of shape {spatial}')


def _full_state(state, like):
    """DYN/leaky_integrator.py:89-90: a one-element state is broadcast."""
    if state.numel() == 1:
        return state.reshape(()) * torch.ones(like.shape[:-1])
    return state.reshape(like.shape[:-1])


# --------------------------------------------------------------------------
# leaky integrator
# --------------------------------------------------------------------------
def li_fwd(x, decay, state, w_scale, threshold=None):
    """Leaky-integrator forward.  DYN/leaky_integrator.py:50-100, 210-231.

    y[t] = rs0(y[t-1] * (4096 - trunc(decay)), 12) + trunc(w * x[t]);
    out[t] = y[t] / w;  y is cleared after a step with y >= threshold * w
    (only when threshold * w > 0; ``None`` means -1, i.e. no reset).
    """
    thr = -1 if threshold is None else threshold
    thr = thr * w_scale                       # python number, :218
    state = _full_state(state, x)
    y_prev = (state * w_scale).detach().to(I64)
    mult = ONE - neuron_shaped(decay.detach(), x.shape).to(I64)
    out = torch.zeros_like(x)
    for t in range(x.shape[-1]):
        y = rs0(y_prev * mult) + (w_scale * x[..., t]).to(I64)
        if thr > 0:
            fired = y >= thr                  # int64 vs python float: compared as float32
            y_prev = y * (fired < 0.5)
        else:
            y_prev = y
        out[..., t] = y / w_scale             # int64 -> float32, then divide
    return out


def li_bwd(grad_out, out, decay):
    """Leaky-integrator backward.  DYN/leaky_integrator.py:234-259.

    g[T-1] = go[T-1];  g[t] = (1 - decay/4096) * g[t+1] + go[t];
    grad_decay = sum g[..., 1:] * out[..., :-1] over batch, time and space.
    """
    a = 1 - neuron_shaped(decay, grad_out.shape) / ONE
    T = grad_out.shape[-1]
    g = torch.zeros_like(grad_out)
    g[..., T - 1] = grad_out[..., T - 1]
    for t in range(T - 2, -1, -1):
        g[..., t] = a * g[..., t + 1] + grad_out[..., t]
    gd = g[..., 1:] * out[..., :-1]
    return g, _reduce_param_grad(gd, decay.numel())


def _reduce_param_grad(gd, n_param):
    """Shared -> [1]; otherwise sum over batch and time, then space.  :249-257."""
    if n_param == 1:
        return gd.flatten().sum(dim=0, keepdim=True)
    gd = gd.sum(dim=[0, -1])
    if gd.dim() != 1:
        gd = gd.reshape(gd.shape[0], -1).sum(dim=1)
    return gd


def li_persistent_state(state, spike):
    """DYN/leaky_integrator.py:103-119."""
    return state * (1 - (spike > 0).to(state.dtype))


# --------------------------------------------------------------------------
# adaptive threshold + refractory
# --------------------------------------------------------------------------
def ath_fwd(x, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale):
    """Adaptive threshold forward.  DYN/adaptive_threshold.py:51-126, 237-274.

    r = rs0(r * (4096 - rd), 12);  th = rs0((th - th0) * (4096 - td), 12) + th0;
    outputs th / w and r / w (values before the spike update);
    s = trunc(w * x[t]) >= th + r;  th += step * s;  r += 2 * th_before * s.
    """
    th_prev = (_full_state(th_state, x) * w_scale).detach().to(I64)
    r_prev = (_full_state(ref_state, x) * w_scale).detach().to(I64)
    th_mult = ONE - neuron_shaped(th_decay.detach(), x.shape).to(I64)
    r_mult = ONE - neuron_shaped(ref_decay.detach(), x.shape).to(I64)
    step = int(th_scale * w_scale)
    base = int(th0 * w_scale)
    th_out = torch.zeros_like(x)
    r_out = torch.zeros_like(x)
    for t in range(x.shape[-1]):
        r = rs0(r_prev * r_mult)
        th = rs0((th_prev - base) * th_mult) + base
        u = (w_scale * x[..., t]).to(I64)
        fired = u >= (th + r)
        th_prev = th + step * (fired > 0.5)
        r_prev = r + 2 * th * (fired > 0.5)
        th_out[..., t] = th / w_scale
        r_out[..., t] = r / w_scale
    return th_out, r_out


def ath_persistent_ref_state(ref_state, spike, th_state):
    """DYN/adaptive_threshold.py:133-151."""
    return ref_state + 2 * (spike > 0).to(ref_state.dtype) * th_state


def ath_persistent_th_state(th_state, spike, th_step):
    """DYN/adaptive_threshold.py:154-172."""
    return th_state + (spike > 0).to(th_state.dtype) * th_step


def apth_fwd(re_in, im_in, im_state, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale):
    """Adaptive phase threshold forward.  DYN/adaptive_phase_th.py:51-131, 234-284.

    Threshold / refractory recurrences of ath_fwd; the spike condition is
    trunc(w*re) >= th + r  and  trunc(w*im) >= 0  and  previous trunc(w*im) < 0.
    """
    th_prev = (_full_state(th_state, re_in) * w_scale).detach().to(I64)
    r_prev = (_full_state(ref_state, re_in) * w_scale).detach().to(I64)
    th_mult = ONE - neuron_shaped(th_decay.detach(), re_in.shape).to(I64)
    r_mult = ONE - neuron_shaped(ref_decay.detach(), re_in.shape).to(I64)
    step = int(th_scale * w_scale)
    base = int(th0 * w_scale)
    im_old = (w_scale * _full_state(im_state, im_in)).to(I64)
    th_out = torch.zeros_like(re_in)
    r_out = torch.zeros_like(re_in)
    for t in range(re_in.shape[-1]):
        r = rs0(r_prev * r_mult)
        th = rs0((th_prev - base) * th_mult) + base
        re = (w_scale * re_in[..., t]).to(I64)
        im = (w_scale * im_in[..., t]).to(I64)
        fired = (re >= (th + r)) * (im >= 0) * (im_old < 0)
        th_prev = th + step * (fired > 0.5)
        r_prev = r + 2 * th * (fired > 0.5)
        th_out[..., t] = th / w_scale
        r_out[..., t] = r / w_scale
        im_old = im
    return th_out, r_out


def adres_fwd(xr, xi, sin_decay, cos_decay, ref_decay, th_decay,
              re_state, im_state, ref_state, th_state, th_scale, th0, w_scale):
    """Adaptive resonator forward.  DYN/adaptive_resonator.py:49-158, 379-436.

    res_fwd without reset, plus ath-style threshold / refractory recurrences whose spike
    condition is the integer compare im >= th + r.  Backward is res_bwd (:439-520).
    """
    re_prev = (_full_state(re_state, xr) * w_scale).detach().to(I64)
    im_prev = (_full_state(im_state, xi) * w_scale).detach().to(I64)
    th_prev = (_full_state(th_state, xr) * w_scale).detach().to(I64)
    r_prev = (_full_state(ref_state, xr) * w_scale).detach().to(I64)
    s = neuron_shaped(sin_decay.detach(), xr.shape).to(I64)
    c = neuron_shaped(cos_decay.detach(), xr.shape).to(I64)
    th_mult = ONE - neuron_shaped(th_decay.detach(), xr.shape).to(I64)
    r_mult = ONE - neuron_shaped(ref_decay.detach(), xr.shape).to(I64)
    step = int(th_scale * w_scale)
    base = int(th0 * w_scale)
    outs = [torch.zeros_like(xr) for _ in range(4)]
    for t in range(xr.shape[-1]):
        r = rs0(r_prev * r_mult)
        th = rs0((th_prev - base) * th_mult) + base
        re = rs0(c * re_prev) - rs0(s * im_prev) + (w_scale * xr[..., t]).to(I64)
        im = rs0(s * re_prev) + rs0(c * im_prev) + (w_scale * xi[..., t]).to(I64)
        fired = (im >= (th + r)).to(I64)
        re_prev, im_prev = re, im
        th_prev = th + step * (fired > 0.5)
        r_prev = r + 2 * th * (fired > 0.5)
        for o, v in zip(outs, (re, im, th, r)):
            o[..., t] = v / w_scale
    return tuple(outs)


# --------------------------------------------------------------------------
# resonator
# --------------------------------------------------------------------------
def res_fwd(xr, xi, sin_decay, cos_decay, re_state, im_state, w_scale, threshold=None):
    """Resonator forward.  DYN/resonator.py:49-132, 333-376.

    re = rs0(c * re', 12) - rs0(s * im', 12) + trunc(w * xr[t])
    im = rs0(s * re', 12) + rs0(c * im', 12) + trunc(w * xi[t])
    with c, s = trunc(cos_decay), trunc(sin_decay).  If threshold * w >= 0 and
    im >= threshold * w:  re' = 0, im' = threshold * w - 1 (through float32).
    """
    thr = -1 if threshold is None else threshold
    thr = thr * w_scale
    re_prev = (_full_state(re_state, xr) * w_scale).detach().to(I64)
    im_prev = (_full_state(im_state, xi) * w_scale).detach().to(I64)
    s = neuron_shaped(sin_decay.detach(), xr.shape).to(I64)
    c = neuron_shaped(cos_decay.detach(), xr.shape).to(I64)
    re_out = torch.zeros_like(xr)
    im_out = torch.zeros_like(xi)
    for t in range(xr.shape[-1]):
        re = rs0(c * re_prev) - rs0(s * im_prev) + (w_scale * xr[..., t]).to(I64)
        im = rs0(s * re_prev) + rs0(c * im_prev) + (w_scale * xi[..., t]).to(I64)
        if thr >= 0:
            fired = (im >= thr).to(I64)
            re_prev = ((1 - fired) * re).to(I64)
            # int64 * python float promotes to float32: the kept value makes a
            # float32 round trip as well (:365-368)
            im_prev = (fired * (thr - 1) + (1 - fired) * im).to(I64)
        else:
            re_prev, im_prev = re, im
        re_out[..., t] = re / w_scale
        im_out[..., t] = im / w_scale
    return re_out, im_out


def res_bwd(g_re, g_im, re, im, sin_decay, cos_decay):
    """Resonator backward.  DYN/resonator.py:379-467.

    gr[t] = c * gr[t+1] + s * gi[t+1] + g_re[t];  gi[t] = -s * gr[t+1] + c * gi[t+1] + g_im[t]
    with c, s = decay / 4096;  grad_sin = sum(-gr[1:] * im[:-1] + gi[1:] * re[:-1]),
    grad_cos = sum(gr[1:] * re[:-1] + gi[1:] * im[:-1]).
    """
    c = neuron_shaped(cos_decay, g_re.shape) / ONE
    s = neuron_shaped(sin_decay, g_re.shape) / ONE
    T = g_re.shape[-1]
    gr = torch.zeros_like(g_re)
    gi = torch.zeros_like(g_im)
    gr[..., T - 1] = g_re[..., T - 1]
    gi[..., T - 1] = g_im[..., T - 1]
    for t in range(T - 2, -1, -1):
        gr[..., t] = c * gr[..., t + 1] + s * gi[..., t + 1] + g_re[..., t]
        gi[..., t] = -s * gr[..., t + 1] + c * gi[..., t + 1] + g_im[..., t]
    for name, v in (('grad_real', g_re), ('grad_imag', g_im),
                    ('grad_real_input', gr), ('grad_imag_input', gi)):
        if torch.isnan(v).any():
            raise Exception(f'{name} has NaN.')
    g_sin = -gr[..., 1:] * im[..., :-1] + gi[..., 1:] * re[..., :-1]
    g_cos = gr[..., 1:] * re[..., :-1] + gi[..., 1:] * im[..., :-1]
    n = cos_decay.numel()
    return gr, gi, _reduce_param_grad(g_sin, n), _reduce_param_grad(g_cos, n)


def res_persistent_real_state(real_state, spike):
    """DYN/resonator.py:135-151."""
    return real_state * (1 - (spike > 0).to(real_state.dtype))


def res_persistent_imag_state(imag_state, spike, threshold, scale):
    """DYN/resonator.py:154-174."""
    s = (spike > 0).to(imag_state.dtype)
    return s * (threshold - 1 / scale) + (1 - s) * imag_state


# --------------------------------------------------------------------------
# spike functions
# --------------------------------------------------------------------------
def _as_f32_scalar(v, like):
    return v if torch.is_tensor(v) else torch.tensor(v, dtype=like.dtype)


def spike_fwd(voltage, threshold, graded=False, scale=1):
    """S/spike/spike.py:64-87."""
    if graded:
        return ((voltage >= threshold) * voltage / scale).to(voltage.dtype)
    return (voltage >= threshold).to(voltage.dtype)


def spike_bwd(grad_spikes, voltage, threshold, tau_rho, scale_rho, graded=False):
    """S/spike/spike.py:10-23, 113-126.  tau/scale are float32 0-dim tensors there."""
    threshold = _as_f32_scalar(threshold, voltage)
    tau = torch.tensor(tau_rho, dtype=voltage.dtype)
    rho = torch.tensor(scale_rho, dtype=voltage.dtype)
    if not graded:
        d = rho / 2 / tau * torch.exp(-torch.abs(voltage - threshold) / tau)
    else:
        d = rho * torch.exp(torch.clamp(voltage - threshold, max=0) / tau)
    return d * grad_spikes


def cspike_fwd(real, imag, threshold, imag_last=0, graded=False, scale=1):
    """S/spike/complex.py:49-92.  spike = (re >= th) & (im[t-1] < 0) & (im[t] >= 0)."""
    prev = torch.zeros_like(imag)
    prev[..., 1:] = imag[..., :-1]
    prev[..., 0] = imag_last
    if graded:
        return (real * (real >= threshold) * (prev < 0) * (imag >= 0) / scale).to(real.dtype)
    return ((real >= threshold) * (prev < 0) * (imag >= 0)).to(real.dtype)


def cspike_bwd(grad_out, real, imag, threshold, tau_rho, scale_rho, graded=False):
    """S/spike/complex.py:117-167."""
    threshold = _as_f32_scalar(threshold, real)
    tau = torch.tensor(tau_rho, dtype=real.dtype)
    rho = torch.tensor(scale_rho, dtype=real.dtype)
    if graded:
        d_re = torch.exp(-(threshold - real).clamp(0) / tau)
    else:
        d_re = 1 / 2 / tau * torch.exp(-torch.abs(real - threshold) / tau)
    d_im = 1 / 2 / tau * torch.exp(-torch.abs(imag) / tau)
    step_re = 1 / 2 * (1 + torch.sign(real - threshold) * (1 - 2 * tau * d_re))
    g_re = rho * d_re * d_im
    g_im = -rho / tau * torch.sign(imag) * d_im * step_re
    return grad_out * g_re, grad_out * g_im


# --------------------------------------------------------------------------
# time shift
# --------------------------------------------------------------------------
def _shift_rows(x2d, k):
    out = torch.zeros_like(x2d)
    T = x2d.shape[-1]
    if k == 0:
        return x2d.clone()
    if abs(k) >= T:
        return out
    if k > 0:
        out[..., k:] = x2d[..., :-k]
    else:
        out[..., :k] = x2d[..., -k:]
    return out


def shift(x, shift_val, sampling_time=1):
    """S/utils/time/shift.py:46-143.

    Scalar (or one-element tensor): every row moves by int(shift / Ts) steps,
    zero filled.  Tensor with more than one element: one shift per neuron of
    shape[1:-1]; the CPU branch divides by Ts twice for that case
    (:82 then :56), the accelerated branch once (S/utils/time/shift.cu:68) --
    they agree for Ts == 1, which is all the oracle is asked for; other Ts use
    the single division.
    """
    if x.dim() <= 1:
        raise AssertionError(f'Expected input to have at least two dimension. Found {x.shape=}.')
    if torch.is_tensor(shift_val) and shift_val.numel() > 1:
        if int(np.prod(x.shape[1:-1])) != shift_val.numel():
            raise Exception('Expected spatial dimension of input and shift_val to be same. '
                            f'Found {x.shape=}, {shift_val.shape=}.')
        rows = x.reshape(x.shape[0], -1, x.shape[-1])
        out = torch.zeros_like(rows)
        steps = shift_val.flatten() / sampling_time
        for i in range(rows.shape[1]):
            out[:, i] = _shift_rows(rows[:, i], int(steps[i].item()))
        return out.reshape(x.shape)
    if torch.is_tensor(shift_val):
        shift_val = shift_val.item()
    k = int(shift_val / sampling_time)
    return _shift_rows(x.reshape(-1, x.shape[-1]), k).reshape(x.shape)


# --------------------------------------------------------------------------
# temporal filter
# --------------------------------------------------------------------------
def conv_fwd(x, filt, sampling_time=1):
    """Causal y[t] = Ts * sum_i f[i] x[t-i].  S/utils/filter/conv.py:48-58."""
    import torch.nn.functional as F
    K = filt.numel()
    pad = F.pad(x.reshape(x.shape[0], 1, 1, -1, x.shape[-1]), (K - 1, 0, 0, 0, 0, 0))
    return F.conv3d(pad, torch.flip(filt.reshape(1, 1, 1, 1, -1), dims=[-1])).reshape(x.shape) * sampling_time


def conv_bwd(x, filt, sampling_time=1):
    """Anti-causal y[t] = Ts * sum_i f[i] x[t+i] (adjoint of conv_fwd).  conv.py:61-71."""
    import torch.nn.functional as F
    K = filt.numel()
    pad = F.pad(x.reshape(x.shape[0], 1, 1, -1, x.shape[-1]), (0, K - 1, 0, 0, 0, 0))
    return F.conv3d(pad, filt.reshape(1, 1, 1, 1, -1)).reshape(x.shape) * sampling_time


# --------------------------------------------------------------------------
# axonal delay (caller of shift + conv)
# --------------------------------------------------------------------------
def delay_fwd(x, delay_val, sampling_time=1):
    """S/axon/delay.py:178-199: output = shift(input, delay)."""
    return shift(x, delay_val, sampling_time)


def delay_bwd(grad_out, out, delay_val, grad_scale=1, sampling_time=1):
    """S/axon/delay.py:201-221."""
    diff = torch.tensor([-1, 1], dtype=grad_out.dtype) / sampling_time
    out_diff = conv_fwd(out, diff, 1)
    g_delay = torch.sum(grad_out * out_diff, [0, -1], keepdim=True) \
        .reshape(grad_out.shape[1:-1]) * sampling_time
    neg = -delay_val if torch.is_tensor(delay_val) else -delay_val
    return shift(grad_out, neg, sampling_time), g_delay * grad_scale


# --------------------------------------------------------------------------
# sigma-delta
# --------------------------------------------------------------------------
def delta_fwd(x, threshold, pre_state, residual_state, error_state, cum_error=False):
    """Delta unit forward.  S/axon/delta.py:10-46.  Returns (events, delta_input, residual, error)."""
    out = torch.zeros_like(x)
    delta_input = torch.zeros_like(x)
    pre = pre_state * torch.ones(x.shape[:-1])
    residual = residual_state * torch.ones(x.shape[:-1])
    error = (error_state * torch.ones(x.shape[:-1])).clone()
    for t in range(x.shape[-1]):
        delta = x[..., t] - pre + residual
        delta_input[..., t] = delta
        if cum_error:
            error = error + delta
            out[..., t] = torch.where(torch.abs(error) >= threshold, delta, 0 * delta)
            error = error * (1 - (torch.abs(out[..., t]) > 0).to(x.dtype))
        else:
            out[..., t] = torch.where(torch.abs(delta) >= threshold, delta, 0 * delta)
        residual = delta - out[..., t]
        pre = x[..., t]
    return out, delta_input, residual, error


def delta_bwd(grad_out, delta_input, threshold, tau_grad, scale_grad):
    """Delta unit backward.  S/axon/delta.py:68-103.  threshold has 1 or C elements.

    The reference subtracts its [C, 1, ...] threshold from the [N, C, ..., T] delta without
    adding the time axis, which mis-broadcasts (or raises) for per-channel thresholds; the
    per-channel alignment its forward pass uses is what is restated here.
    """
    tau = torch.tensor(tau_grad, dtype=grad_out.dtype)
    scale = torch.tensor(scale_grad, dtype=grad_out.dtype)
    thr = threshold if threshold.numel() == 1 else threshold.reshape([-1] + [1] * (delta_input.dim() - 2))
    sub = torch.abs(delta_input) - thr
    g_thr = torch.where(sub > 0, -delta_input * (scale * torch.exp(-torch.abs(sub) / tau)) / thr,
                        -torch.sign(delta_input)) * grad_out
    g_in = torch.zeros_like(grad_out)
    g_in[..., :-1] = grad_out[..., :-1] - grad_out[..., 1:]
    g_in[..., -1] = grad_out[..., -1]
    if threshold.numel() == 1:
        g_thr = torch.unsqueeze(torch.sum(g_thr), dim=0)
    else:
        g_thr = torch.sum(g_thr.reshape(delta_input.shape[0], delta_input.shape[1], -1), dim=[0, -1]) \
            .reshape(threshold.shape)
    return g_in, g_thr


def quantize_floor(x, step):
    """S/utils/quantize.py:38-48 (forward of the floor quantiser)."""
    return torch.floor(x / step) * step


def sigma_fwd(x, pre_state=None):
    """Sigma decoder.  S/dendrite/sigma.py:63-70: cumulative sum along time (+ carried state)."""
    out = torch.cumsum(x, dim=-1)
    if pre_state is not None:
        out = out + pre_state.unsqueeze(-1)
    return out


# --------------------------------------------------------------------------- convolution synapse
def conv_synapse(x, weight, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    """synapse/layer.py:297-323 in the reference: ``F.conv3d`` of an NCHWT tensor with a weight of
    [Co, Ci / groups, kh, kw, 1], no bias -- a spatial convolution applied at every time step.  The arithmetic is
    torch's (a dependency of the reference, torch ^2.9, not its own code): evaluated here in float64 and rounded once,
    and pinned by a direct evaluation of the defining sum on small cases (tests/test_oracle_spec.py)."""
    import torch.nn.functional as F
    out = F.conv3d(x.double(), weight.double(), None, tuple(stride) + (1,), tuple(padding) + (0,),
                   tuple(dilation) + (1,), groups)
    return out.float()


# --------------------------------------------------------------------------- recurrent layer
def recurrent_cuba_fwd(z, rec, i_decay, v_decay, i_state, v_state, w_scale, threshold, graded=False):
    """Recurrent CUBA layer, S/utils/recurrent.py:45-81 with the CUBA neuron called one step at a
    time (S/neuron/cuba.py:356-421, persistent state): feedback = s[t-1] @ R^T, the neuron's current
    and voltage LI run one step each from the carried float32 states, a spike resets the carried
    voltage; a graded spike carries the voltage (scale 1, S/neuron/cuba.py:403-409).
    z: [N, C, T]; rec = R [C, C].  Returns (spikes, voltage, current_state, voltage_state)."""
    spikes = torch.zeros_like(z)
    voltage = torch.zeros_like(z)
    cur_state = _full_state(i_state, z[..., :1])
    vol_state = _full_state(v_state, z[..., :1])
    s = torch.zeros(z.shape[:-1])
    rec_t = rec.transpose(0, 1)
    for t in range(z.shape[-1]):
        dend = (z[..., t] + torch.matmul(s, rec_t)).unsqueeze(-1)
        cur = li_fwd(dend, i_decay, cur_state, w_scale)
        vol = li_fwd(cur, v_decay, vol_state, w_scale, threshold)
        spk = spike_fwd(vol, threshold, graded, 1)
        cur_state = cur[..., -1]
        vol_state = li_persistent_state(vol[..., -1], spk[..., -1])
        s = spk[..., 0]
        spikes[..., t] = s
        voltage[..., t] = vol[..., 0]
    return spikes, voltage, cur_state, vol_state


def recurrent_alif_fwd(z, rec, decays, states, th_step, th0, w_scale, graded=False):
    """Recurrent ALIF layer: the same loop with the ALIF neuron called one step at a time
    (S/neuron/alif.py:383-623, persistent state).  decays / states = (current, voltage, threshold,
    refractory).  The voltage is not reset; a spike adds th_step to the carried threshold and twice the
    threshold to the carried refractory state (DYN/adaptive_threshold.py:133-172).
    Returns (spikes, voltage, theta = threshold + refractory, states after the last step)."""
    spikes, voltage, theta = torch.zeros_like(z), torch.zeros_like(z), torch.zeros_like(z)
    cur_state, vol_state, th_state, ref_state = (_full_state(x, z[..., :1]) for x in states)
    s = torch.zeros(z.shape[:-1])
    rec_t = rec.transpose(0, 1)
    for t in range(z.shape[-1]):
        dend = (z[..., t] + torch.matmul(s, rec_t)).unsqueeze(-1)
        cur = li_fwd(dend, decays[0], cur_state, w_scale)
        vol = li_fwd(cur, decays[1], vol_state, w_scale)
        th, ref = ath_fwd(vol, ref_state, decays[3], th_state, decays[2], th_step, th0, w_scale)
        spk = spike_fwd(vol, th + ref, graded, 1)
        cur_state, vol_state = cur[..., -1], vol[..., -1]
        ref_state = ath_persistent_ref_state(ref[..., -1], spk[..., -1], th[..., -1])
        th_state = ath_persistent_th_state(th[..., -1], spk[..., -1], th_step)
        s = spk[..., 0]
        spikes[..., t] = s
        voltage[..., t] = vol[..., 0]
        theta[..., t] = (th + ref)[..., 0]
    return spikes, voltage, theta, (cur_state, vol_state, th_state, ref_state)


def recurrent_cuba_bwd(grad_x, spikes, voltage, rec, threshold, tau_rho, scale_rho, graded=False):
    """S/utils/recurrent.py:83-112: the carried neuron state is a constant, so a step contributes the
    spike surrogate (the two one-step LI backward passes are identities); the gradient reaches step
    t-1 through R.  threshold: a number, or for an ALIF layer the tensor threshold + refractory of
    every step.  Returns (grad_z, grad_R)."""
    grad_z = torch.zeros_like(grad_x)
    carry = torch.zeros(grad_x.shape[:-1])
    for t in range(grad_x.shape[-1] - 1, -1, -1):
        gs = carry + grad_x[..., t]
        th = threshold[..., t:t + 1] if torch.is_tensor(threshold) and threshold.dim() > 0 else threshold
        gd = spike_bwd(gs.unsqueeze(-1), voltage[..., t:t + 1], th, tau_rho, scale_rho, graded)[..., 0]
        grad_z[..., t] = gd
        carry = torch.matmul(gd, rec)
    grad_out = grad_z[..., 1:].transpose(0, 1).reshape(grad_z.shape[1], -1)
    spikes_in = spikes[..., :-1].transpose(1, 2).reshape(-1, spikes.shape[1])
    return grad_z, torch.matmul(grad_out, spikes_in)
