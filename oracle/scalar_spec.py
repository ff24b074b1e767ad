"""Scalar big-integer statement of the fixed-point recurrences.

TEST INFRASTRUCTURE ONLY (see slayer_oracle.py).  One neuron, one python loop,
unbounded python ints, written from the arithmetic rules rather than from the
vectorised code, so that it can pin slayer_oracle.py by brute force on small
inputs.  float32 effects (input scaling, int -> float32 output conversion, the
float32 threshold compare) are made explicit with numpy.float32.

Rules restated (citations relative to /root/reference/src/lava/lib/dl/slayer/):
  rs0       utils/int_utils.py:29-31      truncating shift, sign(+1 iff x > 0)
  LI        neuron/dynamics/leaky_integrator.py:214-231
  ATH       neuron/dynamics/adaptive_threshold.py:243-274
  RES       neuron/dynamics/resonator.py:343-376
  APTH      neuron/dynamics/adaptive_phase_th.py:241-284
  ADRES     neuron/dynamics/adaptive_resonator.py:386-436
"""

import numpy as np

f32 = np.float32


def trunc_div_4096(p):
    """Integer p / 4096 rounded toward zero, for a python int."""
    return p // 4096 if p >= 0 else -((-p) // 4096)


def to_int(x_f32):
    """float32 -> integer truncation toward zero."""
    return int(np.trunc(f32(x_f32)))


def li(x, decay, state, w, threshold=None):
    """Returns (out list of float32, spikes list of bool)."""
    thr = (-1 if threshold is None else threshold) * w
    y = to_int(f32(state) * f32(w))
    m = 4096 - to_int(decay)
    out, fired_seq = [], []
    for xt in x:
        y = trunc_div_4096(y * m) + to_int(f32(w) * f32(xt))
        out.append(f32(y) / f32(w))
        fired = thr > 0 and f32(y) >= f32(thr)
        fired_seq.append(bool(fired))
        if fired:
            y = 0
    return out, fired_seq


def ath(x, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w):
    """Returns (threshold list, refractory list, spikes list)."""
    th = to_int(f32(th_state) * f32(w))
    r = to_int(f32(ref_state) * f32(w))
    mt = 4096 - to_int(th_decay)
    mr = 4096 - to_int(ref_decay)
    step = int(th_scale * w)
    base = int(th0 * w)
    th_out, r_out, fired_seq = [], [], []
    for xt in x:
        r = trunc_div_4096(r * mr)
        th = trunc_div_4096((th - base) * mt) + base
        th_out.append(f32(th) / f32(w))
        r_out.append(f32(r) / f32(w))
        fired = to_int(f32(w) * f32(xt)) >= th + r
        fired_seq.append(bool(fired))
        if fired:
            r += 2 * th
            th += step
    return th_out, r_out, fired_seq


def res(xr, xi, sin_decay, cos_decay, re_state, im_state, w, threshold=None):
    """Returns (re list, im list, spikes list).  Exact while abs(im) <= 2**24."""
    thr = (-1 if threshold is None else threshold) * w
    re = to_int(f32(re_state) * f32(w))
    im = to_int(f32(im_state) * f32(w))
    s = to_int(sin_decay)
    c = to_int(cos_decay)
    re_out, im_out, fired_seq = [], [], []
    for a, b in zip(xr, xi):
        re_n = trunc_div_4096(c * re) - trunc_div_4096(s * im) + to_int(f32(w) * f32(a))
        im_n = trunc_div_4096(s * re) + trunc_div_4096(c * im) + to_int(f32(w) * f32(b))
        re_out.append(f32(re_n) / f32(w))
        im_out.append(f32(im_n) / f32(w))
        fired = thr >= 0 and f32(im_n) >= f32(thr)
        fired_seq.append(bool(fired))
        if fired:
            re, im = 0, to_int(f32(thr - 1))
        else:
            re, im = re_n, im_n
    return re_out, im_out, fired_seq


def apth(xr, xi, im_state, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w):
    """neuron/dynamics/adaptive_phase_th.py:241-284.  Returns (threshold, refractory, spikes)."""
    th = to_int(f32(th_state) * f32(w))
    r = to_int(f32(ref_state) * f32(w))
    mt = 4096 - to_int(th_decay)
    mr = 4096 - to_int(ref_decay)
    step = int(th_scale * w)
    base = int(th0 * w)
    im_old = to_int(f32(w) * f32(im_state))
    th_out, r_out, fired_seq = [], [], []
    for a, b in zip(xr, xi):
        r = trunc_div_4096(r * mr)
        th = trunc_div_4096((th - base) * mt) + base
        th_out.append(f32(th) / f32(w))
        r_out.append(f32(r) / f32(w))
        re, im = to_int(f32(w) * f32(a)), to_int(f32(w) * f32(b))
        fired = re >= th + r and im >= 0 and im_old < 0
        fired_seq.append(bool(fired))
        if fired:
            r += 2 * th
            th += step
        im_old = im
    return th_out, r_out, fired_seq


def adres(xr, xi, sin_decay, cos_decay, ref_decay, th_decay, re_state, im_state, ref_state, th_state,
          th_scale, th0, w):
    """neuron/dynamics/adaptive_resonator.py:386-436.  Returns (re, im, threshold, refractory, spikes)."""
    re = to_int(f32(re_state) * f32(w))
    im = to_int(f32(im_state) * f32(w))
    th = to_int(f32(th_state) * f32(w))
    r = to_int(f32(ref_state) * f32(w))
    s, c = to_int(sin_decay), to_int(cos_decay)
    mt = 4096 - to_int(th_decay)
    mr = 4096 - to_int(ref_decay)
    step = int(th_scale * w)
    base = int(th0 * w)
    outs = ([], [], [], [], [])
    for a, b in zip(xr, xi):
        r = trunc_div_4096(r * mr)
        th = trunc_div_4096((th - base) * mt) + base
        re, im = (trunc_div_4096(c * re) - trunc_div_4096(s * im) + to_int(f32(w) * f32(a)),
                  trunc_div_4096(s * re) + trunc_div_4096(c * im) + to_int(f32(w) * f32(b)))
        for o, v in zip(outs, (re, im, th, r)):
            o.append(f32(v) / f32(w))
        fired = im >= th + r
        outs[4].append(bool(fired))
        if fired:
            r += 2 * th
            th += step
    return outs
