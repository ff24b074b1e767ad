/*
 * slayer_hip.h -- C ABI of libslayer_hip.so, the MI355X (gfx950) implementation of
 * lava-dl SLAYER's neuron-dynamics and temporal-op kernels.
 *
 * Every entry point replaces one function of the reference's JIT-built CUDA
 * modules (citations are relative to src/lava/lib/dl/slayer/ in lava-nc/lava-dl);
 * the arithmetic follows the reference's CPU branch, which is the semantic
 * definition (int64 states on the CPU, float32 tensors at every op boundary).
 *
 * Conventions
 *   - All tensor pointers are DEVICE pointers to contiguous float32 data laid out
 *     [M neurons][T steps], time innermost (M = numel / T).
 *   - Nothing is allocated, freed or synchronised inside; work is enqueued on
 *     `stream` (a hipStream_t passed as void*, NULL = the null stream) of the
 *     device that is current when the call is made.
 *   - Inputs are never written.  Outputs are fully overwritten.
 *   - Return value: 0 on success, a positive hipError_t from the launch, or a
 *     negative SLAYER_E* code for arguments the kernels cannot honour (nothing is
 *     launched in that case).
 *   - Per-neuron parameter addressing (decays) follows the reference kernels:
 *     num_params == 1 -> shared;  otherwise neuron m uses
 *     param[(m % neurons_per_batch) / (neurons_per_batch / num_params)]
 *     (leaky_integrator.cu:46-52,145-147): num_params == C is per channel,
 *     num_params == C*H*W is per neuron.
 *   - States: num_states == 1 broadcasts one value, otherwise num_states == M.
 *   - Integer states are held in 32 bits with 64-bit products (as the reference
 *     kernels do, leaky_integrator.cu:43,61); results equal the int64 CPU branch
 *     (leaky_integrator.py:210-231) while no intermediate leaves 32 bits.  That is
 *     not left to chance: every forward kernel watches the states it stores and
 *     raises a process-wide flag (slayer_range_status) when one comes within a
 *     factor of two of the limit -- before anything can have overflowed.
 */
#ifndef SLAYER_HIP_H
#define SLAYER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLAYER_ABI_VERSION 4

#define SLAYER_EINVAL   (-1)   /* inconsistent sizes (M, T, neurons_per_batch, num_params, ...) */
#define SLAYER_ENULL    (-2)   /* a required pointer is NULL */
#define SLAYER_ERANGE   (-3)   /* a size exceeds what the kernels index (M*T >= 2^40, T >= 2^31, min(K, T) > 12288 ...) */
#define SLAYER_ESCRATCH (-4)   /* a size exceeds the library's built-in scratch buffer (slayer_li_bwd_static) */
#define SLAYER_ENOFLAG  (-5)   /* the range flag could not be set up (slayer_range_status) */

int slayer_abi_version(void);

/* Axonal delays folded into a fused neuron block (slayer_cuba_fwd/bwd, slayer_alif_fwd/bwd, slayer_rf_fwd/bwd),
 * so that the shift before a neuron and the delay after it (block/base.py:15-39,549-553: step_delay, then the
 * learnable axon/delay.py Delay; utils/time/shift.py:94-143 for the shift itself) cost no pass over the
 * tensor of their own.  A host structure; the tables are device pointers.
 *   forward : the neuron sees x[t] = in[t - kin] (zero where t - kin is outside [0, T)) and its spikes
 *             leave as spike_out[t + kout] = s[t]; spike_out[kout - 1] = out_head[m] when out_head is given
 *             (the last spike of the previous call: step_delay with persistent state), every other position
 *             no spike reaches is 0.  State traces (current, voltage, ...) are stored unshifted.
 *   backward: pass the same structure; grad_spikes is taken as the gradient of the delayed spikes and read as
 *             g[t] = grad_spikes[t + kout], grad_in is stored as the gradient of `in`: grad_in[t - kin].
 *   kin  = in_steps  + trunc(in_shift [m % neurons_per_batch] / sampling_time)   (any sign)
 *   kout = out_steps + trunc(out_delay[m % neurons_per_batch] / sampling_time)   (any sign)
 * as slayer_shift computes them.  Passing NULL instead of a structure means no delays at all. */
typedef struct slayer_delays {
    const float *in_shift;   /* neurons_per_batch floats in time units, or NULL */
    const float *out_delay;  /* neurons_per_batch floats in time units, or NULL */
    const float *out_head;   /* M floats, or NULL; forward only */
    float *spike_last;       /* M floats, or NULL; forward only: receives s[T-1], the spike of the last step, which
                              * a delayed spike tensor no longer holds (step_delay's buffer, persistent state) */
    int64_t in_steps;        /* whole steps added to every neuron's input shift */
    int64_t out_steps;       /* whole steps added to every neuron's output delay (step_delay: 1) */
    float sampling_time;     /* divides the table entries; must not be 0 when a table is given */
    /* backward only, all three or none: the gradient of out_delay as the learnable Delay computes it
     * (axon/delay.py:201-221): grad_out_delay[j] = sum over the batch and t of
     * grad_spikes[t] * (delayed_spikes[t-1] - delayed_spikes[t]) / sampling_time for neuron j of a batch element.
     * Tensors of 2^20 elements and more get it from the backward scan itself, which reads the gradient anyway (one more
     * tensor read instead of a pass of its own over two); smaller ones from slayer_delay_bwd, launched inside. */
    const float *delayed_spikes; /* M*T floats: the delayed spike tensor the forward pass stored */
    float *grad_out_delay;       /* neurons_per_batch floats */
    float *grad_workspace;       /* M + 64 * neurons_per_batch floats of scratch */
} slayer_delays;

/* Text for a return code of this library (hipGetErrorString for positive codes). */
const char *slayer_error_string(int code);

/* ---- range of the 32-bit states -------------------------------------------------------- */

/* The reference's CPU branch holds its fixed-point states in int64 (leaky_integrator.py:213, resonator.py:340), its
 * CUDA kernels and this library in int32 (leaky_integrator.cu:61 notes the overflow).  Here an overflow cannot pass
 * unnoticed: every forward entry point (slayer_li_fwd, slayer_ath_fwd, slayer_apth_fwd, slayer_res_fwd,
 * slayer_adres_fwd, slayer_cuba_fwd, slayer_alif_fwd, slayer_rf_fwd, slayer_*_recurrent_fwd) raises a sticky,
 * process-wide flag when
 *   - a state it stores (or is handed as initial state) reaches 2^30 in magnitude (2^29 for the real / imaginary
 *     states of the resonator family, whose step adds two products; 2^28 for threshold and refractory states, whose
 *     spike adds the step and twice the threshold), in units of 1 / w_scale, or
 *   - a decay multiplier (4096 - decay; sin / cos decay) exceeds 8191 in magnitude, or
 *   - a scaled threshold step, base threshold or reset value is itself beyond the bound of the state it enters.
 * While the flag is clear, no sum or product of a launch that has completed left 32 bits, and its results are those
 * of the 64-bit evaluation, bit for bit.  Once it is raised, the results of the launches since it was last clear are
 * suspect (sums saturate at the int32 limits instead of wrapping); the *_naive entry points evaluate in 64 bits.
 * The flag is one word of pinned host memory that the kernels write and the host reads in place: reading it costs
 * no device call and no synchronisation, and tells about every launch that has completed.
 *
 * slayer_range_status: *raised (may be NULL) receives 1 when the flag is up, else 0; clear != 0 lowers it.
 * Returns 0, or SLAYER_ENOFLAG when the word could not be set up (then no kernel reports anything).  The word is set
 * up by the first call of this function or of any forward entry point, with one hipHostMalloc of 64 bytes: make
 * that first call outside a stream capture.  Neither function has a counterpart in the reference. */
int slayer_range_status(int *raised, int clear);

/* Host address of the flag word (non-zero = raised), for polling without a call; NULL when it could not be set up. */
const volatile unsigned *slayer_range_word(void);

/* 1 when the float backward entry points (slayer_li_bwd, slayer_res_bwd, slayer_cuba_bwd, slayer_alif_bwd,
 * slayer_rf_bwd) evaluate a tensor of this shape as wave scans (grad_in then equals a step-by-step evaluation to
 * a few ulp of the largest terms), 0 when they walk it step by step (grad_in bit-identical to it); 16-byte
 * aligned tensors assumed.  For callers that compare the two, like the reference's debug cross-check
 * (leaky_integrator.py:168-205). */
int slayer_bwd_takes_scan(int64_t M, int64_t neurons_per_batch, int64_t T);

/* ---- leaky integrator ---------------------------------------------------------------- */

/* Replaces LIDynamicsFwd (neuron/dynamics/leaky_integrator.cu:112-153); arithmetic of
 * _li_dynamics_fwd (neuron/dynamics/leaky_integrator.py:210-231).
 * y = rs0(y * (4096 - trunc(decay)), 12) + trunc(w * in[t]);  out[t] = float(y) / w;
 * if thr_scaled > 0 and float(y) >= float(thr_scaled):  y = 0.
 * thr_scaled = threshold * w_scale computed by the caller in double (pass -w_scale for "no threshold"). */
int slayer_li_fwd(float *out, const float *in, const float *decay, const float *state,
                  double thr_scaled, int w_scale,
                  int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t num_states,
                  int64_t T, void *stream);

/* Replaces LIDynamicsBwd (leaky_integrator.cu:155-200); arithmetic of _li_dynamics_bwd
 * (leaky_integrator.py:234-259).
 * grad_in[T-1] = grad_out[T-1];  grad_in[t] = (1 - decay/4096) * grad_in[t+1] + grad_out[t];
 * grad_decay[j] = sum over the neurons that use decay j of sum_t grad_in[t+1] * out[t].
 * grad_decay (num_decays floats) may be NULL to skip the parameter gradient.
 * workspace: M + 64 * num_decays floats of scratch (per-neuron partial sums, then slice sums),
 * required iff grad_decay != NULL; its contents on return are unspecified.  Given without grad_decay it
 * receives the per-neuron sums (workspace[m] = sum_t grad_in[m][t+1] * out[m][t]) and nothing is reduced. */
int slayer_li_bwd(float *grad_in, float *grad_decay, const float *grad_out, const float *out,
                  const float *decay, float *workspace,
                  int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                  int64_t T, void *stream);

/* slayer_li_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same arguments without `workspace`, same kernels, same
 * results bit for bit.  It has no counterpart in the reference.  The scratch is a buffer built into the
 * library (5 MiB of device memory per GPU, held until the process ends); the call allocates and frees
 * nothing.  Limits: M <= SLAYER_LI_BWD_STATIC_MAX_ROWS and num_decays <= SLAYER_LI_BWD_STATIC_MAX_DECAYS,
 * else SLAYER_ESCRATCH is returned and nothing is launched.  All calls on one GPU share the one buffer:
 * calls that overlap on the same GPU (different streams, or threads) race; serialise them.
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress, which may load the code object):
 * make that call outside a stream capture, as a warm-up; later calls on that device only launch.
 * With grad_decay == NULL nothing is summed and the scratch is not touched (slayer_li_bwd given a workspace
 * without grad_decay would leave the per-neuron sums there; this entry point has no place to hand them out). */
#define SLAYER_LI_BWD_STATIC_MAX_ROWS   (1 << 20)
#define SLAYER_LI_BWD_STATIC_MAX_DECAYS 4096
int slayer_li_bwd_static(float *grad_in, float *grad_decay, const float *grad_out, const float *out,
                         const float *decay,
                         int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                         int64_t T, void *stream);

/* ---- adaptive threshold + refractory ---------------------------------------------------- */

/* Replaces AThDynamicsFwd (neuron/dynamics/adaptive_threshold.cu:81-131) with the CPU
 * branch's rounding (_ath_dynamics_fwd, neuron/dynamics/adaptive_threshold.py:237-274):
 * r = rs0(r * (4096 - rd), 12);  th = rs0((th - th0) * (4096 - td), 12) + th0;
 * th_out[t] = th / w;  ref_out[t] = r / w;  s = trunc(w * in[t]) >= th + r;
 * th += th_step * s;  r += 2 * th_before_step * s.
 * th_step_scaled = int(th_scale * w_scale), th0_scaled = int(th0 * w_scale), both taken by the caller. */
int slayer_ath_fwd(float *th_out, float *ref_out, const float *in,
                   const float *ref_state, const float *ref_decay,
                   const float *th_state, const float *th_decay,
                   int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                   int64_t M, int64_t neurons_per_batch,
                   int64_t num_ref_decays, int64_t num_th_decays,
                   int64_t num_ref_states, int64_t num_th_states,
                   int64_t T, void *stream);

/* Replaces APThDynamicsFwd (neuron/dynamics/adaptive_phase_th.cu:25-88 kernel, host function and
 * exports at its end); arithmetic of _APTHDynamicsFwd (neuron/dynamics/adaptive_phase_th.py:234-284).
 * Threshold / refractory recurrences as in slayer_ath_fwd; a step spikes when
 * trunc(w*re_in[t]) >= th + r and trunc(w*im_in[t]) >= 0 and the previous imaginary sample was < 0
 * (im_state seeds the previous sample of step 0). */
int slayer_apth_fwd(float *th_out, float *ref_out, const float *re_in, const float *im_in,
                    const float *im_state, const float *ref_state, const float *ref_decay,
                    const float *th_state, const float *th_decay,
                    int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                    int64_t M, int64_t neurons_per_batch,
                    int64_t num_ref_decays, int64_t num_th_decays,
                    int64_t num_im_states, int64_t num_ref_states, int64_t num_th_states,
                    int64_t T, void *stream);

/* ---- resonator ------------------------------------------------------------------------------ */

/* Replaces ResDynamicsFwd (neuron/dynamics/resonator.cu:151-198); arithmetic of
 * _res_dynamics_fwd (neuron/dynamics/resonator.py:333-376).
 * re = rs0(c*re', 12) - rs0(s*im', 12) + trunc(w*re_in[t]);
 * im = rs0(s*re', 12) + rs0(c*im', 12) + trunc(w*im_in[t]);   c, s = trunc(cos_decay), trunc(sin_decay)
 * if thr_scaled >= 0 and float(im) >= float(thr_scaled): re' = 0, im' = trunc(float(thr_scaled - 1)). */
int slayer_res_fwd(float *re_out, float *im_out, const float *re_in, const float *im_in,
                   const float *sin_decay, const float *cos_decay,
                   const float *re_state, const float *im_state,
                   double thr_scaled, int w_scale,
                   int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                   int64_t num_re_states, int64_t num_im_states,
                   int64_t T, void *stream);

/* Replaces ResDynamicsBwd (resonator.cu:200-262); arithmetic of _res_dynamics_bwd
 * (resonator.py:379-467) without its host-side NaN scans (the Python caller does those).
 * gr[t] = c*gr[t+1] + s*gi[t+1] + g_re[t];  gi[t] = -s*gr[t+1] + c*gi[t+1] + g_im[t];  c, s = decay/4096
 * grad_sin[j] = sum(-gr[t+1]*im[t] + gi[t+1]*re[t]);  grad_cos[j] = sum(gr[t+1]*re[t] + gi[t+1]*im[t]).
 * grad_sin/grad_cos (num_decays floats each) may both be NULL.
 * workspace: 2 * M + 128 * num_decays floats, required iff the parameter gradients are requested. */
int slayer_res_bwd(float *g_re_in, float *g_im_in, float *grad_sin, float *grad_cos,
                   const float *g_re, const float *g_im, const float *re, const float *im,
                   const float *sin_decay, const float *cos_decay, float *workspace,
                   int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                   int64_t T, void *stream);

/* Replaces AdResDynamicsFwd (neuron/dynamics/adaptive_resonator.cu:25-126 kernel and its host
 * function); arithmetic of _AdResDynamicsFwd (neuron/dynamics/adaptive_resonator.py:379-436):
 * the resonator recurrence without reset plus threshold / refractory recurrences whose spike
 * condition is im >= th + r (integer compare).  Its backward pass is slayer_res_bwd. */
int slayer_adres_fwd(float *re_out, float *im_out, float *th_out, float *ref_out,
                     const float *re_in, const float *im_in,
                     const float *sin_decay, const float *cos_decay,
                     const float *ref_decay, const float *th_decay,
                     const float *re_state, const float *im_state,
                     const float *ref_state, const float *th_state,
                     int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                     int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                     int64_t num_ref_decays, int64_t num_th_decays,
                     int64_t num_re_states, int64_t num_im_states,
                     int64_t num_ref_states, int64_t num_th_states,
                     int64_t T, void *stream);

/* ---- spike functions (elementwise; they replace chains of torch ops, not a .cu) ----------- */

/* Threshold convention of the four spike entry points: threshold == NULL -> the scalar
 * threshold_value applies everywhere; otherwise threshold points at num_threshold device floats,
 * num_threshold == 1 (one value, read on the device) or == numel (elementwise). */

/* Spike.forward (spike/spike.py:64-87).  graded != 0: out = (v >= th) * v / scale. */
int slayer_spike_fwd(float *spikes, const float *voltage, const float *threshold,
                     int64_t num_threshold, float threshold_value, int graded, float scale,
                     int64_t numel, void *stream);

/* Spike.backward / _spike_backward (spike/spike.py:10-23,113-126).
 * binary: rho/2/tau * exp(-|v - th| / tau) * g;   graded: rho * exp(min(v - th, 0) / tau) * g. */
int slayer_spike_bwd(float *grad_voltage, const float *grad_spikes, const float *voltage,
                     const float *threshold, int64_t num_threshold, float threshold_value,
                     float tau_rho, float scale_rho, int graded, int64_t numel, void *stream);

/* complex.Spike.forward (spike/complex.py:49-92): (re >= th) * (im[t-1] < 0) * (im[t] >= 0)
 * with im[-1] = imag_last[m] (num_last == 1 broadcasts; imag_last == NULL -> imag_last_value).
 * graded != 0 multiplies by re / scale. */
int slayer_cspike_fwd(float *spikes, const float *re, const float *im, const float *threshold,
                      int64_t num_threshold, float threshold_value,
                      const float *imag_last, int64_t num_last, float imag_last_value,
                      int graded, float scale, int64_t M, int64_t T, void *stream);

/* complex.Spike.backward (spike/complex.py:117-167). */
int slayer_cspike_bwd(float *grad_re, float *grad_im, const float *grad_spikes,
                      const float *re, const float *im, const float *threshold,
                      int64_t num_threshold, float threshold_value,
                      float tau_rho, float scale_rho, int graded, int64_t numel, void *stream);

/* ---- time shift --------------------------------------------------------------------------- */

/* Replaces both shift() overloads (utils/time/shift.cu:157-209, launchers :80-155); semantics of _shift_group /
 * _shift_individual (utils/time/shift.py:46-91).  out[m][t] = in[m][t - k] (zero outside [0,T)),
 * lut == NULL: every row moves by scalar_steps, the caller's int(shift / sampling_time) (python
 * double arithmetic, as _shift_group does); otherwise lut holds neurons_per_batch device floats and
 * row m moves by trunc(lut[m % neurons_per_batch] / sampling_time), divided in float32. */
int slayer_shift(float *out, const float *in, const float *lut, int64_t scalar_steps,
                 float sampling_time, int64_t M, int64_t neurons_per_batch, int64_t T, void *stream);

/* Backward of the learnable axonal delay, _delayFunction.backward (axon/delay.py:201-221: conv with
 * [-1, 1] / Ts, product, sum, shift -- four passes) in one: grad_in[m][t] = grad_out[m][t + k_m] with k_m as
 * in slayer_shift (lut == NULL: scalar_steps), and, when grad_sum is not NULL,
 * grad_sum[j] = sum over the batch and time of grad_out * ((-1/Ts) out[t] + (1/Ts) out[t-1]) for the
 * neurons_per_batch neurons of a batch element (the caller scales by Ts and grad_scale as the reference does).
 * workspace: M + 64 * neurons_per_batch floats, only read and written when grad_sum is wanted.
 * grad_in may be NULL when only the sums are wanted (a fused block's backward pass reads the gradient
 * back through the delay itself): 8 instead of 12 bytes per neuron-timestep. */
int slayer_delay_bwd(float *grad_in, float *grad_sum, const float *grad_out, const float *out,
                     const float *lut, int64_t scalar_steps, float sampling_time, float *workspace,
                     int64_t M, int64_t neurons_per_batch, int64_t T, void *stream);

/* ---- temporal filter ---------------------------------------------------------------------- */

/* Replaces conv fwd (utils/filter/conv.cu:80-125): out[m][t] = Ts * sum_{i<K, t-i>=0} filt[i] * in[m][t-i].
 * Any K: only the first min(K, T) taps can meet a sample of the row, and only they are read (SLAYER_ERANGE when
 * min(K, T) > 12288: rows and filters both longer than that).  float32 throughout; for 32 < K <= 128 the products are formed on the matrix
 * cores from three bfloat16 parts per operand (each operand to within 2^-27, sums in float32): as close to the
 * exact sum as float32 multiply-adds, for every finite operand of at least about 3e-33 in magnitude (smaller
 * ones enter with an absolute error of up to 1.2e-38). */
int slayer_conv(float *out, const float *in, const float *filt, int64_t K, float sampling_time,
                int64_t M, int64_t T, void *stream);

/* Replaces conv bwd (utils/filter/conv.cu:127-172): out[m][t] = Ts * sum_{i<K, t+i<T} filt[i] * in[m][t+i]. */
int slayer_corr(float *out, const float *in, const float *filt, int64_t K, float sampling_time,
                int64_t M, int64_t T, void *stream);

/* ---- convolution synapse ------------------------------------------------------------------ */

/* Replaces the F.conv3d call of the convolution synapse (synapse/layer.py:297-323: a kernel of (kh, kw, 1) over
 * [N, C, H, W, T], no bias, one group) for time-innermost tensors, without leaving that layout:
 * out[n][co][ho][wo][t] = sum over ci, y, x of weight[co][ci][y][x] *
 *                         in[n][ci][ho * stride_h + y * dil_h - pad_h][wo * stride_w + x * dil_w - pad_w][t]
 * (zero outside the image), Ho = (H + 2 pad_h - dil_h (kh - 1) - 1) / stride_h + 1, Wo likewise; weight is
 * [Co][Ci][kh][kw] (the reference's [Co][Ci][kh][kw][1]).  float32 operands and accumulation on the matrix cores
 * (on the vector units when Ci = Co = 1: the pooling layers, which fold their channels into the image height).
 * The gradient of the input is the same call on the gradient with the weights transposed and flipped.
 * Rows of any length from four steps on, float-aligned tensors.  SLAYER_ERANGE for what the kernel does not take
 * (T < 4, a batch entry of 2 GiB or more, more than about 860 taps Ci * kh * kw): the caller keeps its library
 * convolution for those. */
int slayer_conv_synapse(float *out, const float *in, const float *weight,
                        int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                        int64_t kh, int64_t kw, int64_t stride_h, int64_t stride_w,
                        int64_t pad_h, int64_t pad_w, int64_t dil_h, int64_t dil_w, void *stream);

/* The gradient of the synapse's input for any stride (what autograd obtains from conv3d's backward, and what the
 * transposed convolution of synapse/layer.py:513-560 computes as a layer of its own):
 * grad_in[n][ci][h][w][t] = sum over co, y, x of weight_t[ci][co][y][x] *
 *                           grad_out[n][co][(h + pad_h - y * dil_h) / stride_h][(w + pad_w - x * dil_w) / stride_w][t]
 * over the taps whose two quotients are exact and lie inside grad_out's [Ho][Wo].  N, Ci, Co, H, W, kh ... dil_w are
 * those of the forward call; weight_t is [Ci][Co][kh][kw] (the forward weights with the channel axes exchanged,
 * not flipped).  One launch per residue class of the pixels modulo the strides (stride_h * stride_w launches, each
 * a plain convolution over the taps that class meets); a single launch on the vector units when Ci = Co = 1 (the
 * pooling layers).  SLAYER_ERANGE as for slayer_conv_synapse, and for strides above 16 or images beyond 65535
 * pixels a side. */
int slayer_conv_synapse_input_grad(float *grad_in, const float *grad_out, const float *weight_t,
                                   int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                                   int64_t kh, int64_t kw, int64_t stride_h, int64_t stride_w,
                                   int64_t pad_h, int64_t pad_w, int64_t dil_h, int64_t dil_w, void *stream);

/* The gradient of the synapse's weights (what autograd obtains from conv3d's backward, synapse/layer.py:297-323):
 * grad_weight[co][ci][y][x] = sum over n, ho, wo, t of grad_out[n][co][ho][wo][t] *
 *                             in[n][ci][ho * stride_h + y * dil_h - pad_h][wo * stride_w + x * dil_w - pad_w][t],
 * reduced along time on the matrix cores (float32), the partial tiles of the waves added in double in a fixed
 * order.  workspace: slayer_conv_synapse_wgrad_workspace(...) floats of device memory, 16-byte aligned, contents
 * undefined afterwards (that function returns a negative error code for sizes the entry point refuses).  Same
 * limits as slayer_conv_synapse, up to 4096 taps. */
int64_t slayer_conv_synapse_wgrad_workspace(int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                                            int64_t kh, int64_t kw, int64_t stride_h, int64_t pad_h, int64_t dil_h);
int slayer_conv_synapse_wgrad(float *grad_weight, const float *grad_out, const float *in,
                              int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                              int64_t kh, int64_t kw, int64_t stride_h, int64_t stride_w,
                              int64_t pad_h, int64_t pad_w, int64_t dil_h, int64_t dil_w,
                              float *workspace, int64_t workspace_floats, void *stream);

/* ---- sigma-delta ---------------------------------------------------------------------------- */

/* _DeltaUnit.forward (axon/delta.py:10-66; a python time loop in the reference, no kernel there):
 * delta = in[t] - pre + residual;  delta_out[t] = delta;
 * cum_error == 0:  y = |delta| >= thr ? delta : 0;
 * cum_error != 0:  error += delta;  y = |error| >= thr ? delta : 0;  error = 0 after an event;
 * residual = delta - y;  pre = in[t].  out[t] = y, or floor(y / quant_step) * quant_step when
 * quant_step > 0 (the floor quantiser Delta.forward applies to its result, axon/delta.py:318).
 * residual_out / error_out receive the final states (M floats each).  threshold follows the decay
 * addressing (one value or one per channel); states are one value or M. */
int slayer_delta_fwd(float *out, float *delta_out, float *residual_out, float *error_out,
                     const float *in, const float *threshold, const float *pre_state,
                     const float *residual_state, const float *error_state,
                     int cum_error, float quant_step,
                     int64_t M, int64_t neurons_per_batch, int64_t num_thresholds,
                     int64_t num_pre, int64_t num_residual, int64_t num_error,
                     int64_t T, void *stream);

/* _DeltaUnit.backward (axon/delta.py:68-103): grad_in[t] = grad_out[t] - grad_out[t+1];
 * grad_threshold[j] = sum of (|d| - thr > 0 ? -d * scale_grad * exp(-||d| - thr| / tau_grad) / thr
 *                                          : -sign(d)) * grad_out over the neurons of threshold j.
 * grad_threshold may be NULL; workspace: M + 64 * num_thresholds floats when it is not. */
int slayer_delta_bwd(float *grad_in, float *grad_threshold, const float *grad_out,
                     const float *delta, const float *threshold, float *workspace,
                     float tau_grad, float scale_grad,
                     int64_t M, int64_t neurons_per_batch, int64_t num_thresholds,
                     int64_t T, void *stream);

/* Running sum along time, sequential float32 adds (dendrite/sigma.py:63 uses torch.cumsum):
 * out[t] = state + in[0] + ... + in[t]; reverse != 0 sums from the last step backwards (the
 * gradient of the forward sum).  state == NULL starts from 0. */
int slayer_cumsum(float *out, const float *in, const float *state, int64_t num_states,
                  int reverse, int64_t M, int64_t T, void *stream);

/* ---- fused CUBA neuron -------------------------------------------------------------------------- */

/* Decays of the fused neuron entry points (slayer_cuba_*, slayer_alif_*, slayer_*_recurrent_fwd): the neuron
 * classes hand their kernels quantize(decay) (neuron/cuba.py:356-374, utils/quantize.py:18-26,52-81: torch.round, i.e. to nearest,
 * ties to even); these entry points do that rounding themselves, so a caller may pass the parameter as it is.
 * The operator entry points (slayer_li_fwd, slayer_ath_fwd, ...) truncate like the kernels they replace. */

/* No single counterpart in the reference: one launch for what cuba.Neuron.forward does with three
 * (neuron/cuba.py:356-374 + :401-410 = leaky_integrator.dynamics, leaky_integrator.dynamics with
 * threshold, Spike.forward).  Bit-identical to slayer_li_fwd -> slayer_li_fwd -> slayer_spike_fwd
 * (each intermediate is rounded to float32 exactly as at the operator boundaries); it only saves the
 * re-reading of the intermediates: 16 instead of 24 bytes per neuron-timestep.
 * thr_scaled = (threshold + eps) * w_scale for the reset (double, <= 0 disables it),
 * spike_threshold = threshold + eps for the spike compare on the float32 voltage.
 * cur_out may be NULL when the current trace is not wanted (no decay gradient in the backward pass):
 * 12 bytes per neuron-timestep; vol_out may be NULL as well when no backward pass will follow
 * (inference): 8 bytes.  cur_last_out / vol_last_out ([M], may be NULL) receive the current and the
 * voltage of the last step, i.e. current[..., -1] and voltage[..., -1], which is what a persistent
 * state needs. */
int slayer_cuba_fwd(float *cur_out, float *vol_out, float *spk_out, float *cur_last_out, float *vol_last_out,
                    const float *in,
                    const float *i_decay, const float *v_decay,
                    const float *i_state, const float *v_state,
                    double thr_scaled, float spike_threshold, int graded, float spike_scale, int w_scale,
                    int64_t M, int64_t neurons_per_batch, int64_t num_i_decays, int64_t num_v_decays,
                    int64_t num_i_states, int64_t num_v_states, int64_t T,
                    const slayer_delays *delays, void *stream);

/* Backward of the above = slayer_spike_bwd -> slayer_li_bwd (voltage) -> slayer_li_bwd (current) in
 * one launch (16 instead of 36 bytes per neuron-timestep); grad_in is bit-identical to the chain.
 * grad_i_decay / grad_v_decay may both be NULL (then current may be NULL too and is not read: 12 bytes
 * per neuron-timestep); workspace: 2*M + 64*(num_i_decays + num_v_decays) floats when they are not. */
int slayer_cuba_bwd(float *grad_in, float *grad_i_decay, float *grad_v_decay,
                    const float *grad_spikes, const float *voltage, const float *current,
                    const float *i_decay, const float *v_decay,
                    float spike_threshold, float tau_rho, float scale_rho, int graded, float *workspace,
                    int64_t M, int64_t neurons_per_batch, int64_t num_i_decays, int64_t num_v_decays,
                    int64_t T, const slayer_delays *delays, void *stream);

/* ---- fused resonate-and-fire neuron ------------------------------------------------------------- */

/* One launch for what rf.Neuron.forward does with two operators (neuron/rf.py:429-436 + :463-471 =
 * resonator.dynamics without threshold, complex.Spike.forward); bit-identical to slayer_res_fwd ->
 * slayer_cspike_fwd, 20 instead of 28 bytes per neuron-timestep.  imag_last is the imaginary sample
 * before step 0 (num_last == 1 broadcasts).  re_out / im_out may both be NULL when no backward pass
 * will follow (inference: 12 bytes); re_last_out / im_last_out ([M], both or neither NULL) receive
 * real[..., -1] and imag[..., -1] for a persistent state.  w_scale must be positive (SLAYER_EINVAL
 * otherwise): the spike conditions are decided on the integer states. */
int slayer_rf_fwd(float *re_out, float *im_out, float *spk_out, float *re_last_out, float *im_last_out,
                  const float *re_in, const float *im_in,
                  const float *sin_decay, const float *cos_decay,
                  const float *re_state, const float *im_state, const float *imag_last,
                  float spike_threshold, int graded, float spike_scale, int w_scale,
                  int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                  int64_t num_re_states, int64_t num_im_states, int64_t num_last,
                  int64_t T, const slayer_delays *delays, void *stream);

/* Backward of the above = slayer_cspike_bwd -> slayer_res_bwd in one launch (20 instead of 44 bytes
 * per neuron-timestep); the input gradients are bit-identical to the chain.  grad_sin / grad_cos may
 * both be NULL; workspace: 2*M + 128*num_decays floats when they are not. */
int slayer_rf_bwd(float *g_re_in, float *g_im_in, float *grad_sin, float *grad_cos,
                  const float *grad_spikes, const float *re, const float *im,
                  const float *sin_decay, const float *cos_decay,
                  float spike_threshold, float tau_rho, float scale_rho, int graded, float *workspace,
                  int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t T, const slayer_delays *delays, void *stream);

/* ---- fused adaptive-threshold LIF neuron ---------------------------------------------------- */

/* One launch for what alif.Neuron.forward does with five operators (neuron/alif.py:499-525 + :557-568 =
 * leaky_integrator.dynamics twice without reset, adaptive_threshold.dynamics, threshold + refractory,
 * Spike.forward); bit-identical to that chain, 20 instead of 52 bytes per neuron-timestep.
 * theta_out receives threshold + refractory (what the spike compares against and what the backward pass
 * needs); th_last_out / ref_last_out ([M], both or neither NULL) receive the threshold and refractory
 * values of the last step, i.e. threshold[..., -1] and refractory[..., -1] of the separate operator.
 * cur_out may be NULL when the current trace is not wanted (no decay gradient in the backward pass):
 * 16 bytes per neuron-timestep; vol_out and theta_out may be NULL as well (together with cur_out) when
 * no backward pass will follow (inference: 8 bytes).  cur_last_out / vol_last_out ([M], may be NULL)
 * receive current[..., -1] and voltage[..., -1]. */
int slayer_alif_fwd(float *cur_out, float *vol_out, float *theta_out, float *spk_out,
                    float *cur_last_out, float *vol_last_out, float *th_last_out, float *ref_last_out,
                    const float *in,
                    const float *i_decay, const float *v_decay, const float *th_decay, const float *ref_decay,
                    const float *i_state, const float *v_state, const float *th_state, const float *ref_state,
                    int64_t th_step_scaled, int64_t th0_scaled, int graded, float spike_scale, int w_scale,
                    int64_t M, int64_t neurons_per_batch,
                    int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays, int64_t num_ref_decays,
                    int64_t num_i_states, int64_t num_v_states, int64_t num_th_states, int64_t num_ref_states,
                    int64_t T, const slayer_delays *delays, void *stream);

/* Backward of the above = slayer_spike_bwd with a threshold tensor -> slayer_li_bwd twice, in one launch
 * (20 instead of 40 bytes per neuron-timestep); grad_in is bit-identical to the chain.  grad_i_decay /
 * grad_v_decay may both be NULL (then current may be NULL too and is not read: 16 bytes per
 * neuron-timestep); workspace: 2*M + 64*(num_i_decays + num_v_decays) floats otherwise. */
int slayer_alif_bwd(float *grad_in, float *grad_i_decay, float *grad_v_decay,
                    const float *grad_spikes, const float *voltage, const float *theta, const float *current,
                    const float *i_decay, const float *v_decay,
                    float tau_rho, float scale_rho, int graded, float *workspace,
                    int64_t M, int64_t neurons_per_batch, int64_t num_i_decays, int64_t num_v_decays,
                    int64_t T, const slayer_delays *delays, void *stream);

/* ---- recurrent layer (CUBA or ALIF neurons) ---------------------------------------------------- */

/* The time loop of utils/recurrent.py:45-81 (CustomRecurrent.forward) for a CUBA neuron
 * (neuron/cuba.py:356-421 called one step at a time), in one launch:
 *   feedback[t] = R s[t-1],  s[t] = neuron(z[t] + feedback[t]),  s[-1] = 0.
 * z, spk_out, vol_out: [N][C][T]; rec_t = R^T followed by a row of zeros, [C + 1][C] (row j = the
 * weights from neuron j; the kernel pads its spike lists with the index of the zero row);
 * decays [1] or [C]; states [1] or [N*C] are the neuron's persistent current / voltage before the
 * first step.  vol_out is the voltage trace the backward pass needs; cur_last_out / vol_last_out
 * ([N*C]) are the current and the (un-reset) voltage of the last step.  graded != 0: a spike carries
 * voltage / spike_scale instead of 1 (spike/spike.py:77-87), into spk_out and into the feedback.
 * C <= 1024.
 * Equal to calling the neuron one step at a time (the state between two calls makes the same float32
 * round trip) whenever the feedback sums are exact in float32, e.g. with quantised weights. */
int slayer_cuba_recurrent_fwd(float *spk_out, float *vol_out, float *cur_last_out, float *vol_last_out,
                              const float *z, const float *rec_t,
                              const float *i_decay, const float *v_decay,
                              const float *i_state, const float *v_state,
                              float spike_threshold, int graded, float spike_scale, int w_scale,
                              int64_t N, int64_t C, int64_t num_i_decays, int64_t num_v_decays,
                              int64_t num_i_states, int64_t num_v_states, int64_t T, void *stream);

/* The same loop for an ALIF neuron (neuron/alif.py:383-623 called one step at a time): a step decays the
 * refractory state and the threshold (towards th0), spikes where voltage >= threshold + refractory, and hands
 * threshold + spike * th_step, refractory + 2 * spike * threshold and the voltage (no reset) to the next step
 * as float32 (neuron/dynamics/adaptive_threshold.py:133-172).  theta_out [N][C][T] receives threshold +
 * refractory of every step (the backward pass needs it); th_last_out / ref_last_out ([N*C]) the decayed
 * threshold and refractory state of the last step, before that step's spike is added.  th_step is the
 * neuron's threshold step in state units (float), th0_scaled = base threshold * w_scale.  Otherwise as above. */
int slayer_alif_recurrent_fwd(float *spk_out, float *vol_out, float *theta_out,
                              float *cur_last_out, float *vol_last_out, float *th_last_out, float *ref_last_out,
                              const float *z, const float *rec_t,
                              const float *i_decay, const float *v_decay, const float *th_decay, const float *ref_decay,
                              const float *i_state, const float *v_state, const float *th_state, const float *ref_state,
                              float th_step, int64_t th0_scaled, int graded, float spike_scale, int w_scale,
                              int64_t N, int64_t C,
                              int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays, int64_t num_ref_decays,
                              int64_t num_i_states, int64_t num_v_states, int64_t num_th_states, int64_t num_ref_states,
                              int64_t T, void *stream);

/* Backward of the loop as utils/recurrent.py:83-112 differentiates it (the carried neuron state is a
 * constant, a step contributes its spike surrogate, the gradient reaches step t-1 through R):
 * grad_z[t] = surrogate(voltage[t] - threshold[t]) * (grad_spikes[t] + (grad_z[t+1] R));  rec = R, [C][C].
 * theta: [N][C][T] thresholds of an ALIF layer (theta_out above), or NULL for the constant spike_threshold.
 * graded selects the surrogate of graded spikes (spike/spike.py:7-19,113-126).
 * The gradient of R is the product grad_z[:, :, 1:] x spikes[:, :, :-1] and is left to the caller. */
int slayer_recurrent_bwd(float *grad_z, const float *grad_spikes, const float *voltage, const float *theta,
                         const float *rec, float spike_threshold, float tau_rho, float scale_rho, int graded,
                         int64_t N, int64_t C, int64_t T, void *stream);

/* The same loops, one launch per time step: for layers of any width up to 16384 neurons (C a multiple of 4).
 * A step multiplies the weight matrix with the spikes of the previous step for the whole batch (the matrix is read
 * once per step, on the matrix cores in float32) and runs one neuron step on the result; the launches follow each
 * other on `stream`.  Same arguments, results and arithmetic as slayer_cuba_recurrent_fwd / slayer_alif_recurrent_fwd
 * except: `rec` is R itself, [C][C] (row c = the weights that reach neuron c); the *_last outputs are 16-byte
 * aligned; the feedback of a step is summed in a fixed order of its own (equal bits whenever the sums are exact in
 * float32, e.g. quantised weights and binary spikes); `workspace` is device memory of at least
 * slayer_recurrent_steps_workspace(N, C, T, alif) floats, 16-byte aligned, whose contents are undefined afterwards
 * (time-major copies of the tensors, the weight matrix in the order the matrix cores read it, the states and the
 * spikes that one step hands to the next).
 * slayer_recurrent_steps_workspace returns the number of floats (with_theta != 0: an ALIF layer), or a negative
 * error code for sizes the entry points refuse (SLAYER_ERANGE: C % 4 != 0, C > 16384, N * C >= 2^29). */
int64_t slayer_recurrent_steps_workspace(int64_t N, int64_t C, int64_t T, int with_theta);
int slayer_cuba_recurrent_steps_fwd(float *spk_out, float *vol_out, float *cur_last_out, float *vol_last_out,
                                    const float *z, const float *rec,
                                    const float *i_decay, const float *v_decay,
                                    const float *i_state, const float *v_state,
                                    float spike_threshold, int graded, float spike_scale, int w_scale,
                                    int64_t N, int64_t C, int64_t num_i_decays, int64_t num_v_decays,
                                    int64_t num_i_states, int64_t num_v_states, int64_t T,
                                    float *workspace, int64_t workspace_floats, void *stream);
int slayer_alif_recurrent_steps_fwd(float *spk_out, float *vol_out, float *theta_out,
                                    float *cur_last_out, float *vol_last_out, float *th_last_out, float *ref_last_out,
                                    const float *z, const float *rec,
                                    const float *i_decay, const float *v_decay, const float *th_decay,
                                    const float *ref_decay,
                                    const float *i_state, const float *v_state, const float *th_state,
                                    const float *ref_state,
                                    float th_step, int64_t th0_scaled, int graded, float spike_scale, int w_scale,
                                    int64_t N, int64_t C,
                                    int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays,
                                    int64_t num_ref_decays,
                                    int64_t num_i_states, int64_t num_v_states, int64_t num_th_states,
                                    int64_t num_ref_states,
                                    int64_t T, float *workspace, int64_t workspace_floats, void *stream);

/* slayer_recurrent_bwd one launch per time step (see above); rec = R, [C][C], as for slayer_recurrent_bwd.
 * Workspace as above (with_theta = theta != NULL). */
int slayer_recurrent_steps_bwd(float *grad_z, const float *grad_spikes, const float *voltage, const float *theta,
                               const float *rec, float spike_threshold, float tau_rho, float scale_rho, int graded,
                               int64_t N, int64_t C, int64_t T,
                               float *workspace, int64_t workspace_floats, void *stream);

/* ---- cross-check implementations (debug mode) ------------------------------------------------ */

/* The reference's debug mode runs its CPU loop next to its kernel and raises on a difference
 * (neuron/dynamics/leaky_integrator.py:134-155,168-205; adaptive_threshold.py:191-225;
 * resonator.py:196-236,254-300).  These entry points are the second implementation for that check
 * here: one thread per neuron, 64-bit integer state, plain global accesses.  Same arguments and
 * results as the entry points without the suffix (the backward variants return grad_input only). */
int slayer_li_fwd_naive(float *out, const float *in, const float *decay, const float *state,
                        double thr_scaled, int w_scale,
                        int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t num_states,
                        int64_t T, void *stream);
int slayer_li_bwd_naive(float *grad_in, const float *grad_out, const float *decay,
                        int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t T, void *stream);
int slayer_ath_fwd_naive(float *th_out, float *ref_out, const float *in,
                         const float *ref_state, const float *ref_decay,
                         const float *th_state, const float *th_decay,
                         int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                         int64_t M, int64_t neurons_per_batch,
                         int64_t num_ref_decays, int64_t num_th_decays,
                         int64_t num_ref_states, int64_t num_th_states,
                         int64_t T, void *stream);
int slayer_res_fwd_naive(float *re_out, float *im_out, const float *re_in, const float *im_in,
                         const float *sin_decay, const float *cos_decay,
                         const float *re_state, const float *im_state,
                         double thr_scaled, int w_scale,
                         int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                         int64_t num_re_states, int64_t num_im_states,
                         int64_t T, void *stream);
int slayer_res_bwd_naive(float *g_re_in, float *g_im_in, const float *g_re, const float *g_im,
                         const float *sin_decay, const float *cos_decay,
                         int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t T, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SLAYER_HIP_H */
