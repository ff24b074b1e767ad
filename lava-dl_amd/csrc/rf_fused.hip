// Fused resonate-and-fire neuron: resonator recurrence (no reset) + phase-threshold spike in one
// pass (reads 8 B, writes 12 B per neuron-timestep instead of 28 B for the two operators), and the
// matching backward pass (complex-spike surrogate -> reverse-time rotation; reads 12 B, writes 8 B
// instead of 44 B).  Intermediates are rounded exactly as at the operator boundaries, so results
// are bit-identical to chaining resonator.dynamics and complex.Spike.
#include "common.h"
#include "tile.h"

namespace slayer {

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);  // li.hip
int launch_reduce_param_grad_pair(float* grad_a, float* grad_b, const float* partial, float* scratch, int64_t M,
                                  int64_t npb, int64_t num_a, int64_t num_b, hipStream_t stream);  // li.hip
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip

// Integer tiles: inputs are scaled and truncated on the way into LDS, the states leave the sequential
// loop as integers together with the spike decision (taken on the integers: real part above the largest
// state whose output value is still below the threshold, previous imaginary state negative, new one not),
// and become output values and spikes on the way out.
// SHIFT: both inputs are read through an axonal delay and the spikes are stored through one (see Shifts).
template <bool POW2, bool GRADED, bool SHIFT = false>
struct RfFwd {
    static constexpr int kIn = 2, kOut = 3;          // out: real, imag, spikes
    static constexpr bool kReverse = false;
    static constexpr unsigned kShiftIn = SHIFT ? 3u : 0u, kShiftOut = SHIFT ? 4u : 0u;
    static constexpr bool kTransforms = true;
    static constexpr int kCopyWaves = SHIFT ? 4 : 2;     // the shifted copies cost the copy waves more instructions
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[2];
        float* out[3];
        float *re_last, *im_last;                   // [M] real / imaginary part of the last step, or nullptr
        const float *sin_decay, *cos_decay, *re_state, *im_state, *imag_last;
        float w, inv_w, spike_scale;
        int fire_above;                             // a real state above this is at or over the spike threshold
        int64_t npb, nd, n_rs, n_is, n_last;
        Shifts shifts;
        unsigned* range_flag;
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int o) { return o < 2 ? 29 : 0; }     // real, imag (two products per step); not the spike flags
    int re, im, im_prev, s, c, fire_above, fired_last;
    float w, inv_w, spike_scale;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; spike_scale = p.spike_scale; fire_above = p.fire_above;
        re = im = im_prev = s = c = fired_last = 0;
        if (valid) {
            re = trunc_i32(p.re_state[p.n_rs == 1 ? 0 : m] * w);
            im = trunc_i32(p.im_state[p.n_is == 1 ? 0 : m] * w);
            const int64_t j = param_index(m, p.npb, p.nd);
            s = trunc_i32(p.sin_decay[j]);
            c = trunc_i32(p.cos_decay[j]);
            im_prev = (p.imag_last[p.n_last == 1 ? 0 : m] < 0.0f) ? -1 : 0;      // only its sign matters
            check_multiplier(s, p.range_flag); check_multiplier(c, p.range_flag);
            check_state(re, 29, p.range_flag); check_state(im, 29, p.range_flag);
        }
    }
    __device__ __forceinline__ void pre(float4 (&x)[2]) const {
        x[0] = to_state(x[0], w);
        x[1] = to_state(x[1], w);
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[3]) {
        const int re_n = add_sat(rs0_12(c, re) - rs0_12(s, im), __float_as_int(x[0]));
        const int im_n = add_sat(rs0_12(s, re) + rs0_12(c, im), __float_as_int(x[1]));
        const bool fired = (re_n > fire_above) & (im_prev < 0) & (im_n >= 0);
        re = re_n; im = im_n; im_prev = im_n;
        if (SHIFT) fired_last = fired ? 1 : 0;
        o[0] = __int_as_float(re_n);
        o[1] = __int_as_float(im_n);
        o[2] = __int_as_float(fired ? 1 : 0);
    }
    // the reference multiplies the real part by the three conditions one after the other: a spike that
    // does not fire is a zero with the sign of the real part
    __device__ __forceinline__ float spike(float r, float flag) const {
        const bool fired = __float_as_int(flag) != 0;
        if (GRADED) return (fired ? r : r * 0.0f) / spike_scale;
        return fired ? 1.0f : 0.0f;
    }
    __device__ __forceinline__ void post(float4 (&y)[3]) const {
        y[0] = from_state<POW2>(y[0], w, inv_w);
        y[1] = from_state<POW2>(y[1], w, inv_w);
        y[2] = make_float4(spike(y[0].x, y[2].x), spike(y[0].y, y[2].y), spike(y[0].z, y[2].z), spike(y[0].w, y[2].w));
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.re_last) {
            p.re_last[m] = from_state<POW2>(__int_as_float(re), w, inv_w);
            p.im_last[m] = from_state<POW2>(__int_as_float(im), w, inv_w);
        }
        if (SHIFT && valid && p.shifts.last)
            p.shifts.last[m] = spike(from_state<POW2>(__int_as_float(re), w, inv_w), __int_as_float(fired_last));
    }
};

// The spike surrogate does not depend on the recurrence.  STAGED = true evaluates it on the way into LDS (by
// the copy waves of the multi-wave kernel) and the sequential wave keeps only the rotation: without decay
// gradients its two results take the places of real and imag; with them real and imag are still needed for
// the partial sums, so a fourth input slot without a tensor behind it receives the second result.
// SHIFT: the gradient of the spikes is read back through the output delay, both input gradients are stored
// back through the input shift.
template <bool GRADED, bool DECAY_GRAD, bool STAGED, bool SHIFT = false>
struct RfBwd {
    static_assert(DECAY_GRAD || STAGED, "without decay gradients the surrogate is always staged");
    static constexpr unsigned kShiftIn = SHIFT ? 1u : 0u, kShiftOut = SHIFT ? 3u : 0u;
    static constexpr int kIn = (DECAY_GRAD && STAGED) ? 4 : 3;     // grad of spikes, saved real, saved imag[, free slot]
    static constexpr int kOut = 2;
    static constexpr bool kTransforms = STAGED;
    static constexpr int kCopyWaves = STAGED ? (SHIFT ? 8 : 4) : 1;
    static constexpr bool kReverse = true;
    static constexpr int64_t kRows32Below = 4096, kRows16Below = 4096;     // exp per step: keep all lanes busy
    struct Params {
        const float* in[kIn];
        float* out[2];
        const float *sin_decay, *cos_decay;
        float *partial_sin, *partial_cos;
        float spike_thr, tau, rho;
        int64_t npb, nd;
        Shifts shifts;
    };
    float c, s, gr, gi, acc_s, acc_c, thr, tau, rho, half_over_tau, two_tau, neg_rho_over_tau, inv_tau;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        thr = p.spike_thr; tau = p.tau; rho = p.rho;
        half_over_tau = (1.0f / 2.0f) / tau;
        inv_tau = 1.0f / tau;
        two_tau = 2.0f * tau;
        neg_rho_over_tau = (-rho) / tau;
        c = s = gr = gi = acc_s = acc_c = 0.f;
        if (valid) {
            const int64_t j = param_index(m, p.npb, p.nd);
            c = p.cos_decay[j] / 4096.0f;
            s = p.sin_decay[j] / 4096.0f;
        }
    }
    // complex spike surrogate (same expression order as the stand-alone kernel)
    __device__ __forceinline__ void surrogate(float g, float r, float i, float& g_re, float& g_im) const {
        float d_re;
        if (GRADED) d_re = expf(-fmaxf(thr - r, 0.0f) * inv_tau);
        else d_re = half_over_tau * expf(-fabsf(r - thr) * inv_tau);
        const float d_im = half_over_tau * expf(-fabsf(i) * inv_tau);
        const float dr = r - thr;
        const float sg_r = dr > 0.0f ? 1.0f : (dr < 0.0f ? -1.0f : (dr == 0.0f ? 0.0f : dr));
        const float sg_i = i > 0.0f ? 1.0f : (i < 0.0f ? -1.0f : (i == 0.0f ? 0.0f : i));
        const float step_re = 0.5f * (1.0f + sg_r * (1.0f - two_tau * d_re));
        g_re = g * ((rho * d_re) * d_im);
        g_im = g * (((neg_rho_over_tau * sg_i) * d_im) * step_re);
    }
    __device__ __forceinline__ void pre(float4 (&x)[kIn]) const {
        float4 a, b;
        surrogate(x[0].x, x[1].x, x[2].x, a.x, b.x);
        surrogate(x[0].y, x[1].y, x[2].y, a.y, b.y);
        surrogate(x[0].z, x[1].z, x[2].z, a.z, b.z);
        surrogate(x[0].w, x[1].w, x[2].w, a.w, b.w);
        if (DECAY_GRAD) { x[0] = a; x[kIn - 1] = b; }
        else { x[1] = a; x[2] = b; }
    }
    __device__ __forceinline__ void post(float4 (&)[2]) const {}
    __device__ __forceinline__ void step(const float (&x)[kIn], float (&o)[2]) {
        float g_re, g_im;
        if (DECAY_GRAD) {
            const float r = x[1], i = x[2];
            if (STAGED) { g_re = x[0]; g_im = x[kIn - 1]; }
            else surrogate(x[0], r, i, g_re, g_im);
            // gr, gi still hold the gradients of step t+1
            acc_s = __fmaf_rn(gi, r, __fmaf_rn(-gr, i, acc_s));
            acc_c = __fmaf_rn(gi, i, __fmaf_rn(gr, r, acc_c));
        } else {
            g_re = x[1];
            g_im = x[2];
        }
        // reverse-time rotation
        const float ngr = (c * gr + s * gi) + g_re;
        const float ngi = ((-s) * gr + c * gi) + g_im;
        gr = ngr; gi = ngi;
        o[0] = ngr; o[1] = ngi;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (DECAY_GRAD && valid && p.partial_sin) { p.partial_sin[m] = acc_s; p.partial_cos[m] = acc_c; }
    }
};

bool bwd_scan_usable(int64_t M, int64_t npb, int64_t T);                // scan.hip
int launch_res_bwd_scan(float* g_re_in, float* g_im_in, float* partial_sin, float* partial_cos, const float* g_re,
                        const float* g_im, const float* re, const float* im, const float* sin_decay,
                        const float* cos_decay, int surrogate, float spike_thr, float tau, float rho, int64_t M,
                        int64_t npb, int64_t num_decays, int64_t T, const Shifts* shifts,
                        hipStream_t stream);       // scan.hip

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_rf_fwd(float* re_out, float* im_out, float* spk_out, float* re_last_out, float* im_last_out,
                             const float* re_in, const float* im_in,
                             const float* sin_decay, const float* cos_decay,
                             const float* re_state, const float* im_state, const float* imag_last,
                             float spike_threshold, int graded, float spike_scale, int w_scale,
                             int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                             int64_t num_re_states, int64_t num_im_states, int64_t num_last,
                             int64_t T, const slayer_delays* delays, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_delays(delays, M, neurons_per_batch)) return e;
    if (M == 0 || T == 0) return 0;
    if (!spk_out || !re_in || !im_in || !sin_decay || !cos_decay || !re_state || !im_state || !imag_last)
        return SLAYER_ENULL;
    if ((re_out == nullptr) != (im_out == nullptr) || (re_last_out == nullptr) != (im_last_out == nullptr))
        return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    for (int64_t n : {num_re_states, num_im_states, num_last})
        if (int e = check_states(M, n)) return e;
    if (w_scale <= 0) return SLAYER_EINVAL;
    const float w = (float)w_scale;
    const int fire = fire_above_scaled(spike_threshold, w, is_pow2(w_scale));
    hipStream_t st = (hipStream_t)stream;
    const Shifts sh = forward_shifts(delays, neurons_per_batch);
#define SLAYER_RF_S(P, G, S)                                                                                     \
    do {                                                                                                         \
        RfFwd<P, G, S>::Params p{{re_in, im_in}, {re_out, im_out, spk_out}, re_last_out, im_last_out, sin_decay, \
                                 cos_decay, re_state, im_state, imag_last, w, 1.0f / w, spike_scale, fire,       \
                                 neurons_per_batch, num_decays, num_re_states, num_im_states, num_last, sh,      \
                                 range_flag_device()};                                                           \
        return launch_stream<RfFwd<P, G, S>>(p, M, T, st);                                                       \
    } while (0)
#define SLAYER_RF(P, G)                                                                                          \
    do {                                                                                                         \
        if (delays) SLAYER_RF_S(P, G, true);                                                                     \
        SLAYER_RF_S(P, G, false);                                                                                \
    } while (0)
    if (is_pow2(w_scale)) { if (graded) SLAYER_RF(true, true); else SLAYER_RF(true, false); }
    if (graded) SLAYER_RF(false, true);
    SLAYER_RF(false, false);
#undef SLAYER_RF
#undef SLAYER_RF_S
}

extern "C" int slayer_rf_bwd(float* g_re_in, float* g_im_in, float* grad_sin, float* grad_cos,
                             const float* grad_spikes, const float* re, const float* im,
                             const float* sin_decay, const float* cos_decay,
                             float spike_threshold, float tau_rho, float scale_rho, int graded, float* workspace,
                             int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t T,
                             const slayer_delays* delays, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_delays(delays, M, neurons_per_batch)) return e;
    if (int e = check_params(M > 0 ? M : neurons_per_batch, neurons_per_batch, num_decays)) return e;
    if ((grad_sin == nullptr) != (grad_cos == nullptr)) return SLAYER_ENULL;
    const bool want = grad_sin != nullptr;
    if (want && !workspace && M > 0) return SLAYER_ENULL;
    hipStream_t st = (hipStream_t)stream;
    bool in_scan = false;
    if (M > 0 && T > 0) {
        if (!g_re_in || !g_im_in || !grad_spikes || !re || !im || !sin_decay || !cos_decay) return SLAYER_ENULL;
        const Shifts sh = backward_shifts(delays, neurons_per_batch);
#define SLAYER_RF_BWD_H(G, D, S, H)                                                                               \
    do {                                                                                                          \
        using Op = RfBwd<G, D, S, H>;                                                                             \
        Op::Params p{{grad_spikes, re, im}, {g_re_in, g_im_in}, sin_decay, cos_decay,                             \
                     want ? workspace : nullptr, want ? workspace + M : nullptr,                                  \
                     spike_threshold, tau_rho, scale_rho, neurons_per_batch, num_decays, sh};                     \
        if (!S || stream_fits_multiwave<Op>(p, M, T)) {                                                           \
            if (int e = launch_stream<Op>(p, M, T, st)) return e;                                                 \
            done = true;                                                                                          \
        }                                                                                                         \
    } while (0)
#define SLAYER_RF_BWD(G, D, S)                                                                                    \
    do {                                                                                                          \
        if (delays) SLAYER_RF_BWD_H(G, D, S, true); else SLAYER_RF_BWD_H(G, D, S, false);                         \
    } while (0)
        // The staged forms pay off in the multi-wave kernel (three times faster there); the one-wave kernel
        // gains nothing from the split, so large tensors take the unstaged form (partial sums dropped when
        // the decay gradients are not wanted).
        bool done = false;
        if (bwd_scan_usable(M, neurons_per_batch, T) && aligned16(g_re_in) && aligned16(g_im_in) &&
            aligned16(grad_spikes) && aligned16(re) && aligned16(im)) {
            // large tensors: surrogate + complex recurrence as a wave scan over a linear stream
            if (int e = launch_res_bwd_scan(g_re_in, g_im_in, want ? workspace : nullptr, want ? workspace + M : nullptr,
                                            grad_spikes, nullptr, re, im, sin_decay, cos_decay, graded ? 2 : 1,
                                            spike_threshold, tau_rho, scale_rho, M, neurons_per_batch, num_decays,
                                            T, delays ? &sh : nullptr, st))
                return e;
            done = true;
            in_scan = true;
        }
        if (done) {}
        else if (graded) { if (want) SLAYER_RF_BWD(true, true, true); else SLAYER_RF_BWD(true, false, true); }
        else { if (want) SLAYER_RF_BWD(false, true, true); else SLAYER_RF_BWD(false, false, true); }
        if (!done) { if (graded) SLAYER_RF_BWD(true, true, false); else SLAYER_RF_BWD(false, true, false); }
#undef SLAYER_RF_BWD
#undef SLAYER_RF_BWD_H
    }
    if (int e = finish_delay_gradient(delays, grad_spikes, in_scan, M, neurons_per_batch, T, st)) return e;
    if (want) {
        if (M == 0 || T == 0) {
            if (int e = launch_zero_fill(grad_sin, num_decays, st)) return e;
            return launch_zero_fill(grad_cos, num_decays, st);
        }
        return launch_reduce_param_grad_pair(grad_sin, grad_cos, workspace, workspace + 2 * M, M, neurons_per_batch, num_decays,
                                             num_decays, st);
    }
    return 0;
}
