// Fused adaptive-threshold LIF neuron: current integrator -> voltage integrator (no reset) ->
// threshold / refractory recurrences -> spike against threshold + refractory, in one pass over the
// input (reads 4 B, writes 16 B per neuron-timestep instead of 52 B for the five separate
// operators), and the matching backward pass (spike surrogate with a per-step threshold -> voltage
// gradient -> current gradient; reads 16 B, writes 4 B instead of 40 B).  Intermediates make the
// same float32 round trips as at the operator boundaries, so results are bit-identical to the chain.
#include "common.h"
#include "tile.h"

namespace slayer {

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);  // li.hip
int launch_reduce_param_grad_pair(float* grad_a, float* grad_b, const float* partial, float* scratch, int64_t M,
                                  int64_t npb, int64_t num_a, int64_t num_b, hipStream_t stream);  // li.hip
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip
bool bwd_scan_usable(int64_t M, int64_t npb, int64_t T);                // scan.hip
int launch_cuba_bwd_scan(float* grad_in, float* partial_i, float* partial_v, const float* grad_spikes,
                         const float* voltage, const float* theta, const float* current, const float* i_decay,
                         const float* v_decay, float spike_thr, float tau, float rho, bool graded,
                         int64_t M, int64_t npb, int64_t n_id, int64_t n_vd, int64_t T, const Shifts* shifts,
                         hipStream_t stream);   // scan.hip

// KEEP_CURRENT = false leaves the current trace out (a caller that wants no decay gradient does not
// need it): 16 instead of 20 bytes per neuron-timestep.
//
// Integer tiles: the input is scaled and truncated on the way into LDS; current, voltage, threshold and
// refractory state leave the sequential loop as integers in four tiles and become current, voltage,
// threshold + refractory and spikes on the way out (the tile of the refractory state carries the spikes
// to memory).
// SHIFT: the input is read through an axonal delay and the spikes are stored through one (see Shifts).
template <bool POW2, bool GRADED, bool KEEP_CURRENT, bool SHIFT = false>
struct AlifFwd {
    static constexpr int kIn = 1, kOut = KEEP_CURRENT ? 4 : 3;   // out: [current,] voltage, threshold + refractory, spikes
    static constexpr int kVol = kOut - 3, kTheta = kOut - 2, kSpk = kOut - 1;
    static constexpr unsigned kShiftIn = SHIFT ? 1u : 0u, kShiftOut = SHIFT ? (1u << kSpk) : 0u;
    static constexpr int kCopyWaves = SHIFT ? 4 : 2;     // the shifted copies cost the copy waves more instructions
    static constexpr bool kReverse = false;
    static constexpr bool kTransforms = true;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[1];
        float* out[kOut];
        float *cur_last, *vol_last, *th_last, *ref_last;   // [M] values of the last step, or nullptr
        const float *i_decay, *v_decay, *th_decay, *ref_decay, *i_state, *v_state, *th_state, *ref_state;
        int step, base;
        float w, inv_w, spike_scale;
        int64_t npb, n_id, n_vd, n_td, n_rd, n_is, n_vs, n_ts, n_rs;
        Shifts shifts;
        unsigned* range_flag;
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int o) { return o >= kTheta ? 28 : 30; }   // threshold / refractory : current, voltage
    int yc, yv, th, r, th_out, r_out, mi, mv, mt, mr, th_step, base;
    float w, inv_w, spike_scale;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; spike_scale = p.spike_scale; th_step = p.step; base = p.base;
        yc = yv = th = r = th_out = r_out = mi = mv = mt = mr = 0;
        if (valid) {
            yc = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m] * w);
            yv = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
            th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
            r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
            mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m, p.npb, p.n_id)]));
            mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m, p.npb, p.n_vd)]));
            mt = 4096 - trunc_i32(rintf(p.th_decay[param_index(m, p.npb, p.n_td)]));
            mr = 4096 - trunc_i32(rintf(p.ref_decay[param_index(m, p.npb, p.n_rd)]));
            check_multiplier(mi, p.range_flag); check_multiplier(mv, p.range_flag);
            check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
            check_state(yc, 30, p.range_flag); check_state(yv, 30, p.range_flag);
            check_state(th, 28, p.range_flag); check_state(r, 28, p.range_flag);
        }
    }
    // what the next operator reads of a state: trunc(w * (float(y) / w)); for a power of two the scaling
    // is exact and only the int -> float32 rounding remains
    __device__ __forceinline__ int reread(int y) const {
        const float f = (float)y;
        return POW2 ? trunc_i32(f) : trunc_i32(w * (f / w));
    }
    __device__ __forceinline__ void pre(float4 (&x)[1]) const { x[0] = to_state(x[0], w); }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[kOut]) {
        yc = add_sat(rs0_12(yc, mi), __float_as_int(x[0]));
        yv = add_sat(rs0_12(yv, mv), reread(yc));               // the voltage op reads the float32 current
        r = rs0_12(r, mr);
        th = rs0_12(th - base, mt) + base;
        th_out = th; r_out = r;
        const bool fired = reread(yv) >= th + r;                // the threshold op reads the float32 voltage
        r += fired ? 2 * th : 0;
        th += fired ? th_step : 0;
        if (KEEP_CURRENT) o[0] = __int_as_float(yc);
        o[kVol] = __int_as_float(yv);
        o[kTheta] = __int_as_float(th_out);
        o[kSpk] = __int_as_float(r_out);
    }
    // The same step as two Ops for the staged multi-wave kernel: current and voltage recurrences, and the
    // threshold / refractory recurrences reading the voltage out of its tile one chunk later.
    static constexpr int kStages = 2;
    struct Stage0 {
        static constexpr int kIn = 1, kOut = KEEP_CURRENT ? 2 : 1;
        static constexpr bool kReverse = false, kTileMapped = true;
        static constexpr int in_tile(int) { return 0; }
        static constexpr int out_tile(int o) { return o; }       // [current,] voltage: tiles 0 .. kVol
        int yc, yv, mi, mv;
        float w, inv_w;
        __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
            w = p.w; inv_w = p.inv_w; yc = yv = mi = mv = 0;
            if (valid) {
                yc = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m] * w);
                yv = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
                mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m, p.npb, p.n_id)]));
                mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m, p.npb, p.n_vd)]));
                check_multiplier(mi, p.range_flag); check_multiplier(mv, p.range_flag);
                check_state(yc, 30, p.range_flag); check_state(yv, 30, p.range_flag);
            }
        }
        __device__ __forceinline__ void step(const float (&x)[1], float (&o)[kOut]) {
            yc = add_sat(rs0_12(yc, mi), __float_as_int(x[0]));
            const float cf = (float)yc;
            yv = add_sat(rs0_12(yv, mv), POW2 ? trunc_i32(cf) : trunc_i32(w * (cf / w)));
            if (KEEP_CURRENT) o[0] = __int_as_float(yc);
            o[kVol] = __int_as_float(yv);
        }
        __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
            if (valid && p.cur_last) p.cur_last[m] = from_state<POW2>(__int_as_float(yc), w, inv_w);
            if (valid && p.vol_last) p.vol_last[m] = from_state<POW2>(__int_as_float(yv), w, inv_w);
        }
    };
    struct Stage1 {
        static constexpr int kIn = 1, kOut = 2;
        static constexpr bool kReverse = false, kTileMapped = true;
        static constexpr int in_tile(int) { return kVol; }
        static constexpr int out_tile(int o) { return kTheta + o; }   // threshold, refractory state
        int th, r, th_out, r_out, yv_last, mt, mr, th_step, base;
        float w, inv_w, spike_scale;
        __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
            w = p.w; inv_w = p.inv_w; spike_scale = p.spike_scale; th_step = p.step; base = p.base;
            th = r = th_out = r_out = yv_last = mt = mr = 0;
            if (valid) {
                th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
                r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
                yv_last = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
                mt = 4096 - trunc_i32(rintf(p.th_decay[param_index(m, p.npb, p.n_td)]));
                mr = 4096 - trunc_i32(rintf(p.ref_decay[param_index(m, p.npb, p.n_rd)]));
                check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
                check_state(th, 28, p.range_flag); check_state(r, 28, p.range_flag);
            }
        }
        __device__ __forceinline__ void step(const float (&x)[1], float (&o)[2]) {
            const int yv = __float_as_int(x[0]);
            const float vf = (float)yv;
            r = rs0_12(r, mr);
            th = rs0_12(th - base, mt) + base;
            th_out = th; r_out = r; yv_last = yv;
            const bool fired = (POW2 ? trunc_i32(vf) : trunc_i32(w * (vf / w))) >= th + r;
            r += fired ? 2 * th : 0;
            th += fired ? th_step : 0;
            o[0] = __int_as_float(th_out);
            o[1] = __int_as_float(r_out);
        }
        __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
            const float thf = from_state<POW2>(__int_as_float(th_out), w, inv_w);
            const float rf = from_state<POW2>(__int_as_float(r_out), w, inv_w);
            if (valid && p.th_last) { p.th_last[m] = thf; p.ref_last[m] = rf; }
            if (SHIFT && valid && p.shifts.last) {
                const float vol = from_state<POW2>(__int_as_float(yv_last), w, inv_w);
                const float h = (vol >= thf + rf) ? 1.0f : 0.0f;
                p.shifts.last[m] = GRADED ? (h * vol) / spike_scale : h;
            }
        }
    };
    __device__ __forceinline__ float spike(float vol, float theta) const {
        const float h = (vol >= theta) ? 1.0f : 0.0f;
        return GRADED ? (h * vol) / spike_scale : h;
    }
    __device__ __forceinline__ void post(float4 (&y)[kOut]) const {
        if (KEEP_CURRENT) y[0] = from_state<POW2>(y[0], w, inv_w);
        const float4 vol = from_state<POW2>(y[kVol], w, inv_w);
        const float4 thf = from_state<POW2>(y[kTheta], w, inv_w), rf = from_state<POW2>(y[kSpk], w, inv_w);
        const float4 theta = make_float4(thf.x + rf.x, thf.y + rf.y, thf.z + rf.z, thf.w + rf.w);
        y[kVol] = vol;
        y[kTheta] = theta;
        y[kSpk] = make_float4(spike(vol.x, theta.x), spike(vol.y, theta.y), spike(vol.z, theta.z), spike(vol.w, theta.w));
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.th_last) {
            p.th_last[m] = from_state<POW2>(__int_as_float(th_out), w, inv_w);
            p.ref_last[m] = from_state<POW2>(__int_as_float(r_out), w, inv_w);
        }
        if (valid && p.cur_last) p.cur_last[m] = from_state<POW2>(__int_as_float(yc), w, inv_w);
        if (valid && p.vol_last) p.vol_last[m] = from_state<POW2>(__int_as_float(yv), w, inv_w);
        if (SHIFT && valid && p.shifts.last) {
            const float thf = from_state<POW2>(__int_as_float(th_out), w, inv_w);
            const float rf = from_state<POW2>(__int_as_float(r_out), w, inv_w);
            p.shifts.last[m] = spike(from_state<POW2>(__int_as_float(yv), w, inv_w), thf + rf);
        }
    }
};

// DECAY_GRAD = false drops the saved current and both decay-gradient sums (16 instead of 20 bytes).
// SHIFT: the gradient of the spikes is read back through the output delay, the gradient of the input is stored
// back through the input shift.
template <bool GRADED, bool DECAY_GRAD, bool SHIFT = false>
struct AlifBwd {
    static constexpr int kIn = DECAY_GRAD ? 4 : 3, kOut = 1;   // in: grad of spikes, voltage, threshold + refractory[, current]
    static constexpr bool kReverse = true;
    static constexpr unsigned kShiftIn = SHIFT ? 1u : 0u, kShiftOut = SHIFT ? 1u : 0u;
    static constexpr int64_t kRows32Below = 4096, kRows16Below = 4096;     // exp per step: keep all lanes busy
    struct Params {
        const float* in[kIn];
        float* out[1];
        const float *i_decay, *v_decay;
        float *partial_i, *partial_v;                // per-neuron decay gradients, or nullptr
        float tau, rho;
        int64_t npb, n_id, n_vd;
        Shifts shifts;
    };
    float ai, av, gc, gx, acc_i, acc_v, tau, rho, lead, inv_tau;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        tau = p.tau; rho = p.rho;
        lead = (rho / 2.0f) / tau;
        inv_tau = 1.0f / tau;
        ai = av = gc = gx = acc_i = acc_v = 0.f;
        if (valid) {
            ai = 1.0f - rintf(p.i_decay[param_index(m, p.npb, p.n_id)]) / 4096.0f;
            av = 1.0f - rintf(p.v_decay[param_index(m, p.npb, p.n_vd)]) / 4096.0f;
        }
    }
    // The surrogate does not depend on the recurrence, so it is evaluated on the way into LDS (by all
    // 64 lanes, or by the copy waves of the multi-wave kernel) and takes the place of the incoming gradient.
    static constexpr bool kTransforms = true;
    static constexpr int kCopyWaves = SHIFT ? 8 : 4;
    __device__ __forceinline__ float surrogate(float g, float v, float theta) const {
        const float d = v - theta;
        return GRADED ? (rho * expf(fminf(d, 0.0f) * inv_tau)) * g : (lead * expf(-fabsf(d) * inv_tau)) * g;
    }
    __device__ __forceinline__ void pre(float4 (&x)[kIn]) const {
        x[0] = make_float4(surrogate(x[0].x, x[1].x, x[2].x), surrogate(x[0].y, x[1].y, x[2].y),
                           surrogate(x[0].z, x[1].z, x[2].z), surrogate(x[0].w, x[1].w, x[2].w));
    }
    __device__ __forceinline__ void post(float4 (&)[1]) const {}
    __device__ __forceinline__ void step(const float (&x)[kIn], float (&o)[1]) {
        const float gv = x[0];
        if (DECAY_GRAD) {
            acc_v = __fmaf_rn(gc, x[1], acc_v);      // gc, gx still hold the gradients of step t+1
            acc_i = __fmaf_rn(gx, x[kIn - 1], acc_i);
        }
        gc = av * gc + gv;
        gx = ai * gx + gc;
        o[0] = gx;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (DECAY_GRAD && valid && p.partial_i) { p.partial_i[m] = acc_i; p.partial_v[m] = acc_v; }
    }
};

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_alif_fwd(float* cur_out, float* vol_out, float* theta_out, float* spk_out,
                               float* cur_last_out, float* vol_last_out, float* th_last_out, float* ref_last_out,
                               const float* in,
                               const float* i_decay, const float* v_decay, const float* th_decay, const float* ref_decay,
                               const float* i_state, const float* v_state, const float* th_state, const float* ref_state,
                               int64_t th_step_scaled, int64_t th0_scaled, int graded, float spike_scale, int w_scale,
                               int64_t M, int64_t neurons_per_batch,
                               int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays, int64_t num_ref_decays,
                               int64_t num_i_states, int64_t num_v_states, int64_t num_th_states, int64_t num_ref_states,
                               int64_t T, const slayer_delays* delays, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_delays(delays, M, neurons_per_batch)) return e;
    if (M == 0 || T == 0) return 0;
    if (!spk_out || !in || !i_decay || !v_decay || !th_decay || !ref_decay ||
        !i_state || !v_state || !th_state || !ref_state)
        return SLAYER_ENULL;
    if ((th_last_out == nullptr) != (ref_last_out == nullptr)) return SLAYER_ENULL;
    if ((vol_out == nullptr) != (theta_out == nullptr) || (vol_out == nullptr && cur_out != nullptr)) return SLAYER_ENULL;
    for (int64_t n : {num_i_decays, num_v_decays, num_th_decays, num_ref_decays})
        if (int e = check_params(M, neurons_per_batch, n)) return e;
    for (int64_t n : {num_i_states, num_v_states, num_th_states, num_ref_states})
        if (int e = check_states(M, n)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const int64_t lim = 0x7fffffffLL;
    if (th_step_scaled > lim || th_step_scaled < -lim || th0_scaled > lim || th0_scaled < -lim) return SLAYER_ERANGE;
    const float w = (float)w_scale;
    hipStream_t st = (hipStream_t)stream;
#define SLAYER_ALIF_ARGS cur_last_out, vol_last_out, th_last_out, ref_last_out, i_decay, v_decay, th_decay, ref_decay, i_state,       \
                         v_state, th_state, ref_state, (int)th_step_scaled, (int)th0_scaled, w, 1.0f / w,         \
                         spike_scale, neurons_per_batch, num_i_decays, num_v_decays, num_th_decays,               \
                         num_ref_decays, num_i_states, num_v_states, num_th_states, num_ref_states, sh, flag
    const Shifts sh = forward_shifts(delays, neurons_per_batch);
    unsigned* flag = range_flag_for_threshold(th_step_scaled, th0_scaled);
#define SLAYER_ALIF_S(P, G, S)                                                                                    \
    do {                                                                                                          \
        if (cur_out) {                                                                                            \
            AlifFwd<P, G, true, S>::Params p{{in}, {cur_out, vol_out, theta_out, spk_out}, SLAYER_ALIF_ARGS};     \
            return launch_stream<AlifFwd<P, G, true, S>>(p, M, T, st);                                            \
        }                                                                                                         \
        AlifFwd<P, G, false, S>::Params p{{in}, {vol_out, theta_out, spk_out}, SLAYER_ALIF_ARGS};                 \
        return launch_stream<AlifFwd<P, G, false, S>>(p, M, T, st);                                               \
    } while (0)
#define SLAYER_ALIF(P, G)                                                                                         \
    do {                                                                                                          \
        if (delays) SLAYER_ALIF_S(P, G, true);                                                                    \
        SLAYER_ALIF_S(P, G, false);                                                                               \
    } while (0)
    if (is_pow2(w_scale)) { if (graded) SLAYER_ALIF(true, true); else SLAYER_ALIF(true, false); }
    if (graded) SLAYER_ALIF(false, true);
    SLAYER_ALIF(false, false);
#undef SLAYER_ALIF
#undef SLAYER_ALIF_S
#undef SLAYER_ALIF_ARGS
}

extern "C" int slayer_alif_bwd(float* grad_in, float* grad_i_decay, float* grad_v_decay,
                               const float* grad_spikes, const float* voltage, const float* theta, const float* current,
                               const float* i_decay, const float* v_decay,
                               float tau_rho, float scale_rho, int graded, float* workspace,
                               int64_t M, int64_t neurons_per_batch, int64_t num_i_decays, int64_t num_v_decays,
                               int64_t T, const slayer_delays* delays, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_delays(delays, M, neurons_per_batch)) return e;
    const int64_t mm = M > 0 ? M : neurons_per_batch;
    if (int e = check_params(mm, neurons_per_batch, num_i_decays)) return e;
    if (int e = check_params(mm, neurons_per_batch, num_v_decays)) return e;
    if ((grad_i_decay == nullptr) != (grad_v_decay == nullptr)) return SLAYER_ENULL;
    const bool want = grad_i_decay != nullptr;
    if (want && !workspace && M > 0) return SLAYER_ENULL;
    hipStream_t st = (hipStream_t)stream;
    bool in_scan = false;
    if (M > 0 && T > 0) {
        if (!grad_in || !grad_spikes || !voltage || !theta || !i_decay || !v_decay || (want && !current))
            return SLAYER_ENULL;
        const Shifts sh = backward_shifts(delays, neurons_per_batch);
        // large tensors: the two recurrences as wave scans over a linear stream
        if (bwd_scan_usable(M, neurons_per_batch, T) && aligned16(grad_in) && aligned16(grad_spikes) &&
            aligned16(voltage) && aligned16(theta) && aligned16(current)) {
            in_scan = true;
            if (int e = launch_cuba_bwd_scan(grad_in, want ? workspace : nullptr, want ? workspace + M : nullptr,
                                             grad_spikes, voltage, theta, want ? current : nullptr, i_decay, v_decay,
                                             0.0f, tau_rho, scale_rho, graded != 0, M, neurons_per_batch,
                                             num_i_decays, num_v_decays, T, delays ? &sh : nullptr, st))
                return e;
        } else {
#define SLAYER_ALIF_BWD_S(G, S)                                                                                   \
    do {                                                                                                          \
        if (want) {                                                                                               \
            AlifBwd<G, true, S>::Params p{{grad_spikes, voltage, theta, current}, {grad_in}, i_decay, v_decay,    \
                                          workspace, workspace + M, tau_rho, scale_rho, neurons_per_batch,        \
                                          num_i_decays, num_v_decays, sh};                                        \
            if (int e = launch_stream<AlifBwd<G, true, S>>(p, M, T, st)) return e;                                \
        } else {                                                                                                  \
            AlifBwd<G, false, S>::Params p{{grad_spikes, voltage, theta}, {grad_in}, i_decay, v_decay, nullptr,   \
                                           nullptr, tau_rho, scale_rho, neurons_per_batch, num_i_decays,          \
                                           num_v_decays, sh};                                                     \
            if (int e = launch_stream<AlifBwd<G, false, S>>(p, M, T, st)) return e;                               \
        }                                                                                                         \
    } while (0)
#define SLAYER_ALIF_BWD(G)                                                                                        \
    do {                                                                                                          \
        if (delays) SLAYER_ALIF_BWD_S(G, true); else SLAYER_ALIF_BWD_S(G, false);                                 \
    } while (0)
        if (graded) SLAYER_ALIF_BWD(true); else SLAYER_ALIF_BWD(false);
#undef SLAYER_ALIF_BWD
#undef SLAYER_ALIF_BWD_S
        }
    }
    if (int e = finish_delay_gradient(delays, grad_spikes, in_scan, M, neurons_per_batch, T, st)) return e;
    if (want) {
        if (M == 0 || T == 0) {
            if (int e = launch_zero_fill(grad_i_decay, num_i_decays, st)) return e;
            return launch_zero_fill(grad_v_decay, num_v_decays, st);
        }
        return launch_reduce_param_grad_pair(grad_i_decay, grad_v_decay, workspace, workspace + 2 * M, M, neurons_per_batch, num_i_decays,
                                             num_v_decays, st);
    }
    return 0;
}
