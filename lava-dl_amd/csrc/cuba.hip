// Fused CUBA neuron: current integrator -> voltage integrator with reset -> spike in one pass
// over the input (reads 4 B, writes 12 B per neuron-timestep instead of 24 B for the three
// separate operators), and the matching backward pass (spike surrogate -> voltage gradient
// -> current gradient; reads 12 B, writes 4 B instead of 36 B).  Every intermediate still makes
// the float32 round trip it makes at the operator boundaries (state -> float32 / w -> trunc(w * .)),
// so the results are bit-identical to chaining the separate kernels.
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
// need it): 12 instead of 16 bytes per neuron-timestep.
// SHIFT: the input is read through an axonal delay and the spikes are stored through one (see Shifts).
template <bool POW2, bool GRADED, bool KEEP_CURRENT, bool SHIFT = false>
struct CubaFwd {
    static constexpr int kIn = 1, kOut = KEEP_CURRENT ? 2 : 1;     // out: [current,] voltage
    static constexpr int kVol = kOut - 1;
    static constexpr int kDerived = 1;               // spikes: a function of the voltage alone
    static constexpr unsigned kShiftIn = SHIFT ? 1u : 0u, kShiftOut = SHIFT ? (1u << kOut) : 0u;
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    static constexpr bool kLongPiecesOnAliasedRows = true;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[1];
        float* out[kOut + 1];
        float *cur_last, *vol_last;                  // [M] current / voltage of the last step, or nullptr
        const float *i_decay, *v_decay, *i_state, *v_state;
        float w, inv_w, spike_thr, spike_scale;
        int fire_above;                              // voltage reset when the state exceeds this
        int64_t npb, n_id, n_vd, n_is, n_vs;
        Shifts shifts;
        unsigned* range_flag;
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int) { return 30; }
    static constexpr bool kTransforms = true;        // integer tiles, see to_state / from_state
    static constexpr int kCopyWaves = SHIFT ? 8 : 2;     // the shifted copies cost the copy waves more instructions
    int yc, yv, yv_out, mi, mv, fire_above;
    float w, inv_w, spike_thr, spike_scale;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        yv_out = 0;
        w = p.w; inv_w = p.inv_w; fire_above = p.fire_above; spike_thr = p.spike_thr; spike_scale = p.spike_scale;
        yc = yv = mi = mv = 0;
        if (valid) {
            yc = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m] * w);
            yv = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
            mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m, p.npb, p.n_id)]));
            mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m, p.npb, p.n_vd)]));
            check_multiplier(mi, p.range_flag); check_multiplier(mv, p.range_flag);
            check_state(yc, 30, p.range_flag); check_state(yv, 30, p.range_flag);
        }
    }
    __device__ __forceinline__ void pre(float4 (&x)[1]) const { x[0] = to_state(x[0], w); }
    __device__ __forceinline__ void post(float4 (&o)[kOut]) const {
#pragma unroll
        for (int i = 0; i < kOut; ++i) o[i] = from_state<POW2>(o[i], w, inv_w);
    }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[kOut]) {
        yc = add_sat(rs0_12(yc, mi), __float_as_int(x[0]));
        // the voltage op reads the float32 current: trunc(w * (float(yc) / w)); for a power of two
        // the scaling is exact and only the int -> float32 rounding remains
        const float cf = (float)yc;
        const int yn = add_sat(rs0_12(yv, mv), POW2 ? trunc_i32(cf) : trunc_i32(w * (cf / w)));
        yv = (yn > fire_above) ? 0 : yn;             // float(yn) >= threshold, decided on the integer
        yv_out = yn;
        if (KEEP_CURRENT) o[0] = __int_as_float(yc);
        o[kVol] = __int_as_float(yn);
    }
    // The same step as two Ops for the staged multi-wave kernel: the current recurrence, and the voltage
    // recurrence one chunk later.  What the voltage op reads of the current (the float32 round trip) is worked
    // out by the first wave and left in the voltage tile, where the second wave replaces it with the voltage:
    // that evens out the two steps (8 and 9 instructions instead of 6 and 11).
    static constexpr int kStages = 2;
    static constexpr bool kStagedWhenLarge = true;
    struct Stage0 {
        static constexpr int kIn = 1, kOut = KEEP_CURRENT ? 2 : 1;
        static constexpr bool kReverse = false, kTileMapped = true;
        static constexpr int in_tile(int) { return 0; }
        static constexpr int out_tile(int o) { return o; }       // [current,] what the voltage op reads of it
        int yc, mi;
        float w, inv_w;
        __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
            w = p.w; inv_w = p.inv_w; yc = mi = 0;
            if (valid) {
                yc = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m] * w);
                mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m, p.npb, p.n_id)]));
                check_multiplier(mi, p.range_flag); check_state(yc, 30, p.range_flag);
            }
        }
        __device__ __forceinline__ void step(const float (&x)[1], float (&o)[kOut]) {
            yc = add_sat(rs0_12(yc, mi), __float_as_int(x[0]));
            const float cf = (float)yc;
            if (KEEP_CURRENT) o[0] = __int_as_float(yc);
            o[kVol] = __int_as_float(POW2 ? trunc_i32(cf) : trunc_i32(w * (cf / w)));
        }
        __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
            if (valid && p.cur_last) p.cur_last[m] = from_state<POW2>(__int_as_float(yc), w, inv_w);
        }
    };
    struct Stage1 {
        static constexpr int kIn = 1, kOut = 1;
        static constexpr bool kReverse = false, kTileMapped = true;
        static constexpr int in_tile(int) { return kVol; }
        static constexpr int out_tile(int) { return kVol; }      // in place
        int yv, yv_out, mv, fire_above;
        float w, inv_w, spike_thr, spike_scale;
        __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
            w = p.w; inv_w = p.inv_w; fire_above = p.fire_above; spike_thr = p.spike_thr; spike_scale = p.spike_scale;
            yv = yv_out = mv = 0;
            if (valid) {
                yv = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
                mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m, p.npb, p.n_vd)]));
                check_multiplier(mv, p.range_flag); check_state(yv, 30, p.range_flag);
            }
        }
        __device__ __forceinline__ void step(const float (&x)[1], float (&o)[1]) {
            const int yn = add_sat(rs0_12(yv, mv), __float_as_int(x[0]));
            yv = (yn > fire_above) ? 0 : yn;
            yv_out = yn;
            o[0] = __int_as_float(yn);
        }
        __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
            const float vol = from_state<POW2>(__int_as_float(yv_out), w, inv_w);
            if (valid && p.vol_last) p.vol_last[m] = vol;
            if (SHIFT && valid && p.shifts.last) {
                const float h = (vol >= spike_thr) ? 1.0f : 0.0f;
                p.shifts.last[m] = GRADED ? (h * vol) / spike_scale : h;
            }
        }
    };
    __device__ __forceinline__ float spike(float vol) const {
        const float h = (vol >= spike_thr) ? 1.0f : 0.0f;
        return GRADED ? (h * vol) / spike_scale : h;
    }
    __device__ __forceinline__ float4 derive(const float4 (&y)[kOut]) const {
        return make_float4(spike(y[kVol].x), spike(y[kVol].y), spike(y[kVol].z), spike(y[kVol].w));
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.cur_last) p.cur_last[m] = from_state<POW2>(__int_as_float(yc), w, inv_w);
        if (valid && p.vol_last) p.vol_last[m] = from_state<POW2>(__int_as_float(yv_out), w, inv_w);
        if (SHIFT && valid && p.shifts.last) p.shifts.last[m] = spike(from_state<POW2>(__int_as_float(yv_out), w, inv_w));
    }
};

// DECAY_GRAD = false drops the saved current and both decay-gradient sums: 12 instead of 16 bytes
// per neuron-timestep.
// SHIFT: the gradient of the spikes is read back through the output delay and the gradient of the input is
// stored back through the input shift (the forward pass's Shifts with the sides swapped and the signs flipped).
template <bool GRADED, bool DECAY_GRAD, bool SHIFT = false>
struct CubaBwd {
    static constexpr int kIn = DECAY_GRAD ? 3 : 2, kOut = 1;   // in: grad of spikes, saved voltage[, saved current]
    static constexpr bool kReverse = true;
    static constexpr unsigned kShiftIn = SHIFT ? 1u : 0u, kShiftOut = SHIFT ? 1u : 0u;
    static constexpr int64_t kRows32Below = 4096, kRows16Below = 4096;     // exp per step: keep all lanes busy
    struct Params {
        const float* in[kIn];
        float* out[1];
        const float *i_decay, *v_decay;
        float *partial_i, *partial_v;                // per-neuron decay gradients (DECAY_GRAD only)
        float spike_thr, tau, rho;
        int64_t npb, n_id, n_vd;
        Shifts shifts;
    };
    float ai, av, gc, gx, acc_i, acc_v, spike_thr, tau, rho, lead, inv_tau;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        spike_thr = p.spike_thr; tau = p.tau; rho = p.rho;
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
    static constexpr int kCopyWaves = 8;
    __device__ __forceinline__ float surrogate(float g, float v) const {
        const float d = v - spike_thr;
        return GRADED ? (rho * expf(fminf(d, 0.0f) * inv_tau)) * g : (lead * expf(-fabsf(d) * inv_tau)) * g;
    }
    __device__ __forceinline__ void pre(float4 (&x)[kIn]) const {
        x[0] = make_float4(surrogate(x[0].x, x[1].x), surrogate(x[0].y, x[1].y), surrogate(x[0].z, x[1].z),
                           surrogate(x[0].w, x[1].w));
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

extern "C" int slayer_cuba_fwd(float* cur_out, float* vol_out, float* spk_out, float* cur_last_out,
                               float* vol_last_out, const float* in,
                               const float* i_decay, const float* v_decay,
                               const float* i_state, const float* v_state,
                               double thr_scaled, float spike_threshold, int graded, float spike_scale, int w_scale,
                               int64_t M, int64_t neurons_per_batch, int64_t num_i_decays, int64_t num_v_decays,
                               int64_t num_i_states, int64_t num_v_states, int64_t T,
                               const slayer_delays* delays, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_delays(delays, M, neurons_per_batch)) return e;
    if (M == 0 || T == 0) return 0;
    if (!spk_out || !in || !i_decay || !v_decay || !i_state || !v_state) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_i_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_v_decays)) return e;
    if (int e = check_states(M, num_i_states)) return e;
    if (int e = check_states(M, num_v_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const float w = (float)w_scale;
    const int fa = fire_above(thr_scaled > 0 ? (float)thr_scaled : __builtin_inff());
    hipStream_t st = (hipStream_t)stream;
    const Shifts sh = forward_shifts(delays, neurons_per_batch);
#define SLAYER_CUBA_S(P, G, S)                                                                                   \
    do {                                                                                                         \
        if (cur_out) {                                                                                           \
            CubaFwd<P, G, true, S>::Params p{{in}, {cur_out, vol_out, spk_out}, cur_last_out, vol_last_out,      \
                                             i_decay, v_decay, i_state, v_state, w, 1.0f / w, spike_threshold,   \
                                             spike_scale, fa, neurons_per_batch, num_i_decays, num_v_decays,     \
                                             num_i_states, num_v_states, sh, range_flag_device()};               \
            return launch_stream<CubaFwd<P, G, true, S>>(p, M, T, st);                                           \
        }                                                                                                        \
        CubaFwd<P, G, false, S>::Params p{{in}, {vol_out, spk_out}, cur_last_out, vol_last_out, i_decay,         \
                                          v_decay, i_state, v_state, w, 1.0f / w, spike_threshold, spike_scale,  \
                                          fa, neurons_per_batch, num_i_decays, num_v_decays, num_i_states,       \
                                          num_v_states, sh, range_flag_device()};                                \
        return launch_stream<CubaFwd<P, G, false, S>>(p, M, T, st);                                              \
    } while (0)
#define SLAYER_CUBA(P, G)                                                                                        \
    do {                                                                                                         \
        if (delays) SLAYER_CUBA_S(P, G, true);                                                                   \
        SLAYER_CUBA_S(P, G, false);                                                                              \
    } while (0)
    if (is_pow2(w_scale)) { if (graded) SLAYER_CUBA(true, true); else SLAYER_CUBA(true, false); }
    if (graded) SLAYER_CUBA(false, true);
    SLAYER_CUBA(false, false);
#undef SLAYER_CUBA
#undef SLAYER_CUBA_S
}

extern "C" int slayer_cuba_bwd(float* grad_in, float* grad_i_decay, float* grad_v_decay,
                               const float* grad_spikes, const float* voltage, const float* current,
                               const float* i_decay, const float* v_decay,
                               float spike_threshold, float tau_rho, float scale_rho, int graded, float* workspace,
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
        if (!grad_in || !grad_spikes || !voltage || !i_decay || !v_decay || (want && !current)) return SLAYER_ENULL;
        const Shifts sh = backward_shifts(delays, neurons_per_batch);
        // large tensors: the two recurrences as wave scans over a linear stream
        if (bwd_scan_usable(M, neurons_per_batch, T) && aligned16(grad_in) && aligned16(grad_spikes) &&
            aligned16(voltage) && aligned16(current)) {
            in_scan = true;
            if (int e = launch_cuba_bwd_scan(grad_in, want ? workspace : nullptr, want ? workspace + M : nullptr,
                                             grad_spikes, voltage, nullptr, want ? current : nullptr, i_decay, v_decay,
                                             spike_threshold, tau_rho, scale_rho, graded != 0, M, neurons_per_batch,
                                             num_i_decays, num_v_decays, T, delays ? &sh : nullptr, st))
                return e;
        } else {
#define SLAYER_CUBA_BWD_S(G, S)                                                                                  \
    do {                                                                                                         \
        if (want) {                                                                                              \
            CubaBwd<G, true, S>::Params p{{grad_spikes, voltage, current}, {grad_in}, i_decay, v_decay,          \
                                          workspace, workspace + M, spike_threshold, tau_rho, scale_rho,         \
                                          neurons_per_batch, num_i_decays, num_v_decays, sh};                    \
            if (int e = launch_stream<CubaBwd<G, true, S>>(p, M, T, st)) return e;                               \
        } else {                                                                                                 \
            CubaBwd<G, false, S>::Params p{{grad_spikes, voltage}, {grad_in}, i_decay, v_decay, nullptr,         \
                                           nullptr, spike_threshold, tau_rho, scale_rho, neurons_per_batch,      \
                                           num_i_decays, num_v_decays, sh};                                      \
            if (int e = launch_stream<CubaBwd<G, false, S>>(p, M, T, st)) return e;                              \
        }                                                                                                        \
    } while (0)
#define SLAYER_CUBA_BWD(G)                                                                                       \
    do {                                                                                                         \
        if (delays) SLAYER_CUBA_BWD_S(G, true); else SLAYER_CUBA_BWD_S(G, false);                                \
    } while (0)
        if (graded) SLAYER_CUBA_BWD(true); else SLAYER_CUBA_BWD(false);
#undef SLAYER_CUBA_BWD
#undef SLAYER_CUBA_BWD_S
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
