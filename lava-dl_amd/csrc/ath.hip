// Adaptive threshold + refractory dynamics (forward only; the op has no gradient).
#include "common.h"
#include "tile.h"

namespace slayer {

template <bool POW2>
struct AthFwd {
    static constexpr int kIn = 1, kOut = 2;      // out: threshold trace, refractory trace
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[1];
        float* out[2];
        const float *ref_state, *ref_decay, *th_state, *th_decay;
        int step, base;
        float w, inv_w;
        int64_t npb, n_rd, n_td, n_rs, n_ts;
        unsigned* range_flag;
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int) { return 28; }
    static constexpr bool kTransforms = true;    // integer tiles, see to_state / from_state
    static constexpr int kCopyWaves = 2;
    int th, r, mt, mr, th_step, base;
    float w, inv_w;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; th_step = p.step; base = p.base;
        th = r = mt = mr = 0;
        if (valid) {
            th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
            r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
            mt = 4096 - trunc_i32(p.th_decay[param_index(m, p.npb, p.n_td)]);
            mr = 4096 - trunc_i32(p.ref_decay[param_index(m, p.npb, p.n_rd)]);
            check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
            check_state(th, 28, p.range_flag); check_state(r, 28, p.range_flag);
        }
    }
    __device__ __forceinline__ void pre(float4 (&x)[1]) const { x[0] = to_state(x[0], w); }
    __device__ __forceinline__ void post(float4 (&o)[2]) const {
        o[0] = from_state<POW2>(o[0], w, inv_w);
        o[1] = from_state<POW2>(o[1], w, inv_w);
    }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[2]) {
        r = rs0_12(r, mr);
        th = rs0_12(th - base, mt) + base;
        o[0] = __int_as_float(th);
        o[1] = __int_as_float(r);
        const bool fired = __float_as_int(x[0]) >= th + r;
        r += fired ? 2 * th : 0;
        th += fired ? th_step : 0;
    }
    __device__ __forceinline__ void finish(const Params&, int64_t, bool) {}
};

// Adaptive phase threshold: the same threshold / refractory recurrences, driven by a complex
// trace; a step spikes when real >= th + r while the imaginary part crosses zero upwards.
template <bool POW2>
struct ApthFwd {
    static constexpr int kIn = 2, kOut = 2;      // in: real, imag;  out: threshold, refractory
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    struct Params {
        const float* in[2];
        float* out[2];
        const float *im_state, *ref_state, *ref_decay, *th_state, *th_decay;
        int step, base;
        float w, inv_w;
        int64_t npb, n_rd, n_td, n_is, n_rs, n_ts;
        unsigned* range_flag;
    };
    int th, r, mt, mr, th_step, base, im_old;
    unsigned range_acc;                          // float tiles: the states are range-checked in the loop
    float w, inv_w;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; th_step = p.step; base = p.base;
        th = r = mt = mr = im_old = 0;
        range_acc = 0u;
        if (valid) {
            th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
            r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
            im_old = trunc_i32(w * p.im_state[p.n_is == 1 ? 0 : m]);
            mt = 4096 - trunc_i32(p.th_decay[param_index(m, p.npb, p.n_td)]);
            mr = 4096 - trunc_i32(p.ref_decay[param_index(m, p.npb, p.n_rd)]);
            check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
            check_state(th, 28, p.range_flag); check_state(r, 28, p.range_flag);
        }
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[2]) {
        r = rs0_12(r, mr);
        th = rs0_12(th - base, mt) + base;
        range_acc |= ((unsigned)th + (1u << 28)) | ((unsigned)r + (1u << 28));
        const float thf = (float)th, rf = (float)r;
        o[0] = POW2 ? thf * inv_w : thf / w;
        o[1] = POW2 ? rf * inv_w : rf / w;
        const int re = trunc_i32(w * x[0]), im = trunc_i32(w * x[1]);
        const bool fired = (re >= th + r) && (im >= 0) && (im_old < 0);
        r += fired ? 2 * th : 0;
        th += fired ? th_step : 0;
        im_old = im;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t, bool) {
        if (range_exceeded(range_acc, 28)) raise_range_flag(p.range_flag);
    }
};

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_ath_fwd(float* th_out, float* ref_out, const float* in,
                              const float* ref_state, const float* ref_decay,
                              const float* th_state, const float* th_decay,
                              int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                              int64_t M, int64_t neurons_per_batch,
                              int64_t num_ref_decays, int64_t num_th_decays,
                              int64_t num_ref_states, int64_t num_th_states,
                              int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!th_out || !ref_out || !in || !ref_state || !ref_decay || !th_state || !th_decay) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_ref_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_th_decays)) return e;
    if (int e = check_states(M, num_ref_states)) return e;
    if (int e = check_states(M, num_th_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const int64_t lim = 0x7fffffffLL;
    if (th_step_scaled > lim || th_step_scaled < -lim || th0_scaled > lim || th0_scaled < -lim) return SLAYER_ERANGE;
    unsigned* flag = range_flag_for_threshold(th_step_scaled, th0_scaled);
    const float w = (float)w_scale;
    if (is_pow2(w_scale)) {
        AthFwd<true>::Params p{{in}, {th_out, ref_out}, ref_state, ref_decay, th_state, th_decay,
                               (int)th_step_scaled, (int)th0_scaled, w, 1.0f / w, neurons_per_batch,
                               num_ref_decays, num_th_decays, num_ref_states, num_th_states, flag};
        return launch_stream<AthFwd<true>>(p, M, T, (hipStream_t)stream);
    }
    AthFwd<false>::Params p{{in}, {th_out, ref_out}, ref_state, ref_decay, th_state, th_decay,
                            (int)th_step_scaled, (int)th0_scaled, w, 1.0f / w, neurons_per_batch,
                            num_ref_decays, num_th_decays, num_ref_states, num_th_states, flag};
    return launch_stream<AthFwd<false>>(p, M, T, (hipStream_t)stream);
}

extern "C" int slayer_apth_fwd(float* th_out, float* ref_out, const float* re_in, const float* im_in,
                               const float* im_state, const float* ref_state, const float* ref_decay,
                               const float* th_state, const float* th_decay,
                               int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                               int64_t M, int64_t neurons_per_batch,
                               int64_t num_ref_decays, int64_t num_th_decays,
                               int64_t num_im_states, int64_t num_ref_states, int64_t num_th_states,
                               int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!th_out || !ref_out || !re_in || !im_in || !im_state || !ref_state || !ref_decay || !th_state || !th_decay)
        return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_ref_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_th_decays)) return e;
    if (int e = check_states(M, num_im_states)) return e;
    if (int e = check_states(M, num_ref_states)) return e;
    if (int e = check_states(M, num_th_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const int64_t lim = 0x7fffffffLL;
    if (th_step_scaled > lim || th_step_scaled < -lim || th0_scaled > lim || th0_scaled < -lim) return SLAYER_ERANGE;
    unsigned* flag = range_flag_for_threshold(th_step_scaled, th0_scaled);
    const float w = (float)w_scale;
    if (is_pow2(w_scale)) {
        ApthFwd<true>::Params p{{re_in, im_in}, {th_out, ref_out}, im_state, ref_state, ref_decay, th_state, th_decay,
                                (int)th_step_scaled, (int)th0_scaled, w, 1.0f / w, neurons_per_batch,
                                num_ref_decays, num_th_decays, num_im_states, num_ref_states, num_th_states, flag};
        return launch_stream<ApthFwd<true>>(p, M, T, (hipStream_t)stream);
    }
    ApthFwd<false>::Params p{{re_in, im_in}, {th_out, ref_out}, im_state, ref_state, ref_decay, th_state, th_decay,
                             (int)th_step_scaled, (int)th0_scaled, w, 1.0f / w, neurons_per_batch,
                             num_ref_decays, num_th_decays, num_im_states, num_ref_states, num_th_states, flag};
    return launch_stream<ApthFwd<false>>(p, M, T, (hipStream_t)stream);
}
