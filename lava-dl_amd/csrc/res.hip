// Resonator: complex rotating-decay fixed-point recurrence and its reverse-time gradient.
#include "common.h"
#include "tile.h"

namespace slayer {

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);  // li.hip
int launch_reduce_param_grad_pair(float* grad_a, float* grad_b, const float* partial, float* scratch, int64_t M,
                                  int64_t npb, int64_t num_a, int64_t num_b, hipStream_t stream);  // li.hip
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip

template <bool POW2, bool HAS_THR>
struct ResFwd {
    static constexpr int kIn = 2, kOut = 2;
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 32768;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[2];
        float* out[2];
        const float *sin_decay, *cos_decay, *re_state, *im_state;
        float w, inv_w;
        int fire_above, im_reset;                // reset when the imaginary state exceeds fire_above
        int64_t npb, num_decays, n_rs, n_is;
        unsigned* range_flag;
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int) { return 29; }     // two products per step
    static constexpr bool kTransforms = true;    // integer tiles, see to_state / from_state
    int re, im, s, c, fire_above, im_reset;
    float w, inv_w;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; fire_above = p.fire_above; im_reset = p.im_reset;
        re = im = s = c = 0;
        if (valid) {
            re = trunc_i32(p.re_state[p.n_rs == 1 ? 0 : m] * w);
            im = trunc_i32(p.im_state[p.n_is == 1 ? 0 : m] * w);
            const int64_t j = param_index(m, p.npb, p.num_decays);
            s = trunc_i32(p.sin_decay[j]);
            c = trunc_i32(p.cos_decay[j]);
            check_multiplier(s, p.range_flag); check_multiplier(c, p.range_flag);
            check_state(re, 29, p.range_flag); check_state(im, 29, p.range_flag);
        }
    }
    __device__ __forceinline__ void pre(float4 (&x)[2]) const {
        x[0] = to_state(x[0], w);
        x[1] = to_state(x[1], w);
    }
    __device__ __forceinline__ void post(float4 (&o)[2]) const {
        o[0] = from_state<POW2>(o[0], w, inv_w);
        o[1] = from_state<POW2>(o[1], w, inv_w);
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[2]) {
        const int re_n = add_sat(rs0_12(c, re) - rs0_12(s, im), __float_as_int(x[0]));
        const int im_n = add_sat(rs0_12(s, re) + rs0_12(c, im), __float_as_int(x[1]));
        o[0] = __int_as_float(re_n);
        o[1] = __int_as_float(im_n);
        if (HAS_THR) {
            // float(im_n) >= threshold, decided on the integer; the kept imaginary state makes a
            // float32 round trip, as the mixed int/float expression of the CPU branch does
            const bool fired = im_n > fire_above;
            re = fired ? 0 : re_n;
            im = fired ? im_reset : trunc_i32((float)im_n);
        } else {
            re = re_n;
            im = im_n;
        }
    }
    __device__ __forceinline__ void finish(const Params&, int64_t, bool) {}
};

// Adaptive resonator: the resonator recurrence (no reset) with an adaptive threshold and a
// refractory state driven by the imaginary part; four output traces.
template <bool POW2>
struct AdResFwd {
    static constexpr int kIn = 2, kOut = 4;      // out: real, imag, threshold, refractory
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = 16384;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[2];
        float* out[4];
        const float *sin_decay, *cos_decay, *ref_decay, *th_decay;
        const float *re_state, *im_state, *ref_state, *th_state;
        int step, base;
        float w, inv_w;
        int64_t npb, nd, n_rd, n_td, n_res, n_ims, n_rs, n_ts;
        unsigned* range_flag;
    };
    int re, im, s, c, th, r, mt, mr, th_step, base;
    unsigned acc_res, acc_th;                    // float tiles: the states are range-checked in the loop
    float w, inv_w;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; th_step = p.step; base = p.base;
        re = im = s = c = th = r = mt = mr = 0;
        acc_res = acc_th = 0u;
        if (valid) {
            re = trunc_i32(p.re_state[p.n_res == 1 ? 0 : m] * w);
            im = trunc_i32(p.im_state[p.n_ims == 1 ? 0 : m] * w);
            th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
            r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
            const int64_t j = param_index(m, p.npb, p.nd);
            s = trunc_i32(p.sin_decay[j]);
            c = trunc_i32(p.cos_decay[j]);
            mt = 4096 - trunc_i32(p.th_decay[param_index(m, p.npb, p.n_td)]);
            mr = 4096 - trunc_i32(p.ref_decay[param_index(m, p.npb, p.n_rd)]);
            check_multiplier(s, p.range_flag); check_multiplier(c, p.range_flag);
            check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
            check_state(re, 29, p.range_flag); check_state(im, 29, p.range_flag);
            check_state(th, 28, p.range_flag); check_state(r, 28, p.range_flag);
        }
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[4]) {
        r = rs0_12(r, mr);
        th = rs0_12(th - base, mt) + base;
        const int re_n = add_sat(rs0_12(c, re) - rs0_12(s, im), trunc_i32(w * x[0]));
        const int im_n = add_sat(rs0_12(s, re) + rs0_12(c, im), trunc_i32(w * x[1]));
        acc_res |= ((unsigned)re_n + (1u << 29)) | ((unsigned)im_n + (1u << 29));
        acc_th |= ((unsigned)th + (1u << 28)) | ((unsigned)r + (1u << 28));
        const float ref = (float)re_n, imf = (float)im_n, thf = (float)th, rf = (float)r;
        o[0] = POW2 ? ref * inv_w : ref / w;
        o[1] = POW2 ? imf * inv_w : imf / w;
        o[2] = POW2 ? thf * inv_w : thf / w;
        o[3] = POW2 ? rf * inv_w : rf / w;
        const bool fired = im_n >= th + r;
        r += fired ? 2 * th : 0;
        th += fired ? th_step : 0;
        re = re_n;
        im = im_n;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t, bool) {
        if (range_exceeded(acc_res, 29) || range_exceeded(acc_th, 28)) raise_range_flag(p.range_flag);
    }
};

struct ResBwd {
    static constexpr int kIn = 4, kOut = 2;      // in: g_re, g_im, saved re, saved im
    static constexpr bool kReverse = true;
    static constexpr int kCopyWaves = 2;
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = 16384;
    struct Params {
        const float* in[4];
        float* out[2];
        const float *sin_decay, *cos_decay;
        float *partial_sin, *partial_cos;        // per-neuron sums, or nullptr
        int64_t npb, num_decays;
    };
    float c, s, gr, gi, acc_s, acc_c;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        c = s = gr = gi = acc_s = acc_c = 0.f;
        if (valid) {
            const int64_t j = param_index(m, p.npb, p.num_decays);
            c = p.cos_decay[j] / 4096.0f;
            s = p.sin_decay[j] / 4096.0f;
        }
    }
    __device__ __forceinline__ void step(const float (&x)[4], float (&o)[2]) {
        // gr, gi still hold the gradients of step t+1; x[2], x[3] are re[t], im[t]
        acc_s = __fmaf_rn(gi, x[2], __fmaf_rn(-gr, x[3], acc_s));
        acc_c = __fmaf_rn(gi, x[3], __fmaf_rn(gr, x[2], acc_c));
        const float ngr = (c * gr + s * gi) + x[0];
        const float ngi = ((-s) * gr + c * gi) + x[1];
        gr = ngr; gi = ngi;
        o[0] = ngr; o[1] = ngi;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.partial_sin) { p.partial_sin[m] = acc_s; p.partial_cos[m] = acc_c; }
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

template <bool POW2, bool HAS_THR>
static int res_fwd_launch(float* re_out, float* im_out, const float* re_in, const float* im_in,
                          const float* sin_decay, const float* cos_decay, const float* re_state,
                          const float* im_state, float thr, int im_reset, float w,
                          int64_t M, int64_t npb, int64_t nd, int64_t n_rs, int64_t n_is, int64_t T,
                          hipStream_t stream) {
    using Op = ResFwd<POW2, HAS_THR>;
    typename Op::Params p{{re_in, im_in}, {re_out, im_out}, sin_decay, cos_decay, re_state, im_state,
                          w, 1.0f / w, fire_above(thr), im_reset, npb, nd, n_rs, n_is, range_flag_device()};
    if (HAS_THR && (im_reset >= (1 << 29) || im_reset < -(1 << 29))) range_flag_raise_from_host();
    return launch_stream<Op>(p, M, T, stream);
}

extern "C" int slayer_res_fwd(float* re_out, float* im_out, const float* re_in, const float* im_in,
                              const float* sin_decay, const float* cos_decay,
                              const float* re_state, const float* im_state,
                              double thr_scaled, int w_scale,
                              int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                              int64_t num_re_states, int64_t num_im_states,
                              int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!re_out || !im_out || !re_in || !im_in || !sin_decay || !cos_decay || !re_state || !im_state)
        return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    if (int e = check_states(M, num_re_states)) return e;
    if (int e = check_states(M, num_im_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const float w = (float)w_scale;
    const bool has_thr = thr_scaled >= 0;
    const float thr = (float)thr_scaled;
    const int im_reset = has_thr ? (int)(float)(thr_scaled - 1.0) : 0;
    hipStream_t st = (hipStream_t)stream;
#define SLAYER_RES_ARGS re_out, im_out, re_in, im_in, sin_decay, cos_decay, re_state, im_state, thr, im_reset, w, \
                        M, neurons_per_batch, num_decays, num_re_states, num_im_states, T, st
    if (is_pow2(w_scale))
        return has_thr ? res_fwd_launch<true, true>(SLAYER_RES_ARGS) : res_fwd_launch<true, false>(SLAYER_RES_ARGS);
    return has_thr ? res_fwd_launch<false, true>(SLAYER_RES_ARGS) : res_fwd_launch<false, false>(SLAYER_RES_ARGS);
#undef SLAYER_RES_ARGS
}

extern "C" int slayer_res_bwd(float* g_re_in, float* g_im_in, float* grad_sin, float* grad_cos,
                              const float* g_re, const float* g_im, const float* re, const float* im,
                              const float* sin_decay, const float* cos_decay, float* workspace,
                              int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                              int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_params(M > 0 ? M : neurons_per_batch, neurons_per_batch, num_decays)) return e;
    if ((grad_sin == nullptr) != (grad_cos == nullptr)) return SLAYER_ENULL;
    const bool want = grad_sin != nullptr;
    if (want && !workspace && M > 0) return SLAYER_ENULL;
    hipStream_t st = (hipStream_t)stream;
    if (M > 0 && T > 0) {
        if (!g_re_in || !g_im_in || !g_re || !g_im || !re || !im || !sin_decay || !cos_decay) return SLAYER_ENULL;
        if (bwd_scan_usable(M, neurons_per_batch, T) && aligned16(g_re_in) && aligned16(g_im_in) && aligned16(g_re) &&
            aligned16(g_im) && aligned16(re) && aligned16(im)) {
            // large tensors: the complex recurrence as a wave scan over a linear stream
            if (int e = launch_res_bwd_scan(g_re_in, g_im_in, want ? workspace : nullptr, want ? workspace + M : nullptr,
                                            g_re, g_im, re, im, sin_decay, cos_decay, 0, 0.0f, 1.0f, 0.0f, M,
                                            neurons_per_batch, num_decays, T, nullptr, st))
                return e;
        } else {
            ResBwd::Params p{{g_re, g_im, re, im}, {g_re_in, g_im_in}, sin_decay, cos_decay,
                             want ? workspace : nullptr, want ? workspace + M : nullptr,
                             neurons_per_batch, num_decays};
            if (int e = launch_stream<ResBwd>(p, M, T, st)) return e;
        }
    }
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

extern "C" int slayer_adres_fwd(float* re_out, float* im_out, float* th_out, float* ref_out,
                                const float* re_in, const float* im_in,
                                const float* sin_decay, const float* cos_decay,
                                const float* ref_decay, const float* th_decay,
                                const float* re_state, const float* im_state,
                                const float* ref_state, const float* th_state,
                                int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                                int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                                int64_t num_ref_decays, int64_t num_th_decays,
                                int64_t num_re_states, int64_t num_im_states,
                                int64_t num_ref_states, int64_t num_th_states,
                                int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!re_out || !im_out || !th_out || !ref_out || !re_in || !im_in || !sin_decay || !cos_decay || !ref_decay ||
        !th_decay || !re_state || !im_state || !ref_state || !th_state)
        return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_ref_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_th_decays)) return e;
    for (int64_t n : {num_re_states, num_im_states, num_ref_states, num_th_states})
        if (int e = check_states(M, n)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const int64_t lim = 0x7fffffffLL;
    if (th_step_scaled > lim || th_step_scaled < -lim || th0_scaled > lim || th0_scaled < -lim) return SLAYER_ERANGE;
    unsigned* flag = range_flag_for_threshold(th_step_scaled, th0_scaled);
    const float w = (float)w_scale;
    hipStream_t st = (hipStream_t)stream;
    if (is_pow2(w_scale)) {
        AdResFwd<true>::Params p{{re_in, im_in}, {re_out, im_out, th_out, ref_out}, sin_decay, cos_decay, ref_decay,
                                 th_decay, re_state, im_state, ref_state, th_state, (int)th_step_scaled,
                                 (int)th0_scaled, w, 1.0f / w, neurons_per_batch, num_decays, num_ref_decays,
                                 num_th_decays, num_re_states, num_im_states, num_ref_states, num_th_states, flag};
        return launch_stream<AdResFwd<true>>(p, M, T, st);
    }
    AdResFwd<false>::Params p{{re_in, im_in}, {re_out, im_out, th_out, ref_out}, sin_decay, cos_decay, ref_decay,
                              th_decay, re_state, im_state, ref_state, th_state, (int)th_step_scaled,
                              (int)th0_scaled, w, 1.0f / w, neurons_per_batch, num_decays, num_ref_decays,
                              num_th_decays, num_re_states, num_im_states, num_ref_states, num_th_states, flag};
    return launch_stream<AdResFwd<false>>(p, M, T, st);
}
