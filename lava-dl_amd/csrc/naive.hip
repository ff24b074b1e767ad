// Independent one-thread-per-neuron implementations with 64-bit integer state.  They exist for the
// debug=True mode of the python operators, which runs both implementations and raises on any
// difference (the role the CPU-loop-versus-kernel check plays in the reference).  Simple on purpose:
// plain loops over time, direct global accesses, no staging -- slow, and exact even where a state
// leaves the 32-bit range of the streaming kernels.
#include "common.h"
#include "tile.h"

namespace slayer {

__device__ __forceinline__ long long rs0_12_i64(long long p) {
    return p >= 0 ? (p >> 12) : -((-p) >> 12);
}
__device__ __forceinline__ long long trunc_i64(float x) { return (long long)x; }

__global__ void li_fwd_naive(float* out, const float* in, const float* decay, const float* state, float thr,
                             float w, int64_t M, int64_t npb, int64_t nd, int64_t ns, int T) {
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    long long y = trunc_i64(state[ns == 1 ? 0 : m] * w);
    const long long mult = 4096 - trunc_i64(decay[param_index(m, npb, nd)]);
    for (int t = 0; t < T; ++t) {
        const long long yn = rs0_12_i64(y * mult) + trunc_i64(w * in[m * T + t]);
        const float yf = (float)yn;
        out[m * T + t] = yf / w;
        y = (yf >= thr) ? 0 : yn;
    }
}

__global__ void li_bwd_naive(float* gin, const float* gout, const float* decay, int64_t M, int64_t npb,
                             int64_t nd, int T) {
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    const float a = 1.0f - decay[param_index(m, npb, nd)] / 4096.0f;
    float g = 0.0f;
    for (int t = T - 1; t >= 0; --t) {
        g = a * g + gout[m * T + t];
        gin[m * T + t] = g;
    }
}

__global__ void ath_fwd_naive(float* th_out, float* ref_out, const float* in, const float* ref_state,
                              const float* ref_decay, const float* th_state, const float* th_decay,
                              long long step, long long base, float w, int64_t M, int64_t npb,
                              int64_t n_rd, int64_t n_td, int64_t n_rs, int64_t n_ts, int T) {
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    long long th = trunc_i64(th_state[n_ts == 1 ? 0 : m] * w);
    long long r = trunc_i64(ref_state[n_rs == 1 ? 0 : m] * w);
    const long long mt = 4096 - trunc_i64(th_decay[param_index(m, npb, n_td)]);
    const long long mr = 4096 - trunc_i64(ref_decay[param_index(m, npb, n_rd)]);
    for (int t = 0; t < T; ++t) {
        r = rs0_12_i64(r * mr);
        th = rs0_12_i64((th - base) * mt) + base;
        th_out[m * T + t] = (float)th / w;
        ref_out[m * T + t] = (float)r / w;
        if (trunc_i64(w * in[m * T + t]) >= th + r) {
            r += 2 * th;
            th += step;
        }
    }
}

__global__ void res_fwd_naive(float* re_out, float* im_out, const float* re_in, const float* im_in,
                              const float* sin_decay, const float* cos_decay, const float* re_state,
                              const float* im_state, float thr, int has_thr, long long im_reset, float w,
                              int64_t M, int64_t npb, int64_t nd, int64_t n_rs, int64_t n_is, int T) {
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    long long re = trunc_i64(re_state[n_rs == 1 ? 0 : m] * w);
    long long im = trunc_i64(im_state[n_is == 1 ? 0 : m] * w);
    const int64_t j = param_index(m, npb, nd);
    const long long s = trunc_i64(sin_decay[j]), c = trunc_i64(cos_decay[j]);
    for (int t = 0; t < T; ++t) {
        const long long re_n = rs0_12_i64(c * re) - rs0_12_i64(s * im) + trunc_i64(w * re_in[m * T + t]);
        const long long im_n = rs0_12_i64(s * re) + rs0_12_i64(c * im) + trunc_i64(w * im_in[m * T + t]);
        const float imf = (float)im_n;
        re_out[m * T + t] = (float)re_n / w;
        im_out[m * T + t] = imf / w;
        if (has_thr) {
            const bool fired = imf >= thr;
            re = fired ? 0 : re_n;
            im = fired ? im_reset : trunc_i64(imf);
        } else {
            re = re_n;
            im = im_n;
        }
    }
}

__global__ void res_bwd_naive(float* gr_out, float* gi_out, const float* g_re, const float* g_im,
                              const float* sin_decay, const float* cos_decay, int64_t M, int64_t npb,
                              int64_t nd, int T) {
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    const int64_t j = param_index(m, npb, nd);
    const float c = cos_decay[j] / 4096.0f, s = sin_decay[j] / 4096.0f;
    float gr = 0.0f, gi = 0.0f;
    for (int t = T - 1; t >= 0; --t) {
        const float ngr = (c * gr + s * gi) + g_re[m * T + t];
        const float ngi = ((-s) * gr + c * gi) + g_im[m * T + t];
        gr = ngr; gi = ngi;
        gr_out[m * T + t] = gr;
        gi_out[m * T + t] = gi;
    }
}

}  // namespace slayer

using namespace slayer;

#define NAIVE_LAUNCH(kernel, M, stream, ...) \
    hipLaunchKernelGGL(kernel, dim3((unsigned)(((M) + 255) / 256)), dim3(256), 0, (hipStream_t)(stream), __VA_ARGS__)

extern "C" int slayer_li_fwd_naive(float* out, const float* in, const float* decay, const float* state,
                                   double thr_scaled, int w_scale, int64_t M, int64_t neurons_per_batch,
                                   int64_t num_decays, int64_t num_states, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in || !decay || !state) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    if (int e = check_states(M, num_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const float thr = thr_scaled > 0 ? (float)thr_scaled : __builtin_inff();
    NAIVE_LAUNCH(li_fwd_naive, M, stream, out, in, decay, state, thr, (float)w_scale, M, neurons_per_batch,
                 num_decays, num_states, (int)T);
    return (int)hipGetLastError();
}

extern "C" int slayer_li_bwd_naive(float* grad_in, const float* grad_out, const float* decay, int64_t M,
                                   int64_t neurons_per_batch, int64_t num_decays, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!grad_in || !grad_out || !decay) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    NAIVE_LAUNCH(li_bwd_naive, M, stream, grad_in, grad_out, decay, M, neurons_per_batch, num_decays, (int)T);
    return (int)hipGetLastError();
}

extern "C" int slayer_ath_fwd_naive(float* th_out, float* ref_out, const float* in,
                                    const float* ref_state, const float* ref_decay,
                                    const float* th_state, const float* th_decay,
                                    int64_t th_step_scaled, int64_t th0_scaled, int w_scale,
                                    int64_t M, int64_t neurons_per_batch,
                                    int64_t num_ref_decays, int64_t num_th_decays,
                                    int64_t num_ref_states, int64_t num_th_states, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!th_out || !ref_out || !in || !ref_state || !ref_decay || !th_state || !th_decay) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_ref_decays)) return e;
    if (int e = check_params(M, neurons_per_batch, num_th_decays)) return e;
    if (int e = check_states(M, num_ref_states)) return e;
    if (int e = check_states(M, num_th_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    NAIVE_LAUNCH(ath_fwd_naive, M, stream, th_out, ref_out, in, ref_state, ref_decay, th_state, th_decay,
                 (long long)th_step_scaled, (long long)th0_scaled, (float)w_scale, M, neurons_per_batch,
                 num_ref_decays, num_th_decays, num_ref_states, num_th_states, (int)T);
    return (int)hipGetLastError();
}

extern "C" int slayer_res_fwd_naive(float* re_out, float* im_out, const float* re_in, const float* im_in,
                                    const float* sin_decay, const float* cos_decay,
                                    const float* re_state, const float* im_state,
                                    double thr_scaled, int w_scale, int64_t M, int64_t neurons_per_batch,
                                    int64_t num_decays, int64_t num_re_states, int64_t num_im_states,
                                    int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!re_out || !im_out || !re_in || !im_in || !sin_decay || !cos_decay || !re_state || !im_state)
        return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    if (int e = check_states(M, num_re_states)) return e;
    if (int e = check_states(M, num_im_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const int has_thr = thr_scaled >= 0;
    NAIVE_LAUNCH(res_fwd_naive, M, stream, re_out, im_out, re_in, im_in, sin_decay, cos_decay, re_state, im_state,
                 (float)thr_scaled, has_thr, has_thr ? (long long)(float)(thr_scaled - 1.0) : 0LL, (float)w_scale,
                 M, neurons_per_batch, num_decays, num_re_states, num_im_states, (int)T);
    return (int)hipGetLastError();
}

extern "C" int slayer_res_bwd_naive(float* g_re_in, float* g_im_in, const float* g_re, const float* g_im,
                                    const float* sin_decay, const float* cos_decay, int64_t M,
                                    int64_t neurons_per_batch, int64_t num_decays, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!g_re_in || !g_im_in || !g_re || !g_im || !sin_decay || !cos_decay) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    NAIVE_LAUNCH(res_bwd_naive, M, stream, g_re_in, g_im_in, g_re, g_im, sin_decay, cos_decay, M,
                 neurons_per_batch, num_decays, (int)T);
    return (int)hipGetLastError();
}
