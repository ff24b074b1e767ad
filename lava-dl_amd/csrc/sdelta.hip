// Sigma-delta pair: delta encoder (difference + threshold, float state per neuron) forward and
// backward, and the running sum of the sigma decoder in both time directions.  Same neuron x
// time-chunk staging as the integer dynamics; the arithmetic is float32 in the reference's order.
#include "common.h"
#include "tile.h"

namespace slayer {

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);   // li.hip
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip

template <bool CUM, bool QUANT>
struct DeltaFwd {
    static constexpr int kIn = 1, kOut = 2;          // out: (quantised) events, delta before thresholding
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = 65536;
    struct Params {
        const float* in[1];
        float* out[2];
        const float *threshold, *pre_state, *residual_state, *error_state;
        float *residual_out, *error_out;             // final states, one per neuron
        float step;                                  // quantisation step of the events (QUANT)
        int64_t npb, n_thr, n_pre, n_res, n_err;
    };
    float pre, residual, error, thr, q;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        pre = residual = error = 0.f; thr = 1.f; q = p.step;
        if (valid) {
            pre = p.pre_state[p.n_pre == 1 ? 0 : m];
            residual = p.residual_state[p.n_res == 1 ? 0 : m];
            error = p.error_state[p.n_err == 1 ? 0 : m];
            thr = p.threshold[param_index(m, p.npb, p.n_thr)];
        }
    }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[2]) {
        const float delta = (x[0] - pre) + residual;
        float y;
        if (CUM) {
            error = error + delta;
            y = (fabsf(error) >= thr) ? delta : 0.0f * delta;
            error = error * ((fabsf(y) > 0.0f) ? 0.0f : 1.0f);
        } else {
            y = (fabsf(delta) >= thr) ? delta : 0.0f * delta;
        }
        residual = delta - y;
        pre = x[0];
        o[0] = QUANT ? floorf(y / q) * q : y;
        o[1] = delta;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid) { p.residual_out[m] = residual; p.error_out[m] = error; }
    }
};

struct DeltaBwd {
    static constexpr int kIn = 2, kOut = 1;          // in: grad of the events, saved delta;  out: grad_input
    static constexpr bool kReverse = true;
    static constexpr int kDuoRows = 32;          // light float recurrence: shorter rows per wave, longer segments
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = kAlways;
    struct Params {
        const float* in[2];
        float* out[1];
        const float* threshold;
        float* partial;                              // per-neuron threshold gradient, or nullptr
        float tau, scale;
        int64_t npb, n_thr;
    };
    float g_next, acc, thr, tau, scale;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        g_next = acc = 0.f; thr = 1.f; tau = p.tau; scale = p.scale;
        if (valid) thr = p.threshold[param_index(m, p.npb, p.n_thr)];
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[1]) {
        const float g = x[0], d = x[1];
        o[0] = g - g_next;                           // grad[t] - grad[t+1]; the last step sees 0
        g_next = g;
        const float sub = fabsf(d) - thr;
        const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : d);
        const float gth = (sub > 0.f) ? ((-d) * (scale * expf(-fabsf(sub) / tau))) / thr : -sgn;
        acc += gth * g;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.partial) p.partial[m] = acc;
    }
};

// The backward pass of the delta unit is not a recurrence: grad_input[t] = g[t] - g[t+1] (0 past the last step)
// and the threshold gradient is a sum over time of an elementwise expression.  With T % 4 == 0 and 16-byte aligned
// tensors it runs as a row walk: one wave per row, 64 quads per pass, g[t+1] of a quad's last step from the
// neighbouring address; the expression (an exp and two divisions per sample) is then evaluated by all 64 lanes
// instead of sitting in a sequential loop of 16 or 32 lanes ([4,16,8192,300]: 947 -> 394 us).  The per-row sums go
// through the same deterministic reduction as before (their order of summation within a row changes).
// L lanes walk a row (a power of two up to 64: short rows share a wave, 64 / L of them).
template <int L>
__global__ __launch_bounds__(256) void delta_bwd_rows_kernel(float* __restrict__ grad_in, float* __restrict__ partial,
                                                             const float* __restrict__ grad_out,
                                                             const float* __restrict__ delta,
                                                             const float* __restrict__ threshold, float tau,
                                                             float scale, int64_t M, int64_t npb, int64_t n_thr, int T) {
    constexpr int kRowsPerWave = kWave / L;
    const int sub_row = threadIdx.x / L, lane = threadIdx.x % L;
    const int64_t m = ((int64_t)blockIdx.x * 4 + threadIdx.y) * kRowsPerWave + sub_row;
    const bool live = m < M;
    const int64_t mm = live ? m : 0;
    const float thr = threshold[param_index(mm, npb, n_thr)];
    const float* g = grad_out + (size_t)mm * (size_t)T;
    const float* d = delta + (size_t)mm * (size_t)T;
    float* dst = grad_in + (size_t)mm * (size_t)T;
    float acc = 0.f;
    auto term = [&](float gg, float dd) {
        const float sub = fabsf(dd) - thr;
        const float sgn = dd > 0.f ? 1.f : (dd < 0.f ? -1.f : dd);
        const float gth = (sub > 0.f) ? ((-dd) * (scale * expf(-fabsf(sub) / tau))) / thr : -sgn;
        return gth * gg;
    };
    if (live) {
        for (int t = 4 * lane; t < T; t += 4 * L) {
            const float4 gv = *reinterpret_cast<const float4*>(g + t);
            const float4 dv = *reinterpret_cast<const float4*>(d + t);
            const float next = t + 4 < T ? g[t + 4] : 0.f;
            *reinterpret_cast<float4*>(dst + t) = make_float4(gv.x - gv.y, gv.y - gv.z, gv.z - gv.w, gv.w - next);
            if (partial) {
                acc += term(gv.w, dv.w);
                acc += term(gv.z, dv.z);
                acc += term(gv.y, dv.y);
                acc += term(gv.x, dv.x);
            }
        }
    }
    if (partial) {
#pragma unroll
        for (int k = L / 2; k >= 1; k >>= 1) acc += __shfl_xor(acc, k);
        if (live && lane == 0) partial[m] = acc;
    }
}

template <bool REVERSE>
struct RunningSum {
    static constexpr int kIn = 1, kOut = 1;
    static constexpr bool kReverse = REVERSE;
    static constexpr int kDuoRows = 32;          // light float recurrence: shorter rows per wave, longer segments
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = kAlways;
    struct Params {
        const float* in[1];
        float* out[1];
        const float* state;                          // initial value per neuron, or nullptr for 0
        int64_t n_state;
    };
    float y;
    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        y = (valid && p.state) ? p.state[p.n_state == 1 ? 0 : m] : 0.f;
    }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[1]) { y = y + x[0]; o[0] = y; }
    __device__ __forceinline__ void finish(const Params&, int64_t, bool) {}
};

template <bool CUM, bool QUANT>
static int delta_fwd_launch(const typename DeltaFwd<CUM, QUANT>::Params& p, int64_t M, int64_t T, hipStream_t st) {
    return launch_stream<DeltaFwd<CUM, QUANT>>(p, M, T, st);
}

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_delta_fwd(float* out, float* delta_out, float* residual_out, float* error_out,
                                const float* in, const float* threshold, const float* pre_state,
                                const float* residual_state, const float* error_state,
                                int cum_error, float quant_step,
                                int64_t M, int64_t neurons_per_batch, int64_t num_thresholds,
                                int64_t num_pre, int64_t num_residual, int64_t num_error,
                                int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0) return 0;
    if (!residual_out || !error_out || !threshold || !pre_state || !residual_state || !error_state) return SLAYER_ENULL;
    if (T > 0 && (!out || !delta_out || !in)) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_thresholds)) return e;
    for (int64_t n : {num_pre, num_residual, num_error})
        if (int e = check_states(M, n)) return e;
    if (T == 0) return SLAYER_EINVAL;                // the final states would not be defined by a launch
    hipStream_t st = (hipStream_t)stream;
    const bool quant = quant_step > 0.0f;
#define SLAYER_DELTA(C, Q)                                                                                      \
    do {                                                                                                        \
        DeltaFwd<C, Q>::Params p{{in}, {out, delta_out}, threshold, pre_state, residual_state, error_state,       \
                                 residual_out, error_out, quant_step, neurons_per_batch, num_thresholds,         \
                                 num_pre, num_residual, num_error};                                              \
        return delta_fwd_launch<C, Q>(p, M, T, st);                                                              \
    } while (0)
    if (cum_error) { if (quant) SLAYER_DELTA(true, true); else SLAYER_DELTA(true, false); }
    if (quant) SLAYER_DELTA(false, true);
    SLAYER_DELTA(false, false);
#undef SLAYER_DELTA
}

extern "C" int slayer_delta_bwd(float* grad_in, float* grad_threshold, const float* grad_out,
                                const float* delta, const float* threshold, float* workspace,
                                float tau_grad, float scale_grad,
                                int64_t M, int64_t neurons_per_batch, int64_t num_thresholds,
                                int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_params(M > 0 ? M : neurons_per_batch, neurons_per_batch, num_thresholds)) return e;
    if (grad_threshold && !workspace && M > 0) return SLAYER_ENULL;
    hipStream_t st = (hipStream_t)stream;
    if (M > 0 && T > 0) {
        if (!grad_in || !grad_out || !delta || !threshold) return SLAYER_ENULL;
        if (T % 4 == 0 && aligned16(grad_in) && aligned16(grad_out) && aligned16(delta) && M / 4 < 0x7fffffffLL) {
            const int64_t quads = T / 4;
#define SLAYER_DELTA_ROWS(L)                                                                                      \
    hipLaunchKernelGGL(delta_bwd_rows_kernel<L>, dim3((unsigned)((M + 4 * (64 / L) - 1) / (4 * (64 / L)))),       \
                       dim3(64, 4), 0, st, grad_in, grad_threshold ? workspace : nullptr, grad_out, delta,        \
                       threshold, tau_grad, scale_grad, M, neurons_per_batch, num_thresholds, (int)T)
            if (quads > 32) SLAYER_DELTA_ROWS(64);
            else if (quads > 16) SLAYER_DELTA_ROWS(32);
            else if (quads > 8) SLAYER_DELTA_ROWS(16);
            else if (quads > 4) SLAYER_DELTA_ROWS(8);
            else SLAYER_DELTA_ROWS(4);
#undef SLAYER_DELTA_ROWS
            if (int e = (int)hipGetLastError()) return e;
        } else {
            DeltaBwd::Params p{{grad_out, delta}, {grad_in}, threshold, grad_threshold ? workspace : nullptr,
                               tau_grad, scale_grad, neurons_per_batch, num_thresholds};
            if (int e = launch_stream<DeltaBwd>(p, M, T, st)) return e;
        }
    }
    if (grad_threshold) {
        if (M == 0 || T == 0) return launch_zero_fill(grad_threshold, num_thresholds, st);
        return launch_reduce_param_grad(grad_threshold, workspace, workspace + M, M, neurons_per_batch,
                                        num_thresholds, st);
    }
    return 0;
}

extern "C" int slayer_cumsum(float* out, const float* in, const float* state, int64_t num_states,
                             int reverse, int64_t M, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in) return SLAYER_ENULL;
    if (state)
        if (int e = check_states(M, num_states)) return e;
    hipStream_t st = (hipStream_t)stream;
    if (reverse) {
        RunningSum<true>::Params p{{in}, {out}, state, num_states};
        return launch_stream<RunningSum<true>>(p, M, T, st);
    }
    RunningSum<false>::Params p{{in}, {out}, state, num_states};
    return launch_stream<RunningSum<false>>(p, M, T, st);
}
