// Spike functions: Heaviside / phase-threshold forward and relaxed-delta backward.
// Elementwise: one lane handles four consecutive samples (one dwordx4 per tensor), one
// workgroup per 1024 samples, no grid-stride loop (measured fastest for pure streaming on
// MI355X); tensors larger than the last-level cache use non-temporal accesses.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kEltBlock = 256;
constexpr int64_t kStreamingBytes = (int64_t)64 << 20;

// Work item g < nq handles samples [4g, 4g+4); items nq .. nq+tail-1 handle the n % 4 leftovers
// (or every sample one by one when the bases are not 16-byte aligned: nq == 0).
struct EltSplit {
    int64_t nq, items;
    unsigned grid;
};
inline EltSplit elt_split(int64_t n, bool aligned) {
    EltSplit s;
    s.nq = aligned ? n / 4 : 0;
    s.items = s.nq + (n - 4 * s.nq);
    s.grid = (unsigned)((s.items + kEltBlock - 1) / kEltBlock);
    return s;
}

template <bool TENSOR_TH, bool GRADED, bool STREAM>
__global__ __launch_bounds__(kEltBlock) void spike_fwd_kernel(float* __restrict__ s, const float* __restrict__ v,
                                                              const float* __restrict__ th, float th0, float scale,
                                                              int64_t n, int64_t nq) {
    if (!TENSOR_TH && th) th0 = th[0];
    auto f = [&](float x, float t) -> float {
        const float h = (x >= t) ? 1.0f : 0.0f;
        return GRADED ? (h * x) / scale : h;
    };
    const int64_t g = (int64_t)blockIdx.x * kEltBlock + threadIdx.x;
    if (g < nq) {
        const float4 x = load4(v + 4 * g, STREAM);
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = load4(th + 4 * g, STREAM);
        store4(s + 4 * g, make_float4(f(x.x, t.x), f(x.y, t.y), f(x.z, t.z), f(x.w, t.w)), STREAM);
    } else {
        const int64_t i = 4 * nq + (g - nq);
        if (i < n) s[i] = f(v[i], TENSOR_TH ? th[i] : th0);
    }
}

template <bool TENSOR_TH, bool GRADED, bool STREAM>
__global__ __launch_bounds__(kEltBlock) void spike_bwd_kernel(float* __restrict__ gv, const float* __restrict__ gs,
                                                              const float* __restrict__ v, const float* __restrict__ th,
                                                              float th0, float tau, float rho, int64_t n, int64_t nq) {
    if (!TENSOR_TH && th) th0 = th[0];
    const float lead = (rho / 2.0f) / tau;       // scale_rho / 2 / tau_rho, left to right
    // The exponent is (v - threshold) * (1 / tau) where the reference divides by tau: at most an ulp and a half
    // apart in the exponent (identical for tau = 1), far inside the 1e-5 bar of the float gradients, and it takes
    // the ten instructions of a correctly rounded division out of every sample -- which is what held the fused
    // backward scans below their memory rate.  Every kernel that evaluates a surrogate does the same, so fused
    // and unfused paths stay bit-identical to each other.
    const float inv_tau = 1.0f / tau;
    auto f = [&](float x, float t, float g) -> float {
        const float d = x - t;
        if (GRADED) return (rho * expf(fminf(d, 0.0f) * inv_tau)) * g;
        return (lead * expf(-fabsf(d) * inv_tau)) * g;
    };
    const int64_t k = (int64_t)blockIdx.x * kEltBlock + threadIdx.x;
    if (k < nq) {
        const float4 x = load4(v + 4 * k, STREAM);
        const float4 g = load4(gs + 4 * k, STREAM);
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = load4(th + 4 * k, STREAM);
        store4(gv + 4 * k, make_float4(f(x.x, t.x, g.x), f(x.y, t.y, g.y), f(x.z, t.z, g.z), f(x.w, t.w, g.w)),
               STREAM);
    } else {
        const int64_t i = 4 * nq + (k - nq);
        if (i < n) gv[i] = f(v[i], TENSOR_TH ? th[i] : th0, gs[i]);
    }
}

// One lane per four consecutive samples of a row (T % 4 == 0 path) or per sample; the previous
// imaginary sample of a quad's first element is the neighbouring address (or imag_last at t == 0).
template <bool TENSOR_TH, bool GRADED, bool VEC4>
__global__ __launch_bounds__(kEltBlock) void cspike_fwd_kernel(float* __restrict__ s, const float* __restrict__ re,
                                                               const float* __restrict__ im,
                                                               const float* __restrict__ th, float th0,
                                                               const float* __restrict__ last, int64_t num_last,
                                                               float last0, float scale, int64_t M, int T,
                                                               int64_t items) {
    if (!TENSOR_TH && th) th0 = th[0];
    auto f = [&](float r, float thr, float prev, float cur) -> float {
        const float a = (r >= thr) ? 1.0f : 0.0f, b = (prev < 0.0f) ? 1.0f : 0.0f, c = (cur >= 0.0f) ? 1.0f : 0.0f;
        return GRADED ? (((r * a) * b) * c) / scale : (a * b) * c;
    };
    const int64_t g = (int64_t)blockIdx.x * kEltBlock + threadIdx.x;
    if (g >= items) return;
    if (VEC4) {
        const int64_t i = 4 * g;
        const int64_t m = i / T;
        const int t = (int)(i - m * T);
        const float4 c = load4(im + i, true), r = load4(re + i, true);
        const float p0 = (t == 0) ? (last ? last[num_last == 1 ? 0 : m] : last0) : im[i - 1];
        float4 h = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) h = load4(th + i, true);
        store4(s + i, make_float4(f(r.x, h.x, p0, c.x), f(r.y, h.y, c.x, c.y), f(r.z, h.z, c.y, c.z),
                                  f(r.w, h.w, c.z, c.w)), true);
    } else {
        const int64_t m = g / T;
        const int t = (int)(g - m * T);
        const float prev = (t == 0) ? (last ? last[num_last == 1 ? 0 : m] : last0) : im[g - 1];
        s[g] = f(re[g], TENSOR_TH ? th[g] : th0, prev, im[g]);
    }
}

template <bool TENSOR_TH, bool GRADED, bool STREAM>
__global__ __launch_bounds__(kEltBlock) void cspike_bwd_kernel(float* __restrict__ gre, float* __restrict__ gim,
                                                               const float* __restrict__ gs,
                                                               const float* __restrict__ re,
                                                               const float* __restrict__ im,
                                                               const float* __restrict__ th, float th0, float tau,
                                                               float rho, int64_t n, int64_t nq) {
    if (!TENSOR_TH && th) th0 = th[0];
    const float half_over_tau = (1.0f / 2.0f) / tau;   // 1 / 2 / tau_rho
    const float inv_tau = 1.0f / tau;
    const float two_tau = 2.0f * tau;
    const float neg_rho_over_tau = (-rho) / tau;
    auto sign = [](float x) -> float { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : (x == 0.0f ? 0.0f : x)); };
    auto f = [&](float r, float i, float t, float g, float& o_re, float& o_im) {
        float d_re;
        if (GRADED) d_re = expf(-fmaxf(t - r, 0.0f) * inv_tau);
        else d_re = half_over_tau * expf(-fabsf(r - t) * inv_tau);
        const float d_im = half_over_tau * expf(-fabsf(i) * inv_tau);
        const float step_re = 0.5f * (1.0f + sign(r - t) * (1.0f - two_tau * d_re));
        o_re = g * ((rho * d_re) * d_im);
        o_im = g * (((neg_rho_over_tau * sign(i)) * d_im) * step_re);
    };
    const int64_t k = (int64_t)blockIdx.x * kEltBlock + threadIdx.x;
    if (k < nq) {
        const float4 r = load4(re + 4 * k, STREAM), i = load4(im + 4 * k, STREAM), g = load4(gs + 4 * k, STREAM);
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = load4(th + 4 * k, STREAM);
        float4 a, b;
        f(r.x, i.x, t.x, g.x, a.x, b.x);
        f(r.y, i.y, t.y, g.y, a.y, b.y);
        f(r.z, i.z, t.z, g.z, a.z, b.z);
        f(r.w, i.w, t.w, g.w, a.w, b.w);
        store4(gre + 4 * k, a, STREAM);
        store4(gim + 4 * k, b, STREAM);
    } else {
        const int64_t j = 4 * nq + (k - nq);
        if (j < n) f(re[j], im[j], TENSOR_TH ? th[j] : th0, gs[j], gre[j], gim[j]);
    }
}

}  // namespace slayer

using namespace slayer;

#define SLAYER_LAUNCH3(kernel, b0, b1, b2, grid, stream, ...)                                              \
    do {                                                                                                   \
        const int sel = ((b0) ? 4 : 0) | ((b1) ? 2 : 0) | ((b2) ? 1 : 0);                                  \
        const dim3 g_(grid), t_(kEltBlock);                                                                \
        switch (sel) {                                                                                     \
            case 0: hipLaunchKernelGGL((kernel<false, false, false>), g_, t_, 0, stream, __VA_ARGS__); break; \
            case 1: hipLaunchKernelGGL((kernel<false, false, true>), g_, t_, 0, stream, __VA_ARGS__); break;  \
            case 2: hipLaunchKernelGGL((kernel<false, true, false>), g_, t_, 0, stream, __VA_ARGS__); break;  \
            case 3: hipLaunchKernelGGL((kernel<false, true, true>), g_, t_, 0, stream, __VA_ARGS__); break;   \
            case 4: hipLaunchKernelGGL((kernel<true, false, false>), g_, t_, 0, stream, __VA_ARGS__); break;  \
            case 5: hipLaunchKernelGGL((kernel<true, false, true>), g_, t_, 0, stream, __VA_ARGS__); break;   \
            case 6: hipLaunchKernelGGL((kernel<true, true, false>), g_, t_, 0, stream, __VA_ARGS__); break;   \
            default: hipLaunchKernelGGL((kernel<true, true, true>), g_, t_, 0, stream, __VA_ARGS__); break;   \
        }                                                                                                  \
    } while (0)

static int check_threshold(const float* threshold, int64_t num_threshold, int64_t numel) {
    if (!threshold) return 0;
    return (num_threshold == 1 || num_threshold == numel) ? 0 : SLAYER_EINVAL;
}

// The dwordx4 paths need 16-byte aligned bases; everything torch allocates is, views may not be.
static bool all_aligned(std::initializer_list<const void*> ps) {
    for (const void* p : ps)
        if (p && !aligned16(p)) return false;
    return true;
}

static int check_numel(int64_t numel) {
    if (numel < 0) return SLAYER_EINVAL;
    if (numel > kMaxNumel) return SLAYER_ERANGE;
    return 0;
}

extern "C" int slayer_spike_fwd(float* spikes, const float* voltage, const float* threshold,
                                int64_t num_threshold, float threshold_value, int graded, float scale,
                                int64_t numel, void* stream) {
    if (int e = check_numel(numel)) return e;
    if (numel == 0) return 0;
    if (!spikes || !voltage) return SLAYER_ENULL;
    if (int e = check_threshold(threshold, num_threshold, numel)) return e;
    const bool tt = threshold && num_threshold != 1;
    const EltSplit sp = elt_split(numel, all_aligned({spikes, voltage, tt ? threshold : nullptr}));
    hipStream_t st = (hipStream_t)stream;
    SLAYER_LAUNCH3(spike_fwd_kernel, tt, graded != 0, numel * 4 > kStreamingBytes, sp.grid, st,
                   spikes, voltage, threshold, threshold_value, scale, numel, sp.nq);
    return (int)hipGetLastError();
}

extern "C" int slayer_spike_bwd(float* grad_voltage, const float* grad_spikes, const float* voltage,
                                const float* threshold, int64_t num_threshold, float threshold_value,
                                float tau_rho, float scale_rho, int graded, int64_t numel, void* stream) {
    if (int e = check_numel(numel)) return e;
    if (numel == 0) return 0;
    if (!grad_voltage || !grad_spikes || !voltage) return SLAYER_ENULL;
    if (int e = check_threshold(threshold, num_threshold, numel)) return e;
    const bool tt = threshold && num_threshold != 1;
    const EltSplit sp = elt_split(numel, all_aligned({grad_voltage, grad_spikes, voltage, tt ? threshold : nullptr}));
    hipStream_t st = (hipStream_t)stream;
    SLAYER_LAUNCH3(spike_bwd_kernel, tt, graded != 0, numel * 4 > kStreamingBytes, sp.grid, st,
                   grad_voltage, grad_spikes, voltage, threshold, threshold_value, tau_rho, scale_rho, numel, sp.nq);
    return (int)hipGetLastError();
}

extern "C" int slayer_cspike_fwd(float* spikes, const float* re, const float* im, const float* threshold,
                                 int64_t num_threshold, float threshold_value,
                                 const float* imag_last, int64_t num_last, float imag_last_value,
                                 int graded, float scale, int64_t M, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!spikes || !re || !im) return SLAYER_ENULL;
    if (int e = check_threshold(threshold, num_threshold, M * T)) return e;
    if (imag_last)
        if (int e = check_states(M, num_last)) return e;
    const bool tt = threshold && num_threshold != 1;
    const bool vec = (T % 4 == 0) && all_aligned({spikes, re, im, tt ? threshold : nullptr});
    const int64_t items = vec ? M * T / 4 : M * T;
    const unsigned grid = (unsigned)((items + kEltBlock - 1) / kEltBlock);
    hipStream_t st = (hipStream_t)stream;
    SLAYER_LAUNCH3(cspike_fwd_kernel, tt, graded != 0, vec, grid, st,
                   spikes, re, im, threshold, threshold_value, imag_last, num_last, imag_last_value, scale, M, (int)T,
                   items);
    return (int)hipGetLastError();
}

extern "C" int slayer_cspike_bwd(float* grad_re, float* grad_im, const float* grad_spikes,
                                 const float* re, const float* im, const float* threshold,
                                 int64_t num_threshold, float threshold_value, float tau_rho, float scale_rho,
                                 int graded, int64_t numel, void* stream) {
    if (int e = check_numel(numel)) return e;
    if (numel == 0) return 0;
    if (!grad_re || !grad_im || !grad_spikes || !re || !im) return SLAYER_ENULL;
    if (int e = check_threshold(threshold, num_threshold, numel)) return e;
    const bool tt = threshold && num_threshold != 1;
    const EltSplit sp = elt_split(numel, all_aligned({grad_re, grad_im, grad_spikes, re, im, tt ? threshold : nullptr}));
    hipStream_t st = (hipStream_t)stream;
    SLAYER_LAUNCH3(cspike_bwd_kernel, tt, graded != 0, numel * 4 > kStreamingBytes, sp.grid, st,
                   grad_re, grad_im, grad_spikes, re, im, threshold, threshold_value, tau_rho, scale_rho, numel, sp.nq);
    return (int)hipGetLastError();
}
