// Spike functions: Heaviside / phase-threshold forward and relaxed-delta backward.
// Elementwise over the flat tensor, four samples per lane (dwordx4), grid-stride.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kEltBlock = 256;

inline unsigned elt_grid(int64_t work_items) {
    // enough workgroups to cover 256 CUs several times over; the loop strides the rest
    int64_t blocks = (work_items + kEltBlock - 1) / kEltBlock;
    const int64_t cap = 256 * 32;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

template <bool TENSOR_TH, bool GRADED>
__global__ __launch_bounds__(kEltBlock) void spike_fwd_kernel(float* __restrict__ s, const float* __restrict__ v,
                                                              const float* __restrict__ th, float scale, int64_t n,
                                                              int64_t nq) {
    const float th0 = TENSOR_TH ? 0.f : th[0];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    auto f = [&](float x, float t) -> float {
        const float h = (x >= t) ? 1.0f : 0.0f;
        return GRADED ? (h * x) / scale : h;
    };
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nq; i += stride) {
        const float4 x = reinterpret_cast<const float4*>(v)[i];
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = reinterpret_cast<const float4*>(th)[i];
        reinterpret_cast<float4*>(s)[i] = make_float4(f(x.x, t.x), f(x.y, t.y), f(x.z, t.z), f(x.w, t.w));
    }
    for (int64_t i = (nq << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        s[i] = f(v[i], TENSOR_TH ? th[i] : th0);
}

template <bool TENSOR_TH, bool GRADED>
__global__ __launch_bounds__(kEltBlock) void spike_bwd_kernel(float* __restrict__ gv, const float* __restrict__ gs,
                                                              const float* __restrict__ v, const float* __restrict__ th,
                                                              float tau, float rho, int64_t n, int64_t nq) {
    const float th0 = TENSOR_TH ? 0.f : th[0];
    const float lead = (rho / 2.0f) / tau;       // scale_rho / 2 / tau_rho, left to right
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    auto f = [&](float x, float t, float g) -> float {
        const float d = x - t;
        if (GRADED) return (rho * expf(fminf(d, 0.0f) / tau)) * g;
        return (lead * expf(-fabsf(d) / tau)) * g;
    };
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nq; i += stride) {
        const float4 x = reinterpret_cast<const float4*>(v)[i];
        const float4 g = reinterpret_cast<const float4*>(gs)[i];
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = reinterpret_cast<const float4*>(th)[i];
        reinterpret_cast<float4*>(gv)[i] =
            make_float4(f(x.x, t.x, g.x), f(x.y, t.y, g.y), f(x.z, t.z, g.z), f(x.w, t.w, g.w));
    }
    for (int64_t i = (nq << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        gv[i] = f(v[i], TENSOR_TH ? th[i] : th0, gs[i]);
}

// One lane per sample; the previous imaginary sample comes from the neighbouring
// address (same cache line except at 128-byte boundaries) or from imag_last at t == 0.
template <bool TENSOR_TH, bool GRADED>
__global__ __launch_bounds__(kEltBlock) void cspike_fwd_kernel(float* __restrict__ s, const float* __restrict__ re,
                                                               const float* __restrict__ im,
                                                               const float* __restrict__ th,
                                                               const float* __restrict__ last, int64_t num_last,
                                                               float scale, int64_t M, int T) {
    const float th0 = TENSOR_TH ? 0.f : th[0];
    const int64_t n = M * (int64_t)T;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t m = i / T;
        const int t = (int)(i - m * T);
        const float cur = im[i];
        const float prev = (t == 0) ? last[num_last == 1 ? 0 : m] : im[i - 1];
        const float r = re[i];
        const float thr = TENSOR_TH ? th[i] : th0;
        const float a = (r >= thr) ? 1.0f : 0.0f, b = (prev < 0.0f) ? 1.0f : 0.0f, c = (cur >= 0.0f) ? 1.0f : 0.0f;
        s[i] = GRADED ? (((r * a) * b) * c) / scale : (a * b) * c;
    }
}

template <bool TENSOR_TH, bool GRADED>
__global__ __launch_bounds__(kEltBlock) void cspike_bwd_kernel(float* __restrict__ gre, float* __restrict__ gim,
                                                               const float* __restrict__ gs,
                                                               const float* __restrict__ re,
                                                               const float* __restrict__ im,
                                                               const float* __restrict__ th, float tau, float rho,
                                                               int64_t n, int64_t nq) {
    const float th0 = TENSOR_TH ? 0.f : th[0];
    const float half_over_tau = (1.0f / 2.0f) / tau;   // 1 / 2 / tau_rho
    const float two_tau = 2.0f * tau;
    const float neg_rho_over_tau = (-rho) / tau;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    auto sign = [](float x) -> float { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : (x == 0.0f ? 0.0f : x)); };
    auto f = [&](float r, float i, float t, float g, float& o_re, float& o_im) {
        float d_re;
        if (GRADED) d_re = expf(-fmaxf(t - r, 0.0f) / tau);
        else d_re = half_over_tau * expf(-fabsf(r - t) / tau);
        const float d_im = half_over_tau * expf(-fabsf(i) / tau);
        const float step_re = 0.5f * (1.0f + sign(r - t) * (1.0f - two_tau * d_re));
        o_re = g * ((rho * d_re) * d_im);
        o_im = g * (((neg_rho_over_tau * sign(i)) * d_im) * step_re);
    };
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nq; k += stride) {
        const float4 r = reinterpret_cast<const float4*>(re)[k];
        const float4 i = reinterpret_cast<const float4*>(im)[k];
        const float4 g = reinterpret_cast<const float4*>(gs)[k];
        float4 t = make_float4(th0, th0, th0, th0);
        if (TENSOR_TH) t = reinterpret_cast<const float4*>(th)[k];
        float4 a, b;
        f(r.x, i.x, t.x, g.x, a.x, b.x);
        f(r.y, i.y, t.y, g.y, a.y, b.y);
        f(r.z, i.z, t.z, g.z, a.z, b.z);
        f(r.w, i.w, t.w, g.w, a.w, b.w);
        reinterpret_cast<float4*>(gre)[k] = a;
        reinterpret_cast<float4*>(gim)[k] = b;
    }
    for (int64_t k = (nq << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += stride)
        f(re[k], im[k], TENSOR_TH ? th[k] : th0, gs[k], gre[k], gim[k]);
}

}  // namespace slayer

using namespace slayer;

#define SLAYER_DISPATCH2(kernel, b0, b1, grid, stream, ...)                                                   \
    do {                                                                                                      \
        if (b0) {                                                                                             \
            if (b1) hipLaunchKernelGGL((kernel<true, true>), dim3(grid), dim3(kEltBlock), 0, stream, __VA_ARGS__);  \
            else hipLaunchKernelGGL((kernel<true, false>), dim3(grid), dim3(kEltBlock), 0, stream, __VA_ARGS__);    \
        } else {                                                                                              \
            if (b1) hipLaunchKernelGGL((kernel<false, true>), dim3(grid), dim3(kEltBlock), 0, stream, __VA_ARGS__); \
            else hipLaunchKernelGGL((kernel<false, false>), dim3(grid), dim3(kEltBlock), 0, stream, __VA_ARGS__);   \
        }                                                                                                     \
    } while (0)

static int check_threshold(int64_t num_threshold, int64_t numel) {
    return (num_threshold == 1 || num_threshold == numel) ? 0 : SLAYER_EINVAL;
}

// The float4 paths need 16-byte aligned bases; everything torch allocates is, views may not be.
static bool all_aligned(std::initializer_list<const void*> ps) {
    for (const void* p : ps)
        if (p && !aligned16(p)) return false;
    return true;
}

extern "C" int slayer_spike_fwd(float* spikes, const float* voltage, const float* threshold,
                                int64_t num_threshold, int graded, float scale, int64_t numel, void* stream) {
    if (numel < 0) return SLAYER_EINVAL;
    if (numel == 0) return 0;
    if (numel > kMaxNumel) return SLAYER_ERANGE;
    if (!spikes || !voltage || !threshold) return SLAYER_ENULL;
    if (int e = check_threshold(num_threshold, numel)) return e;
    const bool tt = num_threshold != 1;
    const int64_t nq = all_aligned({spikes, voltage, tt ? threshold : nullptr}) ? numel / 4 : 0;
    hipStream_t st = (hipStream_t)stream;
    SLAYER_DISPATCH2(spike_fwd_kernel, tt, graded != 0, elt_grid(nq ? nq + 3 : numel), st,
                     spikes, voltage, threshold, scale, numel, nq);
    return (int)hipGetLastError();
}

extern "C" int slayer_spike_bwd(float* grad_voltage, const float* grad_spikes, const float* voltage,
                                const float* threshold, int64_t num_threshold,
                                float tau_rho, float scale_rho, int graded, int64_t numel, void* stream) {
    if (numel < 0) return SLAYER_EINVAL;
    if (numel == 0) return 0;
    if (numel > kMaxNumel) return SLAYER_ERANGE;
    if (!grad_voltage || !grad_spikes || !voltage || !threshold) return SLAYER_ENULL;
    if (int e = check_threshold(num_threshold, numel)) return e;
    const bool tt = num_threshold != 1;
    const int64_t nq = all_aligned({grad_voltage, grad_spikes, voltage, tt ? threshold : nullptr}) ? numel / 4 : 0;
    hipStream_t st = (hipStream_t)stream;
    SLAYER_DISPATCH2(spike_bwd_kernel, tt, graded != 0, elt_grid(nq ? nq + 3 : numel), st,
                     grad_voltage, grad_spikes, voltage, threshold, tau_rho, scale_rho, numel, nq);
    return (int)hipGetLastError();
}

extern "C" int slayer_cspike_fwd(float* spikes, const float* re, const float* im, const float* threshold,
                                 int64_t num_threshold, const float* imag_last, int64_t num_last,
                                 int graded, float scale, int64_t M, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!spikes || !re || !im || !threshold || !imag_last) return SLAYER_ENULL;
    if (int e = check_threshold(num_threshold, M * T)) return e;
    if (int e = check_states(M, num_last)) return e;
    hipStream_t st = (hipStream_t)stream;
    SLAYER_DISPATCH2(cspike_fwd_kernel, num_threshold != 1, graded != 0, elt_grid(M * T), st,
                     spikes, re, im, threshold, imag_last, num_last, scale, M, (int)T);
    return (int)hipGetLastError();
}

extern "C" int slayer_cspike_bwd(float* grad_re, float* grad_im, const float* grad_spikes,
                                 const float* re, const float* im, const float* threshold,
                                 int64_t num_threshold, float tau_rho, float scale_rho, int graded,
                                 int64_t numel, void* stream) {
    if (numel < 0) return SLAYER_EINVAL;
    if (numel == 0) return 0;
    if (numel > kMaxNumel) return SLAYER_ERANGE;
    if (!grad_re || !grad_im || !grad_spikes || !re || !im || !threshold) return SLAYER_ENULL;
    if (int e = check_threshold(num_threshold, numel)) return e;
    const bool tt = num_threshold != 1;
    const int64_t nq = all_aligned({grad_re, grad_im, grad_spikes, re, im, tt ? threshold : nullptr}) ? numel / 4 : 0;
    hipStream_t st = (hipStream_t)stream;
    SLAYER_DISPATCH2(cspike_bwd_kernel, tt, graded != 0, elt_grid(nq ? nq + 3 : numel), st,
                     grad_re, grad_im, grad_spikes, re, im, threshold, tau_rho, scale_rho, numel, nq);
    return (int)hipGetLastError();
}
