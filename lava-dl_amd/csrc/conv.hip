// Causal temporal convolution and its adjoint (anti-causal correlation).
//   conv: out[m][t] = Ts * sum_{i<K, t-i>=0} f[i] * in[m][t-i]
//   corr: out[m][t] = Ts * sum_{i<K, t+i<T } f[i] * in[m][t+i]
// One wavefront produces kSeg consecutive outputs of one row.  The input window
// (segment + K-1 halo) is staged in LDS once, so each input sample is fetched from
// HBM once per segment instead of K times; taps accumulate in ascending order.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kOutPerLane = 8;
constexpr int kSeg = kWave * kOutPerLane;      // outputs per workgroup
constexpr int kMaxTaps = 4096;

template <bool CORR>
__global__ __launch_bounds__(kWave) void conv_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                     const float* __restrict__ filt, int K, float ts,
                                                     int64_t M, int T, unsigned segs_per_row) {
    extern __shared__ float win[];             // kSeg + K - 1 input samples, then K taps
    float* taps = win + kSeg + K - 1;
    const int lane = threadIdx.x;
    const unsigned m = blockIdx.x / segs_per_row;
    const int t0 = (int)(blockIdx.x - m * segs_per_row) * kSeg;
    const float* row = in + (size_t)m * (size_t)T;
    const int wstart = CORR ? t0 : t0 - (K - 1);
    const int wlen = kSeg + K - 1;
    for (int p = lane; p < wlen; p += kWave) {
        const int t = wstart + p;
        win[p] = (t >= 0 && t < T) ? row[t] : 0.0f;
    }
    for (int i = lane; i < K; i += kWave) taps[i] = filt[i];
    __syncthreads();

    float acc[kOutPerLane];
#pragma unroll
    for (int r = 0; r < kOutPerLane; ++r) acc[r] = 0.0f;
    // output o = lane + 64*r;  conv reads win[(K-1) + o - i], corr reads win[o + i]
    const float* base = win + lane + (CORR ? 0 : K - 1);
    for (int i = 0; i < K; ++i) {
        const float f = taps[i];
        const float* x = CORR ? base + i : base - i;
#pragma unroll
        for (int r = 0; r < kOutPerLane; ++r) acc[r] = __fmaf_rn(f, x[kWave * r], acc[r]);
    }
    float* dst = out + (size_t)m * (size_t)T;
#pragma unroll
    for (int r = 0; r < kOutPerLane; ++r) {
        const int t = t0 + lane + kWave * r;
        if (t < T) dst[t] = acc[r] * ts;
    }
}

template <bool CORR>
static int conv_launch(float* out, const float* in, const float* filt, int64_t K, float ts,
                       int64_t M, int64_t T, hipStream_t stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in || !filt) return SLAYER_ENULL;
    if (K < 1) return SLAYER_EINVAL;
    if (K > kMaxTaps) return SLAYER_ERANGE;
    const unsigned segs = (unsigned)((T + kSeg - 1) / kSeg);
    const int64_t blocks = M * (int64_t)segs;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const size_t lds = sizeof(float) * (size_t)(kSeg + 2 * K - 1);
    hipLaunchKernelGGL((conv_kernel<CORR>), dim3((unsigned)blocks), dim3(kWave), lds, stream,
                       out, in, filt, (int)K, ts, M, (int)T, segs);
    return (int)hipGetLastError();
}

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_conv(float* out, const float* in, const float* filt, int64_t K, float sampling_time,
                           int64_t M, int64_t T, void* stream) {
    return conv_launch<false>(out, in, filt, K, sampling_time, M, T, (hipStream_t)stream);
}

extern "C" int slayer_corr(float* out, const float* in, const float* filt, int64_t K, float sampling_time,
                           int64_t M, int64_t T, void* stream) {
    return conv_launch<true>(out, in, filt, K, sampling_time, M, T, (hipStream_t)stream);
}
