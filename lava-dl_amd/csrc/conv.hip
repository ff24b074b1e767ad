// Causal temporal convolution and its adjoint (anti-causal correlation).
//   conv: out[m][t] = Ts * sum_{i<K, t-i>=0} f[i] * in[m][t-i]
//   corr: out[m][t] = Ts * sum_{i<K, t+i<T } f[i] * in[m][t+i]
//
// One wavefront produces 512 consecutive outputs of one row.  The input window (segment plus a
// K-1 halo) is staged in LDS once, so each input sample is fetched from HBM once per segment
// instead of K times.  A lane owns 8 consecutive outputs and keeps the 8 inputs they need for
// the current tap in registers; moving to the next tap replaces exactly one of them, so the
// inner loop is one LDS read and 8 FMAs per tap (FMA-issue bound: with K = 64 the kernel does
// 128 flop per 8 bytes, beyond what HBM could feed).  The window is stored with one pad word
// per 8 samples, which makes the lane-stride-8 reads bank-conflict free.  Taps are read with
// wave-uniform addresses (scalar loads) and accumulate in ascending order.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kOutPerLane = 8;
constexpr int kSeg = kWave * kOutPerLane;      // outputs per workgroup
constexpr int kMaxTaps = 4096;

// LDS index of window position p (one pad word per 8 samples).  For p = 8*lane + d this is
// 9*lane + d + (d >> 3): the lane part is computed once, the rest is wave-uniform (scalar ALU).
__device__ __forceinline__ int padded(int p) { return p + (p >> 3); }
constexpr int kFront = 8;      // unused samples in front of the window keep every index non-negative

template <bool CORR, bool VEC4>
__global__ __launch_bounds__(kWave) void conv_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                     const float* __restrict__ filt, int K, float ts,
                                                     int64_t M, int T, unsigned segs_per_row) {
    extern __shared__ float win[];             // padded(kFront + kSeg + K - 1) input samples
    const int lane = threadIdx.x;
    const unsigned m = blockIdx.x / segs_per_row;
    const int t0 = (int)(blockIdx.x - m * segs_per_row) * kSeg;
    const float* row = in + (size_t)m * (size_t)T;
    // window position p holds input step wstart + p
    const int wstart = CORR ? t0 : t0 - (K - 1);
    const int wlen = kSeg + K - 1;
    for (int p = lane; p < wlen; p += kWave) {
        const int t = wstart + p;
        win[padded(p + kFront)] = (t >= 0 && t < T) ? row[t] : 0.0f;
    }
    __syncthreads();

    // output r of this lane is step t0 + 8*lane + r.  At tap i it needs window position
    //   conv: (K-1) + 8*lane + r - i        corr: 8*lane + r + i
    // kept in v[(r - i) & 7] (conv) or v[(r + i) & 7] (corr): stepping i replaces one slot.
    float acc[kOutPerLane], v[kOutPerLane];
    const float* mine = win + 9 * lane;                       // padded(8 * lane)
    const int base = kFront + (CORR ? 0 : K - 1);             // wave-uniform part of the position
#pragma unroll
    for (int r = 0; r < kOutPerLane; ++r) {
        acc[r] = 0.0f;
        v[r] = mine[padded(base + r)];
    }
    int i = 0;
    for (; i + 8 <= K; i += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float f = filt[i + u];
#pragma unroll
            for (int r = 0; r < kOutPerLane; ++r)
                acc[r] = __fmaf_rn(f, v[CORR ? ((r + u) & 7) : ((r - u) & 7)], acc[r]);
            // slot of the sample that drops out receives the one needed by the next tap
            if (CORR) v[u & 7] = mine[padded(base + 8 + i + u)];
            else v[(7 - u) & 7] = mine[padded(base - 1 - (i + u))];
        }
    }
    // remaining K % 8 taps: i is a multiple of 8 here, so slot indices restart at u = 0
    for (int u = 0; i + u < K; ++u) {
        const float f = filt[i + u];
#pragma unroll
        for (int r = 0; r < kOutPerLane; ++r) {
            const int s = CORR ? ((r + u) & 7) : ((r - u) & 7);
            float x = v[0];
#pragma unroll
            for (int j = 1; j < 8; ++j) x = (s == j) ? v[j] : x;
            acc[r] = __fmaf_rn(f, x, acc[r]);
        }
        const float nv = CORR ? mine[padded(base + 8 + i + u)] : mine[padded(base - 1 - (i + u))];
        const int slot = CORR ? (u & 7) : ((7 - u) & 7);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (slot == j) ? nv : v[j];
    }

    const int t = t0 + 8 * lane;
    float* dst = out + (size_t)m * (size_t)T + t;
    if (VEC4 && t + 8 <= T) {
        *reinterpret_cast<float4*>(dst) = make_float4(acc[0] * ts, acc[1] * ts, acc[2] * ts, acc[3] * ts);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(acc[4] * ts, acc[5] * ts, acc[6] * ts, acc[7] * ts);
    } else {
#pragma unroll
        for (int r = 0; r < kOutPerLane; ++r)
            if (t + r < T) dst[r] = acc[r] * ts;
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
    const int wlen = kFront + kSeg + (int)K;                   // one spare sample behind the window
    const size_t lds = sizeof(float) * (size_t)(wlen + (wlen >> 3) + 1);
    const bool vec = (T % 4 == 0) && aligned16(out);
    if (vec)
        hipLaunchKernelGGL((conv_kernel<CORR, true>), dim3((unsigned)blocks), dim3(kWave), lds, stream,
                           out, in, filt, (int)K, ts, M, (int)T, segs);
    else
        hipLaunchKernelGGL((conv_kernel<CORR, false>), dim3((unsigned)blocks), dim3(kWave), lds, stream,
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
