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

// ---------------------------------------------------------------------------------------------
// Matrix-core form for 8 < K <= 128 (T % 4 == 0, 16-byte aligned tensors).  A tile of 16 output steps of 16
// rows is a [16 x (16 + KPAD)] Toeplitz matrix of taps times the [(16 + KPAD) x 16] window of inputs:
// v_mfma_f32_16x16x4_f32 with D[i][j] = output step i of row j, four input samples per instruction.  With
// K = 64 the window is 80 samples, so 64 of 80 multiply-adds are useful (the FMA form above issues 82
// instructions per 64 useful FMAs at half the rate).  Lane l works for row l % 16 and quad l / 16: it loads
// the 4 samples [16 g + 4 (l / 16), +4) of window group g straight from memory (a float4), which are exactly
// the B operands of the group's four instructions (sample 4 k + r of a group goes to summation slot k of
// instruction r), keeps the Toeplitz operands of all groups in registers (they do not depend on the tile),
// and receives 4 consecutive output steps of its row (a float4 store).  Stepping to the next tile moves
// every window group down by one, so a tile costs one new load per lane; no LDS, no barrier.
// Window samples outside a filter's support meet a zero tap instead of being skipped, so an Inf or NaN in the
// input also reaches the up to 16 + KPAD - K neighbouring outputs whose window holds it (0 * Inf); finite
// inputs, the only ones this path sees, give the same sums.
typedef float mfma_f4 __attribute__((ext_vector_type(4)));

template <int KPAD, bool CORR>
__global__ __launch_bounds__(kWave) void conv_mfma_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                          const float* __restrict__ filt, int K, float ts,
                                                          int64_t M, int T, int span, unsigned spans_per_row) {
    constexpr int G = KPAD / 16 + 1;        // window groups of 16 samples per tile
    constexpr int RING = KPAD <= 64 ? 8 : 16;
    const int lane = threadIdx.x;
    const int j = lane & 15, kq = lane >> 4;
    const int64_t rowgroup = blockIdx.x / spans_per_row;
    const int tbeg = (int)(blockIdx.x - rowgroup * spans_per_row) * span;
    const int tend = tbeg + span < T ? tbeg + span : T;
    const int64_t m0 = rowgroup * 16;
    const int rows = (int)((M - m0) < 16 ? (M - m0) : 16);
    // raw buffer accesses over the wave's rows: a lane that must not touch memory (row beyond the tensor,
    // step outside [0, T)) gets an out-of-range offset, reads zeros and has its store dropped; no branch
    // surrounds a memory instruction, so the loads issued ahead stay in flight across the loop's waits
    const unsigned wave_bytes = (unsigned)rows * (unsigned)T * 4u;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(in + m0 * (int64_t)T, wave_bytes);
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(out + m0 * (int64_t)T, wave_bytes);
    const bool row_ok = j < rows;
    const int row_off = j * T * 4;

    // Toeplitz operands: lane (output step i = l % 16, slot kq) of instruction (g, r) holds the tap that
    // links output step i with window sample 16 g + 4 kq + r
    float a[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = CORR ? (16 * g + 4 * kq + r) - j : j + KPAD - (16 * g + 4 * kq + r);
            a[g][r] = (idx >= 0 && idx < K) ? filt[idx] : 0.0f;
        }

    // window group g of the tile at t0 starts at step t0 - KPAD + 16 g (conv) or t0 + 16 g (corr)
    auto load = [&](int step) -> float4 {
        const bool ok = row_ok && (unsigned)step < (unsigned)T;
        return buf_load4<false>(src, ok ? row_off + step * 4 : kOutOfRange);
    };
    // Window groups live in a ring of RING registers (absolute group q of the span, starting at step
    // first + 16 q, sits in slot q % RING): tile n reads groups n .. n + G - 1 and then refills the slot of
    // group n, which no later tile needs, with group n + RING -- P = RING - G tiles before its first use.
    // The loop body is RING tiles, so every slot index is a compile-time constant.
    const int first = (CORR ? tbeg : tbeg - KPAD) + 4 * kq;
    float4 x[RING];
    // each load is preceded by a store that falls out of range (dropped by the hardware): the loop is then
    // entered in the state its back edge leaves, and the wait at its top can leave the youngest loads in
    // flight instead of draining everything
#pragma unroll
    for (int q = 0; q < RING; ++q) {
        buf_store4<false>(dst, kOutOfRange + 16 * q, make_float4(0.f, 0.f, 0.f, 0.f));
        x[q] = load(first + 16 * q);
    }

    for (int t0 = tbeg; t0 < tend; t0 += 16 * RING) {
#pragma unroll
        for (int u = 0; u < RING; ++u) {
            mfma_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float4 xv = x[(u + g) % RING];
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][0], xv.x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][1], xv.y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][2], xv.z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][3], xv.w, acc, 0, 0, 0);
            }
            // tiles past the end of the span (the last pass of the loop may hold some) store nothing
            const int t = t0 + 16 * u + 4 * kq;
            buf_store4<false>(dst, (row_ok && t < tend) ? row_off + t * 4 : kOutOfRange,
                              make_float4(acc[0] * ts, acc[1] * ts, acc[2] * ts, acc[3] * ts));
            x[u] = load(first + (t0 - tbeg) + 16 * (u + RING));
        }
    }
}

template <bool CORR>
static int conv_mfma_launch(float* out, const float* in, const float* filt, int K, float ts, int64_t M, int64_t T,
                            hipStream_t stream) {
    const int64_t rowgroups = (M + 15) / 16;
    // about four waves per SIMD on 256 compute units when the rows alone do not provide them; a span is a
    // whole number of loop passes (RING tiles of 16 outputs) and is preceded by KPAD samples of warm-up
    const int64_t pass = 16 * (K <= 64 ? 8 : 16);
    int64_t spans = (4096 + rowgroups - 1) / rowgroups;
    const int64_t max_spans = (T + pass - 1) / pass;
    if (spans > max_spans) spans = max_spans;
    if (spans < 1) spans = 1;
    const int64_t span = (((T + spans - 1) / spans) + pass - 1) / pass * pass;
    spans = (T + span - 1) / span;
    const int64_t blocks = rowgroups * spans;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    // No non-temporal accesses here: a load or store covers 64 bytes per row, half a cache line, and the caches
    // put the halves together (measured: non-temporal accesses cost 25-85 % on large tensors).
#define SLAYER_CONV_MFMA(KP)                                                                                      \
    hipLaunchKernelGGL((conv_mfma_kernel<KP, CORR>), dim3((unsigned)blocks), dim3(kWave), 0, stream, out, in, filt, \
                       K, ts, M, (int)T, (int)span, (unsigned)spans)
    if (K <= 16) SLAYER_CONV_MFMA(16);
    else if (K <= 32) SLAYER_CONV_MFMA(32);
    else if (K <= 64) SLAYER_CONV_MFMA(64);
    else SLAYER_CONV_MFMA(128);
#undef SLAYER_CONV_MFMA
    return (int)hipGetLastError();
}

template <bool CORR>
static int conv_launch(float* out, const float* in, const float* filt, int64_t K, float ts,
                       int64_t M, int64_t T, hipStream_t stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in || !filt) return SLAYER_ENULL;
    if (K < 1) return SLAYER_EINVAL;
    if (K > kMaxTaps) return SLAYER_ERANGE;
    if (K > 8 && K <= 128 && T % 4 == 0 && T <= (1 << 22) && aligned16(out) && aligned16(in))
        return conv_mfma_launch<CORR>(out, in, filt, (int)K, ts, M, T, stream);
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
