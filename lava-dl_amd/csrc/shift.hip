// Time shift: out[m][t] = in[m][t - k_m], zero filled.  Pure data movement.
#include "common.h"
#include "tile.h"

namespace slayer {

// One lane per output quad (4 consecutive steps of one row); lanes of a wave cover
// consecutive quads of a row, so loads and stores are contiguous along time.
// VEC4: T % 4 == 0 and 16-byte aligned bases -> dwordx4 stores, and dwordx4 loads
// whenever the row's shift is a multiple of 4.
template <bool VEC4>
__global__ __launch_bounds__(256) void shift_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                    const float* __restrict__ lut, int scalar_steps, float ts,
                                                    int64_t M, int64_t npb, int T, unsigned quads_per_row,
                                                    unsigned blocks_per_row) {
    // blockDim = (64, 4): x walks quads of a row, y picks one of 4 rows
    const unsigned rowgroup = blockIdx.x / blocks_per_row;
    const unsigned seg = blockIdx.x - rowgroup * blocks_per_row;
    const int64_t m = (int64_t)rowgroup * 4 + threadIdx.y;
    const unsigned q = seg * 64 + threadIdx.x;
    if (m >= M || q >= quads_per_row) return;
    const int k = lut ? (int)(lut[m % npb] / ts) : scalar_steps;
    const int t = (int)(q * 4);
    const float* row = in + (size_t)m * (size_t)T;
    float* dst = out + (size_t)m * (size_t)T + t;
    const int64_t s = (int64_t)t - (int64_t)k;       // source step of the first element
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (VEC4 && (k & 3) == 0) {
        if (s >= 0 && s < T) v = *reinterpret_cast<const float4*>(row + s);
    } else {
        if (s + 0 >= 0 && s + 0 < T) v.x = row[s + 0];
        if (s + 1 >= 0 && s + 1 < T) v.y = row[s + 1];
        if (s + 2 >= 0 && s + 2 < T) v.z = row[s + 2];
        if (s + 3 >= 0 && s + 3 < T) v.w = row[s + 3];
    }
    if (VEC4) {
        *reinterpret_cast<float4*>(dst) = v;
    } else {
        if (t + 0 < T) dst[0] = v.x;
        if (t + 1 < T) dst[1] = v.y;
        if (t + 2 < T) dst[2] = v.z;
        if (t + 3 < T) dst[3] = v.w;
    }
}

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_shift(float* out, const float* in, const float* lut, int64_t scalar_steps,
                            float sampling_time, int64_t M, int64_t neurons_per_batch, int64_t T,
                            void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in) return SLAYER_ENULL;
    if (neurons_per_batch <= 0 || M % neurons_per_batch != 0) return SLAYER_EINVAL;
    if (lut && sampling_time == 0.0f) return SLAYER_EINVAL;
    // any |shift| >= T empties the row; clamp so the step count fits an int
    const int64_t kk = scalar_steps > T ? T : (scalar_steps < -T ? -T : scalar_steps);
    const unsigned quads = (unsigned)((T + 3) / 4);
    const unsigned bpr = (quads + 63) / 64;
    const int64_t blocks = ((M + 3) / 4) * (int64_t)bpr;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const bool vec = (T % 4 == 0) && aligned16(out) && aligned16(in);
    hipStream_t st = (hipStream_t)stream;
    if (vec)
        hipLaunchKernelGGL((shift_kernel<true>), dim3((unsigned)blocks), dim3(64, 4), 0, st, out, in, lut,
                           (int)kk, sampling_time, M, neurons_per_batch, (int)T, quads, bpr);
    else
        hipLaunchKernelGGL((shift_kernel<false>), dim3((unsigned)blocks), dim3(64, 4), 0, st, out, in, lut,
                           (int)kk, sampling_time, M, neurons_per_batch, (int)T, quads, bpr);
    return (int)hipGetLastError();
}
