// Time shift: out[m][t] = in[m][t - k_m], zero filled.  Pure data movement.
#include "common.h"
#include "tile.h"

namespace slayer {

// One lane per output quad (4 consecutive steps of one row); lanes of a wave cover
// consecutive quads of a row, so loads and stores are contiguous along time.
// VEC4: T % 4 == 0 and 16-byte aligned bases -> dwordx4 stores, and one dwordx4 load per quad whose
// source lies wholly inside the row, at a dword-aligned address when the row's shift is not a multiple of 4
// (the quads that straddle an end of the row load sample by sample).  Without VEC4 the stores are 16 bytes at
// dword-aligned addresses too, except for a row's last, partial quad.

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
    } else if (s >= 0 && s + 3 < T) {
        v = load_quad_dword_aligned(row + s);
    } else {
        if (s + 0 >= 0 && s + 0 < T) v.x = row[s + 0];
        if (s + 1 >= 0 && s + 1 < T) v.y = row[s + 1];
        if (s + 2 >= 0 && s + 2 < T) v.z = row[s + 2];
        if (s + 3 >= 0 && s + 3 < T) v.w = row[s + 3];
    }
    if (VEC4) {
        *reinterpret_cast<float4*>(dst) = v;
    } else if (t + 3 < T) {
        store_quad_dword_aligned(dst, v);
    } else {
        if (t + 0 < T) dst[0] = v.x;
        if (t + 1 < T) dst[1] = v.y;
        if (t + 2 < T) dst[2] = v.z;
        if (t + 3 < T) dst[3] = v.w;
    }
}

// Backward of a learnable delay in one pass: grad_in[m][t] = grad_out[m][t + k_m] (the shift undone) and,
// per row, sum_t grad_out[t] * ((-1/Ts) out[t] + (1/Ts) out[t-1]), the gradient with respect to the delay
// before it is summed over the batch.  One wave walks one row, 64 quads at a time; out[t-1] of a quad's
// first element is the neighbouring address (0 at t = 0).
template <bool VEC4>
__global__ __launch_bounds__(256) void delay_bwd_kernel(float* __restrict__ grad_in, float* __restrict__ partial,
                                                        const float* __restrict__ grad_out,
                                                        const float* __restrict__ out,
                                                        const float* __restrict__ lut, int scalar_steps, float ts,
                                                        float f0, float f1, int64_t M, int64_t npb, int T) {
    const int64_t m = (int64_t)blockIdx.x * 4 + threadIdx.y;
    if (m >= M) return;
    const int k = lut ? (int)(lut[m % npb] / ts) : scalar_steps;
    const float* g = grad_out + (size_t)m * (size_t)T;
    const float* y = out + (size_t)m * (size_t)T;
    float* dst = grad_in + (size_t)m * (size_t)T;
    float acc = 0.f;
    for (int t = 4 * (int)threadIdx.x; t < T; t += 256) {
        float4 gv = make_float4(0.f, 0.f, 0.f, 0.f), yv = gv, sv = gv;
        const int64_t s = (int64_t)t + (int64_t)k;       // source step of the first element of the shifted quad
        if (VEC4) {
            gv = *reinterpret_cast<const float4*>(g + t);
            yv = *reinterpret_cast<const float4*>(y + t);
        } else {
            if (t + 0 < T) { gv.x = g[t + 0]; yv.x = y[t + 0]; }
            if (t + 1 < T) { gv.y = g[t + 1]; yv.y = y[t + 1]; }
            if (t + 2 < T) { gv.z = g[t + 2]; yv.z = y[t + 2]; }
            if (t + 3 < T) { gv.w = g[t + 3]; yv.w = y[t + 3]; }
        }
        if (!grad_in) {
            // sums only: the shifted copy of the gradient is not wanted
        } else if (VEC4 && (k & 3) == 0) {
            if (s >= 0 && s < T) sv = *reinterpret_cast<const float4*>(g + s);
        } else if (VEC4 && s >= 0 && s + 3 < T) {
            sv = load_quad_dword_aligned(g + s);
        } else {
            if (s + 0 >= 0 && s + 0 < T) sv.x = g[s + 0];
            if (s + 1 >= 0 && s + 1 < T) sv.y = g[s + 1];
            if (s + 2 >= 0 && s + 2 < T) sv.z = g[s + 2];
            if (s + 3 >= 0 && s + 3 < T) sv.w = g[s + 3];
        }
        const float prev = t > 0 ? y[t - 1] : 0.f;
        if (partial) {
            // steps past T-1 hold zeros in gv and add nothing
            acc = __fmaf_rn(gv.x, f0 * yv.x + f1 * prev, acc);
            acc = __fmaf_rn(gv.y, f0 * yv.y + f1 * yv.x, acc);
            acc = __fmaf_rn(gv.z, f0 * yv.z + f1 * yv.y, acc);
            acc = __fmaf_rn(gv.w, f0 * yv.w + f1 * yv.z, acc);
        }
        if (!grad_in) {
        } else if (VEC4) {
            *reinterpret_cast<float4*>(dst + t) = sv;
        } else {
            if (t + 0 < T) dst[t + 0] = sv.x;
            if (t + 1 < T) dst[t + 1] = sv.y;
            if (t + 2 < T) dst[t + 2] = sv.z;
            if (t + 3 < T) dst[t + 3] = sv.w;
        }
    }
    if (partial) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d);
        if (threadIdx.x == 0) partial[m] = acc;
    }
}

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);   // li.hip
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip

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

extern "C" int slayer_delay_bwd(float* grad_in, float* grad_sum, const float* grad_out, const float* out,
                                const float* lut, int64_t scalar_steps, float sampling_time, float* workspace,
                                int64_t M, int64_t neurons_per_batch, int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (neurons_per_batch <= 0 || M % neurons_per_batch != 0) return SLAYER_EINVAL;
    if (sampling_time == 0.0f) return SLAYER_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (M == 0 || T == 0) return grad_sum ? launch_zero_fill(grad_sum, neurons_per_batch, st) : 0;
    if (!grad_out || !out || (!grad_in && !grad_sum)) return SLAYER_ENULL;
    if (grad_sum && !workspace) return SLAYER_ENULL;
    const int64_t kk = scalar_steps > T ? T : (scalar_steps < -T ? -T : scalar_steps);
    const int64_t blocks = (M + 3) / 4;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const bool vec = (T % 4 == 0) && aligned16(grad_in) && aligned16(grad_out) && aligned16(out);   // NULL counts as aligned
    const float f0 = -1.0f / sampling_time, f1 = 1.0f / sampling_time;
    float* partial = grad_sum ? workspace : nullptr;
    if (vec)
        hipLaunchKernelGGL((delay_bwd_kernel<true>), dim3((unsigned)blocks), dim3(64, 4), 0, st, grad_in, partial,
                           grad_out, out, lut, (int)kk, sampling_time, f0, f1, M, neurons_per_batch, (int)T);
    else
        hipLaunchKernelGGL((delay_bwd_kernel<false>), dim3((unsigned)blocks), dim3(64, 4), 0, st, grad_in, partial,
                           grad_out, out, lut, (int)kk, sampling_time, f0, f1, M, neurons_per_batch, (int)T);
    if (int e = (int)hipGetLastError()) return e;
    if (grad_sum)
        return launch_reduce_param_grad(grad_sum, workspace, workspace + M, M, neurons_per_batch,
                                        neurons_per_batch, st);
    return 0;
}
