// Recurrent CUBA layer: the whole time loop of
//   feedback[t] = R s[t-1];  s[t] = neuron(z[t] + feedback[t])
// in one launch per direction.  The reference runs this loop in Python with one neuron call per
// time step (utils/recurrent.py:45-112), i.e. a dozen launches per step; here one workgroup owns
// one batch sample, one thread one neuron, and a step costs one barrier: the spikes of step t-1
// travel as a bit mask through LDS and the feedback is the sum of the columns of R they select
// (binary spikes), read as rows of R^T so that neighbouring threads read neighbouring addresses.
// rec_t carries one extra all-zero row: lists of spiking neurons are padded with its index.
//
// A neuron called one step at a time carries its state between the calls as float32
// (current, voltage * (1 - spike)); the kernel makes the same round trip, so it matches that loop
// bit for bit whenever the feedback sum is exact in float32 (quantised weights), and to float32
// summation order otherwise.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kMaxRecurrent = 1024;      // neurons per sample = threads per workgroup
constexpr int kGather = 16;              // rows of the weight matrix a thread keeps in flight

template <bool POW2, bool VEC4>
__global__ __launch_bounds__(kMaxRecurrent) void cuba_recurrent_fwd_kernel(
    float* __restrict__ spk_out, float* __restrict__ vol_out, float* __restrict__ cur_last, float* __restrict__ vol_last,
    const float* __restrict__ z, const float* __restrict__ rec_t, const float* __restrict__ i_decay,
    const float* __restrict__ v_decay, const float* __restrict__ i_state, const float* __restrict__ v_state,
    int64_t n_id, int64_t n_vd, int64_t n_is, int64_t n_vs, float w, float inv_w, float spike_thr, int C, int T) {
    // spikes of the previous step: per wave a count and the indices of its neurons that fired, padded
    // to a multiple of kGather with C, the index of the all-zero row that ends rec_t
    __shared__ int counts[2][kMaxRecurrent / kWave];
    __shared__ __attribute__((aligned(16))) int fired_list[2][kMaxRecurrent];
    const int c = threadIdx.x;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    const bool live = c < C;
    const int64_t m = (int64_t)blockIdx.x * C + (live ? c : 0);
    const float* zrow = z + m * (int64_t)T;
    float* srow = spk_out + m * (int64_t)T;
    float* vrow = vol_out + m * (int64_t)T;

    int yc = 0, yv = 0, mi = 0, mv = 0;
    if (live) {
        yc = trunc_i32(i_state[n_is == 1 ? 0 : m] * w);
        yv = trunc_i32(v_state[n_vs == 1 ? 0 : m] * w);
        mi = 4096 - trunc_i32(i_decay[param_index(m, C, n_id)]);
        mv = 4096 - trunc_i32(v_decay[param_index(m, C, n_vd)]);
    }
    float cur = 0.f, vol = 0.f;
    float4 zq = make_float4(0.f, 0.f, 0.f, 0.f), sq = zq, vq = zq;

    for (int t = 0; t < T; ++t) {
        // feedback from the spikes of step t-1 (none before the first step)
        float fb = 0.f;
        if (t > 0) {
            for (int wv = 0; wv < waves; ++wv) {
                const int cnt = __builtin_amdgcn_readfirstlane(counts[(t - 1) & 1][wv]);
                const int4* seg = reinterpret_cast<const int4*>(&fired_list[(t - 1) & 1][wv * kWave]);
                for (int k = 0; k < cnt; k += kGather) {           // kGather rows of R^T in flight at a time
                    int row[kGather];
#pragma unroll
                    for (int q = 0; q < kGather / 4; ++q) {
                        const int4 i4 = seg[k / 4 + q];
                        row[4 * q] = i4.x; row[4 * q + 1] = i4.y; row[4 * q + 2] = i4.z; row[4 * q + 3] = i4.w;
                    }
                    float v[kGather];
#pragma unroll
                    for (int q = 0; q < kGather; ++q) v[q] = live ? rec_t[row[q] * C + c] : 0.f;
#pragma unroll
                    for (int q = 0; q < kGather; ++q) fb += v[q];
                }
            }
        }
        float zt;
        if (VEC4) {
            if ((t & 3) == 0 && live) zq = *reinterpret_cast<const float4*>(zrow + t);
            zt = (t & 3) == 0 ? zq.x : (t & 3) == 1 ? zq.y : (t & 3) == 2 ? zq.z : zq.w;
        } else {
            zt = live ? zrow[t] : 0.f;
        }
        const float dend = zt + fb;
        // one step of current and voltage, each starting from the float32 state the previous call left
        yc = rs0_12(yc, mi) + trunc_i32(w * dend);
        const float cf = (float)yc;
        cur = POW2 ? cf * inv_w : cf / w;
        const int yn = rs0_12(yv, mv) + trunc_i32(w * cur);
        const float vf = (float)yn;
        vol = POW2 ? vf * inv_w : vf / w;
        const bool fired = live && vol >= spike_thr;
        if (POW2) {
            yv = fired ? 0 : yn;
        } else {                               // the carried float32 states are rescaled by the next call
            yc = trunc_i32(cur * w);
            yv = fired ? 0 : trunc_i32(vol * w);
        }
        {
            const unsigned long long ballot = __ballot(fired);
            const int lane = c & (kWave - 1);
            const int cnt = __builtin_popcountll(ballot);
            const int below = __builtin_popcountll(ballot & ((1ull << lane) - 1ull));   // fired lanes below this one
            int* seg = &fired_list[t & 1][(c / kWave) * kWave];
            if (fired) {
                seg[below] = c;
            } else {                                   // the lanes that did not fire write the padding
                const int slot = cnt + (lane - below);
                if (slot < ((cnt + kGather - 1) & ~(kGather - 1))) seg[slot] = C;
            }
            if (lane == 0) counts[t & 1][c / kWave] = cnt;
        }
        const float s = fired ? 1.0f : 0.0f;
        if (VEC4) {
            if ((t & 3) == 0) { sq.x = s; vq.x = vol; }
            else if ((t & 3) == 1) { sq.y = s; vq.y = vol; }
            else if ((t & 3) == 2) { sq.z = s; vq.z = vol; }
            else {
                sq.w = s; vq.w = vol;
                if (live) {
                    *reinterpret_cast<float4*>(srow + t - 3) = sq;
                    *reinterpret_cast<float4*>(vrow + t - 3) = vq;
                }
            }
        } else if (live) {
            srow[t] = s;
            vrow[t] = vol;
        }
        __syncthreads();
    }
    if (live) {
        cur_last[m] = cur;
        vol_last[m] = vol;
    }
}

// Backward through the loop as the reference differentiates it (utils/recurrent.py:83-112): the
// state carried between the one-step neuron calls is a constant, so a step contributes the spike
// surrogate only, and the gradient reaches step t-1 through R.
template <bool VEC4>
__global__ __launch_bounds__(kMaxRecurrent) void cuba_recurrent_bwd_kernel(
    float* __restrict__ grad_z, const float* __restrict__ grad_spikes, const float* __restrict__ voltage,
    const float* __restrict__ rec, float spike_thr, float tau, float rho, int C, int T) {
    __shared__ float gd_s[2][kMaxRecurrent];
    const int c = threadIdx.x;
    const bool live = c < C;
    const int64_t m = (int64_t)blockIdx.x * C + (live ? c : 0);
    const float* grow = grad_spikes + m * (int64_t)T;
    const float* vrow = voltage + m * (int64_t)T;
    float* orow = grad_z + m * (int64_t)T;
    const float lead = (rho / 2.0f) / tau;
    float carry = 0.f;
    float4 gq = make_float4(0.f, 0.f, 0.f, 0.f), vq = gq, oq = gq;

    for (int t = T - 1; t >= 0; --t) {
        float g, v;
        if (VEC4) {
            if ((t & 3) == 3 && live) {
                gq = *reinterpret_cast<const float4*>(grow + t - 3);
                vq = *reinterpret_cast<const float4*>(vrow + t - 3);
            }
            g = (t & 3) == 0 ? gq.x : (t & 3) == 1 ? gq.y : (t & 3) == 2 ? gq.z : gq.w;
            v = (t & 3) == 0 ? vq.x : (t & 3) == 1 ? vq.y : (t & 3) == 2 ? vq.z : vq.w;
        } else {
            g = live ? grow[t] : 0.f;
            v = live ? vrow[t] : 0.f;
        }
        const float gs = carry + g;
        const float gd = live ? (lead * expf(-fabsf(v - spike_thr) / tau)) * gs : 0.f;
        if (VEC4) {
            if ((t & 3) == 3) oq.w = gd;
            else if ((t & 3) == 2) oq.z = gd;
            else if ((t & 3) == 1) oq.y = gd;
            else {
                oq.x = gd;
                if (live) *reinterpret_cast<float4*>(orow + t) = oq;
            }
        } else if (live) {
            orow[t] = gd;
        }
        gd_s[t & 1][c] = gd;
        __syncthreads();
        // gradient handed to step t-1: (grad of the feedback) R, this thread's column
        carry = 0.f;
        if (live && t > 0) {
            const float* col = rec + c;
            const float* gd = gd_s[t & 1];
            int cc = 0;
            for (; cc + 16 <= C; cc += 16) {       // sixteen rows of R in flight at a time
                float r[16];
#pragma unroll
                for (int k = 0; k < 16; ++k) r[k] = col[(int64_t)(cc + k) * C];
#pragma unroll
                for (int k = 0; k < 16; ++k) carry = __fmaf_rn(gd[cc + k], r[k], carry);
            }
            for (; cc < C; ++cc) carry = __fmaf_rn(gd[cc], col[(int64_t)cc * C], carry);
        }
    }
}

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_cuba_recurrent_fwd(float* spk_out, float* vol_out, float* cur_last_out, float* vol_last_out,
                                         const float* z, const float* rec_t,
                                         const float* i_decay, const float* v_decay,
                                         const float* i_state, const float* v_state,
                                         float spike_threshold, int w_scale,
                                         int64_t N, int64_t C, int64_t num_i_decays, int64_t num_v_decays,
                                         int64_t num_i_states, int64_t num_v_states, int64_t T, void* stream) {
    if (N < 0 || C < 0 || T < 0) return SLAYER_EINVAL;
    if (C > kMaxRecurrent || T > 0x7fffffffLL || N > 0x7fffffffLL) return SLAYER_ERANGE;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!spk_out || !vol_out || !cur_last_out || !vol_last_out || !z || !rec_t || !i_decay || !v_decay || !i_state ||
        !v_state)
        return SLAYER_ENULL;
    if (int e = check_params(N * C, C, num_i_decays)) return e;
    if (int e = check_params(N * C, C, num_v_decays)) return e;
    if (int e = check_states(N * C, num_i_states)) return e;
    if (int e = check_states(N * C, num_v_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const float w = (float)w_scale;
    const bool vec = (T % 4) == 0 && aligned16(z) && aligned16(spk_out) && aligned16(vol_out);
    const dim3 grid((unsigned)N), block((unsigned)((C + kWave - 1) / kWave * kWave));
    hipStream_t st = (hipStream_t)stream;
#define SLAYER_REC(P, V)                                                                                          \
    hipLaunchKernelGGL((cuba_recurrent_fwd_kernel<P, V>), grid, block, 0, st, spk_out, vol_out, cur_last_out,     \
                       vol_last_out, z, rec_t, i_decay, v_decay, i_state, v_state, num_i_decays, num_v_decays,    \
                       num_i_states, num_v_states, w, 1.0f / w, spike_threshold, (int)C, (int)T)
    if (is_pow2(w_scale)) { if (vec) SLAYER_REC(true, true); else SLAYER_REC(true, false); }
    else { if (vec) SLAYER_REC(false, true); else SLAYER_REC(false, false); }
#undef SLAYER_REC
    return (int)hipGetLastError();
}

extern "C" int slayer_cuba_recurrent_bwd(float* grad_z, const float* grad_spikes, const float* voltage,
                                         const float* rec, float spike_threshold, float tau_rho, float scale_rho,
                                         int64_t N, int64_t C, int64_t T, void* stream) {
    if (N < 0 || C < 0 || T < 0) return SLAYER_EINVAL;
    if (C > kMaxRecurrent || T > 0x7fffffffLL || N > 0x7fffffffLL) return SLAYER_ERANGE;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!grad_z || !grad_spikes || !voltage || !rec) return SLAYER_ENULL;
    const bool vec = (T % 4) == 0 && aligned16(grad_z) && aligned16(grad_spikes) && aligned16(voltage);
    const dim3 grid((unsigned)N), block((unsigned)((C + kWave - 1) / kWave * kWave));
    hipStream_t st = (hipStream_t)stream;
    if (vec)
        hipLaunchKernelGGL((cuba_recurrent_bwd_kernel<true>), grid, block, 0, st, grad_z, grad_spikes, voltage, rec,
                           spike_threshold, tau_rho, scale_rho, (int)C, (int)T);
    else
        hipLaunchKernelGGL((cuba_recurrent_bwd_kernel<false>), grid, block, 0, st, grad_z, grad_spikes, voltage, rec,
                           spike_threshold, tau_rho, scale_rho, (int)C, (int)T);
    return (int)hipGetLastError();
}
