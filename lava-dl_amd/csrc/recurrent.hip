// Recurrent layer of CUBA or ALIF neurons: the whole time loop of
//   feedback[t] = R s[t-1];  s[t] = neuron(z[t] + feedback[t])
// in one launch per direction.  The reference runs this loop in Python with one neuron call per
// time step (utils/recurrent.py:45-112), i.e. a dozen launches per step; here one workgroup owns
// one batch sample, one thread one neuron, and a step costs one barrier: the neurons that fired at
// step t-1 travel as per-wave index lists through LDS and the feedback is the sum of the columns of
// R they select (times the spike's value for graded spikes), read as rows of R^T so that
// neighbouring threads read neighbouring addresses.  rec_t carries one extra all-zero row: the lists
// are padded with its index.
//
// A neuron called one step at a time carries its state between the calls as float32 (CUBA: current,
// voltage * (1 - spike); ALIF: current, voltage, threshold + spike * step, refractory + 2 * spike *
// threshold); the kernel makes the same round trip, so it matches that loop bit for bit whenever the
// feedback sum is exact in float32 (quantised weights, and for graded spikes quantised voltages that
// keep the products exact), and to float32 summation order otherwise.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kMaxRecurrent = 1024;      // neurons per sample = threads per workgroup
constexpr int kGather = 16;              // rows of the weight matrix a thread keeps in flight

struct RecurrentFwd {
    float *spk, *vol, *theta;                                 // [N][C][T]; theta: ALIF only
    float *cur_last, *vol_last, *th_last, *ref_last;          // [N*C]; th / ref: ALIF only
    const float *z, *rec_t;
    const float *i_decay, *v_decay, *th_decay, *ref_decay, *i_state, *v_state, *th_state, *ref_state;
    int64_t n_id, n_vd, n_td, n_rd, n_is, n_vs, n_ts, n_rs;
    float w, inv_w, spike_thr, spike_scale, th_step_f;
    int base;
    int C, T;
    unsigned* range_flag;                                     // see raise_range_flag in tile.h
};

template <bool ALIF, bool GRADED, bool POW2, bool VEC4>
__global__ __launch_bounds__(kMaxRecurrent) void recurrent_fwd_kernel(const RecurrentFwd p) {
    // spikes of the previous step: per wave a count and the indices of its neurons that fired, padded
    // to a multiple of kGather with C, the index of the all-zero row that ends rec_t; graded spikes
    // bring their values along (0 in the padding)
    __shared__ int counts[2][kMaxRecurrent / kWave];
    __shared__ __attribute__((aligned(16))) int fired_list[2][kMaxRecurrent];
    __shared__ __attribute__((aligned(16))) float fired_value[GRADED ? 2 : 1][GRADED ? kMaxRecurrent : 4];
    const int C = p.C, T = p.T;
    const float w = p.w, inv_w = p.inv_w;
    const float* __restrict__ rec_t = p.rec_t;
    const int c = threadIdx.x;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    const bool live = c < C;
    const int64_t m = (int64_t)blockIdx.x * C + (live ? c : 0);
    const float* zrow = p.z + m * (int64_t)T;
    float* srow = p.spk + m * (int64_t)T;
    float* vrow = p.vol + m * (int64_t)T;
    float* trow = ALIF ? p.theta + m * (int64_t)T : nullptr;
    auto from = [&](int y) -> float { const float f = (float)y; return POW2 ? f * inv_w : f / w; };

    int yc = 0, yv = 0, th = 0, r = 0, mi = 0, mv = 0, mt = 0, mr = 0;
    unsigned acc_lif = 0u, acc_th = 0u;                       // range of the states, see range_bits in tile.h
    if (live) {
        yc = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m] * w);
        yv = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m] * w);
        mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m, C, p.n_id)]));
        mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m, C, p.n_vd)]));
        if (ALIF) {
            th = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m] * w);
            r = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m] * w);
            mt = 4096 - trunc_i32(rintf(p.th_decay[param_index(m, C, p.n_td)]));
            mr = 4096 - trunc_i32(rintf(p.ref_decay[param_index(m, C, p.n_rd)]));
            check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag);
        }
        check_multiplier(mi, p.range_flag); check_multiplier(mv, p.range_flag);
        acc_lif = ((unsigned)yc + (1u << 30)) | ((unsigned)yv + (1u << 30));
        acc_th = ((unsigned)th + (1u << 28)) | ((unsigned)r + (1u << 28));
    }
    float cur = 0.f, vol = 0.f, thf = 0.f, rf = 0.f;
    float4 zq = make_float4(0.f, 0.f, 0.f, 0.f), sq = zq, vq = zq, tq = zq;

    for (int t = 0; t < T; ++t) {
        // feedback from the spikes of step t-1 (none before the first step)
        float fb = 0.f;
        if (t > 0) {
            for (int wv = 0; wv < waves; ++wv) {
                const int cnt = __builtin_amdgcn_readfirstlane(counts[(t - 1) & 1][wv]);
                const int4* seg = reinterpret_cast<const int4*>(&fired_list[(t - 1) & 1][wv * kWave]);
                const float4* val = reinterpret_cast<const float4*>(&fired_value[GRADED ? (t - 1) & 1 : 0][GRADED ? wv * kWave : 0]);
                for (int k = 0; k < cnt; k += kGather) {           // kGather rows of R^T in flight at a time
                    int row[kGather];
                    float sv[kGather];
#pragma unroll
                    for (int q = 0; q < kGather / 4; ++q) {
                        const int4 i4 = seg[k / 4 + q];
                        row[4 * q] = i4.x; row[4 * q + 1] = i4.y; row[4 * q + 2] = i4.z; row[4 * q + 3] = i4.w;
                        if (GRADED) {
                            const float4 f4 = val[k / 4 + q];
                            sv[4 * q] = f4.x; sv[4 * q + 1] = f4.y; sv[4 * q + 2] = f4.z; sv[4 * q + 3] = f4.w;
                        }
                    }
                    float v[kGather];
#pragma unroll
                    for (int q = 0; q < kGather; ++q) v[q] = live ? rec_t[row[q] * C + c] : 0.f;
#pragma unroll
                    for (int q = 0; q < kGather; ++q) fb += GRADED ? sv[q] * v[q] : v[q];
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
        // one step of every state, each starting from the float32 value the previous call left and
        // handing a float32 value to the next operator
        yc = add_sat(rs0_12(yc, mi), trunc_i32(w * dend));
        cur = from(yc);
        yc = trunc_i32(w * cur);
        const int yn = add_sat(rs0_12(yv, mv), yc);
        acc_lif |= ((unsigned)yc + (1u << 30)) | ((unsigned)yn + (1u << 30));
        vol = from(yn);
        float theta = p.spike_thr;
        if (ALIF) {
            r = rs0_12(r, mr);
            th = rs0_12(th - p.base, mt) + p.base;
            acc_th |= ((unsigned)th + (1u << 28)) | ((unsigned)r + (1u << 28));
            thf = from(th);
            rf = from(r);
            theta = thf + rf;
        }
        const bool fired = live && vol >= theta;
        const float s = GRADED ? ((fired ? 1.0f : 0.0f) * vol) / p.spike_scale : (fired ? 1.0f : 0.0f);
        const bool spiked = live && s > 0.0f;           // what the carried states and the feedback see
        if (ALIF) {
            yv = trunc_i32(w * vol);
            r = trunc_i32((spiked ? rf + 2.0f * thf : rf) * w);
            th = trunc_i32((spiked ? thf + p.th_step_f : thf) * w);
        } else {
            yv = spiked ? 0 : trunc_i32(w * vol);
        }
        {
            // a graded spike that is not positive still takes part in the feedback with its value
            const bool listed = GRADED ? (live && s != 0.0f) : fired;
            const unsigned long long ballot = __ballot(listed);
            const int lane = c & (kWave - 1);
            const int cnt = __builtin_popcountll(ballot);
            const int below = __builtin_popcountll(ballot & ((1ull << lane) - 1ull));   // listed lanes below this one
            int* seg = &fired_list[t & 1][(c / kWave) * kWave];
            if (listed) {
                seg[below] = c;
                if (GRADED) fired_value[t & 1][(c / kWave) * kWave + below] = s;
            } else {                                   // the other lanes write the padding
                const int slot = cnt + (lane - below);
                if (slot < ((cnt + kGather - 1) & ~(kGather - 1))) {
                    seg[slot] = C;
                    if (GRADED) fired_value[t & 1][(c / kWave) * kWave + slot] = 0.0f;
                }
            }
            if (lane == 0) counts[t & 1][c / kWave] = cnt;
        }
        if (VEC4) {
            if ((t & 3) == 0) { sq.x = s; vq.x = vol; tq.x = theta; }
            else if ((t & 3) == 1) { sq.y = s; vq.y = vol; tq.y = theta; }
            else if ((t & 3) == 2) { sq.z = s; vq.z = vol; tq.z = theta; }
            else {
                sq.w = s; vq.w = vol; tq.w = theta;
                if (live) {
                    *reinterpret_cast<float4*>(srow + t - 3) = sq;
                    *reinterpret_cast<float4*>(vrow + t - 3) = vq;
                    if (ALIF) *reinterpret_cast<float4*>(trow + t - 3) = tq;
                }
            }
        } else if (live) {
            srow[t] = s;
            vrow[t] = vol;
            if (ALIF) trow[t] = theta;
        }
        __syncthreads();
    }
    if (live && (range_exceeded(acc_lif, 30) || range_exceeded(acc_th, 28))) raise_range_flag(p.range_flag);
    if (live) {
        p.cur_last[m] = cur;
        p.vol_last[m] = vol;
        if (ALIF) {
            p.th_last[m] = thf;
            p.ref_last[m] = rf;
        }
    }
}

// Backward through the loop as the reference differentiates it (utils/recurrent.py:83-112): the
// state carried between the one-step neuron calls is a constant, so a step contributes the spike
// surrogate only, and the gradient reaches step t-1 through R.
template <bool THETA, bool GRADED, bool VEC4>
__global__ __launch_bounds__(kMaxRecurrent) void recurrent_bwd_kernel(
    float* __restrict__ grad_z, const float* __restrict__ grad_spikes, const float* __restrict__ voltage,
    const float* __restrict__ theta, const float* __restrict__ rec, float spike_thr, float tau, float rho, int C,
    int T) {
    __shared__ float gd_s[2][kMaxRecurrent];
    const int c = threadIdx.x;
    const bool live = c < C;
    const int64_t m = (int64_t)blockIdx.x * C + (live ? c : 0);
    const float* grow = grad_spikes + m * (int64_t)T;
    const float* vrow = voltage + m * (int64_t)T;
    const float* trow = THETA ? theta + m * (int64_t)T : nullptr;
    float* orow = grad_z + m * (int64_t)T;
    const float lead = (rho / 2.0f) / tau;
    const float inv_tau = 1.0f / tau;
    float carry = 0.f;
    float4 gq = make_float4(0.f, 0.f, 0.f, 0.f), vq = gq, oq = gq, tq = gq;

    for (int t = T - 1; t >= 0; --t) {
        float g, v, th = spike_thr;
        if (VEC4) {
            if ((t & 3) == 3 && live) {
                gq = *reinterpret_cast<const float4*>(grow + t - 3);
                vq = *reinterpret_cast<const float4*>(vrow + t - 3);
                if (THETA) tq = *reinterpret_cast<const float4*>(trow + t - 3);
            }
            g = (t & 3) == 0 ? gq.x : (t & 3) == 1 ? gq.y : (t & 3) == 2 ? gq.z : gq.w;
            v = (t & 3) == 0 ? vq.x : (t & 3) == 1 ? vq.y : (t & 3) == 2 ? vq.z : vq.w;
            if (THETA) th = (t & 3) == 0 ? tq.x : (t & 3) == 1 ? tq.y : (t & 3) == 2 ? tq.z : tq.w;
        } else {
            g = live ? grow[t] : 0.f;
            v = live ? vrow[t] : 0.f;
            if (THETA) th = live ? trow[t] : 0.f;
        }
        const float gs = carry + g;
        const float d = v - th;
        const float factor = GRADED ? rho * expf(fminf(d, 0.0f) * inv_tau) : lead * expf(-fabsf(d) * inv_tau);
        const float gd = live ? factor * gs : 0.f;
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

namespace {

int check_recurrent_sizes(int64_t N, int64_t C, int64_t T) {
    if (N < 0 || C < 0 || T < 0) return SLAYER_EINVAL;
    if (C > kMaxRecurrent || T > 0x7fffffffLL || N > 0x7fffffffLL) return SLAYER_ERANGE;
    return 0;
}

template <bool ALIF>
int launch_recurrent_fwd(RecurrentFwd p, int graded, int w_scale, int64_t N, hipStream_t st) {
    bool vec = (p.T % 4) == 0 && aligned16(p.z) && aligned16(p.spk) && aligned16(p.vol);
    if (ALIF) vec = vec && aligned16(p.theta);
    const dim3 grid((unsigned)N), block((unsigned)((p.C + kWave - 1) / kWave * kWave));
    const bool pow2 = is_pow2(w_scale);
#define SLAYER_REC(G, P, V) hipLaunchKernelGGL((recurrent_fwd_kernel<ALIF, G, P, V>), grid, block, 0, st, p)
#define SLAYER_REC2(G)                                                                                        \
    do {                                                                                                      \
        if (pow2) { if (vec) SLAYER_REC(G, true, true); else SLAYER_REC(G, true, false); }                    \
        else { if (vec) SLAYER_REC(G, false, true); else SLAYER_REC(G, false, false); }                       \
    } while (0)
    if (graded) SLAYER_REC2(true); else SLAYER_REC2(false);
#undef SLAYER_REC2
#undef SLAYER_REC
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int slayer_cuba_recurrent_fwd(float* spk_out, float* vol_out, float* cur_last_out, float* vol_last_out,
                                         const float* z, const float* rec_t,
                                         const float* i_decay, const float* v_decay,
                                         const float* i_state, const float* v_state,
                                         float spike_threshold, int graded, float spike_scale, int w_scale,
                                         int64_t N, int64_t C, int64_t num_i_decays, int64_t num_v_decays,
                                         int64_t num_i_states, int64_t num_v_states, int64_t T, void* stream) {
    if (int e = check_recurrent_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!spk_out || !vol_out || !cur_last_out || !vol_last_out || !z || !rec_t || !i_decay || !v_decay || !i_state ||
        !v_state)
        return SLAYER_ENULL;
    if (int e = check_params(N * C, C, num_i_decays)) return e;
    if (int e = check_params(N * C, C, num_v_decays)) return e;
    if (int e = check_states(N * C, num_i_states)) return e;
    if (int e = check_states(N * C, num_v_states)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    RecurrentFwd p{};
    p.spk = spk_out; p.vol = vol_out; p.cur_last = cur_last_out; p.vol_last = vol_last_out;
    p.z = z; p.rec_t = rec_t; p.i_decay = i_decay; p.v_decay = v_decay; p.i_state = i_state; p.v_state = v_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_is = num_i_states; p.n_vs = num_v_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / p.w; p.spike_thr = spike_threshold; p.spike_scale = spike_scale;
    p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_device();
    return launch_recurrent_fwd<false>(p, graded, w_scale, N, (hipStream_t)stream);
}

extern "C" int slayer_alif_recurrent_fwd(float* spk_out, float* vol_out, float* theta_out,
                                         float* cur_last_out, float* vol_last_out, float* th_last_out,
                                         float* ref_last_out, const float* z, const float* rec_t,
                                         const float* i_decay, const float* v_decay, const float* th_decay,
                                         const float* ref_decay, const float* i_state, const float* v_state,
                                         const float* th_state, const float* ref_state,
                                         float th_step, int64_t th0_scaled, int graded, float spike_scale, int w_scale,
                                         int64_t N, int64_t C,
                                         int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays,
                                         int64_t num_ref_decays, int64_t num_i_states, int64_t num_v_states,
                                         int64_t num_th_states, int64_t num_ref_states, int64_t T, void* stream) {
    if (int e = check_recurrent_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!spk_out || !vol_out || !theta_out || !cur_last_out || !vol_last_out || !th_last_out || !ref_last_out || !z ||
        !rec_t || !i_decay || !v_decay || !th_decay || !ref_decay || !i_state || !v_state || !th_state || !ref_state)
        return SLAYER_ENULL;
    for (int64_t n : {num_i_decays, num_v_decays, num_th_decays, num_ref_decays})
        if (int e = check_params(N * C, C, n)) return e;
    for (int64_t n : {num_i_states, num_v_states, num_th_states, num_ref_states})
        if (int e = check_states(N * C, n)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    if (th0_scaled > 0x7fffffffLL || th0_scaled < -0x7fffffffLL) return SLAYER_ERANGE;
    RecurrentFwd p{};
    p.spk = spk_out; p.vol = vol_out; p.theta = theta_out;
    p.cur_last = cur_last_out; p.vol_last = vol_last_out; p.th_last = th_last_out; p.ref_last = ref_last_out;
    p.z = z; p.rec_t = rec_t;
    p.i_decay = i_decay; p.v_decay = v_decay; p.th_decay = th_decay; p.ref_decay = ref_decay;
    p.i_state = i_state; p.v_state = v_state; p.th_state = th_state; p.ref_state = ref_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_td = num_th_decays; p.n_rd = num_ref_decays;
    p.n_is = num_i_states; p.n_vs = num_v_states; p.n_ts = num_th_states; p.n_rs = num_ref_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / p.w; p.spike_scale = spike_scale; p.th_step_f = th_step;
    p.base = (int)th0_scaled;
    p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_for_threshold(0, th0_scaled);
    return launch_recurrent_fwd<true>(p, graded, w_scale, N, (hipStream_t)stream);
}

extern "C" int slayer_recurrent_bwd(float* grad_z, const float* grad_spikes, const float* voltage, const float* theta,
                                    const float* rec, float spike_threshold, float tau_rho, float scale_rho,
                                    int graded, int64_t N, int64_t C, int64_t T, void* stream) {
    if (int e = check_recurrent_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!grad_z || !grad_spikes || !voltage || !rec) return SLAYER_ENULL;
    const bool vec = (T % 4) == 0 && aligned16(grad_z) && aligned16(grad_spikes) && aligned16(voltage) &&
                     (!theta || aligned16(theta));
    const dim3 grid((unsigned)N), block((unsigned)((C + kWave - 1) / kWave * kWave));
    hipStream_t st = (hipStream_t)stream;
#define SLAYER_RB(TH, G, V)                                                                                     \
    hipLaunchKernelGGL((recurrent_bwd_kernel<TH, G, V>), grid, block, 0, st, grad_z, grad_spikes, voltage, theta, \
                       rec, spike_threshold, tau_rho, scale_rho, (int)C, (int)T)
#define SLAYER_RB2(TH, G) do { if (vec) SLAYER_RB(TH, G, true); else SLAYER_RB(TH, G, false); } while (0)
    if (theta) { if (graded) SLAYER_RB2(true, true); else SLAYER_RB2(true, false); }
    else { if (graded) SLAYER_RB2(false, true); else SLAYER_RB2(false, false); }
#undef SLAYER_RB2
#undef SLAYER_RB
    return (int)hipGetLastError();
}
