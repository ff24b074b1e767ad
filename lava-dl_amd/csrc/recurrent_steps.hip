// Recurrent layer of CUBA or ALIF neurons, one launch per time step: the form for layers too wide for one
// workgroup per sample (recurrent.hip), where re-reading the weight matrix per sample is what a step costs.
//
//   feedback[t] = R s[t-1];  s[t] = neuron(z[t] + feedback[t])          (utils/recurrent.py:45-112 in the reference)
//
// A step is one product of the [C x C] weight matrix with the [N x C] spikes of the previous step -- the matrix
// is read once per step for the whole batch -- followed by one neuron step of every (sample, neuron).  A workgroup
// owns 16 neurons for up to 64 samples: its eight waves each take an eighth of the sum over the presynaptic
// neurons on the matrix cores (v_mfma_f32_16x16x4_f32: float32 operands and accumulation; the products of a 0/1
// spike are exact, and so is every partial sum of quantised weights), the partial sums meet in LDS, and the first
// waves run the neuron step on the result: lane (q, j) of a 16 x 16 result tile holds neurons 4q .. 4q+3 of sample
// j, a quad of neighbouring floats in every time-major tensor.  The launches of consecutive steps follow each
// other in the stream; what a step hands to the next lies in memory: the spikes (the slab of the time-major spike
// tensor just written) and the integer states.
//
// The tensors of the interface are [N, C, T] with time innermost; a step touches one sample of every row.  The
// input is therefore copied to a time-major workspace ([T][N][C]) once, the steps read and write slabs of
// [N][C] floats, and the outputs are copied back at the end: four or five passes over the tensors against T
// passes over the weight matrix.
//
// The backward pass has the same shape (the reference's convention, utils/recurrent.py:83-112: the state carried
// between two steps is a constant): grad_dendrite[t] = surrogate(v[t], theta[t]) * (grad_spike[t] + grad_dendrite[t+1] R),
// the product taken with the transposed matrix so that both directions read weight rows along the summed index.
#include "common.h"
#include "tile.h"

namespace slayer {

constexpr int kStepWaves = 8;            // waves per workgroup: each takes an eighth of the sum over k
constexpr int kStepUnroll = 4;           // blocks of 16 k a wave keeps in flight
constexpr int kStepMaxC = 16384;         // 32-bit byte offsets into the weight matrix

typedef float step_f4 __attribute__((ext_vector_type(4)));

// dst[t][m] = src[m][t] (TO_TIME_MAJOR) or dst[m][t] = src[t][m]: 64 x 64 tiles through LDS, 256 threads.
template <bool TO_TIME_MAJOR>
__global__ __launch_bounds__(256) void time_major_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                         int64_t M, int T) {
    __shared__ float tile[64][65];
    const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
    const int64_t m0 = (int64_t)blockIdx.x * 64;
    const int t0 = blockIdx.y * 64;
    if (TO_TIME_MAJOR) {
#pragma unroll 4
        for (int r = y; r < 64; r += 4)
            tile[r][x] = (m0 + r < M && t0 + x < T) ? src[(m0 + r) * (int64_t)T + t0 + x] : 0.f;
        __syncthreads();
#pragma unroll 4
        for (int r = y; r < 64; r += 4)
            if (t0 + r < T && m0 + x < M) dst[(int64_t)(t0 + r) * M + m0 + x] = tile[x][r];
    } else {
#pragma unroll 4
        for (int r = y; r < 64; r += 4)
            tile[r][x] = (t0 + r < T && m0 + x < M) ? src[(int64_t)(t0 + r) * M + m0 + x] : 0.f;
        __syncthreads();
#pragma unroll 4
        for (int r = y; r < 64; r += 4)
            if (m0 + r < M && t0 + x < T) dst[(m0 + r) * (int64_t)T + t0 + x] = tile[x][r];
    }
}

// sum over k of w[c0 + 4q + i][k] * act[n0 + 16 s + j][k] for this thread's (s, q, j) = (tid / 64, lane / 16,
// lane % 16), i = 0 .. 3: valid in the threads tid < 64 NT, after one workgroup barrier.  Lane (kk, j) of a wave
// loads k = kb + 4 kk .. + 3 of weight row c0 + j and of sample row n0 + 16 s + j; element e of the two quads are
// the operands of one matrix product, so a block of 16 k is four of them.
template <int NT>
__device__ __forceinline__ float4 step_product(const float* __restrict__ w, const float* __restrict__ act, int N,
                                               int C, int n0, int c0, float4 (*red)[NT][kWave]) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kk = lane >> 4, j = lane & 15;
    const int w_rows = (C - c0) < 16 ? (C - c0) : 16;
    const int a_rows = (N - n0) < 16 * NT ? (N - n0) : 16 * NT;
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(w + (int64_t)c0 * C, (unsigned)(w_rows * C * 4));
    const __amdgpu_buffer_rsrc_t ar = make_rsrc(act + (int64_t)n0 * C, (unsigned)(a_rows * C * 4));
    const bool w_ok = j < w_rows;
    step_f4 acc[NT][2];
#pragma unroll
    for (int s = 0; s < NT; ++s) acc[s][0] = acc[s][1] = step_f4{0.f, 0.f, 0.f, 0.f};
    for (int kb = wave * 16; kb < C; kb += kStepWaves * 16 * kStepUnroll) {
        float4 wq[kStepUnroll], aq[kStepUnroll][NT];
#pragma unroll
        for (int u = 0; u < kStepUnroll; ++u) {
            const int k = kb + u * (kStepWaves * 16) + 4 * kk;
            const bool ok = k < C;                                       // C is a whole number of quads
            wq[u] = buf_load4<false>(wr, (ok && w_ok) ? (j * C + k) * 4 : kOutOfRange);
#pragma unroll
            for (int s = 0; s < NT; ++s)
                aq[u][s] = buf_load4<false>(ar, (ok && 16 * s + j < a_rows) ? ((16 * s + j) * C + k) * 4 : kOutOfRange);
        }
#pragma unroll
        for (int u = 0; u < kStepUnroll; ++u) {
#pragma unroll
            for (int s = 0; s < NT; ++s) {
                acc[s][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u].x, aq[u][s].x, acc[s][0], 0, 0, 0);
                acc[s][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u].y, aq[u][s].y, acc[s][1], 0, 0, 0);
                acc[s][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u].z, aq[u][s].z, acc[s][0], 0, 0, 0);
                acc[s][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u].w, aq[u][s].w, acc[s][1], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int s = 0; s < NT; ++s)
        red[wave][s][lane] = make_float4(acc[s][0][0] + acc[s][1][0], acc[s][0][1] + acc[s][1][1],
                                         acc[s][0][2] + acc[s][1][2], acc[s][0][3] + acc[s][1][3]);
    __syncthreads();
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    if (tid < NT * kWave) {
        const int s = tid >> 6;
#pragma unroll
        for (int wv = 0; wv < kStepWaves; ++wv) {
            const float4 v = red[wv][s][lane];
            sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
        }
    }
    return sum;
}

struct StepFwd {
    float *spk_t, *vol_t, *theta_t;                           // [T][N][C]; theta: ALIF only
    const float* z_t;                                         // [T][N][C]
    int* carried;                                             // [4][N][C]: current, voltage, threshold, refractory
    float *cur_last, *vol_last, *th_last, *ref_last;          // [N*C]; th / ref: ALIF only
    const float* rec;                                         // [C][C]
    const float *i_decay, *v_decay, *th_decay, *ref_decay, *i_state, *v_state, *th_state, *ref_state;
    int64_t n_id, n_vd, n_td, n_rd, n_is, n_vs, n_ts, n_rs;
    float w, inv_w, spike_thr, spike_scale, th_step_f;
    int base;
    int N, C, T;
    unsigned* range_flag;                                     // see raise_range_flag in tile.h
};

// One step of the layer for 16 neurons x 16 NT samples.  The neuron step is that of recurrent_fwd_kernel
// (recurrent.hip), state by state: each starts from the float32 value the previous step left and hands a float32
// value on, as between two one-step neuron calls.
template <bool ALIF, bool GRADED, bool POW2, int NT>
__global__ __launch_bounds__(kStepWaves * kWave) void recurrent_step_fwd_kernel(const StepFwd p, const int t) {
    __shared__ float4 red[kStepWaves][NT][kWave];
    const int C = p.C, N = p.N;
    const int c0 = blockIdx.x * 16, n0 = blockIdx.y * 16 * NT;
    const int64_t slab = (int64_t)N * C;
    float4 fb = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t > 0) fb = step_product<NT>(p.rec, p.spk_t + (t - 1) * slab, N, C, n0, c0, red);
    const int tid = threadIdx.x;
    if (tid >= NT * kWave) return;
    const int lane = tid & (kWave - 1);
    const int n = n0 + 16 * (tid >> 6) + (lane & 15), c = c0 + 4 * (lane >> 4);
    if (n >= N || c >= C) return;
    const int64_t m = (int64_t)n * C + c;                     // first of this thread's four neurons
    const float w = p.w, inv_w = p.inv_w;
    auto from = [&](int y) -> float { const float f = (float)y; return POW2 ? f * inv_w : f / w; };
    const float4 z4 = *reinterpret_cast<const float4*>(p.z_t + t * slab + m);
    const float zs[4] = {z4.x, z4.y, z4.z, z4.w}, fbs[4] = {fb.x, fb.y, fb.z, fb.w};
    int yc[4], yv[4], th[4] = {0, 0, 0, 0}, r[4] = {0, 0, 0, 0};
    if (t == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            yc[i] = trunc_i32(p.i_state[p.n_is == 1 ? 0 : m + i] * w);
            yv[i] = trunc_i32(p.v_state[p.n_vs == 1 ? 0 : m + i] * w);
            if (ALIF) {
                th[i] = trunc_i32(p.th_state[p.n_ts == 1 ? 0 : m + i] * w);
                r[i] = trunc_i32(p.ref_state[p.n_rs == 1 ? 0 : m + i] * w);
            }
        }
    } else {
        const int4 a = *reinterpret_cast<const int4*>(p.carried + m);
        const int4 b = *reinterpret_cast<const int4*>(p.carried + slab + m);
        yc[0] = a.x; yc[1] = a.y; yc[2] = a.z; yc[3] = a.w;
        yv[0] = b.x; yv[1] = b.y; yv[2] = b.z; yv[3] = b.w;
        if (ALIF) {
            const int4 d = *reinterpret_cast<const int4*>(p.carried + 2 * slab + m);
            const int4 e = *reinterpret_cast<const int4*>(p.carried + 3 * slab + m);
            th[0] = d.x; th[1] = d.y; th[2] = d.z; th[3] = d.w;
            r[0] = e.x; r[1] = e.y; r[2] = e.z; r[3] = e.w;
        }
    }
    unsigned acc_lif = 0u, acc_th = 0u;                       // range of the states, see range_bits in tile.h
    float so[4], vo[4], to[4], co[4], tho[4], ro[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int mi = 4096 - trunc_i32(rintf(p.i_decay[param_index(m + i, C, p.n_id)]));
        const int mv = 4096 - trunc_i32(rintf(p.v_decay[param_index(m + i, C, p.n_vd)]));
        int mt = 0, mr = 0;
        if (ALIF) {
            mt = 4096 - trunc_i32(rintf(p.th_decay[param_index(m + i, C, p.n_td)]));
            mr = 4096 - trunc_i32(rintf(p.ref_decay[param_index(m + i, C, p.n_rd)]));
        }
        if (t == 0) {
            check_multiplier(mi, p.range_flag); check_multiplier(mv, p.range_flag);
            if (ALIF) { check_multiplier(mt, p.range_flag); check_multiplier(mr, p.range_flag); }
            acc_lif |= ((unsigned)yc[i] + (1u << 30)) | ((unsigned)yv[i] + (1u << 30));
            acc_th |= ((unsigned)th[i] + (1u << 28)) | ((unsigned)r[i] + (1u << 28));
        }
        const float dend = zs[i] + fbs[i];
        yc[i] = add_sat(rs0_12(yc[i], mi), trunc_i32(w * dend));
        const float cur = from(yc[i]);
        yc[i] = trunc_i32(w * cur);
        const int yn = add_sat(rs0_12(yv[i], mv), yc[i]);
        acc_lif |= ((unsigned)yc[i] + (1u << 30)) | ((unsigned)yn + (1u << 30));
        const float vol = from(yn);
        float theta = p.spike_thr, thf = 0.f, rf = 0.f;
        if (ALIF) {
            r[i] = rs0_12(r[i], mr);
            th[i] = rs0_12(th[i] - p.base, mt) + p.base;
            acc_th |= ((unsigned)th[i] + (1u << 28)) | ((unsigned)r[i] + (1u << 28));
            thf = from(th[i]);
            rf = from(r[i]);
            theta = thf + rf;
        }
        const bool fired = vol >= theta;
        const float s = GRADED ? ((fired ? 1.0f : 0.0f) * vol) / p.spike_scale : (fired ? 1.0f : 0.0f);
        const bool spiked = s > 0.0f;                          // what the carried states see
        if (ALIF) {
            yv[i] = trunc_i32(w * vol);
            r[i] = trunc_i32((spiked ? rf + 2.0f * thf : rf) * w);
            th[i] = trunc_i32((spiked ? thf + p.th_step_f : thf) * w);
        } else {
            yv[i] = spiked ? 0 : trunc_i32(w * vol);
        }
        so[i] = s; vo[i] = vol; to[i] = theta; co[i] = cur; tho[i] = thf; ro[i] = rf;
    }
    if (range_exceeded(acc_lif, 30) || range_exceeded(acc_th, 28)) raise_range_flag(p.range_flag);
    *reinterpret_cast<float4*>(p.spk_t + t * slab + m) = make_float4(so[0], so[1], so[2], so[3]);
    *reinterpret_cast<float4*>(p.vol_t + t * slab + m) = make_float4(vo[0], vo[1], vo[2], vo[3]);
    if (ALIF) *reinterpret_cast<float4*>(p.theta_t + t * slab + m) = make_float4(to[0], to[1], to[2], to[3]);
    if (t == p.T - 1) {
        *reinterpret_cast<float4*>(p.cur_last + m) = make_float4(co[0], co[1], co[2], co[3]);
        *reinterpret_cast<float4*>(p.vol_last + m) = make_float4(vo[0], vo[1], vo[2], vo[3]);
        if (ALIF) {
            *reinterpret_cast<float4*>(p.th_last + m) = make_float4(tho[0], tho[1], tho[2], tho[3]);
            *reinterpret_cast<float4*>(p.ref_last + m) = make_float4(ro[0], ro[1], ro[2], ro[3]);
        }
    } else {
        *reinterpret_cast<int4*>(p.carried + m) = make_int4(yc[0], yc[1], yc[2], yc[3]);
        *reinterpret_cast<int4*>(p.carried + slab + m) = make_int4(yv[0], yv[1], yv[2], yv[3]);
        if (ALIF) {
            *reinterpret_cast<int4*>(p.carried + 2 * slab + m) = make_int4(th[0], th[1], th[2], th[3]);
            *reinterpret_cast<int4*>(p.carried + 3 * slab + m) = make_int4(r[0], r[1], r[2], r[3]);
        }
    }
}

struct StepBwd {
    float* gz_t;                                              // [T][N][C]: gradient of the dendrite input
    const float *g_t, *v_t, *theta_t;                         // [T][N][C]; theta: ALIF only
    const float* rec_t;                                       // [C][C]: the weight matrix transposed
    float spike_thr, tau, rho;
    int N, C, T;
};

template <bool THETA, bool GRADED, int NT>
__global__ __launch_bounds__(kStepWaves * kWave) void recurrent_step_bwd_kernel(const StepBwd p, const int t) {
    __shared__ float4 red[kStepWaves][NT][kWave];
    const int C = p.C, N = p.N;
    const int c0 = blockIdx.x * 16, n0 = blockIdx.y * 16 * NT;
    const int64_t slab = (int64_t)N * C;
    float4 carry = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t < p.T - 1) carry = step_product<NT>(p.rec_t, p.gz_t + (t + 1) * slab, N, C, n0, c0, red);
    const int tid = threadIdx.x;
    if (tid >= NT * kWave) return;
    const int lane = tid & (kWave - 1);
    const int n = n0 + 16 * (tid >> 6) + (lane & 15), c = c0 + 4 * (lane >> 4);
    if (n >= N || c >= C) return;
    const int64_t at = t * slab + (int64_t)n * C + c;
    const float4 g4 = *reinterpret_cast<const float4*>(p.g_t + at);
    const float4 v4 = *reinterpret_cast<const float4*>(p.v_t + at);
    float4 th4 = make_float4(p.spike_thr, p.spike_thr, p.spike_thr, p.spike_thr);
    if (THETA) th4 = *reinterpret_cast<const float4*>(p.theta_t + at);
    const float lead = (p.rho / 2.0f) / p.tau, inv_tau = 1.0f / p.tau;
    auto one = [&](float cy, float g, float v, float th) -> float {
        const float gs = cy + g;
        const float d = v - th;
        const float factor = GRADED ? p.rho * expf(fminf(d, 0.0f) * inv_tau) : lead * expf(-fabsf(d) * inv_tau);
        return factor * gs;
    };
    *reinterpret_cast<float4*>(p.gz_t + at) = make_float4(one(carry.x, g4.x, v4.x, th4.x), one(carry.y, g4.y, v4.y, th4.y),
                                                          one(carry.z, g4.z, v4.z, th4.z), one(carry.w, g4.w, v4.w, th4.w));
}

}  // namespace slayer

using namespace slayer;

namespace {

int check_step_sizes(int64_t N, int64_t C, int64_t T) {
    if (N < 0 || C < 0 || T < 0) return SLAYER_EINVAL;
    // whole quads of neurons, 32-bit byte offsets inside the weight matrix and a slab of [N][C] floats
    if ((C % 4) != 0 || C > kStepMaxC || N * C >= ((int64_t)1 << 29) || T > 0x7fffffffLL || N > 0x7fffffffLL ||
        (N + 63) / 64 > 65535 || (T + 63) / 64 > 65535)
        return SLAYER_ERANGE;
    return 0;
}

int64_t step_workspace_floats(int64_t N, int64_t C, int64_t T, int with_theta) {
    return (3 + (with_theta ? 1 : 0)) * N * C * T + 4 * N * C;
}

void launch_time_major(float* dst, const float* src, int64_t M, int64_t T, bool to_time_major, hipStream_t st) {
    // rows in the y dimension when there are more than the x dimension of a grid takes
    const dim3 grid((unsigned)((M + 63) / 64), (unsigned)((T + 63) / 64));
    if (to_time_major)
        hipLaunchKernelGGL((time_major_kernel<true>), grid, dim3(256), 0, st, dst, src, M, (int)T);
    else
        hipLaunchKernelGGL((time_major_kernel<false>), grid, dim3(256), 0, st, dst, src, M, (int)T);
}

// sample tiles per workgroup: as many as the batch needs, up to four
int step_sample_tiles(int64_t N) { return N <= 16 ? 1 : (N <= 32 ? 2 : 4); }

template <bool ALIF>
int launch_step_fwd(StepFwd p, int graded, int w_scale, hipStream_t st) {
    const int nt = step_sample_tiles(p.N);
    const dim3 grid((unsigned)((p.C + 15) / 16), (unsigned)((p.N + 16 * nt - 1) / (16 * nt)));
    const dim3 block(kStepWaves * kWave);
    const bool pow2 = is_pow2(w_scale);
    for (int t = 0; t < p.T; ++t) {
#define SLAYER_STEP(G, P, NT) hipLaunchKernelGGL((recurrent_step_fwd_kernel<ALIF, G, P, NT>), grid, block, 0, st, p, t)
#define SLAYER_STEP_NT(G, P)                                                                         \
        do {                                                                                             \
            if (nt == 1) SLAYER_STEP(G, P, 1); else if (nt == 2) SLAYER_STEP(G, P, 2); else SLAYER_STEP(G, P, 4); \
        } while (0)
        if (graded) { if (pow2) SLAYER_STEP_NT(true, true); else SLAYER_STEP_NT(true, false); }
        else { if (pow2) SLAYER_STEP_NT(false, true); else SLAYER_STEP_NT(false, false); }
#undef SLAYER_STEP_NT
#undef SLAYER_STEP
    }
    return (int)hipGetLastError();
}

// common part of the two forward entry points: copies in, the steps, copies out
template <bool ALIF>
int run_steps_fwd(StepFwd p, float* spk, float* vol, float* theta, const float* z, int graded, int w_scale,
                  float* workspace, int64_t workspace_floats, hipStream_t st) {
    const int64_t N = p.N, C = p.C, T = p.T, nct = N * C * T;
    if (workspace_floats < step_workspace_floats(N, C, T, ALIF ? 1 : 0)) return SLAYER_ERANGE;
    if (!aligned16(workspace) || !aligned16(p.rec) || !aligned16(p.cur_last) || !aligned16(p.vol_last) ||
        (ALIF && (!aligned16(p.th_last) || !aligned16(p.ref_last))))
        return SLAYER_ERANGE;
    float* zt = workspace;
    p.z_t = zt;
    p.spk_t = workspace + nct;
    p.vol_t = workspace + 2 * nct;
    p.theta_t = ALIF ? workspace + 3 * nct : nullptr;
    p.carried = reinterpret_cast<int*>(workspace + (3 + (ALIF ? 1 : 0)) * nct);
    launch_time_major(zt, z, N * C, T, true, st);
    if (int e = launch_step_fwd<ALIF>(p, graded, w_scale, st)) return e;
    launch_time_major(spk, p.spk_t, N * C, T, false, st);
    launch_time_major(vol, p.vol_t, N * C, T, false, st);
    if (ALIF) launch_time_major(theta, p.theta_t, N * C, T, false, st);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int64_t slayer_recurrent_steps_workspace(int64_t N, int64_t C, int64_t T, int with_theta) {
    if (int e = check_step_sizes(N, C, T)) return e;
    return step_workspace_floats(N, C, T, with_theta);
}

extern "C" int slayer_cuba_recurrent_steps_fwd(float* spk_out, float* vol_out, float* cur_last_out, float* vol_last_out,
                                               const float* z, const float* rec,
                                               const float* i_decay, const float* v_decay,
                                               const float* i_state, const float* v_state,
                                               float spike_threshold, int graded, float spike_scale, int w_scale,
                                               int64_t N, int64_t C, int64_t num_i_decays, int64_t num_v_decays,
                                               int64_t num_i_states, int64_t num_v_states, int64_t T,
                                               float* workspace, int64_t workspace_floats, void* stream) {
    if (int e = check_step_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!spk_out || !vol_out || !cur_last_out || !vol_last_out || !z || !rec || !i_decay || !v_decay || !i_state ||
        !v_state || !workspace)
        return SLAYER_ENULL;
    if (int e = check_params(N * C, C, num_i_decays)) return e;
    if (int e = check_params(N * C, C, num_v_decays)) return e;
    if (int e = check_states(N * C, num_i_states)) return e;
    if (int e = check_states(N * C, num_v_states)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    StepFwd p{};
    p.cur_last = cur_last_out; p.vol_last = vol_last_out;
    p.rec = rec;
    p.i_decay = i_decay; p.v_decay = v_decay; p.i_state = i_state; p.v_state = v_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_is = num_i_states; p.n_vs = num_v_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / (float)w_scale;
    p.spike_thr = spike_threshold; p.spike_scale = spike_scale;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_device();
    return run_steps_fwd<false>(p, spk_out, vol_out, nullptr, z, graded, w_scale, workspace, workspace_floats,
                                (hipStream_t)stream);
}

extern "C" int slayer_alif_recurrent_steps_fwd(float* spk_out, float* vol_out, float* theta_out,
                                               float* cur_last_out, float* vol_last_out, float* th_last_out,
                                               float* ref_last_out, const float* z, const float* rec,
                                               const float* i_decay, const float* v_decay, const float* th_decay,
                                               const float* ref_decay, const float* i_state, const float* v_state,
                                               const float* th_state, const float* ref_state,
                                               float th_step, int64_t th0_scaled, int graded, float spike_scale,
                                               int w_scale, int64_t N, int64_t C,
                                               int64_t num_i_decays, int64_t num_v_decays, int64_t num_th_decays,
                                               int64_t num_ref_decays, int64_t num_i_states, int64_t num_v_states,
                                               int64_t num_th_states, int64_t num_ref_states, int64_t T,
                                               float* workspace, int64_t workspace_floats, void* stream) {
    if (int e = check_step_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!spk_out || !vol_out || !theta_out || !cur_last_out || !vol_last_out || !th_last_out || !ref_last_out || !z ||
        !rec || !i_decay || !v_decay || !th_decay || !ref_decay || !i_state || !v_state || !th_state || !ref_state ||
        !workspace)
        return SLAYER_ENULL;
    for (int64_t n : {num_i_decays, num_v_decays, num_th_decays, num_ref_decays})
        if (int e = check_params(N * C, C, n)) return e;
    for (int64_t n : {num_i_states, num_v_states, num_th_states, num_ref_states})
        if (int e = check_states(N * C, n)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    if (th0_scaled > 0x7fffffffLL || th0_scaled < -0x7fffffffLL) return SLAYER_ERANGE;
    StepFwd p{};
    p.cur_last = cur_last_out; p.vol_last = vol_last_out; p.th_last = th_last_out; p.ref_last = ref_last_out;
    p.rec = rec;
    p.i_decay = i_decay; p.v_decay = v_decay; p.th_decay = th_decay; p.ref_decay = ref_decay;
    p.i_state = i_state; p.v_state = v_state; p.th_state = th_state; p.ref_state = ref_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_td = num_th_decays; p.n_rd = num_ref_decays;
    p.n_is = num_i_states; p.n_vs = num_v_states; p.n_ts = num_th_states; p.n_rs = num_ref_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / (float)w_scale;
    p.spike_scale = spike_scale; p.th_step_f = th_step;
    p.base = (int)th0_scaled;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_for_threshold(0, th0_scaled);
    return run_steps_fwd<true>(p, spk_out, vol_out, theta_out, z, graded, w_scale, workspace, workspace_floats,
                               (hipStream_t)stream);
}

extern "C" int slayer_recurrent_steps_bwd(float* grad_z, const float* grad_spikes, const float* voltage,
                                          const float* theta, const float* rec_t, float spike_threshold,
                                          float tau_rho, float scale_rho, int graded, int64_t N, int64_t C, int64_t T,
                                          float* workspace, int64_t workspace_floats, void* stream) {
    if (int e = check_step_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!grad_z || !grad_spikes || !voltage || !rec_t || !workspace) return SLAYER_ENULL;
    if (workspace_floats < step_workspace_floats(N, C, T, theta ? 1 : 0)) return SLAYER_ERANGE;
    if (!aligned16(workspace) || !aligned16(rec_t)) return SLAYER_ERANGE;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nct = N * C * T;
    float* g_t = workspace;
    float* v_t = workspace + nct;
    float* gz_t = workspace + 2 * nct;
    float* th_t = theta ? workspace + 3 * nct : nullptr;
    launch_time_major(g_t, grad_spikes, N * C, T, true, st);
    launch_time_major(v_t, voltage, N * C, T, true, st);
    if (theta) launch_time_major(th_t, theta, N * C, T, true, st);
    StepBwd p{};
    p.gz_t = gz_t; p.g_t = g_t; p.v_t = v_t; p.theta_t = th_t; p.rec_t = rec_t;
    p.spike_thr = spike_threshold; p.tau = tau_rho; p.rho = scale_rho;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    const int nt = step_sample_tiles(N);
    const dim3 grid((unsigned)((C + 15) / 16), (unsigned)((N + 16 * nt - 1) / (16 * nt)));
    const dim3 block(kStepWaves * kWave);
    for (int t = (int)T - 1; t >= 0; --t) {
#define SLAYER_SB(TH, G, NT) hipLaunchKernelGGL((recurrent_step_bwd_kernel<TH, G, NT>), grid, block, 0, st, p, t)
#define SLAYER_SB_NT(TH, G)                                                                            \
        do {                                                                                           \
            if (nt == 1) SLAYER_SB(TH, G, 1); else if (nt == 2) SLAYER_SB(TH, G, 2); else SLAYER_SB(TH, G, 4); \
        } while (0)
        if (theta) { if (graded) SLAYER_SB_NT(true, true); else SLAYER_SB_NT(true, false); }
        else { if (graded) SLAYER_SB_NT(false, true); else SLAYER_SB_NT(false, false); }
#undef SLAYER_SB_NT
#undef SLAYER_SB
    }
    launch_time_major(grad_z, gz_t, N * C, T, false, st);
    return (int)hipGetLastError();
}
