// Recurrent layer of CUBA or ALIF neurons, one launch per time step: the form for layers too wide for one
// workgroup per sample (recurrent.hip), where re-reading the weight matrix per sample is what a step costs.
//
//   feedback[t] = R s[t-1];  s[t] = neuron(z[t] + feedback[t])          (utils/recurrent.py:45-112 in the reference)
//
// A step is one product of the [C x C] weight matrix with the [N x C] spikes of the previous step -- the matrix
// is read once per step for the whole batch -- followed by one neuron step of every (sample, neuron).  A workgroup
// owns 16 neurons for up to 64 samples: its four waves each take a quarter of the sum over the presynaptic
// neurons on the matrix cores (v_mfma_f32_16x16x4_f32: float32 operands and accumulation; the products of a 0/1
// spike are exact, and so is every partial sum of quantised weights), the partial sums meet in LDS, and the first
// waves run the neuron step on the result: lane (q, j) of a 16 x 16 result tile holds neurons 4q .. 4q+3 of sample
// j, a quad of neighbouring floats in every time-major tensor.  The launches of consecutive steps follow each
// other in the stream; what a step hands to the next lies in memory: the spikes (the slab of the time-major spike
// tensor just written) and the integer states.
//
// Both operands of the product are read in the order the matrix cores want them: the weight matrix is re-packed
// once per call (pack_weights_kernel: per tile of 16 neurons and block of 16 k, the 64 quads of the 64 lanes one
// after the other -- a wave-wide load is one contiguous kilobyte instead of sixteen rows a power of two apart), and
// a step leaves its spikes in the same order next to the time-major slab (the quad a lane of the neuron step holds
// is the quad the same lane of the next step's product loads).
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

#ifndef SLAYER_STEP_WAVES
#define SLAYER_STEP_WAVES 4
#endif
#ifndef SLAYER_STEP_QUADS
#define SLAYER_STEP_QUADS 16
#endif
constexpr int kStepWaves = SLAYER_STEP_WAVES;   // waves per workgroup: each takes its share of the sum over k
constexpr int kStepQuads = SLAYER_STEP_QUADS;   // operand quads (weights and activations) a lane keeps in flight
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

// Packed operands.  Weights: wp[tile][kb][lane] (float4) = w[16 tile + j][16 kb + 4 kk .. + 3] for lane = 16 kk + j,
// zero beyond the matrix.  Activations: ap[kb][s][lane] (float4) = act[16 s + j][16 kb + 4 kk .. + 3], zero beyond
// the batch and the layer; S = sample tiles, a multiple of the tiles a workgroup takes.
template <bool TRANSPOSED>
__global__ __launch_bounds__(kWave) void pack_weights_kernel(float4* __restrict__ wp, const float* __restrict__ w, int C,
                                                             int KB) {
    const int lane = threadIdx.x, kk = lane >> 4, j = lane & 15;
    const int kb = blockIdx.x, tile = blockIdx.y;
    const int row = 16 * tile + j, k = 16 * kb + 4 * kk;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const bool ok = row < C && k + e < C;
        v[e] = ok ? (TRANSPOSED ? w[(int64_t)(k + e) * C + row] : w[(int64_t)row * C + k + e]) : 0.f;
    }
    wp[((int64_t)tile * KB + kb) * kWave + lane] = make_float4(v[0], v[1], v[2], v[3]);
}

// sum over k of w[c0 + 4q + i][k] * act[n0 + 16 s + j][k] for this thread's (s, q, j) = (tid / 64, lane / 16,
// lane % 16), i = 0 .. 3: valid in the threads tid < 64 NT, after one workgroup barrier.  Element e of a lane's two
// quads are the operands of one matrix product, so a block of 16 k is four of them; wave v takes blocks v, v + 4, ...
template <int NT>
__device__ __forceinline__ float4 step_product(const float4* __restrict__ wp, const float4* __restrict__ ap, int KB,
                                               int S, int s0, float4 (*red)[NT][kWave]) {
    constexpr int kStepUnroll = kStepQuads / (1 + NT) < 2 ? 2 : kStepQuads / (1 + NT);
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    step_f4 acc[NT][2];
#pragma unroll
    for (int s = 0; s < NT; ++s) acc[s][0] = acc[s][1] = step_f4{0.f, 0.f, 0.f, 0.f};
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int kb0 = wave; kb0 < KB; kb0 += kStepWaves * kStepUnroll) {
        float4 wq[kStepUnroll], aq[kStepUnroll][NT];
#pragma unroll
        for (int u = 0; u < kStepUnroll; ++u) {
            const int kb = kb0 + u * kStepWaves;
            const bool ok = kb < KB;                                     // the same for the whole wave
            const int at = ok ? kb : kb0;
            wq[u] = wp[(int64_t)at * kWave + lane];
            if (!ok) wq[u] = zero;
#pragma unroll
            for (int s = 0; s < NT; ++s) aq[u][s] = ap[((int64_t)at * S + s0 + s) * kWave + lane];
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
    float4 sum = zero;
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
    const float4* rec_packed;                                 // see pack_weights_kernel
    float4* spk_packed;                                       // two buffers of [KB][S][64] quads, written in turn
    int KB, S;                                                // blocks of 16 neurons, sample tiles
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
    const int s0 = blockIdx.y * NT;
    const int64_t packed = (int64_t)p.KB * p.S * kWave;       // quads of one buffer of packed spikes
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const bool worker = tid < NT * kWave;                     // the threads that run the neuron step
    const int n = n0 + 16 * (tid >> 6) + (lane & 15), c = c0 + 4 * (lane >> 4);
    const bool valid = worker && n < N && c < C;
    const int64_t m = valid ? (int64_t)n * C + c : 0;         // first of this thread's four neurons
    const float w = p.w, inv_w = p.inv_w;
    auto from = [&](int y) -> float { const float f = (float)y; return POW2 ? f * inv_w : f / w; };
    // what the neuron step reads is on its way while the product runs
    float4 z4 = make_float4(0.f, 0.f, 0.f, 0.f);
    int yc[4] = {0, 0, 0, 0}, yv[4] = {0, 0, 0, 0}, th[4] = {0, 0, 0, 0}, r[4] = {0, 0, 0, 0};
    int mi[4] = {0, 0, 0, 0}, mv[4] = {0, 0, 0, 0}, mt[4] = {0, 0, 0, 0}, mr[4] = {0, 0, 0, 0};
    if (valid) {
        z4 = *reinterpret_cast<const float4*>(p.z_t + t * slab + m);
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
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // one decay for the layer or one per neuron (neuron c + i of its sample)
            mi[i] = 4096 - trunc_i32(rintf(p.i_decay[p.n_id == 1 ? 0 : c + i]));
            mv[i] = 4096 - trunc_i32(rintf(p.v_decay[p.n_vd == 1 ? 0 : c + i]));
            if (ALIF) {
                mt[i] = 4096 - trunc_i32(rintf(p.th_decay[p.n_td == 1 ? 0 : c + i]));
                mr[i] = 4096 - trunc_i32(rintf(p.ref_decay[p.n_rd == 1 ? 0 : c + i]));
            }
        }
    }
    float4 fb = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t > 0)
        fb = step_product<NT>(p.rec_packed + (int64_t)blockIdx.x * p.KB * kWave, p.spk_packed + ((t - 1) & 1) * packed,
                              p.KB, p.S, s0, red);
    if (!worker) return;
    // where the next step's product finds this thread's four spikes
    float4* hand_on = p.spk_packed + (t & 1) * packed + ((int64_t)blockIdx.x * p.S + s0 + (tid >> 6)) * kWave + lane;
    if (!valid) {
        *hand_on = make_float4(0.f, 0.f, 0.f, 0.f);
        return;
    }
    const float zs[4] = {z4.x, z4.y, z4.z, z4.w}, fbs[4] = {fb.x, fb.y, fb.z, fb.w};
    unsigned acc_lif = 0u, acc_th = 0u;                       // range of the states, see range_bits in tile.h
    float so[4], vo[4], to[4], co[4], tho[4], ro[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (t == 0) {
            check_multiplier(mi[i], p.range_flag); check_multiplier(mv[i], p.range_flag);
            if (ALIF) { check_multiplier(mt[i], p.range_flag); check_multiplier(mr[i], p.range_flag); }
            acc_lif |= ((unsigned)yc[i] + (1u << 30)) | ((unsigned)yv[i] + (1u << 30));
            acc_th |= ((unsigned)th[i] + (1u << 28)) | ((unsigned)r[i] + (1u << 28));
        }
        const float dend = zs[i] + fbs[i];
        yc[i] = add_sat(rs0_12(yc[i], mi[i]), trunc_i32(w * dend));
        const float cur = from(yc[i]);
        yc[i] = trunc_i32(w * cur);
        const int yn = add_sat(rs0_12(yv[i], mv[i]), yc[i]);
        acc_lif |= ((unsigned)yc[i] + (1u << 30)) | ((unsigned)yn + (1u << 30));
        const float vol = from(yn);
        float theta = p.spike_thr, thf = 0.f, rf = 0.f;
        if (ALIF) {
            r[i] = rs0_12(r[i], mr[i]);
            th[i] = rs0_12(th[i] - p.base, mt[i]) + p.base;
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
    *hand_on = make_float4(so[0], so[1], so[2], so[3]);
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
    const float4* rec_packed;                                 // the transposed matrix, see pack_weights_kernel
    float4* gz_packed;                                        // two buffers of [KB][S][64] quads, written in turn
    int KB, S;
    float spike_thr, tau, rho;
    int N, C, T;
};

template <bool THETA, bool GRADED, int NT>
__global__ __launch_bounds__(kStepWaves * kWave) void recurrent_step_bwd_kernel(const StepBwd p, const int t) {
    __shared__ float4 red[kStepWaves][NT][kWave];
    const int C = p.C, N = p.N;
    const int c0 = blockIdx.x * 16, n0 = blockIdx.y * 16 * NT;
    const int64_t slab = (int64_t)N * C;
    const int s0 = blockIdx.y * NT;
    const int64_t packed = (int64_t)p.KB * p.S * kWave;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const bool worker = tid < NT * kWave;
    const int n = n0 + 16 * (tid >> 6) + (lane & 15), c = c0 + 4 * (lane >> 4);
    const bool valid = worker && n < N && c < C;
    const int64_t at = valid ? t * slab + (int64_t)n * C + c : 0;
    // what the step reads is on its way while the product runs
    float4 g4 = make_float4(0.f, 0.f, 0.f, 0.f), v4 = g4;
    float4 th4 = make_float4(p.spike_thr, p.spike_thr, p.spike_thr, p.spike_thr);
    if (valid) {
        g4 = *reinterpret_cast<const float4*>(p.g_t + at);
        v4 = *reinterpret_cast<const float4*>(p.v_t + at);
        if (THETA) th4 = *reinterpret_cast<const float4*>(p.theta_t + at);
    }
    float4 carry = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t < p.T - 1)
        carry = step_product<NT>(p.rec_packed + (int64_t)blockIdx.x * p.KB * kWave, p.gz_packed + ((t + 1) & 1) * packed,
                                 p.KB, p.S, s0, red);
    if (!worker) return;
    float4* hand_on = p.gz_packed + (t & 1) * packed + ((int64_t)blockIdx.x * p.S + s0 + (tid >> 6)) * kWave + lane;
    if (!valid) {
        *hand_on = make_float4(0.f, 0.f, 0.f, 0.f);
        return;
    }
    const float lead = (p.rho / 2.0f) / p.tau, inv_tau = 1.0f / p.tau;
    auto one = [&](float cy, float g, float v, float th) -> float {
        const float gs = cy + g;
        const float d = v - th;
        const float factor = GRADED ? p.rho * expf(fminf(d, 0.0f) * inv_tau) : lead * expf(-fabsf(d) * inv_tau);
        return factor * gs;
    };
    const float4 gd = make_float4(one(carry.x, g4.x, v4.x, th4.x), one(carry.y, g4.y, v4.y, th4.y),
                                  one(carry.z, g4.z, v4.z, th4.z), one(carry.w, g4.w, v4.w, th4.w));
    *reinterpret_cast<float4*>(p.gz_t + at) = gd;
    *hand_on = gd;
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

// sample tiles per workgroup (1, 2 or 4): one while that still leaves the chip with no more than one workgroup per
// compute unit (the workgroups of one neuron tile share their weights through the L2), more for larger problems
int step_sample_tiles(int64_t N, int64_t C) {
    const int64_t tiles = (N + 15) / 16, KB = (C + 15) / 16;
    int nt = 1;
    while (nt < 4 && nt < tiles && KB * ((tiles + nt - 1) / nt) > 256) nt *= 2;
    return nt;
}

// what the workspace holds: the time-major tensors, the states between two steps, the packed weights and two
// buffers of packed activations
struct StepLayout {
    int64_t nct, carried, KB, S, weights, packed;             // floats, except KB (blocks of 16) and S (sample tiles)
    int64_t total(int tensors) const { return tensors * nct + carried + weights + 2 * packed; }
};
StepLayout step_layout(int64_t N, int64_t C, int64_t T) {
    StepLayout l;
    const int nt = step_sample_tiles(N, C);
    l.nct = N * C * T;
    l.carried = 4 * N * C;
    l.KB = (C + 15) / 16;
    l.S = (N + 16 * nt - 1) / (16 * nt) * nt;
    l.weights = l.KB * l.KB * 256;
    l.packed = l.KB * l.S * 256;
    return l;
}

int64_t step_workspace_floats(int64_t N, int64_t C, int64_t T, int with_theta) {
    return step_layout(N, C, T).total(3 + (with_theta ? 1 : 0));
}

void launch_pack_weights(float* packed, const float* w, int64_t C, bool transposed, hipStream_t st) {
    const int KB = (int)((C + 15) / 16);
    const dim3 grid((unsigned)KB, (unsigned)KB);
    if (transposed)
        hipLaunchKernelGGL((pack_weights_kernel<true>), grid, dim3(kWave), 0, st, reinterpret_cast<float4*>(packed), w,
                           (int)C, KB);
    else
        hipLaunchKernelGGL((pack_weights_kernel<false>), grid, dim3(kWave), 0, st, reinterpret_cast<float4*>(packed), w,
                           (int)C, KB);
}

void launch_time_major(float* dst, const float* src, int64_t M, int64_t T, bool to_time_major, hipStream_t st) {
    // rows in the y dimension when there are more than the x dimension of a grid takes
    const dim3 grid((unsigned)((M + 63) / 64), (unsigned)((T + 63) / 64));
    if (to_time_major)
        hipLaunchKernelGGL((time_major_kernel<true>), grid, dim3(256), 0, st, dst, src, M, (int)T);
    else
        hipLaunchKernelGGL((time_major_kernel<false>), grid, dim3(256), 0, st, dst, src, M, (int)T);
}

template <bool ALIF>
int launch_step_fwd(StepFwd p, int graded, int w_scale, hipStream_t st) {
    const int nt = step_sample_tiles(p.N, p.C);
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
int run_steps_fwd(StepFwd p, float* spk, float* vol, float* theta, const float* z, const float* rec, int graded, int w_scale,
                  float* workspace, int64_t workspace_floats, hipStream_t st) {
    const int64_t N = p.N, C = p.C, T = p.T;
    const StepLayout l = step_layout(N, C, T);
    const int64_t nct = l.nct;
    const int tensors = 3 + (ALIF ? 1 : 0);
    if (workspace_floats < l.total(tensors)) return SLAYER_ERANGE;
    if (!aligned16(workspace) || !aligned16(p.cur_last) || !aligned16(p.vol_last) ||
        (ALIF && (!aligned16(p.th_last) || !aligned16(p.ref_last))))
        return SLAYER_ERANGE;
    float* zt = workspace;
    p.z_t = zt;
    p.spk_t = workspace + nct;
    p.vol_t = workspace + 2 * nct;
    p.theta_t = ALIF ? workspace + 3 * nct : nullptr;
    p.carried = reinterpret_cast<int*>(workspace + tensors * nct);
    float* wp = workspace + tensors * nct + l.carried;
    p.rec_packed = reinterpret_cast<const float4*>(wp);
    p.spk_packed = reinterpret_cast<float4*>(wp + l.weights);
    p.KB = (int)l.KB; p.S = (int)l.S;
    launch_pack_weights(wp, rec, C, false, st);
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
    for (int64_t n : {num_i_decays, num_v_decays})
        if (n != 1 && n != C) return SLAYER_EINVAL;
    if (int e = check_states(N * C, num_i_states)) return e;
    if (int e = check_states(N * C, num_v_states)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    StepFwd p{};
    p.cur_last = cur_last_out; p.vol_last = vol_last_out;
    p.i_decay = i_decay; p.v_decay = v_decay; p.i_state = i_state; p.v_state = v_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_is = num_i_states; p.n_vs = num_v_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / (float)w_scale;
    p.spike_thr = spike_threshold; p.spike_scale = spike_scale;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_device();
    return run_steps_fwd<false>(p, spk_out, vol_out, nullptr, z, rec, graded, w_scale, workspace, workspace_floats,
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
        if (n != 1 && n != C) return SLAYER_EINVAL;
    for (int64_t n : {num_i_states, num_v_states, num_th_states, num_ref_states})
        if (int e = check_states(N * C, n)) return e;
    if (w_scale == 0 || (graded && spike_scale == 0.0f)) return SLAYER_EINVAL;
    if (th0_scaled > 0x7fffffffLL || th0_scaled < -0x7fffffffLL) return SLAYER_ERANGE;
    StepFwd p{};
    p.cur_last = cur_last_out; p.vol_last = vol_last_out; p.th_last = th_last_out; p.ref_last = ref_last_out;
    p.i_decay = i_decay; p.v_decay = v_decay; p.th_decay = th_decay; p.ref_decay = ref_decay;
    p.i_state = i_state; p.v_state = v_state; p.th_state = th_state; p.ref_state = ref_state;
    p.n_id = num_i_decays; p.n_vd = num_v_decays; p.n_td = num_th_decays; p.n_rd = num_ref_decays;
    p.n_is = num_i_states; p.n_vs = num_v_states; p.n_ts = num_th_states; p.n_rs = num_ref_states;
    p.w = (float)w_scale; p.inv_w = 1.0f / (float)w_scale;
    p.spike_scale = spike_scale; p.th_step_f = th_step;
    p.base = (int)th0_scaled;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    p.range_flag = range_flag_for_threshold(0, th0_scaled);
    return run_steps_fwd<true>(p, spk_out, vol_out, theta_out, z, rec, graded, w_scale, workspace, workspace_floats,
                               (hipStream_t)stream);
}

extern "C" int slayer_recurrent_steps_bwd(float* grad_z, const float* grad_spikes, const float* voltage,
                                          const float* theta, const float* rec, float spike_threshold,
                                          float tau_rho, float scale_rho, int graded, int64_t N, int64_t C, int64_t T,
                                          float* workspace, int64_t workspace_floats, void* stream) {
    if (int e = check_step_sizes(N, C, T)) return e;
    if (N == 0 || C == 0 || T == 0) return 0;
    if (!grad_z || !grad_spikes || !voltage || !rec || !workspace) return SLAYER_ENULL;
    const StepLayout l = step_layout(N, C, T);
    const int tensors = 3 + (theta ? 1 : 0);
    if (workspace_floats < l.total(tensors)) return SLAYER_ERANGE;
    if (!aligned16(workspace)) return SLAYER_ERANGE;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nct = l.nct;
    float* g_t = workspace;
    float* v_t = workspace + nct;
    float* gz_t = workspace + 2 * nct;
    float* th_t = theta ? workspace + 3 * nct : nullptr;
    float* wp = workspace + tensors * nct + l.carried;
    launch_pack_weights(wp, rec, C, true, st);
    launch_time_major(g_t, grad_spikes, N * C, T, true, st);
    launch_time_major(v_t, voltage, N * C, T, true, st);
    if (theta) launch_time_major(th_t, theta, N * C, T, true, st);
    StepBwd p{};
    p.gz_t = gz_t; p.g_t = g_t; p.v_t = v_t; p.theta_t = th_t;
    p.rec_packed = reinterpret_cast<const float4*>(wp);
    p.gz_packed = reinterpret_cast<float4*>(wp + l.weights);
    p.KB = (int)l.KB; p.S = (int)l.S;
    p.spike_thr = spike_threshold; p.tau = tau_rho; p.rho = scale_rho;
    p.N = (int)N; p.C = (int)C; p.T = (int)T;
    const int nt = step_sample_tiles(N, C);
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
