// Convolution synapse on time-innermost tensors.
//
// A SLAYER conv synapse is a spatial convolution applied at every time step (synapse/layer.py:297-323 in the
// reference: F.conv3d with a kernel of (kh, kw, 1) on [N, C, H, W, T]).  A library conv3d wants channels last: it
// transposes the tensor there and back around its kernel, three passes over tensors whose innermost axis is already
// the one the neuron kernels walk.  Here the tensors stay as they are: for an output pixel (n, h, w) and a tile of
// 64 time steps the [Co x 64] result is the [Co x K] weight matrix (K = Ci * kh * kw) times the [K x 64] matrix
// whose row k is the input row of tap k -- 64 consecutive floats of the input as it lies in memory.  One wavefront
// takes 16 output channels x 64 steps of one pixel at a time on the matrix cores (v_mfma_f32_16x16x4_f32: float32
// operands, float32 accumulation) and walks along the image row, so neighbouring pixels find their shared input
// rows in the cache; a wave-wide load is four input rows of 256 bytes, a wave-wide store four output rows.
//
// Lane (kk, j) = (lane / 16, lane % 16) loads steps 4j .. 4j+3 of tap 4g + kk for tap group g: element e of that
// quad is the B operand of the e-th of four matrix products, whose column j stands for step 4j + e; lane (q, j) of a
// result then holds output channels 4q .. 4q+3 of step 4j + e, i.e. over e a quad of consecutive steps per channel.
#include "common.h"
#include "tile.h"

namespace slayer {

typedef float syn_f4 __attribute__((ext_vector_type(4)));

constexpr int kSynTile = 64;            // time steps per tile
constexpr int kSynWaves = 4;            // waves per workgroup: same output channels, same image row, different tiles

struct SynapseConv {
    float* out;
    const float* in;
    const float* weight;                // [Co][Ci][kh][kw]
    int N, Ci, Co, H, W, Ho, Wo, T;
    int kh, kw, sh, sw, ph, pw, dh, dw;
    int K, KG;                          // taps, groups of four taps
    int ttiles, wsplit;                 // tiles of 64 steps per row, pieces an image row is cut into
};

// LDS: the weights of this workgroup's 16 output channels, tap-major (row k holds the 16 channels), and per tap the
// offset of its input row relative to the pixel's own position and its (row, column) displacement in the image.
template <bool STREAM>
__global__ __launch_bounds__(kSynWaves * kWave) void synapse_conv_kernel(const SynapseConv p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int Kp = p.KG * 4;
    float* wt = lds;                                    // [Kp][16]
    int* tap_off = reinterpret_cast<int*>(lds + Kp * 16);   // [Kp] bytes
    int* tap_dy = tap_off + Kp;                         // [Kp]
    int* tap_dx = tap_dy + Kp;                          // [Kp]

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup -> (batch entry, block of 16 output channels, output row, piece of the row, group of time tiles)
    int b = blockIdx.x;
    const int tgroups = (p.ttiles + kSynWaves - 1) / kSynWaves;
    const int tg = b % tgroups; b /= tgroups;
    const int piece = b % p.wsplit; b /= p.wsplit;
    const int ho = b % p.Ho; b /= p.Ho;
    const int cob = b % ((p.Co + 15) / 16);
    const int n = b / ((p.Co + 15) / 16);
    const int co0 = cob * 16;

    for (int i = tid; i < Kp * 16; i += kSynWaves * kWave) {
        const int k = i >> 4, m = i & 15;
        wt[i] = (k < p.K && co0 + m < p.Co) ? p.weight[(int64_t)(co0 + m) * p.K + k] : 0.0f;
    }
    for (int k = tid; k < Kp; k += kSynWaves * kWave) {
        const int ci = k / (p.kh * p.kw), r = k - ci * (p.kh * p.kw), y = r / p.kw, x = r - y * p.kw;
        const int dy = y * p.dh - p.ph, dx = x * p.dw - p.pw;
        tap_dy[k] = k < p.K ? dy : (1 << 28);                            // a tap that does not exist: always outside
        tap_dx[k] = dx;
        tap_off[k] = (((ci * p.H + dy) * p.W) + dx) * p.T * 4;
    }
    __syncthreads();

    const int tile = tg * kSynWaves + wave;
    if (tile >= p.ttiles) return;
    const int t0 = tile * kSynTile;
    const int kk = lane >> 4, j = lane & 15;
    const bool t_ok = t0 + 4 * j < p.T;                                  // T is a whole number of quads
    const int hin = ho * p.sh;                                           // image row of tap (0, 0) before padding
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho * p.Wo * p.T;
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(p.out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));

    const int per = (p.Wo + p.wsplit - 1) / p.wsplit;
    const int w_lo = piece * per, w_hi = (w_lo + per) < p.Wo ? (w_lo + per) : p.Wo;
    for (int wo = w_lo; wo < w_hi; ++wo) {
        const int win = wo * p.sw;
        const int pix = ((hin * p.W) + win) * p.T * 4 + (t0 + 4 * j) * 4;    // byte offset of tap (0,0,0)'s quad
        syn_f4 acc[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = syn_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
        for (int g = 0; g < p.KG; ++g) {
            const int k = 4 * g + kk;
            const int yy = hin + tap_dy[k], xx = win + tap_dx[k];
            const bool ok = t_ok && (unsigned)yy < (unsigned)p.H && (unsigned)xx < (unsigned)p.W;
            const float4 q = buf_load4<false>(src, ok ? pix + tap_off[k] : kOutOfRange);
            const float a = wt[k * 16 + j];
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, q.x, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, q.y, acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, q.z, acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, q.w, acc[3], 0, 0, 0);
        }
        // lane (kk, j): output channels co0 + 4 kk + i, steps t0 + 4 j + e
        const int opix = ((ho * p.Wo) + wo) * p.T * 4 + (t0 + 4 * j) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int co = co0 + 4 * kk + i;
            const bool ok = t_ok && co < p.Co;
            buf_store4<STREAM>(dst, ok ? co * (p.Ho * p.Wo * p.T * 4) + opix : kOutOfRange,
                               make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]));
        }
    }
}

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_conv_synapse(float* out, const float* in, const float* weight,
                                   int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                                   int64_t kh, int64_t kw, int64_t stride_h, int64_t stride_w,
                                   int64_t pad_h, int64_t pad_w, int64_t dil_h, int64_t dil_w, void* stream) {
    if (N < 0 || Ci < 1 || Co < 1 || H < 1 || W < 1 || T < 0 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
        pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1)
        return SLAYER_EINVAL;
    const int64_t Ho = (H + 2 * pad_h - dil_h * (kh - 1) - 1) / stride_h + 1;
    const int64_t Wo = (W + 2 * pad_w - dil_w * (kw - 1) - 1) / stride_w + 1;
    if (Ho < 1 || Wo < 1) return SLAYER_EINVAL;
    if (N == 0 || T == 0) return 0;
    if (!out || !in || !weight) return SLAYER_ENULL;
    // whole quads of time steps at 16-byte addresses, 32-bit byte offsets inside one batch entry
    if ((T % 4) != 0 || !aligned16(out) || !aligned16(in)) return SLAYER_ERANGE;
    const int64_t K = Ci * kh * kw, lim = (int64_t)1 << 31;
    if (Ci * H * W * T * 4 >= lim || Co * Ho * Wo * T * 4 >= lim || K > 4096 || pad_h > 4096 || pad_w > 4096 ||
        H * stride_h > (1 << 20) || W * stride_w > (1 << 20))
        return SLAYER_ERANGE;
    SynapseConv p;
    p.out = out; p.in = in; p.weight = weight;
    p.N = (int)N; p.Ci = (int)Ci; p.Co = (int)Co; p.H = (int)H; p.W = (int)W; p.Ho = (int)Ho; p.Wo = (int)Wo; p.T = (int)T;
    p.kh = (int)kh; p.kw = (int)kw; p.sh = (int)stride_h; p.sw = (int)stride_w; p.ph = (int)pad_h; p.pw = (int)pad_w;
    p.dh = (int)dil_h; p.dw = (int)dil_w;
    p.K = (int)K; p.KG = (int)((K + 3) / 4);
    p.ttiles = (int)((T + kSynTile - 1) / kSynTile);
    // enough workgroups to fill the chip several times over, image rows cut into as few pieces as that takes
    const int64_t tgroups = (p.ttiles + kSynWaves - 1) / kSynWaves;
    const int64_t base = N * ((Co + 15) / 16) * Ho * tgroups;
    int wsplit = 1;
    while (base * wsplit < 8 * 256 && wsplit * 2 <= Wo) wsplit *= 2;
    p.wsplit = wsplit;
    const int64_t blocks = base * wsplit;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const size_t lds = (size_t)p.KG * 4 * (16 * sizeof(float) + 3 * sizeof(int));
    if (lds > 64 * 1024) return SLAYER_ERANGE;
    const bool streaming = N * Co * Ho * Wo * T * 4 > ((int64_t)64 << 20);
    if (streaming)
        hipLaunchKernelGGL((synapse_conv_kernel<true>), dim3((unsigned)blocks), dim3(kSynWaves * kWave), lds,
                           (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL((synapse_conv_kernel<false>), dim3((unsigned)blocks), dim3(kSynWaves * kWave), lds,
                           (hipStream_t)stream, p);
    return (int)hipGetLastError();
}
