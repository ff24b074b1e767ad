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

constexpr int kSynChunk = 6;            // tap groups whose loads are in flight together

struct SynapseConv {
    float* out;
    const float* in;
    const float* weight;                // [Co][Ci][kh][kw]
    int N, Ci, Co, H, W, Ho, Wo, T;
    int kh, kw, sh, sw, ph, pw, dh, dw;
    int K, KG;                          // taps, groups of four taps (a whole number of chunks, padded with null taps)
    int ttiles, wsplit;                 // tiles of 64 steps per row, pieces an image row is cut into
    int items;                          // (tile, piece, output row) triples of one (batch entry, channel block)
};

// LDS: the weights of this workgroup's 16 output channels, tap-major (row k holds the 16 channels), and per tap the
// offset of its input row relative to the pixel's own position and its (row, column) displacement in the image.
// A workgroup's four waves take four consecutive items of one (batch entry, channel block): an item is one tile
// of 64 steps of a piece of one output row.
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
    // workgroup -> (batch entry, block of 16 output channels, four items)
    const int groups = (p.items + kSynWaves - 1) / kSynWaves;
    int b = blockIdx.x;
    const int ig = b % groups; b /= groups;
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

    const int item = ig * kSynWaves + wave;
    if (item >= p.items) return;
    const int tile = item % p.ttiles;
    const int piece = (item / p.ttiles) % p.wsplit;
    const int ho = item / (p.ttiles * p.wsplit);
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
        for (int g0 = 0; g0 < p.KG; g0 += kSynChunk) {
            float4 q[kSynChunk];
            float a[kSynChunk];
#pragma unroll
            for (int u = 0; u < kSynChunk; ++u) {
                const int k = 4 * (g0 + u) + kk;
                const int yy = hin + tap_dy[k], xx = win + tap_dx[k];
                const bool ok = t_ok && (unsigned)yy < (unsigned)p.H && (unsigned)xx < (unsigned)p.W;
                q[u] = buf_load4<false>(src, ok ? pix + tap_off[k] : kOutOfRange);
                a[u] = wt[k * 16 + j];
            }
#pragma unroll
            for (int u = 0; u < kSynChunk; ++u) {
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].x, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].y, acc[1], 0, 0, 0);
                acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].z, acc[2], 0, 0, 0);
                acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].w, acc[3], 0, 0, 0);
            }
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

// The common case -- unit stride and dilation along the image row, KW taps per row -- takes PIX neighbouring
// output pixels at a time: they share their input columns (PIX + KW - 1 of them instead of PIX * KW), so a group of
// four (input channel, kernel row) pairs costs PIX + KW - 1 loads for PIX * KW * 4 matrix products.  Measured on
// [32,8,32,32,300] -> 16 channels, 3x3: the one-pixel form is bound by what the caches deliver to the loads
// (18 KB per pixel and tile of 64 steps), not by the matrix cores.
// LDS: weights as above (tap k = pair * KW + x, pair = ci * kh + y), and per pair the byte offset of its input row
// relative to the pixel block's own position and its row displacement.
template <int KW, int PIX, bool STREAM>
__global__ __launch_bounds__(kSynWaves * kWave) void synapse_conv_row_kernel(const SynapseConv p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int PG = p.KG;                                // groups of four pairs
    const int Kp = PG * 4 * KW;
    float* wt = lds;                                    // [Kp][16]
    int* pair_off = reinterpret_cast<int*>(lds + Kp * 16);  // [4 PG] bytes
    int* pair_dy = pair_off + 4 * PG;                   // [4 PG]

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int groups = (p.items + kSynWaves - 1) / kSynWaves;
    int b = blockIdx.x;
    const int ig = b % groups; b /= groups;
    const int cob = b % ((p.Co + 15) / 16);
    const int n = b / ((p.Co + 15) / 16);
    const int co0 = cob * 16;

    for (int i = tid; i < Kp * 16; i += kSynWaves * kWave) {
        const int k = i >> 4, m = i & 15;
        wt[i] = (k < p.K && co0 + m < p.Co) ? p.weight[(int64_t)(co0 + m) * p.K + k] : 0.0f;
    }
    for (int pr = tid; pr < 4 * PG; pr += kSynWaves * kWave) {
        const int ci = pr / p.kh, y = pr - ci * p.kh;
        const int dy = y * p.dh - p.ph;
        pair_dy[pr] = pr < p.Ci * p.kh ? dy : (1 << 28);                 // a pair that does not exist: always outside
        pair_off[pr] = (((ci * p.H + dy) * p.W) - p.pw) * p.T * 4;
    }
    __syncthreads();

    const int item = ig * kSynWaves + wave;
    if (item >= p.items) return;
    const int tile = item % p.ttiles;
    const int piece = (item / p.ttiles) % p.wsplit;
    const int ho = item / (p.ttiles * p.wsplit);
    const int t0 = tile * kSynTile;
    const int kk = lane >> 4, j = lane & 15;
    const bool t_ok = t0 + 4 * j < p.T;                                  // T is a whole number of quads
    const int hin = ho * p.sh;
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho * p.Wo * p.T;
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(p.out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));
    const int col = p.T * 4;                                             // bytes from a pixel to its right neighbour

    const int per = ((p.Wo + p.wsplit - 1) / p.wsplit + PIX - 1) / PIX * PIX;
    const int w_lo = piece * per, w_hi = (w_lo + per) < p.Wo ? (w_lo + per) : p.Wo;
    for (int wo0 = w_lo; wo0 < w_hi; wo0 += PIX) {
        const int pix = ((hin * p.W) + wo0) * col + (t0 + 4 * j) * 4;
        syn_f4 acc[PIX][4];
#pragma unroll
        for (int i = 0; i < PIX; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][e] = syn_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
        for (int g = 0; g < PG; ++g) {
            const int pr = 4 * g + kk;
            const bool row_ok = t_ok && (unsigned)(hin + pair_dy[pr]) < (unsigned)p.H;
            const int base = pix + pair_off[pr];
            float4 q[PIX + KW - 1];
#pragma unroll
            for (int c = 0; c < PIX + KW - 1; ++c) {
                const bool ok = row_ok && (unsigned)(wo0 + c - p.pw) < (unsigned)p.W;
                q[c] = buf_load4<false>(src, ok ? base + c * col : kOutOfRange);
            }
            float a[KW];
#pragma unroll
            for (int x = 0; x < KW; ++x) a[x] = wt[(pr * KW + x) * 16 + j];
#pragma unroll
            for (int x = 0; x < KW; ++x) {
#pragma unroll
                for (int i = 0; i < PIX; ++i) {
                    acc[i][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], q[i + x].x, acc[i][0], 0, 0, 0);
                    acc[i][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], q[i + x].y, acc[i][1], 0, 0, 0);
                    acc[i][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], q[i + x].z, acc[i][2], 0, 0, 0);
                    acc[i][3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], q[i + x].w, acc[i][3], 0, 0, 0);
                }
            }
        }
        // lane (kk, j): output channels co0 + 4 kk + i, steps t0 + 4 j + e
#pragma unroll
        for (int px = 0; px < PIX; ++px) {
            const int opix = ((ho * p.Wo) + wo0 + px) * col + (t0 + 4 * j) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int co = co0 + 4 * kk + i;
                const bool ok = t_ok && co < p.Co && wo0 + px < w_hi;
                buf_store4<STREAM>(dst, ok ? co * (p.Ho * p.Wo * col) + opix : kOutOfRange,
                                   make_float4(acc[px][0][i], acc[px][1][i], acc[px][2][i], acc[px][3][i]));
            }
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
    p.K = (int)K;
    p.ttiles = (int)((T + kSynTile - 1) / kSynTile);
    // blocks of four neighbouring pixels that share their input columns: unit stride and dilation along the row
#ifndef SLAYER_SYN_PIX
#define SLAYER_SYN_PIX 4
#endif
    constexpr int kRowPix = SLAYER_SYN_PIX;
    const bool rows = stride_w == 1 && dil_w == 1 && (kw == 3 || kw == 5) && Wo >= kRowPix;
    // enough waves for four rounds of the chip (16 waves on each of 256 compute units), so that the last, partly
    // filled round weighs little; image rows cut into as few pieces as that takes
    const int64_t base = N * ((Co + 15) / 16) * Ho * p.ttiles;
    int wsplit = 1;
    while (base * wsplit < 16 * 1024 && wsplit * 2 * (rows ? kRowPix : 1) <= Wo) wsplit *= 2;
    p.wsplit = wsplit;
    const int64_t items = Ho * wsplit * p.ttiles;
    if (items > 0x7fffffffLL) return SLAYER_ERANGE;
    p.items = (int)items;
    const int64_t blocks = N * ((Co + 15) / 16) * ((items + kSynWaves - 1) / kSynWaves);
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const bool streaming = N * Co * Ho * Wo * T * 4 > ((int64_t)64 << 20);
    const dim3 grid((unsigned)blocks), block(kSynWaves * kWave);
    hipStream_t st = (hipStream_t)stream;
    if (rows) {
        p.KG = (int)((Ci * kh + 3) / 4);                                  // groups of four (channel, kernel row) pairs
        const size_t lds = (size_t)p.KG * 4 * (kw * 16 * sizeof(float) + 2 * sizeof(int));
        if (lds > 64 * 1024) return SLAYER_ERANGE;
#define SLAYER_SYN_ROW(KW)                                                                                          \
        do {                                                                                                        \
            if (streaming) hipLaunchKernelGGL((synapse_conv_row_kernel<KW, kRowPix, true>), grid, block, lds, st, p); \
            else hipLaunchKernelGGL((synapse_conv_row_kernel<KW, kRowPix, false>), grid, block, lds, st, p);         \
        } while (0)
        if (kw == 3) SLAYER_SYN_ROW(3); else SLAYER_SYN_ROW(5);
#undef SLAYER_SYN_ROW
        return (int)hipGetLastError();
    }
    p.KG = (int)(((K + 3) / 4 + kSynChunk - 1) / kSynChunk * kSynChunk);
    const size_t lds = (size_t)p.KG * 4 * (16 * sizeof(float) + 3 * sizeof(int));
    if (lds > 64 * 1024) return SLAYER_ERANGE;
    if (streaming)
        hipLaunchKernelGGL((synapse_conv_kernel<true>), grid, block, lds, st, p);
    else
        hipLaunchKernelGGL((synapse_conv_kernel<false>), grid, block, lds, st, p);
    return (int)hipGetLastError();
}
