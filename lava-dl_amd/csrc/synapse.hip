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

int launch_zero_fill(float* p, int64_t n, hipStream_t stream);          // li.hip

typedef float syn_f4 __attribute__((ext_vector_type(4)));

// Rows of any length (T >= 4): a quad of steps is a 16-byte access at a dword-aligned address, and the last quad of
// a row may hold fewer than four steps (nv of them).  Such a quad is loaded four steps before the end of its row --
// never beyond it -- and moved into place: element e of the result is element e + 4 - nv of what was loaded, zero
// behind the row's end.  Stores leave the steps that do not exist out.
struct SynQuad {
    int t_load;                         // step the quad is loaded at
    int nv;                             // steps of the quad that exist (<= 0: none, the lane loads nothing)
    template <bool TAIL>
    __device__ __forceinline__ void set(int t, int t_end) {
        nv = t_end - t;
        t_load = (TAIL && nv > 0 && nv < 4) ? t_end - 4 : t;
    }
    __device__ __forceinline__ bool any() const { return nv > 0; }
    __device__ __forceinline__ bool partial() const { return nv > 0 && nv < 4; }
    // TAIL: the rows are not whole quads (decided on the host: a test per load would sit between the loads)
    template <bool TAIL>
    __device__ __forceinline__ float4 place(float4 q) const {
        if (!TAIL || !__any(partial())) return q;                        // only the tile that holds the end of the rows
        const int d = partial() ? 4 - nv : 0;
        const float a[4] = {q.x, q.y, q.z, q.w};
        float r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = e + d;
            r[e] = i == 0 ? a[0] : (i == 1 ? a[1] : (i == 2 ? a[2] : (i == 3 ? a[3] : 0.f)));
        }
        return make_float4(r[0], r[1], r[2], r[3]);
    }
};
// the quad v at byte offset off, of which the first nv elements exist (nv <= 0: nothing is stored)
template <bool STREAM, bool TAIL>
__device__ __forceinline__ void syn_store_quad(__amdgpu_buffer_rsrc_t dst, bool on, int off, int nv, float4 v) {
    buf_store4<STREAM>(dst, (on && nv >= 4) ? off : kOutOfRange, v);
    if (TAIL && __any(on && nv > 0 && nv < 4)) {                                 // only the tile that holds the end of the rows
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 3; ++i) buf_store1<false>(dst, (on && nv < 4 && i < nv) ? off + 4 * i : kOutOfRange, e[i]);
    }
}

// Workgroups are handed to the chip's eight XCDs round-robin by their index, and each XCD has an L2 of its own.
// Neighbouring work items of the kernels below share most of what they read (an input row serves the output rows
// above and below it and the neighbouring time shares of the weight gradient), so taken in index order every XCD
// fetched nearly every row for itself: FETCH_SIZE read 5.0 x the input tensor for the forward kernel on
// [32,8,32,32,300] -> 16 channels, 1.4 x with the permuted index below, by which XCD x gets the x-th contiguous eighth
// of the work.
constexpr int kXcds = 8;
__device__ __forceinline__ int xcd_contiguous(int b, int nb) {
    const int x = b % kXcds, slot = b / kXcds, q = nb / kXcds, r = nb % kXcds;
    return x * q + (x < r ? x : r) + slot;
}

constexpr int kSynTile = 64;            // time steps per tile
constexpr int kSynWaves = 4;            // waves per workgroup: same output channels, same image row, different tiles

constexpr int kSynChunk = 6;            // tap groups whose loads are in flight together (fewer for filters of a few taps)

struct SynapseConv {
    float* out;
    const float* in;
    const float* weight;                // [Co][Ci][kh_full][kw_full]
    int N, Ci, Co, H, W, Ho, Wo, T;
    int kh, kw, sh, sw, ph, pw, dh, dw; // ph, pw: may be negative (a window that begins inside the image)
    int K, KG;                          // taps, groups of four taps (a whole number of chunks, padded with null taps)
    int ttiles, wsplit;                 // tiles of 64 steps per row, pieces an image row is cut into
    int items;                          // (tile, piece, output row) triples of one (batch entry, channel block)
    // The taps may be a sub-lattice of a larger filter and the outputs a sub-lattice of a larger image (identity for
    // a plain convolution): row iy of the kh x kw taps is row ky0 + iy * kys of the weight tensor's kh_full rows,
    // output pixel (ho, wo) is pixel (oy0 + ho * oys, ox0 + wo * oxs) of a tensor [Co][Ho_full][Wo_full][T].
    int kh_full, kw_full, ky0, kys, kx0, kxs;
    int Ho_full, Wo_full, oy0, oys, ox0, oxs;
    __device__ __forceinline__ int weight_index(int ci, int iy, int ix) const {
        return (ci * kh_full + ky0 + iy * kys) * kw_full + kx0 + ix * kxs;
    }
    __device__ __forceinline__ int out_pixel(int ho, int wo) const {     // in pixels of the full output image
        return (oy0 + ho * oys) * Wo_full + ox0 + wo * oxs;
    }
};

// The gradient of the input of a convolution with strides (what conv_transpose3d computes, the ConvTranspose synapse
// of synapse/layer.py:513-560 in the reference) is one plain convolution per residue class of the output pixels: the
// pixels (ry + m sh, rx + m' sw) meet only the taps y with (ry + ph - y dh) divisible by sh (x likewise), and over
// m, m' those taps slide across the source with unit stride.  Each class is a launch of the kernels below on its
// sub-lattices of taps and of outputs (slayer_conv_synapse_input_grad), a fraction 1 / (sh sw) of the taps each.
//
// LDS: the weights of this workgroup's 16 output channels, tap-major (row k holds the 16 channels), and per tap the
// offset of its input row relative to the pixel's own position and its (row, column) displacement in the image.
// A workgroup's four waves take four consecutive items of one (batch entry, channel block): an item is one tile
// of 64 steps of a piece of one output row.
template <bool STREAM, bool TAIL, int CHUNK>
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
    int b = xcd_contiguous(blockIdx.x, gridDim.x);
    const int ig = b % groups; b /= groups;
    const int cob = b % ((p.Co + 15) / 16);
    const int n = b / ((p.Co + 15) / 16);
    const int co0 = cob * 16;

    const int64_t k_full = (int64_t)p.Ci * p.kh_full * p.kw_full;
    for (int i = tid; i < Kp * 16; i += kSynWaves * kWave) {
        const int k = i >> 4, m = i & 15;
        const int ci = k / (p.kh * p.kw), r = k - ci * (p.kh * p.kw), y = r / p.kw, x = r - y * p.kw;
        wt[i] = (k < p.K && co0 + m < p.Co) ? p.weight[(int64_t)(co0 + m) * k_full + p.weight_index(ci, y, x)] : 0.0f;
    }
    for (int k = tid; k < Kp; k += kSynWaves * kWave) {
        const int ci = k / (p.kh * p.kw), r = k - ci * (p.kh * p.kw), y = r / p.kw, x = r - y * p.kw;
        const int dy = y * p.dh - p.ph;
        const int dx = x * p.dw - p.pw;
        tap_dy[k] = k < p.K ? dy : (1 << 28);                             // a tap that does not exist: always outside
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
    SynQuad tq;
    tq.template set<TAIL>(t0 + 4 * j, p.T);
    const int nv = tq.nv;
    const bool t_ok = tq.any();
    const int hin = ho * p.sh;                                           // image row of tap (0, 0) before padding
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho_full * p.Wo_full * p.T;
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(p.out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));

    const int per = (p.Wo + p.wsplit - 1) / p.wsplit;
    const int w_lo = piece * per, w_hi = (w_lo + per) < p.Wo ? (w_lo + per) : p.Wo;
    for (int wo = w_lo; wo < w_hi; ++wo) {
        const int win = wo * p.sw;
        const int pix = ((hin * p.W) + win) * p.T * 4 + tq.t_load * 4;   // byte offset of tap (0,0,0)'s quad
        syn_f4 acc[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = syn_f4{0.f, 0.f, 0.f, 0.f};
        for (int g0 = 0; g0 < p.KG; g0 += CHUNK) {
            float4 q[CHUNK];
            float a[CHUNK];
#pragma unroll
            for (int u = 0; u < CHUNK; ++u) {
                const int k = 4 * (g0 + u) + kk;
                const int yy = hin + tap_dy[k], xx = win + tap_dx[k];
                const bool ok = t_ok && (unsigned)yy < (unsigned)p.H && (unsigned)xx < (unsigned)p.W;
                q[u] = tq.template place<TAIL>(buf_load4<false>(src, ok ? pix + tap_off[k] : kOutOfRange));
                a[u] = wt[k * 16 + j];
            }
#pragma unroll
            for (int u = 0; u < CHUNK; ++u) {
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].x, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].y, acc[1], 0, 0, 0);
                acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].z, acc[2], 0, 0, 0);
                acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], q[u].w, acc[3], 0, 0, 0);
            }
        }
        // lane (kk, j): output channels co0 + 4 kk + i, steps t0 + 4 j + e
        const int opix = p.out_pixel(ho, wo) * p.T * 4 + (t0 + 4 * j) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int co = co0 + 4 * kk + i;
            syn_store_quad<STREAM, TAIL>(dst, co < p.Co, co * (p.Ho_full * p.Wo_full * p.T * 4) + opix, nv,
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
template <int KW, int PIX, bool STREAM, bool TAIL>
__device__ __forceinline__ void synapse_conv_row(const SynapseConv& p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int PG = p.KG;                                // groups of four pairs
    const int Kp = PG * 4 * KW;
    float* wt = lds;                                    // [Kp][16]
    int* pair_off = reinterpret_cast<int*>(lds + Kp * 16);  // [4 PG] bytes
    int* pair_dy = pair_off + 4 * PG;                   // [4 PG]

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int groups = (p.items + kSynWaves - 1) / kSynWaves;
    int b = xcd_contiguous(blockIdx.x, gridDim.x);
    const int ig = b % groups; b /= groups;
    const int cob = b % ((p.Co + 15) / 16);
    const int n = b / ((p.Co + 15) / 16);
    const int co0 = cob * 16;

    const int64_t k_full = (int64_t)p.Ci * p.kh_full * p.kw_full;
    // eight loads of a thread in flight at a time (one after the other they were a fifth of a workgroup's life)
    for (int i0 = tid; i0 < Kp * 16; i0 += 8 * kSynWaves * kWave) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kSynWaves * kWave;
            const int k = i >> 4, m = i & 15;
            const int pr = k / KW, x = k - pr * KW, ci = pr / p.kh, y = pr - ci * p.kh;
            v[u] = (k < p.K && co0 + m < p.Co) ? p.weight[(int64_t)(co0 + m) * k_full + p.weight_index(ci, y, x)] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kSynWaves * kWave;
            if (i < Kp * 16) wt[i] = v[u];
        }
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
    SynQuad tq;
    tq.template set<TAIL>(t0 + 4 * j, p.T);
    const int nv = tq.nv;
    const bool t_ok = tq.any();
    const int hin = ho * p.sh;
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho_full * p.Wo_full * p.T;
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(p.out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));
    const int col = p.T * 4;                                             // bytes from a pixel to its right neighbour

    const int per = ((p.Wo + p.wsplit - 1) / p.wsplit + PIX - 1) / PIX * PIX;
    const int w_lo = piece * per, w_hi = (w_lo + per) < p.Wo ? (w_lo + per) : p.Wo;
    for (int wo0 = w_lo; wo0 < w_hi; wo0 += PIX) {
        const int pix = ((hin * p.W) + wo0) * col + tq.t_load * 4;
        syn_f4 acc[PIX][4];
#pragma unroll
        for (int i = 0; i < PIX; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][e] = syn_f4{0.f, 0.f, 0.f, 0.f};
        for (int g = 0; g < PG; ++g) {
            const int pr = 4 * g + kk;
            const bool row_ok = t_ok && (unsigned)(hin + pair_dy[pr]) < (unsigned)p.H;
            const int base = pix + pair_off[pr];
            float4 q[PIX + KW - 1];
#pragma unroll
            for (int c = 0; c < PIX + KW - 1; ++c) {
                const bool ok = row_ok && (unsigned)(wo0 + c - p.pw) < (unsigned)p.W;
                q[c] = tq.template place<TAIL>(buf_load4<false>(src, ok ? base + c * col : kOutOfRange));
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
            const int opix = p.out_pixel(ho, wo0 + px) * col + (t0 + 4 * j) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int co = co0 + 4 * kk + i;
                syn_store_quad<STREAM, TAIL>(dst, co < p.Co && wo0 + px < w_hi, co * (p.Ho_full * p.Wo_full * col) + opix, nv,
                                       make_float4(acc[px][0][i], acc[px][1][i], acc[px][2][i], acc[px][3][i]));
            }
        }
    }
}

// Rows of whole quads at five waves per SIMD (88 registers, no spills; four waves otherwise: 2-3 % slower); the
// forms for rows that end inside a quad need a few registers more and keep the compiler's own choice.
template <int KW, int PIX, bool STREAM>
__global__ __launch_bounds__(kSynWaves * kWave) __attribute__((amdgpu_waves_per_eu(5)))
void synapse_conv_row_kernel(const SynapseConv p) { synapse_conv_row<KW, PIX, STREAM, false>(p); }
template <int KW, int PIX, bool STREAM>
__global__ __launch_bounds__(kSynWaves * kWave) void synapse_conv_row_tail_kernel(const SynapseConv p) {
    synapse_conv_row<KW, PIX, STREAM, true>(p);
}

// One input and one output channel (the pooling layers, which fold their channels into the image height,
// synapse/layer.py:438-508 and :770-838 in the reference): there is no contraction for the matrix cores, and a wave
// that owns 16 channels x 64 steps of one pixel would move 256 bytes per instruction.  One thread per quad of output
// steps on the vector units instead: a block row of the grid is ROWS image rows of the output, grid.z the batch.
// SPREAD: the gradient of the input (the unpooling layer's forward pass): output pixel (h, w) sums the taps (y, x)
// whose source coordinates (h + ph - y dh) / sh, (w + pw - x dw) / sw are exact.  Which taps those are depends on
// h mod sh alone: a table in LDS lists them per residue (at most ny per residue: tap_y, and quot_y = the quotient
// less h / sh; likewise nx, tap_x, quot_x), so that a pixel visits ny * nx slots -- one for a pooling window that is
// as large as its stride -- instead of all kh * kw taps.
constexpr int kPlaneThreads = 256;
#ifndef SLAYER_PLANE_ROWS_SUM
#define SLAYER_PLANE_ROWS_SUM 1
#endif
#ifndef SLAYER_PLANE_ROWS_SPREAD
#define SLAYER_PLANE_ROWS_SPREAD 8
#endif
constexpr int kPlaneRowsSum = SLAYER_PLANE_ROWS_SUM, kPlaneRowsSpread = SLAYER_PLANE_ROWS_SPREAD;
template <bool SPREAD, bool STREAM, bool TAIL, int ROWS>
__global__ __launch_bounds__(kPlaneThreads) void synapse_plane_kernel(const SynapseConv p, int quads, int ny, int nx) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* wt = lds;                                                      // [kh * kw]
    int* quot_y = reinterpret_cast<int*>(lds + p.kh * p.kw);              // SPREAD: [sh * ny]
    int* tap_y = quot_y + p.sh * ny;                                      //         [sh * ny], times kw
    int* quot_x = tap_y + p.sh * ny;                                      //         [sw * nx]
    int* tap_x = quot_x + p.sw * nx;                                      //         [sw * nx]
    const int none = 1 << 28;
    for (int i = threadIdx.x; i < p.kh * p.kw; i += kPlaneThreads) wt[i] = p.weight[i];
    if (SPREAD) {
        for (int r = threadIdx.x; r < p.sh + p.sw; r += kPlaneThreads) {
            const bool rows = r < p.sh;
            const int res = rows ? r : r - p.sh, k = rows ? p.kh : p.kw, stride = rows ? p.sh : p.sw;
            const int pad = rows ? p.ph : p.pw, dil = rows ? p.dh : p.dw, slots = rows ? ny : nx;
            int* quot = (rows ? quot_y : quot_x) + res * slots;
            int* tap = (rows ? tap_y : tap_x) + res * slots;
            int found = 0;
            for (int y = 0; y < k; ++y) {
                const int c = res + pad - y * dil;
                if (c % stride == 0) { quot[found] = c / stride; tap[found] = rows ? y * p.kw : y; ++found; }
            }
            for (; found < slots; ++found) { quot[found] = none; tap[found] = 0; }
        }
    }
    __syncthreads();
    const int n = blockIdx.z;
    const int idx = blockIdx.x * kPlaneThreads + threadIdx.x;
    const int wo = idx / quads, j = idx - wo * quads;
    const bool on = wo < p.Wo;
    SynQuad tq;
    tq.template set<TAIL>(4 * j, p.T);
    const bool lane_on = on && tq.any();
    const int64_t in_plane = (int64_t)p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Ho * p.Wo * p.T;
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(p.out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));
    // SPREAD: the pixel as quotient and residue of the strides (the rows' are the same for the whole block)
    const int wq = SPREAD ? wo / p.sw : 0, rx = SPREAD ? (on ? wo - wq * p.sw : 0) : 0;
    // A block takes ROWS image rows at once: the tables above are set up once for all of them, and a slot is
    // loaded for all the rows before the first product waits for it.
    const int ho0 = blockIdx.y * ROWS;
    int hq[ROWS], ry[ROWS];
    float4 acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        hq[r] = SPREAD ? (ho0 + r) / p.sh : 0;
        ry[r] = SPREAD ? (ho0 + r < p.Ho ? ho0 + r - hq[r] * p.sh : 0) : 0;
        acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int y = 0; y < (SPREAD ? ny : p.kh); ++y) {
        int row_off[ROWS], w_row[ROWS];                                   // source row of this slot or none, its weights
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int yy = SPREAD ? hq[r] + quot_y[ry[r] * ny + y] : (ho0 + r) * p.sh + y * p.dh - p.ph;
            row_off[r] = (ho0 + r < p.Ho && (unsigned)yy < (unsigned)p.H) ? yy * p.W : -1;
            w_row[r] = SPREAD ? tap_y[ry[r] * ny + y] : y * p.kw;
        }
        for (int x = 0; x < (SPREAD ? nx : p.kw); ++x) {
            const int xx = SPREAD ? wq + quot_x[rx * nx + x] : wo * p.sw + x * p.dw - p.pw;
            const int w_col = SPREAD ? tap_x[rx * nx + x] : x;
            const bool ok = lane_on && (unsigned)xx < (unsigned)p.W;
            float4 q[ROWS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                q[r] = buf_load4<false>(src, (ok && row_off[r] >= 0) ? ((row_off[r] + xx) * p.T + tq.t_load) * 4 : kOutOfRange);
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const float f = wt[w_row[r] + w_col];
                const float4 v = tq.template place<TAIL>(q[r]);
                acc[r].x = __fmaf_rn(f, v.x, acc[r].x); acc[r].y = __fmaf_rn(f, v.y, acc[r].y);
                acc[r].z = __fmaf_rn(f, v.z, acc[r].z); acc[r].w = __fmaf_rn(f, v.w, acc[r].w);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
        syn_store_quad<STREAM, TAIL>(dst, on && ho0 + r < p.Ho, (((ho0 + r) * p.Wo + wo) * p.T + 4 * j) * 4, tq.nv, acc[r]);
}

// Gradient of the weights: grad_w[co][k] = sum over batch, output pixels and time of grad_out[co][pixel][t] *
// (input row of tap k at that pixel)[t] -- a [Co x P] x [P x K] product with P = N * Ho * Wo * T positions, reduced
// along time on the matrix cores: lane (kk, j) loads steps 4 kk .. 4 kk + 3 of a 16-step group of the gradient row of
// channel co0 + j (the A operand of four products) and of the input row of tap 16 tt + j (the B operand), so that
// a group of 16 steps costs 1 + NTT loads and 4 NTT products and adds to NTT accumulator tiles [16 channels x 16
// taps].  A wave owns one output row of one batch entry and a share of the time axis, walks the row pixel by pixel
// and leaves its tiles in the workspace; synapse_wgrad_reduce_kernel adds the tiles of all waves in double, in a
// fixed order.  Filters of more than 16 NTT taps take several passes (grid dimension z).
struct SynapseWgrad {
    float* partial;                     // [items][passes][NTT][64] quads
    const float* grad_out;
    const float* in;
    int N, Ci, Co, H, W, Ho, Wo, T;
    int kh, kw, sh, sw, ph, pw, dh, dw;
    int K, passes;                      // taps, passes of 16 NTT taps
    int tparts, tlen;                   // shares of the time axis, steps per share (a multiple of 32)
    int items;                          // (share of time, output row) pairs of one (batch entry, channel block)
};

template <int NTT, bool TAIL>
__global__ __launch_bounds__(kSynWaves * kWave) void synapse_wgrad_kernel(const SynapseWgrad p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int Kp = NTT * 16;
    int* tap_off = reinterpret_cast<int*>(lds);         // [Kp] bytes
    int* tap_dy = tap_off + Kp;                         // [Kp]
    int* tap_dx = tap_dy + Kp;                          // [Kp]

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int groups = (p.items + kSynWaves - 1) / kSynWaves;
    const int cobs = (p.Co + 15) / 16;
    int b = xcd_contiguous(blockIdx.x, gridDim.x);
    const int ig = b % groups; b /= groups;
    const int cob = b % cobs;
    const int n = b / cobs;
    const int co0 = cob * 16;
    const int pass = blockIdx.y;
    const int k0 = pass * Kp;

    for (int kl = tid; kl < Kp; kl += kSynWaves * kWave) {
        const int k = k0 + kl;
        const int ci = k / (p.kh * p.kw), r = k - ci * (p.kh * p.kw), y = r / p.kw, x = r - y * p.kw;
        const int dy = y * p.dh - p.ph, dx = x * p.dw - p.pw;
        tap_dy[kl] = k < p.K ? dy : (1 << 28);                           // a tap that does not exist: always outside
        tap_dx[kl] = dx;
        tap_off[kl] = (((ci * p.H + dy) * p.W) + dx) * p.T * 4;
    }
    __syncthreads();

    const int item = ig * kSynWaves + wave;
    if (item >= p.items) return;
    const int tpart = item % p.tparts;
    const int ho = item / p.tparts;
    const int kk = lane >> 4, j = lane & 15;
    const int hin = ho * p.sh;
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho * p.Wo * p.T;
    const __amdgpu_buffer_rsrc_t grd = make_rsrc(p.grad_out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));
    const int col = p.T * 4;
    const bool co_ok = co0 + j < p.Co;
    const int g_row = (co0 + j) * (p.Ho * p.Wo * col) + ho * p.Wo * col;  // gradient row of this lane's channel
    // this lane's taps: offset of the input row relative to the pixel, and whether its image row exists
    int my_off[NTT], my_dx[NTT];
    bool my_row[NTT];
#pragma unroll
    for (int tt = 0; tt < NTT; ++tt) {
        my_off[tt] = tap_off[16 * tt + j];
        my_dx[tt] = tap_dx[16 * tt + j];
        my_row[tt] = (unsigned)(hin + tap_dy[16 * tt + j]) < (unsigned)p.H;
    }
    syn_f4 acc[NTT][2];                                                  // two chains per tile: no product waits for the one before
#pragma unroll
    for (int tt = 0; tt < NTT; ++tt) acc[tt][0] = acc[tt][1] = syn_f4{0.f, 0.f, 0.f, 0.f};

    const int t_lo = tpart * p.tlen, t_hi = (t_lo + p.tlen) < p.T ? (t_lo + p.tlen) : p.T;
    for (int t0 = t_lo; t0 < t_hi; t0 += 32) {                           // one 128-byte line of every row per visit
        for (int wo = 0; wo < p.Wo; ++wo) {
            const int win = wo * p.sw;
            const int pix = ((hin * p.W) + win) * col;
            float4 g[2], q[2][NTT];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int t = t0 + 16 * u + 4 * kk;
                SynQuad tq;                                              // the shares are whole quads; a row's last quad may not be
                tq.template set<TAIL>(t, t_hi);
                const bool t_ok = tq.any();
                g[u] = tq.template place<TAIL>(buf_load4<false>(grd, (t_ok && co_ok) ? g_row + wo * col + tq.t_load * 4 : kOutOfRange));
#pragma unroll
                for (int tt = 0; tt < NTT; ++tt) {
                    const bool ok = t_ok && my_row[tt] && (unsigned)(win + my_dx[tt]) < (unsigned)p.W;
                    q[u][tt] = tq.template place<TAIL>(buf_load4<false>(src, ok ? pix + my_off[tt] + tq.t_load * 4 : kOutOfRange));
                }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int tt = 0; tt < NTT; ++tt) {
                    acc[tt][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(g[u].x, q[u][tt].x, acc[tt][0], 0, 0, 0);
                    acc[tt][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(g[u].y, q[u][tt].y, acc[tt][1], 0, 0, 0);
                }
#pragma unroll
                for (int tt = 0; tt < NTT; ++tt) {
                    acc[tt][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(g[u].z, q[u][tt].z, acc[tt][0], 0, 0, 0);
                    acc[tt][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(g[u].w, q[u][tt].w, acc[tt][1], 0, 0, 0);
                }
            }
        }
    }
    // lane (q, j) of tile tt: channels co0 + 4 q + i, tap k0 + 16 tt + j
    float4* dst = reinterpret_cast<float4*>(p.partial) +
                  ((((int64_t)(n * cobs + cob) * p.items + item) * p.passes + pass) * NTT) * kWave + lane;
#pragma unroll
    for (int tt = 0; tt < NTT; ++tt)
        dst[tt * kWave] = make_float4(acc[tt][0][0] + acc[tt][1][0], acc[tt][0][1] + acc[tt][1][1],
                                      acc[tt][0][2] + acc[tt][1][2], acc[tt][0][3] + acc[tt][1][3]);
}

// The common case again (unit stride and dilation along the image row, KW taps per row): the taps of a tile are 16
// (input channel, kernel row) pairs at one input column, and that column meets KW output pixels, one per tap of the
// row -- so the wave walks the input columns of its image row, keeps the gradient quads of the last KW pixels in
// registers (one new load per column), and a column costs 1 + NPT loads for KW * NPT * 4 products per 16 steps instead
// of 1 + KW * NPT / ... loads of the form above.  Accumulator tile (x, pt): [16 channels x 16 pairs] for tap x.
#ifndef SLAYER_WGRAD_GROUPS
#define SLAYER_WGRAD_GROUPS 4
#endif
constexpr int kWgU = SLAYER_WGRAD_GROUPS;      // groups of 16 steps per visit of a column

template <int KW, int NPT, bool TAIL>
__global__ __launch_bounds__(kSynWaves * kWave) void synapse_wgrad_row_kernel(const SynapseWgrad p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int Pp = NPT * 16;
    int* pair_off = reinterpret_cast<int*>(lds);        // [Pp] bytes, relative to the start of the wave's image row
    int* pair_dy = pair_off + Pp;                       // [Pp]

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int groups = (p.items + kSynWaves - 1) / kSynWaves;
    const int cobs = (p.Co + 15) / 16;
    int b = xcd_contiguous(blockIdx.x, gridDim.x);
    const int ig = b % groups; b /= groups;
    const int cob = b % cobs;
    const int n = b / cobs;
    const int co0 = cob * 16;
    const int pass = blockIdx.y;
    const int col = p.T * 4;

    for (int pl = tid; pl < Pp; pl += kSynWaves * kWave) {
        const int pr = pass * Pp + pl;
        const int ci = pr / p.kh, y = pr - ci * p.kh;
        const int dy = y * p.dh - p.ph;
        pair_dy[pl] = pr < p.Ci * p.kh ? dy : (1 << 28);                 // a pair that does not exist: always outside
        pair_off[pl] = ((ci * p.H + dy) * p.W) * col;
    }
    __syncthreads();

    const int item = ig * kSynWaves + wave;
    if (item >= p.items) return;
    const int tpart = item % p.tparts;
    const int ho = item / p.tparts;
    const int kk = lane >> 4, j = lane & 15;
    const int hin = ho * p.sh;
    const int64_t in_plane = (int64_t)p.Ci * p.H * p.W * p.T;
    const __amdgpu_buffer_rsrc_t src = make_rsrc(p.in + (int64_t)n * in_plane, (unsigned)(in_plane * 4));
    const int64_t out_plane = (int64_t)p.Co * p.Ho * p.Wo * p.T;
    const __amdgpu_buffer_rsrc_t grd = make_rsrc(p.grad_out + (int64_t)n * out_plane, (unsigned)(out_plane * 4));
    const bool co_ok = co0 + j < p.Co;
    const int g_row = (co0 + j) * (p.Ho * p.Wo * col) + ho * p.Wo * col;  // gradient row of this lane's channel
    const int s_row = hin * p.W * col;                                   // the wave's image row, before the pairs' offsets
    int my_off[NPT];
    bool my_row[NPT];
#pragma unroll
    for (int pt = 0; pt < NPT; ++pt) {
        my_off[pt] = s_row + pair_off[16 * pt + j];
        my_row[pt] = (unsigned)(hin + pair_dy[16 * pt + j]) < (unsigned)p.H;
    }
    syn_f4 acc[KW][NPT];
#pragma unroll
    for (int x = 0; x < KW; ++x)
#pragma unroll
        for (int pt = 0; pt < NPT; ++pt) acc[x][pt] = syn_f4{0.f, 0.f, 0.f, 0.f};

    const int t_lo = tpart * p.tlen, t_hi = (t_lo + p.tlen) < p.T ? (t_lo + p.tlen) : p.T;
    for (int t0 = t_lo; t0 < t_hi; t0 += 16 * kWgU) {                    // whole 128-byte lines of every row per visit
        int toff[kWgU];
        bool t_ok[kWgU];
        SynQuad tq[kWgU];
#pragma unroll
        for (int u = 0; u < kWgU; ++u) {
            const int t = t0 + 16 * u + 4 * kk;
            tq[u].template set<TAIL>(t, t_hi);                                          // the shares are whole quads; a row's last quad may not be
            t_ok[u] = tq[u].any();
            toff[u] = tq[u].t_load * 4;
        }
        auto grad_at = [&](int wo, int u) {
            return tq[u].template place<TAIL>(buf_load4<false>(
                grd, (t_ok[u] && co_ok && (unsigned)wo < (unsigned)p.Wo) ? g_row + wo * col + toff[u] : kOutOfRange));
        };
        // gw[x][u]: the gradient at pixel c + pw - x for the column c at hand; gw[0] arrives with the column
        float4 gw[KW][kWgU];
#pragma unroll
        for (int x = 1; x < KW; ++x)
#pragma unroll
            for (int u = 0; u < kWgU; ++u) gw[x][u] = grad_at(p.pw - x, u);
        for (int c = 0; c < p.W; ++c) {
            float4 q[kWgU][NPT];
#pragma unroll
            for (int u = 0; u < kWgU; ++u) {
                gw[0][u] = grad_at(c + p.pw, u);
#pragma unroll
                for (int pt = 0; pt < NPT; ++pt)
                    q[u][pt] = tq[u].template place<TAIL>(buf_load4<false>(
                        src, (t_ok[u] && my_row[pt]) ? my_off[pt] + c * col + toff[u] : kOutOfRange));
            }
#pragma unroll
            for (int u = 0; u < kWgU; ++u) {
#pragma unroll
                for (int x = 0; x < KW; ++x)
#pragma unroll
                    for (int pt = 0; pt < NPT; ++pt) {
                        acc[x][pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(gw[x][u].x, q[u][pt].x, acc[x][pt], 0, 0, 0);
                    }
#pragma unroll
                for (int x = 0; x < KW; ++x)
#pragma unroll
                    for (int pt = 0; pt < NPT; ++pt) {
                        acc[x][pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(gw[x][u].y, q[u][pt].y, acc[x][pt], 0, 0, 0);
                    }
#pragma unroll
                for (int x = 0; x < KW; ++x)
#pragma unroll
                    for (int pt = 0; pt < NPT; ++pt) {
                        acc[x][pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(gw[x][u].z, q[u][pt].z, acc[x][pt], 0, 0, 0);
                    }
#pragma unroll
                for (int x = 0; x < KW; ++x)
#pragma unroll
                    for (int pt = 0; pt < NPT; ++pt) {
                        acc[x][pt] = __builtin_amdgcn_mfma_f32_16x16x4f32(gw[x][u].w, q[u][pt].w, acc[x][pt], 0, 0, 0);
                    }
            }
#pragma unroll
            for (int x = KW - 1; x >= 1; --x)
#pragma unroll
                for (int u = 0; u < kWgU; ++u) gw[x][u] = gw[x - 1][u];
        }
    }
    // lane (q, j) of tile (x, pt): channels co0 + 4 q + i, pair 16 (pass NPT + pt) + j, tap x of its row
    float4* dst = reinterpret_cast<float4*>(p.partial) +
                  ((((int64_t)(n * cobs + cob) * p.items + item) * p.passes + pass) * (KW * NPT)) * kWave + lane;
#pragma unroll
    for (int x = 0; x < KW; ++x)
#pragma unroll
        for (int pt = 0; pt < NPT; ++pt)
            dst[(x * NPT + pt) * kWave] = make_float4(acc[x][pt][0], acc[x][pt][1], acc[x][pt][2], acc[x][pt][3]);
}

// grad_w[co][k] = sum over batch entries and items of the waves' tiles, in double, in a fixed order, in two
// launches: block (tile, chunk) adds the tiles of its chunk of the (batch entry, item) pairs -- sixteen partial sums
// (every sixteenth pair each), then those in turn -- into stage[chunk][tile]; the second launch adds the chunks and
// writes the gradient.  `tiles` tiles per wave and pass; tile tl holds taps k = 16 (pass tiles + tl) + j
// (row_kw == 0) or, for the row kernel, pairs 16 (pass npt + tl % npt) + j at tap x = tl / npt of their row:
// k = pair * row_kw + x.
constexpr int kWgradParts = 16;
constexpr int kWgradChunks = 32;
__global__ __launch_bounds__(kWgradParts * kWave) void synapse_wgrad_reduce_kernel(
        double* __restrict__ stage, const float* __restrict__ partial, int N, int Co, int items, int passes, int tiles) {
    __shared__ double sums[kWgradParts][kWave][4];
    const int lane = threadIdx.x & (kWave - 1), part = threadIdx.x >> 6;
    const int tl = blockIdx.x % tiles;
    int b = blockIdx.x / tiles;
    const int pass = b % passes;
    const int cob = b / passes;
    const int cobs = (Co + 15) / 16;
    double s[4] = {0.0, 0.0, 0.0, 0.0};
    const float4* src = reinterpret_cast<const float4*>(partial);
    const int64_t total = (int64_t)N * items;
    const int64_t per = (total + kWgradChunks - 1) / kWgradChunks;
    const int64_t lo = blockIdx.y * per, hi = (lo + per) < total ? (lo + per) : total;
    for (int64_t at = lo + part; at < hi; at += kWgradParts) {
        const int64_t n = at / items, item = at - n * items;
        const float4 v = src[((((n * cobs + cob) * items + item) * passes + pass) * tiles + tl) * kWave + lane];
        s[0] += v.x; s[1] += v.y; s[2] += v.z; s[3] += v.w;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) sums[part][lane][i] = s[i];
    __syncthreads();
    if (part != 0) return;
    double* dst = stage + (((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * kWave + lane) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        double tot = 0.0;
        for (int pp = 0; pp < kWgradParts; ++pp) tot += sums[pp][lane][i];
        dst[i] = tot;
    }
}

__global__ __launch_bounds__(kWave) void synapse_wgrad_final_kernel(float* __restrict__ grad_w,
                                                                     const double* __restrict__ stage, int Co, int K,
                                                                     int passes, int tiles, int row_kw, int npt) {
    const int lane = threadIdx.x, q = lane >> 4, j = lane & 15;
    const int tl = blockIdx.x % tiles;
    int b = blockIdx.x / tiles;
    const int pass = b % passes;
    const int cob = b / passes;
    int k;
    if (row_kw == 0) {
        k = (pass * tiles + tl) * 16 + j;
    } else {
        const int x = tl / npt, pt = tl - x * npt;
        const int pair = (pass * npt + pt) * 16 + j;
        k = pair * row_kw + x;
        if (pair * row_kw >= K) k = K;                                   // a pair that does not exist
    }
    double tot[4] = {0.0, 0.0, 0.0, 0.0};
    for (int c = 0; c < kWgradChunks; ++c) {
        const double* src = stage + (((int64_t)c * gridDim.x + blockIdx.x) * kWave + lane) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) tot[i] += src[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int co = cob * 16 + 4 * q + i;
        if (co < Co && k < K) grad_w[(int64_t)co * K + k] = (float)tot[i];
    }
}

}  // namespace slayer

using namespace slayer;

namespace {

#ifndef SLAYER_SYN_PIX
#define SLAYER_SYN_PIX 4
#endif

// One launch of the convolution kernels for the geometry in p (tensors, sizes, taps and sub-lattices filled in by the
// caller): the row kernel for unit stride and dilation along the image row with 2, 3 or 5 taps per row, else the
// one-pixel kernel with as many tap groups in flight as the filter has, up to six.  A filter without taps (K = 0)
// clears its outputs.
int launch_synapse_conv(SynapseConv p, bool streaming, hipStream_t st) {
    // Non-temporal stores only for the classes of a transposed convolution, which leave every line they touch
    // unfinished for the next launch.  A plain convolution finishes the lines that two of its tiles share within
    // microseconds, and the L2 puts the pieces together if it is allowed to keep them: [32,8,32,32,300] -> 16 channels
    // forward 378 -> 329 us with cached stores (the transposed 4x4 stride-2 classes 251 -> 288 us).
    if (p.oys == 1 && p.oxs == 1) streaming = false;
    constexpr int kRowPix = SLAYER_SYN_PIX;
    const int64_t K = (int64_t)p.Ci * p.kh * p.kw;
    p.K = (int)K;
    p.ttiles = (p.T + kSynTile - 1) / kSynTile;
    // blocks of four neighbouring pixels that share their input columns: unit stride and dilation along the row
    const bool rows = p.sw == 1 && p.dw == 1 && (p.kw == 2 || p.kw == 3 || p.kw == 5) && p.Wo >= kRowPix;
    // enough waves for four rounds of the chip (16 waves on each of 256 compute units), so that the last, partly
    // filled round weighs little; image rows cut into as few pieces as that takes
    const int64_t cobs = (p.Co + 15) / 16;
    const int64_t base = (int64_t)p.N * cobs * p.Ho * p.ttiles;
    int wsplit = 1;
    while (base * wsplit < 16 * 1024 && wsplit * 2 * (rows ? kRowPix : 1) <= p.Wo) wsplit *= 2;
    p.wsplit = wsplit;
    const int64_t items = (int64_t)p.Ho * wsplit * p.ttiles;
    if (items > 0x7fffffffLL) return SLAYER_ERANGE;
    p.items = (int)items;
    const int64_t blocks = p.N * cobs * ((items + kSynWaves - 1) / kSynWaves);
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
    const bool tail = (p.T % 4) != 0;                                     // rows that end inside a quad
    const dim3 grid((unsigned)blocks), block(kSynWaves * kWave);
    if (rows) {
        p.KG = (p.Ci * p.kh + 3) / 4;                                     // groups of four (channel, kernel row) pairs
        const size_t lds = (size_t)p.KG * 4 * (p.kw * 16 * sizeof(float) + 2 * sizeof(int));
        if (lds > 64 * 1024) return SLAYER_ERANGE;
#define SLAYER_SYN_ROW_T(KERNEL, KW)                                                                      \
        do {                                                                                             \
            if (streaming) hipLaunchKernelGGL((KERNEL<KW, kRowPix, true>), grid, block, lds, st, p);      \
            else hipLaunchKernelGGL((KERNEL<KW, kRowPix, false>), grid, block, lds, st, p);               \
        } while (0)
#define SLAYER_SYN_ROW(KW)                                                                                \
        do { if (tail) SLAYER_SYN_ROW_T(synapse_conv_row_tail_kernel, KW); else SLAYER_SYN_ROW_T(synapse_conv_row_kernel, KW); } while (0)
        if (p.kw == 2) SLAYER_SYN_ROW(2); else if (p.kw == 3) SLAYER_SYN_ROW(3); else SLAYER_SYN_ROW(5);
#undef SLAYER_SYN_ROW_T
#undef SLAYER_SYN_ROW
        return (int)hipGetLastError();
    }
    const int groups = (int)((K + 3) / 4);
    const int chunk = groups <= 1 ? 1 : (groups == 2 ? 2 : kSynChunk);
    p.KG = (groups + chunk - 1) / chunk * chunk;
    const size_t lds = (size_t)p.KG * 4 * (16 * sizeof(float) + 3 * sizeof(int));
    if (lds > 64 * 1024) return SLAYER_ERANGE;
#define SLAYER_SYN_ONE(S, TL, CH) hipLaunchKernelGGL((synapse_conv_kernel<S, TL, CH>), grid, block, lds, st, p)
#define SLAYER_SYN_CH(S, TL) \
    do { if (chunk == 1) SLAYER_SYN_ONE(S, TL, 1); else if (chunk == 2) SLAYER_SYN_ONE(S, TL, 2); else SLAYER_SYN_ONE(S, TL, kSynChunk); } while (0)
    if (streaming) { if (tail) SLAYER_SYN_CH(true, true); else SLAYER_SYN_CH(true, false); }
    else { if (tail) SLAYER_SYN_CH(false, true); else SLAYER_SYN_CH(false, false); }
#undef SLAYER_SYN_CH
#undef SLAYER_SYN_ONE
    return (int)hipGetLastError();
}

// the most taps of a filter row of k taps that pixels of one residue (mod stride) meet in a transposed convolution
int most_taps_per_residue(int k, int stride, int pad, int dil) {
    int most = 0;
    for (int r = 0; r < stride; ++r) {
        int found = 0;
        for (int y = 0; y < k; ++y) found += (r + pad - y * dil) % stride == 0;
        most = found > most ? found : most;
    }
    return most;
}

// The one-channel form (synapse_plane_kernel) for a plain convolution (spread = false: p as for
// launch_synapse_conv) or for the gradient of its input (spread = true: p.in the gradient of the output [H][W],
// p.out the gradient of the input [Ho][Wo], strides, padding and dilation those of the convolution).
// false: not a geometry it takes.
bool launch_synapse_plane(const SynapseConv& p, bool spread, bool streaming, hipStream_t st, int* code) {
    const int64_t quads = (p.T + 3) / 4;
    const int64_t blocks = ((int64_t)p.Wo * quads + kPlaneThreads - 1) / kPlaneThreads;
    if (p.Ci != 1 || p.Co != 1 || p.N > 65535 || blocks > 0x7fffffffLL || p.kh * p.kw > 1024) return false;
    const int ny = spread ? most_taps_per_residue(p.kh, p.sh, p.ph, p.dh) : 0;
    const int nx = spread ? most_taps_per_residue(p.kw, p.sw, p.pw, p.dw) : 0;
    const size_t lds = ((size_t)p.kh * p.kw + 2 * ((size_t)p.sh * ny + (size_t)p.sw * nx)) * 4;
    if (lds > 48 * 1024) return false;
    const int rows = spread ? kPlaneRowsSpread : kPlaneRowsSum;
    if ((p.Ho + rows - 1) / rows > 65535) return false;                   // grid.y
    const dim3 grid((unsigned)blocks, (unsigned)((p.Ho + rows - 1) / rows), (unsigned)p.N), block(kPlaneThreads);
    const bool tail = (p.T % 4) != 0;
#define SLAYER_SYN_PLANE(SP, S, TL)                                                                                      \
    hipLaunchKernelGGL((synapse_plane_kernel<SP, S, TL, (SP ? kPlaneRowsSpread : kPlaneRowsSum)>), grid, block, lds, st, p, \
                       (int)quads, ny, nx)
#define SLAYER_SYN_PLANE_T(SP, S) do { if (tail) SLAYER_SYN_PLANE(SP, S, true); else SLAYER_SYN_PLANE(SP, S, false); } while (0)
    if (spread) { if (streaming) SLAYER_SYN_PLANE_T(true, true); else SLAYER_SYN_PLANE_T(true, false); }
    else { if (streaming) SLAYER_SYN_PLANE_T(false, true); else SLAYER_SYN_PLANE_T(false, false); }
#undef SLAYER_SYN_PLANE_T
#undef SLAYER_SYN_PLANE
    *code = (int)hipGetLastError();
    return true;
}

// the taps y of a filter row that output pixels of residue r (mod stride) meet in a transposed convolution:
// (r + pad - y * dil) divisible by stride; they are y_last, y_last - step, ... (count of them), and the source
// coordinate of y_last for the first pixel of the class, (r + pad - y_last * dil) / stride, is `first`
struct TapClass { int count, y_last, step, first; };
TapClass tap_class(int r, int k, int stride, int pad, int dil) {
    TapClass c{0, 0, 1, 0};
    int y_first = -1;
    for (int y = 0; y < k; ++y) {
        if ((r + pad - y * dil) % stride != 0) continue;
        if (c.count == 0) y_first = y;
        else if (c.count == 1) c.step = y - y_first;
        c.y_last = y;
        ++c.count;
    }
    if (c.count) {
        const int num = r + pad - c.y_last * dil;                         // divisible by stride, of either sign
        c.first = num / stride;
    }
    return c;
}

}  // namespace

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
    // 32-bit byte offsets inside one batch entry; rows of any length from four steps on (16-byte accesses at
    // dword-aligned addresses)
    if (T < 4) return SLAYER_ERANGE;
    const int64_t K = Ci * kh * kw, lim = (int64_t)1 << 31;
    if (Ci * H * W * T * 4 >= lim || Co * Ho * Wo * T * 4 >= lim || K > 4096 || pad_h > 4096 || pad_w > 4096 ||
        H * stride_h > (1 << 20) || W * stride_w > (1 << 20))
        return SLAYER_ERANGE;
    SynapseConv p;
    p.out = out; p.in = in; p.weight = weight;
    p.N = (int)N; p.Ci = (int)Ci; p.Co = (int)Co; p.H = (int)H; p.W = (int)W; p.Ho = (int)Ho; p.Wo = (int)Wo; p.T = (int)T;
    p.kh = (int)kh; p.kw = (int)kw; p.sh = (int)stride_h; p.sw = (int)stride_w; p.ph = (int)pad_h; p.pw = (int)pad_w;
    p.dh = (int)dil_h; p.dw = (int)dil_w;
    p.kh_full = p.kh; p.kw_full = p.kw; p.ky0 = p.kx0 = 0; p.kys = p.kxs = 1;
    p.Ho_full = p.Ho; p.Wo_full = p.Wo; p.oy0 = p.ox0 = 0; p.oys = p.oxs = 1;
    const bool streaming = N * Co * Ho * Wo * T * 4 > ((int64_t)64 << 20);
    int code = 0;
    if (launch_synapse_plane(p, false, streaming, (hipStream_t)stream, &code)) return code;
    return launch_synapse_conv(p, streaming, (hipStream_t)stream);
}

namespace {

// The form of the weight-gradient kernels for a geometry: the row kernel (tiles of 16 (channel, kernel row) pairs,
// row_kw taps each) for unit stride and dilation along the image row with 3 or 5 taps per row, else tiles of 16
// taps; `tiles` accumulator tiles per wave and pass; the shares the time axis is cut into.
struct WgradForm { int row_kw, npt, tiles; };
WgradForm wgrad_form(int64_t Ci, int64_t kh, int64_t kw, int64_t stride_w, int64_t dil_w) {
    WgradForm f;
    if (stride_w == 1 && dil_w == 1 && (kw == 3 || kw == 5)) {
        const int64_t pairs = Ci * kh;
        f.row_kw = (int)kw;
        f.npt = pairs <= 16 ? 1 : 2;
        f.tiles = f.row_kw * f.npt;
    } else {
        const int64_t K = Ci * kh * kw;
        f.row_kw = 0;
        f.npt = 0;
        f.tiles = K <= 16 ? 1 : (K <= 32 ? 2 : 5);
    }
    return f;
}
void wgrad_shape(int64_t N, int64_t Ci, int64_t Co, int64_t Ho, int64_t T, int64_t kh, int64_t kw, const WgradForm& f,
                 SynapseWgrad& p) {
    if (f.row_kw) p.passes = (int)((Ci * kh + 16 * f.npt - 1) / (16 * f.npt));
    else p.passes = (int)((Ci * kh * kw + 16 * f.tiles - 1) / (16 * f.tiles));
    // about four thousand waves (one per SIMD and occupancy slot), shares of whole visits of 64 steps: a wave's
    // set-up (tables, the gradient window) is paid once per share
#ifndef SLAYER_WGRAD_WAVES
#define SLAYER_WGRAD_WAVES 4096
#endif
    const int64_t base = N * ((Co + 15) / 16) * Ho;
    const int64_t visits = (T + 63) / 64;
    int64_t parts = (SLAYER_WGRAD_WAVES + base - 1) / base;
    parts = parts > visits ? visits : (parts < 1 ? 1 : parts);
    const int64_t len = (visits + parts - 1) / parts * 64;
    p.tparts = (int)((T + len - 1) / len);
    p.tlen = (int)len;
    p.items = (int)(Ho * p.tparts);
}

}  // namespace

extern "C" int64_t slayer_conv_synapse_wgrad_workspace(int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W,
                                                       int64_t T, int64_t kh, int64_t kw, int64_t stride_h,
                                                       int64_t pad_h, int64_t dil_h) {
    if (N < 0 || Ci < 1 || Co < 1 || H < 1 || W < 1 || T < 0 || kh < 1 || kw < 1 || stride_h < 1 || pad_h < 0 ||
        dil_h < 1)
        return SLAYER_EINVAL;
    const int64_t Ho = (H + 2 * pad_h - dil_h * (kh - 1) - 1) / stride_h + 1;
    if (Ho < 1) return SLAYER_EINVAL;
    const int64_t K = Ci * kh * kw;
    if (K > 4096 || Ho > (1 << 20) || T > (1 << 24)) return SLAYER_ERANGE;
    // enough for either form of the kernel (which one runs depends on stride and dilation along the image row)
    int64_t need = 0;
    for (int64_t stride_w : {1, 2}) {
        const WgradForm f = wgrad_form(Ci, kh, kw, stride_w, 1);
        SynapseWgrad p;
        wgrad_shape(N, Ci, Co, Ho, T, kh, kw, f, p);
        const int64_t floats = (N * p.items + 2 * kWgradChunks) * ((Co + 15) / 16) * p.passes * f.tiles * 256;
        need = floats > need ? floats : need;
    }
    return need;
}

extern "C" int slayer_conv_synapse_wgrad(float* grad_weight, const float* grad_out, const float* in,
                                         int64_t N, int64_t Ci, int64_t Co, int64_t H, int64_t W, int64_t T,
                                         int64_t kh, int64_t kw, int64_t stride_h, int64_t stride_w,
                                         int64_t pad_h, int64_t pad_w, int64_t dil_h, int64_t dil_w,
                                         float* workspace, int64_t workspace_floats, void* stream) {
    if (N < 0 || Ci < 1 || Co < 1 || H < 1 || W < 1 || T < 0 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
        pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1)
        return SLAYER_EINVAL;
    const int64_t Ho = (H + 2 * pad_h - dil_h * (kh - 1) - 1) / stride_h + 1;
    const int64_t Wo = (W + 2 * pad_w - dil_w * (kw - 1) - 1) / stride_w + 1;
    if (Ho < 1 || Wo < 1) return SLAYER_EINVAL;
    if (!grad_weight) return SLAYER_ENULL;
    const int64_t K = Ci * kh * kw, lim = (int64_t)1 << 31;
    hipStream_t st = (hipStream_t)stream;
    if (N == 0 || T == 0) return launch_zero_fill(grad_weight, Co * K, st);
    if (!grad_out || !in || !workspace) return SLAYER_ENULL;
    if (T < 4 || !aligned16(workspace)) return SLAYER_ERANGE;
    if (Ci * H * W * T * 4 >= lim || Co * Ho * Wo * T * 4 >= lim || K > 4096 || pad_h > 4096 || pad_w > 4096 ||
        H * stride_h > (1 << 20) || W * stride_w > (1 << 20) || Ho > (1 << 20) || T > (1 << 24))
        return SLAYER_ERANGE;
    SynapseWgrad p;
    p.partial = workspace; p.grad_out = grad_out; p.in = in;
    p.N = (int)N; p.Ci = (int)Ci; p.Co = (int)Co; p.H = (int)H; p.W = (int)W; p.Ho = (int)Ho; p.Wo = (int)Wo; p.T = (int)T;
    p.kh = (int)kh; p.kw = (int)kw; p.sh = (int)stride_h; p.sw = (int)stride_w; p.ph = (int)pad_h; p.pw = (int)pad_w;
    p.dh = (int)dil_h; p.dw = (int)dil_w;
    p.K = (int)K;
    const WgradForm f = wgrad_form(Ci, kh, kw, stride_w, dil_w);
    wgrad_shape(N, Ci, Co, Ho, T, kh, kw, f, p);
    const int64_t cobs = (Co + 15) / 16;
    // the waves' tiles, then the chunk sums of the first reduction launch (doubles)
    const int64_t tile_floats = N * cobs * p.items * p.passes * f.tiles * 256;
    const int64_t stage_floats = 2 * kWgradChunks * cobs * p.passes * f.tiles * 256;
    if (workspace_floats < tile_floats + stage_floats) return SLAYER_ERANGE;
    double* stage = reinterpret_cast<double*>(workspace + tile_floats);
    const int64_t blocks = N * cobs * ((p.items + kSynWaves - 1) / kSynWaves);
    if (blocks > 0x7fffffffLL || p.passes > 65535) return SLAYER_ERANGE;
    const dim3 grid((unsigned)blocks, (unsigned)p.passes), block(kSynWaves * kWave);
    const bool tail = (T % 4) != 0;                                       // rows that end inside a quad
#define SLAYER_WGRAD(NTT)                                                                                              \
    do {                                                                                                               \
        if (tail) hipLaunchKernelGGL((synapse_wgrad_kernel<NTT, true>), grid, block, NTT * 16 * 3 * sizeof(int), st, p); \
        else hipLaunchKernelGGL((synapse_wgrad_kernel<NTT, false>), grid, block, NTT * 16 * 3 * sizeof(int), st, p);    \
    } while (0)
#define SLAYER_WGRAD_ROW(KW, NPT)                                                                                      \
    do {                                                                                                               \
        if (tail) hipLaunchKernelGGL((synapse_wgrad_row_kernel<KW, NPT, true>), grid, block, NPT * 16 * 2 * sizeof(int), st, p); \
        else hipLaunchKernelGGL((synapse_wgrad_row_kernel<KW, NPT, false>), grid, block, NPT * 16 * 2 * sizeof(int), st, p);    \
    } while (0)
    if (f.row_kw == 3) { if (f.npt == 1) SLAYER_WGRAD_ROW(3, 1); else SLAYER_WGRAD_ROW(3, 2); }
    else if (f.row_kw == 5) { if (f.npt == 1) SLAYER_WGRAD_ROW(5, 1); else SLAYER_WGRAD_ROW(5, 2); }
    else if (f.tiles == 1) SLAYER_WGRAD(1);
    else if (f.tiles == 2) SLAYER_WGRAD(2);
    else SLAYER_WGRAD(5);
#undef SLAYER_WGRAD_ROW
#undef SLAYER_WGRAD
    const unsigned tile_blocks = (unsigned)(cobs * p.passes * f.tiles);
    hipLaunchKernelGGL(synapse_wgrad_reduce_kernel, dim3(tile_blocks, kWgradChunks), dim3(kWgradParts * kWave), 0, st,
                       stage, workspace, (int)N, (int)Co, p.items, p.passes, f.tiles);
    hipLaunchKernelGGL(synapse_wgrad_final_kernel, dim3(tile_blocks), dim3(kWave), 0, st, grad_weight, stage, (int)Co,
                       (int)K, p.passes, f.tiles, f.row_kw, f.npt);
    return (int)hipGetLastError();
}

// The gradient of the input of slayer_conv_synapse for any stride (and, read as a layer of its own, the transposed
// convolution): one plain convolution per residue class of the pixels of grad_in, see SynapseConv.
extern "C" int slayer_conv_synapse_input_grad(float* grad_in, const float* grad_out, const float* weight_t,
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
    if (!grad_in || !grad_out || !weight_t) return SLAYER_ENULL;
    if (T < 4) return SLAYER_ERANGE;
    const int64_t K = Co * kh * kw, lim = (int64_t)1 << 31;
    if (Ci * H * W * T * 4 >= lim || Co * Ho * Wo * T * 4 >= lim || K > 4096 || pad_h > 4096 || pad_w > 4096 ||
        dil_h > 4096 || dil_w > 4096 || H + pad_h >= (1 << 16) || W + pad_w >= (1 << 16) || stride_h > 16 || stride_w > 16)
        return SLAYER_ERANGE;
    SynapseConv p;
    p.out = grad_in; p.in = grad_out; p.weight = weight_t;
    // in the kernels' names: the source is the gradient of the output, the result the gradient of the input
    p.N = (int)N; p.Ci = (int)Co; p.Co = (int)Ci; p.H = (int)Ho; p.W = (int)Wo; p.T = (int)T;
    p.sh = p.sw = 1;
    p.kh_full = (int)kh; p.kw_full = (int)kw; p.Ho_full = (int)H; p.Wo_full = (int)W;
    p.oys = (int)stride_h; p.oxs = (int)stride_w;
    const bool streaming = N * Ci * H * W * T * 4 > ((int64_t)64 << 20);
    {
        SynapseConv q = p;                                                // one channel: every class in one launch
        q.Ho = (int)H; q.Wo = (int)W; q.kh = (int)kh; q.kw = (int)kw; q.sh = (int)stride_h; q.sw = (int)stride_w;
        q.ph = (int)pad_h; q.pw = (int)pad_w; q.dh = (int)dil_h; q.dw = (int)dil_w;
        int code = 0;
        if (launch_synapse_plane(q, true, streaming, (hipStream_t)stream, &code)) return code;
    }
    for (int ry = 0; ry < (int)stride_h && ry < (int)H; ++ry) {
        const TapClass cy = tap_class(ry, (int)kh, (int)stride_h, (int)pad_h, (int)dil_h);
        for (int rx = 0; rx < (int)stride_w && rx < (int)W; ++rx) {
            const TapClass cx = tap_class(rx, (int)kw, (int)stride_w, (int)pad_w, (int)dil_w);
            p.oy0 = ry; p.ox0 = rx;
            p.Ho = ((int)H - ry + (int)stride_h - 1) / (int)stride_h;
            p.Wo = ((int)W - rx + (int)stride_w - 1) / (int)stride_w;
            const bool none = cy.count == 0 || cx.count == 0;            // pixels no tap reaches: zeros
            // the taps in the order of rising source coordinate: from the last one down, a step of
            // step * dil / stride pixels of the source each
            p.kh = none ? 0 : cy.count; p.kw = none ? 0 : cx.count;
            p.ky0 = cy.y_last; p.kys = -cy.step; p.kx0 = cx.y_last; p.kxs = -cx.step;
            p.dh = cy.count > 1 ? cy.step * (int)dil_h / (int)stride_h : 1;
            p.dw = cx.count > 1 ? cx.step * (int)dil_w / (int)stride_w : 1;
            p.ph = -cy.first; p.pw = -cx.first;
            const int code = launch_synapse_conv(p, streaming, (hipStream_t)stream);
            if (code != 0) return code;
        }
    }
    return 0;
}
