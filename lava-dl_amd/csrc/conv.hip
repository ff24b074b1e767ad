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
constexpr int kMaxTaps = 12288;          // window of 512 + K samples in 64 KB of LDS

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
// Matrix-core form for 8 < K <= 128 (T >= 16, M * T a whole number of quads, 16-byte aligned tensors).  The tensor is walked as one
// flat stream of M * T samples in tiles of 256 consecutive samples, each seen as 16 blocks of 16 output steps:
// D[i][n] = output 16 n + i of the tile is the [16 x (16 + KPAD)] Toeplitz matrix of taps times the
// [(16 + KPAD) x 16] matrix whose column n is the window of block n (v_mfma_f32_16x16x4_f32, four window samples
// per instruction).  With K = 64 the window is 80 samples, so 64 of 80 multiply-adds are useful (the FMA form
// above issues 82 instructions per 64 useful FMAs at half the rate).  The window of block n, shifted by 16
// samples, is the window of block n + 1: the B operands of all window groups are the same 256 (+ KPAD) samples,
// read at different offsets.  So a tile costs one wave-wide load of 1 KB of consecutive bytes (lane l: samples
// [4 l, 4 l + 4) of the tile), kept in an LDS ring of four tiles, and one wave-wide store that covers the tile's
// 1 KB (lane (kq, n) of the result holds the outputs 16 n + 4 kq .. + 3; passing the result through LDS to store
// in lane order as well changes nothing): whole 128-byte lines in both directions, every input byte fetched once
// (plus one tile per wave for the window of its first or last tile).
// In the ring a tile is stored quad-transposed (quad 4 n + kq at slot 16 kq + n), which makes the operand reads
// (lane (kq, n) reads slot 16 kq + n + g of group g, spilling into the neighbouring tile) conflict-free.
// The Toeplitz operands do not depend on the tile and stay in registers (4 per window group).
//
// Rows: a block's window must not see the neighbouring row.  Every lane masks the window quads of its block that
// lie outside the row of the block (it reads a quad of zeros instead).  Where rows are not whole quads (ANYT: T % 4
// != 0) a row begins or ends inside a quad: the samples of such a quad that belong to the other row are replaced by
// zeros one by one, and an output quad that straddles two rows takes each output from its own row's view.  A block that holds
// the end of one row and the start of the next (T % 16 != 0) needs both views: such a tile is multiplied twice,
// once with every block seeing the row of its first output and once the row of its last output, and every output
// quad takes the result of its own row.
// Window samples outside a filter's support meet a zero tap instead of being skipped, so an Inf or NaN in the
// input also reaches the up to 16 + KPAD - K neighbouring outputs of its row whose window holds it (0 * Inf);
// finite inputs, the only ones this path sees, give the same sums.
typedef float mfma_f4 __attribute__((ext_vector_type(4)));
typedef __bf16 mfma_bf8 __attribute__((ext_vector_type(8)));

constexpr int kConvTile = 256;             // samples per tile
constexpr int kConvRing = 4;               // tiles in the LDS ring = tiles per loop pass

// A float as the sum of three bfloat16 numbers, each the rounding to nearest of what the parts before it leave
// (|second| <= 2^-9, |third| <= 2^-18 of the value, what the three leave out <= 2^-27), four floats at a time:
// part t of the quad as four bfloat16 in two dwords.
struct SplitQuad { uint2 part[3]; };
typedef __bf16 conv_bf2 __attribute__((ext_vector_type(2)));
typedef float conv_f2 __attribute__((ext_vector_type(2)));
// two floats rounded to bfloat16 in one dword; a and b become what the rounding left
__device__ __forceinline__ unsigned round_pair(float& a, float& b) {
    const conv_bf2 h = __builtin_convertvector(conv_f2{a, b}, conv_bf2);
    const conv_f2 back = __builtin_convertvector(h, conv_f2);
    a -= back.x;
    b -= back.y;
    return __builtin_bit_cast(unsigned, h);
}
// A finite float beyond the largest bfloat16 (3.3895e38 .. 3.4028e38) rounds to an infinite first part, and what
// that leaves is an infinity of the other sign -- which nothing else produces (an infinite or NaN value leaves a
// NaN), so it marks exactly this case.  Such a value then takes the largest bfloat16 as its first part instead; the
// parts after it hold the rest as usual.  Rare: a wave-uniform branch that no ordinary tensor enters.
__device__ __forceinline__ bool is_inf(float x) { return __builtin_isinf(x); }
__device__ __forceinline__ void clamp_first_part(float orig, float& rest, unsigned& pair, int half) {
    if (is_inf(rest)) {
        const unsigned top = (__float_as_uint(orig) >> 16 & 0x8000u) | 0x7f7fu;      // +-3.3895e38 as bfloat16
        pair = half ? (pair & 0x0000ffffu) | (top << 16) : (pair & 0xffff0000u) | top;
        rest = orig - __uint_as_float(top << 16);
    }
}
__device__ __forceinline__ SplitQuad split_quad(float4 v) {
    SplitQuad q;
    const float4 orig = v;
    q.part[0].x = round_pair(v.x, v.y);
    q.part[0].y = round_pair(v.z, v.w);
    if (__any(is_inf(v.x) || is_inf(v.y) || is_inf(v.z) || is_inf(v.w))) {
        clamp_first_part(orig.x, v.x, q.part[0].x, 0);
        clamp_first_part(orig.y, v.y, q.part[0].x, 1);
        clamp_first_part(orig.z, v.z, q.part[0].y, 0);
        clamp_first_part(orig.w, v.w, q.part[0].y, 1);
    }
#pragma unroll
    for (int t = 1; t < 3; ++t) {
        q.part[t].x = round_pair(v.x, v.y);
        q.part[t].y = round_pair(v.z, v.w);
    }
    return q;
}
// d += A * B over 32 window samples (two quads per lane).  An odd last group is paired with zeros rather than given
// to the 16-sample instruction: that instruction, fed the accumulator of a 32-sample one, returned half of the
// accumulator without the products of the instruction before it on this toolchain.
__device__ __forceinline__ mfma_f4 mfma_pair(uint2 a0, uint2 a1, uint2 b0, uint2 b1, mfma_f4 d) {
    const uint4 a = make_uint4(a0.x, a0.y, a1.x, a1.y), b = make_uint4(b0.x, b0.y, b1.x, b1.y);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mfma_bf8, a), __builtin_bit_cast(mfma_bf8, b), d, 0, 0, 0);
}

// What both matrix kernels share: the tiles of a wave, its addressing and the ring slots of its operands.
template <int KPAD, bool CORR>
struct ConvWave {
    static constexpr int G = KPAD / 16 + 1;        // window groups of 16 samples per block
    static constexpr int kZero = kConvRing * 64;   // ring slot that holds a quad of zeros
    // Step s writes tile w0 + s into the ring (w0 = -1: the conv window reaches back into the previous tile;
    // corr reaches forward, so its tile s is written one step before tile s - 1 is computed) and computes tile
    // s - 1.  Loads run kConvRing steps ahead of their ring write, in registers.
    static constexpr int w0 = CORR ? 0 : -1;
    int lane, n, kq;
    int mine, lead, floor0, lend, steps, wslot, wq;
    int opnd[G];
    __amdgpu_buffer_rsrc_t src, dst;

    __device__ __forceinline__ void init(float* out, const float* in, int64_t total, int T, int tiles_per_wave) {
        lane = threadIdx.x;
        n = lane & 15;
        kq = lane >> 4;
        // this wave's tiles: samples [first, last) of the flat tensor; its accesses are relative to the row that
        // holds `first`, through a descriptor that ends with the tensor
        const int64_t first = (int64_t)blockIdx.x * tiles_per_wave * kConvTile;
        const int64_t rest = total - first;
        mine = (int)(rest < (int64_t)tiles_per_wave * kConvTile ? rest : (int64_t)tiles_per_wave * kConvTile);
        const int64_t row0 = first / T;
        lead = (int)(first - row0 * T);                 // samples of row0 in front of `first`
        // offsets below are relative to `origin`, one tile in front of `first` (the conv window reaches back)
        const int64_t origin = first - kConvTile;
        const int64_t avail = total - origin;           // samples from origin to the end of the tensor
        const int bound = (int)(avail < (int64_t)(tiles_per_wave + 2) * kConvTile ? avail
                                                                                  : (int64_t)(tiles_per_wave + 2) * kConvTile);
        src = make_rsrc(in + origin, (unsigned)bound * 4u);
        dst = make_rsrc(out + origin, (unsigned)bound * 4u);
        floor0 = origin < 0 ? kConvTile : 0;            // nothing in front of the tensor
        // Ring slot (in quads) of the operand of group g, relative to the ring position of the tile being computed:
        // the window of block n starts KPAD samples before the block (conv) or with it (corr), so group g is block
        // b = n + g - KPAD / 16 (conv) or n + g (corr) of the tile, or of its neighbour when b leaves [0, 16).
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int b = n + g - (CORR ? 0 : KPAD / 16);
            const int tile = b < 0 ? -1 : (b >= 16 ? 1 : 0);
            opnd[g] = ((tile * 64 + 16 * kq + (b - 16 * tile)) + kConvRing * 64) & (kConvRing * 64 - 1);
        }
        wslot = 16 * (lane & 3) + (lane >> 2);          // where this lane's loaded quad goes within a tile
        // sample (relative to `first`) of the first window quad of this lane: group g adds 16 g
        wq = 16 * n + 4 * kq - (CORR ? 0 : KPAD);
        lend = kConvTile + mine + (CORR ? kConvTile : 0);   // relative to origin: last sample a tile may read
        steps = (mine + kConvTile - 1) / kConvTile + 1;
    }
    // Toeplitz operand: the tap that links output step n of a block with window sample 16 g + 4 kq + r
    __device__ __forceinline__ float tap(const float* filt, int K, int g, int r) const {
        const int idx = CORR ? (16 * g + 4 * kq + r) - n : n + KPAD - (16 * g + 4 * kq + r);
        return (idx >= 0 && idx < K) ? filt[idx] : 0.0f;
    }
    // this lane's quad of a tile of the wave (tile -1 / tile count: the neighbours the windows reach into)
    __device__ __forceinline__ float4 load(int tile) const {
        const int t = (tile + 1) * kConvTile + 4 * lane;          // relative to origin
        return buf_load4<false>(src, (t >= floor0 && t < lend) ? t * 4 : kOutOfRange);
    }
};

template <int KPAD, bool CORR, bool ANYT = false>
__global__ __launch_bounds__(kWave) void conv_mfma_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                          const float* __restrict__ filt, int K, float ts,
                                                          int64_t total, int T, int tiles_per_wave) {
    using W = ConvWave<KPAD, CORR>;
    constexpr int G = W::G, kZero = W::kZero, w0 = W::w0;
    __shared__ __attribute__((aligned(16))) float4 ring[kConvRing * 64 + 1];
    W wv;
    wv.init(out, in, total, T, tiles_per_wave);
    const int lane = wv.lane, n = wv.n, kq = wv.kq, mine = wv.mine, lead = wv.lead, wslot = wv.wslot, wq = wv.wq;
    const int* opnd = wv.opnd;
    const __amdgpu_buffer_rsrc_t dst = wv.dst;
    if (lane == 0) ring[kZero] = make_float4(0.f, 0.f, 0.f, 0.f);
    float a[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) a[g][r] = wv.tap(filt, K, g, r);
    auto load = [&](int tile) -> float4 { return wv.load(tile); };
    float4 stage[kConvRing];
    // each load is preceded by a store that falls out of range (dropped by the hardware): the loop is then
    // entered in the state its back edge leaves, and the wait at its top can leave the youngest loads in
    // flight instead of draining everything
#pragma unroll
    for (int u = 0; u < kConvRing; ++u) {
        buf_store4<false>(dst, kOutOfRange + 16 * u, make_float4(0.f, 0.f, 0.f, 0.f));
        stage[u] = load(w0 + u);
    }
    const int steps = wv.steps;
    for (int s0 = 0; s0 < steps; s0 += kConvRing) {
#pragma unroll
        for (int u = 0; u < kConvRing; ++u) {
            // ring position of tile w0 + s is (s & 3) = u: s0 is a multiple of the ring length
            ring[u * 64 + wslot] = stage[u];
            stage[u] = load(w0 + s0 + u + kConvRing);
            // tile s - 1 sits at ring position (u - 1 - w0) & 3
            const int here = ((u - 1 - w0 + kConvRing) & (kConvRing - 1)) * 64;
            // the first step computes no tile and the last pass may hold steps past the end of the wave's tiles:
            // they skip the matrix work (a wave-uniform branch without memory instructions inside) and store
            // out of range
            const int tile0 = (s0 + u - 1) * kConvTile;               // relative to `first`
            mfma_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
            if (s0 + u >= 1 && tile0 < mine) {
                // rows of the first and the last output of this lane's block, as sample ranges relative to `first`
                const int o0 = tile0 + 16 * n + lead;                 // relative to the start of row0
                const int ra = o0 / T;
                const int lo_a = ra * T - lead, rb_more = (o0 - ra * T + 15 >= T) ? T : 0;
                auto multiply = [&](mfma_f4 d, int g, int lo) -> mfma_f4 {
                    const int q = tile0 + wq + 16 * g;                // first sample of the quad
                    const bool ok = ANYT ? (q + 3 >= lo && q < lo + T) : (q >= lo && q < lo + T);
                    float4 xv = ring[ok ? ((here + opnd[g]) & (kConvRing * 64 - 1)) : kZero];
                    if (ANYT) {                                       // a row may begin or end inside the quad
                        const unsigned rel = (unsigned)(q - lo);
                        xv.x = rel < (unsigned)T ? xv.x : 0.0f;
                        xv.y = rel + 1u < (unsigned)T ? xv.y : 0.0f;
                        xv.z = rel + 2u < (unsigned)T ? xv.z : 0.0f;
                        xv.w = rel + 3u < (unsigned)T ? xv.w : 0.0f;
                    }
                    d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][0], xv.x, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][1], xv.y, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][2], xv.z, d, 0, 0, 0);
                    return __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][3], xv.w, d, 0, 0, 0);
                };
                // every block sees the row of its first output (conv) or of its last output (corr) ...
                const int lo_full = lo_a + (CORR ? rb_more : 0);
#pragma unroll
                for (int g = 0; g < G; ++g) acc = multiply(acc, g, lo_full);
                // ... and the outputs of a block's other row take their own view.  They are the last outputs
                // of the previous row (corr) or the first ones of the next row (conv), and inside their row their
                // window holds samples of this block only: one window group, the block itself.
                if (__any(rb_more != 0)) {
                    mfma_f4 other = {0.0f, 0.0f, 0.0f, 0.0f};
                    other = multiply(other, CORR ? 0 : G - 1, lo_a + (CORR ? 0 : rb_more));
                    const int oq = tile0 + 16 * n + 4 * kq;           // this lane's output quad
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool in_next = oq + (ANYT ? j : 0) >= lo_a + T;
                        acc[j] = (rb_more != 0 && in_next != CORR) ? other[j] : acc[j];
                    }
                }
            }
            const int t = tile0 + 16 * n + 4 * kq;
            buf_store4<false>(dst, (s0 + u >= 1 && t < mine) ? (t + kConvTile) * 4 : kOutOfRange,
                              make_float4(acc[0] * ts, acc[1] * ts, acc[2] * ts, acc[3] * ts));
        }
    }
}

// The same kernel for more than 32 taps, where the float instruction (one pass of the matrix pipe per 4 window
// samples) is what bounds it: every tap and every sample is split into three bfloat16 parts that add up to it
// to within 2^-27 (each part the rounding to nearest of what the parts before it leave), and the products of the
// parts are taken with the bfloat16 instruction (one pass per 32 window samples: two window groups at a time) --
// part i of the taps with part j of the samples for i + j <= 2, six products, each exact, summed in float32.  What
// is left out (i + j >= 3 and the remainders) is below 2^-25 of a product: less than the rounding of a float sum.
// The parts are made once per sample on the way into the ring (three planes of four bfloat16 per quad).
// A part that is zero in every lane of a tile and its neighbour (wave-uniform: spikes, small
// integers, anything of at most 8 significant bits has no second and third part) is left out together with its
// products, which then are exactly zero: such inputs cost three products instead of six.
// Range: a finite value beyond the largest bfloat16 (3.3895e38) takes that as its first part (split_quad), so
// every finite float32 is covered; parts below the smallest normal float32 are lost, so a tap or sample below about
// 3e-33 in magnitude enters with an absolute error of up to 1.2e-38 (3.38e38 * 1e-38 gives 3.3834).
// Measured against the float form (conv on 3 % spikes / corr on normal random data, us): [524288,300] K = 64
// 293 / 307 -> 265 / 306, K = 128 464 / 469 -> 310 / 422; [65536,2000] K = 64 245 / 255 -> 221 / 241, K = 128
// 350 / 361 -> 228 / 316; [8192,1500] K = 64 36 / 30 -> 32 / 31.  Up to 32 taps the float form is as fast or
// faster (memory-bound; the split costs about 25 vector instructions per quad) and stays.
template <int KPAD, bool CORR, bool ANYT = false>
__global__ __launch_bounds__(kWave) void conv_mfma_split_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                          const float* __restrict__ filt, int K, float ts,
                                                          int64_t total, int T, int tiles_per_wave) {
    using W = ConvWave<KPAD, CORR>;
    constexpr int G = W::G, kZero = W::kZero, w0 = W::w0;
    __shared__ __attribute__((aligned(16))) uint2 ring[3][kConvRing * 64 + 2];
    W wv;
    wv.init(out, in, total, T, tiles_per_wave);
    const int lane = wv.lane, n = wv.n, kq = wv.kq, mine = wv.mine, lead = wv.lead, wslot = wv.wslot, wq = wv.wq;
    const int* opnd = wv.opnd;
    const __amdgpu_buffer_rsrc_t dst = wv.dst;
    if (lane < 3) ring[lane][kZero] = make_uint2(0u, 0u);
    // the taps in three parts, and whether any lane holds a non-zero second / third part of a tap
    SplitQuad a[G];
    bool a_part[3] = {true, false, false};
#pragma unroll
    for (int g = 0; g < G; ++g) {
        a[g] = split_quad(make_float4(wv.tap(filt, K, g, 0), wv.tap(filt, K, g, 1), wv.tap(filt, K, g, 2), wv.tap(filt, K, g, 3)));
        a_part[1] = a_part[1] || __any((a[g].part[1].x | a[g].part[1].y) != 0u);
        a_part[2] = a_part[2] || __any((a[g].part[2].x | a[g].part[2].y) != 0u);
    }
    auto load = [&](int tile) -> float4 { return wv.load(tile); };
    float4 stage[kConvRing];
    // does the tile at a ring position hold a non-zero second / third part?  (Spikes and other values of at most
    // eight significant bits do not: their products with those parts are left out.)
    bool mid_at[kConvRing] = {false, false, false, false}, low_at[kConvRing] = {false, false, false, false};
    // each load is preceded by a store that falls out of range (dropped by the hardware): the loop is then
    // entered in the state its back edge leaves, and the wait at its top can leave the youngest loads in
    // flight instead of draining everything
#pragma unroll
    for (int u = 0; u < kConvRing; ++u) {
        buf_store4<false>(dst, kOutOfRange + 16 * u, make_float4(0.f, 0.f, 0.f, 0.f));
        stage[u] = load(w0 + u);
    }
    const int steps = wv.steps;
    for (int s0 = 0; s0 < steps; s0 += kConvRing) {
#pragma unroll
        for (int u = 0; u < kConvRing; ++u) {
            // ring position of tile w0 + s is (s & 3) = u: s0 is a multiple of the ring length
            {
                const SplitQuad q = split_quad(stage[u]);
                ring[0][u * 64 + wslot] = q.part[0];
                ring[1][u * 64 + wslot] = q.part[1];
                ring[2][u * 64 + wslot] = q.part[2];
                mid_at[u] = __any((q.part[1].x | q.part[1].y) != 0u);
                low_at[u] = __any((q.part[2].x | q.part[2].y) != 0u);
            }
            stage[u] = load(w0 + s0 + u + kConvRing);
            // tile s - 1 sits at ring position (u - 1 - w0) & 3; its windows reach into the tile before it (conv)
            // or after it (corr)
            constexpr int kRingMask = kConvRing - 1;
            const int at = (u - 1 - w0 + kConvRing) & kRingMask, beside = (at + (CORR ? 1 : kConvRing - 1)) & kRingMask;
            const int here = at * 64;
            const bool b_part[3] = {true, mid_at[at] || mid_at[beside], low_at[at] || low_at[beside]};
            // the first step computes no tile and the last pass may hold steps past the end of the wave's tiles:
            // they skip the matrix work (a wave-uniform branch without memory instructions inside) and store
            // out of range
            const int tile0 = (s0 + u - 1) * kConvTile;               // relative to `first`
            mfma_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
            if (s0 + u >= 1 && tile0 < mine) {
                // rows of the first and the last output of this lane's block, as sample ranges relative to `first`
                const int o0 = tile0 + 16 * n + lead;                 // relative to the start of row0
                const int ra = o0 / T;
                const int lo_a = ra * T - lead, rb_more = (o0 - ra * T + 15 >= T) ? T : 0;
                // slot of the window quad of group g as the row [lo, lo + T) sees it, and which of its samples the
                // row holds (ANYT: a row may begin or end inside the quad), as masks over the two dwords
                auto slot_of = [&](int g, int lo, uint2& keep) -> int {
                    const int q = tile0 + wq + 16 * g;                // first sample of the quad
                    const bool ok = ANYT ? (q + 3 >= lo && q < lo + T) : (q >= lo && q < lo + T);
                    if (ANYT) {
                        const unsigned rel = (unsigned)(q - lo);
                        keep.x = (rel < (unsigned)T ? 0x0000ffffu : 0u) | (rel + 1u < (unsigned)T ? 0xffff0000u : 0u);
                        keep.y = (rel + 2u < (unsigned)T ? 0x0000ffffu : 0u) | (rel + 3u < (unsigned)T ? 0xffff0000u : 0u);
                    }
                    return ok ? ((here + opnd[g]) & (kConvRing * 64 - 1)) : kZero;
                };
                // the products of the parts of the taps with the parts of the samples over the window groups [g0, g1)
                auto multiply = [&](mfma_f4 d, int g0, int g1, int lo) -> mfma_f4 {
                    int slot[G];
                    uint2 keep[G];
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        if (g >= g0 && g < g1) slot[g] = slot_of(g, lo, keep[g]);
                    auto term = [&](mfma_f4 d, int ta, int tb) -> mfma_f4 {
                        uint2 x[G];
#pragma unroll
                        for (int g = 0; g < G; ++g)
                            if (g >= g0 && g < g1) {
                                x[g] = ring[tb][slot[g]];
                                if (ANYT) { x[g].x &= keep[g].x; x[g].y &= keep[g].y; }
                            }
#pragma unroll
                        for (int h = 0; h < (G + 1) / 2; ++h) {            // two groups per instruction
                            const int g = g0 + 2 * h;
                            if (g + 1 < g1) d = mfma_pair(a[g].part[ta], a[g + 1].part[ta], x[g], x[g + 1], d);
                            else if (g < g1) d = mfma_pair(a[g].part[ta], make_uint2(0u, 0u), x[g], make_uint2(0u, 0u), d);
                        }
                        return d;
                    };
                    // smallest products first; parts that are zero throughout (wave-uniform) are left out.  (Reading
                    // every part of the samples once and keeping two accumulators is slower at K = 64: 376 -> 395 us
                    // on 524 288 rows of 300 dense samples.)
                    if (a_part[2]) d = term(d, 2, 0);
                    if (a_part[1] && b_part[1]) d = term(d, 1, 1);
                    if (b_part[2]) d = term(d, 0, 2);
                    if (a_part[1]) d = term(d, 1, 0);
                    if (b_part[1]) d = term(d, 0, 1);
                    return term(d, 0, 0);
                };
                // every block sees the row of its first output (conv) or of its last output (corr) ...
                acc = multiply(acc, 0, G, lo_a + (CORR ? rb_more : 0));
                // ... and the outputs of a block's other row take their own view.  They are the last outputs
                // of the previous row (corr) or the first ones of the next row (conv), and inside their row their
                // window holds samples of this block only: one window group, the block itself.
                if (__any(rb_more != 0)) {
                    mfma_f4 other = {0.0f, 0.0f, 0.0f, 0.0f};
                    constexpr int gb = CORR ? 0 : G - 1;
                    other = multiply(other, gb, gb + 1, lo_a + (CORR ? 0 : rb_more));
                    const int oq = tile0 + 16 * n + 4 * kq;           // this lane's output quad
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool in_next = oq + (ANYT ? j : 0) >= lo_a + T;
                        acc[j] = (rb_more != 0 && in_next != CORR) ? other[j] : acc[j];
                    }
                }
            }
            const int t = tile0 + 16 * n + 4 * kq;
            buf_store4<false>(dst, (s0 + u >= 1 && t < mine) ? (t + kConvTile) * 4 : kOutOfRange,
                              make_float4(acc[0] * ts, acc[1] * ts, acc[2] * ts, acc[3] * ts));
        }
    }
}

template <bool CORR, bool ANYT>
static int conv_mfma_launch(float* out, const float* in, const float* filt, int K, float ts, int64_t M, int64_t T,
                            hipStream_t stream) {
    // Tiles per wave (a whole number of loop passes of consecutive tiles; every wave reads one tile more than it
    // writes): few, so that the waves in flight together walk the tensor as one narrow front -- up to 16 taps, where
    // a wave's set-up is 8 tap loads, 8 tiles per wave run at 5.7-6.0 TB/s against 4.8 with 64 ([524288,300]
    // 260 -> 217 us, [65536,2000] 212 -> 182 us) -- but enough to pay for the set-up of the longer filters (20 to
    // 36 tap loads and their split: 32 tiles, 330 -> 276 us against 8 at K = 64), and no more than leaves about
    // three thousand waves to a small tensor ([8192,1500], K = 64: 30.1 us with 8 tiles, 27.7 with 12-16, 34.7 with 32).
    const int64_t total = M * T;
    const int64_t tiles = (total + kConvTile - 1) / kConvTile;
    const int64_t cap = K <= 16 ? 8 : 32;
    int64_t per_wave = (tiles / 3072 + kConvRing - 1) / kConvRing * kConvRing;
    if (per_wave < kConvRing) per_wave = kConvRing;
    if (per_wave > cap) per_wave = cap;
    const int64_t blocks = (tiles + per_wave - 1) / per_wave;
    if (blocks > 0x7fffffffLL) return SLAYER_ERANGE;
#define SLAYER_CONV_MFMA(KP)                                                                                      \
    hipLaunchKernelGGL((conv_mfma_kernel<KP, CORR, ANYT>), dim3((unsigned)blocks), dim3(kWave), 0, stream, out, in, filt, \
                       K, ts, total, (int)T, (int)per_wave)
#define SLAYER_CONV_MFMA_SPLIT(KP)                                                                                \
    hipLaunchKernelGGL((conv_mfma_split_kernel<KP, CORR, ANYT>), dim3((unsigned)blocks), dim3(kWave), 0, stream, out, \
                       in, filt, K, ts, total, (int)T, (int)per_wave)
    // up to 32 taps the float instructions keep up with memory; beyond that the three-part bfloat16 form is faster
    if (K <= 16) SLAYER_CONV_MFMA(16);
    else if (K <= 32) SLAYER_CONV_MFMA(32);
    else if (K <= 64) SLAYER_CONV_MFMA_SPLIT(64);
    else SLAYER_CONV_MFMA_SPLIT(128);
#undef SLAYER_CONV_MFMA_SPLIT
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
    // tap i meets sample t - i (conv) or t + i (corr) of the same row: taps from T on meet nothing and are not read
    // (the reference's kernels skip them one by one, utils/filter/conv.cu:42-46)
    if (K > T) K = T;
    if (K > kMaxTaps) return SLAYER_ERANGE;
    // the matrix kernel walks the tensor as one flat stream of whole quads: rows of any length from 16 steps on, as
    // long as the tensor as a whole is a whole number of quads
    if (K > 8 && K <= 128 && (M * T) % 4 == 0 && T >= 16 && T <= (1 << 22) && aligned16(out) && aligned16(in))
        return T % 4 == 0 ? conv_mfma_launch<CORR, false>(out, in, filt, (int)K, ts, M, T, stream)
                          : conv_mfma_launch<CORR, true>(out, in, filt, (int)K, ts, M, T, stream);
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
