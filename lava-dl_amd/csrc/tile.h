// Neuron x time-chunk streaming engine shared by every sequential-in-time kernel.
//
// Tensors are [M][T] float32 with time innermost.  One 64-lane wavefront (one
// workgroup) owns 64 consecutive neurons (rows) and walks the time axis in chunks
// of TC steps (TC = 32 for 64 rows):
//
//   global --dwordx4, coalesced along time--> registers --ds_write_b128--> LDS tile
//   LDS tile: lane j runs the recurrence over row j, 4 steps per ds_read_b128,
//             results overwrite the tile in place (ds_write_b128)
//   LDS tile --ds_read_b128--> registers --dwordx4, coalesced--> global
//
// The loads for chunk k+1 are issued before chunk k is computed, so HBM latency
// hides behind the sequential arithmetic.  Rows are padded by 4 floats (16 B):
// with a pitch of TC+4 floats both access patterns (lane = (row, quad) for the
// copies; lane = row for the recurrence) touch 8 distinct 16-byte bank groups
// per 8 consecutive lanes, i.e. they run at the conflict-free b128 rate.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace slayer {

constexpr int kWave = 64;

// (a * b) >> 12 rounded toward zero.  The 64-bit product is biased by 4095 when it is
// negative; its sign is the sign bit of a ^ b whenever the product is non-zero, and a
// zero product gives 0 with either bias, so no second multiply is needed for the sign.
__device__ __forceinline__ int rs0_12(int a, int b) {
    const long long bias = (long long)(((a ^ b) >> 31) & 4095);
    return (int)(((long long)a * (long long)b + bias) >> 12);
}

// Streaming (non-temporal) 16-byte global accesses: tensors on this path are read once and
// written once, so they should not displace each other in L2.
typedef float vf4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load4(const float* p, bool streaming) {
    if (streaming) {
        const vf4 v = __builtin_nontemporal_load(reinterpret_cast<const vf4*>(p));
        return make_float4(v.x, v.y, v.z, v.w);
    }
    return *reinterpret_cast<const float4*>(p);
}
__device__ __forceinline__ void store4(float* p, float4 v, bool streaming) {
    if (streaming) {
        vf4 u; u.x = v.x; u.y = v.y; u.z = v.z; u.w = v.w;
        __builtin_nontemporal_store(u, reinterpret_cast<vf4*>(p));
    } else {
        *reinterpret_cast<float4*>(p) = v;
    }
}

// float32 -> int32 toward zero; out-of-range values saturate (v_cvt_i32_f32).
__device__ __forceinline__ int trunc_i32(float x) { return (int)x; }

__device__ __forceinline__ int64_t param_index(int64_t m, int64_t npb, int64_t num_params) {
    return num_params > 1 ? (m % npb) / (npb / num_params) : 0;
}

// A tile is R rows x TC steps with R * TC = 2048 samples (8 KB per tensor): R = 64 rows when
// there are plenty of neurons, fewer rows and longer chunks when there are few, so that small
// problems still spread over all compute units (lanes >= R only help with the copies).
constexpr int kTileSamples = 2048;

template <int R>
struct TileGeom {
    static constexpr int kRows = R;
    static constexpr int kChunk = kTileSamples / R;          // TC: steps per chunk
    static_assert(R == 64 || R == 32 || R == 16, "rows per wave");
    static constexpr int kPitch = kChunk + 4;                // floats per LDS row
    static constexpr int kQuads = kChunk / 4;                // float4 per row
    static constexpr int kRowsPerPass = kWave / kQuads;      // rows one wave-wide access covers
    static constexpr int kPasses = R / kRowsPerPass;
    static_assert(kRowsPerPass >= 1 && kPasses >= 1, "tile geometry");
    static constexpr int kTileFloats = R * kPitch;
};

// An Op provides:
//   static constexpr int kIn, kOut;  static constexpr bool kReverse;
//   static constexpr int64_t kRows32Below, kRows16Below;   (rows-per-wave policy, see launch_stream)
//   struct Params { const float* in[kIn]; float* out[kOut]; ... };
//   __device__ void init(const Params&, int64_t m, bool valid);
//   __device__ void step(const float (&x)[kIn], float (&y)[kOut]);
//   __device__ void finish(const Params&, int64_t m, bool valid);
//
// Line alignment (VEC4 path).  A row of T floats starts wherever m*T falls, so a fixed
// time grid would cut every row segment across 128-byte lines and each line would be
// fetched (and partially written) twice.  Instead every row gets its own phase
// a = (float index of the row start) mod 32 and tile column j of chunk k holds step
// t = k*TC + j - a: the segments a wave-wide access touches then start on 128-byte
// boundaries.  Lanes simply skip the columns that fall before step 0 or after step T-1.
//
// Boundary lines (VEC4 path).  Unless T is a multiple of 32, the last line of row r is also
// the first line of row r+1.  Writing it in two pieces at two different times costs a
// read-modify-write in memory for each piece (measured: ~16% of the kernel at T = 300), so
// output quads that fall in such a shared line are collected in an LDS buffer of 65 lines
// (one per row boundary of the wave) and written once, whole, after the last chunk.  Only
// the two lines shared with neighbouring workgroups are still written in pieces.
template <class Op, int R, bool VEC4, bool STREAM>
__global__ __launch_bounds__(kWave) void stream_kernel(typename Op::Params prm, int64_t M, int T) {
    using G = TileGeom<R>;
    constexpr int TC = G::kChunk;
    constexpr int NI = Op::kIn, NO = Op::kOut, NT = NI > NO ? NI : NO;
    __shared__ __attribute__((aligned(16))) float tile[NT][G::kTileFloats];
    __shared__ __attribute__((aligned(16))) float bline[VEC4 ? NO : 1][VEC4 ? (R + 1) * 32 : 4];

    const int lane = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.x * R;
    const int rows = (int)((M - m0) < R ? (M - m0) : R);

    Op op;
    op.init(prm, m0 + lane, lane < rows);

    // phase of a row: float index of its first sample modulo one 128-byte line
    const unsigned base_f = (unsigned)(reinterpret_cast<uintptr_t>(prm.in[0]) >> 2);
    auto phase = [&](int r) -> int {
        return VEC4 ? (int)((base_f + (unsigned)(m0 + r) * (unsigned)T) & 31u) : 0;
    };
    const int a_lane = phase(lane);

    int last = (lane < rows) ? (a_lane + T - 1) / TC : 0;    // last chunk this row needs
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_xor(last, d);
        last = o > last ? o : last;
    }
    const int nchunks = last + 1;

    // rows shorter than a line could start and end inside the same line; they keep direct stores
    const bool route = VEC4 && T >= 32;

    const int crow = lane / G::kQuads;      // row within a pass (copy pattern)
    const int cq = lane % G::kQuads;        // quad within the row

    float4 stage[NI][G::kPasses];

    auto fetch = [&](int chunk) {
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
            const int t = chunk * TC + 4 * cq - phase(r);
            const int64_t off = (int64_t)(m0 + r) * (int64_t)T + (int64_t)t;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < rows) {
                    const float* src = prm.in[i] + off;
                    if (VEC4) {
                        if (t >= 0 && t < T) v = load4(src, STREAM);
                    } else {
                        if (t + 0 < T) v.x = src[0];
                        if (t + 1 < T) v.y = src[1];
                        if (t + 2 < T) v.z = src[2];
                        if (t + 3 < T) v.w = src[3];
                    }
                }
                stage[i][p] = v;
            }
        }
    };

    fetch(Op::kReverse ? nchunks - 1 : 0);

    for (int k = 0; k < nchunks; ++k) {
        const int chunk = Op::kReverse ? nchunks - 1 - k : k;

        // staged registers -> LDS
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
#pragma unroll
            for (int i = 0; i < NI; ++i)
                *reinterpret_cast<float4*>(&tile[i][r * G::kPitch + 4 * cq]) = stage[i][p];
        }
        __syncthreads();

        if (k + 1 < nchunks) fetch(Op::kReverse ? chunk - 1 : chunk + 1);

        // sequential recurrence: lane = neuron; columns outside [0, T) are skipped
        const int tl = chunk * TC - a_lane;           // step held by column 0 of this lane's row
#pragma unroll 2
        for (int q = 0; q < G::kQuads; ++q) {
            const int qq = Op::kReverse ? G::kQuads - 1 - q : q;
            const int t = tl + 4 * qq;
            if (lane < R && t >= 0 && t < T) {
                float xin[NI][4], yout[NO][4];
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const float4 v = *reinterpret_cast<const float4*>(&tile[i][lane * G::kPitch + 4 * qq]);
                    xin[i][0] = v.x; xin[i][1] = v.y; xin[i][2] = v.z; xin[i][3] = v.w;
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int ss = Op::kReverse ? 3 - s : s;
                    float x[NI], y[NO];
#pragma unroll
                    for (int i = 0; i < NI; ++i) x[i] = xin[i][ss];
                    op.step(x, y);
#pragma unroll
                    for (int o = 0; o < NO; ++o) yout[o][ss] = y[o];
                }
#pragma unroll
                for (int o = 0; o < NO; ++o)
                    *reinterpret_cast<float4*>(&tile[o][lane * G::kPitch + 4 * qq]) =
                        make_float4(yout[o][0], yout[o][1], yout[o][2], yout[o][3]);
            }
        }
        __syncthreads();

        // LDS -> global (quads of a line shared with a neighbouring row go to the boundary buffer)
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
            const int a = phase(r);
            const int pos = chunk * TC + 4 * cq;          // position in the row's line-aligned window
            const int t = pos - a;
            const int64_t off = (int64_t)(m0 + r) * (int64_t)T + (int64_t)t;
            const int end = a + T;                        // window position one past the last step
            const int last_full = end & ~31;
#pragma unroll
            for (int o = 0; o < NO; ++o) {
                const float4 v = *reinterpret_cast<const float4*>(&tile[o][r * G::kPitch + 4 * cq]);
                if (r < rows) {
                    float* dst = prm.out[o] + off;
                    if (VEC4) {
                        if (t >= 0 && t < T) {
                            if (route && a != 0 && pos < 32)
                                *reinterpret_cast<float4*>(&bline[o][r * 32 + pos]) = v;
                            else if (route && pos >= last_full)   // only when end is not a line multiple
                                *reinterpret_cast<float4*>(&bline[o][(r + 1) * 32 + (pos - last_full)]) = v;
                            else
                                store4(dst, v, STREAM);
                        }
                    } else {
                        if (t + 0 < T) dst[0] = v.x;
                        if (t + 1 < T) dst[1] = v.y;
                        if (t + 2 < T) dst[2] = v.z;
                        if (t + 3 < T) dst[3] = v.w;
                    }
                }
            }
        }
        __syncthreads();
    }

    if (route) {
        // boundary line b holds the tail of row b-1 (columns < phase(b)) and the head of row b
        for (int i = lane; i < (R + 1) * 8; i += kWave) {
            const int b = i >> 3, col = (i & 7) * 4;
            const int a = phase(b);
            const bool owned = (col < a) ? (b >= 1 && b - 1 < rows) : (b < rows);
            if (a != 0 && b <= rows && owned) {
                const int64_t off = (int64_t)(m0 + b) * (int64_t)T - a + col;
#pragma unroll
                for (int o = 0; o < NO; ++o)
                    store4(prm.out[o] + off, *reinterpret_cast<const float4*>(&bline[o][b * 32 + col]), STREAM);
            }
        }
    }
    op.finish(prm, m0 + lane, lane < rows);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launch helper: picks the dwordx4 path when T and every pointer allow it, non-temporal global
// accesses when the tensors are too large to be reused out of the last-level cache, and the
// rows-per-wave geometry from the number of neurons.
template <class Op, int R>
int launch_stream_rows(const typename Op::Params& prm, int64_t M, int64_t T, bool vec, bool streaming,
                       hipStream_t stream) {
    const dim3 grid((unsigned)((M + R - 1) / R)), block(kWave);
    if (!vec)
        hipLaunchKernelGGL((stream_kernel<Op, R, false, false>), grid, block, 0, stream, prm, M, (int)T);
    else if (streaming)
        hipLaunchKernelGGL((stream_kernel<Op, R, true, true>), grid, block, 0, stream, prm, M, (int)T);
    else
        hipLaunchKernelGGL((stream_kernel<Op, R, true, false>), grid, block, 0, stream, prm, M, (int)T);
    return (int)hipGetLastError();
}

// Rows per wave.  An Op states below how many neurons it wants 32 and 16 rows per wave
// (kRows32Below, kRows16Below; measured on MI355X): arithmetic-heavy forward recurrences keep all
// 64 lanes busy until the problem gets small, the light float backward passes prefer 16 rows
// and 512-byte row segments at every size.
constexpr int64_t kAlways = (int64_t)1 << 62;

template <class Op>
int launch_stream(const typename Op::Params& prm, int64_t M, int64_t T, hipStream_t stream) {
    if (M == 0 || T == 0) return 0;
    bool vec = (T % 4) == 0;
    for (int i = 0; i < Op::kIn; ++i) vec = vec && aligned16(prm.in[i]);
    for (int o = 0; o < Op::kOut; ++o) vec = vec && aligned16(prm.out[o]);
    const bool streaming = M * T * 4 > ((int64_t)64 << 20);
    if (M < Op::kRows16Below) return launch_stream_rows<Op, 16>(prm, M, T, vec, streaming, stream);
    if constexpr (Op::kRows16Below < kAlways && Op::kRows16Below < Op::kRows32Below)
        if (M < Op::kRows32Below) return launch_stream_rows<Op, 32>(prm, M, T, vec, streaming, stream);
    if constexpr (Op::kRows32Below < kAlways)
        return launch_stream_rows<Op, 64>(prm, M, T, vec, streaming, stream);
    return 0;   // not reached: every neuron count is covered by the branches above
}

}  // namespace slayer
