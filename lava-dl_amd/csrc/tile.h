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
#include <type_traits>
#include "../../include/slayer_hip.h"

namespace slayer {

constexpr int kWave = 64;

// (a * b) >> 12 rounded toward zero.  The 64-bit product is biased by 4095 when it is
// negative; its sign is the sign bit of a ^ b whenever the product is non-zero, and a
// zero product gives 0 with either bias, so no second multiply is needed for the sign.
__device__ __forceinline__ int rs0_12(int a, int b) {
    const long long bias = (long long)(((a ^ b) >> 31) & 4095);
    return (int)(((long long)a * (long long)b + bias) >> 12);
}

// a + b held inside the int32 range (v_add_i32 with clamp: one instruction, as the wrapping add).  The state
// updates use it so that a sum that leaves the range ends at the limit, where the range check of the copy-out
// sees it, instead of wrapping to an innocent-looking value.
__device__ __forceinline__ int add_sat(int a, int b) { return __builtin_elementwise_add_sat(a, b); }

// Range of the 32-bit states.  The kernels follow the reference's 64-bit evaluation bit for bit while no
// intermediate leaves 32 bits.  That is guaranteed while every stored state stays below a bound that leaves room
// for one more step (2^30 for a single decayed state plus input, 2^29 for the two-product resonator step, 2^28 for
// threshold / refractory states, whose spike adds step and twice the threshold) and every decay multiplier is at
// most 8191 in magnitude: an Op with integer tiles names the bound of each output tile (range_log2), the copy-out
// tests every value it stores on its way (off the sequential chain), the Op's init tests the multipliers, and
// either raises the process-wide flag behind Params::range_flag (pinned host memory that the device can write).
__device__ __forceinline__ void raise_range_flag(unsigned* flag) {
    if (flag) *reinterpret_cast<volatile unsigned*>(flag) = 1u;
}
__device__ __forceinline__ void check_multiplier(int mult, unsigned* flag) {
    if (mult > 8191 || mult < -8191) raise_range_flag(flag);
}
#ifndef SLAYER_RANGE_CHECK
#define SLAYER_RANGE_CHECK 1             // 0: a build without the copy-out's range test, to measure what it costs
#endif
template <class Op, class = void>
struct RangeChecked { static constexpr bool value = false; };
template <class Op>
struct RangeChecked<Op, decltype((void)Op::kRangeChecked)> { static constexpr bool value = Op::kRangeChecked && SLAYER_RANGE_CHECK != 0; };
// Smallest and largest value seen (integer bit patterns in float registers): two three-way minima / maxima per
// quad, the cheapest form for the copy waves, whose instruction count is what bounds the kernels on few rows.
struct RangeSpan {
    int lo, hi;
    __device__ __forceinline__ void reset() { lo = 0; hi = 0; }
    __device__ __forceinline__ void track(float4 q) {
        const int x = __float_as_int(q.x), y = __float_as_int(q.y), z = __float_as_int(q.z), w = __float_as_int(q.w);
        hi = max(max(hi, x), y); hi = max(max(hi, z), w);
        lo = min(min(lo, x), y); lo = min(min(lo, z), w);
    }
    __device__ __forceinline__ bool exceeded(int log2_bound) const {
        return hi >= (1 << log2_bound) || lo < -(1 << log2_bound);
    }
};
// the same test for states that are watched inside a sequential loop: accumulates v + 2^L for a quad; a value
// outside [-2^L, 2^L) sets a bit at or above bit L + 1
__device__ __forceinline__ unsigned range_bits(float4 q, int log2_bound) {
    const unsigned b = 1u << log2_bound;
    return (__float_as_uint(q.x) + b) | (__float_as_uint(q.y) + b) | (__float_as_uint(q.z) + b) | (__float_as_uint(q.w) + b);
}
__device__ __forceinline__ bool range_exceeded(unsigned acc, int log2_bound) { return (acc >> (log2_bound + 1)) != 0u; }
// an initial state (never stored, so never seen by the copy-out) against the bound of its tile
__device__ __forceinline__ void check_state(int y, int log2_bound, unsigned* flag) {
    if (range_exceeded((unsigned)y + (1u << log2_bound), log2_bound)) raise_range_flag(flag);
}

// Largest integer y whose float32 conversion is below thr: (float)y >= thr  <=>  y > fire_above(thr),
// so a recurrence can take its reset decision on the integer state.  INT_MAX (never fires) for
// thresholds beyond the int range, NaN or +inf.
inline int fire_above(float thr) {
    if (!(thr <= 2147483648.0f)) return 0x7fffffff;
    if (thr <= -2147483648.0f) return (int)0x80000000;     // every state fires except the most negative one
    long long c = (long long)__builtin_ceil((double)thr);   // candidate for the smallest firing state
    while (c > -2147483648LL && (float)(c - 1) >= thr) --c;
    while (c <= 2147483647LL && (float)c < thr) ++c;
    return (int)(c - 1);
}

// The same for a compare made on the converted state: largest integer y whose output value
// (float32(y) * (1 / w) for a power-of-two w, float32(y) / w otherwise, w > 0) is below thr, found by
// bisection with the very operations the kernels use (both are monotone in y).
inline int fire_above_scaled(float thr, float w, bool pow2) {
    const float inv_w = 1.0f / w;
    auto below = [&](long long y) {
        const float f = (float)y;
        return (pow2 ? f * inv_w : f / w) < thr;
    };
    long long lo = -2147483648LL, hi = 2147483647LL;
    if (!(thr == thr) || below(hi)) return (int)hi;      // NaN or beyond every state: never fires
    if (!below(lo)) return (int)lo;                      // every state fires except the most negative one
    while (hi - lo > 1) {
        const long long mid = lo + (hi - lo) / 2;
        if (below(mid)) lo = mid; else hi = mid;
    }
    return (int)lo;
}

// Integer tiles: an Op with kTransforms can keep its fixed-point states in LDS as integers (bit
// patterns in float registers).  Inputs are scaled and truncated on the way in, states converted
// and scaled back on the way out.
__device__ __forceinline__ float to_state(float x, float w) { return __int_as_float((int)(w * x)); }
__device__ __forceinline__ float4 to_state(float4 x, float w) {
    return make_float4(to_state(x.x, w), to_state(x.y, w), to_state(x.z, w), to_state(x.w, w));
}
template <bool POW2>
__device__ __forceinline__ float from_state(float s, float w, float inv_w) {
    const float f = (float)__float_as_int(s);
    return POW2 ? f * inv_w : f / w;
}
template <bool POW2>
__device__ __forceinline__ float4 from_state(float4 s, float w, float inv_w) {
    return make_float4(from_state<POW2>(s.x, w, inv_w), from_state<POW2>(s.y, w, inv_w),
                       from_state<POW2>(s.z, w, inv_w), from_state<POW2>(s.w, w, inv_w));
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

// 16-byte accesses at addresses that are only dword-aligned (rows of a length that is not a multiple of 4, or
// shifted by such a count): the hardware takes them, the type tells the compiler not to assume more.
typedef float quad_align4 __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ float4 load_quad_dword_aligned(const float* p) {
    const quad_align4 v = *reinterpret_cast<const quad_align4*>(p);
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_quad_dword_aligned(float* p, float4 f) {
    quad_align4 v;
    v.x = f.x; v.y = f.y; v.z = f.z; v.w = f.w;
    *reinterpret_cast<quad_align4*>(p) = v;
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

template <int R, int S = kTileSamples>
struct TileGeom {
    static constexpr int kRows = R;
    static constexpr int kChunk = S / R;                     // TC: steps per chunk
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
//   optionally static constexpr bool kTransforms = true and
//     __device__ void pre(float4 (&x)[kIn]) const;  __device__ void post(float4 (&y)[kOut]) const;
//     elementwise maps (wave-uniform members only) applied to the input quads on their way into LDS
//     and to the output quads on their way out, so that work that does not belong to the
//     sequential dependency chain (scaling, int <-> float conversion) is done by all 64 lanes in
//     the copy phases, or by the copy waves of the multi-wave kernel;
//   optionally static constexpr int kDerived = 1 and
//     __device__ float4 derive(const float4 (&y)[kOut]) const;   (uses wave-uniform members only)
//     an extra output, Params::out[kOut], that is an elementwise function of the other outputs of
//     the same step: it is computed while a quad is copied out and needs neither an LDS tile nor
//     boundary registers
//   static constexpr int64_t kRows32Below, kRows16Below;   (rows-per-wave policy, see launch_stream)
//   static constexpr bool kLongPiecesOnAliasedRows;        (optional, see row_stride_aliases)
//   struct Params { const float* in[kIn]; float* out[kOut]; ... };   (a null out[] entry is not stored, a null
//     in[] entry other than in[0] reads as zeros: a slot for pre() to fill)
//   __device__ void init(const Params&, int64_t m, bool valid);
//   __device__ void step(const float (&x)[kIn], float (&y)[kOut]);
//   __device__ void finish(const Params&, int64_t m, bool valid);

template <class Op, class = void>
struct HasTransforms { static constexpr bool value = false; };
template <class Op>
struct HasTransforms<Op, decltype((void)Op::kTransforms)> { static constexpr bool value = Op::kTransforms; };

template <class Op, class = void>
struct DerivedCount { static constexpr int value = 0; };
template <class Op>
struct DerivedCount<Op, decltype((void)Op::kDerived)> { static constexpr int value = Op::kDerived; };

// Time shifts folded into the copies (an axonal delay on either side of a neuron costs no pass of its own).
//   static constexpr unsigned kShiftIn  = bit mask over in[]:  input i is read shifted, the recurrence sees
//                                         x[t] = in[i][t - kin] (zero where t - kin falls outside [0, T));
//   static constexpr unsigned kShiftOut = bit mask over out[] (bit kOut = the derived output): output o is
//                                         stored shifted, out[o][t + kout] = y[t]; samples that leave [0, T)
//                                         are dropped and the positions no sample reaches are filled with
//                                         zeros (the one just before the first sample with head[m], if given).
// An Op that sets either carries `Shifts shifts;` in its Params.  kin and kout are per row:
// steps + trunc(lut[m % npb] / ts), any sign.  Shifted tensors still move 16 bytes per lane and instruction,
// at dword-aligned addresses (a row's shift need not be a multiple of 4 and differs from row to row); only the
// quads that straddle an end of their row take extra work.  Everything else is unchanged.
struct Shifts {
    const float* in_lut;     // per-neuron input shift in time units, npb entries, or nullptr
    const float* out_lut;    // per-neuron output shift, npb entries, or nullptr
    const float* head;       // [M] value of the sample before step 0 of a shifted output (lands at kout - 1), or nullptr
    float* last;             // [M] receives the shifted output's sample of step T-1 (written by Op::finish), or nullptr
    int in_steps, out_steps; // scalar parts, in steps
    int sign;                // +1, or -1 for a backward pass (undoes the forward pass's shifts)
    float ts;                // sampling time the lut entries are divided by
    int64_t npb;
    // backward scans only: the delayed spikes the forward pass stored and the per-row sums of
    // grad[t] * (delayed[t-1] - delayed[t]) / ts they leave for the delay gradient, or nullptr
    const float* delayed;
    float* delay_partial;
};

// prm.shifts, or no shifts at all for an Op whose Params carry none
template <class P, class = void>
struct ShiftsOf { static __host__ __device__ __forceinline__ Shifts get(const P&) { return Shifts{nullptr, nullptr, nullptr, nullptr, 0, 0, 1, 1.0f, 1}; } };
template <class P>
struct ShiftsOf<P, decltype((void)sizeof(((P*)nullptr)->shifts))> {
    static __host__ __device__ __forceinline__ const Shifts& get(const P& p) { return p.shifts; }
};

template <class Op, class = void>
struct ShiftInMask { static constexpr unsigned value = 0; };
template <class Op>
struct ShiftInMask<Op, decltype((void)Op::kShiftIn)> { static constexpr unsigned value = Op::kShiftIn; };
template <class Op, class = void>
struct ShiftOutMask { static constexpr unsigned value = 0; };
template <class Op>
struct ShiftOutMask<Op, decltype((void)Op::kShiftOut)> { static constexpr unsigned value = Op::kShiftOut; };

// steps + trunc(lut / ts), the sum held inside [-(T+1), T+1]: a shift of T steps already empties the row, T+1
// stands for everything beyond (the sample before the first, `head`, then falls off the row too).  The terms are
// added before the sum is clamped (two large terms of opposite sign leave a small shift); a table entry beyond
// +-2^30 steps counts as +-2^30.
__host__ __device__ __forceinline__ int clamp_shift(int64_t k, int T) {
    const int64_t lim = (int64_t)T + 1;
    return (int)(k > lim ? lim : (k < -lim ? -lim : k));
}
__device__ __forceinline__ int row_shift(const float* lut, int steps, float ts, int64_t m, int64_t npb, int T) {
    int64_t k = steps;
    if (lut) {
        const float q = lut[m % npb] / ts;
        const float lim = 1073741824.0f;
        k += !(q == q) ? 0 : (q >= lim ? (1 << 30) : (q <= -lim ? -(1 << 30) : (int)q));
    }
    return clamp_shift(k, T);
}

__device__ __forceinline__ int in_shift_of(const Shifts& sh, int64_t m, int T) {
    return sh.sign * row_shift(sh.in_lut, sh.in_steps, sh.ts, m, sh.npb, T);
}
__device__ __forceinline__ int out_shift_of(const Shifts& sh, int64_t m, int T) {
    return sh.sign * row_shift(sh.out_lut, sh.out_steps, sh.ts, m, sh.npb, T);
}

// ---------------------------------------------------------------------------------------------
// Buffer addressing.  Global accesses of the dwordx4 path go through raw buffer instructions whose
// descriptor covers exactly the rows of this wave: a lane that must not touch memory (column
// outside [0, T), row beyond the tensor) gets an offset past the end, for which the hardware
// returns zero / drops the store.  There are no branches around memory instructions, so their
// count per chunk is static and the loads of chunk k+1 can be waited for with an exact vmcnt
// while the stores of chunk k are still in flight.
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
constexpr int kOutOfRange = (int)0x80000000;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)bytes, 0x00020000);
}
template <bool STREAM>
__device__ __forceinline__ float4 buf_load4(__amdgpu_buffer_rsrc_t r, int byte_off) {
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, STREAM ? 2 : 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
template <bool STREAM>
__device__ __forceinline__ void buf_store4(__amdgpu_buffer_rsrc_t r, int byte_off, float4 f) {
    v4u v;
    v.x = __float_as_uint(f.x); v.y = __float_as_uint(f.y); v.z = __float_as_uint(f.z); v.w = __float_as_uint(f.w);
    __builtin_amdgcn_raw_buffer_store_b128(v, r, byte_off, 0, STREAM ? 2 : 0);
}

template <bool STREAM>
__device__ __forceinline__ float buf_load1(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, STREAM ? 2 : 0));
}
template <bool STREAM>
__device__ __forceinline__ void buf_store1(__amdgpu_buffer_rsrc_t r, int byte_off, float f) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(f), r, byte_off, 0, STREAM ? 2 : 0);
}

// ---------------------------------------------------------------------------------------------
// dwordx4 kernel (T % 4 == 0, 16-byte aligned bases).
//
// Line alignment.  A row of T floats starts wherever m*T falls, so a fixed time grid would cut
// every row segment across 128-byte lines and each line would be fetched (and partially written)
// twice.  Instead every row gets its own phase a = (float index of the row start) mod 32 and tile
// column j of chunk k holds step t = k*TC + j - a: the segments a wave-wide access touches then
// start on 128-byte boundaries.  Lanes skip the columns that fall before step 0 or after T-1.
//
// Boundary lines.  Unless T is a multiple of 32, the last line of row r is also the first line of
// row r+1, and the two pieces are produced a whole row apart in time.  Written when produced, each
// piece reaches memory as a partial line, which costs a read-modify-write there (measured: ~16% of
// the kernel at T = 300).  So the piece that comes first (the head of row r+1 in a forward pass,
// the tail of row r in a reverse pass) waits in registers of the lanes that will store the other
// piece, and the eight lanes that cover the line store it whole with one instruction.  Only the
// lines shared with neighbouring workgroups are still written in pieces.
//
// Ownership rule.  A wave completes a shared line only when both rows that meet in it belong to
// the passes this wave owns.  Copy waves that share a tile run without a barrier among themselves
// (one fills a tile buffer with the next chunk right after it has copied the previous chunk out),
// so a quad taken from a row of another wave could already have been overwritten; at the edge of a
// wave's row range the line is therefore written in two pieces, as at the edge of a workgroup.
//
// Interior chunks (every column of every row inside [0, T), no shared line) run a branch-free
// recurrence loop; only the first and the last one or two chunks take the predicated path.
// Everything a wave needs to move the tiles of its R rows between global memory and LDS: buffer
// descriptors, the per-pass copy pattern, the registers the next chunk is prefetched into and the
// registers that hold boundary quads.
//
// A wave can share the job with others: it then owns PASSES of the G::kPasses wave-wide accesses
// that cover a tile, starting at pass first_pass.
//
// UNAL: rows that are not whole quads (T % 4 != 0, or base pointers that are only dword-aligned).  Tile columns
// are still laid on 128-byte lines by the row phases, so quads sit on 16-byte boundaries of memory, but a row
// may now begin and end inside a quad.  Every tensor then takes the path of the shifted ones (with a shift of
// zero unless it really is shifted): 16-byte accesses where the whole quad lies inside the row, the quads that
// straddle an end of the row loaded from the nearest position inside it and stored sample by sample, no line
// completion; the recurrence skips the steps of such a quad that lie outside the row.
template <class Op, int R, bool STREAM, int PASSES = TileGeom<R>::kPasses, int S = kTileSamples, bool UNAL = false>
struct Copier {
    using G = TileGeom<R, S>;
    static constexpr int TC = G::kChunk, NI = Op::kIn, NO = Op::kOut, ND = DerivedCount<Op>::value;
    static constexpr int kPasses = PASSES;
    static_assert(ND == 0 || ND == 1, "at most one derived output");
    static constexpr unsigned SI = ShiftInMask<Op>::value, SO = ShiftOutMask<Op>::value;     // really shifted
    static constexpr unsigned AI = UNAL ? (1u << NI) - 1u : SI, AO = UNAL ? (1u << (NO + ND)) - 1u : SO;   // careful path
    static constexpr bool kShifts = AI != 0 || AO != 0;
    using Tiles = float (*)[G::kTileFloats];

    __amdgpu_buffer_rsrc_t src[NI], dst[NO + ND];
    int step0[kPasses], off0[kPasses];    // step of this lane's quad in chunk 0, its byte offset in the wave's rows
    float4 stage[NI][kPasses];               // prefetched inputs
    float4 keep[NO][kPasses];                // first-produced pieces of shared lines, one quad per pass
    int rows, T, crow, cq, interior_end, first_pass;
    int row_lo, row_hi;                      // rows [row_lo, row_hi) of the tile are copied by this wave
    int kin[kShifts ? kPasses : 1], kout[kShifts ? kPasses : 1];   // shifts of this lane's row in each pass
    int kout_row;                            // output shift of row `lane` (lane = row), for fill_unreached
    RangeSpan range_seen[RangeChecked<Op>::value ? NO : 1];  // of the states this wave stored
    // wave-uniform: chunks [in_first, in_last] hold only quads whose shifted source lies wholly inside its row,
    // chunks [out_first, out_last] only quads whose shifted destination does (for every row of this wave)
    int in_first, in_last, out_first, out_last;
    bool route;

    __device__ __forceinline__ void init(const typename Op::Params& prm, int64_t m0, int rows_, int T_, int lane,
                                         unsigned base_f, int first_pass_ = 0) {
        rows = rows_; T = T_; first_pass = first_pass_;
#pragma unroll
        for (int o = 0; o < (RangeChecked<Op>::value ? NO : 1); ++o) range_seen[o].reset();
        row_lo = first_pass * G::kRowsPerPass;
        row_hi = (first_pass + kPasses) * G::kRowsPerPass;
        if (row_hi > rows) row_hi = rows;
        const unsigned wave_bytes = (unsigned)rows * (unsigned)T * 4u;
#pragma unroll
        for (int i = 0; i < NI; ++i)         // an input the caller does not have: every load falls out of range, reads 0
            src[i] = prm.in[i] ? make_rsrc(prm.in[i] + m0 * (int64_t)T, wave_bytes) : make_rsrc(nullptr, 0);
#pragma unroll
        for (int o = 0; o < NO + ND; ++o)    // an output the caller does not want: every store falls out of range
            dst[o] = prm.out[o] ? make_rsrc(prm.out[o] + m0 * (int64_t)T, wave_bytes) : make_rsrc(nullptr, 0);
        crow = lane / G::kQuads;                // row within a pass
        cq = lane % G::kQuads;                  // quad within the row
        // chunks [1, interior_end) hold only valid columns and touch no shared line, for every phase
        interior_end = (T & ~31) / TC;
        // rows shorter than a line could start and end inside the same line; they keep direct stores
        route = T >= 32 && !UNAL;
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int r = (first_pass + p) * G::kRowsPerPass + crow;
            step0[p] = 4 * cq - (int)((base_f + (unsigned)(m0 + r) * (unsigned)T) & 31u);
            off0[p] = (r * T + step0[p]) * 4;
#pragma unroll
            for (int o = 0; o < NO; ++o) keep[o][p] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if constexpr (kShifts) {
            // lane l works out the shifts of row l once (a table look-up with a 64-bit modulo and a division);
            // the passes pick theirs up from that lane
            const Shifts sh = ShiftsOf<typename Op::Params>::get(prm);
            const bool mine = lane >= row_lo && lane < row_hi;
            const int kin_row = (SI != 0 && mine) ? in_shift_of(sh, m0 + lane, T) : 0;
            kout_row = (SO != 0 && mine) ? out_shift_of(sh, m0 + lane, T) : 0;
#pragma unroll
            for (int p = 0; p < kPasses; ++p) {
                const int r = (first_pass + p) * G::kRowsPerPass + crow;
                kin[p] = __shfl(kin_row, r);
                kout[p] = __shfl(kout_row, r);
            }
            int in_max = kin_row > 0 ? kin_row : 0, in_min = kin_row < 0 ? kin_row : 0;
            int out_max = kout_row > 0 ? kout_row : 0, out_min = kout_row < 0 ? kout_row : 0;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                int o;
                o = __shfl_xor(in_max, d); in_max = o > in_max ? o : in_max;
                o = __shfl_xor(in_min, d); in_min = o < in_min ? o : in_min;
                o = __shfl_xor(out_max, d); out_max = o > out_max ? o : out_max;
                o = __shfl_xor(out_min, d); out_min = o < out_min ? o : out_min;
            }
            // chunk c holds steps c*TC - 31 .. (c+1)*TC - 1 over all phases; a quad starts at t, its source at
            // s = t - kin, its destination at u = t + kout; both must lie in [0, T - 4]
            in_first = (31 + in_max + TC - 1) / TC;
            in_last = (T + in_min) / TC - 1;
            out_first = (31 - out_min + TC - 1) / TC;
            out_last = (T - out_max) / TC - 1;
            in_first = __builtin_amdgcn_readfirstlane(in_first); in_last = __builtin_amdgcn_readfirstlane(in_last);
            out_first = __builtin_amdgcn_readfirstlane(out_first); out_last = __builtin_amdgcn_readfirstlane(out_last);
        }
    }

    __device__ __forceinline__ bool whole_in(int chunk) const { return chunk >= in_first && chunk <= in_last; }
    __device__ __forceinline__ bool whole_out(int chunk) const { return chunk >= out_first && chunk <= out_last; }

    // The positions of a shifted output that no sample reaches: [0, kout) for a delay, [T + kout, T) for an
    // advance.  Row after row of this wave's rows, 64 positions per instruction.
    __device__ __forceinline__ void fill_unreached(const typename Op::Params& prm, int64_t m0, int lane) const {
        if constexpr (SO != 0) {
            const Shifts sh = ShiftsOf<typename Op::Params>::get(prm);
            for (int r = row_lo; r < row_hi; ++r) {
                const int k = __builtin_amdgcn_readlane(kout_row, r);
                const int mag = k < 0 ? -k : k;
                const int len = mag > T ? T : mag;
                for (int j0 = 0; j0 < len; j0 += kWave) {
                    const int j = j0 + lane;
                    const bool ok = j < len;
                    const int u = k < 0 ? T - len + j : j;
                    float v = 0.f;
                    if (ok && sh.head && k > 0 && j == k - 1) v = sh.head[m0 + r];
#pragma unroll
                    for (int o = 0; o < NO + ND; ++o)
                        if (((SO >> o) & 1u) != 0) buf_store1<STREAM>(dst[o], ok ? (r * T + u) * 4 : kOutOfRange, v);
                }
            }
        }
    }

    __device__ __forceinline__ bool interior(int chunk) const { return chunk >= 1 && chunk < interior_end; }

    // global -> registers; past the last chunk (or before the first) every lane is out of range
    __device__ __forceinline__ void fetch_into(float4 (&buf)[NI][kPasses], int chunk) const {
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int t = step0[p] + chunk * TC;
            const bool ok = UNAL ? (t > -4 && t < T) : (unsigned)t < (unsigned)T;   // some step of the quad is in the row
            const int off = ok ? off0[p] + chunk * (TC * 4) : kOutOfRange;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                if (((AI >> i) & 1u) != 0) {
                    // the quad wanted is samples s .. s+3 of the row, s = t - kin (a multiple of 4 only by chance:
                    // the load is dword-aligned).  One 16-byte load at the nearest position that lies inside
                    // the row; to_tiles() moves the samples into place when the two differ.
                    const int ki = ((SI >> i) & 1u) != 0 ? kin[p] : 0;
                    if (whole_in(chunk)) {
                        buf[i][p] = buf_load4<STREAM>(src[i], ok ? off0[p] + chunk * (TC * 4) - 4 * ki : kOutOfRange);
                    } else {
                        const int s = t - ki;
                        const int sc = s < 0 ? 0 : (s > T - 4 ? T - 4 : s);
                        const bool some = ok && s > -4 && s < T;
                        buf[i][p] = buf_load4<STREAM>(src[i], some ? off0[p] + 4 * (sc - step0[p]) : kOutOfRange);
                    }
                } else {
                    buf[i][p] = buf_load4<STREAM>(src[i], off);
                }
            }
        }
    }
    __device__ __forceinline__ void fetch(int chunk) { fetch_into(stage, chunk); }

    // registers -> LDS
    // A shifted input whose quad straddles an end of its row was loaded from the nearest position inside the
    // row: element e of the quad is element e + d of what was loaded, d = wanted - loaded position, or zero.
    __device__ __forceinline__ float4 place(float4 q, int d) const {
        const float a[4] = {q.x, q.y, q.z, q.w};
        float r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = e + d;
            r[e] = j == 0 ? a[0] : (j == 1 ? a[1] : (j == 2 ? a[2] : (j == 3 ? a[3] : 0.f)));
        }
        return make_float4(r[0], r[1], r[2], r[3]);
    }

    __device__ __forceinline__ void stage_to_tiles(const Op& op, Tiles tile, int chunk) const {
        to_tiles(op, tile, stage, chunk);
    }
    // `chunk` is the chunk `buf` was fetched for
    __device__ __forceinline__ void to_tiles(const Op& op, Tiles tile, const float4 (&buf)[NI][kPasses],
                                             int chunk) const {
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int r = (first_pass + p) * G::kRowsPerPass + crow;
            float4 x[NI];
#pragma unroll
            for (int i = 0; i < NI; ++i) x[i] = buf[i][p];
            if (AI != 0 && !whole_in(chunk)) {
                auto offset_of = [&](int ki) {        // wanted minus loaded position of a quad read through shift ki
                    const int s = step0[p] + chunk * TC - ki;
                    const int sc = s < 0 ? 0 : (s > T - 4 ? T - 4 : s);
                    return (s > -4 && s < T) ? s - sc : 0;
                };
                const int d = offset_of(SI != 0 ? kin[p] : 0), d0 = (UNAL && SI != AI) ? offset_of(0) : 0;
                if (__any((d | d0) != 0)) {           // rare: only where a row begins or ends
#pragma unroll
                    for (int i = 0; i < NI; ++i) {
                        if (((SI >> i) & 1u) != 0) x[i] = place(x[i], d);
                        else if (((AI >> i) & 1u) != 0) x[i] = place(x[i], d0);
                    }
                }
            }
            if constexpr (HasTransforms<Op>::value) op.pre(x);
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<float4*>(&tile[i][r * G::kPitch + 4 * cq]) = x[i];
        }
    }

    // Stores that fall out of range (dropped by the hardware), as many as one chunk issues: the
    // chunk loop is then entered in the same state its back edge leaves -- a chunk of loads
    // followed by a chunk of stores in flight -- and the wait for the loads at the top of every
    // iteration can leave the stores of the previous chunk in flight instead of draining them.
    __device__ __forceinline__ void prime_stores() const {
#pragma unroll
        for (int p = 0; p < kPasses; ++p)
#pragma unroll
            for (int o = 0; o < NO + ND; ++o) { // distinct offsets, or the compiler merges them into one store
                buf_store4<STREAM>(dst[o], kOutOfRange + 16 * p, make_float4(0.f, 0.f, 0.f, 0.f));
            }
    }

    // Raises the range flag when a state this wave stored came too close to the 32-bit limit (see range_bits).
    __device__ __forceinline__ void report_range(const typename Op::Params& prm) const {
        if constexpr (RangeChecked<Op>::value) {
            bool bad = false;
#pragma unroll
            for (int o = 0; o < NO; ++o)
                if (Op::range_log2(o) != 0) bad = bad || range_seen[o].exceeded(Op::range_log2(o));
            if (bad) raise_range_flag(prm.range_flag);
        }
    }

    // LDS -> global.  On edge chunks the line shared by rows r and r+1 is completed before it is
    // stored: in a forward pass the lanes that copy the last line of row r fill its slots past
    // the end of the row with the head of row r+1, which they fetched from that row's tile in
    // chunk 0; in a reverse pass the lanes that copy the first line of row r+1 fill its slots
    // before the start of the row with the tail of row r, fetched in the chunk that held it.
    // Either way the fetched quad waits in keep[][p] and leaves with the regular store of its
    // lane, so every chunk issues the same number of stores.
    __device__ __forceinline__ void copy_out(const Op& op, Tiles tile, int chunk) {
        const bool inner = interior(chunk);
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int r = (first_pass + p) * G::kRowsPerPass + crow;
            const int t = step0[p] + chunk * TC;
            int off = off0[p] + chunk * (TC * 4);
            float4 v[NO], own[NO];                                  // own: this lane's quad, for shifted outputs
#pragma unroll
            for (int o = 0; o < NO; ++o) own[o] = v[o] = *reinterpret_cast<const float4*>(&tile[o][r * G::kPitch + 4 * cq]);
            if constexpr (RangeChecked<Op>::value) {
                // only quads that hold steps of the row: the tiles of a chunk number that names no chunk (before
                // the first, after the last) were never filled.  Interior chunks hold nothing else.
                if (inner) {
#pragma unroll
                    for (int o = 0; o < NO; ++o)
                        if (Op::range_log2(o) != 0) range_seen[o].track(v[o]);
                } else {
                    const bool counted = UNAL ? (t > -4 && t < T) : (unsigned)t < (unsigned)T;
                    const float4 none = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                    for (int o = 0; o < NO; ++o)
                        if (Op::range_log2(o) != 0) range_seen[o].track(counted ? v[o] : none);
                }
            }
            if (!inner) {
                const int a = 4 * cq - step0[p];                   // phase of row r
                const bool valid = (unsigned)t < (unsigned)T;
                if (!valid) off = kOutOfRange;
                const int a_next = (a + T) & 31;                   // phase of row r+1
                const int tail_pos = (a + T) & ~31;                // window position of row r's partial last line
                const int prev_tail_pos = (((a - T) & 31) + T) & ~31;   // the same for row r-1
                // the pieces of a line shared with a neighbouring row that this wave copies too
                const bool prev_mine = r > row_lo && r < row_hi;       // row r-1 is one of this wave's rows
                const bool next_mine = r + 1 < row_hi;                 // row r+1 is one of this wave's rows
                const bool own_head = route && prev_mine && a != 0 && cq < 8 && 4 * cq >= a;
                const bool own_tail = route && valid && next_mine && 4 * cq + chunk * TC >= tail_pos;
                bool take, release;
                int idx;                                           // tile position of the quad to take
                if (Op::kReverse) {
                    // slot cq of row r's first line, before the row starts: tail of row r-1
                    const bool slot = route && prev_mine && a != 0 && cq < 8 && 4 * cq < a;
                    const int kp = prev_tail_pos / TC;
                    take = slot && chunk == kp;
                    release = slot && chunk == 0;
                    idx = (r - 1) * G::kPitch + (prev_tail_pos - kp * TC) + 4 * cq;
                    if (own_tail) off = kOutOfRange;               // stored by row r+1's lanes in chunk 0
                } else {
                    // slot j of row r's last line, past the end of the row: head of row r+1
                    const int kt = tail_pos / TC;
                    const int j = cq - (tail_pos - kt * TC) / 4;
                    const bool slot = route && next_mine && a_next != 0 && j >= 0 && j < 8 && 4 * j >= a_next;
                    take = slot && chunk == 0;
                    release = slot && chunk == kt;
                    idx = (r + 1) * G::kPitch + 4 * j;
                    if (own_head && chunk == 0) off = kOutOfRange; // stored by row r-1's lanes with its tail
                }
                if (!take) idx = 0;
                if (release) off = off0[p] + chunk * (TC * 4);
#pragma unroll
                for (int o = 0; o < NO; ++o) {
                    const float4 other = *reinterpret_cast<const float4*>(&tile[o][idx]);
                    if (take) keep[o][p] = other;
                    if (release) v[o] = keep[o][p];
                }
            }
            if constexpr (HasTransforms<Op>::value) op.post(v);
            // A shifted output leaves from the lane that computed it (no completed lines: its quads do not fall
            // on line boundaries anyway), sample t + e to position t + e + kout of the row: one dword-aligned
            // 16-byte store when the whole quad lands inside the row; a quad that straddles an end of the row
            // (only in the first or last few chunks) leaves sample by sample.
            const bool careful = AO != 0 && !(inner && whole_out(chunk));   // a quad of this chunk may straddle an end of its row
            if (careful) {
                if (inner) {
#pragma unroll
                    for (int o = 0; o < NO; ++o) own[o] = v[o];
                } else {
                    if constexpr (HasTransforms<Op>::value) op.post(own);
                }
            } else if (AO != 0) {
#pragma unroll
                for (int o = 0; o < NO; ++o) own[o] = v[o];
            }
            const bool t_some = UNAL ? (t > -4 && t < T) : (unsigned)t < (unsigned)T;
            const bool t_whole = t >= 0 && t <= T - 4;
            // Sample t + e of the quad goes to position t + e + ko of the row.  A really shifted tensor is never
            // stored with the streaming hint: each of its stores ends in a partial line that the next chunk
            // completes, so the line has to wait in the cache.
            auto store_through = [&](__amdgpu_buffer_rsrc_t d, float4 q, int ko, bool shifted) {
                const int ubase = off0[p] + chunk * (TC * 4) + 4 * ko;
                const int u = t + ko;
                const bool whole = !careful || (t_some && t_whole && u >= 0 && u <= T - 4);
                const bool part = careful && t_some && !whole && u > -4 && u < T;
                if (shifted || !STREAM) buf_store4<false>(d, whole ? ubase : kOutOfRange, q);
                else buf_store4<true>(d, whole ? ubase : kOutOfRange, q);
                if (careful && __any(part)) {
                    const float e[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        buf_store1<false>(d, (part && (unsigned)(t + j) < (unsigned)T && (unsigned)(u + j) < (unsigned)T)
                                                 ? ubase + 4 * j : kOutOfRange, e[j]);
                }
            };
#pragma unroll
            for (int o = 0; o < NO; ++o) {
                if (((SO >> o) & 1u) != 0) store_through(dst[o], own[o], kout[p], true);
                else if (((AO >> o) & 1u) != 0) store_through(dst[o], own[o], 0, false);
                else buf_store4<STREAM>(dst[o], off, v[o]);
            }
            if constexpr (ND == 1) {
                if constexpr (((SO >> NO) & 1u) != 0) store_through(dst[NO], op.derive(own), kout[p], true);
                else if constexpr (((AO >> NO) & 1u) != 0) store_through(dst[NO], op.derive(own), 0, false);
                else buf_store4<STREAM>(dst[NO], off, op.derive(v));
            }
        }
    }
};

// Phase of a row (float index of its first sample modulo one 128-byte line) and the number of
// chunks the wave's rows span, the same value in every lane.
template <int TC>
__device__ __forceinline__ int chunk_count(int a_lane, bool valid, int T) {
    int last = valid ? (a_lane + T - 1) / TC : 0;    // last chunk this row needs
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_xor(last, d);
        last = o > last ? o : last;
    }
    return last + 1;
}

// Which tile an Op's i-th input / o-th output lives in: its own index, unless the Op is one stage of a
// staged Op (kTileMapped) and names the tiles of the whole Op it reads and writes.
template <class Op, class = void>
struct TileMap {
    static constexpr int in(int i) { return i; }
    static constexpr int out(int o) { return o; }
};
template <class Op>
struct TileMap<Op, decltype((void)Op::kTileMapped)> {
    static constexpr int in(int i) { return Op::in_tile(i); }
    static constexpr int out(int o) { return Op::out_tile(o); }
};

// The sequential part: lane = neuron, one chunk of the tiles in place.
// EXACT: rows may begin and end inside a quad (see Copier, UNAL); on the edge chunks the steps of a quad that lie
// outside the row are then skipped one by one.
template <class Op, int R, int UNROLL, int S = kTileSamples, bool EXACT = false>
__device__ __forceinline__ void run_chunk(Op& op, float (*tile)[TileGeom<R, S>::kTileFloats], int lane, int chunk,
                                          bool inner, int a_lane, int T) {
    using G = TileGeom<R, S>;
    constexpr int NI = Op::kIn, NO = Op::kOut;
    auto run_quad = [&](int qq) {
        float xin[NI][4], yout[NO][4];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const float4 v = *reinterpret_cast<const float4*>(&tile[TileMap<Op>::in(i)][lane * G::kPitch + 4 * qq]);
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
            *reinterpret_cast<float4*>(&tile[TileMap<Op>::out(o)][lane * G::kPitch + 4 * qq]) =
                make_float4(yout[o][0], yout[o][1], yout[o][2], yout[o][3]);
    };
    if (inner) {
        if (lane < R) {
#pragma unroll UNROLL
            for (int q = 0; q < G::kQuads; ++q) run_quad(Op::kReverse ? G::kQuads - 1 - q : q);
        }
    } else if (!EXACT) {
        const int tl = chunk * G::kChunk - a_lane;       // step held by column 0 of this lane's row
        for (int q = 0; q < G::kQuads; ++q) {
            const int qq = Op::kReverse ? G::kQuads - 1 - q : q;
            if (lane < R && (unsigned)(tl + 4 * qq) < (unsigned)T) run_quad(qq);
        }
    } else {
        const int tl = chunk * G::kChunk - a_lane;
        for (int q = 0; q < G::kQuads; ++q) {
            const int qq = Op::kReverse ? G::kQuads - 1 - q : q;
            const int t0 = tl + 4 * qq;                  // step of the quad's first column
            if (lane < R && t0 > -4 && t0 < T) {
                if (t0 >= 0 && t0 <= T - 4) {
                    run_quad(qq);
                } else {
                    float xin[NI][4], yout[NO][4];
#pragma unroll
                    for (int i = 0; i < NI; ++i) {
                        const float4 v = *reinterpret_cast<const float4*>(&tile[TileMap<Op>::in(i)][lane * G::kPitch + 4 * qq]);
                        xin[i][0] = v.x; xin[i][1] = v.y; xin[i][2] = v.z; xin[i][3] = v.w;
                    }
#pragma unroll
                    for (int st = 0; st < 4; ++st) {
                        const int ss = Op::kReverse ? 3 - st : st;
                        float x[NI], y[NO];
#pragma unroll
                        for (int i = 0; i < NI; ++i) x[i] = xin[i][ss];
#pragma unroll
                        for (int o = 0; o < NO; ++o) y[o] = 0.f;
                        if ((unsigned)(t0 + ss) < (unsigned)T) op.step(x, y);    // steps outside the row leave the state alone
#pragma unroll
                        for (int o = 0; o < NO; ++o) yout[o][ss] = y[o];
                    }
#pragma unroll
                    for (int o = 0; o < NO; ++o)
                        *reinterpret_cast<float4*>(&tile[TileMap<Op>::out(o)][lane * G::kPitch + 4 * qq]) =
                            make_float4(yout[o][0], yout[o][1], yout[o][2], yout[o][3]);
                }
            }
        }
    }
}

template <class Op, int R, bool STREAM>
__global__ __launch_bounds__(kWave) void stream_kernel(typename Op::Params prm, int64_t M, int T) {
    using G = TileGeom<R>;
    constexpr int TC = G::kChunk;
    constexpr int NI = Op::kIn, NO = Op::kOut, NT = NI > NO ? NI : NO;
    __shared__ __attribute__((aligned(16))) float tile[NT][G::kTileFloats];

    const int lane = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.x * R;
    const int rows = (int)((M - m0) < R ? (M - m0) : R);

    Op op;
    op.init(prm, m0 + lane, lane < rows);

    const unsigned base_f = (unsigned)(reinterpret_cast<uintptr_t>(prm.in[0]) >> 2);
    const int a_lane = (int)((base_f + (unsigned)(m0 + lane) * (unsigned)T) & 31u);
    const int nchunks = chunk_count<TC>(a_lane, lane < rows, T);

    Copier<Op, R, STREAM> io;
    io.init(prm, m0, rows, T, lane, base_f);
    io.fetch(Op::kReverse ? nchunks - 1 : 0);
    io.fill_unreached(prm, m0, lane);
    io.prime_stores();

    for (int k = 0; k < nchunks; ++k) {
        const int chunk = Op::kReverse ? nchunks - 1 - k : k;
        io.stage_to_tiles(op, tile, chunk);
        __syncthreads();
        io.fetch(Op::kReverse ? chunk - 1 : chunk + 1);
        run_chunk<Op, R, 4>(op, tile, lane, chunk, io.interior(chunk), a_lane, T);
        __syncthreads();
        io.copy_out(op, tile, chunk);
        __syncthreads();
    }
    io.report_range(prm);
    op.finish(prm, m0 + lane, lane < rows);
}

// Variant for problems too small to fill the machine with one wave per R rows.  There the run
// time is the number of steps times the latency of one step of the sequential wave, so that wave
// does nothing else: wave 0 runs the recurrence chunk after chunk, NCOPY more waves move the tiles
// (prefetch, LDS fill, boundary lines, stores) through a second set of tiles, each owning an equal
// share of the wave-wide accesses that cover a tile; one barrier per chunk.
//   barrier j: chunk j is in tiles[j & 1] and the recurrence of chunk j-1 is done.
// A chunk is a few hundred nanoseconds of recurrence, less than a trip to memory, so the copy
// waves keep the loads of two chunks in flight (chunk j waits in fetched[j & 1]).  All waves run
// an even number of chunks; a surplus chunk lies outside every row and neither computes nor stores.
template <class Op, int R, bool STREAM, int NCOPY, int S = kTileSamples, bool UNAL = false>
__global__ __launch_bounds__((1 + NCOPY) * kWave) void stream_kernel_duo(typename Op::Params prm, int64_t M, int T) {
    using G = TileGeom<R, S>;
    constexpr int TC = G::kChunk;
    constexpr int NI = Op::kIn, NO = Op::kOut, NT = NI > NO ? NI : NO;
    constexpr int PASSES = G::kPasses / NCOPY;
    static_assert(PASSES * NCOPY == G::kPasses, "copy waves share the passes evenly");
    __shared__ __attribute__((aligned(16))) float tiles[2][NT][G::kTileFloats];

    const int lane = threadIdx.x & (kWave - 1);
    const int role = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // wave-uniform
    const int64_t m0 = (int64_t)blockIdx.x * R;
    const int rows = (int)((M - m0) < R ? (M - m0) : R);
    const unsigned base_f = (unsigned)(reinterpret_cast<uintptr_t>(prm.in[0]) >> 2);
    const int a_lane = (int)((base_f + (unsigned)(m0 + lane) * (unsigned)T) & 31u);
    const int nchunks = chunk_count<TC>(a_lane, lane < rows, T);
    const int nloop = (nchunks + 1) & ~1;
    const int interior_end = (T & ~31) / TC;
    // k-th chunk in processing order; values outside [0, nchunks) name no chunk
    auto chunk_of = [&](int k) { return Op::kReverse ? nchunks - 1 - k : k; };

    if (role == 0) {
        Op op;
        op.init(prm, m0 + lane, lane < rows);
        for (int k = 0; k < nloop; ++k) {
            const int chunk = chunk_of(k);
            __syncthreads();                                   // barrier k
            if (k < nchunks)
                run_chunk<Op, R, 4, S, UNAL>(op, tiles[k & 1], lane, chunk, chunk >= 1 && chunk < interior_end, a_lane, T);
        }
        __syncthreads();                                       // barrier nloop
        op.finish(prm, m0 + lane, lane < rows);
    } else {
        Op uni;                                                // wave-uniform members only (pre, post, derive)
        uni.init(prm, 0, false);
        Copier<Op, R, STREAM, PASSES, S, UNAL> io;
        io.init(prm, m0, rows, T, lane, base_f, (role - 1) * PASSES);
        float4 fetched[2][NI][PASSES];
        io.fetch_into(fetched[0], chunk_of(0));
        io.fetch_into(fetched[1], chunk_of(1));
        io.prime_stores();
        io.to_tiles(uni, tiles[0], fetched[0], chunk_of(0));
        io.fetch_into(fetched[0], chunk_of(2));
        __syncthreads();                                       // barrier 0
        io.fill_unreached(prm, m0, lane);                      // while the sequential wave works on chunk 0
        for (int k = 0; k < nloop; k += 2) {
            // wave 0 works on tiles[0] (chunk k); tiles[1] still holds the results of chunk k-1
            io.copy_out(uni, tiles[1], chunk_of(k - 1));
            io.to_tiles(uni, tiles[1], fetched[1], chunk_of(k + 1));
            io.fetch_into(fetched[1], chunk_of(k + 3));
            __syncthreads();                                   // barrier k+1
            io.copy_out(uni, tiles[0], chunk_of(k));
            io.to_tiles(uni, tiles[0], fetched[0], chunk_of(k + 2));
            io.fetch_into(fetched[0], chunk_of(k + 4));
            __syncthreads();                                   // barrier k+2
        }
        io.copy_out(uni, tiles[1], chunk_of(nloop - 1));
        io.report_range(prm);
    }
}

// The multi-wave kernel for an Op whose step is a chain of two recurrences, the second reading what the
// first produced (kStages = 2, Stage0 / Stage1: Ops of their own that name the tiles they read and write).
// The two recurrences run in two waves, the second one chunk behind the first, so a step of the workgroup
// costs the longer of the two instead of their sum; that is what bounds the kernel while all workgroups are
// resident.  Three sets of tiles rotate:
//   period j (between barriers j and j+1): wave 0 runs stage 0 on chunk j in tiles[j % 3], wave 1 runs stage 1
//   on chunk j-1 in tiles[(j-1) % 3], the copy waves store chunk j-2 from tiles[(j+1) % 3], refill them with
//   chunk j+1 and issue the loads of chunk j+4 (three chunks of loads in flight).
// Every wave passes the same number of barriers; chunk numbers outside [0, nchunks) name no chunk.
template <class Op, int R, bool STREAM, int NCOPY, bool UNAL = false>
__global__ __launch_bounds__((2 + NCOPY) * kWave) void stream_kernel_staged(typename Op::Params prm, int64_t M, int T) {
    using G = TileGeom<R>;
    constexpr int TC = G::kChunk;
    constexpr int NI = Op::kIn, NO = Op::kOut, NT = NI > NO ? NI : NO;
    constexpr int PASSES = G::kPasses / NCOPY;
    static_assert(PASSES * NCOPY == G::kPasses, "copy waves share the passes evenly");
    static_assert(Op::kStages == 2 && !Op::kReverse, "two forward stages");
    __shared__ __attribute__((aligned(16))) float tiles[3][NT][G::kTileFloats];

    const int lane = threadIdx.x & (kWave - 1);
    const int role = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // wave-uniform
    const int64_t m0 = (int64_t)blockIdx.x * R;
    const int rows = (int)((M - m0) < R ? (M - m0) : R);
    const unsigned base_f = (unsigned)(reinterpret_cast<uintptr_t>(prm.in[0]) >> 2);
    const int a_lane = (int)((base_f + (unsigned)(m0 + lane) * (unsigned)T) & 31u);
    const int nchunks = chunk_count<TC>(a_lane, lane < rows, T);
    const int periods = (nchunks + 2 + 2) / 3 * 3;          // the last chunk leaves in period nchunks + 1
    const int interior_end = (T & ~31) / TC;

    auto sequential = [&](auto& stage, int lag) {
        stage.init(prm, m0 + lane, lane < rows);
        for (int j = 0; j < periods; j += 3) {
#pragma unroll
            for (int h = 0; h < 3; ++h) {
                const int chunk = j + h - lag;
                __syncthreads();                               // barrier j+h
                if (chunk >= 0 && chunk < nchunks)
                    run_chunk<typename std::remove_reference<decltype(stage)>::type, R, 4, kTileSamples, UNAL>(
                        stage, tiles[(h + 3 - lag) % 3], lane, chunk, chunk >= 1 && chunk < interior_end, a_lane, T);
            }
        }
        __syncthreads();                                       // barrier `periods`
        stage.finish(prm, m0 + lane, lane < rows);
    };
    if (role == 0) {
        typename Op::Stage0 st;
        sequential(st, 0);
    } else if (role == 1) {
        typename Op::Stage1 st;
        sequential(st, 1);
    } else {
        Op uni;                                                // wave-uniform members only (pre, post, derive)
        uni.init(prm, 0, false);
        Copier<Op, R, STREAM, PASSES, kTileSamples, UNAL> io;
        io.init(prm, m0, rows, T, lane, base_f, (role - 2) * PASSES);
        float4 fetched[3][NI][PASSES];
#pragma unroll
        for (int d = 0; d < 3; ++d) io.fetch_into(fetched[d], d);
        io.prime_stores();
        io.to_tiles(uni, tiles[0], fetched[0], 0);
        io.fetch_into(fetched[0], 3);
        __syncthreads();                                       // barrier 0
        io.fill_unreached(prm, m0, lane);                      // while the first wave works on chunk 0
        for (int j = 0; j < periods; j += 3) {
#pragma unroll
            for (int h = 0; h < 3; ++h) {
                io.copy_out(uni, tiles[(h + 1) % 3], j + h - 2);
                io.to_tiles(uni, tiles[(h + 1) % 3], fetched[(h + 1) % 3], j + h + 1);
                io.fetch_into(fetched[(h + 1) % 3], j + h + 4);
                __syncthreads();                               // barrier j+h+1
            }
        }
        io.report_range(prm);
    }
}

// ---------------------------------------------------------------------------------------------
// Rows that are not whole quads (T % 4 != 0, bases that are only dword-aligned) and are short (fewer than
// kUnalignedMinSteps steps; longer ones take the multi-wave kernels in their UNAL form) or longer than 2^22 steps:
// same tiling, 16-byte accesses at dword-aligned addresses for whole quads, no phase, no prefetch, no boundary
// handling.  Bit-exact.
template <class Op, int R>
__global__ __launch_bounds__(kWave) void stream_kernel_scalar(typename Op::Params prm, int64_t M, int T) {
    using G = TileGeom<R>;
    constexpr int TC = G::kChunk;
    constexpr int NI = Op::kIn, NO = Op::kOut, ND = DerivedCount<Op>::value, NT = NI > NO ? NI : NO;
    __shared__ __attribute__((aligned(16))) float tile[NT][G::kTileFloats];

    const int lane = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.x * R;
    const int rows = (int)((M - m0) < R ? (M - m0) : R);

    Op op;
    op.init(prm, m0 + lane, lane < rows);

    const int nchunks = (T + TC - 1) / TC;
    const int crow = lane / G::kQuads;
    const int cq = lane % G::kQuads;

    constexpr unsigned SI = ShiftInMask<Op>::value, SO = ShiftOutMask<Op>::value;
    constexpr bool kShifts = SI != 0 || SO != 0;
    int kin[kShifts ? G::kPasses : 1], kout[kShifts ? G::kPasses : 1];
    if constexpr (kShifts) {
        const auto& sh = prm.shifts;
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
            kin[p] = (SI != 0 && r < rows) ? in_shift_of(sh, m0 + r, T) : 0;
            kout[p] = (SO != 0 && r < rows) ? out_shift_of(sh, m0 + r, T) : 0;
        }
        if constexpr (SO != 0) {
            // positions of a shifted output that no sample reaches (see Copier::fill_unreached)
            for (int r = 0; r < rows; ++r) {
                const int kr = out_shift_of(sh, m0 + r, T);
                const int mag = kr < 0 ? -kr : kr;
                const int len = mag > T ? T : mag;
                for (int j = lane; j < len; j += kWave) {
                    const int64_t pos = (int64_t)(m0 + r) * (int64_t)T + (kr < 0 ? T - len + j : j);
                    const float v = (sh.head && kr > 0 && j == kr - 1) ? sh.head[m0 + r] : 0.f;
#pragma unroll
                    for (int o = 0; o < NO + ND; ++o)
                        if (((SO >> o) & 1u) != 0 && prm.out[o]) prm.out[o][pos] = v;
                }
            }
        }
    }

    for (int k = 0; k < nchunks; ++k) {
        const int chunk = Op::kReverse ? nchunks - 1 - k : k;
        const int t = chunk * TC + 4 * cq;
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
            const int64_t off = (int64_t)(m0 + r) * (int64_t)T + (int64_t)t;
            float4 x[NI];
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);      // zero fill: steps past T-1 must be no-ops
                if (r < rows && prm.in[i]) {
                    const int ki = ((SI >> i) & 1u) != 0 ? kin[p] : 0;   // sample t + e - ki, if the row has it
                    const float* src = prm.in[i] + off - ki;
                    const int s = t - ki;
                    if (t + 3 < T && s >= 0 && s + 3 < T) {
                        v = load_quad_dword_aligned(src);        // the whole quad exists: one 16-byte access
                    } else {
                        if (t + 0 < T && (unsigned)(s + 0) < (unsigned)T) v.x = src[0];
                        if (t + 1 < T && (unsigned)(s + 1) < (unsigned)T) v.y = src[1];
                        if (t + 2 < T && (unsigned)(s + 2) < (unsigned)T) v.z = src[2];
                        if (t + 3 < T && (unsigned)(s + 3) < (unsigned)T) v.w = src[3];
                    }
                }
                x[i] = v;
            }
            if constexpr (HasTransforms<Op>::value) op.pre(x);
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<float4*>(&tile[i][r * G::kPitch + 4 * cq]) = x[i];
        }
        __syncthreads();

        for (int q = 0; q < G::kQuads; ++q) {
            const int qq = Op::kReverse ? G::kQuads - 1 - q : q;
            if (lane < R && chunk * TC + 4 * qq < T) {
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
#pragma unroll
                    for (int o = 0; o < NO; ++o) y[o] = 0.f;
                    if (chunk * TC + 4 * qq + ss < T) op.step(x, y);   // steps past T-1 must not touch the state
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

#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int r = p * G::kRowsPerPass + crow;
            const int64_t off = (int64_t)(m0 + r) * (int64_t)T + (int64_t)t;
            float4 y[NO], v[NO + ND];
#pragma unroll
            for (int o = 0; o < NO; ++o) y[o] = *reinterpret_cast<const float4*>(&tile[o][r * G::kPitch + 4 * cq]);
            if constexpr (RangeChecked<Op>::value) {
#pragma unroll
                for (int o = 0; o < NO; ++o)
                    if (Op::range_log2(o) != 0 && r < rows && t < T &&       // a quad past the row's end was never written
                        range_exceeded(range_bits(y[o], Op::range_log2(o)), Op::range_log2(o)))
                        raise_range_flag(prm.range_flag);
            }
            if constexpr (HasTransforms<Op>::value) op.post(y);
#pragma unroll
            for (int o = 0; o < NO; ++o) v[o] = y[o];
            if constexpr (ND == 1) v[NO] = op.derive(y);
#pragma unroll
            for (int o = 0; o < NO + ND; ++o) {
                if (r < rows && prm.out[o]) {
                    const int ko = ((SO >> o) & 1u) != 0 ? kout[p] : 0;  // sample t + e goes to t + e + ko
                    float* d = prm.out[o] + off + ko;
                    const int u = t + ko;
                    if (t + 3 < T && u >= 0 && u + 3 < T) {
                        store_quad_dword_aligned(d, v[o]);       // the whole quad lands inside the row
                    } else {
                        if (t + 0 < T && (unsigned)(u + 0) < (unsigned)T) d[0] = v[o].x;
                        if (t + 1 < T && (unsigned)(u + 1) < (unsigned)T) d[1] = v[o].y;
                        if (t + 2 < T && (unsigned)(u + 2) < (unsigned)T) d[2] = v[o].z;
                        if (t + 3 < T && (unsigned)(u + 3) < (unsigned)T) d[3] = v[o].w;
                    }
                }
            }
        }
        __syncthreads();
    }
    op.finish(prm, m0 + lane, lane < rows);
}

// The Shifts of a forward pass (input read through in_shift, designated output stored through out_delay)
// and of the matching backward pass: the gradient arriving at the delayed output is read back through the
// output delay, the gradient of the input is stored back through the input shift.
inline int steps_to_int(int64_t k) {
    const int64_t lim = (int64_t)1 << 30;
    return (int)(k > lim ? lim : (k < -lim ? -lim : k));
}
inline Shifts forward_shifts(const slayer_delays* d, int64_t npb) {
    Shifts s{nullptr, nullptr, nullptr, nullptr, 0, 0, 1, 1.0f, npb > 0 ? npb : 1};
    if (d) {
        s.in_lut = d->in_shift; s.out_lut = d->out_delay; s.head = d->out_head; s.last = d->spike_last;
        s.in_steps = steps_to_int(d->in_steps); s.out_steps = steps_to_int(d->out_steps);
        if (d->sampling_time != 0.0f) s.ts = d->sampling_time;
    }
    return s;
}
inline Shifts backward_shifts(const slayer_delays* d, int64_t npb) {
    Shifts s{nullptr, nullptr, nullptr, nullptr, 0, 0, -1, 1.0f, npb > 0 ? npb : 1};
    if (d) {
        s.in_lut = d->out_delay; s.out_lut = d->in_shift;
        s.in_steps = steps_to_int(d->out_steps); s.out_steps = steps_to_int(d->in_steps);
        if (d->sampling_time != 0.0f) s.ts = d->sampling_time;
        s.delayed = d->delayed_spikes; s.delay_partial = d->grad_workspace;
    }
    return s;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int64_t kAlways = (int64_t)1 << 62;

// Rows per workgroup of the multi-wave kernel: 64 unless the Op says otherwise (kDuoRows).
template <class Op, class = void>
struct DuoRows { static constexpr int value = 64; };
template <class Op>
struct DuoRows<Op, decltype((void)Op::kDuoRows)> { static constexpr int value = Op::kDuoRows; };

// Copy waves per workgroup of the multi-wave kernel: 1 unless the Op says otherwise (kCopyWaves; an Op
// whose pre() is expensive wants more, so that the sequential wave does not wait for its tiles).
template <class Op, class = void>
struct CopyWaves { static constexpr int value = 1; };
template <class Op>
struct CopyWaves<Op, decltype((void)Op::kCopyWaves)> { static constexpr int value = Op::kCopyWaves; };

// Workgroups of the multi-wave kernel that one compute unit holds at a time (LDS and registers).
template <class Op, int R, bool STREAM, bool UNAL = false>
int duo_groups_per_cu() {
    static const int n = [] {
        int v = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, stream_kernel_duo<Op, R, STREAM, CopyWaves<Op>::value, kTileSamples, UNAL>,
                                                         (1 + CopyWaves<Op>::value) * kWave, 0) != hipSuccess)
            v = 0;
        return v;
    }();
    return n;
}

inline int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) cached[dev] = n;
    }
    return cached[dev];
}

template <class Op, int R>
int launch_stream_rows(const typename Op::Params& prm, int64_t M, int64_t T, bool vec, bool streaming,
                       hipStream_t stream) {
    const dim3 grid((unsigned)((M + R - 1) / R)), block(kWave);
    if (!vec)
        hipLaunchKernelGGL((stream_kernel_scalar<Op, R>), grid, block, 0, stream, prm, M, (int)T);
    else if (streaming)
        hipLaunchKernelGGL((stream_kernel<Op, R, true>), grid, block, 0, stream, prm, M, (int)T);
    else
        hipLaunchKernelGGL((stream_kernel<Op, R, false>), grid, block, 0, stream, prm, M, (int)T);
    return (int)hipGetLastError();
}

// Launch policy (thresholds measured on MI355X).
//  * dwordx4 path when T and every pointer allow it, else the dword fallback;
//  * non-temporal global accesses when the tensors are too large to be reused out of the
//    last-level cache;
//  * while every workgroup of the multi-wave kernel is resident at once, run time is set by the
//    latency of the sequential wave and that kernel is 10-40% faster (all 64 lanes hold a row);
//  * beyond that the one-wave kernel, with the rows per wave the Op asks for (kRows32Below,
//    kRows16Below): integer forward recurrences and backward passes with an exp per step keep all
//    64 lanes busy, the light float backward passes prefer 16 rows and 512-byte row segments.
// True when launch_stream would pick the dwordx4 path for these operands.
template <class Op>
bool stream_vectorizes(const typename Op::Params& prm, int64_t T) {
    // the dwordx4 kernels address a wave's rows with 32-bit byte offsets: 64 * T * 4 must stay below 2^31
    bool vec = (T % 4) == 0 && T <= (1 << 22);
    for (int i = 0; i < Op::kIn; ++i) vec = vec && aligned16(prm.in[i]);
    for (int o = 0; o < Op::kOut + DerivedCount<Op>::value; ++o) vec = vec && aligned16(prm.out[o]);
    return vec;
}

inline bool stream_is_large(int64_t M, int64_t T) { return M * T * 4 > ((int64_t)64 << 20); }

// True when launch_stream would run the multi-wave kernel: dwordx4 path and every workgroup resident at once.
template <class Op>
bool stream_fits_multiwave(const typename Op::Params& prm, int64_t M, int64_t T) {
    if (M == 0 || T == 0 || !stream_vectorizes<Op>(prm, T)) return false;
    constexpr int RD = DuoRows<Op>::value;
    const int per_cu = stream_is_large(M, T) ? duo_groups_per_cu<Op, RD, true>() : duo_groups_per_cu<Op, RD, false>();
    return (M + RD - 1) / RD <= (int64_t)per_cu * compute_units();
}

// Rows a multiple of 2 KB apart (or within 64 bytes of one: T = 512, 1024, 2048, also 500) put the same columns
// of every row on few memory channels, and a wave-wide access that touches eight rows (128-byte pieces) is served
// by them one after the other: a plain copy in that pattern drops from 5.0 to 3.6 TB/s at T = 1024
// (measured with a stand-alone copy program).  512-byte pieces of two rows per access (16 rows per wave) do not suffer;
// Ops whose recurrence is light enough to run on 16 lanes per wave ask for them (kLongPiecesOnAliasedRows:
// LI forward 311 -> 265 us, fused CUBA forward 616 -> 542 us at [2400,64,1024]; the adaptive-threshold and
// resonator recurrences lose more on the idle lanes than they gain).
inline bool row_stride_aliases(int64_t T) {
    const int64_t r = (T * 4) % 2048;
    return T >= 384 && (r <= 64 || r >= 2048 - 64);
}
template <class Op, class = void>
struct LongPiecesOnAliasedRows { static constexpr bool value = false; };
template <class Op>
struct LongPiecesOnAliasedRows<Op, decltype((void)Op::kLongPiecesOnAliasedRows)> {
    static constexpr bool value = Op::kLongPiecesOnAliasedRows;
};

// Ops that also take the multi-wave kernel when their workgroups outnumber the compute units' slots
// (kMultiwaveWhenLarge): the integer forward recurrences, whose one-wave kernel does copies and recurrence
// one after the other in the same wave.  Measured on [4,16,8192,300] / [4,16,2048,1000] / [4,16,1024,2000]
// tensors against the one-wave kernel: LI 262 -> 248 / 216 -> 212 / 220 -> 217 us, fused CUBA 542 -> 496 /
// 454 -> 436 / 453 -> 451, adaptive threshold 396 -> 377 / 336 -> 326 / 340 -> 339, resonator 525 -> 515 /
// 446 -> 436 / 466 -> 467, fused RF 700 -> 653 / 621 -> 584 / 609 -> 603, fused ALIF 698 -> 681 / 608 -> 583 /
// 611 -> 598.
template <class Op, class = void>
struct MultiwaveWhenLarge { static constexpr bool value = false; };
template <class Op>
struct MultiwaveWhenLarge<Op, decltype((void)Op::kMultiwaveWhenLarge)> {
    static constexpr bool value = Op::kMultiwaveWhenLarge;
};

// Workgroups of the multi-wave kernel a compute unit should hold when they come in several rounds: the fewer
// rows the chip works on at a time, the closer together its memory accesses fall (a plain copy in this access
// pattern gains 10-20 % when the rows in flight drop from all of the tensor to a tenth of it), but a
// workgroup spends its first microseconds waiting for its first tiles and others must cover for it.
constexpr int kGroupsPerCuWhenLarge = 4;

// Rows of a chunk or two are all prologue for a workgroup of several waves: below 128 steps the one-wave kernels
// stay (1 M rows of 16 steps: LI fwd 42 us one-wave, 74 us multi-wave; fused CUBA fwd 72 / 155; 512 K rows of
// 32 steps: 36 / 46 and 52 / 88; at 64 steps even to 25 % behind, from 128 steps on 3-15 % ahead).
constexpr int64_t kMultiwaveWhenLargeMinSteps = 128;

// Dynamic LDS (unused by the kernel) that holds a kernel with `static_lds` bytes to `groups` workgroups per CU.
inline unsigned lds_pad_for(int groups, size_t static_lds) {
    const size_t lds_per_cu = 160 * 1024, want = lds_per_cu / (size_t)(groups + 1) + 256;   // too much for groups + 1
    if (static_lds >= want) return 0;
    const size_t pad = want - static_lds;
    return (unsigned)(pad > 60 * 1024 ? 60 * 1024 : pad);
}
template <class Op, int R, bool STREAM, bool UNAL = false>
unsigned duo_pad_when_large() {
    static const unsigned pad = [] {
        hipFuncAttributes a;
        if (hipFuncGetAttributes(&a, (const void*)stream_kernel_duo<Op, R, STREAM, CopyWaves<Op>::value, kTileSamples, UNAL>) != hipSuccess)
            return 0u;
        return lds_pad_for(kGroupsPerCuWhenLarge, a.sharedSizeBytes);
    }();
    return pad;
}

// Ops made of two chained recurrences (kStages = 2) run them in two waves while every workgroup of that
// kernel is resident.
template <class Op, class = void>
struct StageCount { static constexpr int value = 1; };
template <class Op>
struct StageCount<Op, decltype((void)Op::kStages)> { static constexpr int value = Op::kStages; };

template <class Op, bool STREAM, bool UNAL = false>
int staged_groups_per_cu() {
    static const int n = [] {
        int v = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, stream_kernel_staged<Op, 64, STREAM, CopyWaves<Op>::value, UNAL>,
                                                         (2 + CopyWaves<Op>::value) * kWave, 0) != hipSuccess)
            v = 0;
        return v;
    }();
    return n;
}

// Staged Ops that keep the staged kernel when its workgroups come in several rounds (kStagedWhenLarge).
template <class Op, class = void>
struct StagedWhenLarge { static constexpr bool value = false; };
template <class Op>
struct StagedWhenLarge<Op, decltype((void)Op::kStagedWhenLarge)> { static constexpr bool value = Op::kStagedWhenLarge; };

// (fused CUBA forward, [4,16,8192,300] / [4,16,2048,1000] / [4,16,1024,2000]: 518 -> 494 / 452 -> 437 / 448 -> 443 us
// against the two-wave form; the fused ALIF forward, whose nine to twelve tiles leave room for one workgroup per
// compute unit, loses a quarter at T = 300 and stays with the two-wave form.)
constexpr int kStagedGroupsPerCuWhenLarge = 3;
template <class Op, bool STREAM, bool UNAL = false>
unsigned staged_pad_when_large() {
    static const unsigned pad = [] {
        hipFuncAttributes a;
        if (hipFuncGetAttributes(&a, (const void*)stream_kernel_staged<Op, 64, STREAM, CopyWaves<Op>::value, UNAL>) != hipSuccess)
            return 0u;
        return lds_pad_for(kStagedGroupsPerCuWhenLarge, a.sharedSizeBytes);
    }();
    return pad;
}

// Rows that are not whole quads (T % 4 != 0 or bases that are only dword-aligned): the multi-wave kernels in their
// UNAL form, at every neuron count (the one-wave kernels have no such form; short rows and rows longer than 2^22
// steps stay with the dword kernel).
// On short rows every chunk is an edge chunk and the sample-by-sample handling of the straddling quads outweighs
// what prefetch and overlap bring: measured against the dword kernel, 131 072 rows of 37 / 65 steps lose (fused CUBA
// fwd 36 -> 100 us, 54 -> 100 us), 65 536 rows of 129 steps are even, 32 768 rows of 301 steps win (81 -> 56 us).
constexpr int64_t kUnalignedMinSteps = 256;

template <class Op, bool STREAM>
int launch_stream_unaligned(const typename Op::Params& prm, int64_t M, int64_t T, hipStream_t stream) {
    constexpr int NC = CopyWaves<Op>::value;
    if constexpr (StageCount<Op>::value == 2) {
        const int per_cu = staged_groups_per_cu<Op, STREAM, true>();
        const bool fits = (M + 63) / 64 <= (int64_t)per_cu * compute_units();
        if (per_cu > 0 && (fits || StagedWhenLarge<Op>::value)) {
            const dim3 grid((unsigned)((M + 63) / 64)), block((2 + NC) * kWave);
            const unsigned pad = fits ? 0u : staged_pad_when_large<Op, STREAM, true>();
            hipLaunchKernelGGL((stream_kernel_staged<Op, 64, STREAM, NC, true>), grid, block, pad, stream, prm, M, (int)T);
            return (int)hipGetLastError();
        }
    }
    constexpr int RD = DuoRows<Op>::value;
    const int64_t groups = (M + RD - 1) / RD;
    const bool resident = groups <= (int64_t)duo_groups_per_cu<Op, RD, STREAM, true>() * compute_units();
    const dim3 grid((unsigned)groups), block((1 + NC) * kWave);
    const unsigned pad = resident ? 0u : duo_pad_when_large<Op, RD, STREAM, true>();
    hipLaunchKernelGGL((stream_kernel_duo<Op, RD, STREAM, NC, kTileSamples, true>), grid, block, pad, stream, prm, M, (int)T);
    return (int)hipGetLastError();
}

template <class Op>
int launch_stream(const typename Op::Params& prm, int64_t M, int64_t T, hipStream_t stream) {
    if (M == 0 || T == 0) return 0;
    const bool vec = stream_vectorizes<Op>(prm, T);
    const bool streaming = stream_is_large(M, T);
    if (!vec && T >= kUnalignedMinSteps && T <= (1 << 22))
        return streaming ? launch_stream_unaligned<Op, true>(prm, M, T, stream)
                         : launch_stream_unaligned<Op, false>(prm, M, T, stream);
    const bool long_pieces = LongPiecesOnAliasedRows<Op>::value && row_stride_aliases(T);
    if constexpr (StageCount<Op>::value == 2) {
        const int per_cu = streaming ? staged_groups_per_cu<Op, true>() : staged_groups_per_cu<Op, false>();
        const bool fits = (M + 63) / 64 <= (int64_t)per_cu * compute_units();
        if (vec && per_cu > 0 && (fits || (StagedWhenLarge<Op>::value && !long_pieces && T >= kMultiwaveWhenLargeMinSteps))) {
            constexpr int NC = CopyWaves<Op>::value;
            const dim3 grid((unsigned)((M + 63) / 64)), block((2 + NC) * kWave);
            if (streaming) {
                const unsigned pad = fits ? 0u : staged_pad_when_large<Op, true>();
                hipLaunchKernelGGL((stream_kernel_staged<Op, 64, true, NC>), grid, block, pad, stream, prm, M, (int)T);
            } else {
                const unsigned pad = fits ? 0u : staged_pad_when_large<Op, false>();
                hipLaunchKernelGGL((stream_kernel_staged<Op, 64, false, NC>), grid, block, pad, stream, prm, M, (int)T);
            }
            return (int)hipGetLastError();
        }
    }
    const bool resident = stream_fits_multiwave<Op>(prm, M, T);
    if (resident || (vec && MultiwaveWhenLarge<Op>::value && !long_pieces && T >= kMultiwaveWhenLargeMinSteps)) {
        constexpr int RD = DuoRows<Op>::value;
        constexpr int NC = CopyWaves<Op>::value;
        const dim3 grid((unsigned)((M + RD - 1) / RD)), block((1 + NC) * kWave);
        if (streaming) {
            const unsigned pad = resident ? 0u : duo_pad_when_large<Op, RD, true>();
            hipLaunchKernelGGL((stream_kernel_duo<Op, RD, true, NC>), grid, block, pad, stream, prm, M, (int)T);
        } else {
            const unsigned pad = resident ? 0u : duo_pad_when_large<Op, RD, false>();
            hipLaunchKernelGGL((stream_kernel_duo<Op, RD, false, NC>), grid, block, pad, stream, prm, M, (int)T);
        }
        return (int)hipGetLastError();
    }
    if (M < Op::kRows16Below || (LongPiecesOnAliasedRows<Op>::value && row_stride_aliases(T)))
        return launch_stream_rows<Op, 16>(prm, M, T, vec, streaming, stream);
    if constexpr (Op::kRows16Below < kAlways && Op::kRows16Below < Op::kRows32Below)
        if (M < Op::kRows32Below) return launch_stream_rows<Op, 32>(prm, M, T, vec, streaming, stream);
    if constexpr (Op::kRows32Below < kAlways)
        return launch_stream_rows<Op, 64>(prm, M, T, vec, streaming, stream);
    return 0;   // not reached: every neuron count is covered by the branches above
}

}  // namespace slayer
