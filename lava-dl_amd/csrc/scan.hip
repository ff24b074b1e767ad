// Reverse-time linear recurrences as wave-level scans.
//
// The backward pass of a leaky integrator, g[t] = a * g[t+1] + go[t], is linear in g, so it does not have to
// be walked one step after the other: a lane takes 4 consecutive steps of a row, 64 lanes take 64 consecutive
// quads of the tensor, and a suffix scan over the lanes of (multiplier, offset) pairs hands every lane the
// gradient that enters its quad from later times.  Rows end wherever they end among the lanes: the last quad of
// a row carries multiplier 0, which cuts the chain there.  Memory is read and written as one linear stream
// (1 KB per tensor and wave-wide access, no LDS transpose, no row-segmented access pattern), which is what the
// spike kernels reach 0.8 of the HBM peak with; the row-staged engine stays below 0.7.
//
// Arithmetic: once a lane knows the gradient that enters its quad it evaluates its 4 steps exactly as the
// sequential recurrence does (separate multiply and add), so the result differs from the sequential evaluation
// only through the rounding of that entering value (a few ulp: six combine steps with |a| <= 1).
#include "common.h"
#include "tile.h"
#include <stdlib.h>

namespace slayer {

int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);   // li.hip

constexpr int kScanWaves = 4;           // waves per workgroup, each with a span of rows of its own
constexpr int kScanMaxRows = 64;        // rows per wave at most (LDS tables)

// Cross-lane moves as DPP modifiers (they fold into the VALU instruction that consumes them): the value of the
// lane n below inside a row of 16 lanes (`fill` where there is none), lane 15 / 31 of the rows below for the
// rows in `rows`, and the lane just below across the whole wave.
template <int N>
__device__ __forceinline__ float lane_below_in_row(float v, float fill) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x110 + N, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_bcast15(float v, float fill) {      // rows 1 and 3 <- lane 15 of rows 0 and 2
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x142, 0xa, 0xf, false));
}
__device__ __forceinline__ float row_bcast31(float v, float fill) {      // rows 2 and 3 <- lane 31
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x143, 0xc, 0xf, false));
}
__device__ __forceinline__ float lane_below(float v, float fill) {       // lane l <- lane l - 1, lane 0 <- fill
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x138, 0xf, 0xf, false));
}

// c -> B + A * c applied to c.  A map with multiplier 0 is a cut (the last quad of a row): it lets nothing in, not
// even an Inf or a NaN that a later row produced (0 * Inf would be a NaN), so rows stay independent of each other
// as they are in a step-by-step evaluation.  For finite operands the result is the same bit for bit.
__device__ __forceinline__ float apply_affine(float A, float c, float B) {
    const float v = __fmaf_rn(A, c, B);
    return A == 0.0f ? B : v;
}

// Inclusive scan over the lanes, lowest lane first, of affine maps c -> B + A * c: afterwards (A, B) of lane l is
// the composition of the maps of lanes 0 .. l (lane 0 applied first).
// The plain composition (two instructions per step) is right whenever every partial result is finite: a cut's
// 0 * b is then 0, which is what the cut means.  An Inf or a NaN anywhere in the wave survives into the final B of
// its lane, so one test afterwards finds the rare wave that has one, and that wave repeats the scan with the cut
// taken by a select (0 * Inf would be a NaN and would cross into the row below).  The same bits either way for
// finite operands.
__device__ __forceinline__ void scan_affine(float& A, float& B) {
    const float A0 = A, B0 = B;
#define SLAYER_COMBINE(An, Bn) do { const float an_ = (An), bn_ = (Bn); B = __fmaf_rn(A, bn_, B); A = A * an_; } while (0)
    SLAYER_COMBINE(lane_below_in_row<1>(A, 1.0f), lane_below_in_row<1>(B, 0.0f));
    SLAYER_COMBINE(lane_below_in_row<2>(A, 1.0f), lane_below_in_row<2>(B, 0.0f));
    SLAYER_COMBINE(lane_below_in_row<4>(A, 1.0f), lane_below_in_row<4>(B, 0.0f));
    SLAYER_COMBINE(lane_below_in_row<8>(A, 1.0f), lane_below_in_row<8>(B, 0.0f));
    SLAYER_COMBINE(row_bcast15(A, 1.0f), row_bcast15(B, 0.0f));
    SLAYER_COMBINE(row_bcast31(A, 1.0f), row_bcast31(B, 0.0f));
#undef SLAYER_COMBINE
    if (__any(!(fabsf(B) <= 3.402823466e+38f))) {
        A = A0; B = B0;
#define SLAYER_COMBINE(An, Bn) do { const float an_ = (An), bn_ = (Bn); const bool cut_ = A == 0.0f;            \
        const float b2_ = __fmaf_rn(A, bn_, B), a2_ = A * an_; B = cut_ ? B : b2_; A = cut_ ? 0.0f : a2_; } while (0)
        SLAYER_COMBINE(lane_below_in_row<1>(A, 1.0f), lane_below_in_row<1>(B, 0.0f));
        SLAYER_COMBINE(lane_below_in_row<2>(A, 1.0f), lane_below_in_row<2>(B, 0.0f));
        SLAYER_COMBINE(lane_below_in_row<4>(A, 1.0f), lane_below_in_row<4>(B, 0.0f));
        SLAYER_COMBINE(lane_below_in_row<8>(A, 1.0f), lane_below_in_row<8>(B, 0.0f));
        SLAYER_COMBINE(row_bcast15(A, 1.0f), row_bcast15(B, 0.0f));
        SLAYER_COMBINE(row_bcast31(A, 1.0f), row_bcast31(B, 0.0f));
#undef SLAYER_COMBINE
    }
}

// Inclusive sum over the lanes below that belong to the same run: lane l adds lanes l - reach .. l - 1.
__device__ __forceinline__ float sum_run(float s, int lane, int reach) {
    const int in_row = lane & 15;
    float v;
    v = lane_below_in_row<1>(s, 0.0f); s += reach >= 1 ? v : 0.0f;
    v = lane_below_in_row<2>(s, 0.0f); s += reach >= 2 ? v : 0.0f;
    v = lane_below_in_row<4>(s, 0.0f); s += reach >= 4 ? v : 0.0f;
    v = lane_below_in_row<8>(s, 0.0f); s += reach >= 8 ? v : 0.0f;
    v = row_bcast15(s, 0.0f); s += reach > in_row ? v : 0.0f;               // the run goes on below this row of 16
    v = row_bcast31(s, 0.0f); s += reach > (lane & 31) ? v : 0.0f;         // ... and below this half of the wave
    return s;
}

// ---------------------------------------------------------------------------------------------
// Workgroup-level pieces shared by the scan kernels.
//
// A workgroup of kScanWaves waves owns `rpg` consecutive rows = one contiguous span of rpg * QR quads and walks it
// from its end to its start, 64 * kScanWaves quads per pass (so a span is a few passes and the chip as a whole
// reads and writes memory as one linear stream).  Thread t of a pass holds quad 64 * kScanWaves - 1 - t of the
// pass: a lower lane and a lower wave are a later time, the scans run upwards.  Within a pass the gradient that
// leaves lane 63 of a wave enters lane 0 of the next wave: every wave publishes the map of its 64 quads taken
// together, one barrier, and every wave applies the maps of the waves before it to what the previous pass left.
constexpr int kScanQuads = kScanWaves * kWave;       // quads per pass

struct ScanSpan {
    int tid, lane, wv, rows, nq, npass;
    int64_t row0;
    __device__ __forceinline__ void init(int64_t M, int QR, int rpg) {
        tid = threadIdx.x;
        lane = tid & (kWave - 1);
        wv = __builtin_amdgcn_readfirstlane(tid >> 6);
        row0 = (int64_t)blockIdx.x * rpg;
        rows = (int)((M - row0) < rpg ? (M - row0) : rpg);
        nq = rows * QR;
        npass = (nq + kScanQuads - 1) / kScanQuads;
    }
    // quad of this thread in the span for the pass that is worked on first (the last one in memory)
    __device__ __forceinline__ int first_quad() const { return (npass - 1) * kScanQuads + (kScanQuads - 1 - tid); }
};

// Row and position in the row of a thread's quad, kept up to date from pass to pass.
struct ScanCursor {
    int lq, r, pos;
    __device__ __forceinline__ void init(int lq0, int nq, int QR) {
        lq = lq0;
        r = (lq < nq ? lq : nq - 1) / QR;
        pos = lq - r * QR;                                           // >= QR for a quad past the end of the span
    }
    __device__ __forceinline__ void next(int QR) {
        lq -= kScanQuads;
        pos -= kScanQuads;
        while (pos < 0) { pos += QR; --r; }
        if (r < 0) { r = 0; pos = 0; }                               // before the span: the thread is idle from here on
    }
};

// (row0 mod npb) once with scalar 64-bit arithmetic; row rr of the span then uses parameter
// ((first + rr) mod npb) / per_param, in 32 bits.
__device__ __forceinline__ unsigned scan_first_in_batch(int64_t row0, unsigned npb) {
    return (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)((uint64_t)row0 % (uint64_t)npb));
}

// LDS of one real-valued scan: per pass parity, the map of each wave's 64 quads and what the pass leaves behind.
struct RealStage {
    float A[2][kScanWaves], B[2][kScanWaves], carry[2];
};

// One pass of a real recurrence g[t] = a * g[t+1] + d[t] on this thread's quad d: returns the four results.
// `ent` receives the gradient that entered the quad (0 at the end of a row).  One workgroup barrier.
__device__ __forceinline__ float4 real_stage(RealStage& L, const ScanSpan& sp, int parity, float a, float4 d,
                                             bool active, bool row_end, float& ent) {
    // the quad by itself (nothing entering): h0 is what leaves it, a^4 what an entering gradient is scaled by
    const float h3 = d.w;
    const float h2 = a * h3 + d.z;
    const float h1 = a * h2 + d.y;
    const float h0 = a * h1 + d.x;
    const float a2 = a * a, a3 = a2 * a, a4 = a2 * a2;
    float A = (active && !row_end) ? a4 : 0.0f;                      // the last quad of a row lets nothing in
    float B = active ? h0 : 0.0f;
    scan_affine(A, B);
    if (sp.lane == kWave - 1) { L.A[parity][sp.wv] = A; L.B[parity][sp.wv] = B; }
    __syncthreads();
    // what enters this wave: what the previous pass left, taken through the waves before this one
    float carry = L.carry[parity];
#pragma unroll
    for (int w = 0; w < kScanWaves - 1; ++w)
        if (w < sp.wv) carry = apply_affine(L.A[parity][w], carry, L.B[parity][w]);
    const float leaving = apply_affine(A, carry, B);                 // gradient leaving this thread's quad
    float entering = lane_below(leaving, carry);
    if (row_end || !active) entering = 0.0f;
    ent = entering;
    float4 g;
    g.w = __fmaf_rn(a, entering, h3);
    g.z = __fmaf_rn(a2, entering, h2);
    g.y = __fmaf_rn(a3, entering, h1);
    g.x = __fmaf_rn(a4, entering, h0);
    if (sp.tid == kScanQuads - 1) L.carry[parity ^ 1] = g.x;          // the earliest quad of the pass (always inside the span)
    return g;
}

// sum_t g[t+1] * y[t] over a quad (g[t+1] of its last step is what entered it)
__device__ __forceinline__ float next_step_product(float4 g, float entering, float4 y) {
    return __fmaf_rn(g.y, y.x, __fmaf_rn(g.z, y.y, __fmaf_rn(g.w, y.z, entering * y.w)));
}

// Adds a quad's contribution to the sum of its row: first over the lanes of this wave that hold the same row (the
// row's first quad in the wave sits in the highest lane of the run and collects the lanes below), then into the
// wave's own table, one lane per row.
__device__ __forceinline__ void add_to_row(float* table, float s, const ScanSpan& sp, const ScanCursor& c, int QR,
                                           bool active) {
    if (!active) s = 0.0f;
    const int reach = active ? QR - 1 - c.pos : 0;                   // quads of the row after this one
    s = sum_run(s, sp.lane, reach);
    if (active && (c.pos == 0 || sp.lane == kWave - 1)) table[c.r] += s;
}

// partial[row] = sum over the waves' tables, in wave order
__device__ __forceinline__ void store_row_sums(float* partial, const float (*table)[kScanMaxRows], const ScanSpan& sp) {
    for (int rr = sp.tid; rr < sp.rows; rr += kScanQuads) {
        float s = table[0][rr];
#pragma unroll
        for (int w = 1; w < kScanWaves; ++w) s += table[w][rr];
        partial[sp.row0 + rr] = s;
    }
}

// ---------------------------------------------------------------------------------------------
// Axonal delays folded into a scan (see Shifts in tile.h): the tensor named as shifted input is read as
// x[t] = in[t - kin], the outputs are stored as out[t + kout], row by row.  A lane's quad of four steps then sits at
// a dword-aligned address of its row, or straddles an end of the row.
struct ScanShiftTables { int kin[kScanMaxRows], kout[kScanMaxRows]; };

__device__ __forceinline__ void scan_shift_tables(ScanShiftTables& tab, const Shifts& sh, const ScanSpan& sp, int T) {
    for (int rr = sp.tid; rr < sp.rows; rr += kScanQuads) {
        tab.kin[rr] = in_shift_of(sh, sp.row0 + rr, T);
        tab.kout[rr] = out_shift_of(sh, sp.row0 + rr, T);
    }
}

// element e of the result is element e + d of q, zero outside it
__device__ __forceinline__ float4 scan_place(float4 q, int d) {
    const float a[4] = {q.x, q.y, q.z, q.w};
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int j = e + d;
        r[e] = j == 0 ? a[0] : (j == 1 ? a[1] : (j == 2 ? a[2] : (j == 3 ? a[3] : 0.f)));
    }
    return make_float4(r[0], r[1], r[2], r[3]);
}

// The quad of steps 4*pos .. 4*pos+3 of row r read through the shift k: one 16-byte load at the nearest position
// inside the row (out of range when no sample of the quad exists); `d` is what scan_place() needs afterwards.
__device__ __forceinline__ float4 scan_load_shifted(__amdgpu_buffer_rsrc_t src, bool in_span, int r, int pos, int k,
                                                    int T, int& d) {
    const int s = 4 * pos - k;
    const int sc = s < 0 ? 0 : (s > T - 4 ? T - 4 : s);
    const bool some = in_span && s > -4 && s < T;
    d = some ? s - sc : 0;
    return buf_load4<false>(src, some ? (r * T + sc) * 4 : kOutOfRange);
}

// The quad of steps 4*pos .. of row r stored through the shift k (sample t lands at t + k; samples that leave the
// row are dropped): one 16-byte store when the whole quad lands inside the row, else sample by sample.  Never
// streaming: a shifted quad ends in a partial line that a neighbouring quad completes.
__device__ __forceinline__ void scan_store_shifted(__amdgpu_buffer_rsrc_t dst, bool active, int r, int pos, int k,
                                                   int T, float4 v) {
    const int u = 4 * pos + k;
    const bool whole = active && u >= 0 && u <= T - 4;
    const bool part = active && !whole && u > -4 && u < T;
    const int base = (r * T + u) * 4;
    buf_store4<false>(dst, whole ? base : kOutOfRange, v);
    if (__any(part)) {
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            buf_store1<false>(dst, (part && (unsigned)(u + j) < (unsigned)T) ? base + 4 * j : kOutOfRange, e[j]);
    }
}

// Rows of any length (T >= 4 floats, not a whole number of quads): a row is walked as ceil(T / 4) quads, the last
// of which holds T mod 4 steps followed by steps that do not exist.  Its 16-byte load sits at T - 4, so the wanted
// samples arrive in the upper elements: scan_tail_place() moves them down by `dd` = 4 - T mod 4 (uniform) and
// zeroes the rest, after which the steps that do not exist behave as steps with zero input behind the row's end.
__device__ __forceinline__ float4 scan_load_row(__amdgpu_buffer_rsrc_t src, bool in_span, int r, int pos, int T) {
    const int s = 4 * pos;
    return buf_load4<false>(src, in_span ? (r * T + (s > T - 4 ? T - 4 : s)) * 4 : kOutOfRange);
}
__device__ __forceinline__ float4 scan_tail_place(float4 q, int dd, bool row_end) {
    float4 p = q;
    if (dd == 1) p = make_float4(q.y, q.z, q.w, 0.f);
    else if (dd == 2) p = make_float4(q.z, q.w, 0.f, 0.f);
    else if (dd == 3) p = make_float4(q.w, 0.f, 0.f, 0.f);
    return row_end ? p : q;
}

// The steps of a row's last quad that do not exist (dd of them) hold nothing: a gradient read through a negative
// shift finds samples of the row at their positions, which must not enter the recurrence.
__device__ __forceinline__ float4 scan_tail_mask(float4 q, int dd, bool row_end) {
    return row_end ? make_float4(q.x, dd >= 3 ? 0.f : q.y, dd >= 2 ? 0.f : q.z, dd >= 1 ? 0.f : q.w) : q;
}

// Zeros at the positions of a shifted output that no sample reaches: [0, k) for k > 0, [T + k, T) for k < 0.
__device__ __forceinline__ void scan_fill_unreached(__amdgpu_buffer_rsrc_t dst, const int* kout, const ScanSpan& sp,
                                                    int T) {
    for (int rr = 0; rr < sp.rows; ++rr) {
        const int k = kout[rr];
        const int mag = k < 0 ? -k : k;
        const int len = mag > T ? T : mag;
        for (int j = sp.tid; j < len; j += kScanQuads)
            buf_store1<false>(dst, (rr * T + (k < 0 ? T - len + j : j)) * 4, 0.0f);
    }
}

// The gradient of a learnable output delay, folded into a scan that reads the gradient of the delayed spikes anyway
// (axon/delay.py:201-221 in the reference: sum over t of grad[t] * (out[t-1] - out[t]) / Ts on the delayed tensor).
// A lane's quad of steps t sits at u = t + kf of the delayed tensors (kf: the forward pass's output shift of the
// row), so the lanes of a row cover u in [kf, T + kf); the delayed spikes are zero outside that range except for the
// one sample before it (the head a step delay carries over), so two more terms per row complete the sum: u = kf - 1
// (taken by the lane of the row's first quad) and u = T + kf (by the lane of its last).  All loads are issued for
// every lane, out of range where they do not apply.
struct DelayGradQuads { float4 s; float sp, ag, as, asp, bg, bs, bsp; };

__device__ __forceinline__ float scan_load_at(__amdgpu_buffer_rsrc_t src, bool on, int r, int u, int T) {
    return buf_load1<false>(src, (on && u >= 0 && u < T) ? (r * T + u) * 4 : kOutOfRange);
}
// k: the shift the scan reads the gradient through (minus the forward pass's output shift)
__device__ __forceinline__ void delay_grad_fetch(DelayGradQuads& d, __amdgpu_buffer_rsrc_t src_g, __amdgpu_buffer_rsrc_t src_s,
                                                 bool in_span, int r, int pos, int QR, int k, int T) {
    int unused;
    d.s = scan_load_shifted(src_s, in_span, r, pos, k, T, unused);
    const int kf = -k, u0 = 4 * pos + kf;
    d.sp = scan_load_at(src_s, in_span, r, u0 - 1, T);
    const bool first = in_span && pos == 0 && kf >= 1, last = in_span && pos == QR - 1 && kf < 0;
    d.ag = d.as = d.asp = d.bg = d.bs = d.bsp = 0.0f;
    if (__any(first || last)) {                                       // most waves hold no end of a row
        d.ag = scan_load_at(src_g, first, r, kf - 1, T);
        d.as = scan_load_at(src_s, first, r, kf - 1, T);
        d.asp = scan_load_at(src_s, first, r, kf - 2, T);
        d.bg = scan_load_at(src_g, last, r, T + kf, T);
        d.bs = scan_load_at(src_s, last, r, T + kf, T);
        d.bsp = scan_load_at(src_s, last, r, T + kf - 1, T);
    }
}
// g: the gradient quad in place (zeros where the row has no sample); place: what scan_place needs for d.s
__device__ __forceinline__ float delay_grad_terms(DelayGradQuads& d, float4 g, int place, float inv_ts) {
    if (__any(place != 0)) d.s = scan_place(d.s, place);
    const float f0 = -inv_ts, f1 = inv_ts;
    float acc = 0.0f;
    acc = __fmaf_rn(g.x, f0 * d.s.x + f1 * d.sp, acc);
    acc = __fmaf_rn(g.y, f0 * d.s.y + f1 * d.s.x, acc);
    acc = __fmaf_rn(g.z, f0 * d.s.z + f1 * d.s.y, acc);
    acc = __fmaf_rn(g.w, f0 * d.s.w + f1 * d.s.z, acc);
    acc = __fmaf_rn(d.ag, f0 * d.as + f1 * d.asp, acc);
    acc = __fmaf_rn(d.bg, f0 * d.bs + f1 * d.bsp, acc);
    return acc;
}

// ---------------------------------------------------------------------------------------------
// Leaky integrator backward.  npb (rows per batch element) and per_param (rows of a batch element that share a
// parameter; npb when there is one parameter) are 32-bit: the launcher refuses anything larger.
// ANYT: rows of any length T >= 4 (see scan_load_row); else T = 4 * QR and the span is read as one flat stream.
template <bool PARTIAL, bool STREAM, bool ANYT = false>
__global__ __launch_bounds__(kScanQuads) void li_bwd_scan_kernel(
        float* __restrict__ grad_in, float* __restrict__ partial, const float* __restrict__ grad_out,
        const float* __restrict__ out, const float* __restrict__ decay, int64_t M, int T, int QR, int rpg,
        unsigned npb, unsigned per_param) {
    __shared__ float a_tab[kScanMaxRows];
    __shared__ float row_sum[kScanWaves][kScanMaxRows];
    __shared__ RealStage stage;
    ScanSpan sp;
    sp.init(M, QR, rpg);
    const int nq = sp.nq;
    const int64_t base = sp.row0 * (int64_t)T;                       // first float of the span
    const unsigned span_bytes = (unsigned)(sp.rows * T) * 4u;
    const int dd = (4 - (T & 3)) & 3;
    const __amdgpu_buffer_rsrc_t src_g = make_rsrc(grad_out + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_y = make_rsrc(PARTIAL ? out + base : nullptr, PARTIAL ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(grad_in + base, span_bytes);

    ScanCursor cur, ahead;                           // ahead: the quad of this thread in the pass fetched next
    // Four pass buffers: the pass being worked on and the three after it, requested before anything else (a
    // workgroup lives for a handful of passes: what it reads should be on its way while it sets up).
    auto fetch = [&](float4& go, float4& y, int q) {
        const bool in_span = (unsigned)q < (unsigned)nq;
        if (ANYT) {
            go = scan_load_row(src_g, in_span, ahead.r, ahead.pos, T);
            y = PARTIAL ? scan_load_row(src_y, in_span, ahead.r, ahead.pos, T) : make_float4(0.f, 0.f, 0.f, 0.f);
            ahead.next(QR);
        } else {
            go = buf_load4<STREAM>(src_g, in_span ? q * 16 : kOutOfRange);
            y = PARTIAL ? buf_load4<STREAM>(src_y, in_span ? q * 16 : kOutOfRange) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    const int q0 = sp.first_quad();
    if (ANYT) { cur.init(q0, nq, QR); ahead = cur; }
    float4 go0, y0, go1, y1, go2, y2, go3, y3;
    fetch(go0, y0, q0);
    fetch(go1, y1, q0 - kScanQuads);
    fetch(go2, y2, q0 - 2 * kScanQuads);
    fetch(go3, y3, q0 - 3 * kScanQuads);

    const unsigned first = scan_first_in_batch(sp.row0, npb);
    for (int rr = sp.tid; rr < sp.rows; rr += kScanQuads)
        a_tab[rr] = 1.0f - decay[((first + (unsigned)rr) % npb) / per_param] / 4096.0f;
    if (PARTIAL)
        for (int rr = sp.lane; rr < sp.rows; rr += kWave) row_sum[sp.wv][rr] = 0.0f;
    int parity = (sp.npass - 1) & 1;
    if (sp.tid == 0) stage.carry[parity] = 0.0f;                     // nothing enters the last quad of the span
    __syncthreads();
    if (!ANYT) cur.init(q0, nq, QR);

    // one pass on the quads in (go, y); the buffer is then refilled with the pass four further on
    auto pass = [&](float4& go, float4& y) {
        const bool active = cur.lq < nq;
        const bool row_end = cur.pos == QR - 1;
        if (ANYT && dd != 0) {
            go = scan_tail_place(go, dd, row_end);
            if (PARTIAL) y = scan_tail_place(y, dd, row_end);
        }
        float entering;
        const float4 g = real_stage(stage, sp, parity, a_tab[cur.r], go, active, row_end, entering);
        if (ANYT) scan_store_shifted(dst, active, cur.r, cur.pos, 0, T, g);
        else buf_store4<STREAM>(dst, active ? cur.lq * 16 : kOutOfRange, g);
        if (PARTIAL) add_to_row(row_sum[sp.wv], next_step_product(g, entering, y), sp, cur, QR, active);
        fetch(go, y, cur.lq - 4 * kScanQuads);
        cur.next(QR);
        parity ^= 1;
    };
    for (int left = sp.npass;;) {
        pass(go0, y0); if (--left == 0) break;
        pass(go1, y1); if (--left == 0) break;
        pass(go2, y2); if (--left == 0) break;
        pass(go3, y3); if (--left == 0) break;
    }
    if (PARTIAL) {
        __syncthreads();
        store_row_sums(partial, row_sum, sp);
    }
}

// ---------------------------------------------------------------------------------------------
// Fused CUBA / ALIF backward: spike surrogate, then the voltage and the current recurrence, each as a scan of its
// own with the very arithmetic of li_bwd_scan_kernel -- the input gradient is bit-identical to the spike backward
// kernel followed by two launches of that kernel.  THETA: the spike threshold is a tensor (threshold + refractory
// of the adaptive neuron), else the scalar spike_thr.
// DELAY: also leaves the per-row sums of the output delay's gradient (SHIFT forms only, see delay_grad_fetch).
template <bool GRADED, bool DECAY_GRAD, bool THETA, bool STREAM, int MODE = 0, int NBUF = 3, bool DELAY = false>
__global__ __launch_bounds__(kScanQuads) void cuba_bwd_scan_kernel(
        float* __restrict__ grad_in, float* __restrict__ partial_i, float* __restrict__ partial_v,
        const float* __restrict__ grad_spikes, const float* __restrict__ voltage, const float* __restrict__ theta,
        const float* __restrict__ current, const float* __restrict__ i_decay, const float* __restrict__ v_decay,
        float spike_thr, float tau, float rho, int64_t M, int T, int QR, int rpg,
        unsigned npb, unsigned per_i, unsigned per_v, Shifts shifts) {
    constexpr bool SHIFT = MODE != 0, ANYT = MODE == 2;
    static_assert(!DELAY || SHIFT, "the delay gradient belongs to the forms that read the gradient through a delay");
    __shared__ float ai_tab[kScanMaxRows], av_tab[kScanMaxRows];
    __shared__ float sum_i[kScanWaves][kScanMaxRows], sum_v[kScanWaves][kScanMaxRows];
    __shared__ float sum_d[DELAY ? kScanWaves : 1][DELAY ? kScanMaxRows : 1];
    __shared__ RealStage stage_v, stage_i;
    __shared__ ScanShiftTables shift_tab;
    ScanSpan sp;
    sp.init(M, QR, rpg);
    const int nq = sp.nq;
    const int64_t base = sp.row0 * (int64_t)T;
    const unsigned span_bytes = (unsigned)(sp.rows * T) * 4u;
    const int dd = (4 - (T & 3)) & 3;
    const __amdgpu_buffer_rsrc_t src_g = make_rsrc(grad_spikes + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_v = make_rsrc(voltage + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_t = make_rsrc(THETA ? theta + base : nullptr, THETA ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t src_c = make_rsrc(DECAY_GRAD ? current + base : nullptr, DECAY_GRAD ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t dst = make_rsrc(grad_in + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_s = make_rsrc(DELAY ? shifts.delayed + base : nullptr, DELAY ? span_bytes : 0u);
    const float lead = (rho / 2.0f) / tau;
    const float inv_tau = 1.0f / tau;

    struct Quads { float4 g, v, th, c; int dg; DelayGradQuads dq; };
    // the saved traces (never shifted), then the gradient of the spikes (read through the output delay when SHIFT)
    auto fetch_saved = [&](Quads& x, int q, const ScanCursor& at) {
        const bool in_span = (unsigned)q < (unsigned)nq;
        const float4 none = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ANYT) {
            x.v = scan_load_row(src_v, in_span, at.r, at.pos, T);
            x.th = THETA ? scan_load_row(src_t, in_span, at.r, at.pos, T) : none;
            x.c = DECAY_GRAD ? scan_load_row(src_c, in_span, at.r, at.pos, T) : none;
        } else {
            const int off = in_span ? q * 16 : kOutOfRange;
            x.v = buf_load4<STREAM>(src_v, off);
            x.th = THETA ? buf_load4<STREAM>(src_t, off) : none;
            x.c = DECAY_GRAD ? buf_load4<STREAM>(src_c, off) : none;
        }
    };
    auto fetch_grad = [&](Quads& x, int q, const ScanCursor& at) {
        if (SHIFT) {
            x.g = scan_load_shifted(src_g, (unsigned)q < (unsigned)nq, at.r, at.pos, shift_tab.kin[at.r], T, x.dg);
            if (DELAY)
                delay_grad_fetch(x.dq, src_g, src_s, (unsigned)q < (unsigned)nq, at.r, at.pos, QR, shift_tab.kin[at.r], T);
        } else {
            x.g = buf_load4<STREAM>(src_g, (unsigned)q < (unsigned)nq ? q * 16 : kOutOfRange);
            x.dg = 0;
        }
    };
    // NBUF pass buffers (up to four tensors each): the pass being worked on and the ones after it (spans of up to
    // three passes are requested whole with three buffers; longer spans gain 7-8 % from a fourth)
    const int q0 = sp.first_quad();
    Quads b[NBUF];
    ScanCursor cur, ahead;                           // ahead: the quad of this thread in the pass fetched next
    if (ANYT) {
        cur.init(q0, nq, QR);
        ahead = cur;
#pragma unroll
        for (int h = 0; h < NBUF; ++h) { fetch_saved(b[h], ahead.lq, ahead); ahead.next(QR); }
    } else {
#pragma unroll
        for (int h = 0; h < NBUF; ++h) fetch_saved(b[h], q0 - h * kScanQuads, ahead);
        cur.init(q0, nq, QR);
    }
    ahead = cur;
    if (!SHIFT) {
#pragma unroll
        for (int h = 0; h < NBUF; ++h) fetch_grad(b[h], q0 - h * kScanQuads, ahead);
    }

    const unsigned first = scan_first_in_batch(sp.row0, npb);
    for (int rr = sp.tid; rr < sp.rows; rr += kScanQuads) {
        const unsigned in_batch = (first + (unsigned)rr) % npb;
        ai_tab[rr] = 1.0f - rintf(i_decay[in_batch / per_i]) / 4096.0f;
        av_tab[rr] = 1.0f - rintf(v_decay[in_batch / per_v]) / 4096.0f;
    }
    if (SHIFT) scan_shift_tables(shift_tab, shifts, sp, T);
    if (DECAY_GRAD)
        for (int rr = sp.lane; rr < sp.rows; rr += kWave) { sum_i[sp.wv][rr] = 0.0f; sum_v[sp.wv][rr] = 0.0f; }
    if (DELAY)
        for (int rr = sp.lane; rr < sp.rows; rr += kWave) sum_d[sp.wv][rr] = 0.0f;
    int parity = (sp.npass - 1) & 1;
    if (sp.tid == 0) { stage_v.carry[parity] = 0.0f; stage_i.carry[parity] = 0.0f; }
    __syncthreads();
    if (SHIFT) {                                     // the shifts are known now
#pragma unroll
        for (int h = 0; h < NBUF; ++h) { fetch_grad(b[h], ahead.lq, ahead); ahead.next(QR); }
        scan_fill_unreached(dst, shift_tab.kout, sp, T);
    }

    // the surrogate, expression by expression as the spike backward kernel evaluates it
    auto surrogate = [&](float g, float v, float th) {
        const float d = v - (THETA ? th : spike_thr);
        return GRADED ? (rho * expf(fminf(d, 0.0f) * inv_tau)) * g : (lead * expf(-fabsf(d) * inv_tau)) * g;
    };
    auto pass = [&](Quads& x) {
        const bool active = cur.lq < nq;
        const bool row_end = cur.pos == QR - 1;
        if (SHIFT && __any(x.dg != 0)) x.g = scan_place(x.g, x.dg);      // rare: only where a row begins or ends
        if (ANYT && dd != 0) x.g = scan_tail_mask(x.g, dd, row_end);
        if (DELAY) add_to_row(sum_d[sp.wv], delay_grad_terms(x.dq, x.g, x.dg, 1.0f / shifts.ts), sp, cur, QR, active);
        if (ANYT && dd != 0) {
            x.v = scan_tail_place(x.v, dd, row_end);
            if (THETA) x.th = scan_tail_place(x.th, dd, row_end);
            if (DECAY_GRAD) x.c = scan_tail_place(x.c, dd, row_end);
        }
        const float4 gv = make_float4(surrogate(x.g.x, x.v.x, x.th.x), surrogate(x.g.y, x.v.y, x.th.y),
                                      surrogate(x.g.z, x.v.z, x.th.z), surrogate(x.g.w, x.v.w, x.th.w));
        float ent_v, ent_i;
        const float4 gc = real_stage(stage_v, sp, parity, av_tab[cur.r], gv, active, row_end, ent_v);
        const float4 gx = real_stage(stage_i, sp, parity, ai_tab[cur.r], gc, active, row_end, ent_i);
        if (SHIFT) scan_store_shifted(dst, active, cur.r, cur.pos, shift_tab.kout[cur.r], T, gx);
        else buf_store4<STREAM>(dst, active ? cur.lq * 16 : kOutOfRange, gx);
        if (DECAY_GRAD) {
            add_to_row(sum_v[sp.wv], next_step_product(gc, ent_v, x.v), sp, cur, QR, active);
            add_to_row(sum_i[sp.wv], next_step_product(gx, ent_i, x.c), sp, cur, QR, active);
        }
        fetch_saved(x, cur.lq - NBUF * kScanQuads, ahead);
        if (SHIFT) { fetch_grad(x, ahead.lq, ahead); ahead.next(QR); }
        else fetch_grad(x, cur.lq - NBUF * kScanQuads, ahead);
        cur.next(QR);
        parity ^= 1;
    };
    static_assert(NBUF == 3 || NBUF == 4, "pass buffers");
    for (int left = sp.npass;;) {
        pass(b[0]); if (--left == 0) break;
        pass(b[1]); if (--left == 0) break;
        pass(b[2]); if (--left == 0) break;
        if (NBUF == 4) { pass(b[NBUF - 1]); if (--left == 0) break; }
    }
    if (DECAY_GRAD || DELAY) __syncthreads();
    if (DECAY_GRAD) {
        store_row_sums(partial_i, sum_i, sp);
        store_row_sums(partial_v, sum_v, sp);
    }
    if constexpr (DELAY) store_row_sums(shifts.delay_partial, sum_d, sp);
}

// ---------------------------------------------------------------------------------------------
// Resonator backward: z[t] = mu * z[t+1] + g[t] over complex numbers, z = gr + i gi, mu = (c - i s) with
// c, s = cos_decay / 4096, sin_decay / 4096 (gr[t] = c gr[t+1] + s gi[t+1] + g_re[t],
// gi[t] = -s gr[t+1] + c gi[t+1] + g_im[t]).  Same structure as the real scan with complex maps.
struct Cx { float re, im; };
__device__ __forceinline__ Cx cmul(Cx a, Cx b) {
    return Cx{__fmaf_rn(a.re, b.re, -(a.im * b.im)), __fmaf_rn(a.re, b.im, a.im * b.re)};
}
__device__ __forceinline__ Cx cfma(Cx a, Cx b, Cx c) {            // a * b + c
    return Cx{__fmaf_rn(a.re, b.re, __fmaf_rn(-a.im, b.im, c.re)), __fmaf_rn(a.re, b.im, __fmaf_rn(a.im, b.re, c.im))};
}

struct ComplexStage {
    float Ar[2][kScanWaves], Ai[2][kScanWaves], Br[2][kScanWaves], Bi[2][kScanWaves], cr[2], ci[2];
};

// z -> B + A * z applied to z; a zero multiplier is a cut that lets nothing in (see apply_affine)
__device__ __forceinline__ Cx apply_affine_complex(Cx A, Cx z, Cx B) {
    const Cx v = cfma(A, z, B);
    const bool cut = A.re == 0.0f && A.im == 0.0f;
    return Cx{cut ? B.re : v.re, cut ? B.im : v.im};
}

// inclusive scan over the lanes of complex affine maps z -> B + A * z (see scan_affine: the plain composition
// first, the one with selected cuts only in a wave that holds an Inf or a NaN)
__device__ __forceinline__ void scan_affine_complex(Cx& A, Cx& B) {
    const Cx A0 = A, B0 = B;
#define SLAYER_COMBINE(M) do {                                                                                  \
        const Cx an_{M(A.re, 1.0f), M(A.im, 0.0f)}, bn_{M(B.re, 0.0f), M(B.im, 0.0f)};                          \
        B = cfma(A, bn_, B); A = cmul(A, an_); } while (0)
    SLAYER_COMBINE(lane_below_in_row<1>);
    SLAYER_COMBINE(lane_below_in_row<2>);
    SLAYER_COMBINE(lane_below_in_row<4>);
    SLAYER_COMBINE(lane_below_in_row<8>);
    SLAYER_COMBINE(row_bcast15);
    SLAYER_COMBINE(row_bcast31);
#undef SLAYER_COMBINE
    if (__any(!(fabsf(B.re) <= 3.402823466e+38f) || !(fabsf(B.im) <= 3.402823466e+38f))) {
        A = A0; B = B0;
#define SLAYER_COMBINE(M) do {                                                                                  \
        const Cx an_{M(A.re, 1.0f), M(A.im, 0.0f)}, bn_{M(B.re, 0.0f), M(B.im, 0.0f)};                          \
        const bool cut_ = A.re == 0.0f && A.im == 0.0f;                                                         \
        const Cx b2_ = cfma(A, bn_, B), a2_ = cmul(A, an_);                                                     \
        B = Cx{cut_ ? B.re : b2_.re, cut_ ? B.im : b2_.im};                                                     \
        A = Cx{cut_ ? 0.0f : a2_.re, cut_ ? 0.0f : a2_.im}; } while (0)
        SLAYER_COMBINE(lane_below_in_row<1>);
        SLAYER_COMBINE(lane_below_in_row<2>);
        SLAYER_COMBINE(lane_below_in_row<4>);
        SLAYER_COMBINE(lane_below_in_row<8>);
        SLAYER_COMBINE(row_bcast15);
        SLAYER_COMBINE(row_bcast31);
#undef SLAYER_COMBINE
    }
}

// SURR = 0: g_re / g_im are the incoming gradients of the two states (resonator backward).
// SURR = 1 (binary spikes) / 2 (graded): the fused resonate-and-fire backward -- g_re holds the gradient of the
// spikes, g_im is not read, and the gradients of the states come from the complex spike surrogate of the saved
// states, evaluated as the quads arrive (same expression order as cspike_bwd_kernel, so the result equals the
// chain surrogate -> resonator scan bit for bit); re / im are then read whether or not the sums are wanted.
struct SpikeSurrogate { float thr, tau, rho; };

template <int SURR>
__device__ __forceinline__ void complex_spike_surrogate(const SpikeSurrogate& k, float g, float r, float i,
                                                        float& g_re, float& g_im) {
    const float half_over_tau = (1.0f / 2.0f) / k.tau;
    const float inv_tau = 1.0f / k.tau;
    const float two_tau = 2.0f * k.tau;
    const float neg_rho_over_tau = (-k.rho) / k.tau;
    float d_re;
    if (SURR == 2) d_re = expf(-fmaxf(k.thr - r, 0.0f) * inv_tau);
    else d_re = half_over_tau * expf(-fabsf(r - k.thr) * inv_tau);
    const float d_im = half_over_tau * expf(-fabsf(i) * inv_tau);
    const float dr = r - k.thr;
    const float sg_r = dr > 0.0f ? 1.0f : (dr < 0.0f ? -1.0f : (dr == 0.0f ? 0.0f : dr));
    const float sg_i = i > 0.0f ? 1.0f : (i < 0.0f ? -1.0f : (i == 0.0f ? 0.0f : i));
    const float step_re = 0.5f * (1.0f + sg_r * (1.0f - two_tau * d_re));
    g_re = g * ((k.rho * d_re) * d_im);
    g_im = g * (((neg_rho_over_tau * sg_i) * d_im) * step_re);
}

template <bool PARTIAL, bool STREAM, int SURR, int MODE = 0, int NBUF = 3, bool DELAY = false>
__global__ __launch_bounds__(kScanQuads) void res_bwd_scan_kernel(
        float* __restrict__ g_re_in, float* __restrict__ g_im_in, float* __restrict__ partial_sin,
        float* __restrict__ partial_cos, const float* __restrict__ g_re, const float* __restrict__ g_im,
        const float* __restrict__ re, const float* __restrict__ im, const float* __restrict__ sin_decay,
        const float* __restrict__ cos_decay, SpikeSurrogate surr, int64_t M, int T, int QR, int rpg, unsigned npb,
        unsigned per_param, Shifts shifts) {
    constexpr bool SHIFT = MODE != 0, ANYT = MODE == 2;
    static_assert(MODE != 1 || SURR != 0, "delays are folded into the fused resonate-and-fire form only");
    static_assert(!DELAY || (SHIFT && SURR != 0), "the delay gradient belongs to the forms that read the spike gradient through a delay");
    __shared__ float c_tab[kScanMaxRows], s_tab[kScanMaxRows];
    __shared__ float sum_s[kScanWaves][kScanMaxRows], sum_c[kScanWaves][kScanMaxRows];
    __shared__ float sum_d[DELAY ? kScanWaves : 1][DELAY ? kScanMaxRows : 1];
    __shared__ ComplexStage L;
    __shared__ ScanShiftTables shift_tab;
    ScanSpan sp;
    sp.init(M, QR, rpg);
    const int nq = sp.nq;
    const int64_t base = sp.row0 * (int64_t)T;
    const unsigned span_bytes = (unsigned)(sp.rows * T) * 4u;
    const int dd = (4 - (T & 3)) & 3;
    constexpr bool kStates = PARTIAL || SURR != 0;          // the saved states are read
    const __amdgpu_buffer_rsrc_t src_gr = make_rsrc(g_re + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_gi = make_rsrc(SURR == 0 ? g_im + base : nullptr, SURR == 0 ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t src_re = make_rsrc(kStates ? re + base : nullptr, kStates ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t src_im = make_rsrc(kStates ? im + base : nullptr, kStates ? span_bytes : 0u);
    const __amdgpu_buffer_rsrc_t dst_r = make_rsrc(g_re_in + base, span_bytes), dst_i = make_rsrc(g_im_in + base, span_bytes);
    const __amdgpu_buffer_rsrc_t src_d = make_rsrc(DELAY ? shifts.delayed + base : nullptr, DELAY ? span_bytes : 0u);

    struct Quads { float4 gr, gi, re, im; int dg; DelayGradQuads dq; };
    // the tensors that are never shifted, then the incoming gradient (read through the output delay when SHIFT)
    auto fetch_saved = [&](Quads& x, int q, const ScanCursor& at) {
        const bool in_span = (unsigned)q < (unsigned)nq;
        const float4 none = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ANYT) {
            x.gi = SURR == 0 ? scan_load_row(src_gi, in_span, at.r, at.pos, T) : none;
            x.re = kStates ? scan_load_row(src_re, in_span, at.r, at.pos, T) : none;
            x.im = kStates ? scan_load_row(src_im, in_span, at.r, at.pos, T) : none;
        } else {
            const int off = in_span ? q * 16 : kOutOfRange;
            x.gi = SURR == 0 ? buf_load4<STREAM>(src_gi, off) : none;
            x.re = kStates ? buf_load4<STREAM>(src_re, off) : none;
            x.im = kStates ? buf_load4<STREAM>(src_im, off) : none;
        }
    };
    auto fetch_grad = [&](Quads& x, int q, const ScanCursor& at) {
        if (SHIFT) {
            x.gr = scan_load_shifted(src_gr, (unsigned)q < (unsigned)nq, at.r, at.pos, shift_tab.kin[at.r], T, x.dg);
            if (DELAY)
                delay_grad_fetch(x.dq, src_gr, src_d, (unsigned)q < (unsigned)nq, at.r, at.pos, QR, shift_tab.kin[at.r], T);
        } else {
            x.gr = buf_load4<STREAM>(src_gr, (unsigned)q < (unsigned)nq ? q * 16 : kOutOfRange);
            x.dg = 0;
        }
    };
    const int q0 = sp.first_quad();
    Quads b[NBUF];
    ScanCursor cur, ahead;                           // ahead: the quad of this thread in the pass fetched next
    if (ANYT) {
        cur.init(q0, nq, QR);
        ahead = cur;
#pragma unroll
        for (int h = 0; h < NBUF; ++h) { fetch_saved(b[h], ahead.lq, ahead); ahead.next(QR); }
    } else {
#pragma unroll
        for (int h = 0; h < NBUF; ++h) fetch_saved(b[h], q0 - h * kScanQuads, ahead);
        cur.init(q0, nq, QR);
    }
    ahead = cur;
    if (!SHIFT) {
#pragma unroll
        for (int h = 0; h < NBUF; ++h) fetch_grad(b[h], q0 - h * kScanQuads, ahead);
    }

    const unsigned first = scan_first_in_batch(sp.row0, npb);
    for (int rr = sp.tid; rr < sp.rows; rr += kScanQuads) {
        const unsigned j = ((first + (unsigned)rr) % npb) / per_param;
        c_tab[rr] = cos_decay[j] / 4096.0f;
        s_tab[rr] = sin_decay[j] / 4096.0f;
    }
    if (SHIFT) scan_shift_tables(shift_tab, shifts, sp, T);
    if (PARTIAL)
        for (int rr = sp.lane; rr < sp.rows; rr += kWave) { sum_s[sp.wv][rr] = 0.0f; sum_c[sp.wv][rr] = 0.0f; }
    if (DELAY)
        for (int rr = sp.lane; rr < sp.rows; rr += kWave) sum_d[sp.wv][rr] = 0.0f;
    int parity = (sp.npass - 1) & 1;
    if (sp.tid == 0) { L.cr[parity] = 0.0f; L.ci[parity] = 0.0f; }
    __syncthreads();
    if (SHIFT) {                                     // the shifts are known now
#pragma unroll
        for (int h = 0; h < NBUF; ++h) { fetch_grad(b[h], ahead.lq, ahead); ahead.next(QR); }
        scan_fill_unreached(dst_r, shift_tab.kout, sp, T);
        scan_fill_unreached(dst_i, shift_tab.kout, sp, T);
    }

    auto pass = [&](Quads& x) {
        const bool active = cur.lq < nq;
        const bool row_end = cur.pos == QR - 1;
        const Cx mu{c_tab[cur.r], -s_tab[cur.r]};
        if (SHIFT && __any(x.dg != 0)) x.gr = scan_place(x.gr, x.dg);    // rare: only where a row begins or ends
        if (ANYT && dd != 0) x.gr = scan_tail_mask(x.gr, dd, row_end);
        if (DELAY) add_to_row(sum_d[sp.wv], delay_grad_terms(x.dq, x.gr, x.dg, 1.0f / shifts.ts), sp, cur, QR, active);
        if (ANYT && dd != 0) {
            if (SURR == 0) x.gi = scan_tail_place(x.gi, dd, row_end);
            if (kStates) { x.re = scan_tail_place(x.re, dd, row_end); x.im = scan_tail_place(x.im, dd, row_end); }
        }
        if (SURR != 0) {                   // quads outside the span hold zeros: their gradient is zero too
            const float4 g = x.gr;
            complex_spike_surrogate<SURR>(surr, g.x, x.re.x, x.im.x, x.gr.x, x.gi.x);
            complex_spike_surrogate<SURR>(surr, g.y, x.re.y, x.im.y, x.gr.y, x.gi.y);
            complex_spike_surrogate<SURR>(surr, g.z, x.re.z, x.im.z, x.gr.z, x.gi.z);
            complex_spike_surrogate<SURR>(surr, g.w, x.re.w, x.im.w, x.gr.w, x.gi.w);
        }
        // the quad by itself
        const Cx d0{x.gr.x, x.gi.x}, d1{x.gr.y, x.gi.y}, d2{x.gr.z, x.gi.z}, d3{x.gr.w, x.gi.w};
        const Cx h3 = d3, h2 = cfma(mu, h3, d2), h1 = cfma(mu, h2, d1), h0 = cfma(mu, h1, d0);
        const Cx mu2 = cmul(mu, mu), mu3 = cmul(mu2, mu), mu4 = cmul(mu2, mu2);
        const bool open = active && !row_end;
        Cx A{open ? mu4.re : 0.0f, open ? mu4.im : 0.0f};
        Cx B{active ? h0.re : 0.0f, active ? h0.im : 0.0f};
        scan_affine_complex(A, B);
        if (sp.lane == kWave - 1) {
            L.Ar[parity][sp.wv] = A.re; L.Ai[parity][sp.wv] = A.im;
            L.Br[parity][sp.wv] = B.re; L.Bi[parity][sp.wv] = B.im;
        }
        __syncthreads();
        Cx carry{L.cr[parity], L.ci[parity]};
#pragma unroll
        for (int w = 0; w < kScanWaves - 1; ++w)
            if (w < sp.wv) carry = apply_affine_complex(Cx{L.Ar[parity][w], L.Ai[parity][w]}, carry, Cx{L.Br[parity][w], L.Bi[parity][w]});
        const Cx leaving = apply_affine_complex(A, carry, B);
        Cx ent{lane_below(leaving.re, carry.re), lane_below(leaving.im, carry.im)};
        if (row_end || !active) ent = Cx{0.0f, 0.0f};
        const Cx z3 = cfma(mu, ent, h3), z2 = cfma(mu2, ent, h2), z1 = cfma(mu3, ent, h1), z0 = cfma(mu4, ent, h0);
        if (SHIFT) {
            const int k = shift_tab.kout[cur.r];
            scan_store_shifted(dst_r, active, cur.r, cur.pos, k, T, make_float4(z0.re, z1.re, z2.re, z3.re));
            scan_store_shifted(dst_i, active, cur.r, cur.pos, k, T, make_float4(z0.im, z1.im, z2.im, z3.im));
        } else {
            const int off = active ? cur.lq * 16 : kOutOfRange;
            buf_store4<STREAM>(dst_r, off, make_float4(z0.re, z1.re, z2.re, z3.re));
            buf_store4<STREAM>(dst_i, off, make_float4(z0.im, z1.im, z2.im, z3.im));
        }
        if (sp.tid == kScanQuads - 1) { L.cr[parity ^ 1] = z0.re; L.ci[parity ^ 1] = z0.im; }
        if (PARTIAL) {
            // grad_sin: sum -gr[t+1] im[t] + gi[t+1] re[t];  grad_cos: sum gr[t+1] re[t] + gi[t+1] im[t]
            const float4 nr = make_float4(z1.re, z2.re, z3.re, ent.re), ni = make_float4(z1.im, z2.im, z3.im, ent.im);
            float ss = 0.0f, sc = 0.0f;
            ss = __fmaf_rn(ni.w, x.re.w, __fmaf_rn(-nr.w, x.im.w, ss)); sc = __fmaf_rn(ni.w, x.im.w, __fmaf_rn(nr.w, x.re.w, sc));
            ss = __fmaf_rn(ni.z, x.re.z, __fmaf_rn(-nr.z, x.im.z, ss)); sc = __fmaf_rn(ni.z, x.im.z, __fmaf_rn(nr.z, x.re.z, sc));
            ss = __fmaf_rn(ni.y, x.re.y, __fmaf_rn(-nr.y, x.im.y, ss)); sc = __fmaf_rn(ni.y, x.im.y, __fmaf_rn(nr.y, x.re.y, sc));
            ss = __fmaf_rn(ni.x, x.re.x, __fmaf_rn(-nr.x, x.im.x, ss)); sc = __fmaf_rn(ni.x, x.im.x, __fmaf_rn(nr.x, x.re.x, sc));
            add_to_row(sum_s[sp.wv], ss, sp, cur, QR, active);
            add_to_row(sum_c[sp.wv], sc, sp, cur, QR, active);
        }
        fetch_saved(x, cur.lq - NBUF * kScanQuads, ahead);
        if (SHIFT) { fetch_grad(x, ahead.lq, ahead); ahead.next(QR); }
        else fetch_grad(x, cur.lq - NBUF * kScanQuads, ahead);
        cur.next(QR);
        parity ^= 1;
    };
    static_assert(NBUF == 3 || NBUF == 4, "pass buffers");
    for (int left = sp.npass;;) {
        pass(b[0]); if (--left == 0) break;
        pass(b[1]); if (--left == 0) break;
        pass(b[2]); if (--left == 0) break;
        if (NBUF == 4) { pass(b[NBUF - 1]); if (--left == 0) break; }
    }
    if (PARTIAL || DELAY) __syncthreads();
    if (PARTIAL) {
        store_row_sums(partial_sin, sum_s, sp);
        store_row_sums(partial_cos, sum_c, sp);
    }
    if constexpr (DELAY) store_row_sums(shifts.delay_partial, sum_d, sp);
}

// Rows per workgroup: the fewest rows whose bytes are a whole number of 128-byte lines (so that no line is
// shared between two workgroups), repeated until the span is at least two passes long; at most kScanMaxRows.
inline int scan_rows_per_group(int64_t M, int64_t T) {
    int64_t unit = 32;                                   // rows * T must be a multiple of 32 floats
    for (int64_t t = T; (t & 1) == 0 && unit > 1; t >>= 1) unit >>= 1;
    if (unit > kScanMaxRows) unit = 1;
    int64_t r = unit;
    const int64_t want = 2 * kScanWaves * kWave * 4;     // floats in two passes
    while (r * T < want && r + unit <= kScanMaxRows) r += unit;
    if (r < 1) r = 1;
    if (r > kScanMaxRows) r = kScanMaxRows;
    if (r > M) r = M;
    return (int)r;
}

// Tensors of at least this many elements take the scan (smaller ones keep the sequential kernel, whose
// grad_in is bit-identical to a step-by-step evaluation).  SLAYER_BWD_SCAN_MIN overrides it (tuning).
int64_t bwd_scan_min_elements() {
    static const int64_t v = [] {
        const char* e = getenv("SLAYER_BWD_SCAN_MIN");
        return e ? (int64_t)atoll(e) : (int64_t)1 << 20;
    }();
    return v;
}

// True when the scan kernels can run a problem of this shape: spans addressable with 32 bits, 32-bit row
// arithmetic, large enough (the callers also check that every tensor is 16-byte aligned).  Rows that are not a
// whole number of quads take the any-length form of the kernels, from kScanAnyLengthMinSteps steps on (a short
// row is mostly its partial last quad).
constexpr int64_t kScanAnyLengthMinSteps = 64;
bool bwd_scan_usable(int64_t M, int64_t npb, int64_t T) {
    if (M <= 0 || T < 4 || T > (1 << 22) || M * T < bwd_scan_min_elements()) return false;
    if ((T % 4) != 0 && T < kScanAnyLengthMinSteps) return false;
    return npb > 0 && npb < ((int64_t)1 << 31);
}

struct ScanGrid { dim3 grid; int rpg, QR, passes; bool streaming, ok, any_length; };   // passes: of a full span
static ScanGrid scan_grid(int64_t M, int64_t T) {
    ScanGrid g;
    g.rpg = scan_rows_per_group(M, T);
    const int64_t blocks = (M + g.rpg - 1) / g.rpg;
    g.ok = blocks <= 0x7fffffffLL;
    g.grid = dim3((unsigned)blocks);
    g.QR = (int)((T + 3) / 4);
    g.any_length = (T % 4) != 0;
    g.passes = (int)(((int64_t)g.rpg * g.QR + kScanQuads - 1) / kScanQuads);
    g.streaming = stream_is_large(M, T);
    return g;
}
static unsigned rows_per_param(int64_t npb, int64_t n) { return (unsigned)(n > 1 ? npb / n : npb); }

int launch_li_bwd_scan(float* grad_in, float* partial, const float* grad_out, const float* out, const float* decay,
                       int64_t M, int64_t npb, int64_t num_decays, int64_t T, hipStream_t stream) {
    const ScanGrid g = scan_grid(M, T);
    if (!g.ok) return SLAYER_ERANGE;
#define SLAYER_SCAN(P, S, A)                                                                                     \
    hipLaunchKernelGGL((li_bwd_scan_kernel<P, S, A>), g.grid, dim3(kScanQuads), 0, stream, grad_in, partial,     \
                       grad_out, out, decay, M, (int)T, g.QR, g.rpg, (unsigned)npb, rows_per_param(npb, num_decays))
    if (g.any_length) { if (partial) SLAYER_SCAN(true, false, true); else SLAYER_SCAN(false, false, true); }
    else if (partial) { if (g.streaming) SLAYER_SCAN(true, true, false); else SLAYER_SCAN(true, false, false); }
    else { if (g.streaming) SLAYER_SCAN(false, true, false); else SLAYER_SCAN(false, false, false); }
#undef SLAYER_SCAN
    return (int)hipGetLastError();
}

// theta == nullptr: CUBA (scalar spike threshold); else ALIF.  partial_i / partial_v both or neither.
// shifts: the backward pass's Shifts when axonal delays are folded in (the gradient of the spikes is read back
// through the output delay, the input gradient stored back through the input shift), else nullptr.
int launch_cuba_bwd_scan(float* grad_in, float* partial_i, float* partial_v, const float* grad_spikes,
                         const float* voltage, const float* theta, const float* current, const float* i_decay,
                         const float* v_decay, float spike_thr, float tau, float rho, bool graded,
                         int64_t M, int64_t npb, int64_t n_id, int64_t n_vd, int64_t T, const Shifts* shifts,
                         hipStream_t stream) {
    const ScanGrid g = scan_grid(M, T);
    if (!g.ok) return SLAYER_ERANGE;
    const Shifts sh = shifts ? *shifts : Shifts{nullptr, nullptr, nullptr, nullptr, 0, 0, 1, 1.0f, 1};
#define SLAYER_SCAN_L(G, D, TH, S, SH, NB, DL)                                                                   \
    hipLaunchKernelGGL((cuba_bwd_scan_kernel<G, D, TH, S, SH, NB, DL>), g.grid, dim3(kScanQuads), 0, stream, grad_in, \
                       partial_i, partial_v, grad_spikes, voltage, theta, current, i_decay, v_decay, spike_thr,  \
                       tau, rho, M, (int)T, g.QR, g.rpg, (unsigned)npb, rows_per_param(npb, n_id),               \
                       rows_per_param(npb, n_vd), sh)
#define SLAYER_SCAN_N(G, D, TH, S, SH, NB) do { if (SH != 0 && delay_grad) SLAYER_SCAN_L(G, D, TH, S, SH, NB, (SH != 0)); else SLAYER_SCAN_L(G, D, TH, S, SH, NB, false); } while (0)
#define SLAYER_SCAN(G, D, TH, S, SH) do { if (g.passes > 3) SLAYER_SCAN_N(G, D, TH, S, SH, 4); else SLAYER_SCAN_N(G, D, TH, S, SH, 3); } while (0)
#define SLAYER_SCAN_H(G, D, TH, S) do { if (shifts) SLAYER_SCAN(G, D, TH, S, 1); else SLAYER_SCAN(G, D, TH, S, 0); } while (0)
#define SLAYER_SCAN_S(G, D, TH) do { if (g.any_length) SLAYER_SCAN(G, D, TH, false, 2); else if (g.streaming) SLAYER_SCAN_H(G, D, TH, true); else SLAYER_SCAN_H(G, D, TH, false); } while (0)
#define SLAYER_SCAN_T(G, D) do { if (theta) SLAYER_SCAN_S(G, D, true); else SLAYER_SCAN_S(G, D, false); } while (0)
    const bool want = partial_i != nullptr;
    const bool delay_grad = shifts && sh.delayed && sh.delay_partial;
    if (graded) { if (want) SLAYER_SCAN_T(true, true); else SLAYER_SCAN_T(true, false); }
    else { if (want) SLAYER_SCAN_T(false, true); else SLAYER_SCAN_T(false, false); }
#undef SLAYER_SCAN_T
#undef SLAYER_SCAN_S
#undef SLAYER_SCAN_H
#undef SLAYER_SCAN
#undef SLAYER_SCAN_N
#undef SLAYER_SCAN_L
    return (int)hipGetLastError();
}

// surrogate: 0 = g_re / g_im are the gradients of the states; 1 / 2 = g_re is the gradient of binary / graded
// spikes (g_im unused) and spike_thr, tau, rho parametrise the complex spike surrogate.
int launch_res_bwd_scan(float* g_re_in, float* g_im_in, float* partial_sin, float* partial_cos, const float* g_re,
                        const float* g_im, const float* re, const float* im, const float* sin_decay,
                        const float* cos_decay, int surrogate, float spike_thr, float tau, float rho, int64_t M,
                        int64_t npb, int64_t num_decays, int64_t T, const Shifts* shifts, hipStream_t stream) {
    const ScanGrid g = scan_grid(M, T);
    if (!g.ok) return SLAYER_ERANGE;
    if (shifts && surrogate == 0) return SLAYER_EINVAL;      // delays belong to the fused resonate-and-fire form
    const SpikeSurrogate k{spike_thr, tau, rho};
    const Shifts sh = shifts ? *shifts : Shifts{nullptr, nullptr, nullptr, nullptr, 0, 0, 1, 1.0f, 1};
    const bool delay_grad = shifts && surrogate != 0 && sh.delayed && sh.delay_partial;
#define SLAYER_SCAN_L(P, S, U, SH, NB, DL)                                                                       \
    hipLaunchKernelGGL((res_bwd_scan_kernel<P, S, U, SH, NB, DL>), g.grid, dim3(kScanQuads), 0, stream, g_re_in, g_im_in, \
                       partial_sin, partial_cos, g_re, g_im, re, im, sin_decay, cos_decay, k, M, (int)T, g.QR,   \
                       g.rpg,                                                                                    \
                       (unsigned)npb, rows_per_param(npb, num_decays), sh)
#define SLAYER_SCAN_N(P, S, U, SH, NB) do { if (SH != 0 && U != 0 && delay_grad) SLAYER_SCAN_L(P, S, U, SH, NB, (SH != 0 && U != 0)); else SLAYER_SCAN_L(P, S, U, SH, NB, false); } while (0)
#define SLAYER_SCAN(P, S, U, SH) do { if (g.passes > 3) SLAYER_SCAN_N(P, S, U, SH, 4); else SLAYER_SCAN_N(P, S, U, SH, 3); } while (0)
#define SLAYER_SCAN_S(P, U, SH) do { if (g.any_length) SLAYER_SCAN(P, false, U, 2); else if (g.streaming) SLAYER_SCAN(P, true, U, SH); else SLAYER_SCAN(P, false, U, SH); } while (0)
#define SLAYER_SCAN_P(U, SH) do { if (partial_sin) SLAYER_SCAN_S(true, U, SH); else SLAYER_SCAN_S(false, U, SH); } while (0)
    if (surrogate == 0) SLAYER_SCAN_P(0, 0);
    else if (surrogate == 1) { if (shifts) SLAYER_SCAN_P(1, 1); else SLAYER_SCAN_P(1, 0); }
    else { if (shifts) SLAYER_SCAN_P(2, 1); else SLAYER_SCAN_P(2, 0); }
#undef SLAYER_SCAN_P
#undef SLAYER_SCAN_S
#undef SLAYER_SCAN
#undef SLAYER_SCAN_N
#undef SLAYER_SCAN_L
    return (int)hipGetLastError();
}

}  // namespace slayer
