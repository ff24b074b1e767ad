// Leaky integrator: forward fixed-point recurrence and reverse-time gradient.
#include "common.h"
#include "tile.h"
#include <mutex>

namespace slayer {

// ---------------------------------------------------------------------------------- forward
// RESET = false: no threshold was given, the reset decision is left out of the step (a third of its
// instructions: what a step costs is what bounds the kernel while few neurons keep the chip busy).
template <bool POW2, bool RESET = true>
struct LiFwd {
    static constexpr int kIn = 1, kOut = 1;
    static constexpr bool kReverse = false;
    static constexpr int64_t kRows32Below = 32768, kRows16Below = 8192;
    static constexpr bool kLongPiecesOnAliasedRows = true;
    static constexpr bool kMultiwaveWhenLarge = true;
    struct Params {
        const float* in[1];
        float* out[1];
        const float* decay;
        const float* state;
        float w, inv_w;
        int fire_above;               // reset when the state exceeds this (INT_MAX: reset disabled)
        int64_t npb, num_decays, num_states;
        unsigned* range_flag;         // raised when a state comes within a factor of two of the 32-bit limit
    };
    static constexpr bool kRangeChecked = true;
    static constexpr int range_log2(int) { return 30; }
    // The tiles hold integers (bit patterns in float registers): the input is scaled and truncated
    // on its way into LDS, the state is converted and scaled back on its way out, and the
    // sequential loop is left with the recurrence alone.
    static constexpr bool kTransforms = true;
    static constexpr int kCopyWaves = 2;
    int y, mult, fire_above;
    float w, inv_w;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        w = p.w; inv_w = p.inv_w; fire_above = p.fire_above;
        y = 0; mult = 0;
        if (valid) {
            y = trunc_i32(p.state[p.num_states == 1 ? 0 : m] * w);
            mult = 4096 - trunc_i32(p.decay[param_index(m, p.npb, p.num_decays)]);
            check_multiplier(mult, p.range_flag);
            check_state(y, 30, p.range_flag);
        }
    }
    __device__ __forceinline__ void pre(float4 (&x)[1]) const { x[0] = to_state(x[0], w); }
    __device__ __forceinline__ void post(float4 (&o)[1]) const { o[0] = from_state<POW2>(o[0], w, inv_w); }
    __device__ __forceinline__ void step(const float (&x)[1], float (&o)[1]) {
        const int yn = add_sat(rs0_12(y, mult), __float_as_int(x[0]));
        o[0] = __int_as_float(yn);
        y = (RESET && yn > fire_above) ? 0 : yn;     // (float)yn >= threshold, decided on the integer
    }
    __device__ __forceinline__ void finish(const Params&, int64_t, bool) {}
};

// --------------------------------------------------------------------------------- backward
struct LiBwd {
    static constexpr int kIn = 2, kOut = 1;     // in: grad_out, saved forward output
    static constexpr bool kReverse = true;
    static constexpr int kDuoRows = 32;          // light float recurrence: shorter rows per wave, longer segments
    static constexpr int kCopyWaves = 2;         // 360 -> 240 us on 262 144 unaligned rows of 301 steps; small tensors alike
    static constexpr int64_t kRows32Below = kAlways, kRows16Below = kAlways;
    struct Params {
        const float* in[2];
        float* out[1];
        const float* decay;
        float* partial;               // per-neuron sum_t g[t+1] * out[t], or nullptr
        int64_t npb, num_decays;
    };
    float a, g, acc;

    __device__ __forceinline__ void init(const Params& p, int64_t m, bool valid) {
        g = 0.f; acc = 0.f; a = 0.f;
        if (valid) a = 1.0f - p.decay[param_index(m, p.npb, p.num_decays)] / 4096.0f;
    }
    __device__ __forceinline__ void step(const float (&x)[2], float (&o)[1]) {
        acc = __fmaf_rn(g, x[1], acc);          // g still holds grad_in[t+1]
        g = a * g + x[0];                       // separate multiply and add, as torch evaluates it
        o[0] = g;
    }
    __device__ __forceinline__ void finish(const Params& p, int64_t m, bool valid) {
        if (valid && p.partial) p.partial[m] = acc;
    }
};

// Parameter-gradient reduction: grad[j] = sum of partial[m] over all rows m whose parameter
// index is j.  Two deterministic passes: (j, s) workgroups each sum one slice in double and
// write one float to scratch[j * split + s]; then one lane per parameter adds its `split`
// slice sums in double.  `scratch` is the tail of the caller's workspace.
constexpr int kRedBlock = 256;
constexpr int kRedMaxSplit = 64;

// (blockIdx.z = 1: the second gradient of a pair -- its partial sums follow the first's M, its slice sums the
// first's num_params * kRedMaxSplit)
__global__ __launch_bounds__(kRedBlock) void reduce_param_slices(float* scratch, const float* partial,
                                                                 int64_t M, int64_t npb, int64_t num_params,
                                                                 int split) {
    const int64_t j = blockIdx.x;
    const int s = blockIdx.y;
    partial += (int64_t)blockIdx.z * M;
    scratch += (int64_t)blockIdx.z * num_params * kRedMaxSplit;
    const int64_t block = num_params > 1 ? npb / num_params : npb;   // rows per batch element for parameter j
    const int64_t total = (M / npb) * block;
    const int64_t per = (total + split - 1) / split;
    const int64_t lo = s * per, hi = (lo + per) < total ? (lo + per) : total;
    double acc = 0.0;
    for (int64_t i = lo + threadIdx.x; i < hi; i += kRedBlock) {
        const int64_t n = i / block, b = i - n * block;
        acc += (double)partial[n * npb + j * block + b];
    }
    __shared__ double red[kRedBlock];
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int w = kRedBlock / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) scratch[j * split + s] = (float)red[0];
}

__global__ __launch_bounds__(kRedBlock) void reduce_param_final(float* grad, float* grad_second, const float* scratch,
                                                                int64_t num_params, int split) {
    const int64_t j = (int64_t)blockIdx.x * kRedBlock + threadIdx.x;
    if (j >= num_params) return;
    if (blockIdx.z) { grad = grad_second; scratch += num_params * kRedMaxSplit; }
    double acc = 0.0;
    for (int s = 0; s < split; ++s) acc += (double)scratch[j * split + s];
    grad[j] = (float)acc;
}

__global__ void zero_fill(float* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = 0.0f;
}

// Clears n floats with a kernel (a memset node would not replay reliably inside a captured graph).
int launch_zero_fill(float* p, int64_t n, hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(zero_fill, dim3(1), dim3(256), 0, stream, p, n);
    return (int)hipGetLastError();
}

// Slices per parameter: enough that a slice is a few thousand rows, at most kRedMaxSplit.
int param_grad_split(int64_t M, int64_t npb, int64_t num_params) {
    const int64_t block = num_params > 1 ? npb / num_params : npb;
    const int64_t total = (M / npb) * block;
    int64_t split = total / 2048;
    if (split < 1) split = 1;
    if (split > kRedMaxSplit) split = kRedMaxSplit;
    return (int)split;
}

// scratch needs num_params * kRedMaxSplit floats.
int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream) {
    const int split = param_grad_split(M, npb, num_params);
    hipLaunchKernelGGL(reduce_param_slices, dim3((unsigned)num_params, (unsigned)split), dim3(kRedBlock), 0, stream,
                       scratch, partial, M, npb, num_params, split);
    if (int e = (int)hipGetLastError()) return e;
    hipLaunchKernelGGL(reduce_param_final, dim3((unsigned)((num_params + kRedBlock - 1) / kRedBlock)),
                       dim3(kRedBlock), 0, stream, grad, (float*)nullptr, scratch, num_params, split);
    return (int)hipGetLastError();
}

// Two gradients of one backward pass (both decays of a CUBA or ALIF neuron, sine and cosine of a resonator): their
// partial sums lie one after the other (M floats each), their slice sums likewise (kRedMaxSplit per parameter).
// With as many parameters each, the two reductions share their two launches.
int launch_reduce_param_grad_pair(float* grad_a, float* grad_b, const float* partial, float* scratch, int64_t M,
                                  int64_t npb, int64_t num_a, int64_t num_b, hipStream_t stream) {
    if (num_a != num_b) {
        if (int e = launch_reduce_param_grad(grad_a, partial, scratch, M, npb, num_a, stream)) return e;
        return launch_reduce_param_grad(grad_b, partial + M, scratch + kRedMaxSplit * num_a, M, npb, num_b, stream);
    }
    const int split = param_grad_split(M, npb, num_a);
    hipLaunchKernelGGL(reduce_param_slices, dim3((unsigned)num_a, (unsigned)split, 2), dim3(kRedBlock), 0, stream,
                       scratch, partial, M, npb, num_a, split);
    if (int e = (int)hipGetLastError()) return e;
    hipLaunchKernelGGL(reduce_param_final, dim3((unsigned)((num_a + kRedBlock - 1) / kRedBlock), 1, 2),
                       dim3(kRedBlock), 0, stream, grad_a, grad_b, scratch, num_a, split);
    return (int)hipGetLastError();
}

// Scratch of the entry point that allocates nothing (slayer_li_bwd_static): per-neuron partial sums for
// up to kStaticMaxRows neurons followed by kRedMaxSplit slice sums for each of up to kStaticMaxDecays
// decays.  5 MiB of device memory on every GPU the library runs on, held until the process ends.
constexpr int64_t kStaticMaxRows = SLAYER_LI_BWD_STATIC_MAX_ROWS;
constexpr int64_t kStaticMaxDecays = SLAYER_LI_BWD_STATIC_MAX_DECAYS;
static __device__ __align__(256) float scratch[kStaticMaxRows + kRedMaxSplit * kStaticMaxDecays];

// Device address of `scratch` on the current device (in host code the array's name is only a
// stand-in for the symbol, not an address a kernel could use).  Every GPU holds its own copy, so the
// address is looked up once per device, with that device current.
static int static_scratch(float** out) {
    constexpr int kMaxDevices = 64;
    static float* ptrs[kMaxDevices] = {nullptr};
    static std::mutex lock;
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return SLAYER_ERANGE;
    std::lock_guard<std::mutex> guard(lock);
    if (!ptrs[dev]) {
        float* p = nullptr;
        if (hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch))) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return 0;
}

bool bwd_scan_usable(int64_t M, int64_t npb, int64_t T);   // scan.hip
int launch_li_bwd_scan(float* grad_in, float* partial, const float* grad_out, const float* out, const float* decay,
                       int64_t M, int64_t npb, int64_t num_decays, int64_t T, hipStream_t stream);              // scan.hip

}  // namespace slayer

using namespace slayer;

extern "C" int slayer_li_fwd(float* out, const float* in, const float* decay, const float* state,
                             double thr_scaled, int w_scale,
                             int64_t M, int64_t neurons_per_batch, int64_t num_decays, int64_t num_states,
                             int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (M == 0 || T == 0) return 0;
    if (!out || !in || !decay || !state) return SLAYER_ENULL;
    if (int e = check_params(M, neurons_per_batch, num_decays)) return e;
    if (int e = check_states(M, num_states)) return e;
    if (w_scale == 0) return SLAYER_EINVAL;
    const float w = (float)w_scale;
    const int fa = fire_above(thr_scaled > 0 ? (float)thr_scaled : __builtin_inff());
#define SLAYER_LI_FWD(P, R)                                                                                       \
    do {                                                                                                          \
        LiFwd<P, R>::Params p{{in}, {out}, decay, state, w, 1.0f / w, fa, neurons_per_batch, num_decays, num_states, \
                              range_flag_device()};                                                               \
        return launch_stream<LiFwd<P, R>>(p, M, T, (hipStream_t)stream);                                          \
    } while (0)
    const bool reset = thr_scaled > 0;
    if (is_pow2(w_scale)) { if (reset) SLAYER_LI_FWD(true, true); else SLAYER_LI_FWD(true, false); }
    if (reset) SLAYER_LI_FWD(false, true);
    SLAYER_LI_FWD(false, false);
#undef SLAYER_LI_FWD
}

extern "C" int slayer_li_bwd(float* grad_in, float* grad_decay, const float* grad_out, const float* out,
                             const float* decay, float* workspace,
                             int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                             int64_t T, void* stream) {
    if (int e = check_rows(M, T)) return e;
    if (int e = check_params(M > 0 ? M : neurons_per_batch, neurons_per_batch, num_decays)) return e;
    if (grad_decay && !workspace && M > 0) return SLAYER_ENULL;
    if (M > 0 && T > 0) {
        if (!grad_in || !grad_out || !out || !decay) return SLAYER_ENULL;
        if (bwd_scan_usable(M, neurons_per_batch, T) && aligned16(grad_in) && aligned16(grad_out) && aligned16(out)) {
            if (int e = launch_li_bwd_scan(grad_in, workspace, grad_out, out, decay, M,
                                           neurons_per_batch, num_decays, T, (hipStream_t)stream))
                return e;
        } else {
            LiBwd::Params p{{grad_out, out}, {grad_in}, decay, workspace,
                            neurons_per_batch, num_decays};
            if (int e = launch_stream<LiBwd>(p, M, T, (hipStream_t)stream)) return e;
        }
    }
    if (grad_decay) {
        if (M == 0 || T == 0) return launch_zero_fill(grad_decay, num_decays, (hipStream_t)stream);
        return launch_reduce_param_grad(grad_decay, workspace, workspace + M, M, neurons_per_batch, num_decays,
                                        (hipStream_t)stream);
    }
    return 0;
}

extern "C" int slayer_li_bwd_static(float* grad_in, float* grad_decay, const float* grad_out, const float* out,
                                    const float* decay, int64_t M, int64_t neurons_per_batch, int64_t num_decays,
                                    int64_t T, void* stream) {
    if (M > kStaticMaxRows || num_decays > kStaticMaxDecays) return SLAYER_ESCRATCH;
    float* ws = nullptr;
    if (grad_decay && M > 0)
        if (int e = static_scratch(&ws)) return e;
    // Nothing in the scratch has to start at zero: the streaming kernel writes the partial sum of every
    // row before the reduction reads it, and the reduction writes every slice sum before it adds them.
    return slayer_li_bwd(grad_in, grad_decay, grad_out, out, decay, ws, M, neurons_per_batch, num_decays, T, stream);
}
