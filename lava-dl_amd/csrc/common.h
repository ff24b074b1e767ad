// Host-side argument checks shared by the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/slayer_hip.h"

namespace slayer {

constexpr int64_t kMaxT = (int64_t)1 << 30;
constexpr int64_t kMaxNumel = (int64_t)1 << 40;

inline int check_rows(int64_t M, int64_t T) {
    if (M < 0 || T < 0) return SLAYER_EINVAL;
    if (T > kMaxT || (T > 0 && M > kMaxNumel / T)) return SLAYER_ERANGE;
    if ((M + 63) / 64 > 0x7fffffffLL) return SLAYER_ERANGE;
    return 0;
}

// M rows split into batches of npb rows; a parameter vector of n entries maps onto one batch.
inline int check_params(int64_t M, int64_t npb, int64_t n) {
    if (npb <= 0 || M % npb != 0) return SLAYER_EINVAL;
    if (n < 1 || (n > 1 && npb % n != 0)) return SLAYER_EINVAL;
    return 0;
}

inline int check_states(int64_t M, int64_t n) { return (n == 1 || n == M) ? 0 : SLAYER_EINVAL; }

inline bool is_pow2(int w) { return w > 0 && (w & (w - 1)) == 0; }

// The process-wide range flag of the 32-bit fixed-point states (api.hip): one word of pinned host memory that the
// kernels can write.  range_flag_device() is the address a kernel stores to (nullptr when the word could not be
// set up: the kernels then skip the report); range_flag_raise_from_host() sets it from an entry point, for scaled
// arguments that are already beyond what a state may hold.
unsigned* range_flag_device();
void range_flag_raise_from_host();
// threshold step and base of the adaptive-threshold family: both enter the states, whose bound is 2^28
inline unsigned* range_flag_for_threshold(int64_t step_scaled, int64_t base_scaled) {
    unsigned* flag = range_flag_device();
    const int64_t lim = (int64_t)1 << 28;
    if (step_scaled >= lim || step_scaled <= -lim || base_scaled >= lim || base_scaled <= -lim)
        range_flag_raise_from_host();
    return flag;
}

// Delays folded into a fused block: per-neuron tables need a batch to map onto and a sampling time to
// divide by; the scalar parts must fit the 32-bit step counts of the kernels (a shift of T steps already
// empties a row, so anything beyond +-2^30 is equivalent to it).
inline int check_delays(const slayer_delays* d, int64_t M, int64_t npb) {
    if (!d) return 0;
    if (npb <= 0 || (M > 0 && M % npb != 0)) return SLAYER_EINVAL;
    if ((d->in_shift || d->out_delay) && !(d->sampling_time != 0.0f)) return SLAYER_EINVAL;
    // the delay gradient of a backward pass: all three of its pointers or none, and a sampling time to divide by
    const int given = (d->delayed_spikes != nullptr) + (d->grad_out_delay != nullptr) + (d->grad_workspace != nullptr);
    if (given != 0 && given != 3) return SLAYER_ENULL;
    if (given == 3 && !(d->sampling_time != 0.0f)) return SLAYER_EINVAL;
    return 0;
}

// After the main kernel of a fused backward pass: the gradient of the output delay, when the caller asked for it.
// in_scan: the backward scan has left the per-row sums in grad_workspace; else nothing has been summed yet and the
// stand-alone kernel does the whole job.  (li.hip, shift.hip)
int launch_reduce_param_grad(float* grad, const float* partial, float* scratch, int64_t M, int64_t npb,
                             int64_t num_params, hipStream_t stream);
int launch_zero_fill(float* p, int64_t n, hipStream_t stream);
inline int finish_delay_gradient(const slayer_delays* d, const float* grad_spikes, bool in_scan, int64_t M, int64_t npb,
                                 int64_t T, hipStream_t stream) {
    if (!d || !d->grad_out_delay) return 0;
    if (M == 0 || T == 0) return launch_zero_fill(d->grad_out_delay, npb, stream);
    if (in_scan)
        return launch_reduce_param_grad(d->grad_out_delay, d->grad_workspace, d->grad_workspace + M, M, npb, npb, stream);
    return slayer_delay_bwd(nullptr, d->grad_out_delay, grad_spikes, d->delayed_spikes, nullptr, 0, d->sampling_time,
                            d->grad_workspace, M, npb, T, (void*)stream);
}

}  // namespace slayer
