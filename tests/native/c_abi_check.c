/* The C ABI from plain C: device buffers from hipMalloc, one call of slayer_li_fwd and one of
 * slayer_spike_fwd on a stream, results compared with a scalar restatement of the leaky integrator
 * (neuron/dynamics/leaky_integrator.py:210-231 of the reference: state and input scaled by w and truncated,
 * product with 4096 - decay shifted right by 12 bits toward zero, reset when the state reaches the threshold).
 * Built by __graft_entry__.build(); run by tests/test_gpu_c_abi.py.  Prints "c abi ok" on success. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include "slayer_hip.h"

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
    fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)

static int64_t shift12_toward_zero(int64_t p) { return p >= 0 ? (p >> 12) : -((-p) >> 12); }

int main(void) {
    enum { N = 3, C = 5, T = 44, M = N * C, W = 64 };
    const float threshold = 1.25f;
    float *in = malloc(sizeof(float) * M * T), *out = malloc(sizeof(float) * M * T), *spk = malloc(sizeof(float) * M * T);
    float decay[C], state = 0.25f;
    unsigned s = 12345u;
    for (int i = 0; i < M * T; ++i) {
        s = s * 1664525u + 1013904223u;
        in[i] = (s >> 28) == 0 ? 0.0f : (float)((int)((s >> 8) & 0xff) - 100) / 64.0f * ((s >> 27) & 1);
    }
    for (int c = 0; c < C; ++c) decay[c] = (float)(c * 900);

    float *d_in, *d_out, *d_spk, *d_decay, *d_state;
    CHECK(hipMalloc((void**)&d_in, sizeof(float) * M * T));
    CHECK(hipMalloc((void**)&d_out, sizeof(float) * M * T));
    CHECK(hipMalloc((void**)&d_spk, sizeof(float) * M * T));
    CHECK(hipMalloc((void**)&d_decay, sizeof(decay)));
    CHECK(hipMalloc((void**)&d_state, sizeof(float)));
    hipStream_t stream;
    CHECK(hipStreamCreate(&stream));
    CHECK(hipMemcpyAsync(d_in, in, sizeof(float) * M * T, hipMemcpyHostToDevice, stream));
    CHECK(hipMemcpyAsync(d_decay, decay, sizeof(decay), hipMemcpyHostToDevice, stream));
    CHECK(hipMemcpyAsync(d_state, &state, sizeof(float), hipMemcpyHostToDevice, stream));

    if (slayer_abi_version() != SLAYER_ABI_VERSION) { fprintf(stderr, "unexpected ABI version\n"); return 1; }
    int rc = slayer_li_fwd(d_out, d_in, d_decay, d_state, (double)threshold * W, W, M, C, C, 1, T, (void*)stream);
    if (rc) { fprintf(stderr, "slayer_li_fwd: %s\n", slayer_error_string(rc)); return 1; }
    rc = slayer_spike_fwd(d_spk, d_out, NULL, 0, threshold, 0, 1.0f, (int64_t)M * T, (void*)stream);
    if (rc) { fprintf(stderr, "slayer_spike_fwd: %s\n", slayer_error_string(rc)); return 1; }
    CHECK(hipMemcpyAsync(out, d_out, sizeof(float) * M * T, hipMemcpyDeviceToHost, stream));
    CHECK(hipMemcpyAsync(spk, d_spk, sizeof(float) * M * T, hipMemcpyDeviceToHost, stream));
    CHECK(hipStreamSynchronize(stream));

    int bad = 0, spikes = 0;
    for (int m = 0; m < M; ++m) {
        const int64_t mult = 4096 - (int64_t)decay[m % C];
        int64_t y = (int64_t)(state * W);
        for (int t = 0; t < T; ++t) {
            y = shift12_toward_zero(y * mult) + (int64_t)((float)W * in[m * T + t]);
            const float v = (float)y / (float)W;
            if (out[m * T + t] != v) ++bad;
            const float fired = v >= threshold ? 1.0f : 0.0f;
            if (spk[m * T + t] != fired) ++bad;
            spikes += fired != 0.0f;
            if ((float)y >= threshold * (float)W) y = 0;
        }
    }
    /* this workload stays far below 2^30: the range flag is down after the launches have completed */
    int raised = -1;
    rc = slayer_range_status(&raised, 0);
    if (rc != 0 || raised != 0 || slayer_range_word() == NULL) {
        fprintf(stderr, "range flag: status %d (%s), raised %d, word %p\n", rc, slayer_error_string(rc), raised,
                (const void*)slayer_range_word());
        ++bad;
    }
    /* an argument error comes back as a code, nothing is launched */
    if (slayer_li_fwd(d_out, d_in, d_decay, d_state, 1.0, W, M, 4, C, 1, T, (void*)stream) != SLAYER_EINVAL) ++bad;
    hipFree(d_in); hipFree(d_out); hipFree(d_spk); hipFree(d_decay); hipFree(d_state);
    hipStreamDestroy(stream);
    if (bad || spikes == 0) { fprintf(stderr, "%d mismatches, %d spikes\n", bad, spikes); return 1; }
    printf("c abi ok: %d samples, %d spikes\n", M * T, spikes);
    return 0;
}
