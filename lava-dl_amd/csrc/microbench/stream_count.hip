// What the memory system gives an elementwise kernel as a function of the number of tensors it reads and writes.
//
// One quad (16 bytes) per lane and tensor, 1024 samples per workgroup, non-temporal accesses: the shape of the spike
// kernels (spike.hip) and, tensor count for tensor count, of the scan kernels (scan.hip).  The kernel adds its NR inputs
// and writes the sum to each of its NW outputs; MATH > 0 adds that many exp + division pairs per sample (the cost
// of a spike surrogate).  Tensors are 131 072 000 floats, the size of a [64,1024,2000] tensor.
// Usage: stream_count [stagger=0]   (stagger: bytes by which the base addresses of consecutive tensors are offset
// beyond what hipMalloc returns).  Prints microseconds per launch and GB/s on (NR + NW) * 524 MB.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef float vf4 __attribute__((ext_vector_type(4)));

template <int NR, int NW, int MATH>
__global__ __launch_bounds__(256) void k(float* const* __restrict__ out, const float* const* __restrict__ in, size_t nq) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nq) return;
    vf4 v[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) v[r] = __builtin_nontemporal_load((const vf4*)in[r] + i);
    vf4 acc = v[0];
#pragma unroll
    for (int r = 1; r < NR; ++r) acc += v[r];
#pragma unroll
    for (int m = 0; m < MATH; ++m) {
        acc.x = expf(-fabsf(acc.x)) / 1.5f; acc.y = expf(-fabsf(acc.y)) / 1.5f;
        acc.z = expf(-fabsf(acc.z)) / 1.5f; acc.w = expf(-fabsf(acc.w)) / 1.5f;
    }
#pragma unroll
    for (int w = 0; w < NW; ++w) __builtin_nontemporal_store(acc + (float)w, (vf4*)out[w] + i);
}

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)

int main(int argc, char** argv) {
    const size_t n = 131072000;
    const size_t bytes = n * 4;
    const size_t off = argc > 1 ? (size_t)atol(argv[1]) : 0;
    if (off % 16 != 0 || off > ((size_t)16 << 20)) { printf("stagger: a multiple of 16, at most 16 MB\n"); return 2; }
    float* buf[8];
    for (int i = 0; i < 8; ++i) {
        char* p;
        CHECK(hipMalloc(&p, bytes + 8 * off + 256));
        CHECK(hipMemset(p, 0, bytes + 8 * off));
        buf[i] = (float*)(p + i * off);
    }
    float **din, **dout;
    CHECK(hipMalloc(&din, 64)); CHECK(hipMalloc(&dout, 64));
    CHECK(hipMemcpy(din, buf, 4 * sizeof(float*), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(dout, buf + 4, 4 * sizeof(float*), hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    printf("stagger %zu bytes\n", off);
    auto run = [&](const char* name, int nr, int nw, auto launch) {
        for (int w = 0; w < 2; ++w) launch();
        if (hipDeviceSynchronize() != hipSuccess) { printf("%s failed\n", name); exit(1); }
        (void)hipEventRecord(e0);
        for (int r = 0; r < 10; ++r) launch();
        (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
        float ms = 0; (void)hipEventElapsedTime(&ms, e0, e1); ms /= 10;
        printf("%-28s %8.1f us %7.0f GB/s\n", name, ms * 1e3, (double)(nr + nw) * bytes / ms / 1e6); fflush(stdout);
    };
    const size_t nq = n / 4;
    const unsigned grid = (unsigned)((nq + 255) / 256);
#define RUN(NR, NW, MATH) run(#NR " read, " #NW " written, math " #MATH, NR, NW, [&] { \
        hipLaunchKernelGGL((k<NR, NW, MATH>), dim3(grid), dim3(256), 0, 0, dout, (const float* const*)din, nq); });
    RUN(1, 1, 0) RUN(2, 1, 0) RUN(2, 1, 1) RUN(3, 1, 0) RUN(3, 2, 0) RUN(3, 2, 2) RUN(4, 2, 0) RUN(4, 2, 2) RUN(4, 4, 0)
    return 0;
}
