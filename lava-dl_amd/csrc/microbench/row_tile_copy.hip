// What the memory system gives the access pattern of the streaming engine, with nothing else in the way.
//
// The sequential-in-time kernels (tile.h) give a wave R rows and let it walk time in chunks of TC samples: every
// chunk is R pieces of 4*TC bytes, one per row, a whole row (4*T bytes) apart.  This program copies a [M][T] float
// tensor in exactly that order, with no recurrence and no transposition, and compares
//   lin   : a plain linear copy (one dwordx4 per lane, 4 per thread);
//   reg   : row tiles staged through registers, the next chunk's loads issued before the current chunk's stores
//           (what the engine does);
//   lds   : row tiles loaded straight into LDS (global_load_lds_dwordx4, no staging registers), NBUF tiles per
//           wave so that NBUF-1 chunks are in flight, read back with ds_read_b128 and stored.
//   deep  : `reg` with D chunks of loads in flight per wave and the waves per compute unit held down with unused
//           dynamic LDS: fewer waves with more loads each keep the same bytes in flight on fewer rows (the rows
//           the chip works on at one time are the "front" of the copy);
//   xcd   : `reg` with the workgroups renumbered so that each of the eight XCDs (workgroup index modulo 8) walks a
//           contiguous eighth of the tensor instead of every eighth row block.
// Usage: row_tile_copy [T=384] [timed launches=20] [few|front]     (T a multiple of 128; "few": four patterns only,
// for counter passes; "front": the deep / xcd variants only).  Prints microseconds per copy and GB/s on
// 2 * M * T * 4 bytes.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

typedef float vf4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) float lds_float;
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <int R, int TC, int NBUF>
__global__ __launch_bounds__(64) void lds_copy(float* __restrict__ out, const float* __restrict__ in, int T) {
    constexpr int Q = TC / 4;             // lanes per row piece
    constexpr int RPI = 64 / Q;           // rows per wave-wide instruction
    constexpr int NI = R / RPI;           // instructions per chunk
    // loads and stores leave the counter in issue order: when chunk c is needed, NBUF-1 later chunks of loads and
    // as many chunks of stores may still be outstanding (the counter holds 63 at most)
    constexpr int AHEAD = 2 * (NBUF - 1) * NI > 63 ? 63 : 2 * (NBUF - 1) * NI;
    extern __shared__ __attribute__((aligned(16))) float tiles[];
    lds_float* lt = (lds_float*)tiles;
    const int lane = threadIdx.x;
    const int crow = lane / Q, cq = lane % Q;
    const long m0 = (long)blockIdx.x * R;
    const int nch = T / TC;
    auto issue = [&](int c) {
        lds_float* buf = lt + (c % NBUF) * (R * TC);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const float* g = in + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq;
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(g), buf + i * 256, 16, 0, 0);   // lane l lands at buf + 4*l floats
        }
    };
#pragma unroll
    for (int c = 0; c < NBUF - 1; ++c)
        if (c < nch) issue(c);
    for (int c = 0; c < nch; ++c) {
        if (c + NBUF - 1 < nch) { issue(c + NBUF - 1); wait_vm<AHEAD>(); }
        else wait_vm<0>();
        const unsigned lbase = (unsigned)(size_t)(lt + (c % NBUF) * (R * TC)) + lane * 16;
        vf4 v[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) asm volatile("ds_read_b128 %0, %1" : "=v"(v[i]) : "v"(lbase + i * 1024));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            float* g = out + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq;
            __builtin_nontemporal_store(v[i], (vf4*)g);
        }
    }
}

template <int R, int TC>
__global__ __launch_bounds__(64) void reg_copy(float* __restrict__ out, const float* __restrict__ in, int T) {
    constexpr int Q = TC / 4, RPI = 64 / Q, NI = R / RPI;
    const int lane = threadIdx.x, crow = lane / Q, cq = lane % Q;
    const long m0 = (long)blockIdx.x * R;
    vf4 st[NI];
    const int nch = T / TC;
    auto fetch = [&](int c) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
            st[i] = __builtin_nontemporal_load((const vf4*)(in + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq));
    };
    fetch(0);
    for (int c = 0; c < nch; ++c) {
        vf4 cur[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) cur[i] = st[i];
        if (c + 1 < nch) fetch(c + 1);
#pragma unroll
        for (int i = 0; i < NI; ++i)
            __builtin_nontemporal_store(cur[i], (vf4*)(out + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq));
    }
}

// D chunks of loads in flight per wave (a ring of D register buffers, named statically by unrolling D chunks)
template <int R, int TC, int D>
__global__ __launch_bounds__(64) void deep_copy(float* __restrict__ out, const float* __restrict__ in, int T) {
    constexpr int Q = TC / 4, RPI = 64 / Q, NI = R / RPI;
    extern __shared__ float unused_lds[];                // its size limits the waves per compute unit
    const int lane = threadIdx.x, crow = lane / Q, cq = lane % Q;
    if (T < 0) unused_lds[lane] = 0.f;
    const long m0 = (long)blockIdx.x * R;
    vf4 st[D][NI];
    const int nch = T / TC;
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < nch) {
#pragma unroll
            for (int i = 0; i < NI; ++i)
                st[d][i] = __builtin_nontemporal_load((const vf4*)(in + (m0 + i * RPI + crow) * (long)T + d * TC + 4 * cq));
        }
    for (int c = 0; c < nch; c += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int cc = c + d;
            if (cc < nch) {
                vf4 cur[NI];
#pragma unroll
                for (int i = 0; i < NI; ++i) cur[i] = st[d][i];
                if (cc + D < nch) {
#pragma unroll
                    for (int i = 0; i < NI; ++i)
                        st[d][i] = __builtin_nontemporal_load(
                            (const vf4*)(in + (m0 + i * RPI + crow) * (long)T + (cc + D) * TC + 4 * cq));
                }
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    __builtin_nontemporal_store(cur[i], (vf4*)(out + (m0 + i * RPI + crow) * (long)T + cc * TC + 4 * cq));
            }
        }
    }
}

// `reg` with each XCD walking a contiguous eighth of the tensor (the grid must be a multiple of 8)
template <int R, int TC>
__global__ __launch_bounds__(64) void xcd_copy(float* __restrict__ out, const float* __restrict__ in, int T) {
    constexpr int Q = TC / 4, RPI = 64 / Q, NI = R / RPI;
    const int lane = threadIdx.x, crow = lane / Q, cq = lane % Q;
    const unsigned b = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    const long m0 = (long)b * R;
    vf4 st[NI];
    const int nch = T / TC;
    auto fetch = [&](int c) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
            st[i] = __builtin_nontemporal_load((const vf4*)(in + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq));
    };
    fetch(0);
    for (int c = 0; c < nch; ++c) {
        vf4 cur[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) cur[i] = st[i];
        if (c + 1 < nch) fetch(c + 1);
#pragma unroll
        for (int i = 0; i < NI; ++i)
            __builtin_nontemporal_store(cur[i], (vf4*)(out + (m0 + i * RPI + crow) * (long)T + c * TC + 4 * cq));
    }
}

__global__ __launch_bounds__(256) void lin_copy(vf4* __restrict__ o, const vf4* __restrict__ i, size_t n) {
    const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
    vf4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) { const size_t k = base + u * 256; if (k < n) v[u] = __builtin_nontemporal_load(&i[k]); }
#pragma unroll
    for (int u = 0; u < 4; ++u) { const size_t k = base + u * 256; if (k < n) __builtin_nontemporal_store(v[u], &o[k]); }
}

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)

int main(int argc, char** argv) {
    const int T = argc > 1 ? atoi(argv[1]) : 384;
    const int reps = argc > 2 ? atoi(argv[2]) : 20;
    const bool few = argc > 3 && argv[3][0] == 'f' && argv[3][1] == 'e';
    const bool front = argc > 3 && !few;
    if (T <= 0 || T % 128 != 0 || reps <= 0) { printf("T must be a positive multiple of 128\n"); return 2; }
    const long M = (157286400L / T) / 256 * 256;          // the byte count of a [32,16,32,32,300] tensor
    const size_t bytes = (size_t)M * T * 4;
    float *a, *b;
    CHECK(hipMalloc(&a, bytes));
    CHECK(hipMalloc(&b, bytes));
    CHECK(hipMemset(a, 1, bytes));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    printf("T=%d M=%ld bytes per tensor=%zu\n", T, M, bytes);
    auto run = [&](const char* name, auto launch) {
        for (int w = 0; w < 3; ++w) launch();
        if (hipDeviceSynchronize() != hipSuccess) { printf("%s failed: %s\n", name, hipGetErrorString(hipGetLastError())); exit(1); }
        (void)hipEventRecord(e0);
        for (int r = 0; r < reps; ++r) launch();
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        ms /= reps;
        printf("%-44s %8.1f us %7.0f GB/s\n", name, ms * 1e3, 2.0 * bytes / ms / 1e6);
        fflush(stdout);
    };
    run("lin", [&] { hipLaunchKernelGGL(lin_copy, dim3((unsigned)(bytes / 16 / 1024)), dim3(256), 0, 0, (vf4*)b, (const vf4*)a, bytes / 16); });
#define LDS(R, TC, NBUF) { const size_t sh = (size_t)R * TC * 4 * NBUF; \
        (void)hipFuncSetAttribute((const void*)lds_copy<R, TC, NBUF>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh); \
        char nm[96]; snprintf(nm, 96, "lds  R=%d TC=%d NBUF=%d (%zu KB, %d waves/CU)", R, TC, NBUF, sh / 1024, (int)(160 * 1024 / sh)); \
        run(nm, [&] { hipLaunchKernelGGL((lds_copy<R, TC, NBUF>), dim3((unsigned)(M / R)), dim3(64), sh, 0, b, a, T); }); }
#define REG(R, TC) { char nm[96]; snprintf(nm, 96, "reg  R=%d TC=%d", R, TC); \
        run(nm, [&] { hipLaunchKernelGGL((reg_copy<R, TC>), dim3((unsigned)(M / R)), dim3(64), 0, 0, b, a, T); }); }
#define DEEP(R, TC, D, WPC) { const size_t sh = (size_t)(160 * 1024 / WPC) & ~(size_t)255; \
        (void)hipFuncSetAttribute((const void*)deep_copy<R, TC, D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh); \
        char nm[96]; snprintf(nm, 96, "deep R=%d TC=%d D=%d, %d waves/CU (%ld rows in flight)", R, TC, D, WPC, 256L * WPC * R); \
        run(nm, [&] { hipLaunchKernelGGL((deep_copy<R, TC, D>), dim3((unsigned)(M / R)), dim3(64), sh, 0, b, a, T); }); }
#define DEEPW(R, TC, D) DEEP(R, TC, D, 4) DEEP(R, TC, D, 8) DEEP(R, TC, D, 16) DEEP(R, TC, D, 32)
#define XCD(R, TC) { char nm[96]; snprintf(nm, 96, "xcd  R=%d TC=%d", R, TC); \
        run(nm, [&] { hipLaunchKernelGGL((xcd_copy<R, TC>), dim3((unsigned)(M / R)), dim3(64), 0, 0, b, a, T); }); }
    if (few) { REG(64, 32); REG(16, 128); LDS(64, 32, 4); LDS(16, 128, 4); return 0; }
    if (front) {
        if ((M / 64) % 8 != 0) { printf("front: M / 64 must be a multiple of 8\n"); return 2; }
        REG(64, 32); XCD(64, 32); REG(16, 128); XCD(16, 128);
        DEEPW(64, 32, 1) DEEPW(64, 32, 2) DEEPW(64, 32, 4)
        DEEPW(32, 32, 1) DEEPW(32, 32, 2) DEEPW(32, 32, 4)
        DEEPW(16, 32, 1) DEEPW(16, 32, 2) DEEPW(16, 32, 4)
        DEEPW(16, 128, 1) DEEPW(16, 128, 2)
        return 0;
    }
    REG(64, 32); REG(32, 64); REG(64, 64); REG(16, 128); REG(32, 128);
    LDS(64, 32, 2); LDS(64, 32, 3); LDS(64, 32, 4);
    LDS(64, 64, 2); LDS(64, 64, 3);
    LDS(32, 64, 2); LDS(32, 64, 4);
    LDS(32, 128, 2); LDS(32, 128, 3);
    LDS(64, 128, 2);
    LDS(16, 128, 2); LDS(16, 128, 4);
    return 0;
}
