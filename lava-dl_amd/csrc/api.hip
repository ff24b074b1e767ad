// Library-level entry points: ABI version, error text, the range flag of the fixed-point states.
#include "common.h"
#include <atomic>
#include <mutex>

namespace slayer {

bool bwd_scan_usable(int64_t M, int64_t npb, int64_t T);   // scan.hip

// One word of pinned host memory, mapped into the address space of every device, zero until a kernel (or an entry
// point) raises it.  Host code reads it directly: no copy, no synchronisation, valid for every launch that has
// completed.  Set up on first use; a failure (no device, or a call made while a stream is being captured) leaves
// the kernels without a flag to raise and is tried again on the next call.
static std::atomic<unsigned*> g_range_host{nullptr};
static std::atomic<unsigned*> g_range_device{nullptr};
static std::mutex g_range_lock;

unsigned* range_flag_device() {
    if (unsigned* d = g_range_device.load(std::memory_order_acquire)) return d;
    std::lock_guard<std::mutex> guard(g_range_lock);
    if (unsigned* d = g_range_device.load(std::memory_order_acquire)) return d;
    void* host = nullptr;
    if (hipHostMalloc(&host, 64, hipHostMallocMapped | hipHostMallocPortable) != hipSuccess || !host) {
        (void)hipGetLastError();
        return nullptr;
    }
    for (int i = 0; i < 16; ++i) static_cast<volatile unsigned*>(host)[i] = 0u;
    void* dev = nullptr;
    if (hipHostGetDevicePointer(&dev, host, 0) != hipSuccess || !dev) {
        (void)hipGetLastError();
        (void)hipHostFree(host);
        return nullptr;
    }
    g_range_host.store(static_cast<unsigned*>(host), std::memory_order_release);
    g_range_device.store(static_cast<unsigned*>(dev), std::memory_order_release);
    return static_cast<unsigned*>(dev);
}

void range_flag_raise_from_host() {
    if (range_flag_device())
        *static_cast<volatile unsigned*>(g_range_host.load(std::memory_order_acquire)) = 1u;
}

}  // namespace slayer

extern "C" int slayer_abi_version(void) { return SLAYER_ABI_VERSION; }

extern "C" const char* slayer_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case SLAYER_EINVAL: return "slayer_hip: inconsistent sizes";
        case SLAYER_ENULL: return "slayer_hip: required pointer is NULL";
        case SLAYER_ERANGE: return "slayer_hip: size beyond what the kernels index";
        case SLAYER_ESCRATCH: return "slayer_hip: size beyond the library's built-in scratch buffer";
        case SLAYER_ENOFLAG: return "slayer_hip: the range flag could not be set up (no device, or a stream capture in progress)";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "slayer_hip: unknown error code";
}

extern "C" int slayer_range_status(int* raised, int clear) {
    if (!slayer::range_flag_device()) return SLAYER_ENOFLAG;
    volatile unsigned* word = slayer::g_range_host.load(std::memory_order_acquire);
    if (raised) *raised = *word != 0u ? 1 : 0;
    if (clear) *word = 0u;
    return 0;
}

extern "C" const volatile unsigned* slayer_range_word(void) {
    return slayer::range_flag_device() ? slayer::g_range_host.load(std::memory_order_acquire) : nullptr;
}

extern "C" int slayer_bwd_takes_scan(int64_t M, int64_t neurons_per_batch, int64_t T) {
    return slayer::bwd_scan_usable(M, neurons_per_batch, T) ? 1 : 0;
}
