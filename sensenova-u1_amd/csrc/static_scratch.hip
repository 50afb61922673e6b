// Device scratch memory that belongs to the library image itself, for the entry point that must not allocate
// (callers under HIP graph capture, serving loops and harnesses that forbid hipMalloc): one file-scope array per
// GPU the library runs on, resident from the moment the code object is loaded until the process ends.
//
// In host code the array's name is only a handle for the runtime, not a device address; the address on the
// current device comes from hipGetSymbolAddress, is looked up once per device and cached, and is what every
// kernel argument and copy uses.  Each GPU has its own copy of the array at its own address.
//
// All calls on one GPU share the area and it keeps the last call's contents.  Its users (the K-split partial
// sums and the transient bf16 weight of sngguf_linear_static) overwrite every element they later read, so nothing
// is cleared; two calls that overlap in time on one GPU (different streams) race on it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/sngguf.h"

namespace sngguf {

namespace {
constexpr int64_t kScratchBytes = (int64_t)64 << 20;   // 64 MiB per device
constexpr int kMaxDevices = 64;
}  // namespace

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
std::atomic<void*> g_scratch_ptr[kMaxDevices];
}  // namespace

int64_t static_scratch_bytes() { return kScratchBytes; }

// Address of the array on the current device (looked up on the first call per device; lock-free afterwards:
// concurrent first calls resolve the same address twice, which is harmless).
int static_scratch(void** ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SNGGUF_E_NODEVICE;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return SNGGUF_E_NODEVICE;
        }
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return SNGGUF_OK;
}

}  // namespace sngguf
