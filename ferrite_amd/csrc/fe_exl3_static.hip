// fe_exl3_linear_forward_static: the EXL3 decode forward for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It is fe_exl3_linear_forward with the
// workspace (rotated inputs, split-K partial sums, arrival counters) taken from one file-scope device array instead of
// a fe_exl3_workspace object. Every GPU the library runs on holds its own copy of the array until the process ends.
//
// The array's name is a host-side stand-in, not a device address: host code only ever uses the address that
// hipGetSymbolAddress returned for the current device (static_base), as kernel argument and for clearing.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>

#include "fe_exl3.h"
#include "fe_internal.h"

// counters | rotated inputs | partial sums
static __device__ __align__(256) unsigned char scratch[FE_EXL3_STATIC_BYTES];

namespace {

constexpr size_t kCounterBytes = 16 * 1024;  // 4096 arrival counters: n <= 524288 columns
constexpr size_t kXhBytes = (size_t)FE_EXL3_STATIC_ROWS * 32768 * 2;  // fp16 [rows][k], k <= 32768 at 16 rows
static_assert(kCounterBytes + kXhBytes < FE_EXL3_STATIC_BYTES, "no room for partial sums");
constexpr int kMaxDevices = 64;

std::atomic<void *> g_base[kMaxDevices];  // device address of `scratch` on each device, once taken

// The array's address on the current device `dev`. Nothing is cleared: a file-scope device array is zero when its
// module is loaded, the arrival counters are zero at rest (the program that finishes a column block re-arms its
// counter), and the other two areas are written before they are read. Threads that come here together take the same
// address and store the same value.
int static_setup(int dev) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fe_check_hip(e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol, "hipGetSymbolAddress(scratch)");
    g_base[dev].store(p, std::memory_order_release);
    return 0;
}

}  // namespace

// Called by fe_hip_init for the device it binds (outside any capture).
int fe_exl3_static_setup_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fe_check_hip((int)e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_static_setup", "device ordinal above 63");
    if (g_base[dev].load(std::memory_order_acquire)) return 0;
    return static_setup(dev);
}

extern "C" int fe_exl3_linear_forward_static(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                             int x_dtype, fe_devptr_t y, int y_dtype, uint32_t rows) {
    const char *fn = "fe_exl3_linear_forward_static";
    if (!l || !kern || !x || !y) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fe_check_hip((int)e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fe_set_error(FE_ERR_UNSUPPORTED, fn, "device ordinal above 63");
    // a device the caller made current without fe_hip_init: take the address now (under stream capture HIP may refuse
    // that; fe_hip_init on the device beforehand avoids it)
    if (!g_base[dev].load(std::memory_order_acquire)) FE_TRY(static_setup(dev));
    const fe_devptr_t base = (fe_devptr_t)(uintptr_t)g_base[dev].load(std::memory_order_acquire);
    return fe_exl3_forward_over(l, kern, s, x, x_dtype, y, y_dtype, rows, FE_EXL3_STATIC_ROWS, base, kCounterBytes,
                                base + kCounterBytes, kXhBytes, base + kCounterBytes + kXhBytes,
                                FE_EXL3_STATIC_BYTES - kCounterBytes - kXhBytes, fn);
}
