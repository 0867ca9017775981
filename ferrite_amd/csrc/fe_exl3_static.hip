// fe_exl3_linear_forward_static: the EXL3 decode forward for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It is fe_exl3_linear_forward with the
// workspace (rotated inputs, split-K partial sums, arrival counters) taken from one file-scope device array instead of
// a fe_exl3_workspace object. Every GPU the library runs on holds its own copy of the array until the process ends.
//
// The array's name is a host-side stand-in, not a device address: host code only ever uses the address that
// hipGetSymbolAddress returned for the current device (static_base), as kernel argument and for clearing.
#include <hip/hip_runtime.h>

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

void *g_base[kMaxDevices];  // device address of `scratch` on each device, once set up

__global__ void fe_static_zero(uint32_t *p, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Once per device, with that device current: the array's address on this device, counters cleared (they are zero at
// rest afterwards: the kernel that finishes a column block re-arms its counter).
int static_setup(int dev, hipStream_t s) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fe_check_hip(e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol, "hipGetSymbolAddress(scratch)");
    // a fill kernel, not hipMemsetAsync: the first call may come under stream capture
    fe_static_zero<<<(uint32_t)(kCounterBytes / 4 / 256), 256, 0, s>>>((uint32_t *)p, (uint32_t)(kCounterBytes / 4));
    e = hipGetLastError();
    if (e != hipSuccess) return fe_check_hip((int)e, "fe_static_zero");
    g_base[dev] = p;
    return 0;
}

}  // namespace

// Called by fe_hip_init for the device it binds (set-up outside any capture, synchronized).
int fe_exl3_static_setup_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fe_check_hip((int)e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fe_set_error(FE_ERR_UNSUPPORTED, "fe_exl3_static_setup", "device ordinal above 63");
    if (g_base[dev]) return 0;
    FE_TRY(static_setup(dev, nullptr));
    return fe_check_hip((int)hipDeviceSynchronize(), "hipDeviceSynchronize");
}

extern "C" int fe_exl3_linear_forward_static(const fe_exl3_linear *l, const fe_exl3_kernels *kern, fe_stream_t s, fe_devptr_t x,
                                             int x_dtype, fe_devptr_t y, int y_dtype, uint32_t rows) {
    const char *fn = "fe_exl3_linear_forward_static";
    if (!l || !kern || !x || !y) return fe_set_error(FE_ERR_ARG, fn, "null argument");
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fe_check_hip((int)e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fe_set_error(FE_ERR_UNSUPPORTED, fn, "device ordinal above 63");
    // a device the caller made current without fe_hip_init: set up on the call's stream, ahead of the kernels
    if (!g_base[dev]) FE_TRY(static_setup(dev, (hipStream_t)s));
    const fe_devptr_t base = (fe_devptr_t)(uintptr_t)g_base[dev];
    return fe_exl3_forward_over(l, kern, s, x, x_dtype, y, y_dtype, rows, FE_EXL3_STATIC_ROWS, base, kCounterBytes,
                                base + kCounterBytes, kXhBytes, base + kCounterBytes + kXhBytes,
                                FE_EXL3_STATIC_BYTES - kCounterBytes - kXhBytes, fn);
}
