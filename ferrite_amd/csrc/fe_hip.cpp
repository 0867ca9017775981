// fe_hip: thin extern "C" binding over the HIP module API (see include/fe_hip.h).
#include "fe_hip.h"

#include <hip/hip_runtime_api.h>

// from hip/hip_ext.h, whose templates need the device compiler: a launch with events attached to its own dispatch
extern "C" hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX, uint32_t globalWorkSizeY,
                                               uint32_t globalWorkSizeZ, uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                               uint32_t localWorkSizeZ, size_t sharedMemBytes, hipStream_t hStream,
                                               void **kernelParams, void **extra, hipEvent_t startEvent, hipEvent_t stopEvent,
                                               uint32_t flags);

#include <cstdio>
#include <cstring>
#include <fstream>
#include <mutex>
#include <string>
#include <vector>

#include "fe_internal.h"

namespace {
thread_local std::string g_err;
int g_ordinal = 0;
}  // namespace

int fe_set_error(int code, const char *call, const char *detail) {
    char buf[512];
    snprintf(buf, sizeof buf, "%s: %s (%d)", call, detail ? detail : "", code);
    g_err = buf;
    return code ? code : -1;
}

int fe_check_hip(int code, const char *call) {
    if (code == 0) return 0;
    return fe_set_error(code, call, hipGetErrorString((hipError_t)code));
}

#define HIPCHK(x)                                   \
    do {                                            \
        int _c = fe_check_hip((int)(x), #x);        \
        if (_c) return _c;                          \
    } while (0)

extern "C" {

const char *fe_hip_last_error(void) { return g_err.c_str(); }

int fe_hip_init(int ordinal) {
    HIPCHK(hipInit(0));
    int n = 0;
    HIPCHK(hipGetDeviceCount(&n));
    if (ordinal < 0 || ordinal >= n) return fe_set_error(hipErrorInvalidDevice, "fe_hip_init", "no such device");
    HIPCHK(hipSetDevice(ordinal));
    g_ordinal = ordinal;
    return fe_exl3_static_setup_current_device();
}

int fe_hip_cu_count(int *out) {
    HIPCHK(hipDeviceGetAttribute(out, hipDeviceAttributeMultiprocessorCount, g_ordinal));
    return 0;
}

int fe_hip_device_name(char *buf, size_t len) {
    HIPCHK(hipDeviceGetName(buf, (int)len, g_ordinal));
    return 0;
}

int fe_hip_synchronize(void) {
    HIPCHK(hipDeviceSynchronize());
    return 0;
}

// Debug aids of the allocator (crates/fe-cuda/src/lib.rs:213-228, 299-343), both read from the environment once:
// FE_CANARY=1 gives every allocation a 64 KB tail filled with 0xA5 that fe_hip_canary_tails checks (an overflow into a
// neighbouring allocation raises no fault); FE_ZERO_ALLOC=0 leaves new memory as the driver hands it out instead of
// zeroing it (the default, as in the reference: a kernel that reads memory it never wrote then at least reads the same
// thing every run).
namespace {
constexpr size_t kCanaryPad = 64 << 10;
std::mutex g_canary_lock;
std::vector<std::pair<fe_devptr_t, size_t>> g_canary_live;
// The reference's reading of the two variables (crates/fe-cuda/src/lib.rs:307-316): zeroing is on unless FE_ZERO_ALLOC is
// exactly "0", the canary is on only when FE_CANARY is exactly "1".
bool env_equals(const char *name, const char *value) {
    const char *e = getenv(name);
    return e && strcmp(e, value) == 0;
}
bool canary_on() {
    static const bool on = env_equals("FE_CANARY", "1");
    return on;
}
bool zero_alloc() {
    static const bool on = !env_equals("FE_ZERO_ALLOC", "0");
    return on;
}
}  // namespace

int fe_hip_zero_alloc_on(void) { return zero_alloc() ? 1 : 0; }

int fe_hip_malloc(fe_devptr_t *out, size_t bytes) {
    void *p = nullptr;
    const size_t n = bytes ? bytes : 1;
    HIPCHK(hipMalloc(&p, n + (canary_on() ? kCanaryPad : 0)));
    // (a failure from here on gives the block back before it is reported)
    hipError_t e = hipSuccess;
    if (zero_alloc()) e = hipMemsetD8Async((hipDeviceptr_t)p, 0, n, nullptr);
    if (e == hipSuccess && canary_on()) e = hipMemsetD8Async((hipDeviceptr_t)((char *)p + bytes), 0xA5, kCanaryPad, nullptr);
    if (e == hipSuccess && (zero_alloc() || canary_on())) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) {
        (void)hipFree(p);
        return fe_check_hip((int)e, "fe_hip_malloc: clearing the new block");
    }
    if (canary_on()) {
        std::lock_guard<std::mutex> g(g_canary_lock);
        g_canary_live.emplace_back((fe_devptr_t)p, bytes);
    }
    *out = (fe_devptr_t)p;
    return 0;
}

int fe_hip_free(fe_devptr_t p) {
    if (!p) return 0;
    if (canary_on()) {
        std::lock_guard<std::mutex> g(g_canary_lock);
        for (size_t i = 0; i < g_canary_live.size(); i++)
            if (g_canary_live[i].first == p) {
                g_canary_live.erase(g_canary_live.begin() + (long)i);
                break;
            }
    }
    HIPCHK(hipFree((void *)p));
    return 0;
}

int fe_hip_canary_on(void) { return canary_on() ? 1 : 0; }

int fe_hip_canary_tails(fe_canary_tail *out, size_t cap, size_t *count) {
    if (!count) return fe_set_error(hipErrorInvalidValue, "fe_hip_canary_tails", "null count");
    *count = 0;
    if (!canary_on()) return 0;
    std::vector<std::pair<fe_devptr_t, size_t>> live;
    {
        std::lock_guard<std::mutex> g(g_canary_lock);
        live = g_canary_live;
    }
    HIPCHK(hipDeviceSynchronize());
    std::vector<unsigned char> buf(kCanaryPad);
    for (const auto &e : live) {
        HIPCHK(hipMemcpyDtoH(buf.data(), (hipDeviceptr_t)(e.first + e.second), kCanaryPad));
        size_t bad = 0, first = 0;
        for (size_t i = 0; i < kCanaryPad; i++)
            if (buf[i] != 0xA5) {
                if (!bad) first = i;
                bad++;
            }
        if (!bad) continue;
        if (out && *count < cap) out[*count] = {e.first, e.second, first, bad};
        ++*count;
    }
    return 0;
}

int fe_hip_memset_d8(fe_devptr_t p, uint8_t v, size_t n, fe_stream_t s) {
    HIPCHK(hipMemsetD8Async((hipDeviceptr_t)p, v, n, (hipStream_t)s));
    return 0;
}

int fe_hip_memset_d32(fe_devptr_t p, uint32_t v, size_t n, fe_stream_t s) {
    HIPCHK(hipMemsetD32Async((hipDeviceptr_t)p, (int)v, n, (hipStream_t)s));
    return 0;
}

int fe_hip_memcpy_htod(fe_devptr_t dst, const void *src, size_t bytes) {
    if (!bytes) return 0;
    HIPCHK(hipDeviceSynchronize());
    HIPCHK(hipMemcpyHtoD((hipDeviceptr_t)dst, const_cast<void *>(src), bytes));
    HIPCHK(hipDeviceSynchronize());
    return 0;
}

int fe_hip_memcpy_dtoh(void *dst, fe_devptr_t src, size_t bytes) {
    if (!bytes) return 0;
    HIPCHK(hipDeviceSynchronize());
    HIPCHK(hipMemcpyDtoH(dst, (hipDeviceptr_t)src, bytes));
    return 0;
}

int fe_hip_memcpy_dtod_async(fe_devptr_t dst, fe_devptr_t src, size_t bytes, fe_stream_t s) {
    HIPCHK(hipMemcpyDtoDAsync((hipDeviceptr_t)dst, (hipDeviceptr_t)src, bytes, (hipStream_t)s));
    return 0;
}

int fe_hip_module_load(fe_module_t *out, const void *image, size_t len) {
    (void)len;  // a code object carries its own size
    hipModule_t m = nullptr;
    HIPCHK(hipModuleLoadData(&m, image));
    *out = m;
    return 0;
}

int fe_hip_module_load_file(fe_module_t *out, const char *path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return fe_set_error(hipErrorFileNotFound, "fe_hip_module_load_file", path);
    std::vector<char> img((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    return fe_hip_module_load(out, img.data(), img.size());
}

int fe_hip_module_unload(fe_module_t m) {
    if (!m) return 0;
    HIPCHK(hipModuleUnload((hipModule_t)m));
    return 0;
}

int fe_hip_module_get_function(fe_function_t *out, fe_module_t m, const char *name) {
    hipFunction_t f = nullptr;
    int c = (int)hipModuleGetFunction(&f, (hipModule_t)m, name);
    if (c) return fe_set_error(c, "hipModuleGetFunction", name);
    *out = f;
    return 0;
}

int fe_hip_func_set_max_dyn_lds(fe_function_t f, uint32_t bytes) {
    HIPCHK(hipFuncSetAttribute((const void *)f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return 0;
}

// events for the calling thread's next fe_hip_launch (fe_hip_time_next_launch)
static thread_local fe_event_t t_time_start = nullptr, t_time_stop = nullptr;

int fe_hip_launch(fe_function_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
                  uint32_t lds_bytes, fe_stream_t s, void **params) {
    // the events of fe_hip_time_next_launch belong to this launch, also when it is rejected below
    fe_event_t time_start = t_time_start, time_stop = t_time_stop;
    t_time_start = t_time_stop = nullptr;
    if (!f) return fe_set_error(hipErrorInvalidHandle, "fe_hip_launch", "null function");
    if (!gx || !gy || !gz || !bx || !by || !bz || (uint64_t)bx * by * bz > 1024)
        return fe_set_error(hipErrorInvalidConfiguration, "fe_hip_launch", "empty grid or block, or block > 1024");
    if (time_start || time_stop) {
        // one launch with events attached to its own dispatch: they take the kernel's begin and end timestamps, with no
        // marker packets in the stream around it (global sizes are in work-items here)
        hipEvent_t a = (hipEvent_t)time_start, b = (hipEvent_t)time_stop;
        HIPCHK(hipExtModuleLaunchKernel((hipFunction_t)f, gx * bx, gy * by, gz * bz, bx, by, bz, lds_bytes, (hipStream_t)s, params,
                                        nullptr, a, b, 0));
        return 0;
    }
    HIPCHK(hipModuleLaunchKernel((hipFunction_t)f, gx, gy, gz, bx, by, bz, lds_bytes, (hipStream_t)s, params, nullptr));
    return 0;
}

int fe_hip_time_next_launch(fe_event_t start, fe_event_t stop) {
    t_time_start = start;
    t_time_stop = stop;
    return 0;
}

int fe_hip_stream_create(fe_stream_t *out) {
    hipStream_t s = nullptr;
    HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = s;
    return 0;
}

int fe_hip_stream_destroy(fe_stream_t s) {
    if (!s) return 0;
    HIPCHK(hipStreamDestroy((hipStream_t)s));
    return 0;
}

int fe_hip_stream_sync(fe_stream_t s) {
    HIPCHK(hipStreamSynchronize((hipStream_t)s));
    return 0;
}

int fe_hip_event_create(fe_event_t *out) {
    hipEvent_t e = nullptr;
    HIPCHK(hipEventCreate(&e));
    *out = e;
    return 0;
}

int fe_hip_event_destroy(fe_event_t e) {
    if (!e) return 0;
    HIPCHK(hipEventDestroy((hipEvent_t)e));
    return 0;
}

int fe_hip_event_record(fe_event_t e, fe_stream_t s) {
    HIPCHK(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
    return 0;
}

int fe_hip_event_sync(fe_event_t e) {
    HIPCHK(hipEventSynchronize((hipEvent_t)e));
    return 0;
}

int fe_hip_event_elapsed_ms(float *out, fe_event_t start, fe_event_t stop) {
    HIPCHK(hipEventElapsedTime(out, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

struct fe_graph {
    hipGraph_t g = nullptr;
    hipGraphExec_t e = nullptr;
};

int fe_hip_graph_begin(fe_stream_t s) {
    HIPCHK(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal));
    return 0;
}

int fe_hip_graph_end(fe_stream_t s, fe_graph_t *out) {
    fe_graph *g = new fe_graph;
    int c = fe_check_hip((int)hipStreamEndCapture((hipStream_t)s, &g->g), "hipStreamEndCapture");
    if (!c) c = fe_check_hip((int)hipGraphInstantiate(&g->e, g->g, nullptr, nullptr, 0), "hipGraphInstantiate");
    if (c) {
        if (g->g) (void)hipGraphDestroy(g->g);
        delete g;
        return c;
    }
    *out = g;
    return 0;
}

int fe_hip_graph_launch(fe_graph_t g, fe_stream_t s) {
    if (!g) return fe_set_error(hipErrorInvalidHandle, "fe_hip_graph_launch", "null graph");
    HIPCHK(hipGraphLaunch(((fe_graph *)g)->e, (hipStream_t)s));
    return 0;
}

int fe_hip_graph_destroy(fe_graph_t g) {
    if (!g) return 0;
    fe_graph *p = (fe_graph *)g;
    (void)hipGraphExecDestroy(p->e);
    (void)hipGraphDestroy(p->g);
    delete p;
    return 0;
}

}  // extern "C"
