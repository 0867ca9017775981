/*
 * fe_hip: the thin device-runtime binding under the quantized-linear layers.
 *
 * It replaces the reference's CUDA driver binding (crates/fe-cuda/src/lib.rs, raw symbols in
 * crates/fe-cuda/src/ffi.rs:73-148) with the same small surface over the HIP module API: a device context, linear
 * device memory, code-object modules and functions loaded by name, launches that take an array of pointers to the
 * argument values (the `kernelParams` convention the reference already uses, crates/fe-cuda/src/lib.rs:645-653),
 * streams, events and graph capture. Nothing here knows about the kernels it launches.
 *
 * Every call returns 0 on success or the failing hipError_t value; fe_hip_last_error() names the call and the error
 * (the reference's CuError{code, call}, crates/fe-cuda/src/lib.rs:15-43). Handles are opaque pointers.
 * Threading: one thread drives a context; fe_hip_init binds the device to the calling thread
 * (Context::bind, crates/fe-cuda/src/lib.rs:123-126).
 */
#ifndef FE_HIP_H
#define FE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *fe_stream_t;   /* hipStream_t; NULL is the default stream */
typedef void *fe_event_t;    /* hipEvent_t */
typedef void *fe_module_t;   /* hipModule_t */
typedef void *fe_function_t; /* hipFunction_t */
typedef void *fe_graph_t;    /* instantiated graph (hipGraphExec_t) */
typedef uint64_t fe_devptr_t; /* device address, as the reference's DevPtr(u64) (crates/fe-cuda/src/lib.rs:184-199) */

/* Context::new / bind / sm_count / synchronize (crates/fe-cuda/src/lib.rs:101-177) */
int fe_hip_init(int ordinal);
int fe_hip_cu_count(int *out);
int fe_hip_device_name(char *buf, size_t len);
int fe_hip_synchronize(void);
const char *fe_hip_last_error(void);

/* DeviceBuffer::alloc / zeroed / drop, memset (crates/fe-cuda/src/lib.rs:201-297) */
int fe_hip_malloc(fe_devptr_t *out, size_t bytes);
int fe_hip_free(fe_devptr_t p);
/* Debug aids of the allocator (crates/fe-cuda/src/lib.rs:213-228, 299-343). FE_ZERO_ALLOC=0 in the environment turns
 * off the zeroing of every new allocation (on by default, as in the reference). FE_CANARY=1 gives every allocation a
 * 64 KB tail filled with 0xA5; fe_hip_canary_tails reports, for up to cap of the live allocations whose tail has been
 * written, the base, the size, the offset of the first damaged tail byte and the number of damaged bytes (count: how
 * many there are in all), canary::tails of the reference. Both variables are read once, at the first allocation. */
typedef struct fe_canary_tail {
    fe_devptr_t base;
    size_t bytes, first, damaged;
} fe_canary_tail;
int fe_hip_canary_on(void);
int fe_hip_zero_alloc_on(void); /* 1 unless FE_ZERO_ALLOC is exactly "0" (the canary: on only for FE_CANARY exactly "1") */
int fe_hip_canary_tails(fe_canary_tail *out, size_t cap, size_t *count);
int fe_hip_memset_d8(fe_devptr_t p, uint8_t v, size_t n, fe_stream_t s);
int fe_hip_memset_d32(fe_devptr_t p, uint32_t v, size_t n, fe_stream_t s);
/* Synchronous copies: the device is synchronized before and after, because pageable host memory is not ordered
 * with non-blocking streams (crates/fe-cuda/src/lib.rs:351-371). */
int fe_hip_memcpy_htod(fe_devptr_t dst, const void *src, size_t bytes);
int fe_hip_memcpy_dtoh(void *dst, fe_devptr_t src, size_t bytes);
int fe_hip_memcpy_dtod_async(fe_devptr_t dst, fe_devptr_t src, size_t bytes, fe_stream_t s);

/* Module::load / function, Function::set_max_dynamic_smem (crates/fe-cuda/src/lib.rs:548-602) */
int fe_hip_module_load(fe_module_t *out, const void *image, size_t len);
int fe_hip_module_load_file(fe_module_t *out, const char *path);
int fe_hip_module_unload(fe_module_t m);
int fe_hip_module_get_function(fe_function_t *out, fe_module_t m, const char *name);
int fe_hip_func_set_max_dyn_lds(fe_function_t f, uint32_t bytes);

/* Stream::launch: params[i] points at the i-th argument value (crates/fe-cuda/src/lib.rs:627-674, 709-720) */
int fe_hip_launch(fe_function_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
                  uint32_t lds_bytes, fe_stream_t s, void **params);

/* Stream / Event (crates/fe-cuda/src/lib.rs:678-822) */
int fe_hip_stream_create(fe_stream_t *out);
int fe_hip_stream_destroy(fe_stream_t s);
int fe_hip_stream_sync(fe_stream_t s);
/* Times one kernel by itself: the calling thread's next fe_hip_launch (whichever library call makes it) is launched with
 * `start` and `stop` attached to its dispatch, so fe_hip_event_elapsed_ms(start, stop) after a sync is that kernel's own
 * duration, without the marker packets fe_hip_event_record puts into the stream. Not for a launch under graph capture
 * (a captured launch carries no events). Stream::time
 * (crates/fe-cuda/src/lib.rs:766-774) brackets a closure with two recorded events instead; CUDA has no per-launch form. */
int fe_hip_time_next_launch(fe_event_t start, fe_event_t stop);
int fe_hip_event_create(fe_event_t *out);
int fe_hip_event_destroy(fe_event_t e);
int fe_hip_event_record(fe_event_t e, fe_stream_t s);
int fe_hip_event_sync(fe_event_t e);
int fe_hip_event_elapsed_ms(float *out, fe_event_t start, fe_event_t stop);

/* Stream::begin_capture / end_capture, Graph::launch (crates/fe-cuda/src/lib.rs:825-843) */
int fe_hip_graph_begin(fe_stream_t s);
int fe_hip_graph_end(fe_stream_t s, fe_graph_t *out);
int fe_hip_graph_launch(fe_graph_t g, fe_stream_t s);
int fe_hip_graph_destroy(fe_graph_t g);

#ifdef __cplusplus
}
#endif
#endif
