// Thin HIP runtime shims with the reference's int return convention (0 = ok, positive =
// runtime error code).  Replace the subset of op_init.cu a standalone harness needs
// (csrc/warp34_cuda.h:135,142-164).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/warp34_kv.h"

extern "C" {

const char* warp34_cuda_error_string(int code) {
    if (code < 0) return "host-side error";
    return hipGetErrorString((hipError_t)code);
}
int warp34_get_device_count(int* out_count) {
    if (!out_count) return (int)hipErrorInvalidValue;
    return (int)hipGetDeviceCount(out_count);
}
int warp34_set_device(int device_id) { return (int)hipSetDevice(device_id); }
int warp34_device_synchronize(void) { return (int)hipDeviceSynchronize(); }
int warp34_get_mem_info(size_t* out_free, size_t* out_total) {
    if (!out_free || !out_total) return (int)hipErrorInvalidValue;
    return (int)hipMemGetInfo(out_free, out_total);
}
int warp34_malloc(void** out_ptr, size_t bytes) {
    if (!out_ptr) return (int)hipErrorInvalidValue;
    return (int)hipMalloc(out_ptr, bytes);
}
int warp34_free(void* ptr) { return (int)hipFree(ptr); }
int warp34_memcpy_h2d_async(void* dst, const void* src, size_t bytes, uintptr_t stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream);
}
int warp34_memcpy_d2h_async(void* dst, const void* src, size_t bytes, uintptr_t stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream);
}
int warp34_memcpy_d2d_async(void* dst, const void* src, size_t bytes, uintptr_t stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream);
}
int warp34_memset_async(void* dst, int value, size_t bytes, uintptr_t stream) {
    return (int)hipMemsetAsync(dst, value, bytes, (hipStream_t)stream);
}
int warp34_stream_create(uintptr_t* out_stream) {
    if (!out_stream) return (int)hipErrorInvalidValue;
    hipStream_t s = nullptr;
    const int rc = (int)hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
    *out_stream = (uintptr_t)s;
    return rc;
}
int warp34_stream_destroy(uintptr_t stream) { return (int)hipStreamDestroy((hipStream_t)stream); }
int warp34_stream_synchronize(uintptr_t stream) {
    return (int)hipStreamSynchronize((hipStream_t)stream);
}
int warp34_event_create(uintptr_t* out_event, int enable_timing) {
    if (!out_event) return (int)hipErrorInvalidValue;
    hipEvent_t e = nullptr;
    const int rc = (int)hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming);
    *out_event = (uintptr_t)e;
    return rc;
}
int warp34_event_destroy(uintptr_t event) { return (int)hipEventDestroy((hipEvent_t)event); }
int warp34_event_record(uintptr_t event, uintptr_t stream) {
    return (int)hipEventRecord((hipEvent_t)event, (hipStream_t)stream);
}
int warp34_stream_wait_event(uintptr_t stream, uintptr_t event) {
    return (int)hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0);
}
int warp34_event_synchronize(uintptr_t event) { return (int)hipEventSynchronize((hipEvent_t)event); }
int warp34_event_elapsed_ms(float* out_ms, uintptr_t start_event, uintptr_t end_event) {
    if (!out_ms) return (int)hipErrorInvalidValue;
    return (int)hipEventElapsedTime(out_ms, (hipEvent_t)start_event, (hipEvent_t)end_event);
}

}  // extern "C"
