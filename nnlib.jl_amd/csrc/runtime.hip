// Runtime half of the C ABI: error strings, device selection, memory, streams, events.
#include "common.h"
#include <string.h>

int32_t attention_static_scratch(void **out);   // attention.hip

static thread_local char g_err[512] = "";

int32_t mi_set_error(int32_t code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

MI_API int32_t mi_version(void) { return MI355ATTN_VERSION; }
MI_API const char *mi_last_error_string(void) { return g_err; }

MI_API int32_t mi_device_count(int32_t *count) {
    if (!count) return mi_set_error(MI_EINVAL, "mi_device_count: count is NULL");
    int n = 0;
    MI_HIP_CHECK(hipGetDeviceCount(&n));
    *count = n;
    return MI_OK;
}

MI_API int32_t mi_init(int32_t device) {
    int n = 0;
    MI_HIP_CHECK(hipGetDeviceCount(&n));
    if (device < 0 || device >= n)
        return mi_set_error(MI_EINVAL, "mi_init: device %d out of range (%d visible)", device, n);
    MI_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t p;
    MI_HIP_CHECK(hipGetDeviceProperties(&p, device));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return mi_set_error(MI_EHIP, "mi_init: device %d is %s; this library carries gfx950 code only",
                            device, p.gcnArchName);
    void *scratch = nullptr;   // look the built-in attention workspace of this device up now, not inside a later call
    return attention_static_scratch(&scratch);
}

MI_API int32_t mi_device_name(char *buf, size_t buflen) {
    if (!buf || buflen == 0) return mi_set_error(MI_EINVAL, "mi_device_name: empty buffer");
    int dev = 0;
    MI_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t p;
    MI_HIP_CHECK(hipGetDeviceProperties(&p, dev));
    snprintf(buf, buflen, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
    return MI_OK;
}

MI_API int32_t mi_malloc(void **ptr, size_t bytes) {
    if (!ptr) return mi_set_error(MI_EINVAL, "mi_malloc: ptr is NULL");
    *ptr = nullptr;
    if (bytes == 0) return MI_OK;
    hipError_t e = hipMalloc(ptr, bytes);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        return mi_set_error(MI_ENOMEM, "mi_malloc: out of device memory for %zu bytes", bytes);
    }
    MI_HIP_CHECK(e);
    return MI_OK;
}

MI_API int32_t mi_free(void *ptr) {
    if (!ptr) return MI_OK;
    MI_HIP_CHECK(hipFree(ptr));
    return MI_OK;
}

static int32_t copy(void *dst, const void *src, size_t bytes, hipMemcpyKind kind, mi_stream s, const char *who) {
    if (bytes == 0) return MI_OK;
    if (!dst || !src) return mi_set_error(MI_EINVAL, "%s: null pointer", who);
    MI_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, kind, (hipStream_t)s));
    // host buffers are ordinary pageable memory owned by the caller: finish before returning
    if (kind != hipMemcpyDeviceToDevice) MI_HIP_CHECK(hipStreamSynchronize((hipStream_t)s));
    return MI_OK;
}
MI_API int32_t mi_memcpy_h2d(void *dst, const void *src, size_t bytes, mi_stream s) {
    return copy(dst, src, bytes, hipMemcpyHostToDevice, s, "mi_memcpy_h2d");
}
MI_API int32_t mi_memcpy_d2h(void *dst, const void *src, size_t bytes, mi_stream s) {
    return copy(dst, src, bytes, hipMemcpyDeviceToHost, s, "mi_memcpy_d2h");
}
MI_API int32_t mi_memcpy_d2d(void *dst, const void *src, size_t bytes, mi_stream s) {
    return copy(dst, src, bytes, hipMemcpyDeviceToDevice, s, "mi_memcpy_d2d");
}

__global__ void fill_zero_kernel(uint8_t *p, size_t bytes) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    // 16-byte body when aligned, byte tail otherwise
    if ((((uintptr_t)p) & 15) == 0) {
        size_t n16 = bytes / 16;
        u32x4_t z = {0, 0, 0, 0};
        for (size_t j = i; j < n16; j += stride) ((u32x4_t *)p)[j] = z;
        for (size_t j = n16 * 16 + i; j < bytes; j += stride) p[j] = 0;
    } else {
        for (size_t j = i; j < bytes; j += stride) p[j] = 0;
    }
}

MI_API int32_t mi_fill_zero(void *ptr, size_t bytes, mi_stream s) {
    if (bytes == 0) return MI_OK;
    if (!ptr) return mi_set_error(MI_EINVAL, "mi_fill_zero: null pointer");
    size_t want = (bytes / 16 + 255) / 256;
    int blocks = (int)(want < 1 ? 1 : (want > 4096 ? 4096 : want));
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)s, (uint8_t *)ptr, bytes);
    MI_LAUNCH_CHECK();
    return MI_OK;
}

MI_API int32_t mi_stream_create(mi_stream *s) {
    if (!s) return mi_set_error(MI_EINVAL, "mi_stream_create: null");
    hipStream_t st;
    MI_HIP_CHECK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *s = (mi_stream)st;
    return MI_OK;
}
MI_API int32_t mi_stream_destroy(mi_stream s) {
    if (!s) return MI_OK;
    MI_HIP_CHECK(hipStreamDestroy((hipStream_t)s));
    return MI_OK;
}
MI_API int32_t mi_stream_sync(mi_stream s) {
    MI_HIP_CHECK(hipStreamSynchronize((hipStream_t)s));
    return MI_OK;
}
MI_API int32_t mi_device_sync(void) {
    MI_HIP_CHECK(hipDeviceSynchronize());
    return MI_OK;
}
MI_API int32_t mi_event_create(mi_event *e) {
    if (!e) return mi_set_error(MI_EINVAL, "mi_event_create: null");
    hipEvent_t ev;
    MI_HIP_CHECK(hipEventCreate(&ev));
    *e = (mi_event)ev;
    return MI_OK;
}
MI_API int32_t mi_event_destroy(mi_event e) {
    if (!e) return MI_OK;
    MI_HIP_CHECK(hipEventDestroy((hipEvent_t)e));
    return MI_OK;
}
MI_API int32_t mi_event_record(mi_event e, mi_stream s) {
    if (!e) return mi_set_error(MI_EINVAL, "mi_event_record: null event");
    MI_HIP_CHECK(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
    return MI_OK;
}
MI_API int32_t mi_event_sync(mi_event e) {
    if (!e) return mi_set_error(MI_EINVAL, "mi_event_sync: null event");
    MI_HIP_CHECK(hipEventSynchronize((hipEvent_t)e));
    return MI_OK;
}
MI_API int32_t mi_event_elapsed_ms(mi_event a, mi_event b, float *ms) {
    if (!a || !b || !ms) return mi_set_error(MI_EINVAL, "mi_event_elapsed_ms: null argument");
    MI_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b));
    return MI_OK;
}
