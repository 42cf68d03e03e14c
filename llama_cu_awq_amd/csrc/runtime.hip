// Context, memory, stream and timing entry points of libawq_hip.
// These replace the reference's direct CUDA runtime calls around its hot path
// (llama2_q4.cu:62-136 allocation, :249 upload, :685-713 device/stream, :545-600 events).
#include <stdarg.h>
#include <string.h>

#include <mutex>

#include "common.hpp"

int awq_gemm_device_setup(int device);  // prefill.hip

static std::mutex g_err_mutex;
static char g_err[1024] = "";

void awq_set_error(const char* fmt, ...) {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" {

const char* awq_last_error(void) { return g_err; }

int awq_device_count(int* count) {
    AWQ_REQUIRE(count, AWQ_ERR_ARG, "null count");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e == hipErrorNoDevice) {
        *count = 0;
        return AWQ_OK;
    }
    if (e != hipSuccess) {
        awq_set_error("hipGetDeviceCount failed: %s", hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    *count = n;
    return AWQ_OK;
}

int awq_device_info(int device, char* name, size_t name_bytes, size_t* global_mem_bytes, int* compute_units) {
    hipDeviceProp_t prop;
    AWQ_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (name && name_bytes) {
        strncpy(name, prop.name, name_bytes - 1);
        name[name_bytes - 1] = 0;
    }
    if (global_mem_bytes) *global_mem_bytes = prop.totalGlobalMem;
    if (compute_units) *compute_units = prop.multiProcessorCount;
    return AWQ_OK;
}

// The device is current when this runs.
static int ctx_init(int device, hipStream_t stream, bool owns, awq_ctx** out) {
    // per-device set-up of the batched GEMM (kernel attribute, address of its static workspace): done here so that
    // the entry points themselves neither allocate nor configure anything
    if (int r = awq_gemm_device_setup(device)) {
        if (owns) (void)hipStreamDestroy(stream);
        return r;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) {
        if (owns) (void)hipStreamDestroy(stream);
        awq_set_error("cannot read the compute-unit count of device %d", device);
        return AWQ_ERR_HIP;
    }
    awq_ctx* c = new awq_ctx();
    c->device = device;
    c->cus = cus;
    c->stream = stream;
    c->owns_stream = owns;
    c->probe = nullptr;
    c->gemm_part = nullptr;
    c->gemm_part_bytes = 0;
    c->gemm_counter = nullptr;
    c->gemm_counter_count = 0;
    *out = c;
    return AWQ_OK;
}

int awq_ctx_create(int device, awq_ctx** out) {
    AWQ_REQUIRE(out, AWQ_ERR_ARG, "null out");
    int count = 0;
    AWQ_HIP_TRY(hipGetDeviceCount(&count));
    AWQ_REQUIRE(device >= 0 && device < count, AWQ_ERR_ARG, "no such device");
    AWQ_HIP_TRY(hipSetDevice(device));
    hipStream_t s;
    AWQ_HIP_TRY(hipStreamCreate(&s));  // default priority
    return ctx_init(device, s, true, out);
}

int awq_ctx_create_on_stream(int device, void* hip_stream, awq_ctx** out) {
    AWQ_REQUIRE(out, AWQ_ERR_ARG, "null out");
    AWQ_HIP_TRY(hipSetDevice(device));
    return ctx_init(device, (hipStream_t)hip_stream, false, out);
}

int awq_ctx_destroy(awq_ctx* ctx) {
    if (int r = awq_bind(ctx)) return r;
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->gemm_part) (void)hipFree(ctx->gemm_part);
    if (ctx->gemm_counter) (void)hipFree(ctx->gemm_counter);
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return AWQ_OK;
}

int awq_stream_sync(awq_ctx* ctx) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return AWQ_OK;
}

void* awq_ctx_stream(awq_ctx* ctx) { return ctx ? (void*)ctx->stream : nullptr; }

int awq_malloc(awq_ctx* ctx, void** ptr, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(ptr, AWQ_ERR_ARG, "null ptr");
    AWQ_HIP_TRY(hipMalloc(ptr, bytes ? bytes : 1));
    return AWQ_OK;
}

int awq_free(awq_ctx* ctx, void* ptr) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipFree(ptr));
    return AWQ_OK;
}

int awq_malloc_host(awq_ctx* ctx, void** ptr, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(ptr, AWQ_ERR_ARG, "null ptr");
    AWQ_HIP_TRY(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return AWQ_OK;
}

int awq_free_host(awq_ctx* ctx, void* ptr) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipHostFree(ptr));
    return AWQ_OK;
}

int awq_memcpy_h2d_async(awq_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    return AWQ_OK;
}

int awq_memcpy_h2d(awq_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    AWQ_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return AWQ_OK;
}

int awq_memcpy_d2h(awq_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    AWQ_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return AWQ_OK;
}

int awq_memcpy_d2d_async(awq_ctx* ctx, void* dst, const void* src, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return AWQ_OK;
}

int awq_memset_async(awq_ctx* ctx, void* dst, int value, size_t bytes) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipMemsetAsync(dst, value, bytes, ctx->stream));
    return AWQ_OK;
}

int awq_event_create(awq_ctx* ctx, void** event) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(event, AWQ_ERR_ARG, "null event");
    hipEvent_t e;
    AWQ_HIP_TRY(hipEventCreate(&e));
    *event = (void*)e;
    return AWQ_OK;
}

int awq_event_destroy(awq_ctx* ctx, void* event) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return AWQ_OK;
}

int awq_event_record(awq_ctx* ctx, void* event) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_HIP_TRY(hipEventRecord((hipEvent_t)event, ctx->stream));
    return AWQ_OK;
}

int awq_event_elapsed_ms(awq_ctx* ctx, void* start, void* stop, float* ms) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(ms, AWQ_ERR_ARG, "null ms");
    AWQ_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
    AWQ_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return AWQ_OK;
}

}  // extern "C"
