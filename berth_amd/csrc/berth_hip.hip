// libberth_hip.so: the device runtime behind include/berth_hip.h.  Mirrors the
// used surface of crates/berth-cuda/src/{context,stream,event,buffer,pinned,module}.rs
// over the HIP runtime.  The device of a context is made current before every
// call (crates/berth-cuda/src/context.rs:91-93 binds before each raw call).
#include <hip/hip_runtime.h>

#include "../../include/berth_hip.h"

#include <cstring>
#include <string>

struct berth_hip_context { int ordinal; hipDeviceProp_t prop; };
struct berth_hip_stream { berth_hip_context* ctx; hipStream_t stream; };
struct berth_hip_event { berth_hip_context* ctx; hipEvent_t event; };
struct berth_hip_module { berth_hip_context* ctx; hipModule_t module; };
struct berth_hip_function { berth_hip_module* mod; hipFunction_t fn; };

namespace {
thread_local std::string g_err;

int fail(hipError_t e, const char* what)
{
    g_err = std::string(what) + ": " + hipGetErrorName(e) + " (" + std::to_string((int)e) + "): " +
            hipGetErrorString(e);
    (void)hipGetLastError();
    return (int)e;
}
int ok() { g_err.clear(); return 0; }
#define BH_TRY(call, what) do { hipError_t e_ = (call); if (e_ != hipSuccess) return fail(e_, what); } while (0)
#define BH_BIND(ctx) BH_TRY(hipSetDevice((ctx)->ordinal), "hipSetDevice")
hipStream_t raw(const berth_hip_stream* s) { return s ? s->stream : nullptr; }
}  // namespace

extern "C" {

const char* berth_hip_error_string(int code) { return hipGetErrorString((hipError_t)code); }
const char* berth_hip_last_error(void) { return g_err.c_str(); }

int berth_hip_context_new(int ordinal, berth_hip_context** out)
{
    if (!out) return fail(hipErrorInvalidValue, "context_new");
    int count = 0;
    BH_TRY(hipGetDeviceCount(&count), "hipGetDeviceCount");
    if (ordinal < 0 || ordinal >= count) return fail(hipErrorInvalidDevice, "context_new");
    BH_TRY(hipSetDevice(ordinal), "hipSetDevice");
    BH_TRY(hipFree(nullptr), "primary context");
    berth_hip_context* ctx = new berth_hip_context;
    ctx->ordinal = ordinal;
    hipError_t e = hipGetDeviceProperties(&ctx->prop, ordinal);
    if (e != hipSuccess) { delete ctx; return fail(e, "hipGetDeviceProperties"); }
    *out = ctx;
    return ok();
}
void berth_hip_context_free(berth_hip_context* ctx) { delete ctx; }
int berth_hip_context_ordinal(const berth_hip_context* ctx) { return ctx ? ctx->ordinal : -1; }
int berth_hip_context_multiprocessor_count(const berth_hip_context* ctx, uint32_t* out)
{
    if (!ctx || !out) return fail(hipErrorInvalidValue, "multiprocessor_count");
    *out = (uint32_t)ctx->prop.multiProcessorCount;
    return ok();
}
int berth_hip_context_compute_capability(const berth_hip_context* ctx, int* gfx, char* name, size_t name_len)
{
    if (!ctx) return fail(hipErrorInvalidValue, "compute_capability");
    if (gfx) {
        // "gfx950:sramecc+:xnack-": the digits are major, minor, stepping (hex)
        int v = 0;
        for (const char* p = ctx->prop.gcnArchName + 3; *p && *p != ':'; ++p) {
            int d = (*p >= '0' && *p <= '9') ? *p - '0' : (*p >= 'a' && *p <= 'f') ? *p - 'a' + 10 : 0;
            v = v * 10 + d;
        }
        *gfx = v;
    }
    if (name && name_len) {
        std::strncpy(name, ctx->prop.gcnArchName, name_len - 1);
        name[name_len - 1] = 0;
    }
    return ok();
}
int berth_hip_context_total_memory(const berth_hip_context* ctx, uint64_t* bytes)
{
    if (!ctx || !bytes) return fail(hipErrorInvalidValue, "total_memory");
    *bytes = (uint64_t)ctx->prop.totalGlobalMem;
    return ok();
}
int berth_hip_context_synchronize(const berth_hip_context* ctx)
{
    if (!ctx) return fail(hipErrorInvalidValue, "context_synchronize");
    BH_BIND(ctx);
    BH_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return ok();
}

int berth_hip_stream_new(berth_hip_context* ctx, berth_hip_stream** out)
{
    if (!ctx || !out) return fail(hipErrorInvalidValue, "stream_new");
    BH_BIND(ctx);
    hipStream_t s;
    // default priority only; non-blocking with respect to the null stream
    BH_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    *out = new berth_hip_stream{ctx, s};
    return ok();
}
void berth_hip_stream_free(berth_hip_stream* s)
{
    if (!s) return;
    (void)hipSetDevice(s->ctx->ordinal);
    (void)hipStreamSynchronize(s->stream);
    (void)hipStreamDestroy(s->stream);
    delete s;
}
uint64_t berth_hip_stream_handle(const berth_hip_stream* s) { return (uint64_t)(uintptr_t)raw(s); }
int berth_hip_stream_synchronize(const berth_hip_stream* s)
{
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipStreamSynchronize(raw(s)), "hipStreamSynchronize");
    return ok();
}
int berth_hip_stream_wait_event(const berth_hip_stream* s, const berth_hip_event* e)
{
    if (!e) return fail(hipErrorInvalidValue, "stream_wait_event");
    BH_BIND(e->ctx);
    BH_TRY(hipStreamWaitEvent(raw(s), e->event, 0), "hipStreamWaitEvent");
    return ok();
}

int berth_hip_event_new(berth_hip_context* ctx, berth_hip_event** out)
{
    if (!ctx || !out) return fail(hipErrorInvalidValue, "event_new");
    BH_BIND(ctx);
    hipEvent_t e;
    BH_TRY(hipEventCreate(&e), "hipEventCreate");
    *out = new berth_hip_event{ctx, e};
    return ok();
}
void berth_hip_event_free(berth_hip_event* e)
{
    if (!e) return;
    (void)hipSetDevice(e->ctx->ordinal);
    (void)hipEventDestroy(e->event);
    delete e;
}
int berth_hip_event_record(berth_hip_event* e, const berth_hip_stream* s)
{
    if (!e) return fail(hipErrorInvalidValue, "event_record");
    BH_BIND(e->ctx);
    BH_TRY(hipEventRecord(e->event, raw(s)), "hipEventRecord");
    return ok();
}
int berth_hip_event_synchronize(const berth_hip_event* e)
{
    if (!e) return fail(hipErrorInvalidValue, "event_synchronize");
    BH_BIND(e->ctx);
    BH_TRY(hipEventSynchronize(e->event), "hipEventSynchronize");
    return ok();
}
int berth_hip_event_elapsed_ms(const berth_hip_event* start, const berth_hip_event* end, float* ms)
{
    if (!start || !end || !ms) return fail(hipErrorInvalidValue, "event_elapsed_ms");
    BH_BIND(start->ctx);
    BH_TRY(hipEventElapsedTime(ms, start->event, end->event), "hipEventElapsedTime");
    return ok();
}

int berth_hip_buffer_alloc(berth_hip_context* ctx, size_t bytes, uint64_t* dptr)
{
    if (!ctx || !dptr) return fail(hipErrorInvalidValue, "buffer_alloc");
    BH_BIND(ctx);
    void* p = nullptr;
    if (bytes) BH_TRY(hipMalloc(&p, bytes), "hipMalloc");
    *dptr = (uint64_t)(uintptr_t)p;
    return ok();
}
int berth_hip_buffer_zeroed(berth_hip_context* ctx, const berth_hip_stream* s, size_t bytes, uint64_t* dptr)
{
    int rc = berth_hip_buffer_alloc(ctx, bytes, dptr);
    if (rc) return rc;
    if (bytes) {
        hipError_t e = hipMemsetAsync((void*)(uintptr_t)*dptr, 0, bytes, raw(s));
        if (e == hipSuccess) e = hipStreamSynchronize(raw(s));
        if (e != hipSuccess) { (void)hipFree((void*)(uintptr_t)*dptr); *dptr = 0; return fail(e, "hipMemsetAsync"); }
    }
    return ok();
}
int berth_hip_buffer_free(berth_hip_context* ctx, uint64_t dptr)
{
    if (!ctx) return fail(hipErrorInvalidValue, "buffer_free");
    if (!dptr) return ok();
    BH_BIND(ctx);
    // buffer.rs:275-286: work that still reads the buffer must finish first
    BH_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    BH_TRY(hipFree((void*)(uintptr_t)dptr), "hipFree");
    return ok();
}
int berth_hip_copy_from_host(const berth_hip_stream* s, uint64_t dst, const void* src, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst || !src) return fail(hipErrorInvalidValue, "copy_from_host");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, raw(s)), "hipMemcpyAsync H2D");
    BH_TRY(hipStreamSynchronize(raw(s)), "hipStreamSynchronize");
    return ok();
}
int berth_hip_copy_to_host(const berth_hip_stream* s, void* dst, uint64_t src, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst || !src) return fail(hipErrorInvalidValue, "copy_to_host");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, raw(s)), "hipMemcpyAsync D2H");
    BH_TRY(hipStreamSynchronize(raw(s)), "hipStreamSynchronize");
    return ok();
}
int berth_hip_copy_from_host_async(const berth_hip_stream* s, uint64_t dst, const void* src, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst || !src) return fail(hipErrorInvalidValue, "copy_from_host_async");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, raw(s)), "hipMemcpyAsync H2D");
    return ok();
}
int berth_hip_copy_to_host_async(const berth_hip_stream* s, void* dst, uint64_t src, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst || !src) return fail(hipErrorInvalidValue, "copy_to_host_async");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, raw(s)), "hipMemcpyAsync D2H");
    return ok();
}
int berth_hip_copy_device(const berth_hip_stream* s, uint64_t dst, uint64_t src, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst || !src) return fail(hipErrorInvalidValue, "copy_device");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemcpyAsync((void*)(uintptr_t)dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToDevice, raw(s)), "hipMemcpyAsync D2D");
    return ok();
}
int berth_hip_memset_async(const berth_hip_stream* s, uint64_t dst, int byte, size_t bytes)
{
    if (!bytes) return ok();
    if (!dst) return fail(hipErrorInvalidValue, "memset_async");
    if (s) BH_BIND(s->ctx);
    BH_TRY(hipMemsetAsync((void*)(uintptr_t)dst, byte, bytes, raw(s)), "hipMemsetAsync");
    return ok();
}

int berth_hip_pinned_alloc(berth_hip_context* ctx, size_t bytes, void** out)
{
    if (!ctx || !out) return fail(hipErrorInvalidValue, "pinned_alloc");
    BH_BIND(ctx);
    void* p = nullptr;
    if (bytes) {
        BH_TRY(hipHostMalloc(&p, bytes, hipHostMallocDefault), "hipHostMalloc");
        std::memset(p, 0, bytes);
    }
    *out = p;
    return ok();
}
int berth_hip_pinned_free(berth_hip_context* ctx, void* p)
{
    if (!ctx) return fail(hipErrorInvalidValue, "pinned_free");
    if (!p) return ok();
    BH_BIND(ctx);
    BH_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    BH_TRY(hipHostFree(p), "hipHostFree");
    return ok();
}

int berth_hip_module_load_file(berth_hip_context* ctx, const char* path, berth_hip_module** out)
{
    if (!ctx || !path || !out) return fail(hipErrorInvalidValue, "module_load_file");
    BH_BIND(ctx);
    hipModule_t m;
    BH_TRY(hipModuleLoad(&m, path), "hipModuleLoad");
    *out = new berth_hip_module{ctx, m};
    return ok();
}
int berth_hip_module_load_bytes(berth_hip_context* ctx, const void* image, size_t bytes, berth_hip_module** out)
{
    if (!ctx || !image || !bytes || !out) return fail(hipErrorInvalidValue, "module_load_bytes");
    BH_BIND(ctx);
    hipModule_t m;
    BH_TRY(hipModuleLoadData(&m, image), "hipModuleLoadData");
    *out = new berth_hip_module{ctx, m};
    return ok();
}
void berth_hip_module_free(berth_hip_module* m)
{
    if (!m) return;
    (void)hipSetDevice(m->ctx->ordinal);
    (void)hipDeviceSynchronize();
    (void)hipModuleUnload(m->module);
    delete m;
}
int berth_hip_module_function(berth_hip_module* m, const char* name, berth_hip_function** out)
{
    if (!m || !name || !out) return fail(hipErrorInvalidValue, "module_function");
    BH_BIND(m->ctx);
    hipFunction_t f;
    BH_TRY(hipModuleGetFunction(&f, m->module, name), "hipModuleGetFunction");
    *out = new berth_hip_function{m, f};
    return ok();
}
void berth_hip_function_free(berth_hip_function* f) { delete f; }
int berth_hip_function_set_max_dynamic_shared_bytes(berth_hip_function* f, uint32_t bytes)
{
    if (!f) return fail(hipErrorInvalidValue, "set_max_dynamic_shared_bytes");
    BH_BIND(f->mod->ctx);
    BH_TRY(hipFuncSetAttribute((const void*)f->fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes),
           "hipFuncSetAttribute");
    return ok();
}
int berth_hip_function_launch(berth_hip_function* f, const berth_hip_stream* s,
                              uint32_t gx, uint32_t gy, uint32_t gz,
                              uint32_t bx, uint32_t by, uint32_t bz,
                              uint32_t shared_bytes, void** params)
{
    if (!f) return fail(hipErrorInvalidValue, "function_launch");
    if (!gx || !gy || !gz || !bx || !by || !bz || (uint64_t)bx * by * bz > 1024)
        return fail(hipErrorInvalidConfiguration, "function_launch");
    BH_BIND(f->mod->ctx);
    BH_TRY(hipModuleLaunchKernel(f->fn, gx, gy, gz, bx, by, bz, shared_bytes, raw(s), params, nullptr),
           "hipModuleLaunchKernel");
    return ok();
}

}  // extern "C"
