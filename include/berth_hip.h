/*
 * berth_hip.h — C ABI of libberth_hip.so, the device runtime that stands in for
 * the reference's berth-cuda crate (crates/berth-cuda/src/lib.rs:26-38).  A thin
 * layer over the HIP runtime: context on one device, streams, events, device and
 * pinned buffers, code-object loading and hipModuleLaunchKernel.  Graph capture
 * (crates/berth-cuda/src/graph.rs) is not part of the eager decode path and is
 * not provided.
 *
 * Every function returns 0 on success or the numeric hipError_t on failure
 * (crates/berth-cuda/src/error.rs:9-20 keeps "numeric driver code + text");
 * berth_hip_error_string / berth_hip_last_error give the text.  No HIP type
 * appears in a signature: handles are opaque pointers, device addresses are
 * uint64_t (crates/berth-cuda/src/ptr.rs:12 `DevicePtr`).
 */
#ifndef BERTH_HIP_H
#define BERTH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct berth_hip_context berth_hip_context;   /* context.rs:41 */
typedef struct berth_hip_stream berth_hip_stream;     /* stream.rs:58 */
typedef struct berth_hip_event berth_hip_event;       /* event.rs:14 */
typedef struct berth_hip_module berth_hip_module;     /* module.rs:47 `Cubin` */
typedef struct berth_hip_function berth_hip_function; /* module.rs:104 */

const char* berth_hip_error_string(int code);
const char* berth_hip_last_error(void);               /* thread-local text of the last failure */

/* ---- context.rs:45-93 */
int berth_hip_context_new(int ordinal, berth_hip_context** out);
void berth_hip_context_free(berth_hip_context* ctx);
int berth_hip_context_ordinal(const berth_hip_context* ctx);
int berth_hip_context_multiprocessor_count(const berth_hip_context* ctx, uint32_t* out);
/* compute capability: the gfx target as major*100 + minor*10 + stepping (950) and its name */
int berth_hip_context_compute_capability(const berth_hip_context* ctx, int* gfx, char* name, size_t name_len);
int berth_hip_context_total_memory(const berth_hip_context* ctx, uint64_t* bytes);
int berth_hip_context_synchronize(const berth_hip_context* ctx);

/* ---- stream.rs:25-99 */
int berth_hip_stream_new(berth_hip_context* ctx, berth_hip_stream** out);
void berth_hip_stream_free(berth_hip_stream* s);
/* the raw hipStream_t, the value the kernel shims take as `void* stream` */
uint64_t berth_hip_stream_handle(const berth_hip_stream* s);
int berth_hip_stream_synchronize(const berth_hip_stream* s);
int berth_hip_stream_wait_event(const berth_hip_stream* s, const berth_hip_event* e);

/* ---- event.rs:14-58 */
int berth_hip_event_new(berth_hip_context* ctx, berth_hip_event** out);
void berth_hip_event_free(berth_hip_event* e);
int berth_hip_event_record(berth_hip_event* e, const berth_hip_stream* s);
int berth_hip_event_synchronize(const berth_hip_event* e);
int berth_hip_event_elapsed_ms(const berth_hip_event* start, const berth_hip_event* end, float* ms);

/* ---- buffer.rs:22-286: sizes in bytes; free synchronises the context first */
int berth_hip_buffer_alloc(berth_hip_context* ctx, size_t bytes, uint64_t* dptr);
int berth_hip_buffer_zeroed(berth_hip_context* ctx, const berth_hip_stream* s, size_t bytes, uint64_t* dptr);
int berth_hip_buffer_free(berth_hip_context* ctx, uint64_t dptr);
int berth_hip_copy_from_host(const berth_hip_stream* s, uint64_t dst, const void* src, size_t bytes);        /* sync */
int berth_hip_copy_to_host(const berth_hip_stream* s, void* dst, uint64_t src, size_t bytes);                /* sync */
int berth_hip_copy_from_host_async(const berth_hip_stream* s, uint64_t dst, const void* src, size_t bytes);  /* pinned src */
int berth_hip_copy_to_host_async(const berth_hip_stream* s, void* dst, uint64_t src, size_t bytes);          /* pinned dst */
int berth_hip_copy_device(const berth_hip_stream* s, uint64_t dst, uint64_t src, size_t bytes);
int berth_hip_memset_async(const berth_hip_stream* s, uint64_t dst, int byte, size_t bytes);

/* ---- pinned.rs:17-145: page-locked host memory, always freshly allocated */
int berth_hip_pinned_alloc(berth_hip_context* ctx, size_t bytes, void** out);
int berth_hip_pinned_free(berth_hip_context* ctx, void* p);

/* ---- module.rs:17-180: code objects (.hsaco / .co) and launches */
int berth_hip_module_load_file(berth_hip_context* ctx, const char* path, berth_hip_module** out);
int berth_hip_module_load_bytes(berth_hip_context* ctx, const void* image, size_t bytes, berth_hip_module** out);
void berth_hip_module_free(berth_hip_module* m);
int berth_hip_module_function(berth_hip_module* m, const char* name, berth_hip_function** out);
void berth_hip_function_free(berth_hip_function* f);
int berth_hip_function_set_max_dynamic_shared_bytes(berth_hip_function* f, uint32_t bytes);
/* params: array of pointers to the argument values, as hipModuleLaunchKernel takes them */
int berth_hip_function_launch(berth_hip_function* f, const berth_hip_stream* s,
                              uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                              uint32_t block_x, uint32_t block_y, uint32_t block_z,
                              uint32_t shared_bytes, void** params);

#ifdef __cplusplus
}
#endif
#endif
