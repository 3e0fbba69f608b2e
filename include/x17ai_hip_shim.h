/*
 * x17ai_hip_shim.h -- C ABI of the HIP device shim (libx17ai_hip_shim.so).
 *
 * Drop-in twin of the reference's CUDA driver-API shim: the same 21 entry points with
 * the same argument order, struct layouts, ownership and error convention, so that the
 * Rust side (src/device/cuda/cuda_shim.rs:76-158) only has to change its link names
 * from x17ai_cuda_* to x17ai_hip_*.  C++ side of the reference: cpp/cuda_shim.cpp:189-988,
 * cpp/ffi.hpp.
 *
 * Error convention (cpp/ffi.hpp:84-175): a function returns NULL (or a PtrResult with
 * value != NULL, diagnostic == NULL) on success.  On failure it returns a non-NULL
 * X17DiagnosticBuffer*, which the caller MUST hand to x17ai_move_diagnostic exactly once;
 * that call appends the message to the caller's buffer and frees heap diagnostics.
 * No function throws; no function leaves a different HIP device current than on entry.
 *
 * Handles: X17HipDeviceData* IS the device address (kernels receive it verbatim,
 * cpp/cuda_shim.cpp:90-100).  All other handles are opaque heap objects.
 */
#ifndef X17AI_HIP_SHIM_H
#define X17AI_HIP_SHIM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- caller-owned growable byte buffer (src/util/ffi_buffer.rs:13-103, cpp/ffi.hpp:12-82) */
typedef struct X17FfiSpan {
	char *ptr;
	size_t len;
} X17FfiSpan;

typedef struct X17FfiBufferVMT {
	X17FfiSpan (*span)(void *self);                     /* initialised bytes            */
	X17FfiSpan (*buf_span)(void *self);                 /* whole capacity               */
	X17FfiSpan (*extend)(void *self, size_t additional);/* grow len, return the new tail */
	void (*clear)(void *self);
	void (*set_len)(void *self, size_t new_len);
} X17FfiBufferVMT;

typedef struct X17FfiBuffer {
	void *instance;
	X17FfiBufferVMT const *vmt;
} X17FfiBuffer;

/* ---- opaque handles (src/device/cuda/cuda_shim.rs:19-68) */
typedef struct X17HipContextHandle {
	size_t refcnt_minus_one;   /* the one caller-visible field (cuda_shim.rs:20-24) */
} X17HipContextHandle;
typedef struct X17HipStreamHandle X17HipStreamHandle;
typedef struct X17HipDeviceData X17HipDeviceData;
typedef struct X17HipTimerHandle X17HipTimerHandle;
typedef struct X17HipModuleHandle X17HipModuleHandle;
typedef struct X17HipKernelHandle X17HipKernelHandle;
typedef struct X17DiagnosticBuffer X17DiagnosticBuffer;

/* src/device/cuda/cuda_shim.rs:51-63 -- nine int32 in this order */
typedef struct X17HipKernelAttrs {
	int32_t max_threads_per_block;
	int32_t static_shared_size_bytes;
	int32_t const_size_bytes;
	int32_t local_size_bytes;          /* scratch (spill) bytes per lane */
	int32_t num_regs;
	int32_t ptx_version;
	int32_t binary_version;
	int32_t max_dynamic_shared_size_bytes;
	int32_t preferred_shared_memory_carveout;
} X17HipKernelAttrs;

/* src/device/cuda/cuda_shim.rs:70-74 -- two pointers, returned by value */
#define X17_PTR_RESULT(NAME, T) \
	typedef struct NAME { T *value; X17DiagnosticBuffer *diagnostic; } NAME
X17_PTR_RESULT(X17ContextResult, X17HipContextHandle);
X17_PTR_RESULT(X17StreamResult, X17HipStreamHandle);
X17_PTR_RESULT(X17TimerResult, X17HipTimerHandle);
X17_PTR_RESULT(X17DeviceDataResult, X17HipDeviceData);
X17_PTR_RESULT(X17ModuleResult, X17HipModuleHandle);
X17_PTR_RESULT(X17KernelResult, X17HipKernelHandle);

/* replaces x17ai_move_diagnostic, cpp/cuda_shim.cpp:190-205 (same name: it is device-neutral) */
void x17ai_move_diagnostic(X17DiagnosticBuffer *diag, X17FfiBuffer err);

/* replaces x17ai_cuda_open_context, cpp/cuda_shim.cpp:207-317 */
X17ContextResult x17ai_hip_open_context(size_t device_id);
/* replaces x17ai_cuda_close_context, cpp/cuda_shim.cpp:319-342 */
X17DiagnosticBuffer *x17ai_hip_close_context(X17HipContextHandle *ctx);
/* replaces x17ai_cuda_context_ptr, cpp/cuda_shim.cpp:343-347 */
void *x17ai_hip_context_ptr(X17HipContextHandle *ctx);

/* replaces x17ai_cuda_open_stream, cpp/cuda_shim.cpp:349-387 (one non-blocking stream) */
X17StreamResult x17ai_hip_open_stream(X17HipContextHandle *ctx);
/* replaces x17ai_cuda_close_stream, cpp/cuda_shim.cpp:388-407 */
X17DiagnosticBuffer *x17ai_hip_close_stream(X17HipStreamHandle *stream);
/* replaces x17ai_cuda_synchronize, cpp/cuda_shim.cpp:408-427 */
X17DiagnosticBuffer *x17ai_hip_synchronize(X17HipStreamHandle *stream);

/* replaces x17ai_cuda_create_timer .. timer_elapsed_seconds, cpp/cuda_shim.cpp:432-652 */
X17TimerResult x17ai_hip_create_timer(X17HipContextHandle *ctx, X17HipStreamHandle *stream);
X17DiagnosticBuffer *x17ai_hip_destroy_timer(X17HipTimerHandle *timer);
X17DiagnosticBuffer *x17ai_hip_timer_start(X17HipTimerHandle *timer);
X17DiagnosticBuffer *x17ai_hip_timer_stop(X17HipTimerHandle *timer);
X17DiagnosticBuffer *x17ai_hip_timer_elapsed_seconds(X17HipTimerHandle *timer, double *seconds);

/* replaces x17ai_cuda_alloc / free, cpp/cuda_shim.cpp:654-700 (stream-ordered) */
X17DeviceDataResult x17ai_hip_alloc(X17HipStreamHandle *stream, size_t bytes);
X17DiagnosticBuffer *x17ai_hip_free(X17HipStreamHandle *stream, X17HipDeviceData *ptr);

/* replaces x17ai_cuda_upload_data / download_data, cpp/cuda_shim.cpp:701-760 (async on the stream) */
X17DiagnosticBuffer *x17ai_hip_upload_data(X17HipStreamHandle *stream, uint8_t const *src,
                                           X17HipDeviceData *dst, size_t offset_bytes, size_t size_bytes);
X17DiagnosticBuffer *x17ai_hip_download_data(X17HipStreamHandle *stream, X17HipDeviceData *src,
                                             uint8_t *dst, size_t offset_bytes, size_t size_bytes);

/* replaces x17ai_cuda_load_module / del_module, cpp/cuda_shim.cpp:761-846 (a gfx950 code object) */
X17ModuleResult x17ai_hip_load_module(X17HipContextHandle *ctx, char const *code_object_path);
X17DiagnosticBuffer *x17ai_hip_del_module(X17HipModuleHandle *module);

/* replaces x17ai_cuda_get_kernel, cpp/cuda_shim.cpp:848-905; smem_size = dynamic LDS the
 * launches will ask for */
X17KernelResult x17ai_hip_get_kernel(X17HipModuleHandle *module, char const *name, size_t smem_size);
/* replaces x17ai_cuda_read_kernel_attrs, cpp/cuda_shim.cpp:907-927 */
X17DiagnosticBuffer *x17ai_hip_read_kernel_attrs(X17HipKernelHandle *kernel, X17HipKernelAttrs *attrs);

/* replaces x17ai_cuda_launch_kernel, cpp/cuda_shim.cpp:929-987; args[i] points at the i-th
 * kernel parameter, of which sizeof(parameter) bytes are copied */
X17DiagnosticBuffer *x17ai_hip_launch_kernel(
	X17HipStreamHandle *stream, X17HipKernelHandle *kernel,
	size_t grid_x, size_t grid_y, size_t grid_z,
	size_t block_x, size_t block_y, size_t block_z,
	size_t shared_mem_bytes, void **args);

#ifdef __cplusplus
}
#endif
#endif /* X17AI_HIP_SHIM_H */
