// hip_shim.cpp -- the C-ABI device shim over the HIP runtime/module API.
//
// Replaces cpp/cuda_shim.cpp of the reference (CUDA driver API) entry point by entry
// point; see include/x17ai_hip_shim.h for the contract and the per-symbol citations.
//
// HIP has no retained driver contexts to push and pop: the unit of "current state" is the
// calling thread's current device.  Every entry point that needs a device makes it current
// for the duration of the call and restores the previous one on exit (DeviceScope), which
// is this shim's form of the reference's "no CUDA context may leak across the FFI" rule
// (cpp/ffi.hpp:195-206).
//
// This translation unit is host code only; it is built with hipcc for its include and
// link paths, not for device compilation.

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <bit>
#include <cassert>
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <mutex>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

#include "../../include/x17ai_hip_shim.h"

namespace {

// ---------------------------------------------------------------- diagnostics

struct Diag {
	size_t is_allocated;
	std::string_view message;
	explicit constexpr Diag(std::string_view msg): is_allocated(0), message(msg) {}
};

struct HeapDiag: Diag {
	std::string buffer;
	explicit HeapDiag(std::string_view fallback): Diag(fallback), buffer() { is_allocated = 1; }
	void append(std::string_view s) noexcept {
		try { buffer.append(s); } catch (...) {}
		message = buffer;
	}
	void append(hipError_t e) noexcept {
		char const *name = hipGetErrorName(e);
		char const *text = hipGetErrorString(e);
		append(name != nullptr ? name : "hipErrorUnknown");
		if (text != nullptr) { append(" ("); append(text); append(")"); }
	}
	void append(char const *s) noexcept { append(std::string_view(s)); }
};

inline X17DiagnosticBuffer *as_c(Diag *d) noexcept { return reinterpret_cast<X17DiagnosticBuffer *>(d); }

// A heap diagnostic when memory allows, else the static fallback (never fails).
template<typename... Parts>
X17DiagnosticBuffer *make_diag(Diag *fallback, Parts const &... parts) noexcept {
	try {
		auto d = std::make_unique<HeapDiag>(fallback->message);
		(d->append(parts), ...);
		return as_c(d.release());
	} catch (...) {
		return as_c(fallback);
	}
}

#define X17_DIAG(FALLBACK, ...) \
	([&]() noexcept -> X17DiagnosticBuffer * { \
		static Diag fallback_diag{FALLBACK}; \
		return make_diag(&fallback_diag, __VA_ARGS__); \
	}())

#define X17_STATIC_DIAG(TEXT) \
	([]() noexcept -> X17DiagnosticBuffer * { \
		static Diag fallback_diag{TEXT}; \
		return as_c(&fallback_diag); \
	}())

#define X17_CATCH(FN) \
	catch (std::exception const &e) { \
		return X17_DIAG(FN ": exception thrown.", FN ": exception thrown: ", e.what()); \
	} catch (...) { \
		return X17_STATIC_DIAG(FN ": unknown exception thrown"); \
	}

#define X17_HIP_CHECK(FN, CALLNAME, EXPR) \
	do { \
		hipError_t e_ = (EXPR); \
		if (e_ != hipSuccess) [[unlikely]] { \
			return X17_DIAG(FN ": " CALLNAME " failed.", FN ": " CALLNAME " failed with hip error: ", e_); \
		} \
	} while (0)

// ---------------------------------------------------------------- handles

struct Ctx {
	X17HipContextHandle pub;   // refcnt_minus_one: first field, visible to the caller
	size_t device_id;
	int device;
	size_t arch_major;
	size_t arch_minor;
	size_t wavefront_size;
};

struct Stream {
	int device;
	hipStream_t stream;
};

struct Timer {
	int device;
	hipStream_t stream;
	hipEvent_t start;
	hipEvent_t end;
};

struct Kernel {
	int device;
	hipFunction_t function;
	size_t max_dynamic_smem;
};

// The reference's kernel handle is the CUfunction itself (cpp/cuda_shim.cpp:903) and the ABI has no call that
// releases one; here a handle is a small record, owned by its module and freed with it in x17ai_hip_del_module.
struct Module {
	int device;
	hipModule_t module;
	std::vector<std::unique_ptr<Kernel>> kernels;
	// The code object as read from the file, alive as long as the module.  The module is created from these bytes and
	// not from the path: the runtime keeps the file handles of paths it has loaded, so a code object rebuilt under the
	// same path within one process would be loaded as its previous contents.
	std::vector<char> image;
};

// Makes `device` current for the scope, restores the previous device afterwards.
struct DeviceScope {
	int previous = -1;
	hipError_t error = hipSuccess;
	explicit DeviceScope(int device) noexcept {
		error = hipGetDevice(&previous);
		if (error != hipSuccess) { previous = -1; return; }
		if (previous != device) {
			error = hipSetDevice(device);
		}
	}
	~DeviceScope() {
		if (previous >= 0) {
			int now = -1;
			if (hipGetDevice(&now) == hipSuccess && now != previous) {
				(void)hipSetDevice(previous);
			}
		}
	}
	DeviceScope(DeviceScope const &) = delete;
	DeviceScope &operator=(DeviceScope const &) = delete;
};

std::atomic<bool> hip_initialized{false};
std::mutex hip_init_mutex;

template<typename R>
inline R ok(decltype(R::value) v) noexcept { return R{v, nullptr}; }
template<typename R>
inline R fail(X17DiagnosticBuffer *d) noexcept { return R{nullptr, d}; }

inline bool fits_u32(size_t v) noexcept { return v <= 0xFFFFFFFFull; }
inline bool fits_int(size_t v) noexcept { return v <= 0x7FFFFFFFull; }

} // namespace

extern "C" {

void x17ai_move_diagnostic(X17DiagnosticBuffer *diag_c, X17FfiBuffer err) {
	if (diag_c == nullptr) {
		return;
	}
	try {
		Diag *diag = reinterpret_cast<Diag *>(diag_c);
		std::unique_ptr<HeapDiag> owner;
		if (diag->is_allocated) {
			owner.reset(static_cast<HeapDiag *>(diag));
		}
		std::string_view msg = diag->message;
		if (err.vmt != nullptr && err.vmt->extend != nullptr && !msg.empty()) {
			X17FfiSpan tail = err.vmt->extend(err.instance, msg.size());
			if (tail.ptr != nullptr && tail.len == msg.size()) {
				std::memcpy(tail.ptr, msg.data(), msg.size());
			}
		}
	} catch (...) {}
}

X17ContextResult x17ai_hip_open_context(size_t device_id) {
	using R = X17ContextResult;
	Ctx *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			auto result = std::make_unique<Ctx>();
			result->pub.refcnt_minus_one = 0;
			result->device_id = device_id;

			if (!hip_initialized.load(std::memory_order_acquire)) [[unlikely]] {
				std::lock_guard<std::mutex> lock(hip_init_mutex);
				if (!hip_initialized.load(std::memory_order_relaxed)) {
					X17_HIP_CHECK("x17ai_hip_open_context()", "hipInit()", hipInit(0));
					hip_initialized.store(true, std::memory_order_release);
				}
			}
			if (!fits_int(device_id)) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_open_context(): HIP device ID out of range");
			}
			int count = 0;
			X17_HIP_CHECK("x17ai_hip_open_context()", "hipGetDeviceCount()", hipGetDeviceCount(&count));
			if (int(device_id) >= count) [[unlikely]] {
				return X17_DIAG(
					"x17ai_hip_open_context(): no such HIP device.",
					"x17ai_hip_open_context(): no such HIP device: ", std::to_string(device_id),
					" (device count ", std::to_string(count), ")"
				);
			}
			result->device = int(device_id);

			int major = 0, minor = 0, wave = 0;
			X17_HIP_CHECK("x17ai_hip_open_context()", "hipDeviceGetAttribute(MAJOR)",
				hipDeviceGetAttribute(&major, hipDeviceAttributeComputeCapabilityMajor, result->device));
			X17_HIP_CHECK("x17ai_hip_open_context()", "hipDeviceGetAttribute(MINOR)",
				hipDeviceGetAttribute(&minor, hipDeviceAttributeComputeCapabilityMinor, result->device));
			X17_HIP_CHECK("x17ai_hip_open_context()", "hipDeviceGetAttribute(WARP_SIZE)",
				hipDeviceGetAttribute(&wave, hipDeviceAttributeWarpSize, result->device));
			if (major < 0 || minor < 0 || wave <= 0) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_open_context(): device attributes out of range");
			}
			result->arch_major = size_t(major);
			result->arch_minor = size_t(minor);
			result->wavefront_size = size_t(wave);
			if (!std::has_single_bit(result->wavefront_size)) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_open_context(): wavefront size is not a power of two");
			}
			{
				// Touch the device once so that later calls find its primary state ready.
				DeviceScope scope(result->device);
				X17_HIP_CHECK("x17ai_hip_open_context()", "hipSetDevice()", scope.error);
				X17_HIP_CHECK("x17ai_hip_open_context()", "hipFree(nullptr)", hipFree(nullptr));
			}
			out = result.release();
			return nullptr;
		} X17_CATCH("x17ai_hip_open_context()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(&out->pub);
}

X17DiagnosticBuffer *x17ai_hip_close_context(X17HipContextHandle *context) {
	try {
		assert(context != nullptr);
		if (context->refcnt_minus_one > 0) {
			--context->refcnt_minus_one;
			return nullptr;
		}
		delete reinterpret_cast<Ctx *>(context);
		return nullptr;
	} X17_CATCH("x17ai_hip_close_context()")
}

void *x17ai_hip_context_ptr(X17HipContextHandle *context) {
	assert(context != nullptr);
	// There is no driver context object; the device ordinal (+1, so that it is never NULL)
	// identifies the device the way the CUcontext pointer does for the reference.
	return reinterpret_cast<void *>(uintptr_t(reinterpret_cast<Ctx *>(context)->device) + 1);
}

X17StreamResult x17ai_hip_open_stream(X17HipContextHandle *context) {
	using R = X17StreamResult;
	Stream *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			assert(context != nullptr);
			Ctx *ctx = reinterpret_cast<Ctx *>(context);
			DeviceScope scope(ctx->device);
			X17_HIP_CHECK("x17ai_hip_open_stream()", "hipSetDevice()", scope.error);
			auto result = std::make_unique<Stream>();
			result->device = ctx->device;
			result->stream = nullptr;
			// default priority on purpose; only the non-blocking flag mirrors the reference
			X17_HIP_CHECK("x17ai_hip_open_stream()", "hipStreamCreateWithFlags()",
				hipStreamCreateWithFlags(&result->stream, hipStreamNonBlocking));
			if (result->stream == nullptr) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_open_stream(): hipStreamCreateWithFlags() returned nullptr");
			}
			out = result.release();
			return nullptr;
		} X17_CATCH("x17ai_hip_open_stream()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(reinterpret_cast<X17HipStreamHandle *>(out));
}

X17DiagnosticBuffer *x17ai_hip_close_stream(X17HipStreamHandle *stream_c) {
	try {
		assert(stream_c != nullptr);
		auto stream = std::unique_ptr<Stream>(reinterpret_cast<Stream *>(stream_c));
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_close_stream()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_close_stream()", "hipStreamDestroy()", hipStreamDestroy(stream->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_close_stream()")
}

X17DiagnosticBuffer *x17ai_hip_synchronize(X17HipStreamHandle *stream_c) {
	try {
		assert(stream_c != nullptr);
		Stream *stream = reinterpret_cast<Stream *>(stream_c);
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_synchronize()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_synchronize()", "hipStreamSynchronize()", hipStreamSynchronize(stream->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_synchronize()")
}

X17TimerResult x17ai_hip_create_timer(X17HipContextHandle *context, X17HipStreamHandle *stream_c) {
	using R = X17TimerResult;
	Timer *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			assert(context != nullptr);
			assert(stream_c != nullptr);
			Ctx *ctx = reinterpret_cast<Ctx *>(context);
			Stream *stream = reinterpret_cast<Stream *>(stream_c);
			if (ctx->device != stream->device) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_create_timer(): stream belongs to another device");
			}
			DeviceScope scope(ctx->device);
			X17_HIP_CHECK("x17ai_hip_create_timer()", "hipSetDevice()", scope.error);
			auto result = std::make_unique<Timer>();
			result->device = ctx->device;
			result->stream = stream->stream;
			result->start = nullptr;
			result->end = nullptr;
			X17_HIP_CHECK("x17ai_hip_create_timer()", "hipEventCreate(start)", hipEventCreate(&result->start));
			hipError_t e = hipEventCreate(&result->end);
			if (e != hipSuccess) [[unlikely]] {
				(void)hipEventDestroy(result->start);
				return X17_DIAG(
					"x17ai_hip_create_timer(): hipEventCreate(end) failed.",
					"x17ai_hip_create_timer(): hipEventCreate(end) failed with hip error: ", e
				);
			}
			out = result.release();
			return nullptr;
		} X17_CATCH("x17ai_hip_create_timer()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(reinterpret_cast<X17HipTimerHandle *>(out));
}

X17DiagnosticBuffer *x17ai_hip_destroy_timer(X17HipTimerHandle *timer_c) {
	try {
		assert(timer_c != nullptr);
		auto timer = std::unique_ptr<Timer>(reinterpret_cast<Timer *>(timer_c));
		DeviceScope scope(timer->device);
		X17_HIP_CHECK("x17ai_hip_destroy_timer()", "hipSetDevice()", scope.error);
		X17DiagnosticBuffer *diag = nullptr;
		if (timer->end != nullptr) {
			hipError_t e = hipEventDestroy(timer->end);
			timer->end = nullptr;
			if (e != hipSuccess) [[unlikely]] {
				diag = X17_DIAG(
					"x17ai_hip_destroy_timer(): hipEventDestroy(end) failed.",
					"x17ai_hip_destroy_timer(): hipEventDestroy(end) failed with hip error: ", e
				);
			}
		}
		if (timer->start != nullptr) {
			hipError_t e = hipEventDestroy(timer->start);
			timer->start = nullptr;
			if (e != hipSuccess && diag == nullptr) [[unlikely]] {
				diag = X17_DIAG(
					"x17ai_hip_destroy_timer(): hipEventDestroy(start) failed.",
					"x17ai_hip_destroy_timer(): hipEventDestroy(start) failed with hip error: ", e
				);
			}
		}
		return diag;
	} X17_CATCH("x17ai_hip_destroy_timer()")
}

X17DiagnosticBuffer *x17ai_hip_timer_start(X17HipTimerHandle *timer_c) {
	try {
		assert(timer_c != nullptr);
		Timer *timer = reinterpret_cast<Timer *>(timer_c);
		DeviceScope scope(timer->device);
		X17_HIP_CHECK("x17ai_hip_timer_start()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_timer_start()", "hipEventRecord()", hipEventRecord(timer->start, timer->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_timer_start()")
}

X17DiagnosticBuffer *x17ai_hip_timer_stop(X17HipTimerHandle *timer_c) {
	try {
		assert(timer_c != nullptr);
		Timer *timer = reinterpret_cast<Timer *>(timer_c);
		DeviceScope scope(timer->device);
		X17_HIP_CHECK("x17ai_hip_timer_stop()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_timer_stop()", "hipEventRecord()", hipEventRecord(timer->end, timer->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_timer_stop()")
}

X17DiagnosticBuffer *x17ai_hip_timer_elapsed_seconds(X17HipTimerHandle *timer_c, double *seconds) {
	try {
		assert(timer_c != nullptr);
		assert(seconds != nullptr);
		Timer *timer = reinterpret_cast<Timer *>(timer_c);
		DeviceScope scope(timer->device);
		X17_HIP_CHECK("x17ai_hip_timer_elapsed_seconds()", "hipSetDevice()", scope.error);
		float ms = 0.0f;
		X17_HIP_CHECK("x17ai_hip_timer_elapsed_seconds()", "hipEventElapsedTime()",
			hipEventElapsedTime(&ms, timer->start, timer->end));
		*seconds = double(ms) / 1000.0;
		return nullptr;
	} X17_CATCH("x17ai_hip_timer_elapsed_seconds()")
}

X17DeviceDataResult x17ai_hip_alloc(X17HipStreamHandle *stream_c, size_t bytes) {
	using R = X17DeviceDataResult;
	void *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			assert(stream_c != nullptr);
			Stream *stream = reinterpret_cast<Stream *>(stream_c);
			DeviceScope scope(stream->device);
			X17_HIP_CHECK("x17ai_hip_alloc()", "hipSetDevice()", scope.error);
			void *memory = nullptr;
			X17_HIP_CHECK("x17ai_hip_alloc()", "hipMallocAsync()", hipMallocAsync(&memory, bytes, stream->stream));
			if (memory == nullptr) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_alloc(): hipMallocAsync() returned null pointer");
			}
			out = memory;
			return nullptr;
		} X17_CATCH("x17ai_hip_alloc()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(reinterpret_cast<X17HipDeviceData *>(out));
}

X17DiagnosticBuffer *x17ai_hip_free(X17HipStreamHandle *stream_c, X17HipDeviceData *ptr) {
	try {
		assert(stream_c != nullptr);
		Stream *stream = reinterpret_cast<Stream *>(stream_c);
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_free()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_free()", "hipFreeAsync()", hipFreeAsync(reinterpret_cast<void *>(ptr), stream->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_free()")
}

X17DiagnosticBuffer *x17ai_hip_upload_data(
	X17HipStreamHandle *stream_c, uint8_t const *src, X17HipDeviceData *dst,
	size_t offset_bytes, size_t size_bytes
) {
	try {
		assert(stream_c != nullptr);
		assert(src != nullptr);
		Stream *stream = reinterpret_cast<Stream *>(stream_c);
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_upload_data()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_upload_data()", "hipMemcpyHtoDAsync()",
			hipMemcpyHtoDAsync(
				reinterpret_cast<hipDeviceptr_t>(reinterpret_cast<uint8_t *>(dst) + offset_bytes),
				const_cast<uint8_t *>(src), size_bytes, stream->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_upload_data()")
}

X17DiagnosticBuffer *x17ai_hip_download_data(
	X17HipStreamHandle *stream_c, X17HipDeviceData *src, uint8_t *dst,
	size_t offset_bytes, size_t size_bytes
) {
	try {
		assert(stream_c != nullptr);
		assert(dst != nullptr);
		Stream *stream = reinterpret_cast<Stream *>(stream_c);
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_download_data()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_download_data()", "hipMemcpyDtoHAsync()",
			hipMemcpyDtoHAsync(
				dst, reinterpret_cast<hipDeviceptr_t>(reinterpret_cast<uint8_t *>(src) + offset_bytes),
				size_bytes, stream->stream));
		return nullptr;
	} X17_CATCH("x17ai_hip_download_data()")
}

X17ModuleResult x17ai_hip_load_module(X17HipContextHandle *context, char const *code_object_path) {
	using R = X17ModuleResult;
	Module *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			assert(context != nullptr);
			assert(code_object_path != nullptr);
			Ctx *ctx = reinterpret_cast<Ctx *>(context);
			DeviceScope scope(ctx->device);
			X17_HIP_CHECK("x17ai_hip_load_module()", "hipSetDevice()", scope.error);
			auto result = std::make_unique<Module>();
			result->device = ctx->device;
			result->module = nullptr;
			{
				std::FILE *f = std::fopen(code_object_path, "rb");
				if (f == nullptr) [[unlikely]] {
					return X17_DIAG(
						"x17ai_hip_load_module(): cannot open the code object.",
						"x17ai_hip_load_module(): cannot open ", code_object_path
					);
				}
				char buf[65536];
				size_t got;
				while ((got = std::fread(buf, 1, sizeof buf, f)) > 0) result->image.insert(result->image.end(), buf, buf + got);
				bool const failed = std::ferror(f) != 0;
				std::fclose(f);
				if (failed || result->image.empty()) [[unlikely]] {
					return X17_DIAG(
						"x17ai_hip_load_module(): cannot read the code object.",
						"x17ai_hip_load_module(): cannot read ", code_object_path
					);
				}
			}
			hipError_t e = hipModuleLoadData(&result->module, result->image.data());
			if (e != hipSuccess) [[unlikely]] {
				return X17_DIAG(
					"x17ai_hip_load_module(): hipModuleLoadData() failed.",
					"x17ai_hip_load_module(): hipModuleLoadData(", code_object_path, ") failed with hip error: ", e
				);
			}
			if (result->module == nullptr) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_load_module(): hipModuleLoad() returned nullptr");
			}
			out = result.release();
			return nullptr;
		} X17_CATCH("x17ai_hip_load_module()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(reinterpret_cast<X17HipModuleHandle *>(out));
}

X17DiagnosticBuffer *x17ai_hip_del_module(X17HipModuleHandle *module_c) {
	try {
		assert(module_c != nullptr);
		auto module = std::unique_ptr<Module>(reinterpret_cast<Module *>(module_c));
		DeviceScope scope(module->device);
		X17_HIP_CHECK("x17ai_hip_del_module()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_del_module()", "hipModuleUnload()", hipModuleUnload(module->module));
		return nullptr;
	} X17_CATCH("x17ai_hip_del_module()")
}

X17KernelResult x17ai_hip_get_kernel(X17HipModuleHandle *module_c, char const *name, size_t smem_size) {
	using R = X17KernelResult;
	Kernel *out = nullptr;
	auto run = [&]() -> X17DiagnosticBuffer * {
		try {
			assert(module_c != nullptr);
			assert(name != nullptr);
			Module *module = reinterpret_cast<Module *>(module_c);
			DeviceScope scope(module->device);
			X17_HIP_CHECK("x17ai_hip_get_kernel()", "hipSetDevice()", scope.error);
			auto result = std::make_unique<Kernel>();
			result->device = module->device;
			result->function = nullptr;
			hipError_t e = hipModuleGetFunction(&result->function, module->module, name);
			if (e != hipSuccess) [[unlikely]] {
				return X17_DIAG(
					"x17ai_hip_get_kernel(): hipModuleGetFunction() failed.",
					"x17ai_hip_get_kernel(): hipModuleGetFunction(", name, ") failed with hip error: ", e
				);
			}
			if (result->function == nullptr) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_get_kernel(): hipModuleGetFunction() returned nullptr");
			}
			if (!fits_int(smem_size)) [[unlikely]] {
				return X17_STATIC_DIAG("x17ai_hip_get_kernel(): max dynamic shared memory size is out of range");
			}
			// The LDS a workgroup may ask for is bounded by the device, not by a per-function
			// opt-in as on CUDA; check the request here so that a launch cannot exceed it.
			int lds_per_block = 0;
			X17_HIP_CHECK("x17ai_hip_get_kernel()", "hipDeviceGetAttribute(MaxSharedMemoryPerBlock)",
				hipDeviceGetAttribute(&lds_per_block, hipDeviceAttributeMaxSharedMemoryPerBlock, module->device));
			int static_lds = 0;
			(void)hipFuncGetAttribute(&static_lds, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, result->function);
			if (smem_size + size_t(static_lds > 0 ? static_lds : 0) > size_t(lds_per_block)) [[unlikely]] {
				return X17_DIAG(
					"x17ai_hip_get_kernel(): requested shared memory exceeds the device limit.",
					"x17ai_hip_get_kernel(): requested ", std::to_string(smem_size), " dynamic + ",
					std::to_string(static_lds), " static LDS bytes, device allows ", std::to_string(lds_per_block)
				);
			}
			result->max_dynamic_smem = smem_size;
			out = result.get();
			module->kernels.push_back(std::move(result));
			return nullptr;
		} X17_CATCH("x17ai_hip_get_kernel()")
	};
	X17DiagnosticBuffer *d = run();
	return d != nullptr ? fail<R>(d) : ok<R>(reinterpret_cast<X17HipKernelHandle *>(out));
}

X17DiagnosticBuffer *x17ai_hip_read_kernel_attrs(X17HipKernelHandle *kernel_c, X17HipKernelAttrs *attrs) {
	try {
		assert(kernel_c != nullptr);
		assert(attrs != nullptr);
		Kernel *kernel = reinterpret_cast<Kernel *>(kernel_c);
		DeviceScope scope(kernel->device);
		X17_HIP_CHECK("x17ai_hip_read_kernel_attrs()", "hipSetDevice()", scope.error);
		X17HipKernelAttrs r{};
		struct { hipFunction_attribute attr; char const *name; int32_t *dst; } const wanted[] = {
			{HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, "MAX_THREADS_PER_BLOCK", &r.max_threads_per_block},
			{HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, "SHARED_SIZE_BYTES", &r.static_shared_size_bytes},
			{HIP_FUNC_ATTRIBUTE_CONST_SIZE_BYTES, "CONST_SIZE_BYTES", &r.const_size_bytes},
			{HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, "LOCAL_SIZE_BYTES", &r.local_size_bytes},
			{HIP_FUNC_ATTRIBUTE_NUM_REGS, "NUM_REGS", &r.num_regs},
			{HIP_FUNC_ATTRIBUTE_PTX_VERSION, "PTX_VERSION", &r.ptx_version},
			{HIP_FUNC_ATTRIBUTE_BINARY_VERSION, "BINARY_VERSION", &r.binary_version},
		};
		for (auto const &w : wanted) {
			int value = 0;
			hipError_t e = hipFuncGetAttribute(&value, w.attr, kernel->function);
			if (e != hipSuccess) [[unlikely]] {
				return X17_DIAG(
					"x17ai_hip_read_kernel_attrs(): hipFuncGetAttribute() failed.",
					"x17ai_hip_read_kernel_attrs(): hipFuncGetAttribute(", w.name, ") failed with hip error: ", e
				);
			}
			*w.dst = value;
		}
		r.max_dynamic_shared_size_bytes = int32_t(kernel->max_dynamic_smem);
		r.preferred_shared_memory_carveout = 100;   // LDS is not carved out of a shared cache on CDNA
		*attrs = r;
		return nullptr;
	} X17_CATCH("x17ai_hip_read_kernel_attrs()")
}

X17DiagnosticBuffer *x17ai_hip_launch_kernel(
	X17HipStreamHandle *stream_c, X17HipKernelHandle *kernel_c,
	size_t grid_x, size_t grid_y, size_t grid_z,
	size_t block_x, size_t block_y, size_t block_z,
	size_t shared_mem_bytes, void **args
) {
	try {
		assert(stream_c != nullptr);
		assert(kernel_c != nullptr);
		Stream *stream = reinterpret_cast<Stream *>(stream_c);
		Kernel *kernel = reinterpret_cast<Kernel *>(kernel_c);
		if (
			(grid_x < 1 || !fits_u32(grid_x))
			|| (grid_y < 1 || !fits_u32(grid_y))
			|| (grid_z < 1 || !fits_u32(grid_z))
		) [[unlikely]] {
			return X17_STATIC_DIAG("x17ai_hip_launch_kernel(): grid dimensions are out of range");
		}
		if (
			(block_x < 1 || !fits_u32(block_x))
			|| (block_y < 1 || !fits_u32(block_y))
			|| (block_z < 1 || !fits_u32(block_z))
		) [[unlikely]] {
			return X17_STATIC_DIAG("x17ai_hip_launch_kernel(): block dimensions are out of range");
		}
		if (!fits_u32(shared_mem_bytes)) [[unlikely]] {
			return X17_STATIC_DIAG("x17ai_hip_launch_kernel(): shared memory size is out of range");
		}
		if (shared_mem_bytes > kernel->max_dynamic_smem) [[unlikely]] {
			return X17_STATIC_DIAG(
				"x17ai_hip_launch_kernel(): shared memory size exceeds what x17ai_hip_get_kernel() was told"
			);
		}
		if (stream->device != kernel->device) [[unlikely]] {
			return X17_STATIC_DIAG("x17ai_hip_launch_kernel(): stream and kernel belong to different devices");
		}
		DeviceScope scope(stream->device);
		X17_HIP_CHECK("x17ai_hip_launch_kernel()", "hipSetDevice()", scope.error);
		X17_HIP_CHECK("x17ai_hip_launch_kernel()", "hipModuleLaunchKernel()",
			hipModuleLaunchKernel(
				kernel->function,
				uint32_t(grid_x), uint32_t(grid_y), uint32_t(grid_z),
				uint32_t(block_x), uint32_t(block_y), uint32_t(block_z),
				uint32_t(shared_mem_bytes), stream->stream, args, nullptr));
		return nullptr;
	} X17_CATCH("x17ai_hip_launch_kernel()")
}

} // extern "C"
