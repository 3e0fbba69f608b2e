// x17ai_host.cpp -- implementation of the host-side operator layer (see x17ai_host.hpp for
// the map from each type here to the reference's Rust source) and of its flat C ABI
// (include/x17ai_host.h).

#include "x17ai_host.hpp"
#include <filesystem>
#include "../../../include/x17ai_host.h"

#include <dlfcn.h>
#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <cmath>
#include <algorithm>
#include <cstdio>
#include <functional>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

namespace x17 {

// ================================================================ FfiBuffer (src/util/ffi_buffer.rs)

namespace {
	X17FfiSpan fb_span(void *self) {
		auto *b = static_cast<FfiBufferImpl *>(self);
		return X17FfiSpan{b->data.data(), b->data.size()};
	}
	X17FfiSpan fb_buf_span(void *self) {
		auto *b = static_cast<FfiBufferImpl *>(self);
		return X17FfiSpan{b->data.data(), b->data.capacity()};
	}
	X17FfiSpan fb_extend(void *self, size_t additional) {
		auto *b = static_cast<FfiBufferImpl *>(self);
		size_t old = b->data.size();
		try {
			b->data.resize(old + additional);
		} catch (...) {
			return X17FfiSpan{nullptr, 0};
		}
		return X17FfiSpan{b->data.data() + old, additional};
	}
	void fb_clear(void *self) { static_cast<FfiBufferImpl *>(self)->data.clear(); }
	void fb_set_len(void *self, size_t n) {
		auto *b = static_cast<FfiBufferImpl *>(self);
		if (n <= b->data.capacity()) b->data.resize(n);
	}
	X17FfiBufferVMT const FB_VMT = {fb_span, fb_buf_span, fb_extend, fb_clear, fb_set_len};
}

X17FfiBuffer FfiBufferImpl::as_ffi() { return X17FfiBuffer{this, &FB_VMT}; }

// cuda_shim.rs:176-188
std::string diagnostic_to_string(X17DiagnosticBuffer *diag, char const *fallback) {
	FfiBufferImpl buf;
	x17ai_move_diagnostic(diag, buf.as_ffi());
	return buf.data.empty() ? std::string(fallback) : buf.data;
}

static ErrPack device_error(X17DiagnosticBuffer *diag) {
	return ErrPack{TensorOpError::Device, diagnostic_to_string(diag, "HIP operation failed without diagnostic"), nullptr};
}

static void discard_diagnostic(X17DiagnosticBuffer *diag) {
	if (diag != nullptr) {
		FfiBufferImpl buf;
		x17ai_move_diagnostic(diag, buf.as_ffi());
	}
}

// ================================================================ dtype (src/dtype.rs)

size_t dtype_bytes(DType d) {
	switch (d) {
		case DType::E4m3: return 1;
		case DType::Int8: return 1;
		case DType::Bf16: return 2;
		case DType::F32: return 4;
	}
	return 0;
}

char const *dtype_name(DType d) {
	switch (d) {
		case DType::E4m3: return "e4m3";
		case DType::Int8: return "i8";
		case DType::Bf16: return "bf16";
		case DType::F32: return "f32";
	}
	return "?";
}

// ================================================================ devices

Result<DevicePtr> CpuDevice::new_buffer(size_t bytes) {
	void *p = std::malloc(bytes == 0 ? 1 : bytes);
	if (p == nullptr) return Result<DevicePtr>::err(ErrPack{TensorOpError::Alloc, "host allocation failed", nullptr});
	return Result<DevicePtr>::ok(p);
}
void CpuDevice::drop_buffer(DevicePtr p, size_t) { std::free(p); }
Status CpuDevice::upload_data(uint8_t const *src, DevicePtr dst, size_t bytes) { std::memcpy(dst, src, bytes); return Status::ok(); }
Status CpuDevice::download_data(DevicePtr src, uint8_t *dst, size_t bytes) { std::memcpy(dst, src, bytes); return Status::ok(); }

// cuda_shim.rs:215-237
Result<std::unique_ptr<HipStream>> HipStream::create(size_t device_id) {
	using R = Result<std::unique_ptr<HipStream>>;
	X17ContextResult c = x17ai_hip_open_context(device_id);
	if (c.value == nullptr) return R::err(device_error(c.diagnostic));
	X17StreamResult s = x17ai_hip_open_stream(c.value);
	if (s.value == nullptr) {
		ErrPack e = device_error(s.diagnostic);
		discard_diagnostic(x17ai_hip_close_context(c.value));
		return R::err(std::move(e));
	}
	auto out = std::make_unique<HipStream>();
	out->ctx = c.value;
	out->stream = s.value;
	return R::ok(std::move(out));
}

HipStream::~HipStream() {
	if (stream != nullptr) discard_diagnostic(x17ai_hip_close_stream(stream));
	if (ctx != nullptr) discard_diagnostic(x17ai_hip_close_context(ctx));
}

Status HipStream::synchronize() {
	X17DiagnosticBuffer *d = x17ai_hip_synchronize(stream);
	return d == nullptr ? Status::ok() : Status::err(device_error(d));
}

HipModule::~HipModule() {
	if (module != nullptr) discard_diagnostic(x17ai_hip_del_module(module));
}

HipKernel::~HipKernel() {}

// cuda_shim.rs:464-489
Status HipKernel::launch(HipStream &s, size_t const (&grid)[3], size_t const (&block)[3], size_t smem, void **args) {
	X17DiagnosticBuffer *d = x17ai_hip_launch_kernel(
		s.stream, kernel, grid[0], grid[1], grid[2], block[0], block[1], block[2], smem, args);
	return d == nullptr ? Status::ok() : Status::err(device_error(d));
}

Result<X17HipKernelAttrs> HipKernel::attrs() {
	X17HipKernelAttrs a{};
	X17DiagnosticBuffer *d = x17ai_hip_read_kernel_attrs(kernel, &a);
	if (d != nullptr) return Result<X17HipKernelAttrs>::err(device_error(d));
	return Result<X17HipKernelAttrs>::ok(a);
}

// src/device/cuda.rs:31-38
Result<std::shared_ptr<HipDevice>> HipDevice::create(size_t device_id) {
	using R = Result<std::shared_ptr<HipDevice>>;
	auto s = HipStream::create(device_id);
	if (!s.is_ok()) return R::err(*s.error);
	auto dev = std::make_shared<HipDevice>();
	dev->name_ = "HIP:" + std::to_string(device_id);
	dev->stream = std::move(*s.value);
	return R::ok(std::move(dev));
}

Result<DevicePtr> HipDevice::new_buffer(size_t bytes) {
	X17DeviceDataResult r = x17ai_hip_alloc(stream->stream, bytes);
	if (r.value == nullptr) {
		ErrPack e = device_error(r.diagnostic);
		e.code = TensorOpError::Alloc;
		return Result<DevicePtr>::err(std::move(e));
	}
	return Result<DevicePtr>::ok(static_cast<void *>(r.value));
}

void HipDevice::drop_buffer(DevicePtr p, size_t) {
	discard_diagnostic(x17ai_hip_free(stream->stream, static_cast<X17HipDeviceData *>(p)));
}

Status HipDevice::upload_data(uint8_t const *src, DevicePtr dst, size_t bytes) {
	X17DiagnosticBuffer *d = x17ai_hip_upload_data(stream->stream, src, static_cast<X17HipDeviceData *>(dst), 0, bytes);
	return d == nullptr ? Status::ok() : Status::err(device_error(d));
}

Status HipDevice::download_data(DevicePtr src, uint8_t *dst, size_t bytes) {
	X17DiagnosticBuffer *d = x17ai_hip_download_data(stream->stream, static_cast<X17HipDeviceData *>(src), dst, 0, bytes);
	return d == nullptr ? Status::ok() : Status::err(device_error(d));
}

Result<std::unique_ptr<HipTimer>> HipTimer::create(HipDevice &device) {
	using R = Result<std::unique_ptr<HipTimer>>;
	X17TimerResult r = x17ai_hip_create_timer(device.stream->ctx, device.stream->stream);
	if (r.value == nullptr) return R::err(device_error(r.diagnostic));
	auto t = std::make_unique<HipTimer>();
	t->timer = r.value;
	return R::ok(std::move(t));
}
HipTimer::~HipTimer() { if (timer != nullptr) discard_diagnostic(x17ai_hip_destroy_timer(timer)); }
Status HipTimer::start() { auto *d = x17ai_hip_timer_start(timer); return d == nullptr ? Status::ok() : Status::err(device_error(d)); }
Status HipTimer::stop() { auto *d = x17ai_hip_timer_stop(timer); return d == nullptr ? Status::ok() : Status::err(device_error(d)); }
Result<double> HipTimer::elapsed_seconds() {
	double s = 0.0;
	auto *d = x17ai_hip_timer_elapsed_seconds(timer, &s);
	if (d != nullptr) return Result<double>::err(device_error(d));
	return Result<double>::ok(s);
}

// ================================================================ tensor (src/tensor.rs)

size_t Tensor::elems() const {
	size_t n = 1;
	for (size_t d : shape) n *= d;
	return n;
}

Result<std::shared_ptr<Tensor>> Tensor::new_empty(std::vector<size_t> shape, DType dtype, std::shared_ptr<Device> device) {
	using R = Result<std::shared_ptr<Tensor>>;
	size_t n = 1;
	for (size_t d : shape) {
		if (d != 0 && n > SIZE_MAX / d) return R::err(ErrPack{TensorOpError::Other, "tensor shape overflows usize", nullptr});
		n *= d;
	}
	if (n > SIZE_MAX / dtype_bytes(dtype)) return R::err(ErrPack{TensorOpError::Other, "tensor size in bytes overflows usize", nullptr});
	size_t bytes = n * dtype_bytes(dtype);
	auto buf = device->new_buffer(bytes);
	if (!buf.is_ok()) return R::err(*buf.error);
	auto t = std::make_shared<Tensor>();
	t->dtype = dtype;
	t->shape = std::move(shape);
	t->ptr = *buf.value;
	t->bytes = bytes;
	t->device = std::move(device);
	return R::ok(std::move(t));
}

// ---- safetensors: u64 little-endian header length, a JSON header {name: {dtype, shape, data_offsets}, ...,
// "__metadata__": {...}}, then the tensor bytes.  The header parser below reads just that shape of JSON.
namespace {
struct StEntry { std::string name, dtype; std::vector<size_t> shape; size_t begin = 0, end = 0; };

struct StParser {
	std::string const &s;
	size_t i = 0;
	explicit StParser(std::string const &text): s(text) {}
	void ws() { while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i; }
	bool eat(char c) { ws(); if (i < s.size() && s[i] == c) { ++i; return true; } return false; }
	bool string(std::string &out) {
		ws();
		if (i >= s.size() || s[i] != '"') return false;
		++i;
		out.clear();
		while (i < s.size() && s[i] != '"') {
			if (s[i] == '\\' && i + 1 < s.size()) { ++i; }
			out.push_back(s[i++]);
		}
		return i < s.size() && s[i++] == '"';
	}
	bool number(size_t &out) {
		ws();
		if (i >= s.size() || s[i] < '0' || s[i] > '9') return false;
		out = 0;
		while (i < s.size() && s[i] >= '0' && s[i] <= '9') out = out * 10 + size_t(s[i++] - '0');
		return true;
	}
	bool numbers(std::vector<size_t> &out) {
		if (!eat('[')) return false;
		out.clear();
		if (eat(']')) return true;
		do { size_t v; if (!number(v)) return false; out.push_back(v); } while (eat(','));
		return eat(']');
	}
	// skips any JSON value (used for "__metadata__" and unknown keys)
	bool skip() {
		ws();
		if (i >= s.size()) return false;
		if (s[i] == '"') { std::string t; return string(t); }
		if (s[i] == '{' || s[i] == '[') {
			char open = s[i], close = open == '{' ? '}' : ']';
			++i;
			if (eat(close)) return true;
			do {
				if (open == '{') { std::string k; if (!string(k) || !eat(':')) return false; }
				if (!skip()) return false;
			} while (eat(','));
			return eat(close);
		}
		while (i < s.size() && s[i] != ',' && s[i] != '}' && s[i] != ']') ++i;
		return true;
	}
	bool entry(StEntry &e) {
		if (!eat('{')) return false;
		do {
			std::string key;
			if (!string(key) || !eat(':')) return false;
			if (key == "dtype") { if (!string(e.dtype)) return false; }
			else if (key == "shape") { if (!numbers(e.shape)) return false; }
			else if (key == "data_offsets") {
				std::vector<size_t> o;
				if (!numbers(o) || o.size() != 2) return false;
				e.begin = o[0]; e.end = o[1];
			} else if (!skip()) return false;
		} while (eat(','));
		return eat('}');
	}
	bool header(std::vector<StEntry> &out) {
		if (!eat('{')) return false;
		if (eat('}')) return true;
		do {
			std::string name;
			if (!string(name) || !eat(':')) return false;
			if (name == "__metadata__") { if (!skip()) return false; continue; }
			StEntry e;
			e.name = name;
			if (!entry(e)) return false;
			out.push_back(std::move(e));
		} while (eat(','));
		return eat('}');
	}
};

char const *st_dtype_name(DType d) {      // src/dtype.rs:26-36
	switch (d) {
		case DType::E4m3: return "F8_E4M3";
		case DType::Int8: return "I8";
		case DType::Bf16: return "BF16";
		case DType::F32: return "F32";
	}
	return "?";
}
} // namespace

Result<std::shared_ptr<Tensor>> Tensor::from_safetensors_file(std::string const &path, std::shared_ptr<Device> device) {
	using R = Result<std::shared_ptr<Tensor>>;
	auto bad = [&](std::string const &why) { return R::err(ErrPack{TensorOpError::Io, "invalid safetensors file " + path + ": " + why, nullptr}); };
	std::ifstream f(path, std::ios::binary);
	if (!f) return R::err(ErrPack{TensorOpError::Io, "cannot open " + path, nullptr});
	unsigned char len8[8];
	if (!f.read(reinterpret_cast<char *>(len8), 8)) return bad("shorter than its length field");
	uint64_t n = 0;
	for (int b = 7; b >= 0; --b) n = (n << 8) | len8[b];
	if (n > (uint64_t(1) << 27)) return bad("header length " + std::to_string(n));
	std::string header(size_t(n), '\0');
	if (!f.read(header.data(), std::streamsize(n))) return bad("truncated header");
	std::vector<StEntry> entries;
	StParser p(header);
	if (!p.header(entries)) return bad("header is not the expected JSON");
	if (entries.size() != 1) return bad("expected exactly one tensor, found " + std::to_string(entries.size()));   // tensor.rs:164-177
	StEntry const &e = entries[0];
	DType dtype;
	if (e.dtype == "F8_E4M3") dtype = DType::E4m3;
	else if (e.dtype == "I8") dtype = DType::Int8;
	else if (e.dtype == "BF16") dtype = DType::Bf16;
	else if (e.dtype == "F32") dtype = DType::F32;
	else return R::err(ErrPack{TensorOpError::Other, "unsupported dtype " + e.dtype + " in " + path, nullptr});   // dtype.rs:38-50
	// shape, data_offsets and the file size are checked against each other before anything is allocated
	size_t want = dtype_bytes(dtype);
	for (size_t d : e.shape) {
		if (d != 0 && want > SIZE_MAX / d) return bad("shape overflows usize");
		want *= d;
	}
	if (e.end < e.begin || e.end - e.begin != want) return bad("data_offsets do not match dtype and shape");
	f.seekg(0, std::ios::end);
	uint64_t const file_size = uint64_t(f.tellg());
	if (file_size < 8 + n || file_size - (8 + n) < e.end) return bad("truncated tensor data");
	auto t = Tensor::new_empty(e.shape, dtype, std::move(device));
	if (!t.is_ok()) return t;
	std::vector<char> data((*t.value)->bytes);
	f.seekg(std::streamoff(8 + n + e.begin));
	if (!data.empty() && !f.read(data.data(), std::streamsize(data.size()))) return bad("truncated tensor data");
	Status up = (*t.value)->device->upload_data(reinterpret_cast<uint8_t const *>(data.data()), (*t.value)->ptr, data.size());
	if (!up.is_ok()) return R::err(*up.error);
	// the staging buffer dies here: make sure an asynchronous copy has consumed it
	if (auto *hip = dynamic_cast<HipDevice *>((*t.value)->device.get())) {
		Status sy = hip->synchronize();
		if (!sy.is_ok()) return R::err(*sy.error);
	}
	return t;
}

Status Tensor::save_safetensors_file(std::string const &path) const {
	if (!device || !device->is_cpu()) {
		return Status::err(TensorOpError::Device, "save_safetensors_file requires a CPU tensor; download it first");   // tensor.rs:230-235
	}
	std::error_code ec;
	std::filesystem::path fp(path);
	if (fp.has_parent_path()) {
		std::filesystem::create_directories(fp.parent_path(), ec);
		if (ec) return Status::err(TensorOpError::Io, "failed to create tensor output directory " + fp.parent_path().string() + ": " + ec.message());
	}
	std::string header = "{\"tensor\":{\"dtype\":\"" + std::string(st_dtype_name(dtype)) + "\",\"shape\":[";
	for (size_t i = 0; i < shape.size(); ++i) header += (i ? "," : "") + std::to_string(shape[i]);
	header += "],\"data_offsets\":[0," + std::to_string(bytes) + "]}}";
	while (header.size() % 8 != 0) header.push_back(' ');          // the format pads the header to 8 bytes with spaces
	std::ofstream f(path, std::ios::binary | std::ios::trunc);
	if (!f) return Status::err(TensorOpError::Io, "cannot create " + path);
	uint64_t n = header.size();
	unsigned char len8[8];
	for (int b = 0; b < 8; ++b) len8[b] = (unsigned char)(n >> (8 * b));
	f.write(reinterpret_cast<char const *>(len8), 8);
	f.write(header.data(), std::streamsize(header.size()));
	if (bytes != 0) f.write(static_cast<char const *>(ptr), std::streamsize(bytes));
	if (!f) return Status::err(TensorOpError::Io, "failed to write " + path);
	return Status::ok();
}

Tensor::~Tensor() {
	if (ptr != nullptr && device) device->drop_buffer(ptr, bytes);
}

// ================================================================ tensor_check (src/device/cuda/tensor_check.rs)

namespace tensor_check {
	static std::string shape_str(std::vector<size_t> const &s) {
		std::string out = "[";
		for (size_t i = 0; i < s.size(); ++i) { if (i) out += ", "; out += std::to_string(s[i]); }
		return out + "]";
	}

	static Status dtype_and_device(char const *op, char const *name, Tensor const &t, HipDevice const &dev, DType dtype) {
		if (t.dtype != dtype) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " has dtype " + dtype_name(t.dtype)
				+ ", but should have " + dtype_name(dtype));
		}
		if (!t.is_on_device(&dev)) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " is not on device " + dev.name());
		}
		return Status::ok();
	}

	// tensor_check.rs:19-56; expected < 0 means "any"
	static Status matrix_shape(char const *op, char const *name, Tensor const &t, std::optional<size_t> rows_exp,
	                           std::optional<size_t> cols_exp, HipDevice const &dev, DType dtype, size_t (&out)[2]) {
		if (t.shape.size() != 2) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " must be 2D, got shape " + shape_str(t.shape));
		}
		size_t rows = t.shape[0], cols = t.shape[1];
		if (rows == 0 || cols == 0) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " has zero size " + shape_str(t.shape));
		}
		if (rows_exp && rows != *rows_exp) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " has " + std::to_string(rows)
				+ " rows, but should have " + std::to_string(*rows_exp));
		}
		if (cols_exp && cols != *cols_exp) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " has " + std::to_string(cols)
				+ " columns, but should have " + std::to_string(*cols_exp));
		}
		Status s = dtype_and_device(op, name, t, dev, dtype);
		if (!s.is_ok()) return s;
		out[0] = rows;
		out[1] = cols;
		return Status::ok();
	}

	// tensor_check.rs:58-78
	static Status vector_shape(char const *op, char const *name, Tensor const &t, size_t len, HipDevice const &dev, DType dtype) {
		bool ok = (t.shape.size() == 1 && t.shape[0] == len) || (t.shape.size() == 2 && t.shape[0] == len && t.shape[1] == 1);
		if (!ok) {
			return Status::err(TensorOpError::Other, std::string(op) + " input " + name + " must have shape [" + std::to_string(len)
				+ "] or [" + std::to_string(len) + ", 1], got " + shape_str(t.shape));
		}
		return dtype_and_device(op, name, t, dev, dtype);
	}
}

// ================================================================ kernel_build (src/device/cuda/kernel_build.rs)

namespace kernel_build {
	static std::string lib_dir() {
		Dl_info info{};
		if (dladdr(reinterpret_cast<void *>(&lib_dir), &info) != 0 && info.dli_fname != nullptr) {
			std::string p = info.dli_fname;
			size_t slash = p.rfind('/');
			if (slash != std::string::npos) return p.substr(0, slash);
		}
		return ".";
	}

	std::string kernels_dir() {
		if (char const *e = std::getenv("X17AI_KERNELS_DIR")) return e;
		return lib_dir() + "/../csrc/kernels";
	}

	std::string cache_dir() {
		if (char const *e = std::getenv("X17AI_KERNEL_CACHE")) return e;
		return lib_dir() + "/../cache/kernels";
	}

	static bool read_file(std::string const &path, std::string &out) {
		std::ifstream f(path, std::ios::binary);
		if (!f) return false;
		std::stringstream ss;
		ss << f.rdbuf();
		out = ss.str();
		return true;
	}

	static bool write_file(std::string const &path, std::string const &text, Diagnostics &diag) {
		std::string tmp = path + ".tmp." + std::to_string(getpid());
		{
			std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
			if (!f) { diag.add_error("failed to write generated file " + path); return false; }
			f << text;
		}
		if (std::rename(tmp.c_str(), path.c_str()) != 0) {
			diag.add_error("failed to move generated file into place: " + path);
			return false;
		}
		return true;
	}

	static bool mkdir_p(std::string const &path) {
		std::string cur;
		for (size_t i = 0; i <= path.size(); ++i) {
			if (i == path.size() || path[i] == '/') {
				if (!cur.empty() && cur != ".") {
					if (mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST) return false;
				}
			}
			if (i < path.size()) cur.push_back(path[i]);
		}
		return true;
	}

	static uint64_t fnv1a(uint64_t h, std::string const &s) {
		for (unsigned char ch : s) { h ^= ch; h *= 0x100000001B3ull; }
		return h;
	}

	static bool file_exists(std::string const &p) { struct stat st{}; return stat(p.c_str(), &st) == 0; }

	// Runs a shell command, returns its exit status and captures stdout+stderr.
	static int run_command(std::string const &cmd, std::string &output) {
		output.clear();
		FILE *p = popen((cmd + " 2>&1").c_str(), "r");
		if (p == nullptr) return -1;
		char buf[4096];
		size_t n;
		while ((n = fread(buf, 1, sizeof buf, p)) > 0) output.append(buf, n);
		int rc = pclose(p);
		return rc;
	}

	static std::string shell_quote(std::string const &s) {
		std::string out = "'";
		for (char ch : s) { if (ch == '\'') out += "'\\''"; else out.push_back(ch); }
		return out + "'";
	}

	// The counterpart of kernel_build.rs:200-220 (nvcc flags): gfx950 only, explicit fused
	// multiply-adds only, packed-f32 instructions off.
	static std::string device_flags() {
		return "--offload-arch=gfx950 -O3 -std=c++20 -ffp-contract=off "
		       "-Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument "
		       // gemm_b8.hip names M0 as clobbered by its hand-written direct-to-LDS load; the backend notes that it
		       // does not preserve that register around inline assembly, which is the intent
		       "-Wno-inline-asm";
	}

	std::optional<BuiltKernel> build(std::string const &kernel_name, std::string const &common_text,
	                                 std::string const &source_file, std::string const &meta_source_file,
	                                 Diagnostics &diag) {
		// gemm.rs:377-387 -- the name becomes a directory name
		if (kernel_name.empty() || kernel_name == "." || kernel_name == ".."
			|| kernel_name.find('/') != std::string::npos || kernel_name.find('\\') != std::string::npos) {
			diag.add_error("invalid kernel name \"" + kernel_name + "\"");
			return std::nullopt;
		}
		std::string kdir = kernels_dir();
		BuiltKernel out;
		out.dir_path = cache_dir() + "/" + kernel_name;
		out.common_path = out.dir_path + "/common.h";
		out.code_object_path = out.dir_path + "/kernel.hsaco";
		out.meta_json_path = out.dir_path + "/meta.json";
		std::string key_path = out.dir_path + "/build.key";

		if (!mkdir_p(out.dir_path)) {
			diag.add_error("failed to create kernel cache directory " + out.dir_path);
			return std::nullopt;
		}

		// Key of this build: everything the code object depends on.
		uint64_t h = 0xCBF29CE484222325ull;
		h = fnv1a(h, common_text);
		h = fnv1a(h, device_flags());
		// ... the two sources and, transitively, the headers of the kernels directory they include with #include "..."
		// (common.h is the generated text above), in the order a depth-first walk meets them: a change to another
		// kernel's tile header leaves this key alone.
		std::string text;
		if (!read_file(kdir + "/" + source_file, text)) {
			diag.add_error("kernel source not found: " + kdir + "/" + source_file);
			return std::nullopt;
		}
		if (!read_file(kdir + "/" + meta_source_file, text)) {
			diag.add_error("kernel metadata source not found: " + kdir + "/" + meta_source_file);
			return std::nullopt;
		}
		std::vector<std::string> seen;
		std::function<void(std::string const &)> hash_with_includes = [&](std::string const &file) {
			if (std::find(seen.begin(), seen.end(), file) != seen.end()) return;
			seen.push_back(file);
			std::string body;
			if (!read_file(kdir + "/" + file, body)) return;           // not a file of this directory (common.h, system headers)
			h = fnv1a(h, file);
			h = fnv1a(h, body);
			size_t pos = 0;
			while ((pos = body.find("#include \"", pos)) != std::string::npos) {
				size_t const from = pos + 10, to = body.find('"', from);
				if (to == std::string::npos) break;
				hash_with_includes(body.substr(from, to - from));
				pos = to;
			}
		};
		hash_with_includes(source_file);
		hash_with_includes(meta_source_file);
		char keybuf[32];
		std::snprintf(keybuf, sizeof keybuf, "%016llx", (unsigned long long)h);

		std::string have;
		bool const force = std::getenv("X17AI_FORCE_REBUILD") != nullptr;
		if (!force && read_file(key_path, have) && have == keybuf && file_exists(out.code_object_path) && file_exists(out.meta_json_path)) {
			out.cache_hit = true;
			return out;
		}

		if (!write_file(out.common_path, common_text, diag)) return std::nullopt;

		char const *hipcc_env = std::getenv("X17AI_HIPCC");
		std::string hipcc = hipcc_env != nullptr ? hipcc_env : "/opt/rocm/bin/hipcc";
		std::string log;
		std::string tmp_obj = out.code_object_path + ".tmp." + std::to_string(getpid());
		std::string cmd = shell_quote(hipcc) + " " + device_flags() + " --genco -I" + shell_quote(out.dir_path) + " -I" + shell_quote(kdir)
			+ " " + shell_quote(kdir + "/" + source_file) + " -o " + shell_quote(tmp_obj);
		int rc = run_command(cmd, log);
		if (rc != 0) {
			diag.add_error("hipcc failed for kernel " + kernel_name + " (" + cmd + "):\n" + log);
			return std::nullopt;
		}
		if (!log.empty()) diag.add_warning("hipcc: " + log);
		if (std::rename(tmp_obj.c_str(), out.code_object_path.c_str()) != 0) {
			diag.add_error("failed to move code object into place: " + out.code_object_path);
			return std::nullopt;
		}

		// kernel_build.rs:88-134 -- a host program prints the launch geometry the C++ constants imply
		std::string meta_exe = out.dir_path + "/meta." + std::to_string(getpid());
		cmd = "g++ -std=c++17 -O0 -I" + shell_quote(out.dir_path) + " -I" + shell_quote(kdir) + " "
			+ shell_quote(kdir + "/" + meta_source_file) + " -o " + shell_quote(meta_exe);
		rc = run_command(cmd, log);
		if (rc != 0) {
			diag.add_error("failed to compile the metadata program for " + kernel_name + ":\n" + log);
			return std::nullopt;
		}
		std::string meta_text;
		rc = run_command(shell_quote(meta_exe), meta_text);
		std::remove(meta_exe.c_str());
		if (rc != 0) {
			diag.add_error("the metadata program for " + kernel_name + " failed:\n" + meta_text);
			return std::nullopt;
		}
		if (!write_file(out.meta_json_path, meta_text, diag)) return std::nullopt;
		if (!write_file(key_path, keybuf, diag)) return std::nullopt;
		return out;
	}

	// Flat {"KEY": unsigned, ...} objects only -- all the metadata programs print.
	std::optional<std::vector<std::pair<std::string, size_t>>> read_metadata_json(std::string const &path, Diagnostics &diag) {
		std::string text;
		if (!read_file(path, text)) {
			diag.add_error("failed to read " + path);
			return std::nullopt;
		}
		std::vector<std::pair<std::string, size_t>> out;
		size_t i = 0;
		auto skip = [&]() { while (i < text.size() && (text[i] == ' ' || text[i] == '\n' || text[i] == '\t' || text[i] == '\r')) ++i; };
		skip();
		if (i >= text.size() || text[i] != '{') { diag.add_error("Invalid JSON metadata in " + path); return std::nullopt; }
		++i;
		for (;;) {
			skip();
			if (i < text.size() && text[i] == '}') break;
			if (i >= text.size() || text[i] != '"') { diag.add_error("Invalid JSON metadata in " + path); return std::nullopt; }
			size_t e = text.find('"', i + 1);
			if (e == std::string::npos) { diag.add_error("Invalid JSON metadata in " + path); return std::nullopt; }
			std::string key = text.substr(i + 1, e - i - 1);
			i = e + 1;
			skip();
			if (i >= text.size() || text[i] != ':') { diag.add_error("Invalid JSON metadata in " + path); return std::nullopt; }
			++i;
			skip();
			size_t v = 0, digits = 0;
			while (i < text.size() && text[i] >= '0' && text[i] <= '9') { v = v * 10 + size_t(text[i] - '0'); ++i; ++digits; }
			if (digits == 0) { diag.add_error("Invalid JSON metadata in " + path); return std::nullopt; }
			out.emplace_back(key, v);
			skip();
			if (i < text.size() && text[i] == ',') { ++i; continue; }
		}
		return out;
	}

	std::optional<size_t> meta_get(std::vector<std::pair<std::string, size_t>> const &m, char const *key) {
		for (auto const &kv : m) if (kv.first == key) return kv.second;
		return std::nullopt;
	}

	// kernel_build.rs:161-198
	std::unique_ptr<HipKernel> load_kernel(HipStream &stream, std::string const &path, char const *name, size_t smem, Diagnostics &diag) {
		if (path.find('\0') != std::string::npos) {
			diag.add_error("kernel path contains a NUL byte");
			return nullptr;
		}
		X17ModuleResult m = x17ai_hip_load_module(stream.ctx, path.c_str());
		if (m.value == nullptr) {
			diag.add_error(diagnostic_to_string(m.diagnostic, "failed to load module"));
			return nullptr;
		}
		auto module = std::make_shared<HipModule>();
		module->module = m.value;
		X17KernelResult k = x17ai_hip_get_kernel(module->module, name, smem);
		if (k.value == nullptr) {
			diag.add_error(diagnostic_to_string(k.diagnostic, "failed to get kernel"));
			return nullptr;
		}
		auto kernel = std::make_unique<HipKernel>();
		kernel->module = module;
		kernel->kernel = k.value;
		auto attrs = kernel->attrs();
		if (attrs.is_ok() && attrs.value->local_size_bytes != 0) {
			diag.add_warning("kernel " + path + " spills " + std::to_string(attrs.value->local_size_bytes) + " bytes per lane to scratch");
		}
		return kernel;
	}
}

static std::string format_cpp_f64(double v) {   // gemm.rs:257-259
	char buf[64];
	std::snprintf(buf, sizeof buf, "%.17e", v);
	return buf;
}

// A scale's description ends up in a `//` comment of the generated common.h: keep it on that line.
static std::string one_line(std::string s) {
	for (char &ch : s) if (ch == '\n' || ch == '\r' || ch == '\\') ch = ' ';
	return s;
}

static bool is_pow2(size_t v) { return v != 0 && (v & (v - 1)) == 0; }
static unsigned ctz(size_t v) { unsigned n = 0; while ((v & 1) == 0) { v >>= 1; ++n; } return n; }

// ================================================================ GEMM (src/device/cuda/gemm.rs)

static int kind_of(DType d) { return d == DType::E4m3 ? 1 : 0; }

// Two tensors share bytes.  Tiles that overhang a matrix edge are moved back and recompute rows or columns of their
// neighbour; that is only the same store twice as long as no output aliases an input another workgroup still reads.
static bool overlaps(Tensor const &x, Tensor const &y) {
	auto const xb = reinterpret_cast<uintptr_t>(x.ptr), yb = reinterpret_cast<uintptr_t>(y.ptr);
	return x.bytes != 0 && y.bytes != 0 && xb < yb + y.bytes && yb < xb + x.bytes;
}

std::unique_ptr<GemmKernel> GemmKernel::create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
                                               GemmConfig const &g, EpilogueConfig const &e, bool strict_math, Diagnostics &diag) {
	// gemm.rs:451-476 (the reference aborts with todo!() on these; here they are errors)
	if (g.a.trans) { diag.add_error("transposed GEMM input A is not supported"); return nullptr; }
	if (!g.b.trans) { diag.add_error("non-transposed GEMM input B is not supported"); return nullptr; }
	if (g.a.cols == 0 || g.b.cols == 0) { diag.add_error("empty GEMM dimensions are not supported"); return nullptr; }
	if (g.a.cols != g.b.cols) { diag.add_error("GEMM inputs A and B must have the same number of columns (K)"); return nullptr; }
	if (!g.b.rows) { diag.add_error("GEMM outputs with runtime column count are not supported"); return nullptr; }
	for (DType d : {g.a.dtype, g.b.dtype}) {
		if (d != DType::Int8 && d != DType::E4m3) { diag.add_error(std::string("unsupported GEMM input dtype ") + dtype_name(d)); return nullptr; }
	}
	size_t const b_rows = *g.b.rows;
	int const kind = int(e.index());
	std::ostringstream common;
	common << "// generated by x17::GemmKernel::create for kernel \"" << one_line(kernel_name) << "\"\n";
	common << "#define X17_A_COLS " << g.a.cols << "\n#define X17_B_ROWS " << b_rows << "\n";
	common << "#define X17_A_KIND " << kind_of(g.a.dtype) << "\n#define X17_B_KIND " << kind_of(g.b.dtype) << "\n";
	common << "#define X17_EPILOGUE " << kind << "\n";
	common << "#define X17_STORE " << (g.c_dtype == DType::E4m3 ? 1 : (g.c_dtype == DType::Bf16 ? 2 : 0)) << "\n";
	common << "#define X17_STRICT_MATH " << (strict_math ? 1 : 0) << "\n";
	// One wavefront per SIMD (four waves of 128 x 128, accumulators in the second half of the register file) wherever
	// an operand is e4m3.  e4m3 x e4m3: with the issue order of a K step pinned, a lone wave keeps the matrix core
	// busier than two waves that take turns at the barrier, and the fragments (32 bytes per lane and operand row) of
	// two such waves would not fit: 7-8 % faster than eight waves of 64 x 128.  e4m3 x int8 (f16 matrix cores, both
	// operands widened in registers): a weight row is widened by two waves and a token row by two, 3.5 vector
	// instructions per MFMA instead of 6.4, issued a piece behind each MFMA one round ahead: 7-8 % faster than eight
	// waves of 128 x 64 with the compiler's schedule.
	if (g.a.dtype == DType::E4m3 || g.b.dtype == DType::E4m3) {
		common << "#define X17_GEMM_WAVES_M 2\n#define X17_GEMM_WAVES_N 2\n";
	}

	auto finite_pos = [](double v) { return std::isfinite(v) && v > 0.0; };
	size_t head_dim = 0, sep_dim = 0;
	if (auto const *c = std::get_if<ScaleConfig>(&e)) {
		if (g.c_dtype != DType::Int8) { diag.add_error("Scale epilogue requires an i8 output"); return nullptr; }
		if (!std::isfinite(c->inp_scale.value) || !std::isfinite(c->out_scale.value)) { diag.add_error("invalid Scale epilogue scale values"); return nullptr; }
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->inp_scale.value) << " // " << one_line(c->inp_scale.description) << "\n";
		common << "#define X17_OUT_SCALE " << format_cpp_f64(c->out_scale.value) << " // " << one_line(c->out_scale.description) << "\n";
	} else if (auto const *c = std::get_if<GeGluConfig>(&e)) {
		if (g.c_dtype != DType::E4m3 && g.c_dtype != DType::Int8) { diag.add_error("GeGLU epilogue requires an e4m3 or i8 output"); return nullptr; }
		if (!finite_pos(c->inp_scale.value) || !finite_pos(c->out_scale.value)) { diag.add_error("invalid GeGLU scale values"); return nullptr; }
		if (b_rows % 2 != 0) { diag.add_error("GeGLU GEMM requires an even raw output column count"); return nullptr; }
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->inp_scale.value) << " // " << one_line(c->inp_scale.description) << "\n";
		common << "#define X17_OUT_SCALE " << format_cpp_f64(c->out_scale.value) << " // " << one_line(c->out_scale.description) << "\n";
	} else if (auto const *c = std::get_if<ResidualConfig>(&e)) {
		if (g.c_dtype != DType::E4m3 && g.c_dtype != DType::Int8) { diag.add_error("Residual epilogue requires an e4m3 or i8 output"); return nullptr; }
		if (!finite_pos(c->inp_scale.value) || !finite_pos(c->out_scale.value)) { diag.add_error("invalid residual GEMM scale values"); return nullptr; }
		if (b_rows % 2 != 0) { diag.add_error("Residual GEMM requires an even raw output column count"); return nullptr; }
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->inp_scale.value) << " // " << one_line(c->inp_scale.description) << "\n";
		common << "#define X17_OUT_SCALE " << format_cpp_f64(c->out_scale.value) << " // " << one_line(c->out_scale.description) << "\n";
	} else if (auto const *c = std::get_if<DequantConfig>(&e)) {
		if (g.c_dtype != DType::Bf16) { diag.add_error("Dequant epilogue requires a bf16 output"); return nullptr; }
		if (c->geglu && b_rows % 2 != 0) { diag.add_error("Dequant GeGLU GEMM requires an even raw output column count"); return nullptr; }
		common << "#define X17_DEQ_GEGLU " << (c->geglu ? 1 : 0) << "\n";
		common << "#define X17_INP_SCALE 1.0\n#define X17_OUT_SCALE 1.0\n";      // the scales arrive at run time
	} else if (auto const *c = std::get_if<RMSNormConfig>(&e)) {
		if (g.c_dtype != DType::Int8) { diag.add_error("RMSNorm epilogue requires an i8 output"); return nullptr; }
		if (g.a.dtype != DType::Int8 || g.b.dtype != DType::Int8) { diag.add_error("RMSNorm epilogue requires i8 inputs"); return nullptr; }
		if (!std::isfinite(c->eps) || c->eps < 0.0 || !std::isfinite(c->inp_scale.value) || !std::isfinite(c->out_scale.value)) {
			diag.add_error("invalid RMSNorm epilogue values"); return nullptr;
		}
		if (c->head_dim % 32 != 0 || c->sep_dim % 32 != 0) { diag.add_error("RMSNorm GEMM epilogue dimensions must be multiples of 32"); return nullptr; }
		if (c->head_dim != c->sep_dim || (c->head_dim != 32 && c->head_dim != 64 && c->head_dim != 128)) {
			diag.add_error("RMSNorm GEMM epilogue requires head_dim == sep_dim in {32, 64, 128}"); return nullptr;
		}
		size_t chunk = c->head_dim + c->sep_dim;
		if (!is_pow2(chunk) || b_rows % chunk != 0) { diag.add_error("RMSNorm GEMM raw output columns must be whole K|V heads"); return nullptr; }
		head_dim = c->head_dim;
		sep_dim = c->sep_dim;
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->inp_scale.value) << "\n#define X17_OUT_SCALE " << format_cpp_f64(c->out_scale.value) << "\n";
		common << "#define X17_HEAD_DIM " << c->head_dim << "\n#define X17_EPS " << format_cpp_f64(c->eps) << "\n";
		// gemm.rs:146,152
		common << "#define X17_HEAD_SCALE " << format_cpp_f64(c->out_scale.value * std::sqrt(double(c->head_dim)))
		       << " // (" << one_line(c->out_scale.description) << ") * sqrt(" << c->head_dim << ")\n";
		common << "#define X17_SEP_SCALE " << format_cpp_f64(c->inp_scale.value * c->out_scale.value)
		       << " // (" << one_line(c->inp_scale.description) << ") * (" << one_line(c->out_scale.description) << ")\n";
	}

	size_t q_cols = 0;
	auto rmsnorm_defines = [&](RMSNormConfig const &c, size_t kv_rows) -> bool {
		if (!std::isfinite(c.eps) || c.eps < 0.0 || !std::isfinite(c.inp_scale.value) || !std::isfinite(c.out_scale.value)) {
			diag.add_error("invalid RMSNorm epilogue values"); return false;
		}
		if (c.head_dim != c.sep_dim || (c.head_dim != 32 && c.head_dim != 64 && c.head_dim != 128)) {
			diag.add_error("RMSNorm GEMM epilogue requires head_dim == sep_dim in {32, 64, 128}"); return false;
		}
		if (kv_rows == 0 || kv_rows % (c.head_dim + c.sep_dim) != 0) { diag.add_error("RMSNorm GEMM raw output columns must be whole K|V heads"); return false; }
		common << "#define X17_HEAD_DIM " << c.head_dim << "\n#define X17_EPS " << format_cpp_f64(c.eps) << "\n";
		common << "#define X17_HEAD_SCALE " << format_cpp_f64(c.out_scale.value * std::sqrt(double(c.head_dim)))
		       << " // (" << one_line(c.out_scale.description) << ") * sqrt(" << c.head_dim << ")\n";
		common << "#define X17_SEP_SCALE " << format_cpp_f64(c.inp_scale.value * c.out_scale.value)
		       << " // (" << one_line(c.inp_scale.description) << ") * (" << one_line(c.out_scale.description) << ")\n";
		return true;
	};
	if (auto const *c = std::get_if<QNormConfig>(&e)) {
		if (g.c_dtype != DType::Int8 || g.a.dtype != DType::Int8 || g.b.dtype != DType::Int8) { diag.add_error("QNorm epilogue requires i8 inputs and an i8 output"); return nullptr; }
		if (!std::isfinite(c->eps) || c->eps < 0.0 || !finite_pos(c->out_scale.value) || !finite_pos(c->post_scale.value)) { diag.add_error("invalid QNorm epilogue values"); return nullptr; }
		if (c->head_dim != 32 && c->head_dim != 64 && c->head_dim != 128) { diag.add_error("QNorm GEMM epilogue requires head_dim in {32, 64, 128}"); return nullptr; }
		if (b_rows % c->head_dim != 0) { diag.add_error("QNorm GEMM raw output columns must be whole heads"); return nullptr; }
		head_dim = c->head_dim;
		// X17_INP_SCALE: the factor applied after the learned scales (the old writer's base class carried
		// 1 / sqrt(MODEL_DIM), cuda/qkvg_fwd_i8.cuh:151-159; 1.0 stores the normalised values as they are)
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->post_scale.value) << "\n#define X17_OUT_SCALE " << format_cpp_f64(c->out_scale.value) << "\n";
		common << "#define X17_HEAD_DIM " << c->head_dim << "\n#define X17_EPS " << format_cpp_f64(c->eps) << "\n";
		// cuda/qkvg_fwd_i8.cuh:205
		common << "#define X17_HEAD_SCALE " << format_cpp_f64(c->out_scale.value * std::sqrt(double(c->head_dim)))
		       << " // (" << one_line(c->out_scale.description) << ") * sqrt(" << c->head_dim << ")\n";
	} else if (auto const *c = std::get_if<QkvConfig>(&e)) {
		if (g.c_dtype != DType::Int8 || g.a.dtype != DType::Int8 || g.b.dtype != DType::Int8) { diag.add_error("fused q + kv GEMM requires i8 inputs and i8 outputs"); return nullptr; }
		if (c->q_cols == 0 || c->q_cols >= b_rows || c->q_cols % 256 != 0) {
			diag.add_error("fused q + kv GEMM: q_cols must be a multiple of 256 below the raw output column count"); return nullptr;
		}
		if (!std::isfinite(c->q.inp_scale.value) || !std::isfinite(c->q.out_scale.value)) { diag.add_error("invalid Scale epilogue scale values"); return nullptr; }
		common << "#define X17_INP_SCALE " << format_cpp_f64(c->kv.inp_scale.value) << "\n#define X17_OUT_SCALE " << format_cpp_f64(c->kv.out_scale.value) << "\n";
		common << "#define X17_Q_COLS " << c->q_cols << "\n";
		common << "#define X17_Q_SCALE (" << format_cpp_f64(c->q.inp_scale.value) << " * " << format_cpp_f64(c->q.out_scale.value) << ")"
		       << " // (" << one_line(c->q.inp_scale.description) << ") * (" << one_line(c->q.out_scale.description) << ")\n";
		if (!rmsnorm_defines(c->kv, b_rows - c->q_cols)) return nullptr;
		head_dim = c->kv.head_dim;
		sep_dim = c->kv.sep_dim;
		q_cols = c->q_cols;
	}

	if (g.a.cols % 128 != 0) { diag.add_error("GEMM K must be a multiple of 128, got " + std::to_string(g.a.cols)); return nullptr; }
	// gemm.rs:607-614 (N_PER_BLOCK of the reference's tile)
	if (b_rows % 128 != 0) { diag.add_error("GEMM raw output columns must be a multiple of 128, got " + std::to_string(b_rows)); return nullptr; }
	if (b_rows < 256) { diag.add_error("GEMM raw output columns must be at least one tile (256), got " + std::to_string(b_rows)); return nullptr; }

	auto built = kernel_build::build(kernel_name, common.str(), "gemm_b8.hip", "gemm_meta.cpp", diag);
	if (!built) return nullptr;

	auto meta = kernel_build::read_metadata_json(built->meta_json_path, diag);
	if (!meta) return nullptr;
	auto out = std::make_unique<GemmKernel>();
	auto get = [&](char const *k) { auto v = kernel_build::meta_get(*meta, k); return v ? *v : size_t(0); };
	out->metadata = GemmLauncherMetadata{get("THREADS_PER_BLOCK"), get("SMEM_BYTES"), get("M_PER_BLOCK"), get("N_PER_BLOCK"), get("MAX_BLOCKS")};
	// gemm.rs:561-570
	if (out->metadata.THREADS_PER_BLOCK == 0 || !is_pow2(out->metadata.M_PER_BLOCK) || !is_pow2(out->metadata.N_PER_BLOCK)) {
		diag.add_error("Invalid JSON metadata in " + built->meta_json_path);
		return nullptr;
	}
	// gemm.rs:607-614 accepts raw columns % 128 == 0 (its tile is 64 x 128).  The tile here is wider; a last tile that
	// would overhang is moved back to end at the matrix edge, so the same shapes are accepted from one tile upwards.
	if (b_rows % 128 != 0 || b_rows < out->metadata.N_PER_BLOCK) {
		diag.add_error("GEMM raw output columns (" + std::to_string(b_rows) + ") must be a multiple of 128 and at least the tile width "
			+ std::to_string(out->metadata.N_PER_BLOCK));
		return nullptr;
	}
	out->name = kernel_name;
	out->files = *built;
	out->epilogue_kind = kind;
	out->a_cols = g.a.cols;
	out->b_rows = g.b.rows;
	out->a_dtype = g.a.dtype;
	out->b_dtype = g.b.dtype;
	out->c_dtype = g.c_dtype;
	out->head_dim = head_dim;
	out->sep_dim = sep_dim;
	out->q_cols = q_cols;
	if (auto const *c = std::get_if<DequantConfig>(&e)) out->dequant_geglu = c->geglu;
	if (device) {
		out->kernel = kernel_build::load_kernel(*device->stream, built->code_object_path, "kernel", out->metadata.SMEM_BYTES, diag);
		if (!out->kernel) return nullptr;
		out->device = std::move(device);
	}
	return out;
}

double GemmKernel::n_ops(Tensor const &a, Tensor const &b) const {
	if (a.shape.size() < 2 || b.shape.size() < 2) return 0.0;
	return 2.0 * double(a.shape[a.shape.size() - 2]) * double(a.shape[a.shape.size() - 1]) * double(b.shape[b.shape.size() - 2]);
}

// gemm.rs:591-641 (basic), :661-747 (residual), :767-838 (geglu), :860-918 (rmsnorm)
Status GemmKernel::launch(GemmArgs const &args) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "GEMM kernel " + name + " was built without a device");
	char const *op = epilogue_kind == 2 ? "Residual GEMM" : "GEMM";
	size_t a_shape[2], b_shape[2], c_shape[2], tmp[2];
	Status s = tensor_check::matrix_shape(op, "a", *args.a, std::nullopt, a_cols, *device, a_dtype, a_shape);
	if (!s.is_ok()) return s;
	if (epilogue_kind == 6) return launch_qkv(args, a_shape[0]);
	if (args.b2 != nullptr || args.c2 != nullptr) {
		return Status::err(TensorOpError::Other, "GEMM kernel " + name + " is not a fused q + kv kernel: it takes one weight matrix and one output");
	}
	s = tensor_check::matrix_shape(op, "b", *args.b, b_rows, a_cols, *device, b_dtype, b_shape);
	if (!s.is_ok()) return s;
	size_t const a_rows = a_shape[0], b_rows_v = b_shape[0];
	bool const halves = epilogue_kind == 1 || epilogue_kind == 2 || (epilogue_kind == 4 && dequant_geglu);
	if (halves && b_rows_v % 2 != 0) {
		return Status::err(TensorOpError::Other, std::string(epilogue_kind == 2 ? "Residual" : "GeGLU")
			+ " GEMM requires an even raw output column count, got " + std::to_string(b_rows_v));
	}
	size_t const out_cols = halves ? b_rows_v / 2 : b_rows_v;
	s = tensor_check::matrix_shape(op, "c", *args.c, a_rows, out_cols, *device, c_dtype, c_shape);
	if (!s.is_ok()) return s;
	if (epilogue_kind == 2) {
		if (args.extra == nullptr) return Status::err(TensorOpError::Other, "Residual GEMM needs a residual tensor");
		s = tensor_check::matrix_shape(op, "residual", *args.extra, a_rows, out_cols, *device, DType::Int8, tmp);
		if (!s.is_ok()) return s;
		if (overlaps(*args.c, *args.extra)) {
			return Status::err(TensorOpError::Other, "Residual GEMM output c must not share memory with the residual (no in-place update)");
		}
	}
	if (overlaps(*args.c, *args.a) || overlaps(*args.c, *args.b)) {
		return Status::err(TensorOpError::Other, std::string(op) + " output c must not share memory with an input");
	}
	// gemm.rs:607-614: rows % 64 == 0, raw columns % 128 == 0 (the reference's tile shape); here from one tile upwards
	if (a_rows % 64 != 0 || b_rows_v % 128 != 0 || a_rows < metadata.M_PER_BLOCK || b_rows_v < metadata.N_PER_BLOCK) {
		return Status::err(TensorOpError::Other, std::string(op) + " raw output shape [" + std::to_string(a_rows) + ", "
			+ std::to_string(b_rows_v) + "] must be divisible by [64, 128] (as in the reference) and hold at least one "
			+ std::to_string(metadata.M_PER_BLOCK) + " x " + std::to_string(metadata.N_PER_BLOCK) + " tile of this kernel");
	}
	if (epilogue_kind == 4) {
		if (args.extra == nullptr || args.extra2 == nullptr) {
			return Status::err(TensorOpError::Other, "Dequant GEMM needs a row-scale and a column-scale tensor");
		}
		s = tensor_check::vector_shape(op, "row_scale", *args.extra, a_rows, *device, DType::F32);
		if (!s.is_ok()) return s;
		s = tensor_check::vector_shape(op, "col_scale", *args.extra2, b_rows_v, *device, DType::F32);
		if (!s.is_ok()) return s;
	}
	if (epilogue_kind == 5) {
		if (args.extra == nullptr) return Status::err(TensorOpError::Other, "QNorm GEMM needs a q_norm_scales tensor");
		s = tensor_check::vector_shape(op, "q_norm_scales", *args.extra, b_rows_v, *device, DType::Bf16);
		if (!s.is_ok()) return s;
	}
	if (epilogue_kind == 3) {
		if (args.extra == nullptr) return Status::err(TensorOpError::Other, "RMSNorm GEMM needs an rrms tensor");
		size_t chunk = head_dim + sep_dim;
		size_t rrms_cols = b_rows_v >> ctz(chunk);
		s = tensor_check::matrix_shape(op, "rrms", *args.extra, a_rows, rrms_cols, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
	}
	if (a_rows > 0xFFFFFFFFull || b_rows_v > 0xFFFFFFFFull) {
		return Status::err(TensorOpError::Other, std::string(op) + " sizes exceed 32 bits (the kernel's row counts are u32)");
	}
	size_t grid_x = (a_rows + metadata.M_PER_BLOCK - 1) >> ctz(metadata.M_PER_BLOCK);
	size_t grid_y = (b_rows_v + metadata.N_PER_BLOCK - 1) >> ctz(metadata.N_PER_BLOCK);
	// 8-byte slots passed by address, exactly as gemm.rs:618-631 does; the kernel's u32 parameters
	// read the low halves.
	void *a_ptr = args.a->ptr;
	size_t a_rows_arg = a_rows;
	void *b_ptr = args.b->ptr;
	size_t b_rows_arg = b_rows_v;
	void *c_ptr = args.c->ptr;
	void *extra_ptr = args.extra != nullptr ? args.extra->ptr : nullptr;
	void *extra2_ptr = args.extra2 != nullptr ? args.extra2->ptr : nullptr;
	void *raw_args[7] = {&a_ptr, &a_rows_arg, &b_ptr, &b_rows_arg, &c_ptr, &extra_ptr, &extra2_ptr};
	size_t grid[3] = {grid_x, grid_y, 1};
	if (metadata.MAX_BLOCKS != 0 && grid_x * grid_y > metadata.MAX_BLOCKS) {
		// persistent kernel: the workgroups share the tiles out among themselves
		grid[0] = metadata.MAX_BLOCKS;
		grid[1] = 1;
	}
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// The fused q + kv launch: the checks of gemm.rs:591-641 for the q part and of :860-918 for the kv part.
Status GemmKernel::launch_qkv(GemmArgs const &args, size_t a_rows) {
	char const *op = "fused q + kv GEMM";
	if (args.b == nullptr || args.c == nullptr || args.b2 == nullptr || args.c2 == nullptr || args.extra == nullptr) {
		return Status::err(TensorOpError::Other, "fused q + kv GEMM needs x, the q and kv weights, the q and kv outputs and an rrms tensor");
	}
	size_t const kv_cols = *b_rows - q_cols;
	size_t tmp[2];
	Status s = tensor_check::matrix_shape(op, "q weights", *args.b, q_cols, a_cols, *device, b_dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "kv weights", *args.b2, kv_cols, a_cols, *device, b_dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "q", *args.c, a_rows, q_cols, *device, c_dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "kv", *args.c2, a_rows, kv_cols, *device, c_dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "rrms", *args.extra, a_rows, kv_cols >> ctz(head_dim + sep_dim), *device, DType::F32, tmp);
	if (!s.is_ok()) return s;
	if (a_rows % 64 != 0 || a_rows < metadata.M_PER_BLOCK) {
		return Status::err(TensorOpError::Other, std::string(op) + " token rows (" + std::to_string(a_rows) + ") must be a multiple of 64 and at least the tile height "
			+ std::to_string(metadata.M_PER_BLOCK));
	}
	if (a_rows > 0xFFFFFFFFull) return Status::err(TensorOpError::Other, std::string(op) + " sizes exceed 32 bits (the kernel's row counts are u32)");
	for (Tensor const *o : {args.c, args.c2}) {
		if (overlaps(*o, *args.a) || overlaps(*o, *args.b) || overlaps(*o, *args.b2)) {
			return Status::err(TensorOpError::Other, std::string(op) + " outputs must not share memory with an input");
		}
	}
	void *a_ptr = args.a->ptr;
	size_t a_rows_arg = a_rows;
	void *b_ptr = args.b->ptr;
	size_t b_rows_arg = *b_rows;
	void *c_ptr = args.c->ptr;
	void *rrms_ptr = args.extra->ptr;
	void *b2_ptr = args.b2->ptr;
	void *c2_ptr = args.c2->ptr;
	void *raw_args[8] = {&a_ptr, &a_rows_arg, &b_ptr, &b_rows_arg, &c_ptr, &rrms_ptr, &b2_ptr, &c2_ptr};
	size_t tiles = ((a_rows + metadata.M_PER_BLOCK - 1) >> ctz(metadata.M_PER_BLOCK)) * ((*b_rows + metadata.N_PER_BLOCK - 1) >> ctz(metadata.N_PER_BLOCK));
	size_t grid[3] = {metadata.MAX_BLOCKS != 0 && tiles > metadata.MAX_BLOCKS ? metadata.MAX_BLOCKS : tiles, 1, 1};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// ================================================================ attention (src/device/cuda/attn.rs)

size_t AttnKernelConfig::heads_per_kernel() const { return head_dim == 0 ? 1 : std::max<size_t>(128 / head_dim, 1); }
size_t AttnKernelConfig::head_group_cnt() const { return n_heads / heads_per_kernel(); }
size_t AttnKernelConfig::head_group_dim() const { return heads_per_kernel() * head_dim; }

double AttnKernelConfig::n_ops(size_t seq_len, size_t window_size) const {
	double attended = window_size > 0 ? double(window_size) + 1.0 : double(seq_len) / 2.0 + 0.5;
	return 4.0 * double(n_heads * head_dim) * double(seq_len) * attended;
}

bool AttnKernelConfig::validate(Diagnostics &diag) const {
	if (dtype != DType::Int8) { diag.add_error(std::string("attention kernel config currently requires dtype i8, got ") + dtype_name(dtype)); return false; }
	if (out_dtype != DType::Int8 && !(row_scales && out_dtype == DType::Bf16)) {
		diag.add_error(std::string("attention kernel config writes i8, or bf16 with row scales, got ") + dtype_name(out_dtype));
		return false;
	}
	if (n_heads == 0) { diag.add_error("attention kernel config requires n_heads > 0"); return false; }
	if (head_dim == 0 || head_dim % 32 != 0) {
		diag.add_error("attention kernel config requires head_dim to be a non-zero multiple of 32, got " + std::to_string(head_dim));
		return false;
	}
	size_t hpk = heads_per_kernel();
	if (n_heads % hpk != 0) {
		diag.add_error("attention kernel config requires n_heads (" + std::to_string(n_heads) + ") to be divisible by heads_per_kernel ("
			+ std::to_string(hpk) + ")");
		return false;
	}
	size_t q_cols = n_heads * head_dim, kv_cols = 2 * q_cols;
	if (q_stride < q_cols) { diag.add_error("attention kernel config requires q_stride >= n_heads * head_dim, got " + std::to_string(q_stride) + " vs " + std::to_string(q_cols)); return false; }
	if (kv_stride < kv_cols) { diag.add_error("attention kernel config requires kv_stride >= 2 * n_heads * head_dim, got " + std::to_string(kv_stride) + " vs " + std::to_string(kv_cols)); return false; }
	if (o_stride < q_cols) { diag.add_error("attention kernel config requires o_stride >= n_heads * head_dim, got " + std::to_string(o_stride) + " vs " + std::to_string(q_cols)); return false; }
	if (head_group_dim() % 128 != 0) {
		diag.add_error("attention kernel config requires heads_per_kernel * head_dim to be 128B aligned, got " + std::to_string(head_group_dim()));
		return false;
	}
	return true;
}

std::unique_ptr<AttnKernel> AttnKernel::create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
                                               AttnKernelConfig const &config, bool strict_math, Diagnostics &diag) {
	if (!config.validate(diag)) return nullptr;
	if (config.head_dim != 32 && config.head_dim != 64 && config.head_dim != 128) {
		diag.add_error("attention kernel supports head_dim 32, 64 or 128, got " + std::to_string(config.head_dim));
		return nullptr;
	}
	std::ostringstream common;
	common << "// generated by x17::AttnKernel::create for kernel \"" << one_line(kernel_name) << "\"\n";
	common << "#define X17_N_HEADS " << config.n_heads << "\n#define X17_HEAD_DIM " << config.head_dim << "\n";
	common << "#define X17_Q_STRIDE " << config.q_stride << "\n#define X17_KV_STRIDE " << config.kv_stride << "\n#define X17_O_STRIDE " << config.o_stride << "\n";
	common << "#define X17_STRICT_MATH " << (strict_math ? 1 : 0) << "\n";
	if (config.row_scales) {
		common << "#define X17_ATTN_ROW_SCALES 1\n#define X17_ATTN_OUT_BF16 " << (config.out_dtype == DType::Bf16 ? 1 : 0) << "\n";
	}
	if ((config.backward_q || config.backward_kv) && (config.row_scales || config.out_dtype != DType::Int8)) {
		diag.add_error("the attention backward kernels take FixedI8 operands at the fixed scale (no row scales, i8 forward output)");
		return nullptr;
	}
	if (config.backward_q && config.backward_kv) {
		diag.add_error("an attention kernel is the forward, the backward with respect to q, or the backward with respect to k and v: backward_q and backward_kv are both set");
		return nullptr;
	}
	auto built = config.backward_q  ? kernel_build::build(kernel_name, common.str(), "attn_d_q_i8.hip", "attn_bwd_meta.cpp", diag)
	           : config.backward_kv ? kernel_build::build(kernel_name, common.str(), "attn_d_kv_i8.hip", "attn_bwd_kv_meta.cpp", diag)
	                                : kernel_build::build(kernel_name, common.str(), "attn_fwd_i8.hip", "attn_meta.cpp", diag);
	if (!built) return nullptr;
	auto meta = kernel_build::read_metadata_json(built->meta_json_path, diag);
	if (!meta) return nullptr;
	auto out = std::make_unique<AttnKernel>();
	auto get = [&](char const *k) { auto v = kernel_build::meta_get(*meta, k); return v ? *v : size_t(0); };
	out->metadata = AttnLauncherMetadata{get("THREADS_PER_BLOCK"), get("SMEM_BYTES"), get("Q_PER_BLOCK")};
	// attn.rs:333-342
	if (out->metadata.THREADS_PER_BLOCK == 0 || out->metadata.SMEM_BYTES == 0 || !is_pow2(out->metadata.Q_PER_BLOCK)) {
		diag.add_error("Invalid JSON metadata in " + built->meta_json_path);
		return nullptr;
	}
	out->name = kernel_name;
	out->files = *built;
	out->config = config;
	if (device) {
		out->kernel = kernel_build::load_kernel(*device->stream, built->code_object_path, "kernel", out->metadata.SMEM_BYTES, diag);
		if (!out->kernel) return nullptr;
		out->device = std::move(device);
	}
	return out;
}

// attn.rs:353-447
Status AttnKernel::launch(AttnKernelArgs const &a) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "attention kernel " + name + " was built without a device");
	if (config.backward_q || config.backward_kv) {
		return Status::err(TensorOpError::Other, "attention kernel " + name + " is a backward kernel: use launch_d_q / launch_d_kv");
	}
	size_t shp[2], tmp[2];
	Status s = tensor_check::matrix_shape("attention", "q", *a.q, std::nullopt, config.q_stride, *device, config.dtype, shp);
	if (!s.is_ok()) return s;
	size_t const rows = shp[0];
	s = tensor_check::matrix_shape("attention", "kv", *a.kv, rows, config.kv_stride, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("attention", "sink_k", *a.sink_k, config.n_heads, config.head_dim, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("attention", "sink_v", *a.sink_v, config.n_heads, config.head_dim, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::vector_shape("attention", "attn_temperature", *a.attn_temperature, config.n_heads, *device, DType::F32);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("attention", "out", *a.out, rows, config.o_stride, *device, config.out_dtype, tmp);
	if (!s.is_ok()) return s;
	bool const any_scale = a.q_scale || a.k_scale || a.v_weight || a.sink_v_weight || a.out_scale;
	if (config.row_scales) {
		if (!a.q_scale || !a.k_scale || !a.v_weight || !a.sink_v_weight || !a.out_scale) {
			return Status::err(TensorOpError::Other, "attention kernel " + name + " needs q_scale, k_scale, v_weight, sink_v_weight and out_scale");
		}
		s = tensor_check::matrix_shape("attention", "q_scale", *a.q_scale, config.n_heads, rows, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
		s = tensor_check::matrix_shape("attention", "k_scale", *a.k_scale, config.n_heads, rows, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
		s = tensor_check::matrix_shape("attention", "v_weight", *a.v_weight, config.n_heads, rows, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
		s = tensor_check::vector_shape("attention", "sink_v_weight", *a.sink_v_weight, config.n_heads, *device, DType::F32);
		if (!s.is_ok()) return s;
		s = tensor_check::vector_shape("attention", "out_scale", *a.out_scale, config.n_heads, *device, DType::F32);
		if (!s.is_ok()) return s;
	} else if (any_scale) {
		return Status::err(TensorOpError::Other, "attention kernel " + name + " was built without row scales");
	}
	if (a.l != nullptr) {
		s = tensor_check::matrix_shape("attention", "l", *a.l, config.n_heads, rows, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
	}
	if (overlaps(*a.out, *a.q) || overlaps(*a.out, *a.kv)) {
		// (a last query block that would overhang is moved back and recomputes its neighbour's queries from q)
		return Status::err(TensorOpError::Other, "attention output must not share memory with q or kv");
	}
	if (a.batch == 0 || rows % a.batch != 0) {
		return Status::err(TensorOpError::Other, "attention rows (" + std::to_string(rows) + ") must be divisible by batch (" + std::to_string(a.batch) + ")");
	}
	size_t const seq_len = rows / a.batch;
	// attn.rs:398-404: seq_len % 64 == 0 (the reference's query block).  The query block here is larger; a last block
	// that would overhang starts earlier instead (it recomputes some of its neighbour's queries and stores the same
	// bytes), so the same lengths are accepted from one block upwards.
	if (seq_len % 64 != 0 || seq_len < metadata.Q_PER_BLOCK) {
		return Status::err(TensorOpError::Other, "attention seq_len must be divisible by 64 (as in the reference) and hold at least one query block of "
			+ std::to_string(metadata.Q_PER_BLOCK) + ", got " + std::to_string(seq_len));
	}
	if (a.window_size > 0 && a.window_size % 16 != 0) {
		return Status::err(TensorOpError::Other, "attention window_size must be zero or divisible by 16, got " + std::to_string(a.window_size));
	}
	if (rows > 0xFFFFFFFFull || a.window_size > 0xFFFFFFFFull) {
		return Status::err(TensorOpError::Other, "attention sizes exceed 32 bits");
	}
	size_t seq_len_arg = seq_len;
	void *q_ptr = a.q->ptr, *kv_ptr = a.kv->ptr, *sk = a.sink_k->ptr, *sv = a.sink_v->ptr, *tp = a.attn_temperature->ptr;
	void *out_ptr = a.out->ptr;
	void *l_ptr = a.l != nullptr ? a.l->ptr : nullptr;
	size_t window_arg = a.window_size;
	void *scale_ptrs[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
	if (config.row_scales) {
		Tensor const *t[5] = {a.q_scale, a.k_scale, a.v_weight, a.sink_v_weight, a.out_scale};
		for (int i = 0; i < 5; ++i) scale_ptrs[i] = t[i]->ptr;
	}
	// the plain kernel takes the first nine arguments only
	void *raw_args[14] = {&seq_len_arg, &q_ptr, &kv_ptr, &sk, &sv, &tp, &out_ptr, &l_ptr, &window_arg,
	                      &scale_ptrs[0], &scale_ptrs[1], &scale_ptrs[2], &scale_ptrs[3], &scale_ptrs[4]};
	size_t grid[3] = {(seq_len + metadata.Q_PER_BLOCK - 1) / metadata.Q_PER_BLOCK, config.head_group_cnt(), a.batch};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// The backward with respect to q: the forward's inputs, its output and log-sum-exp, and dO (bf16) -> dQ (bf16), D.
Status AttnKernel::launch_d_q(AttnKernelArgs const &a) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "attention kernel " + name + " was built without a device");
	if (!config.backward_q) return Status::err(TensorOpError::Other, "attention kernel " + name + " is not a backward-with-respect-to-q kernel");
	if (a.l == nullptr || a.d_out == nullptr || a.d_q == nullptr) {
		return Status::err(TensorOpError::Other, "attention backward needs l, d_out and d_q");
	}
	char const *op = "attention backward";
	size_t shp[2], tmp[2];
	Status s = tensor_check::matrix_shape(op, "q", *a.q, std::nullopt, config.q_stride, *device, config.dtype, shp);
	if (!s.is_ok()) return s;
	size_t const rows = shp[0];
	s = tensor_check::matrix_shape(op, "kv", *a.kv, rows, config.kv_stride, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "sink_k", *a.sink_k, config.n_heads, config.head_dim, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "sink_v", *a.sink_v, config.n_heads, config.head_dim, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::vector_shape(op, "attn_temperature", *a.attn_temperature, config.n_heads, *device, DType::F32);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "out", *a.out, rows, config.o_stride, *device, DType::Int8, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "d_out", *a.d_out, rows, config.o_stride, *device, DType::Bf16, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "d_q", *a.d_q, rows, config.q_stride, *device, DType::Bf16, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "l", *a.l, config.n_heads, rows, *device, DType::F32, tmp);
	if (!s.is_ok()) return s;
	if (a.d != nullptr) {
		s = tensor_check::matrix_shape(op, "d", *a.d, config.n_heads, rows, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
	}
	for (Tensor const *in : {a.q, a.kv, a.out, a.d_out}) {
		if (overlaps(*a.d_q, *in)) return Status::err(TensorOpError::Other, "attention backward output d_q must not share memory with an input");
	}
	if (a.batch == 0 || rows % a.batch != 0) {
		return Status::err(TensorOpError::Other, "attention rows (" + std::to_string(rows) + ") must be divisible by batch (" + std::to_string(a.batch) + ")");
	}
	size_t const seq_len = rows / a.batch;
	if (seq_len % 64 != 0 || seq_len < metadata.Q_PER_BLOCK) {
		return Status::err(TensorOpError::Other, "attention seq_len must be divisible by 64 (as in the reference) and hold at least one query block of "
			+ std::to_string(metadata.Q_PER_BLOCK) + ", got " + std::to_string(seq_len));
	}
	if (a.window_size > 0 && a.window_size % 16 != 0) {
		return Status::err(TensorOpError::Other, "attention window_size must be zero or divisible by 16, got " + std::to_string(a.window_size));
	}
	if (rows > 0xFFFFFFFFull || a.window_size > 0xFFFFFFFFull) return Status::err(TensorOpError::Other, "attention sizes exceed 32 bits");
	size_t seq_len_arg = seq_len, window_arg = a.window_size;
	void *q_ptr = a.q->ptr, *kv_ptr = a.kv->ptr, *sk = a.sink_k->ptr, *sv = a.sink_v->ptr, *tp = a.attn_temperature->ptr;
	void *out_ptr = a.out->ptr, *do_ptr = a.d_out->ptr, *dq_ptr = a.d_q->ptr, *l_ptr = a.l->ptr;
	void *d_ptr = a.d != nullptr ? a.d->ptr : nullptr;
	void *raw_args[12] = {&seq_len_arg, &q_ptr, &kv_ptr, &sk, &sv, &tp, &out_ptr, &do_ptr, &dq_ptr, &l_ptr, &d_ptr, &window_arg};
	size_t grid[3] = {(seq_len + metadata.Q_PER_BLOCK - 1) / metadata.Q_PER_BLOCK, config.head_group_cnt(), a.batch};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// The backward with respect to k and v: q, kv, the temperatures, dO (bf16), the forward's L and the dQ pass's D
// -> d_kv (bf16, the layout of kv).
Status AttnKernel::launch_d_kv(AttnKernelArgs const &a) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "attention kernel " + name + " was built without a device");
	if (!config.backward_kv) return Status::err(TensorOpError::Other, "attention kernel " + name + " is not a backward-with-respect-to-k-and-v kernel");
	if (a.l == nullptr || a.d == nullptr || a.d_out == nullptr || a.d_kv == nullptr) {
		return Status::err(TensorOpError::Other, "attention backward (k, v) needs l, d, d_out and d_kv");
	}
	char const *op = "attention backward (k, v)";
	size_t shp[2], tmp[2];
	Status s = tensor_check::matrix_shape(op, "q", *a.q, std::nullopt, config.q_stride, *device, config.dtype, shp);
	if (!s.is_ok()) return s;
	size_t const rows = shp[0];
	s = tensor_check::matrix_shape(op, "kv", *a.kv, rows, config.kv_stride, *device, config.dtype, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::vector_shape(op, "attn_temperature", *a.attn_temperature, config.n_heads, *device, DType::F32);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "d_out", *a.d_out, rows, config.o_stride, *device, DType::Bf16, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "l", *a.l, config.n_heads, rows, *device, DType::F32, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "d", *a.d, config.n_heads, rows, *device, DType::F32, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape(op, "d_kv", *a.d_kv, rows, config.kv_stride, *device, DType::Bf16, tmp);
	if (!s.is_ok()) return s;
	for (Tensor const *in : {a.q, a.kv, a.d_out, a.l, a.d}) {
		if (overlaps(*a.d_kv, *in)) return Status::err(TensorOpError::Other, "attention backward output d_kv must not share memory with an input");
	}
	if (a.batch == 0 || rows % a.batch != 0) {
		return Status::err(TensorOpError::Other, "attention rows (" + std::to_string(rows) + ") must be divisible by batch (" + std::to_string(a.batch) + ")");
	}
	size_t const seq_len = rows / a.batch;
	if (seq_len % 64 != 0 || seq_len < metadata.Q_PER_BLOCK) {
		return Status::err(TensorOpError::Other, "attention seq_len must be divisible by 64 (as in the reference) and hold at least one key block of "
			+ std::to_string(metadata.Q_PER_BLOCK) + ", got " + std::to_string(seq_len));
	}
	if (a.window_size > 0 && a.window_size % 16 != 0) {
		return Status::err(TensorOpError::Other, "attention window_size must be zero or divisible by 16, got " + std::to_string(a.window_size));
	}
	if (rows > 0xFFFFFFFFull || a.window_size > 0xFFFFFFFFull) return Status::err(TensorOpError::Other, "attention sizes exceed 32 bits");
	size_t seq_len_arg = seq_len, window_arg = a.window_size;
	void *q_ptr = a.q->ptr, *kv_ptr = a.kv->ptr, *tp = a.attn_temperature->ptr, *do_ptr = a.d_out->ptr, *l_ptr = a.l->ptr, *d_ptr = a.d->ptr;
	void *dkv_ptr = a.d_kv->ptr;
	void *raw_args[9] = {&seq_len_arg, &q_ptr, &kv_ptr, &tp, &do_ptr, &l_ptr, &d_ptr, &dkv_ptr, &window_arg};
	size_t grid[3] = {(seq_len + metadata.Q_PER_BLOCK - 1) / metadata.Q_PER_BLOCK, config.head_group_cnt(), a.batch};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// ================================================================ rms_norm

std::unique_ptr<RmsNormKernel> RmsNormKernel::create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
                                                     RmsNormConfig const &config, Diagnostics &diag) {
	if (config.in_dtype != DType::E4m3 && config.in_dtype != DType::Bf16) { diag.add_error("rms_norm input must be e4m3 or bf16"); return nullptr; }
	if (config.model_dim == 0 || config.model_dim % 512 != 0) {      // rms_norm.cu:16
		diag.add_error("rms_norm requires model_dim to be a non-zero multiple of 512, got " + std::to_string(config.model_dim));
		return nullptr;
	}
	if (!std::isfinite(config.eps) || config.eps < 0.0) { diag.add_error("invalid rms_norm eps"); return nullptr; }
	std::ostringstream common;
	common << "// generated by x17::RmsNormKernel::create for kernel \"" << one_line(kernel_name) << "\"\n";
	common << "#define X17_MODEL_DIM " << config.model_dim << "\n#define X17_IN_KIND " << (config.in_dtype == DType::E4m3 ? 1 : 2) << "\n";
	common << "#define X17_EPS " << format_cpp_f64(config.eps) << "\n";
	auto built = kernel_build::build(kernel_name, common.str(), "rms_norm.hip", "rms_norm_meta.cpp", diag);
	if (!built) return nullptr;
	auto meta = kernel_build::read_metadata_json(built->meta_json_path, diag);
	if (!meta) return nullptr;
	auto out = std::make_unique<RmsNormKernel>();
	auto get = [&](char const *k) { auto v = kernel_build::meta_get(*meta, k); return v ? *v : size_t(0); };
	out->metadata = RmsNormMetadata{get("THREADS_PER_BLOCK"), get("SMEM_BYTES"), get("ROWS_PER_BLOCK")};
	if (out->metadata.THREADS_PER_BLOCK == 0 || !is_pow2(out->metadata.ROWS_PER_BLOCK)) {
		diag.add_error("Invalid JSON metadata in " + built->meta_json_path);
		return nullptr;
	}
	out->name = kernel_name;
	out->files = *built;
	out->config = config;
	if (device) {
		out->kernel = kernel_build::load_kernel(*device->stream, built->code_object_path, "kernel", out->metadata.SMEM_BYTES, diag);
		if (!out->kernel) return nullptr;
		out->device = std::move(device);
	}
	return out;
}

Status RmsNormKernel::launch(Tensor const &inp, Tensor const &outp) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "rms_norm kernel " + name + " was built without a device");
	size_t shp[2], tmp[2];
	Status s = tensor_check::matrix_shape("rms_norm", "inp", inp, std::nullopt, config.model_dim, *device, config.in_dtype, shp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("rms_norm", "out", outp, shp[0], config.model_dim, *device, DType::Int8, tmp);
	if (!s.is_ok()) return s;
	size_t rows = shp[0];
	if ((rows & (metadata.ROWS_PER_BLOCK - 1)) != 0) {     // rms_norm.cu:127
		return Status::err(TensorOpError::Other, "rms_norm rows must be divisible by " + std::to_string(metadata.ROWS_PER_BLOCK) + ", got " + std::to_string(rows));
	}
	if (rows > 0xFFFFFFFFull) return Status::err(TensorOpError::Other, "rms_norm rows exceed 32 bits");
	void *in_ptr = inp.ptr;
	size_t rows_arg = rows;
	void *out_ptr = outp.ptr;
	void *raw_args[3] = {&in_ptr, &rows_arg, &out_ptr};
	size_t grid[3] = {rows / metadata.ROWS_PER_BLOCK, 1, 1};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

// ================================================================ decode

std::unique_ptr<AttnDecodeKernel> AttnDecodeKernel::create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
                                                           AttnDecodeConfig const &config, bool strict_math, Diagnostics &diag) {
	if (config.n_heads == 0) { diag.add_error("decode kernel requires n_heads > 0"); return nullptr; }
	if (config.head_dim != 32 && config.head_dim != 64 && config.head_dim != 128) {
		diag.add_error("decode kernel supports head_dim 32, 64 or 128, got " + std::to_string(config.head_dim));
		return nullptr;
	}
	if (config.cache_capacity == 0 || config.cache_capacity % 16 != 0) {
		diag.add_error("decode kernel requires a cache capacity that is a non-zero multiple of 16, got " + std::to_string(config.cache_capacity));
		return nullptr;
	}
	std::ostringstream common;
	common << "// generated by x17::AttnDecodeKernel::create for kernel \"" << one_line(kernel_name) << "\"\n";
	common << "#define X17_N_HEADS " << config.n_heads << "\n#define X17_HEAD_DIM " << config.head_dim << "\n";
	common << "#define X17_CACHE_CAPACITY " << config.cache_capacity << "\n";
	common << "#define X17_STRICT_MATH " << (strict_math ? 1 : 0) << "\n";
	if (config.out_dtype != DType::Int8 && !(config.row_scales && config.out_dtype == DType::Bf16)) {
		diag.add_error(std::string("decode kernel writes i8, or bf16 with row scales, got ") + dtype_name(config.out_dtype));
		return nullptr;
	}
	if (config.row_scales) {
		common << "#define X17_ATTN_ROW_SCALES 1\n#define X17_ATTN_OUT_BF16 " << (config.out_dtype == DType::Bf16 ? 1 : 0) << "\n";
	}
	auto built = kernel_build::build(kernel_name, common.str(), "attn_decode_i8.hip", "decode_meta.cpp", diag);
	if (!built) return nullptr;
	auto meta = kernel_build::read_metadata_json(built->meta_json_path, diag);
	if (!meta) return nullptr;
	auto out = std::make_unique<AttnDecodeKernel>();
	auto get = [&](char const *k) { auto v = kernel_build::meta_get(*meta, k); return v ? *v : size_t(0); };
	out->metadata = AttnDecodeMetadata{get("THREADS_PER_BLOCK"), get("SMEM_BYTES"), get("HEADS_PER_BLOCK")};
	if (out->metadata.THREADS_PER_BLOCK == 0 || out->metadata.HEADS_PER_BLOCK == 0 || config.n_heads % out->metadata.HEADS_PER_BLOCK != 0) {
		diag.add_error("Invalid JSON metadata in " + built->meta_json_path);
		return nullptr;
	}
	out->name = kernel_name;
	out->files = *built;
	out->config = config;
	if (device) {
		out->kernel = kernel_build::load_kernel(*device->stream, built->code_object_path, "kernel", out->metadata.SMEM_BYTES, diag);
		if (!out->kernel) return nullptr;
		out->device = std::move(device);
	}
	return out;
}

Status AttnDecodeKernel::launch(AttnDecodeArgs const &a) {
	if (!device || !kernel) return Status::err(TensorOpError::Other, "decode kernel " + name + " was built without a device");
	size_t const width = config.n_heads * config.head_dim;
	size_t shp[2], tmp[2];
	Status s = tensor_check::matrix_shape("decode", "q", *a.q, std::nullopt, width, *device, DType::Int8, shp);
	if (!s.is_ok()) return s;
	size_t const seqs = shp[0];
	if (a.cache->shape.size() != 3 || a.cache->shape[0] != seqs || a.cache->shape[1] != config.cache_capacity || a.cache->shape[2] != 2 * width) {
		return Status::err(TensorOpError::Other, "decode input cache must have shape [" + std::to_string(seqs) + ", "
			+ std::to_string(config.cache_capacity) + ", " + std::to_string(2 * width) + "], got " + tensor_check::shape_str(a.cache->shape));
	}
	s = tensor_check::dtype_and_device("decode", "cache", *a.cache, *device, DType::Int8);
	if (!s.is_ok()) return s;
	// cache_len: one u32 per sequence, stored in an f32-typed tensor of the same width
	s = tensor_check::vector_shape("decode", "cache_len", *a.cache_len, seqs, *device, DType::F32);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("decode", "sink_k", *a.sink_k, config.n_heads, config.head_dim, *device, DType::Int8, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("decode", "sink_v", *a.sink_v, config.n_heads, config.head_dim, *device, DType::Int8, tmp);
	if (!s.is_ok()) return s;
	s = tensor_check::vector_shape("decode", "attn_temperature", *a.attn_temperature, config.n_heads, *device, DType::F32);
	if (!s.is_ok()) return s;
	s = tensor_check::matrix_shape("decode", "out", *a.out, seqs, width, *device, config.out_dtype, tmp);
	if (!s.is_ok()) return s;
	bool const any_scale = a.q_scale || a.k_scale || a.v_weight || a.sink_v_weight || a.out_scale;
	if (config.row_scales) {
		if (!a.q_scale || !a.k_scale || !a.v_weight || !a.sink_v_weight || !a.out_scale) {
			return Status::err(TensorOpError::Other, "decode kernel " + name + " needs q_scale, k_scale, v_weight, sink_v_weight and out_scale");
		}
		s = tensor_check::matrix_shape("decode", "q_scale", *a.q_scale, seqs, config.n_heads, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
		for (auto [label, t] : {std::pair<char const *, Tensor const *>{"k_scale", a.k_scale}, {"v_weight", a.v_weight}}) {
			if (t->shape.size() != 3 || t->shape[0] != seqs || t->shape[1] != config.n_heads || t->shape[2] != config.cache_capacity) {
				return Status::err(TensorOpError::Other, std::string("decode input ") + label + " must have shape [" + std::to_string(seqs) + ", "
					+ std::to_string(config.n_heads) + ", " + std::to_string(config.cache_capacity) + "], got " + tensor_check::shape_str(t->shape));
			}
			s = tensor_check::dtype_and_device("decode", label, *t, *device, DType::F32);
			if (!s.is_ok()) return s;
		}
		s = tensor_check::vector_shape("decode", "sink_v_weight", *a.sink_v_weight, config.n_heads, *device, DType::F32);
		if (!s.is_ok()) return s;
		s = tensor_check::vector_shape("decode", "out_scale", *a.out_scale, config.n_heads, *device, DType::F32);
		if (!s.is_ok()) return s;
	} else if (any_scale) {
		return Status::err(TensorOpError::Other, "decode kernel " + name + " was built without row scales");
	}
	if (a.l != nullptr) {
		s = tensor_check::matrix_shape("decode", "l", *a.l, seqs, config.n_heads, *device, DType::F32, tmp);
		if (!s.is_ok()) return s;
	}
	if (a.window_size > 0 && a.window_size % 16 != 0) {
		return Status::err(TensorOpError::Other, "decode window_size must be zero or divisible by 16, got " + std::to_string(a.window_size));
	}
	if (seqs > 0xFFFFFFFFull || a.window_size > 0xFFFFFFFFull) return Status::err(TensorOpError::Other, "decode sizes exceed 32 bits");
	void *q_ptr = a.q->ptr, *cache_ptr = a.cache->ptr, *len_ptr = a.cache_len->ptr, *sk = a.sink_k->ptr, *sv = a.sink_v->ptr;
	void *tp = a.attn_temperature->ptr, *out_ptr = a.out->ptr;
	void *l_ptr = a.l != nullptr ? a.l->ptr : nullptr;
	size_t window_arg = a.window_size;
	void *scale_ptrs[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
	if (config.row_scales) {
		Tensor const *t[5] = {a.q_scale, a.k_scale, a.v_weight, a.sink_v_weight, a.out_scale};
		for (int i = 0; i < 5; ++i) scale_ptrs[i] = t[i]->ptr;
	}
	// the plain kernel takes the first nine arguments only
	void *raw_args[14] = {&q_ptr, &cache_ptr, &len_ptr, &sk, &sv, &tp, &out_ptr, &l_ptr, &window_arg,
	                      &scale_ptrs[0], &scale_ptrs[1], &scale_ptrs[2], &scale_ptrs[3], &scale_ptrs[4]};
	size_t grid[3] = {config.n_heads / metadata.HEADS_PER_BLOCK, seqs, 1};
	size_t block[3] = {metadata.THREADS_PER_BLOCK, 1, 1};
	return kernel->launch(*device->stream, grid, block, metadata.SMEM_BYTES, raw_args);
}

} // namespace x17

// ================================================================ flat C ABI

using namespace x17;

struct X17hTimer { std::unique_ptr<HipTimer> t; };
struct X17hGemmKernel { std::unique_ptr<GemmKernel> k; };
struct X17hAttnKernel { std::unique_ptr<AttnKernel> k; };
struct X17hRmsNormKernel { std::unique_ptr<RmsNormKernel> k; };
struct X17hDecodeKernel { std::unique_ptr<AttnDecodeKernel> k; };

namespace {
	thread_local std::string g_last_error;
	thread_local std::string g_last_diag;

	int fail(std::string msg) { g_last_error = std::move(msg); return 1; }
	int fail(ErrPack const &e) { g_last_error = e.message; return 1; }
	int from_status(Status const &s) { return s.is_ok() ? 0 : fail(*s.error); }

	void stash_diag(Diagnostics const &d) {
		g_last_diag.clear();
		for (auto const &x : d.list) {
			g_last_diag += x.is_error ? "error: " : "warning: ";
			g_last_diag += x.message;
			g_last_diag += "\n";
		}
	}
	int fail_diag(char const *what, Diagnostics const &d) {
		stash_diag(d);
		std::string msg = std::string("failed to generate ") + what + " kernel; " + std::to_string(d.err_count) + " error(s)";
		for (auto const &x : d.list) if (x.is_error) { msg += "\n" + x.message; }
		return fail(std::move(msg));
	}
	bool valid_dtype(int d) { return d >= 0 && d <= 3; }
}

extern "C" {

char const *x17h_last_error(void) { return g_last_error.c_str(); }
char const *x17h_last_diagnostics(void) { return g_last_diag.c_str(); }

size_t x17h_move_diagnostic_text(void *diag, char *out, size_t capacity) {
	if (out == nullptr || capacity == 0) return 0;
	size_t have = strnlen(out, capacity - 1);
	FfiBufferImpl buf;
	buf.data.assign(out, have);
	if (diag != nullptr) {
		x17ai_move_diagnostic(reinterpret_cast<X17DiagnosticBuffer *>(diag), buf.as_ffi());
	}
	size_t n = buf.data.size() < capacity - 1 ? buf.data.size() : capacity - 1;
	std::memcpy(out, buf.data.data(), n);
	out[n] = 0;
	return n;
}

int x17h_device_new(size_t device_id, X17hDevice **out) {
	try {
		auto r = HipDevice::create(device_id);
		if (!r.is_ok()) return fail(*r.error);
		*out = new X17hDevice{*r.value};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17h_device_free(X17hDevice *d) { delete d; }
int x17h_device_synchronize(X17hDevice *d) { return from_status(d->dev->synchronize()); }
char const *x17h_device_name(X17hDevice *d) { return d->dev->name().c_str(); }

int x17h_tensor_new_empty(X17hDevice *dev, size_t const *shape, size_t ndim, int dtype, X17hTensor **out) {
	try {
		if (!valid_dtype(dtype)) return fail("unknown dtype");
		std::shared_ptr<Device> device;
		if (dev != nullptr) device = dev->dev; else device = std::make_shared<CpuDevice>();
		auto r = Tensor::new_empty(std::vector<size_t>(shape, shape + ndim), DType(dtype), device);
		if (!r.is_ok()) return fail(*r.error);
		*out = new X17hTensor{*r.value};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17h_tensor_free(X17hTensor *t) { delete t; }
int x17h_tensor_upload(X17hTensor *t, void const *src, size_t bytes) {
	if (bytes != t->t->bytes) return fail("upload size " + std::to_string(bytes) + " does not match tensor size " + std::to_string(t->t->bytes));
	return from_status(t->t->device->upload_data(static_cast<uint8_t const *>(src), t->t->ptr, bytes));
}
int x17h_tensor_download(X17hTensor *t, void *dst, size_t bytes) {
	if (bytes != t->t->bytes) return fail("download size " + std::to_string(bytes) + " does not match tensor size " + std::to_string(t->t->bytes));
	return from_status(t->t->device->download_data(t->t->ptr, static_cast<uint8_t *>(dst), bytes));
}
int x17h_tensor_from_safetensors_file(X17hDevice *dev, char const *path, X17hTensor **out, int *dtype, size_t *shape, size_t *ndim) {
	try {
		std::shared_ptr<Device> device;
		if (dev != nullptr) device = dev->dev; else device = std::make_shared<CpuDevice>();
		auto r = Tensor::from_safetensors_file(path, device);
		if (!r.is_ok()) return fail(*r.error);
		if ((*r.value)->shape.size() > 8) return fail("tensors of more than 8 dimensions are not supported here");
		*dtype = int((*r.value)->dtype);
		*ndim = (*r.value)->shape.size();
		for (size_t i = 0; i < *ndim; ++i) shape[i] = (*r.value)->shape[i];
		*out = new X17hTensor{*r.value};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
int x17h_tensor_save_safetensors_file(X17hTensor *t, char const *path) {
	try {
		return from_status(t->t->save_safetensors_file(path));
	} catch (std::exception const &e) { return fail(e.what()); }
}
void *x17h_tensor_device_ptr(X17hTensor *t) { return t->t->ptr; }
size_t x17h_tensor_bytes(X17hTensor *t) { return t->t->bytes; }
int x17h_tensor_reshape(X17hTensor *t, size_t const *shape, size_t ndim) {
	size_t n = 1;
	for (size_t i = 0; i < ndim; ++i) n *= shape[i];
	if (n != t->t->elems()) return fail("cannot reshape: element counts differ");
	t->t->shape.assign(shape, shape + ndim);
	return 0;
}

int x17h_timer_new(X17hDevice *dev, X17hTimer **out) {
	auto r = HipTimer::create(*dev->dev);
	if (!r.is_ok()) return fail(*r.error);
	*out = new X17hTimer{std::move(*r.value)};
	return 0;
}
void x17h_timer_free(X17hTimer *t) { delete t; }
int x17h_timer_start(X17hTimer *t) { return from_status(t->t->start()); }
int x17h_timer_stop(X17hTimer *t) { return from_status(t->t->stop()); }
int x17h_timer_elapsed_seconds(X17hTimer *t, double *seconds) {
	auto r = t->t->elapsed_seconds();
	if (!r.is_ok()) return fail(*r.error);
	*seconds = *r.value;
	return 0;
}

int x17h_gemm_kernel_new(X17hDevice *dev, char const *kernel_name, X17hGemmConfig const *c, X17hGemmKernel **out) {
	try {
		if (!valid_dtype(c->a_dtype) || !valid_dtype(c->b_dtype) || !valid_dtype(c->c_dtype)) return fail("unknown dtype");
		GemmConfig g{
			GemmInputConfig{DType(c->a_dtype), c->a_cols, c->a_rows ? std::optional<size_t>(c->a_rows) : std::nullopt, c->a_trans != 0},
			GemmInputConfig{DType(c->b_dtype), c->b_cols, c->b_rows ? std::optional<size_t>(c->b_rows) : std::nullopt, c->b_trans != 0},
			DType(c->c_dtype)};
		Scale inp{c->inp_scale, "inp_scale"}, outs{c->out_scale, "out_scale"};
		EpilogueConfig e;
		switch (c->epilogue) {
			case X17H_EPI_SCALE: e = ScaleConfig{inp, outs}; break;
			case X17H_EPI_GEGLU: e = GeGluConfig{inp, outs}; break;
			case X17H_EPI_RESIDUAL: e = ResidualConfig{inp, outs}; break;
			case X17H_EPI_RMSNORM: e = RMSNormConfig{c->eps, c->head_dim, c->sep_dim, inp, outs}; break;
			case X17H_EPI_DEQUANT: e = DequantConfig{c->activation == X17H_ACT_GEGLU}; break;
			case X17H_EPI_QNORM: e = QNormConfig{c->eps, c->head_dim, outs, Scale{c->inp_scale == 0.0 ? 1.0 : c->inp_scale, "post_scale"}}; break;
			case X17H_EPI_QKV:
				e = QkvConfig{c->q_cols, ScaleConfig{Scale{c->q_inp_scale, "q inp_scale"}, Scale{c->q_out_scale, "q out_scale"}},
				              RMSNormConfig{c->eps, c->head_dim, c->sep_dim, inp, outs}};
				break;
			default: return fail("unknown epilogue");
		}
		Diagnostics diag;
		auto k = GemmKernel::create(dev != nullptr ? dev->dev : nullptr, kernel_name, g, e, c->strict_math != 0, diag);
		if (!k) return fail_diag("GEMM", diag);
		stash_diag(diag);
		*out = new X17hGemmKernel{std::move(k)};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17h_gemm_kernel_free(X17hGemmKernel *k) { delete k; }
int x17h_gemm_kernel_launch(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b, X17hTensor *c, X17hTensor *extra) {
	if (a == nullptr || b == nullptr || c == nullptr) return fail("GEMM launch needs a, b and c");
	GemmArgs args{a->t.get(), b->t.get(), c->t.get(), extra != nullptr ? extra->t.get() : nullptr};
	return from_status(k->k->launch(args));
}
int x17h_gemm_kernel_launch_dequant(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b, X17hTensor *c,
                                    X17hTensor *row_scale, X17hTensor *col_scale) {
	if (a == nullptr || b == nullptr || c == nullptr || row_scale == nullptr || col_scale == nullptr) {
		return fail("dequant GEMM launch needs a, b, c, row_scale and col_scale");
	}
	GemmArgs args{a->t.get(), b->t.get(), c->t.get(), row_scale->t.get(), col_scale->t.get()};
	return from_status(k->k->launch(args));
}
int x17h_gemm_kernel_launch_qkv(X17hGemmKernel *k, X17hTensor *x, X17hTensor *q_weights, X17hTensor *kv_weights,
                                X17hTensor *q, X17hTensor *kv, X17hTensor *rrms) {
	if (x == nullptr || q_weights == nullptr || kv_weights == nullptr || q == nullptr || kv == nullptr || rrms == nullptr) {
		return fail("fused q + kv GEMM launch needs x, both weight matrices, both outputs and rrms");
	}
	GemmArgs args{x->t.get(), q_weights->t.get(), q->t.get(), rrms->t.get(), nullptr, kv_weights->t.get(), kv->t.get()};
	return from_status(k->k->launch(args));
}
double x17h_gemm_kernel_n_ops(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b) { return k->k->n_ops(*a->t, *b->t); }
int x17h_gemm_kernel_metadata(X17hGemmKernel *k, size_t out[4]) {
	out[0] = k->k->metadata.THREADS_PER_BLOCK; out[1] = k->k->metadata.SMEM_BYTES;
	out[2] = k->k->metadata.M_PER_BLOCK; out[3] = k->k->metadata.N_PER_BLOCK;
	return 0;
}
static int attrs_out(HipKernel *k, int32_t out[9]) {
	if (k == nullptr) return fail("kernel was built without a device");
	auto r = k->attrs();
	if (!r.is_ok()) return fail(*r.error);
	std::memcpy(out, &*r.value, sizeof(int32_t) * 9);
	return 0;
}
int x17h_gemm_kernel_attrs(X17hGemmKernel *k, int32_t out[9]) { return attrs_out(k->k->kernel.get(), out); }

int x17h_attn_kernel_new(X17hDevice *dev, char const *kernel_name, X17hAttnConfig const *c, X17hAttnKernel **out) {
	try {
		if (!valid_dtype(c->dtype)) return fail("unknown dtype");
		if (!valid_dtype(c->out_dtype)) return fail("unknown out_dtype");
		AttnKernelConfig cfg{DType(c->dtype), c->n_heads, c->head_dim, c->q_stride, c->kv_stride, c->o_stride,
		                     c->row_scales != 0, DType(c->out_dtype), c->backward_q != 0, c->backward_kv != 0};
		Diagnostics diag;
		auto k = AttnKernel::create(dev != nullptr ? dev->dev : nullptr, kernel_name, cfg, c->strict_math != 0, diag);
		if (!k) return fail_diag("attention", diag);
		stash_diag(diag);
		*out = new X17hAttnKernel{std::move(k)};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17h_attn_kernel_free(X17hAttnKernel *k) { delete k; }
int x17h_attn_kernel_launch(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k, X17hTensor *sink_v,
                            X17hTensor *temp, X17hTensor *out, X17hTensor *l, size_t window_size, size_t batch) {
	if (!q || !kv || !sink_k || !sink_v || !temp || !out) return fail("attention launch needs q, kv, sinks, temperature and out");
	AttnKernelArgs a{q->t.get(), kv->t.get(), sink_k->t.get(), sink_v->t.get(), temp->t.get(), out->t.get(),
	                 l != nullptr ? l->t.get() : nullptr, window_size, batch};
	return from_status(k->k->launch(a));
}
int x17h_attn_kernel_launch_row_scaled(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k, X17hTensor *sink_v,
                                       X17hTensor *temp, X17hTensor *out, X17hTensor *l, size_t window_size, size_t batch,
                                       X17hTensor *q_scale, X17hTensor *k_scale, X17hTensor *v_weight,
                                       X17hTensor *sink_v_weight, X17hTensor *out_scale) {
	if (!q || !kv || !sink_k || !sink_v || !temp || !out) return fail("attention launch needs q, kv, sinks, temperature and out");
	if (!q_scale || !k_scale || !v_weight || !sink_v_weight || !out_scale) return fail("row-scaled attention launch needs all five scale tensors");
	AttnKernelArgs a{q->t.get(), kv->t.get(), sink_k->t.get(), sink_v->t.get(), temp->t.get(), out->t.get(),
	                 l != nullptr ? l->t.get() : nullptr, window_size, batch,
	                 q_scale->t.get(), k_scale->t.get(), v_weight->t.get(), sink_v_weight->t.get(), out_scale->t.get()};
	return from_status(k->k->launch(a));
}
int x17h_attn_kernel_launch_d_q(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k, X17hTensor *sink_v,
                                X17hTensor *temp, X17hTensor *out, X17hTensor *d_out, X17hTensor *d_q, X17hTensor *l, X17hTensor *d,
                                size_t window_size, size_t batch) {
	if (q == nullptr || kv == nullptr || sink_k == nullptr || sink_v == nullptr || temp == nullptr || out == nullptr
	    || d_out == nullptr || d_q == nullptr || l == nullptr) {
		return fail("attention backward launch needs q, kv, the sinks, the temperatures, out, d_out, d_q and l");
	}
	AttnKernelArgs args{q->t.get(), kv->t.get(), sink_k->t.get(), sink_v->t.get(), temp->t.get(), out->t.get(), l->t.get(), window_size, batch};
	args.d_out = d_out->t.get();
	args.d_q = d_q->t.get();
	args.d = d != nullptr ? d->t.get() : nullptr;
	return from_status(k->k->launch_d_q(args));
}
int x17h_attn_kernel_launch_d_kv(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *temp, X17hTensor *d_out,
                                 X17hTensor *l, X17hTensor *d, X17hTensor *d_kv, size_t window_size, size_t batch) {
	if (q == nullptr || kv == nullptr || temp == nullptr || d_out == nullptr || l == nullptr || d == nullptr || d_kv == nullptr) {
		return fail("attention backward (k, v) launch needs q, kv, the temperatures, d_out, l, d and d_kv");
	}
	AttnKernelArgs args{q->t.get(), kv->t.get(), nullptr, nullptr, temp->t.get(), nullptr, l->t.get(), window_size, batch};
	args.d_out = d_out->t.get();
	args.d = d->t.get();
	args.d_kv = d_kv->t.get();
	return from_status(k->k->launch_d_kv(args));
}
double x17h_attn_kernel_n_ops(X17hAttnKernel *k, size_t seq_len, size_t window_size) { return k->k->config.n_ops(seq_len, window_size); }
int x17h_attn_kernel_metadata(X17hAttnKernel *k, size_t out[3]) {
	out[0] = k->k->metadata.THREADS_PER_BLOCK; out[1] = k->k->metadata.SMEM_BYTES; out[2] = k->k->metadata.Q_PER_BLOCK;
	return 0;
}
int x17h_attn_kernel_attrs(X17hAttnKernel *k, int32_t out[9]) { return attrs_out(k->k->kernel.get(), out); }

int x17h_rms_norm_kernel_new(X17hDevice *dev, char const *kernel_name, int in_dtype, size_t model_dim, double eps, X17hRmsNormKernel **out) {
	try {
		if (!valid_dtype(in_dtype)) return fail("unknown dtype");
		Diagnostics diag;
		auto k = RmsNormKernel::create(dev != nullptr ? dev->dev : nullptr, kernel_name, RmsNormConfig{DType(in_dtype), model_dim, eps}, diag);
		if (!k) return fail_diag("rms_norm", diag);
		stash_diag(diag);
		*out = new X17hRmsNormKernel{std::move(k)};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17h_rms_norm_kernel_free(X17hRmsNormKernel *k) { delete k; }
int x17h_rms_norm_kernel_launch(X17hRmsNormKernel *k, X17hTensor *inp, X17hTensor *out) {
	if (!inp || !out) return fail("rms_norm launch needs inp and out");
	return from_status(k->k->launch(*inp->t, *out->t));
}

int x17h_decode_kernel_new(X17hDevice *dev, char const *kernel_name, size_t n_heads, size_t head_dim, size_t cache_capacity,
                           int strict_math, X17hDecodeKernel **out) {
	try {
		Diagnostics diag;
		auto k = AttnDecodeKernel::create(dev != nullptr ? dev->dev : nullptr, kernel_name,
		                                  AttnDecodeConfig{n_heads, head_dim, cache_capacity}, strict_math != 0, diag);
		if (!k) return fail_diag("decode", diag);
		stash_diag(diag);
		*out = new X17hDecodeKernel{std::move(k)};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
int x17h_decode_kernel_new_row_scaled(X17hDevice *dev, char const *kernel_name, size_t n_heads, size_t head_dim, size_t cache_capacity,
                                      int strict_math, int out_dtype, X17hDecodeKernel **out) {
	try {
		if (!valid_dtype(out_dtype)) return fail("unknown out_dtype");
		Diagnostics diag;
		auto k = AttnDecodeKernel::create(dev != nullptr ? dev->dev : nullptr, kernel_name,
		                                  AttnDecodeConfig{n_heads, head_dim, cache_capacity, true, DType(out_dtype)}, strict_math != 0, diag);
		if (!k) return fail_diag("decode", diag);
		stash_diag(diag);
		*out = new X17hDecodeKernel{std::move(k)};
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
int x17h_decode_kernel_launch_row_scaled(X17hDecodeKernel *k, X17hTensor *q, X17hTensor *cache, X17hTensor *cache_len, X17hTensor *sink_k,
                                         X17hTensor *sink_v, X17hTensor *temp, X17hTensor *out, X17hTensor *l, size_t window_size,
                                         X17hTensor *q_scale, X17hTensor *k_scale, X17hTensor *v_weight,
                                         X17hTensor *sink_v_weight, X17hTensor *out_scale) {
	if (!q || !cache || !cache_len || !sink_k || !sink_v || !temp || !out) return fail("decode launch needs q, cache, cache_len, sinks, temperature and out");
	if (!q_scale || !k_scale || !v_weight || !sink_v_weight || !out_scale) return fail("row-scaled decode launch needs all five scale tensors");
	AttnDecodeArgs a{q->t.get(), cache->t.get(), cache_len->t.get(), sink_k->t.get(), sink_v->t.get(), temp->t.get(), out->t.get(),
	                 l != nullptr ? l->t.get() : nullptr, window_size,
	                 q_scale->t.get(), k_scale->t.get(), v_weight->t.get(), sink_v_weight->t.get(), out_scale->t.get()};
	return from_status(k->k->launch(a));
}
void x17h_decode_kernel_free(X17hDecodeKernel *k) { delete k; }
int x17h_decode_kernel_launch(X17hDecodeKernel *k, X17hTensor *q, X17hTensor *cache, X17hTensor *cache_len, X17hTensor *sink_k,
                              X17hTensor *sink_v, X17hTensor *temp, X17hTensor *out, X17hTensor *l, size_t window_size) {
	if (!q || !cache || !cache_len || !sink_k || !sink_v || !temp || !out) return fail("decode launch needs q, cache, cache_len, sinks, temperature and out");
	AttnDecodeArgs a{q->t.get(), cache->t.get(), cache_len->t.get(), sink_k->t.get(), sink_v->t.get(), temp->t.get(), out->t.get(),
	                 l != nullptr ? l->t.get() : nullptr, window_size};
	return from_status(k->k->launch(a));
}

} // extern "C"
