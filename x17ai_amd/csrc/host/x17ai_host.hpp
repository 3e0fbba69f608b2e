// x17ai_host.hpp -- the host-side operator layer above the C-ABI shim, in C++.
//
// The reference's operator layer for this path is Rust (no Rust toolchain exists where this
// library is built), so it is mirrored here type by type, with the same names, argument
// meaning and error behaviour:
//
//   this file                      reference
//   -----------------------------  -------------------------------------------------------
//   ErrPack, TensorOpError         src/lib.rs (error values, never exceptions across the API)
//   FfiBufferImpl                  src/util/ffi_buffer.rs:13-103
//   HipStream/HipKernel/HipTimer   src/device/cuda/cuda_shim.rs:207-562 (wrappers over the FFI)
//   Device, HipDevice, CpuDevice   src/device.rs:35-67, src/device/cuda.rs:25-101, src/device/cpu.rs
//   DType, Tensor                  src/dtype.rs:1-61, src/tensor.rs:23-256 (contiguous only)
//   tensor_check::*                src/device/cuda/tensor_check.rs:19-101
//   kernel_build::*                src/device/cuda/kernel_build.rs:38-220 (hipcc instead of nvcc)
//   GemmKernel<Epilogue> & co.     src/device/cuda/gemm.rs:28-918
//   AttnKernel & co.               src/device/cuda/attn.rs:45-448
//   RmsNormKernel                  rms_norm.cu:55-113 given the same kernel-object shape
//   AttnDecodeKernel               no reference counterpart (single-token decode, defined in attn_decode_i8.hip)
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <variant>
#include <vector>

#include "../../../include/x17ai_hip_shim.h"

namespace x17 {

// ---------------------------------------------------------------- errors

enum class TensorOpError { Device, Other, Alloc, Io };

struct ErrPack {
	TensorOpError code;
	std::string message;
	std::shared_ptr<ErrPack> nested;
};

template<typename T>
struct Result {
	std::optional<T> value;
	std::optional<ErrPack> error;
	static Result ok(T v) { Result r; r.value = std::move(v); return r; }
	static Result err(ErrPack e) { Result r; r.error = std::move(e); return r; }
	bool is_ok() const { return !error.has_value(); }
};

struct Status {
	std::optional<ErrPack> error;
	static Status ok() { return Status{}; }
	static Status err(TensorOpError c, std::string m) { Status s; s.error = ErrPack{c, std::move(m), nullptr}; return s; }
	static Status err(ErrPack e) { Status s; s.error = std::move(e); return s; }
	bool is_ok() const { return !error.has_value(); }
};

// src/lib.rs Diagnostics: warnings and errors collected while a kernel is generated
struct Diagnostic { bool is_error; std::string message; };
struct Diagnostics {
	std::vector<Diagnostic> list;
	size_t err_count = 0;
	void add_error(std::string m) { list.push_back({true, std::move(m)}); ++err_count; }
	void add_warning(std::string m) { list.push_back({false, std::move(m)}); }
};

// ---------------------------------------------------------------- FfiBuffer over std::string

struct FfiBufferImpl {
	std::string data;
	X17FfiBuffer as_ffi();
};

std::string diagnostic_to_string(X17DiagnosticBuffer *diag, char const *fallback);

// ---------------------------------------------------------------- dtype

enum class DType : int { E4m3 = 0, Int8 = 1, Bf16 = 2, F32 = 3 };
size_t dtype_bytes(DType d);
char const *dtype_name(DType d);

// ---------------------------------------------------------------- device

using DevicePtr = void *;

struct Device {
	virtual ~Device() = default;
	virtual std::string const &name() const = 0;
	virtual bool is_cpu() const { return false; }
	virtual Result<DevicePtr> new_buffer(size_t bytes) = 0;
	virtual void drop_buffer(DevicePtr p, size_t bytes) = 0;
	virtual Status upload_data(uint8_t const *src, DevicePtr dst, size_t bytes) = 0;
	virtual Status download_data(DevicePtr src, uint8_t *dst, size_t bytes) = 0;
};

struct CpuDevice final : Device {
	std::string name_ = "CPU";
	std::string const &name() const override { return name_; }
	bool is_cpu() const override { return true; }
	Result<DevicePtr> new_buffer(size_t bytes) override;
	void drop_buffer(DevicePtr p, size_t bytes) override;
	Status upload_data(uint8_t const *src, DevicePtr dst, size_t bytes) override;
	Status download_data(DevicePtr src, uint8_t *dst, size_t bytes) override;
};

struct HipStream {
	X17HipContextHandle *ctx = nullptr;
	X17HipStreamHandle *stream = nullptr;
	static Result<std::unique_ptr<HipStream>> create(size_t device_id);
	~HipStream();
	Status synchronize();
};

struct HipModule {
	X17HipModuleHandle *module = nullptr;
	~HipModule();
};

struct HipKernel {
	std::shared_ptr<HipModule> module;     // a kernel keeps its module alive (cuda_shim.rs:445-449)
	X17HipKernelHandle *kernel = nullptr;
	Status launch(HipStream &stream, size_t const (&grid)[3], size_t const (&block)[3], size_t smem, void **args);
	Result<X17HipKernelAttrs> attrs();
	~HipKernel();
};

struct HipDevice final : Device {
	std::string name_;
	std::unique_ptr<HipStream> stream;
	static Result<std::shared_ptr<HipDevice>> create(size_t device_id);
	std::string const &name() const override { return name_; }
	Status synchronize() { return stream->synchronize(); }
	Result<DevicePtr> new_buffer(size_t bytes) override;
	void drop_buffer(DevicePtr p, size_t bytes) override;
	Status upload_data(uint8_t const *src, DevicePtr dst, size_t bytes) override;
	Status download_data(DevicePtr src, uint8_t *dst, size_t bytes) override;
};

struct HipTimer {
	X17HipTimerHandle *timer = nullptr;
	static Result<std::unique_ptr<HipTimer>> create(HipDevice &device);
	~HipTimer();
	Status start();
	Status stop();
	Result<double> elapsed_seconds();
};

// ---------------------------------------------------------------- tensor (contiguous, no views)

struct Tensor {
	DType dtype;
	std::vector<size_t> shape;
	DevicePtr ptr = nullptr;
	size_t bytes = 0;
	std::shared_ptr<Device> device;

	static Result<std::shared_ptr<Tensor>> new_empty(std::vector<size_t> shape, DType dtype, std::shared_ptr<Device> device);
	// src/tensor.rs:155-179 -- a safetensors file holding exactly one tensor of dtype F8_E4M3 / I8 / BF16 / F32;
	// the bytes are uploaded as they are (int8 and e4m3 tensors are codes).
	static Result<std::shared_ptr<Tensor>> from_safetensors_file(std::string const &path, std::shared_ptr<Device> device);
	// src/tensor.rs:213-249 -- CPU tensors only; written as the single entry "tensor"; parent directories are created.
	Status save_safetensors_file(std::string const &path) const;
	~Tensor();
	size_t elems() const;
	bool is_on_device(Device const *d) const { return device.get() == d; }   // pointer identity, tensor.rs:87-91
};

// ---------------------------------------------------------------- kernel build

namespace kernel_build {
	struct BuiltKernel {
		std::string dir_path, common_path, code_object_path, meta_json_path;
		bool cache_hit = false;
	};
	// Renders common.h, compiles <source> (a file of csrc/kernels) for gfx950 and runs the meta
	// program, unless an identical build is already cached under <cache>/<name>/.
	std::optional<BuiltKernel> build(std::string const &kernel_name, std::string const &common_text,
	                                 std::string const &source_file, std::string const &meta_source_file,
	                                 Diagnostics &diag);
	std::optional<std::vector<std::pair<std::string, size_t>>> read_metadata_json(std::string const &path, Diagnostics &diag);
	std::string kernels_dir();
	std::string cache_dir();
	std::optional<size_t> meta_get(std::vector<std::pair<std::string, size_t>> const &meta, char const *key);
	// kernel_build.rs:161-198
	std::unique_ptr<HipKernel> load_kernel(HipStream &stream, std::string const &code_object_path, char const *name,
	                                       size_t smem_bytes, Diagnostics &diag);
}

// ---------------------------------------------------------------- GEMM (src/device/cuda/gemm.rs)

struct Scale { double value; std::string description; };
struct ScaleConfig { Scale inp_scale, out_scale; };
struct RMSNormConfig { double eps; size_t head_dim; size_t sep_dim; Scale inp_scale, out_scale; };
struct ResidualConfig { Scale inp_scale, out_scale; };
struct GeGluConfig { Scale inp_scale, out_scale; };
// Run-time per-row and per-column dequantisation scales, bf16 output, optional GeGLU over column pairs
// (no counterpart in gemm.rs: the superset for symmetric per-row / per-channel int8 quantisation).
struct DequantConfig { bool geglu; };
// The reference's older Q writer (cuda/qkvg_fwd_i8.cuh:145-219; hook cuda/gemm_b8.cuh:761-824): every head_dim raw
// columns are one L2-normalised head, multiplied by a learned bf16 scale per column given at launch.
struct QNormConfig { double eps; size_t head_dim; Scale out_scale; Scale post_scale{1.0, "1"}; };   // post_scale: the factor of the old writer's base class (1 = none)
// The q and the kv projection of src/main.rs:387-493 as ONE launch over the same token rows (no counterpart in
// gemm.rs, which launches them one after the other): raw columns [0, q_cols) come from the q weights and go through
// the Scale writer `q`, the remaining b.rows - q_cols come from the kv weights and go through the RMSNorm writer `kv`.
struct QkvConfig { size_t q_cols; ScaleConfig q; RMSNormConfig kv; };
using EpilogueConfig = std::variant<ScaleConfig, GeGluConfig, ResidualConfig, RMSNormConfig, DequantConfig, QNormConfig, QkvConfig>;   // index = X17_EPILOGUE

struct GemmInputConfig { DType dtype; size_t cols; std::optional<size_t> rows; bool trans; };
struct GemmConfig { GemmInputConfig a, b; DType c_dtype; };

// MAX_BLOCKS (0 = one workgroup per tile, as in the reference) caps the grid of the persistent kernel
struct GemmLauncherMetadata { size_t THREADS_PER_BLOCK, SMEM_BYTES, M_PER_BLOCK, N_PER_BLOCK, MAX_BLOCKS; };

struct GemmArgs {
	Tensor const *a; Tensor const *b; Tensor const *c;
	Tensor const *extra;     // rrms (RMSNorm, Qkv), residual (Residual), row scales (Dequant), q_norm_scales (QNorm), else null
	Tensor const *extra2 = nullptr;   // column scales (Dequant epilogue)
	// Qkv only: a = x, b = q weights, c = q, extra = rrms, and the kv weights and the kv output:
	Tensor const *b2 = nullptr;
	Tensor const *c2 = nullptr;
};

struct GemmKernel {
	std::string name;
	kernel_build::BuiltKernel files;
	int epilogue_kind = 0;                // 0 scale, 1 geglu, 2 residual, 3 rmsnorm, 4 dequant, 5 qnorm, 6 fused q + kv
	size_t q_cols = 0;                    // fused q + kv: raw columns that belong to q
	size_t a_cols = 0;
	std::optional<size_t> b_rows;
	DType a_dtype, b_dtype, c_dtype;
	size_t head_dim = 0, sep_dim = 0;
	bool dequant_geglu = false;
	GemmLauncherMetadata metadata{};
	std::shared_ptr<HipDevice> device;    // null for a build-only kernel
	std::unique_ptr<HipKernel> kernel;

	// device == nullptr: generate + compile only (what a build step without a GPU does)
	static std::unique_ptr<GemmKernel> create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
	                                           GemmConfig const &gemm_config, EpilogueConfig const &epilogue_config,
	                                           bool strict_math, Diagnostics &diag);
	Status launch(GemmArgs const &args);
	Status launch_qkv(GemmArgs const &args, size_t a_rows);   // epilogue_kind 6, reached through launch()
	double n_ops(Tensor const &a, Tensor const &b) const;     // 2*M*K*N_raw, gemm.rs:445-449
};

// ---------------------------------------------------------------- attention (src/device/cuda/attn.rs)

struct AttnKernelConfig {
	DType dtype; size_t n_heads, head_dim, q_stride, kv_stride, o_stride;
	// Extension (the reference's codes all share the scale 1/8): one f32 scale per (row, head) for q, k and v.
	// out_dtype is Int8 (FixedI8 codes) or, in the row-scaled build only, Bf16 (real values).
	bool row_scales = false;
	DType out_dtype = DType::Int8;
	// Builds the backward-with-respect-to-q kernel (attn_d_q_i8.hip; the reference's attn_d_q.cuh is its bf16
	// generation) instead of the forward: launched through AttnKernel::launch_d_q.
	bool backward_q = false;
	// Builds the backward-with-respect-to-k-and-v kernel (attn_d_kv_i8.hip; structure of attn_d_kv.cuh): launched
	// through AttnKernel::launch_d_kv.
	bool backward_kv = false;
	size_t heads_per_kernel() const;
	size_t head_group_cnt() const;
	size_t head_group_dim() const;
	double n_ops(size_t seq_len, size_t window_size) const;   // attn.rs:72-84
	bool validate(Diagnostics &diag) const;
};

struct AttnKernelArgs {
	Tensor const *q, *kv, *sink_k, *sink_v, *attn_temperature, *out, *l;   // l may be null
	size_t window_size;
	size_t batch = 1;       // extension: `batch` sequences of seq_len/batch rows, each with its own causal origin
	// row-scaled kernels only: f32 [n_heads, rows] scales of q and k, weights (<= 1) of the value rows, and per head
	// the weight of the sink value and the output scale
	Tensor const *q_scale = nullptr, *k_scale = nullptr, *v_weight = nullptr, *sink_v_weight = nullptr, *out_scale = nullptr;
	// backward_q kernels only: `out` is the forward's output (an input here), `l` its log-sum-exp (required);
	// d_out bf16 [rows, o_stride] in, d_q bf16 [rows, q_stride] out, d f32 [n_heads, rows] out (may be null)
	Tensor const *d_out = nullptr, *d_q = nullptr, *d = nullptr;
	// backward_kv kernels only: q, kv, attn_temperature, d_out, l and d (the dQ pass's D, required) in;
	// d_kv bf16 [rows, kv_stride] out, in the layout of kv (per head dK then dV)
	Tensor const *d_kv = nullptr;
};

struct AttnLauncherMetadata { size_t THREADS_PER_BLOCK, SMEM_BYTES, Q_PER_BLOCK; };

struct AttnKernel {
	std::string name;
	kernel_build::BuiltKernel files;
	AttnKernelConfig config;
	AttnLauncherMetadata metadata{};
	std::shared_ptr<HipDevice> device;
	std::unique_ptr<HipKernel> kernel;
	static std::unique_ptr<AttnKernel> create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
	                                           AttnKernelConfig const &config, bool strict_math, Diagnostics &diag);
	Status launch(AttnKernelArgs const &args);
	Status launch_d_q(AttnKernelArgs const &args);
	Status launch_d_kv(AttnKernelArgs const &args);
};

// ---------------------------------------------------------------- rms_norm, decode

struct RmsNormConfig { DType in_dtype; size_t model_dim; double eps; };
struct RmsNormMetadata { size_t THREADS_PER_BLOCK, SMEM_BYTES, ROWS_PER_BLOCK; };

struct RmsNormKernel {
	std::string name;
	kernel_build::BuiltKernel files;
	RmsNormConfig config;
	RmsNormMetadata metadata{};
	std::shared_ptr<HipDevice> device;
	std::unique_ptr<HipKernel> kernel;
	static std::unique_ptr<RmsNormKernel> create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
	                                              RmsNormConfig const &config, Diagnostics &diag);
	Status launch(Tensor const &inp, Tensor const &out);
};

struct AttnDecodeConfig {
	size_t n_heads, head_dim, cache_capacity;
	bool row_scales = false;             // as AttnKernelConfig::row_scales
	DType out_dtype = DType::Int8;       // Int8, or Bf16 with row scales
};
struct AttnDecodeMetadata { size_t THREADS_PER_BLOCK, SMEM_BYTES, HEADS_PER_BLOCK; };
struct AttnDecodeArgs {
	Tensor const *q, *cache, *cache_len, *sink_k, *sink_v, *attn_temperature, *out, *l;   // l may be null
	size_t window_size;
	// row-scaled kernels only: q_scale [S, H], k_scale and v_weight [S, H, capacity], sink_v_weight and out_scale [H]
	Tensor const *q_scale = nullptr, *k_scale = nullptr, *v_weight = nullptr, *sink_v_weight = nullptr, *out_scale = nullptr;
	// backward_q kernels only: `out` is the forward's output (an input here), `l` its log-sum-exp (required);
	// d_out bf16 [rows, o_stride] in, d_q bf16 [rows, q_stride] out, d f32 [n_heads, rows] out (may be null)
	Tensor const *d_out = nullptr, *d_q = nullptr, *d = nullptr;
	// backward_kv kernels only: q, kv, attn_temperature, d_out, l and d (the dQ pass's D, required) in;
	// d_kv bf16 [rows, kv_stride] out, in the layout of kv (per head dK then dV)
	Tensor const *d_kv = nullptr;
};

struct AttnDecodeKernel {
	std::string name;
	kernel_build::BuiltKernel files;
	AttnDecodeConfig config;
	AttnDecodeMetadata metadata{};
	std::shared_ptr<HipDevice> device;
	std::unique_ptr<HipKernel> kernel;
	static std::unique_ptr<AttnDecodeKernel> create(std::shared_ptr<HipDevice> device, std::string const &kernel_name,
	                                                 AttnDecodeConfig const &config, bool strict_math, Diagnostics &diag);
	Status launch(AttnDecodeArgs const &args);
};

} // namespace x17

// The handles of the flat C ABI (include/x17ai_host.h) that other libraries built on this layer take apart
struct X17hDevice { std::shared_ptr<x17::HipDevice> dev; };
struct X17hTensor { std::shared_ptr<x17::Tensor> t; };
