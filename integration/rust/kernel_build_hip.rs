// src/device/hip/kernel_build.rs -- turns a rendered common.h into a loaded gfx950 kernel
// (twin of src/device/cuda/kernel_build.rs:20-260).
// UNCOMPILED HERE: no Rust toolchain in the image this was written in.
//
// The CUDA side renders three askama templates per kernel (common.cuh, kernel.cu, meta.cu), compiles kernel.cu to
// PTX and then to a cubin, compiles and runs meta.cu for meta.json, and always recompiles (gemm.rs:408-416).  Here
// the kernel sources are fixed files (x17ai_amd/csrc/kernels/*.hip, one `extern "C" kernel` each); only common.h is
// generated -- a list of #defines -- and one hipcc call produces the code object.  The metadata program is plain
// host C++ (the tile headers are constexpr-only), so the host compiler builds it.  A content hash of everything the
// code object depends on is kept beside it (build.key): an unchanged kernel is not compiled again.
// The operator layer in C++ (x17ai_amd/csrc/host/x17ai_host.cpp, namespace kernel_build) does the same steps; its
// tests (tests/test_gpu_cache.py, tests/test_host_cpu.py) are the executable description of this file.

use std::fs;
use std::hash::Hasher;
use std::path::{Path, PathBuf};
use std::process::{Command, Output};

use serde::de::DeserializeOwned;

use crate::{Diagnostics, KernelGeneratorError};

use super::hip_shim::{HipKernel, HipStream};

type Gen<T> = Result<T, KernelGeneratorError>;

/// Flags every device compilation gets.  -ffp-contract=off: the kernels spell out their fused multiply-adds, as the
/// reference's arithmetic is specified operation by operation.  Packed-f32 instructions are kept off.  nvcc's
/// --ftz / --use_fast_math have no counterpart here: the speed builds call the hardware transcendentals explicitly
/// (X17_STRICT_MATH = 0), the strict builds their deterministic definitions.
const DEVICE_FLAGS: &[&str] = &[
	"--offload-arch=gfx950", "-O3", "-std=c++20", "-ffp-contract=off",
	"-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
	"-Wno-unused-command-line-argument", "-Wno-inline-asm",
];

pub(super) struct BuiltKernel {
	pub dir: PathBuf,
	pub code_object: PathBuf,
	pub meta_json: PathBuf,
	pub cache_hit: bool,
}

fn fail<T>(diag: &mut Diagnostics, message: String) -> Gen<T> {
	diag.add_error(message);
	Err(KernelGeneratorError)
}

fn hipcc() -> PathBuf {
	std::env::var_os("X17AI_HIPCC").map_or_else(|| PathBuf::from("/opt/rocm/bin/hipcc"), PathBuf::from)
}

/// Directory of the fixed kernel sources (gemm_b8.hip, attn_fwd_i8.hip, x17_device.h, the *_tile.h headers, ...).
fn kernels_dir() -> PathBuf {
	std::env::var_os("X17AI_KERNELS_DIR").map_or_else(|| PathBuf::from("x17ai_amd/csrc/kernels"), PathBuf::from)
}

fn read(path: &Path, diag: &mut Diagnostics) -> Gen<Vec<u8>> {
	match fs::read(path) {
		Ok(bytes) => Ok(bytes),
		Err(err) => fail(diag, format!("Error reading file {}: {err}", path.display())),
	}
}

/// FNV-1a over the rendered header, the flags, the shared headers and the two sources, in that order
/// (the same key as the C++ operator layer writes, so both sides share one cache).
fn build_key(common_h: &str, source: &Path, meta_source: &Path, diag: &mut Diagnostics) -> Gen<String> {
	struct Fnv(u64);
	impl Hasher for Fnv {
		fn write(&mut self, bytes: &[u8]) {
			for &b in bytes {
				self.0 = (self.0 ^ u64::from(b)).wrapping_mul(0x0000_0100_0000_01B3);
			}
		}
		fn finish(&self) -> u64 {
			self.0
		}
	}
	let mut h = Fnv(0xCBF2_9CE4_8422_2325);
	h.write(common_h.as_bytes());
	// (joined by single spaces this is, byte for byte, the flag string the C++ operator layer hashes: both sides can
	// share one cache directory)
	h.write(DEVICE_FLAGS.join(" ").as_bytes());
	let dir = kernels_dir();
	for shared in ["x17_device.h", "gemm_tile.h", "attn_tile.h", "rms_norm_tile.h", "decode_tile.h"] {
		if let Ok(bytes) = fs::read(dir.join(shared)) {
			h.write(&bytes);
		}
	}
	h.write(&read(source, diag)?);
	h.write(&read(meta_source, diag)?);
	Ok(format!("{:016x}", h.finish()))
}

/// `common_h`: the #define list for this kernel; `source` / `meta_source`: file names inside kernels_dir().
pub(super) fn build(
	cache_dir: &Path,
	kernel_name: &str,
	common_h: &str,
	source: &str,
	meta_source: &str,
	diag: &mut Diagnostics,
) -> Gen<BuiltKernel> {
	// the name becomes a directory name (gemm.rs:377-387)
	if kernel_name.is_empty() || kernel_name == "." || kernel_name == ".." || kernel_name.contains(['/', '\\']) {
		return fail(diag, format!("invalid kernel name {kernel_name:?}"));
	}
	let dir = cache_dir.join(kernel_name);
	if let Err(err) = fs::create_dir_all(&dir) {
		return fail(diag, format!("failed to create kernel cache directory {}: {err}", dir.display()));
	}
	let source = kernels_dir().join(source);
	let meta_source = kernels_dir().join(meta_source);
	let built = BuiltKernel {
		code_object: dir.join("kernel.hsaco"),
		meta_json: dir.join("meta.json"),
		cache_hit: false,
		dir,
	};
	let key_path = built.dir.join("build.key");
	let key = build_key(common_h, &source, &meta_source, diag)?;
	let forced = std::env::var_os("X17AI_FORCE_REBUILD").is_some();
	if !forced
		&& fs::read_to_string(&key_path).is_ok_and(|have| have == key)
		&& built.code_object.exists()
		&& built.meta_json.exists()
	{
		return Ok(BuiltKernel { cache_hit: true, ..built });
	}

	write_generated_file(&built.dir.join("common.h"), common_h, diag)?;

	// device code: one step instead of PTX + cubin (kernel_build.rs:38-86)
	let mut compile = Command::new(hipcc());
	compile.args(DEVICE_FLAGS).arg("--genco").arg("-I").arg(&built.dir).arg("-I").arg(kernels_dir()).arg(&source).arg("-o").arg(&built.code_object);
	run_checked_command(&mut compile, &format!("hipcc failed while compiling {}", source.display()), diag)?;

	// metadata: host program printing the tile constants as JSON (kernel_build.rs:88-131)
	let meta_exe = built.dir.join("meta");
	let mut host = Command::new("g++");
	host.arg("-std=c++17").arg("-I").arg(&built.dir).arg("-I").arg(kernels_dir()).arg(&meta_source).arg("-o").arg(&meta_exe);
	run_checked_command(&mut host, &format!("g++ failed while compiling {}", meta_source.display()), diag)?;
	let printed = run_checked_command(&mut Command::new(&meta_exe), &format!("failed to run metadata executable {}", meta_exe.display()), diag)?;
	if let Err(err) = fs::write(&built.meta_json, printed.stdout) {
		return fail(diag, format!("failed to write generated metadata {}: {err}", built.meta_json.display()));
	}
	// the key goes last: an interrupted build leaves no key and is redone
	if let Err(err) = fs::write(&key_path, key) {
		return fail(diag, format!("failed to write {}: {err}", key_path.display()));
	}
	Ok(built)
}

pub(super) fn write_generated_file(path: &Path, text: &str, diag: &mut Diagnostics) -> Gen<()> {
	match fs::write(path, text) {
		Ok(()) => Ok(()),
		Err(err) => fail(diag, format!("failed to write generated HIP source {}: {err}", path.display())),
	}
}

pub(super) fn read_metadata_json<T: DeserializeOwned>(path: &Path, diag: &mut Diagnostics) -> Gen<T> {
	let text = match fs::read_to_string(path) {
		Ok(text) => text,
		Err(err) => return fail(diag, format!("Error reading file {}: {err}", path.display())),
	};
	match serde_json::from_str(&text) {
		Ok(meta) => Ok(meta),
		Err(err) => fail(diag, format!("Failed to parse JSON data from {}: {err}", path.display())),
	}
}

/// Loads `kernel.hsaco` and resolves its entry point (always named "kernel", gemm.rs:573-575).
pub(super) fn load_kernel(
	stream: &HipStream,
	code_object: &Path,
	kernel_name: &str,
	smem_size: usize,
	diag: &mut Diagnostics,
) -> Gen<HipKernel> {
	let module = match stream.load_module_from_code_object(code_object) {
		Ok(module) => module,
		Err(err) => return fail(diag, format!("failed to load generated HIP module `{}`: {err}", code_object.display())),
	};
	let kernel = match module.get_kernel(kernel_name, smem_size) {
		Ok(kernel) => kernel,
		Err(err) => {
			return fail(diag, format!("failed to load generated HIP kernel `{kernel_name}` from `{}`: {err}", code_object.display()));
		},
	};
	if kernel.has_spills() {
		diag.add_warning(format!(
			"generated HIP kernel `{kernel_name}` from `{}` uses scratch memory: local_size_bytes={}, num_regs={}, max_threads_per_block={}",
			code_object.display(),
			kernel.attrs.local_size_bytes,
			kernel.attrs.num_regs,
			kernel.attrs.max_threads_per_block,
		));
	}
	Ok(kernel)
}

pub(super) fn run_checked_command(command: &mut Command, context: &str, diag: &mut Diagnostics) -> Gen<Output> {
	let shown = format!("{command:?}");
	let output = match command.output() {
		Ok(output) => output,
		Err(err) => return fail(diag, format!("{context}: failed to start {shown}: {err}")),
	};
	if output.status.success() {
		return Ok(output);
	}
	fail(
		diag,
		format!(
			"{context} (status: {})\ncommand: {shown}\nstdout:\n{}\nstderr:\n{}",
			output.status,
			String::from_utf8_lossy(&output.stdout),
			String::from_utf8_lossy(&output.stderr),
		),
	)
}
