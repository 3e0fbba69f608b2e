// build.rs for a tree that carries the HIP device (twin of the reference's build.rs:1-27).
// UNCOMPILED HERE: no Rust toolchain in the image this was written in.
//
// cpp/hip_shim.cpp is x17ai_amd/csrc/hip_shim.cpp, include/x17ai_hip_shim.h its header.  The shim is host-only C++
// over the HIP runtime API: hipcc is used as the C++ driver so that the ROCm include and library paths resolve;
// nothing is compiled for the GPU at this point (kernels are built per configuration at run time, see
// src/device/hip/kernel_build.rs).  libtorch and nvrtc, which the CUDA build links without using, are gone.

use std::env;
use std::path::PathBuf;

fn main() {
	let rocm = PathBuf::from(env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_owned()));

	cc::Build::new()
		.cpp(true)
		.compiler(rocm.join("bin/hipcc"))
		.flag("-std=c++20")
		.flag("-x")
		.flag("c++")
		.define("__HIP_PLATFORM_AMD__", None)
		.include(rocm.join("include"))
		.include("include")
		.file("cpp/hip_shim.cpp")
		.compile("x17ai_hip_shim");

	let lib = rocm.join("lib");
	println!("cargo:rustc-link-search=native={}", lib.display());
	println!("cargo:rustc-link-arg=-Wl,-rpath,{}", lib.display());
	println!("cargo:rustc-link-lib=dylib=amdhip64");

	for path in ["build.rs", "cpp/hip_shim.cpp", "include/x17ai_hip_shim.h"] {
		println!("cargo:rerun-if-changed={path}");
	}
	println!("cargo:rerun-if-env-changed=ROCM_PATH");
}
