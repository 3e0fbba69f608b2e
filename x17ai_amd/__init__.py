"""x17ai_amd -- MI355X-native quantized transformer-block forward path of x17ai.

Python face of the host-side operator layer (libx17ai_host.so), which mirrors the
reference's Rust operator layer (src/device/cuda/{gemm,attn}.rs, src/tensor.rs,
src/device/cuda.rs) and drives the C-ABI device shim (libx17ai_hip_shim.so).

There is no CPU fallback anywhere in this package: every compute call ends in a HIP
kernel launch and raises X17Error if the libraries, the code objects or a GPU are missing.
"""
from ._ffi import X17Error, lib_paths
from .api import (
	BF16, E4M3, F32, INT8,
	AttnDecodeKernel, AttnKernel, AttnKernelConfig, DequantConfig, Device, GeGluConfig, GemmConfig, GemmInputConfig,
	GemmKernel, QkvConfig, QNormConfig, ResidualConfig, RMSNormConfig, RmsNormKernel, ScaleConfig, Tensor, Timer,
)

__all__ = [
	"X17Error", "lib_paths", "BF16", "E4M3", "F32", "INT8", "AttnDecodeKernel", "AttnKernel", "AttnKernelConfig",
	"DequantConfig", "Device", "GeGluConfig", "GemmConfig", "GemmInputConfig", "GemmKernel", "QkvConfig", "QNormConfig",
	"ResidualConfig", "RMSNormConfig",
	"RmsNormKernel", "ScaleConfig", "Tensor", "Timer",
]
