"""Python mirror of the reference's operator API for the quantized block-forward path.

Names and argument meaning follow the Rust side: GemmKernel / GemmConfig / ScaleConfig /
RMSNormConfig / ResidualConfig / GeGluConfig (src/device/cuda/gemm.rs:28-449), AttnKernel /
AttnKernelConfig (src/device/cuda/attn.rs:45-240), Tensor (src/tensor.rs), CudaDevice and
CudaTimer (src/device/cuda.rs) -- here Device and Timer.  Each object owns a handle of the
C++ operator layer; numpy arrays only cross at Tensor.upload / Tensor.download.
"""
from __future__ import annotations

import ctypes
import dataclasses
import os
from typing import Optional, Sequence, Union

import numpy as np

from . import _ffi
from ._ffi import X17Error, check

# DType, src/dtype.rs:1-15
E4M3, INT8, BF16, F32 = 0, 1, 2, 3
_DTYPE_BYTES = {E4M3: 1, INT8: 1, BF16: 2, F32: 4}
_DTYPE_NAME = {E4M3: "e4m3", INT8: "i8", BF16: "bf16", F32: "f32"}


class Device:
	"""CudaDevice::new(device_id), src/device/cuda.rs:31-38 -- one HIP device with one stream."""

	def __init__(self, device_id: int = 0):
		self._h = ctypes.c_void_p()
		check(_ffi.host().x17h_device_new(device_id, ctypes.byref(self._h)))

	def synchronize(self) -> None:
		check(_ffi.host().x17h_device_synchronize(self._h))

	@property
	def name(self) -> str:
		return _ffi.host().x17h_device_name(self._h).decode()

	def close(self) -> None:
		if self._h:
			_ffi.host().x17h_device_free(self._h)
			self._h = ctypes.c_void_p()

	def __del__(self):
		try:
			self.close()
		except Exception:
			pass


class Tensor:
	"""Contiguous tensor = (dtype, shape, device buffer), src/tensor.rs:23-112."""

	def __init__(self, device: Optional[Device], shape: Sequence[int], dtype: int):
		self.device = device
		self.shape = tuple(int(s) for s in shape)
		self.dtype = dtype
		self._h = ctypes.c_void_p()
		arr = (ctypes.c_size_t * len(self.shape))(*self.shape)
		check(_ffi.host().x17h_tensor_new_empty(device._h if device is not None else None, arr, len(self.shape), dtype,
		                                        ctypes.byref(self._h)))

	@classmethod
	def new_empty(cls, shape: Sequence[int], dtype: int, device: Optional[Device]) -> "Tensor":
		return cls(device, shape, dtype)

	@classmethod
	def from_numpy(cls, device: Optional[Device], array: np.ndarray, dtype: int) -> "Tensor":
		t = cls(device, array.shape, dtype)
		t.upload(array)
		return t

	@classmethod
	def from_safetensors_file(cls, path: str, device: Optional[Device]) -> "Tensor":
		"""Tensor::from_safetensors_file, src/tensor.rs:155-179 (what the reference's block_utils.store_tensor
		writes for `*_i8 / _f8 / _bf16 / _f32.safetensors`): exactly one tensor, bytes uploaded unchanged."""
		t = cls.__new__(cls)
		t.device = device
		t._h = ctypes.c_void_p()
		dtype, ndim = ctypes.c_int(), ctypes.c_size_t()
		shape = (ctypes.c_size_t * 8)()
		check(_ffi.host().x17h_tensor_from_safetensors_file(device._h if device is not None else None, os.fsencode(path),
		                                                    ctypes.byref(t._h), ctypes.byref(dtype), shape, ctypes.byref(ndim)))
		t.dtype = dtype.value
		t.shape = tuple(int(shape[i]) for i in range(ndim.value))
		return t

	def save_safetensors_file(self, path: str) -> None:
		"""Tensor::save_safetensors_file, src/tensor.rs:213-249: CPU tensors only (download first)."""
		check(_ffi.host().x17h_tensor_save_safetensors_file(self._h, os.fsencode(path)))

	def to_cpu(self) -> "Tensor":
		"""Tensor::to_cpu + synchronize, src/tensor.rs:98-112."""
		return Tensor.from_numpy(None, self.download(), self.dtype)

	@property
	def nbytes(self) -> int:
		return int(_ffi.host().x17h_tensor_bytes(self._h))

	def upload(self, array: np.ndarray) -> None:
		array = np.ascontiguousarray(array)
		if array.nbytes != self.nbytes:
			raise X17Error(f"upload of {array.nbytes} bytes into a tensor of {self.nbytes} bytes")
		# the copy is asynchronous on the device stream; the source must outlive it
		self._staging = array
		check(_ffi.host().x17h_tensor_upload(self._h, array.ctypes.data_as(ctypes.c_void_p), array.nbytes))

	def download(self, np_dtype=None) -> np.ndarray:
		"""Tensor::to_cpu + synchronize (src/tensor.rs:98-112, src/main.rs:265)."""
		if np_dtype is None:
			np_dtype = {E4M3: np.uint8, INT8: np.int8, BF16: np.uint16, F32: np.float32}[self.dtype]
		out = np.empty(self.shape, dtype=np_dtype)
		if out.nbytes != self.nbytes:
			raise X17Error(f"download of {self.nbytes} bytes into an array of {out.nbytes} bytes")
		check(_ffi.host().x17h_tensor_download(self._h, out.ctypes.data_as(ctypes.c_void_p), out.nbytes))
		if self.device is not None:
			self.device.synchronize()
		return out

	def reshape(self, shape: Sequence[int]) -> "Tensor":
		shape = tuple(int(s) for s in shape)
		arr = (ctypes.c_size_t * len(shape))(*shape)
		check(_ffi.host().x17h_tensor_reshape(self._h, arr, len(shape)))
		self.shape = shape
		return self

	def device_ptr(self) -> int:
		return int(_ffi.host().x17h_tensor_device_ptr(self._h) or 0)

	def close(self) -> None:
		if self._h:
			_ffi.host().x17h_tensor_free(self._h)
			self._h = ctypes.c_void_p()

	def __del__(self):
		try:
			self.close()
		except Exception:
			pass


class Timer:
	"""CudaTimer, src/device/cuda.rs:79-101: a pair of events on the device's stream."""

	def __init__(self, device: Device):
		self.device = device
		self._h = ctypes.c_void_p()
		check(_ffi.host().x17h_timer_new(device._h, ctypes.byref(self._h)))

	def start(self) -> None:
		check(_ffi.host().x17h_timer_start(self._h))

	def stop(self) -> None:
		check(_ffi.host().x17h_timer_stop(self._h))

	def elapsed_seconds(self) -> float:
		s = ctypes.c_double()
		check(_ffi.host().x17h_timer_elapsed_seconds(self._h, ctypes.byref(s)))
		return float(s.value)

	def __del__(self):
		try:
			if self._h:
				_ffi.host().x17h_timer_free(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass


# ---------------------------------------------------------------- GEMM

@dataclasses.dataclass
class GemmInputConfig:          # gemm.rs:59-64
	dtype: int
	cols: int
	rows: Optional[int]
	trans: bool


@dataclasses.dataclass
class GemmConfig:               # gemm.rs:66-70
	a: GemmInputConfig
	b: GemmInputConfig
	c_dtype: int


@dataclasses.dataclass
class ScaleConfig:              # gemm.rs:33-36
	inp_scale: float
	out_scale: float
	kind = 0


@dataclasses.dataclass
class GeGluConfig:              # gemm.rs:52-55
	inp_scale: float
	out_scale: float
	kind = 1


@dataclasses.dataclass
class ResidualConfig:           # gemm.rs:47-50
	inp_scale: float
	out_scale: float
	kind = 2


@dataclasses.dataclass
class RMSNormConfig:            # gemm.rs:38-45
	eps: float
	head_dim: int
	sep_dim: int
	inp_scale: float
	out_scale: float
	kind = 3


@dataclasses.dataclass
class DequantConfig:
	"""No counterpart in gemm.rs: run-time per-row (token) and per-column (output channel) f32 scales,
	bf16 output, optionally GeGLU over column pairs -- symmetric per-row / per-channel int8 quantisation."""
	geglu: bool = False
	inp_scale: float = 1.0
	out_scale: float = 1.0
	kind = 4


@dataclasses.dataclass
class QNormConfig:
	"""The reference's older Q writer (cuda/qkvg_fwd_i8.cuh:145-219; hook cuda/gemm_b8.cuh:761-824): every head_dim
	raw columns are one L2-normalised head, times a learned bf16 scale per column passed at launch.  `inp_scale` is
	the factor applied after the learned scales: the old writer hands its values to a base class built with
	1 / sqrt(MODEL_DIM) (cuda/qkvg_fwd_i8.cuh:151-159) that no longer exists in the reference tree; 1.0 stores them as
	they are, 1 / sqrt(K) is the other reading (the live scaled writer's f32 overload applies its scale,
	cuda/gemm_b8.cuh:307-324)."""
	eps: float
	head_dim: int
	out_scale: float
	inp_scale: float = 1.0
	kind = 5


@dataclasses.dataclass
class QkvConfig:
	"""No counterpart in gemm.rs: the q projection (Scale writer) and the kv projection (RMSNorm writer) of
	src/main.rs:387-493 as one launch over the same token rows.  Raw columns [0, q_cols) are q."""
	q_cols: int
	q: ScaleConfig
	kv: RMSNormConfig
	kind = 6

	# the fields the flat configuration reads for the kv part
	@property
	def inp_scale(self): return self.kv.inp_scale
	@property
	def out_scale(self): return self.kv.out_scale
	@property
	def eps(self): return self.kv.eps
	@property
	def head_dim(self): return self.kv.head_dim
	@property
	def sep_dim(self): return self.kv.sep_dim


EpilogueConfig = Union[ScaleConfig, GeGluConfig, ResidualConfig, RMSNormConfig, DequantConfig, QNormConfig, QkvConfig]


def _attrs_dict(raw) -> dict:
	names = ["max_threads_per_block", "static_shared_size_bytes", "const_size_bytes", "local_size_bytes", "num_regs",
	         "ptx_version", "binary_version", "max_dynamic_shared_size_bytes", "preferred_shared_memory_carveout"]
	return {n: int(raw[i]) for i, n in enumerate(names)}


class GemmKernel:
	"""GemmKernel::<Epilogue>::new / launch / n_ops, src/device/cuda/gemm.rs:350-449.

	`device=None` generates and compiles the code object without loading it (what a build
	step on a machine without a GPU does).  `strict_math` picks the deterministic
	transcendental build (bit-exact against the CPU checker) over the hardware one."""

	def __init__(self, device: Optional[Device], kernel_name: str, gemm_config: GemmConfig,
	             epilogue_config: EpilogueConfig, strict_math: bool = True):
		c = _ffi.GemmConfigC()
		c.a_dtype, c.a_cols, c.a_rows, c.a_trans = gemm_config.a.dtype, gemm_config.a.cols, gemm_config.a.rows or 0, int(gemm_config.a.trans)
		c.b_dtype, c.b_cols, c.b_rows, c.b_trans = gemm_config.b.dtype, gemm_config.b.cols, gemm_config.b.rows or 0, int(gemm_config.b.trans)
		c.c_dtype = gemm_config.c_dtype
		c.epilogue = epilogue_config.kind
		c.inp_scale = epilogue_config.inp_scale
		c.out_scale = epilogue_config.out_scale
		c.eps = getattr(epilogue_config, "eps", 0.0)
		c.head_dim = getattr(epilogue_config, "head_dim", 0)
		c.sep_dim = getattr(epilogue_config, "sep_dim", 0)
		c.strict_math = int(strict_math)
		c.activation = int(bool(getattr(epilogue_config, "geglu", False)))
		if isinstance(epilogue_config, QkvConfig):
			c.q_cols, c.q_inp_scale, c.q_out_scale = epilogue_config.q_cols, epilogue_config.q.inp_scale, epilogue_config.q.out_scale
		self.device = device
		self.name = kernel_name
		self.epilogue_kind = epilogue_config.kind
		self._h = ctypes.c_void_p()
		check(_ffi.host().x17h_gemm_kernel_new(device._h if device is not None else None, kernel_name.encode(),
		                                       ctypes.byref(c), ctypes.byref(self._h)))
		self.diagnostics = _ffi.last_diagnostics()

	def launch(self, a: Tensor, b: Tensor, c: Tensor, extra: Optional[Tensor] = None) -> None:
		check(_ffi.host().x17h_gemm_kernel_launch(self._h, a._h, b._h, c._h, extra._h if extra is not None else None))

	def launch_dequant(self, a: Tensor, b: Tensor, c: Tensor, row_scale: Tensor, col_scale: Tensor) -> None:
		check(_ffi.host().x17h_gemm_kernel_launch_dequant(self._h, a._h, b._h, c._h, row_scale._h, col_scale._h))

	def launch_qkv(self, x: Tensor, q_weights: Tensor, kv_weights: Tensor, q: Tensor, kv: Tensor, rrms: Tensor) -> None:
		"""QkvConfig kernels: q = Scale(x . Wq^T), kv, rrms = RMSNorm(x . Wkv^T) in one launch."""
		check(_ffi.host().x17h_gemm_kernel_launch_qkv(self._h, x._h, q_weights._h, kv_weights._h, q._h, kv._h, rrms._h))

	def n_ops(self, a: Tensor, b: Tensor) -> float:
		return float(_ffi.host().x17h_gemm_kernel_n_ops(self._h, a._h, b._h))

	@property
	def metadata(self) -> dict:
		out = (ctypes.c_size_t * 4)()
		check(_ffi.host().x17h_gemm_kernel_metadata(self._h, out))
		return dict(zip(["THREADS_PER_BLOCK", "SMEM_BYTES", "M_PER_BLOCK", "N_PER_BLOCK"], [int(v) for v in out]))

	@property
	def attrs(self) -> dict:
		out = (ctypes.c_int32 * 9)()
		check(_ffi.host().x17h_gemm_kernel_attrs(self._h, out))
		return _attrs_dict(out)

	def __del__(self):
		try:
			if self._h:
				_ffi.host().x17h_gemm_kernel_free(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass


# ---------------------------------------------------------------- attention

@dataclasses.dataclass
class AttnKernelConfig:         # attn.rs:45-84
	dtype: int
	n_heads: int
	head_dim: int
	q_stride: int
	kv_stride: int
	o_stride: int
	# extension: q/k/v codes with one f32 scale per (row, head); out_dtype INT8 (FixedI8) or, with row scales, BF16
	row_scales: bool = False
	out_dtype: int = INT8
	# builds the backward-with-respect-to-q kernel (attn_d_q_i8.hip) instead of the forward: AttnKernel.launch_d_q
	backward_q: bool = False
	# builds the backward-with-respect-to-k-and-v kernel (attn_d_kv_i8.hip) instead: AttnKernel.launch_d_kv
	backward_kv: bool = False

	def heads_per_kernel(self) -> int:
		return 1 if self.head_dim == 0 else max(128 // self.head_dim, 1)

	def head_group_cnt(self) -> int:
		return self.n_heads // self.heads_per_kernel()


class AttnKernel:
	"""AttnKernel::new / launch, src/device/cuda/attn.rs:156-240."""

	def __init__(self, device: Optional[Device], kernel_name: str, config: AttnKernelConfig, strict_math: bool = True):
		c = _ffi.AttnConfigC(config.dtype, config.n_heads, config.head_dim, config.q_stride, config.kv_stride,
		                     config.o_stride, int(strict_math), int(config.row_scales), config.out_dtype, int(config.backward_q), int(config.backward_kv))
		self.device = device
		self.name = kernel_name
		self.config = config
		self._h = ctypes.c_void_p()
		check(_ffi.host().x17h_attn_kernel_new(device._h if device is not None else None, kernel_name.encode(),
		                                       ctypes.byref(c), ctypes.byref(self._h)))
		self.diagnostics = _ffi.last_diagnostics()

	def launch(self, q: Tensor, kv: Tensor, sink_k: Tensor, sink_v: Tensor, attn_temperature: Tensor, out: Tensor,
	           l: Optional[Tensor], window_size: int, batch: int = 1) -> None:
		check(_ffi.host().x17h_attn_kernel_launch(self._h, q._h, kv._h, sink_k._h, sink_v._h, attn_temperature._h, out._h,
		                                          l._h if l is not None else None, window_size, batch))

	def launch_row_scaled(self, q: Tensor, kv: Tensor, sink_k: Tensor, sink_v: Tensor, attn_temperature: Tensor,
	                      out: Tensor, l: Optional[Tensor], window_size: int, q_scale: Tensor, k_scale: Tensor,
	                      v_weight: Tensor, sink_v_weight: Tensor, out_scale: Tensor, batch: int = 1) -> None:
		"""Launch of a kernel built with config.row_scales: q_scale, k_scale, v_weight are f32 [n_heads, rows]
		(see recipes.attn_row_scale_operands)."""
		check(_ffi.host().x17h_attn_kernel_launch_row_scaled(
			self._h, q._h, kv._h, sink_k._h, sink_v._h, attn_temperature._h, out._h, l._h if l is not None else None,
			window_size, batch, q_scale._h, k_scale._h, v_weight._h, sink_v_weight._h, out_scale._h))

	def launch_d_q(self, q: Tensor, kv: Tensor, sink_k: Tensor, sink_v: Tensor, attn_temperature: Tensor, out: Tensor,
	               d_out: Tensor, d_q: Tensor, l: Tensor, d: Optional[Tensor], window_size: int, batch: int = 1) -> None:
		"""Launch of a kernel built with config.backward_q: the forward's operands, its output `out` (i8) and
		log-sum-exp `l`, dO `d_out` (bf16) -> dQ `d_q` (bf16, with respect to the real q) and D `d` (f32 [H, rows])."""
		check(_ffi.host().x17h_attn_kernel_launch_d_q(
			self._h, q._h, kv._h, sink_k._h, sink_v._h, attn_temperature._h, out._h, d_out._h, d_q._h, l._h,
			d._h if d is not None else None, window_size, batch))

	def launch_d_kv(self, q: Tensor, kv: Tensor, attn_temperature: Tensor, d_out: Tensor, l: Tensor, d: Tensor,
	                d_kv: Tensor, window_size: int, batch: int = 1) -> None:
		"""Launch of a kernel built with config.backward_kv: q, kv, the temperatures, dO `d_out` (bf16), the forward's
		log-sum-exp `l` and the dQ pass's `d` (f32 [H, rows]) -> `d_kv` (bf16 [rows, kv_stride], per head dK then dV,
		with respect to the real k and v)."""
		check(_ffi.host().x17h_attn_kernel_launch_d_kv(
			self._h, q._h, kv._h, attn_temperature._h, d_out._h, l._h, d._h, d_kv._h, window_size, batch))

	def n_ops(self, seq_len: int, window_size: int) -> float:
		return float(_ffi.host().x17h_attn_kernel_n_ops(self._h, seq_len, window_size))

	@property
	def metadata(self) -> dict:
		out = (ctypes.c_size_t * 3)()
		check(_ffi.host().x17h_attn_kernel_metadata(self._h, out))
		return dict(zip(["THREADS_PER_BLOCK", "SMEM_BYTES", "Q_PER_BLOCK"], [int(v) for v in out]))

	@property
	def attrs(self) -> dict:
		out = (ctypes.c_int32 * 9)()
		check(_ffi.host().x17h_attn_kernel_attrs(self._h, out))
		return _attrs_dict(out)

	def __del__(self):
		try:
			if self._h:
				_ffi.host().x17h_attn_kernel_free(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass


class RmsNormKernel:
	"""The reference's stand-alone rms_norm kernel (rms_norm.cu:55-113) as a kernel object."""

	def __init__(self, device: Optional[Device], kernel_name: str, in_dtype: int, model_dim: int, eps: float):
		self.device = device
		self.name = kernel_name
		self._h = ctypes.c_void_p()
		check(_ffi.host().x17h_rms_norm_kernel_new(device._h if device is not None else None, kernel_name.encode(),
		                                           in_dtype, model_dim, eps, ctypes.byref(self._h)))
		self.diagnostics = _ffi.last_diagnostics()

	def launch(self, inp: Tensor, out: Tensor) -> None:
		check(_ffi.host().x17h_rms_norm_kernel_launch(self._h, inp._h, out._h))

	def __del__(self):
		try:
			if self._h:
				_ffi.host().x17h_rms_norm_kernel_free(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass


class AttnDecodeKernel:
	"""Single-token decode against an int8 KV cache (no counterpart in the reference)."""

	def __init__(self, device: Optional[Device], kernel_name: str, n_heads: int, head_dim: int, cache_capacity: int,
	             strict_math: bool = True, row_scales: bool = False, out_dtype: int = INT8):
		self.device = device
		self.name = kernel_name
		self.row_scales = row_scales
		self.out_dtype = out_dtype
		self._h = ctypes.c_void_p()
		dev_h = device._h if device is not None else None
		if row_scales:
			check(_ffi.host().x17h_decode_kernel_new_row_scaled(dev_h, kernel_name.encode(), n_heads, head_dim, cache_capacity,
			                                                    int(strict_math), out_dtype, ctypes.byref(self._h)))
		else:
			if out_dtype != INT8:
				raise X17Error("the decode kernel writes bf16 only with row scales")
			check(_ffi.host().x17h_decode_kernel_new(dev_h, kernel_name.encode(), n_heads, head_dim, cache_capacity,
			                                         int(strict_math), ctypes.byref(self._h)))
		self.diagnostics = _ffi.last_diagnostics()

	def launch_row_scaled(self, q: Tensor, cache: Tensor, cache_len: Tensor, sink_k: Tensor, sink_v: Tensor,
	                      attn_temperature: Tensor, out: Tensor, l: Optional[Tensor], window_size: int, q_scale: Tensor,
	                      k_scale: Tensor, v_weight: Tensor, sink_v_weight: Tensor, out_scale: Tensor) -> None:
		"""q_scale [S, H]; k_scale, v_weight [S, H, capacity]; sink_v_weight, out_scale [H] (all f32)."""
		check(_ffi.host().x17h_decode_kernel_launch_row_scaled(
			self._h, q._h, cache._h, cache_len._h, sink_k._h, sink_v._h, attn_temperature._h, out._h,
			l._h if l is not None else None, window_size, q_scale._h, k_scale._h, v_weight._h, sink_v_weight._h, out_scale._h))

	def launch(self, q: Tensor, cache: Tensor, cache_len: Tensor, sink_k: Tensor, sink_v: Tensor,
	           attn_temperature: Tensor, out: Tensor, l: Optional[Tensor], window_size: int) -> None:
		check(_ffi.host().x17h_decode_kernel_launch(self._h, q._h, cache._h, cache_len._h, sink_k._h, sink_v._h,
		                                            attn_temperature._h, out._h, l._h if l is not None else None, window_size))

	def __del__(self):
		try:
			if self._h:
				_ffi.host().x17h_decode_kernel_free(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass
