"""ctypes declarations for include/x17ai_host.h (the flat C ABI of the operator layer)."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_DIR = os.path.join(_HERE, "lib")


class X17Error(RuntimeError):
	"""An error value returned by the operator layer (the reference's ErrPack<TensorOpError>)."""


def lib_paths() -> dict:
	return {
		"shim": os.path.join(_LIB_DIR, "libx17ai_hip_shim.so"),
		"host": os.path.join(_LIB_DIR, "libx17ai_host.so"),
	}


def kernel_cache_dir() -> str:
	"""Where the operator layer keeps one directory per built kernel (common.h, kernel.hsaco, meta.json)."""
	return os.environ.get("X17AI_KERNEL_CACHE") or os.path.join(_HERE, "cache", "kernels")


class GemmConfigC(ctypes.Structure):
	_fields_ = [
		("a_dtype", ctypes.c_int), ("a_cols", ctypes.c_size_t), ("a_rows", ctypes.c_size_t), ("a_trans", ctypes.c_int),
		("b_dtype", ctypes.c_int), ("b_cols", ctypes.c_size_t), ("b_rows", ctypes.c_size_t), ("b_trans", ctypes.c_int),
		("c_dtype", ctypes.c_int),
		("epilogue", ctypes.c_int),
		("inp_scale", ctypes.c_double),
		("out_scale", ctypes.c_double),
		("eps", ctypes.c_double),
		("head_dim", ctypes.c_size_t),
		("sep_dim", ctypes.c_size_t),
		("strict_math", ctypes.c_int),
		("activation", ctypes.c_int),
		("q_cols", ctypes.c_size_t),
		("q_inp_scale", ctypes.c_double),
		("q_out_scale", ctypes.c_double),
	]


class AttnConfigC(ctypes.Structure):
	_fields_ = [
		("dtype", ctypes.c_int), ("n_heads", ctypes.c_size_t), ("head_dim", ctypes.c_size_t),
		("q_stride", ctypes.c_size_t), ("kv_stride", ctypes.c_size_t), ("o_stride", ctypes.c_size_t),
		("strict_math", ctypes.c_int), ("row_scales", ctypes.c_int), ("out_dtype", ctypes.c_int),
		("backward_q", ctypes.c_int), ("backward_kv", ctypes.c_int),
	]


_host = None


def host() -> ctypes.CDLL:
	"""Loads libx17ai_host.so (which pulls in the shim).  Fails loudly when it was not built."""
	global _host
	if _host is not None:
		return _host
	paths = lib_paths()
	for p in paths.values():
		if not os.path.exists(p):
			raise X17Error(f"{p} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
			               f"(or `make -C x17ai_amd/csrc`) first; there is no CPU fallback")
	# the shim first, globally, so that the host library's dependency resolves to this very file
	ctypes.CDLL(paths["shim"], mode=ctypes.RTLD_GLOBAL)
	h = ctypes.CDLL(paths["host"])
	P = ctypes.c_void_p
	PP = ctypes.POINTER(ctypes.c_void_p)
	SZ = ctypes.c_size_t
	h.x17h_last_error.restype = ctypes.c_char_p
	h.x17h_last_diagnostics.restype = ctypes.c_char_p
	h.x17h_device_new.argtypes = [SZ, PP]
	h.x17h_device_free.argtypes = [P]
	h.x17h_device_free.restype = None
	h.x17h_device_synchronize.argtypes = [P]
	h.x17h_device_name.argtypes = [P]
	h.x17h_device_name.restype = ctypes.c_char_p
	h.x17h_tensor_new_empty.argtypes = [P, ctypes.POINTER(SZ), SZ, ctypes.c_int, PP]
	h.x17h_tensor_free.argtypes = [P]
	h.x17h_tensor_free.restype = None
	h.x17h_tensor_upload.argtypes = [P, P, SZ]
	h.x17h_tensor_download.argtypes = [P, P, SZ]
	h.x17h_tensor_from_safetensors_file.argtypes = [P, ctypes.c_char_p, PP, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(SZ), ctypes.POINTER(SZ)]
	h.x17h_tensor_save_safetensors_file.argtypes = [P, ctypes.c_char_p]
	h.x17h_tensor_device_ptr.argtypes = [P]
	h.x17h_tensor_device_ptr.restype = P
	h.x17h_tensor_bytes.argtypes = [P]
	h.x17h_tensor_bytes.restype = SZ
	h.x17h_tensor_reshape.argtypes = [P, ctypes.POINTER(SZ), SZ]
	h.x17h_timer_new.argtypes = [P, PP]
	h.x17h_timer_free.argtypes = [P]
	h.x17h_timer_free.restype = None
	h.x17h_timer_start.argtypes = [P]
	h.x17h_timer_stop.argtypes = [P]
	h.x17h_timer_elapsed_seconds.argtypes = [P, ctypes.POINTER(ctypes.c_double)]
	h.x17h_gemm_kernel_new.argtypes = [P, ctypes.c_char_p, ctypes.POINTER(GemmConfigC), PP]
	h.x17h_gemm_kernel_free.argtypes = [P]
	h.x17h_gemm_kernel_free.restype = None
	h.x17h_gemm_kernel_launch.argtypes = [P, P, P, P, P]
	h.x17h_gemm_kernel_launch_dequant.argtypes = [P, P, P, P, P, P]
	h.x17h_gemm_kernel_launch_qkv.argtypes = [P, P, P, P, P, P, P]
	h.x17h_gemm_kernel_n_ops.argtypes = [P, P, P]
	h.x17h_gemm_kernel_n_ops.restype = ctypes.c_double
	h.x17h_gemm_kernel_metadata.argtypes = [P, ctypes.POINTER(SZ)]
	h.x17h_gemm_kernel_attrs.argtypes = [P, ctypes.POINTER(ctypes.c_int32)]
	h.x17h_attn_kernel_new.argtypes = [P, ctypes.c_char_p, ctypes.POINTER(AttnConfigC), PP]
	h.x17h_attn_kernel_free.argtypes = [P]
	h.x17h_attn_kernel_free.restype = None
	h.x17h_attn_kernel_launch.argtypes = [P, P, P, P, P, P, P, P, SZ, SZ]
	h.x17h_attn_kernel_launch_row_scaled.argtypes = [P, P, P, P, P, P, P, P, SZ, SZ, P, P, P, P, P]
	h.x17h_attn_kernel_launch_d_q.argtypes = [P, P, P, P, P, P, P, P, P, P, P, SZ, SZ]
	h.x17h_attn_kernel_launch_d_kv.argtypes = [P, P, P, P, P, P, P, P, SZ, SZ]
	h.x17h_attn_kernel_n_ops.argtypes = [P, SZ, SZ]
	h.x17h_attn_kernel_n_ops.restype = ctypes.c_double
	h.x17h_attn_kernel_metadata.argtypes = [P, ctypes.POINTER(SZ)]
	h.x17h_attn_kernel_attrs.argtypes = [P, ctypes.POINTER(ctypes.c_int32)]
	h.x17h_rms_norm_kernel_new.argtypes = [P, ctypes.c_char_p, ctypes.c_int, SZ, ctypes.c_double, PP]
	h.x17h_rms_norm_kernel_free.argtypes = [P]
	h.x17h_rms_norm_kernel_free.restype = None
	h.x17h_rms_norm_kernel_launch.argtypes = [P, P, P]
	h.x17h_decode_kernel_new.argtypes = [P, ctypes.c_char_p, SZ, SZ, SZ, ctypes.c_int, PP]
	h.x17h_decode_kernel_new_row_scaled.argtypes = [P, ctypes.c_char_p, SZ, SZ, SZ, ctypes.c_int, ctypes.c_int, PP]
	h.x17h_decode_kernel_launch_row_scaled.argtypes = [P, P, P, P, P, P, P, P, P, SZ, P, P, P, P, P]
	h.x17h_decode_kernel_free.argtypes = [P]
	h.x17h_decode_kernel_free.restype = None
	h.x17h_decode_kernel_launch.argtypes = [P, P, P, P, P, P, P, P, P, SZ]
	_host = h
	return h


def check(rc: int) -> None:
	if rc != 0:
		raise X17Error(host().x17h_last_error().decode("utf-8", "replace"))


def last_diagnostics() -> str:
	return host().x17h_last_diagnostics().decode("utf-8", "replace")
