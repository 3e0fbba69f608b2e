"""Measurement aids of the benchmark (include/x17ai_probe.h, libx17ai_probe.so): a copy kernel of known size, a loop
of nothing but matrix-core instructions and a loop of one vector instruction.  None of them is on the product path,
none has a counterpart in the reference; bench.py uses them to calibrate its figures against the machine at hand."""
from __future__ import annotations

import ctypes
import os
from typing import Optional

from . import _ffi
from ._ffi import X17Error
from .api import Device, Tensor

_lib = None


def lib() -> ctypes.CDLL:
	global _lib
	if _lib is not None:
		return _lib
	_ffi.host()                                   # the operator layer first: the probe library is built on it
	path = os.path.join(os.path.dirname(_ffi.lib_paths()["host"]), "libx17ai_probe.so")
	if not os.path.exists(path):
		raise X17Error(f"{path} is missing: run `make -C x17ai_amd/csrc` first")
	h = ctypes.CDLL(path)
	P, PP, SZ = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t
	h.x17p_last_error.restype = ctypes.c_char_p
	h.x17p_copy_probe_new.argtypes = [P, PP]
	h.x17p_copy_probe_free.argtypes = [P]
	h.x17p_copy_probe_free.restype = None
	h.x17p_copy_probe_launch.argtypes = [P, P, P]
	h.x17p_mfma_probe_new.argtypes = [P, ctypes.c_int, PP]
	h.x17p_mfma_probe_free.argtypes = [P]
	h.x17p_mfma_probe_free.restype = None
	h.x17p_mfma_probe_launch.argtypes = [P, P, P, SZ, ctypes.POINTER(ctypes.c_double)]
	h.x17p_valu_probe_ops.restype = ctypes.c_int
	h.x17p_valu_probe_op_name.argtypes = [ctypes.c_int]
	h.x17p_valu_probe_op_name.restype = ctypes.c_char_p
	h.x17p_valu_probe_new.argtypes = [P, ctypes.c_int, PP]
	h.x17p_valu_probe_free.argtypes = [P]
	h.x17p_valu_probe_free.restype = None
	h.x17p_valu_probe_launch.argtypes = [P, P, P, SZ, SZ, ctypes.POINTER(ctypes.c_double)]
	_lib = h
	return h


def _check(rc: int) -> None:
	if rc != 0:
		raise X17Error(lib().x17p_last_error().decode(errors="replace"))


class _Probe:
	_free = ""

	def __del__(self):
		try:
			if self._h:
				getattr(lib(), self._free)(self._h)
				self._h = ctypes.c_void_p()
		except Exception:
			pass


class CopyProbe(_Probe):
	"""A plain device-to-device copy kernel of known size (counter calibration)."""
	_free = "x17p_copy_probe_free"

	def __init__(self, device: Optional[Device]):
		self._h = ctypes.c_void_p()
		_check(lib().x17p_copy_probe_new(device._h if device is not None else None, ctypes.byref(self._h)))

	def launch(self, src: Tensor, dst: Tensor) -> None:
		_check(lib().x17p_copy_probe_launch(self._h, src._h, dst._h))


class MfmaProbe(_Probe):
	"""A loop of nothing but matrix-core instructions on register operands: what the matrix cores sustain on given
	operand data.  kind: 0 int8, 1 e4m3, 2 f16."""
	_free = "x17p_mfma_probe_free"

	def __init__(self, device: Optional[Device], kind: int):
		self._h = ctypes.c_void_p()
		_check(lib().x17p_mfma_probe_new(device._h if device is not None else None, kind, ctypes.byref(self._h)))

	def launch(self, operands: Tensor, out: Tensor, iterations: int) -> float:
		"""Returns the number of operations launched."""
		ops = ctypes.c_double()
		_check(lib().x17p_mfma_probe_launch(self._h, operands._h, out._h, iterations, ctypes.byref(ops)))
		return float(ops.value)


def valu_probe_ops() -> list:
	return [lib().x17p_valu_probe_op_name(i).decode() for i in range(lib().x17p_valu_probe_ops())]


class ValuProbe(_Probe):
	"""A loop of one vector (or scalar) instruction on sixteen independent registers, `waves_per_simd` wavefronts on
	every SIMD of the chip: the issue rate of that instruction."""
	_free = "x17p_valu_probe_free"

	def __init__(self, device: Optional[Device], op: int):
		self._h = ctypes.c_void_p()
		_check(lib().x17p_valu_probe_new(device._h if device is not None else None, op, ctypes.byref(self._h)))

	def launch(self, src: Tensor, out: Tensor, waves_per_simd: int, iterations: int) -> float:
		"""Returns the number of wavefront-instructions each SIMD executes."""
		n = ctypes.c_double()
		_check(lib().x17p_valu_probe_launch(self._h, src._h, out._h, waves_per_simd, iterations, ctypes.byref(n)))
		return float(n.value)
