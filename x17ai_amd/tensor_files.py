"""Naming and value conventions of the reference's tensor files (block_utils.py:47-199, src/tensor.rs:155-249).

A tensor file is `<name>_<tag>.safetensors` or `<name>_<tag>.bin` with tag in f32 / i32 / bf16 / i8 / f8:
  * `.safetensors` holds exactly one tensor (any entry name) whose dtype matches the tag;
  * `.bin` holds the raw bytes only, the caller supplies rows x cols (block_utils.py:94-107);
  * i8 files hold FixedI8 codes: real value = code / 8, and the code -128 stands for NaN (block_utils.py:118-124);
  * f8 files hold e4m3 codes of values flushed to zero below 1.9375 * 2^-7 (block_utils.py:126-137).
The kernels take the codes as they are; `real_values` is for reports and comparisons on the host.
"""
from __future__ import annotations

import os
from typing import Optional, Sequence

import numpy as np

from .api import BF16, E4M3, F32, INT8, Device, Tensor
from ._ffi import X17Error

_TAGS = {"f32": F32, "bf16": BF16, "i8": INT8, "f8": E4M3}      # "i32" is a report-only format: no tensor dtype
_EXTENSIONS = (".bin", ".safetensors")


def storage_dtype_tag(file_name: str) -> str:
	"""block_utils.py:55-70: the dtype tag between the last '_' and the extension."""
	base = os.path.basename(file_name)
	stem, ext = os.path.splitext(base)
	if ext not in _EXTENSIONS:
		raise X17Error(f"unsupported tensor file extension {ext!r} in {file_name!r}; expected one of: .bin, .safetensors")
	name, sep, tag = stem.rpartition("_")
	if not sep or not name or tag not in ("f32", "i32", "bf16", "i8", "f8"):
		raise X17Error(f"tensor file name must end with a dtype tag before the extension: {file_name!r}")
	return tag


def load_tensor_file(path: str, device: Optional[Device], shape: Optional[Sequence[int]] = None) -> Tensor:
	"""Loads `<name>_<tag>.safetensors` (shape from the file) or `<name>_<tag>.bin` (shape required) as codes."""
	tag = storage_dtype_tag(path)
	if tag not in _TAGS:
		raise X17Error(f"{path!r}: dtype tag {tag!r} has no tensor dtype on the device")
	dtype = _TAGS[tag]
	if path.endswith(".safetensors"):
		t = Tensor.from_safetensors_file(path, device)
		if t.dtype != dtype:
			raise X17Error(f"{path!r} declares {tag} in its name but stores dtype {t.dtype}")
		if shape is not None and tuple(shape) != t.shape:
			raise X17Error(f"{path!r} holds shape {t.shape}, expected {tuple(shape)}")
		return t
	if shape is None:
		raise X17Error(f"{path!r}: a raw .bin file carries no shape; pass shape=(rows, cols)")
	np_dtype = {F32: np.float32, BF16: np.uint16, INT8: np.int8, E4M3: np.uint8}[dtype]
	want = int(np.prod(shape)) * np.dtype(np_dtype).itemsize
	if os.path.getsize(path) != want:
		raise X17Error(f"{path!r} has {os.path.getsize(path)} bytes, shape {tuple(shape)} of {tag} needs {want}")
	return Tensor.from_numpy(device, np.fromfile(path, dtype=np_dtype).reshape(shape), dtype)


def real_values(codes: np.ndarray, dtype: int) -> np.ndarray:
	"""float32 values of stored codes (block_utils.py:118-124 for i8; the e4m3 dialect of the kernels has no
	subnormals and no NaN: value = 2^(e-7) * (1 + m/8), code 0 and 0x80 are zero)."""
	if dtype == F32:
		return np.asarray(codes, dtype=np.float32)
	if dtype == BF16:
		return (np.asarray(codes, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
	if dtype == INT8:
		c = np.asarray(codes, dtype=np.int8)
		out = c.astype(np.float32) / np.float32(8.0)
		out[c == -128] = np.nan
		return out
	if dtype == E4M3:
		c = np.asarray(codes, dtype=np.uint8).astype(np.uint32)
		bits = (((c & 0x80) << 24) | ((c & 0x7F) << 20)) + np.uint32(120 << 23)
		out = bits.astype(np.uint32).view(np.float32).copy()
		out[(c & 0x7F) == 0] = 0.0
		return out
	raise X17Error(f"unknown dtype {dtype}")
