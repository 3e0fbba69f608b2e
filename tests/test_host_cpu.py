"""Host-side checks that need no GPU: the two shared libraries load and export exactly what
include/*.h declares, errors travel as diagnostics (never exceptions or aborts), kernel
configurations are validated as the reference validates them, and the kernel cache works."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

import x17ai_amd as X
from x17ai_amd import _ffi, recipes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
	text = open(os.path.join(ROOT, "include", header)).read()
	text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
	return sorted(set(re.findall(r"\b(x17(?:ai|h|p)_[a-z0-9_]+)\s*\(", text)))


def _exported(lib):
	out = subprocess.run(["nm", "-D", "--defined-only", lib], check=True, capture_output=True, text=True).stdout
	return sorted(set(l.split()[-1] for l in out.splitlines() if " T " in l))


def test_shim_exports_exactly_the_declared_entry_points():
	declared = _declared("x17ai_hip_shim.h")
	assert len(declared) == 21              # the reference's FFI surface, src/device/cuda/cuda_shim.rs:76-158
	exported = [s for s in _exported(_ffi.lib_paths()["shim"]) if s.startswith("x17ai_")]
	assert exported == declared


def test_host_library_exports_every_declared_entry_point():
	declared = _declared("x17ai_host.h")
	exported = set(_exported(_ffi.lib_paths()["host"]))
	assert declared and not [s for s in declared if s not in exported]


def test_the_product_headers_and_libraries_hold_no_measurement_aids():
	assert sorted(os.listdir(os.path.join(ROOT, "include"))) == ["x17ai_hip_shim.h", "x17ai_host.h"]
	assert not [s for s in _declared("x17ai_host.h") if "probe" in s]
	assert not [s for s in _exported(_ffi.lib_paths()["host"]) if "probe" in s and s.startswith("x17h_")]


def test_the_headers_are_plain_c_and_a_c_program_links_against_both_libraries(tmp_path):
	"""The boundary is a C ABI: both headers compile as strict C99 and as C++17, and a C program that takes the address of
	every declared entry point links against the two libraries (no GPU is touched: nothing is called)."""
	inc = os.path.join(ROOT, "include")
	for header in ("x17ai_hip_shim.h", "x17ai_host.h"):
		subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c", os.path.join(inc, header)], check=True)
		subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c++", os.path.join(inc, header)], check=True)
	names = _declared("x17ai_hip_shim.h") + _declared("x17ai_host.h")
	prog = '#include "x17ai_hip_shim.h"\n#include "x17ai_host.h"\n#include <stdio.h>\nint main(void) {\n\tvoid (*table[])(void) = {\n'
	prog += "".join(f"\t\t(void (*)(void)){n},\n" for n in names)
	prog += '\t};\n\tprintf("%u\\n", (unsigned)(sizeof table / sizeof table[0]));\n\treturn 0;\n}\n'
	exe = str(tmp_path / "links")
	libdir = os.path.dirname(_ffi.lib_paths()["host"])
	subprocess.run(["gcc", "-std=c99", "-x", "c", "-", "-I", inc, "-L", libdir, "-lx17ai_host", "-lx17ai_hip_shim",
	                "-Wl,-rpath," + libdir, "-o", exe], input=prog, text=True, check=True)
	assert int(subprocess.run([exe], capture_output=True, text=True, check=True).stdout) == len(names) > 60


def test_struct_layouts_match_the_reference_ffi(tmp_path):
	# CudaKernelAttrs: nine int32 (cuda_shim.rs:51-63); PtrResult: two pointers (cuda_shim.rs:70-74)
	src = open(os.path.join(ROOT, "include", "x17ai_hip_shim.h")).read()
	body = src[src.index("typedef struct X17HipKernelAttrs {"):src.index("} X17HipKernelAttrs;")]
	assert len(re.findall(r"int32_t\s+\w+;", body)) == 9
	prog = r'''
	#include "x17ai_hip_shim.h"
	#include <stdio.h>
	int main(void) { printf("%zu %zu %zu %zu\n", sizeof(X17HipKernelAttrs), sizeof(X17StreamResult), sizeof(X17FfiBuffer), sizeof(X17FfiSpan)); return 0; }
	'''
	exe = str(tmp_path / "layout_probe")
	subprocess.run(["gcc", "-x", "c", "-", "-I", os.path.join(ROOT, "include"), "-o", exe], input=prog, text=True, check=True)
	assert subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split() == ["36", "16", "16", "16"]


def test_errors_are_diagnostics_not_crashes():
	"""Without a GPU (or with a bad ordinal) opening a device fails with the shim's message, moved
	through x17ai_move_diagnostic into the caller's buffer (cpp/ffi.hpp:84-175)."""
	with pytest.raises(X.X17Error, match=r"x17ai_hip_open_context\(\)"):
		X.Device(10 ** 6)
	# a NULL diagnostic is a no-op; handing one to move_diagnostic must not crash
	shim = ctypes.CDLL(_ffi.lib_paths()["shim"])

	class Buf(ctypes.Structure):
		_fields_ = [("instance", ctypes.c_void_p), ("vmt", ctypes.c_void_p)]
	shim.x17ai_move_diagnostic.argtypes = [ctypes.c_void_p, Buf]
	shim.x17ai_move_diagnostic.restype = None
	shim.x17ai_move_diagnostic(None, Buf(None, None))


def _gemm(a, b, c, k=256, n=256, trans_a=False, trans_b=True, rows=True):
	return X.GemmConfig(X.GemmInputConfig(a, k, None, trans_a), X.GemmInputConfig(b, k, n if rows else None, trans_b), c)


@pytest.mark.parametrize("cfg,epi,msg", [
	(_gemm(X.INT8, X.INT8, X.INT8, trans_a=True), X.ScaleConfig(1.0, 1.0), "transposed GEMM input A"),
	(_gemm(X.INT8, X.INT8, X.INT8, trans_b=False), X.ScaleConfig(1.0, 1.0), "non-transposed GEMM input B"),
	(_gemm(X.INT8, X.INT8, X.INT8, rows=False), X.ScaleConfig(1.0, 1.0), "runtime column count"),
	(_gemm(X.INT8, X.INT8, X.E4M3), X.ScaleConfig(1.0, 1.0), "Scale epilogue requires an i8 output"),
	(_gemm(X.BF16, X.INT8, X.INT8), X.ScaleConfig(1.0, 1.0), "unsupported GEMM input dtype bf16"),
	(_gemm(X.INT8, X.INT8, X.F32), X.GeGluConfig(1.0, 1.0), "GeGLU epilogue requires"),
	(_gemm(X.INT8, X.INT8, X.E4M3), X.GeGluConfig(-1.0, 1.0), "invalid GeGLU scale values"),
	(_gemm(X.INT8, X.INT8, X.E4M3), X.ResidualConfig(1.0, float("nan")), "invalid residual GEMM scale values"),
	(_gemm(X.INT8, X.INT8, X.INT8), X.RMSNormConfig(1e-9, 48, 48, 1.0, 1.0), "multiples of 32"),
	(_gemm(X.INT8, X.INT8, X.INT8), X.RMSNormConfig(1e-9, 32, 64, 1.0, 1.0), "head_dim == sep_dim"),
	(_gemm(X.INT8, X.INT8, X.INT8, k=200), X.ScaleConfig(1.0, 1.0), "multiple of 128"),
	(_gemm(X.INT8, X.INT8, X.INT8, n=192), X.ScaleConfig(1.0, 1.0), "raw output columns must be a multiple of 128"),
	(_gemm(X.INT8, X.INT8, X.INT8, n=128), X.ScaleConfig(1.0, 1.0), "at least one tile"),
	(_gemm(X.INT8, X.INT8, X.INT8), X.QNormConfig(0.0, 48, 8.0), "head_dim in"),
	(_gemm(X.INT8, X.INT8, X.E4M3), X.QNormConfig(0.0, 64, 8.0), "QNorm epilogue requires i8"),
	(_gemm(X.INT8, X.INT8, X.INT8, n=768), X.QkvConfig(128, X.ScaleConfig(1.0, 8.0), X.RMSNormConfig(1e-9, 64, 64, 1.0, 8.0)), "q_cols must be a multiple of 256"),
	(_gemm(X.INT8, X.INT8, X.INT8, n=768), X.QkvConfig(256, X.ScaleConfig(1.0, 8.0), X.RMSNormConfig(1e-9, 64, 32, 1.0, 8.0)), "head_dim == sep_dim"),
])
def test_gemm_kernel_config_validation(cfg, epi, msg):
	with pytest.raises(X.X17Error, match=msg):
		X.GemmKernel(None, "cpu-validation-probe", cfg, epi)


def test_kernel_names_are_path_safe():
	for bad in ("", ".", "..", "a/b", "a\\b"):
		with pytest.raises(X.X17Error, match="invalid kernel name"):
			X.GemmKernel(None, bad, _gemm(X.INT8, X.INT8, X.INT8), X.ScaleConfig(1.0, 1.0))


def test_attention_kernel_config_validation():
	bad = [
		(X.AttnKernelConfig(X.E4M3, 4, 64, 256, 512, 256), "requires dtype i8"),
		(X.AttnKernelConfig(X.INT8, 0, 64, 256, 512, 256), "n_heads > 0"),
		(X.AttnKernelConfig(X.INT8, 4, 48, 256, 512, 256), "multiple of 32"),
		(X.AttnKernelConfig(X.INT8, 3, 64, 192, 384, 192), "divisible by heads_per_kernel"),
		(X.AttnKernelConfig(X.INT8, 4, 64, 128, 512, 256), "q_stride >= n_heads"),
		(X.AttnKernelConfig(X.INT8, 4, 64, 256, 256, 256), "kv_stride >= 2"),
	]
	for cfg, msg in bad:
		with pytest.raises(X.X17Error, match=msg):
			X.AttnKernel(None, "cpu-validation-probe", cfg)
	with pytest.raises(X.X17Error, match="multiple of 512"):
		X.RmsNormKernel(None, "cpu-validation-probe", X.E4M3, 1000, 1e-9)
	with pytest.raises(X.X17Error, match="multiple of 16"):
		X.AttnDecodeKernel(None, "cpu-validation-probe", 4, 64, 100)


def test_kernel_build_metadata_and_cache(tmp_path, monkeypatch):
	"""The code object and meta.json are generated per configuration and reused when nothing changed
	(the reference recompiles on every run, src/device/cuda/gemm.rs:408-416)."""
	monkeypatch.setenv("X17AI_KERNEL_CACHE", str(tmp_path))
	k = recipes.attn_q_kernel(None, 256, 256)
	assert k.metadata == {"THREADS_PER_BLOCK": 512, "SMEM_BYTES": 131072, "M_PER_BLOCK": 256, "N_PER_BLOCK": 256}
	d = tmp_path / k.name
	assert (d / "kernel.hsaco").stat().st_size > 1000
	text = (d / "common.h").read_text()
	assert "#define X17_A_COLS 256" in text and "#define X17_EPILOGUE 0" in text
	# inv_sqrt(256) / 64 printed with 17 significant digits, as gemm.rs:257-259 does
	assert "#define X17_INP_SCALE 9.76562500000000000e-04" in text
	stamp = (d / "kernel.hsaco").stat().st_mtime_ns
	recipes.attn_q_kernel(None, 256, 256)
	assert (d / "kernel.hsaco").stat().st_mtime_ns == stamp
	with pytest.raises(X.X17Error, match="built without a device"):
		k.launch(X.Tensor(None, (256, 256), X.INT8), X.Tensor(None, (256, 256), X.INT8), X.Tensor(None, (256, 256), X.INT8))
	a = k  # n_ops is pure host arithmetic (gemm.rs:445-449)
	assert a.n_ops(X.Tensor(None, (512, 256), X.INT8), X.Tensor(None, (256, 256), X.INT8)) == 2.0 * 512 * 256 * 256


def test_build_key_follows_the_headers_a_kernel_includes(tmp_path, monkeypatch):
	"""The key of a code object covers its generated common.h, the flags, its two sources and, transitively, the headers
	of the kernels directory they include -- not the other kernels' headers: a comment added to the attention tile
	header leaves an rms_norm build alone, one added to rms_norm_tile.h or x17_device.h rebuilds it."""
	import shutil
	from x17ai_amd import _ffi
	src = os.path.join(os.path.dirname(os.path.abspath(_ffi.__file__)), "csrc", "kernels")
	kernels = tmp_path / "kernels"
	shutil.copytree(src, kernels)
	monkeypatch.setenv("X17AI_KERNELS_DIR", str(kernels))
	monkeypatch.setenv("X17AI_KERNEL_CACHE", str(tmp_path / "cache"))
	build = lambda: X.RmsNormKernel(None, "key-probe", X.BF16, 512, 1e-6)
	key_file = tmp_path / "cache" / "key-probe" / "build.key"
	build()
	first = key_file.read_text()
	stamp = (tmp_path / "cache" / "key-probe" / "kernel.hsaco").stat().st_mtime_ns
	with open(kernels / "attn_tile.h", "a") as f:
		f.write("// a change to another kernel's header\n")
	build()
	assert key_file.read_text() == first and (tmp_path / "cache" / "key-probe" / "kernel.hsaco").stat().st_mtime_ns == stamp
	for header in ("rms_norm_tile.h", "x17_device.h"):
		before = key_file.read_text()
		with open(kernels / header, "a") as f:
			f.write("// a change to a header this kernel includes\n")
		build()
		assert key_file.read_text() != before, header


def test_cpu_tensors_round_trip():
	import numpy as np
	t = X.Tensor.from_numpy(None, np.arange(24, dtype=np.int8).reshape(4, 6), X.INT8)
	assert t.download().tolist() == np.arange(24).reshape(4, 6).tolist()
	assert t.reshape((6, 4)).shape == (6, 4)
	with pytest.raises(X.X17Error):
		t.reshape((5, 5))


def test_safetensors_files_round_trip_against_the_safetensors_package(tmp_path):
	"""The on-disk format of the reference's tensors (src/tensor.rs:155-249, block_utils.py:163-199): one tensor per
	file, dtype I8 / F8_E4M3 / BF16 / F32.  Files written by the `safetensors` package load here byte for byte,
	files written here load there, and the reference's error cases are errors."""
	import numpy as np
	import torch
	from safetensors.torch import load_file, save_file
	rng = np.random.default_rng(5)
	cases = {
		X.INT8: torch.from_numpy(rng.integers(-127, 128, (6, 32), dtype=np.int8)),
		X.E4M3: torch.from_numpy(rng.integers(0, 0x7F, (4, 16), dtype=np.uint8)).view(torch.float8_e4m3fn),
		X.BF16: torch.from_numpy(rng.standard_normal((3, 8), dtype=np.float32)).to(torch.bfloat16),
		X.F32: torch.from_numpy(rng.standard_normal((2, 5, 7), dtype=np.float32)),
	}
	for dtype, tensor in cases.items():
		theirs = str(tmp_path / f"t{dtype}_theirs.safetensors")
		save_file({"x_i8": tensor}, theirs, metadata={"note": "written by the package, with a metadata block"})
		t = X.Tensor.from_safetensors_file(theirs, None)
		assert t.dtype == dtype and t.shape == tuple(tensor.shape)
		raw = tensor.view(torch.uint8).numpy() if dtype != X.F32 else tensor.numpy().view(np.uint8)
		assert t.download(np.uint8 if dtype in (X.E4M3,) else None).tobytes() == raw.tobytes()
		ours = str(tmp_path / "sub" / "dir" / f"t{dtype}_ours.safetensors")      # parent directories are created
		t.save_safetensors_file(ours)
		back = load_file(ours)
		assert list(back) == ["tensor"] and back["tensor"].dtype == tensor.dtype and back["tensor"].shape == tensor.shape
		assert back["tensor"].view(torch.uint8).numpy().tobytes() == raw.tobytes()
	two = str(tmp_path / "two.safetensors")
	save_file({"a": cases[X.INT8], "b": cases[X.INT8].clone()}, two)
	with pytest.raises(X.X17Error, match="expected exactly one tensor, found 2"):
		X.Tensor.from_safetensors_file(two, None)
	f16 = str(tmp_path / "f16.safetensors")
	save_file({"a": torch.zeros(4, dtype=torch.float16)}, f16)
	with pytest.raises(X.X17Error, match="unsupported dtype F16"):
		X.Tensor.from_safetensors_file(f16, None)
	with pytest.raises(X.X17Error, match="cannot open"):
		X.Tensor.from_safetensors_file(str(tmp_path / "missing.safetensors"), None)
	junk = tmp_path / "junk.safetensors"
	junk.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00not json at all!")
	with pytest.raises(X.X17Error, match="invalid safetensors file"):
		X.Tensor.from_safetensors_file(str(junk), None)


def test_reference_tensor_file_conventions(tmp_path):
	"""`<name>_<tag>.safetensors|.bin` (block_utils.py:47-124): the tag names the dtype, .bin needs a shape,
	i8 codes are value * 8 with -128 = NaN, f8 codes decode as the kernels decode them."""
	import numpy as np
	import torch
	from safetensors.torch import save_file
	from x17ai_amd import tensor_files as TF
	assert TF.storage_dtype_tag("tmp/block_torch/ffn_y_f8.bin") == "f8"
	assert TF.storage_dtype_tag("attn_out_i8.safetensors") == "i8"
	for bad in ("x.safetensors", "x_i8.npy", "_i8.bin", "x_u8.bin"):
		with pytest.raises(X.X17Error):
			TF.storage_dtype_tag(bad)
	rng = np.random.default_rng(9)
	real = rng.standard_normal((8, 16)).astype(np.float32) * 4
	codes = np.clip(np.rint(real * 8), -127, 127).astype(np.int8)            # block_utils.py:163-166
	codes[0, 0] = -128
	p = str(tmp_path / "x_i8.safetensors")
	save_file({"x": torch.from_numpy(codes)}, p)
	t = TF.load_tensor_file(p, None)
	assert t.dtype == X.INT8 and t.shape == (8, 16)
	vals = TF.real_values(t.download(), t.dtype)
	assert np.isnan(vals[0, 0]) and np.array_equal(vals.ravel()[1:], codes.ravel()[1:].astype(np.float32) / 8)
	raw = str(tmp_path / "x_i8.bin")
	codes.tofile(raw)
	assert np.array_equal(TF.load_tensor_file(raw, None, (8, 16)).download(), codes)
	with pytest.raises(X.X17Error, match="carries no shape"):
		TF.load_tensor_file(raw, None)
	with pytest.raises(X.X17Error, match="needs 256"):
		TF.load_tensor_file(raw, None, (16, 16))
	wrong = str(tmp_path / "y_f8.safetensors")
	save_file({"y": torch.from_numpy(codes)}, wrong)
	with pytest.raises(X.X17Error, match="declares f8"):
		TF.load_tensor_file(wrong, None)
	# every e4m3 code the reference's encoder emits decodes like torch's float8_e4m3fn (normal codes, zero)
	all_codes = np.array([c for c in range(256) if (c & 0x7F) == 0 or (c & 0x78) != 0 and (c & 0x7F) != 0x7F], np.uint8)
	want = torch.from_numpy(all_codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
	assert np.array_equal(TF.real_values(all_codes, X.E4M3), np.abs(want) * np.where(np.signbit(want) & (want != 0), -1, 1))
	bf = torch.from_numpy(real).to(torch.bfloat16)
	assert np.array_equal(TF.real_values(bf.view(torch.int16).numpy().view(np.uint16), X.BF16), bf.to(torch.float32).numpy())


def test_bench_refuses_more_than_one_gpu():
	r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
	assert r.returncode != 0 and "one GPU" in r.stderr


def test_safetensors_header_that_overflows_is_rejected_before_anything_is_allocated(tmp_path):
	"""A header whose shape times the element size wraps around usize, or whose data lies beyond the end of the
	file, is an error (never a tensor whose shape disagrees with its allocation)."""
	import json
	import struct

	def write(name, header: dict, payload: bytes = b""):
		text = json.dumps(header).encode()
		text += b" " * (-len(text) % 8)
		p = tmp_path / name
		p.write_bytes(struct.pack("<Q", len(text)) + text + payload)
		return str(p)

	wraps = write("wrap_f32.safetensors", {"t": {"dtype": "F32", "shape": [2 ** 62], "data_offsets": [0, 0]}})
	with pytest.raises(X.X17Error, match="invalid safetensors file"):
		X.Tensor.from_safetensors_file(wraps, None)
	wraps2 = write("wrap2_i8.safetensors", {"t": {"dtype": "I8", "shape": [2 ** 33, 2 ** 33], "data_offsets": [0, 0]}})
	with pytest.raises(X.X17Error, match="invalid safetensors file"):
		X.Tensor.from_safetensors_file(wraps2, None)
	short = write("short_i8.safetensors", {"t": {"dtype": "I8", "shape": [1 << 20], "data_offsets": [0, 1 << 20]}}, b"\0" * 16)
	with pytest.raises(X.X17Error, match="truncated tensor data"):
		X.Tensor.from_safetensors_file(short, None)
	with pytest.raises(X.X17Error, match="overflows"):
		X.Tensor(None, (2 ** 62,), X.F32)
	ok = write("ok_i8.safetensors", {"t": {"dtype": "I8", "shape": [2, 8], "data_offsets": [0, 16]}}, bytes(range(16)))
	assert X.Tensor.from_safetensors_file(ok, None).download().ravel().tolist() == list(range(16))
