"""The C-ABI device shim driven directly, the way the reference's Rust wrappers drive it
(src/device/cuda/cuda_shim.rs:207-562, src/device/cuda.rs:25-101): open context -> stream -> alloc ->
upload -> load_module -> get_kernel -> read_kernel_attrs -> launch with an array of pointers to 8-byte
argument slots -> timer -> download -> synchronize -> teardown, and the error paths: every failure is a
diagnostic that the caller moves into its own growable buffer through x17ai_move_diagnostic.

The module loaded is the GEMM code object the operator layer builds (int8 x int8, scale epilogue), so
the launch is also checked against the oracle bit for bit.
"""
import ctypes
import math
import os

import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd import _ffi, recipes
from oracle import strict as S
from tests.gpu_common import i8_codes, rng_for

pytestmark = pytest.mark.gpu

P = ctypes.c_void_p
SZ = ctypes.c_size_t


class PtrResult(ctypes.Structure):
	_fields_ = [("value", P), ("diagnostic", P)]


class KernelAttrs(ctypes.Structure):
	_fields_ = [(n, ctypes.c_int32) for n in (
		"max_threads_per_block", "static_shared_size_bytes", "const_size_bytes", "local_size_bytes", "num_regs",
		"ptx_version", "binary_version", "max_dynamic_shared_size_bytes", "preferred_shared_memory_carveout")]


class GrowBuffer:
	"""The caller's message buffer.  x17ai_move_diagnostic wants the five callbacks of
	src/util/ffi_buffer.rs:13-103, which return structs by value (not expressible as ctypes callbacks), so
	the move goes through x17h_move_diagnostic_text: the operator layer's C++ twin of that buffer."""

	def __init__(self, capacity=4096):
		self.mem = ctypes.create_string_buffer(capacity)
		self.capacity = capacity

	@property
	def len(self):
		return len(self.mem.value)

	def take(self, diag):
		host = _ffi.host()
		host.x17h_move_diagnostic_text.argtypes = [P, ctypes.c_char_p, SZ]
		host.x17h_move_diagnostic_text.restype = SZ
		host.x17h_move_diagnostic_text(diag, self.mem, self.capacity)

	def text(self):
		return self.mem.value.decode("utf-8", "replace")


@pytest.fixture(scope="module")
def shim():
	lib = ctypes.CDLL(_ffi.lib_paths()["shim"])
	for f in ("open_context", "open_stream", "create_timer", "alloc", "load_module", "get_kernel"):
		getattr(lib, "x17ai_hip_" + f).restype = PtrResult
	lib.x17ai_hip_open_context.argtypes = [SZ]
	lib.x17ai_hip_open_stream.argtypes = [P]
	lib.x17ai_hip_create_timer.argtypes = [P, P]
	lib.x17ai_hip_alloc.argtypes = [P, SZ]
	lib.x17ai_hip_load_module.argtypes = [P, ctypes.c_char_p]
	lib.x17ai_hip_get_kernel.argtypes = [P, ctypes.c_char_p, SZ]
	for f, args in (("close_context", [P]), ("close_stream", [P]), ("synchronize", [P]), ("destroy_timer", [P]),
	                ("timer_start", [P]), ("timer_stop", [P]), ("timer_elapsed_seconds", [P, ctypes.POINTER(ctypes.c_double)]),
	                ("free", [P, P]), ("upload_data", [P, P, P, SZ, SZ]), ("download_data", [P, P, P, SZ, SZ]),
	                ("del_module", [P]), ("read_kernel_attrs", [P, ctypes.POINTER(KernelAttrs)]),
	                ("launch_kernel", [P, P] + [SZ] * 7 + [ctypes.POINTER(P)])):
		fn = getattr(lib, "x17ai_hip_" + f)
		fn.argtypes = args
		fn.restype = P
	lib.x17ai_hip_context_ptr.argtypes = [P]
	lib.x17ai_hip_context_ptr.restype = P
	return lib


def _ok(shim, diag):
	"""A NULL diagnostic is success; anything else is moved into a buffer and raised."""
	if diag:
		buf = GrowBuffer()
		buf.take(diag)
		raise AssertionError(buf.text())


def _value(shim, res):
	_ok(shim, res.diagnostic)
	assert res.value
	return res.value


def _message(shim, diag):
	assert diag, "expected a diagnostic"
	buf = GrowBuffer()
	buf.take(diag)
	return buf.text()


def test_call_sequence_of_the_reference_wrappers(shim):
	m, k, n = 512, 1024, 512
	built = recipes.attn_q_kernel(None, k, n)            # generates + compiles (or finds) the code object, no device
	meta = built.metadata
	path = os.path.join(_ffi.kernel_cache_dir(), built.name, "kernel.hsaco")
	assert os.path.exists(path)

	ctx = _value(shim, shim.x17ai_hip_open_context(0))
	assert ctypes.cast(ctx, ctypes.POINTER(SZ))[0] == 0           # refcnt_minus_one, the one visible field
	assert shim.x17ai_hip_context_ptr(ctx)
	stream = _value(shim, shim.x17ai_hip_open_stream(ctx))
	timer = _value(shim, shim.x17ai_hip_create_timer(ctx, stream))

	rng = rng_for("shim", m, k, n)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	da = _value(shim, shim.x17ai_hip_alloc(stream, a.nbytes))
	db = _value(shim, shim.x17ai_hip_alloc(stream, b.nbytes))
	dc = _value(shim, shim.x17ai_hip_alloc(stream, m * n))
	_ok(shim, shim.x17ai_hip_upload_data(stream, a.ctypes.data, da, 0, a.nbytes))
	# an upload in two pieces through the offset argument
	half = b.nbytes // 2
	_ok(shim, shim.x17ai_hip_upload_data(stream, b.ctypes.data, db, 0, half))
	_ok(shim, shim.x17ai_hip_upload_data(stream, b.ctypes.data + half, db, half, b.nbytes - half))

	module = _value(shim, shim.x17ai_hip_load_module(ctx, path.encode()))
	kernel = _value(shim, shim.x17ai_hip_get_kernel(module, b"kernel", meta["SMEM_BYTES"]))
	attrs = KernelAttrs()
	_ok(shim, shim.x17ai_hip_read_kernel_attrs(kernel, ctypes.byref(attrs)))
	assert attrs.max_threads_per_block >= meta["THREADS_PER_BLOCK"]
	assert 0 < attrs.num_regs <= 512 and attrs.local_size_bytes == 0
	assert attrs.max_dynamic_shared_size_bytes >= meta["SMEM_BYTES"]

	# 8-byte slots passed by address, as src/device/cuda/gemm.rs:618-631 does; the kernel's u32 parameters
	# read the low halves
	slots = [ctypes.c_uint64(da), ctypes.c_uint64(m), ctypes.c_uint64(db), ctypes.c_uint64(n), ctypes.c_uint64(dc), ctypes.c_uint64(0)]
	args = (P * len(slots))(*[ctypes.cast(ctypes.byref(s), P) for s in slots])
	grid = (m // meta["M_PER_BLOCK"], n // meta["N_PER_BLOCK"], 1)     # the reference's one workgroup per tile
	_ok(shim, shim.x17ai_hip_timer_start(timer))
	_ok(shim, shim.x17ai_hip_launch_kernel(stream, kernel, grid[0], grid[1], grid[2], meta["THREADS_PER_BLOCK"], 1, 1,
	                                      meta["SMEM_BYTES"], args))
	_ok(shim, shim.x17ai_hip_timer_stop(timer))
	got = np.empty((m, n), np.int8)
	_ok(shim, shim.x17ai_hip_download_data(stream, dc, got.ctypes.data, 0, got.nbytes))
	_ok(shim, shim.x17ai_hip_synchronize(stream))
	seconds = ctypes.c_double(-1.0)
	_ok(shim, shim.x17ai_hip_timer_elapsed_seconds(timer, ctypes.byref(seconds)))
	assert 0.0 < seconds.value < 1.0
	want = S.epilogue_scale(S.gemm_i32(a, b), 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(got, want)
	# a download through the offset argument
	tail = np.empty(n, np.int8)
	_ok(shim, shim.x17ai_hip_download_data(stream, dc, tail.ctypes.data, (m - 1) * n, n))
	_ok(shim, shim.x17ai_hip_synchronize(stream))
	assert np.array_equal(tail, want[-1])

	# ---- error paths: diagnostics with a message, never a crash
	msg = _message(shim, shim.x17ai_hip_load_module(ctx, b"/nonexistent/kernel.hsaco").diagnostic)
	assert "x17ai_hip_load_module" in msg and "/nonexistent/kernel.hsaco" in msg
	msg = _message(shim, shim.x17ai_hip_get_kernel(module, b"no_such_entry", 0).diagnostic)
	assert "x17ai_hip_get_kernel" in msg and "no_such_entry" in msg
	msg = _message(shim, shim.x17ai_hip_get_kernel(module, b"kernel", 1 << 20).diagnostic)
	assert "x17ai_hip_get_kernel" in msg                        # more dynamic LDS than a compute unit has
	msg = _message(shim, shim.x17ai_hip_launch_kernel(stream, kernel, 1, 1, 1, 4096, 1, 1, meta["SMEM_BYTES"], args))
	assert "x17ai_hip_launch_kernel" in msg                     # 4096 threads per block
	msg = _message(shim, shim.x17ai_hip_open_context(10 ** 6).diagnostic)
	assert "x17ai_hip_open_context" in msg
	# two diagnostics moved into ONE buffer append, they do not overwrite
	buf = GrowBuffer()
	buf.take(shim.x17ai_hip_load_module(ctx, b"/nonexistent/a.hsaco").diagnostic)
	first = buf.len
	buf.take(shim.x17ai_hip_load_module(ctx, b"/nonexistent/b.hsaco").diagnostic)
	assert buf.len > first and "a.hsaco" in buf.text() and "b.hsaco" in buf.text()
	# the stream still works after the failures
	_ok(shim, shim.x17ai_hip_synchronize(stream))

	# ---- teardown in the wrappers' drop order
	for d in (da, db, dc):
		_ok(shim, shim.x17ai_hip_free(stream, d))
	_ok(shim, shim.x17ai_hip_destroy_timer(timer))
	_ok(shim, shim.x17ai_hip_del_module(module))
	_ok(shim, shim.x17ai_hip_close_stream(stream))
	_ok(shim, shim.x17ai_hip_close_context(ctx))
