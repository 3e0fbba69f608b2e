"""The kernels' hand-written tile requests (global -> LDS, 16 bytes per lane, addresses formed from scalar bases and
lane offsets outside the compiler's view) are audited on the CPU: the index arithmetic lives in gemm_tile.h /
attn_tile.h, the kernels call it, and the audit programs beside them (gemm_requests_audit.cpp,
attn_requests_audit.cpp) are compiled here with a kernel's own generated common.h and enumerate every request of a
launch -- every tile of the persistent walk and K step, every (sequence, head, query block) and step of the request
schedule, overhanging tiles and past-the-end repeats included.  Each must stay inside its operand and each tile's
chunks must be requested exactly once.  No GPU is involved."""
import json
import os
import shutil
import subprocess

import pytest

import x17ai_amd as X
from x17ai_amd import _ffi, recipes

KERNELS = os.path.join(os.path.dirname(os.path.abspath(recipes.__file__)), "csrc", "kernels")
pytestmark = pytest.mark.skipif(shutil.which("g++") is None or shutil.which("hipcc") is None, reason="needs g++ and hipcc")


def _audit(tmp_path, kernel, source, *args):
	"""Compiles `source` against the configuration of `kernel` (a kernel object built without a device) and runs it."""
	exe = os.path.join(str(tmp_path), kernel.name + "." + source.split(".")[0])
	if not os.path.exists(exe):
		subprocess.run(["g++", "-std=c++17", "-O2", "-I" + os.path.join(_ffi.kernel_cache_dir(), kernel.name), "-I" + KERNELS,
		                os.path.join(KERNELS, source), "-o", exe], check=True)
	out = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True)
	return json.loads(out.stdout), out.returncode


GEMMS = [
	("scale, 8 waves, off the grid", lambda: recipes.attn_q_kernel(None, 512, 384), (256, 320, 1024)),
	("K = 128, a single step", lambda: recipes.attn_q_kernel(None, 128, 256), (256, 320)),
	("K = 384: the shortest deep token ring", lambda: recipes.attn_q_kernel(None, 384, 1024), (256, 2048)),
	("GeGLU, config 4 ffn_f", lambda: recipes.ffn_f_kernel(None, 2048, 16384, False), (256, 32768)),
	("L2-norm writer (natural weight rows), off the grid", lambda: recipes.attn_kv_kernel(None, 512, 384, 32), (320, 576)),
	("fused q + kv, 256 + 384 columns", lambda: recipes.attn_qkv_kernel(None, 512, 256, 384, 64), (320, 2048)),
	("fused q + kv, config 4", lambda: recipes.attn_qkv_kernel(None, 2048, 2048, 4096, 128, False), (32768,)),
	("e4m3 x int8, four waves of 128 x 128, config 4 ffn_y", lambda: recipes.ffn_y_kernel(None, 2048, 8192, False), (256, 32768)),
	("e4m3 x e4m3, config 3", lambda: recipes.ffn_f_f8_kernel(None, 4096, 32768, False), (16384,)),
	("mixed, off the grid", lambda: recipes.mixed_gemm_kernel(None, 512, 384, False), (320,)),
]


@pytest.mark.parametrize("label,make,row_counts", GEMMS, ids=[g[0] for g in GEMMS])
def test_gemm_tile_requests_stay_inside_their_operands(tmp_path, label, make, row_counts):
	kern = make()
	for rows in row_counts:
		rep, rc = _audit(tmp_path, kern, "gemm_requests_audit.cpp", rows)
		assert rc == 0 and rep["ok"], (label, rows, rep)
		# the walk reaches the last byte of every operand and never goes beyond
		assert rep["a_extent"] == rep["a_bytes"] and rep["b_extent"] == rep["b_bytes"] and rep["b_kv_extent"] == rep["b_kv_bytes"], (label, rows, rep)
	# the audit sees a request that leaves its operand: the same launch over a token matrix one row short
	rep, rc = _audit(tmp_path, kern, "gemm_requests_audit.cpp", row_counts[0], row_counts[0] - 1)
	assert rc != 0 and not rep["ok"] and "past the end of a" in rep["error"], rep
	# shapes the launcher rejects are not audited as if they could run
	rep, rc = _audit(tmp_path, kern, "gemm_requests_audit.cpp", 192)
	assert rc != 0 and not rep["ok"]


ATTNS = [
	("config 4 speed build", lambda: recipes.attn_kernel(None, 16, 128, False), ((8192, 4, 512), (128, 1, 0), (192, 3, 16), (320, 2, 4096))),
	("config 5 speed build", lambda: recipes.attn_kernel(None, 32, 128, False), ((65536, 1, 4096),)),
	("strict build, head_dim 64 (two staging wavefronts)", lambda: recipes.attn_kernel(None, 2, 64, True), ((1024, 1, 256), (192, 2, 0), (128, 1, 16))),
	("head_dim 32 (one staging wavefront)", lambda: recipes.attn_kernel(None, 4, 32, False), ((768, 1, 64), (192, 1, 0))),
	("row-scaled speed build", lambda: recipes.attn_row_scaled_kernel(None, 8, 64, X.BF16, False), ((1024, 1, 256), (320, 2, 48))),
]


@pytest.mark.parametrize("label,make,shapes", ATTNS, ids=[a[0] for a in ATTNS])
def test_attention_tile_requests_stay_inside_their_sequence(tmp_path, label, make, shapes):
	kern = make()
	for seq_len, batch, window in shapes:
		rep, rc = _audit(tmp_path, kern, "attn_requests_audit.cpp", seq_len, batch, window)
		assert rc == 0 and rep["ok"], (label, seq_len, batch, window, rep)
		assert rep["kv_extent"] == rep["kv_bytes"] and rep["q_extent"] == rep["q_bytes"] and rep["scale_extent_rows"] == rep["rows"], rep
	seq_len, batch, window = shapes[0]
	rep, rc = _audit(tmp_path, kern, "attn_requests_audit.cpp", seq_len, batch, window, seq_len * batch - 1)
	assert rc != 0 and not rep["ok"] and "past the end" in rep["error"], rep
	rep, rc = _audit(tmp_path, kern, "attn_requests_audit.cpp", 96, 1, 0)
	assert rc != 0 and not rep["ok"]


D_KVS = [
	("config 4", lambda: recipes.attn_d_kv_kernel(None, 16, 128, False), ((2048, 16, 512), (128, 1, 0), (192, 3, 16), (320, 2, 4096))),
	("head_dim 64 (two staging wavefronts)", lambda: recipes.attn_d_kv_kernel(None, 8, 64, True), ((1024, 1, 256), (192, 2, 0), (128, 1, 16))),
	("head_dim 32 (one staging wavefront)", lambda: recipes.attn_d_kv_kernel(None, 4, 32, True), ((768, 1, 64), (256, 3, 16))),
]


@pytest.mark.parametrize("label,make,shapes", D_KVS, ids=[a[0] for a in D_KVS])
def test_attention_backward_kv_requests_and_lds_layouts(tmp_path, label, make, shapes):
	"""attn_bwd_kv_tile.h: the three LDS layouts' request maps are the inverses of the readers' offset functions, every
	16-byte position of a tile is requested once, operand reads stay inside their tiles, and every workgroup's walk
	over query tiles covers exactly the queries that see its keys, inside its own sequence and inside q, d_out, L and D."""
	kern = make()
	for seq_len, batch, window in shapes:
		rep, rc = _audit(tmp_path, kern, "attn_bwd_kv_requests_audit.cpp", seq_len, batch, window)
		assert rc == 0 and rep["ok"], (label, seq_len, batch, window, rep)
		assert rep["q_extent"] == rep["q_bytes"] and rep["d_out_extent"] == rep["d_out_bytes"] and rep["ld_extent_rows"] == rep["rows"], rep
	seq_len, batch, window = shapes[0]
	rep, rc = _audit(tmp_path, kern, "attn_bwd_kv_requests_audit.cpp", seq_len, batch, window, seq_len * batch - 1)
	assert rc != 0 and not rep["ok"] and "past the end" in rep["error"], rep
	rep, rc = _audit(tmp_path, kern, "attn_bwd_kv_requests_audit.cpp", 64, 1, 0)
	assert rc != 0 and not rep["ok"]
