"""Compiles, without a GPU, every code object the tests, the smoke check and the benchmark ask for.

The operator layer builds kernels on demand (one code object per configuration, cached by
content hash); a machine that runs the tests should find all of them already built.
"""
from __future__ import annotations

import concurrent.futures
import math
import os
import subprocess

from . import recipes
from .api import E4M3, INT8, BF16, GeGluConfig, GemmConfig, GemmInputConfig, GemmKernel, ScaleConfig

_HERE = os.path.dirname(os.path.abspath(__file__))

TEST_SHAPES = [(256, 128, 256), (512, 1024, 512), (256, 2048, 1024)]


def _specs():
	s = []
	add = s.append
	# ---- tests/test_gpu_gemm.py
	for _, k, n in TEST_SHAPES:
		add(("attn_q", k, n))
		for store in (E4M3, INT8):
			for strict in (True, False):
				add(("ffn_f", k, n, strict, store))
				add(("attn_y", n // 2, k, strict, store))
	add(("acc_probe",))
	add(("e4m3_range",))
	for geglu in (False, True):
		add(("mixed", 1024, 512, geglu))
	for hd in (32, 64, 128):
		for k in (512, 2048):
			add(("attn_kv", k, 512, hd))
	for k, n in ((512, 256), (2048, 512)):
		add(("ffn_y", n // 2, k, True, E4M3, INT8))
	for k, n in ((512, 256), (4096, 512)):
		add(("ffn_f_f8", k, n, True))
	for hd in (32, 64, 128):             # learned-scale Q writer; fused q + kv
		add(("attn_q_norm", 512, 512, hd, 0.0))
		add(("attn_qkv", 512, 256, 512, hd, True))
	add(("attn_q_norm", 2048, 1024, 128, recipes.L2_NORM_EPS))
	add(("attn_q_norm", 512, 512, 64, 0.0, 1.0 / math.sqrt(512)))
	for hd in (64, 128):                 # L2-norm writer on a walk of more tiles than workgroups
		add(("attn_kv", 256, 2048, hd))
	# shapes off the 256-grid (rows % 64, raw columns % 128 as the reference accepts them)
	add(("attn_q", 512, 384))
	add(("ffn_f", 512, 384, True, E4M3))
	add(("attn_y", 192, 512, True, E4M3))
	for hd in (32, 64):
		add(("attn_kv", 512, 384, hd))
	add(("mixed", 512, 384, False))
	for geglu in (False, True):
		add(("dequant", 512, 384, INT8, INT8, geglu, True))
	add(("attn_q_norm", 512, 384, 64, 0.0))
	add(("attn_qkv", 512, 256, 384, 64, True))
	add(("attn_q", 384, 1024))           # the shortest K with the deeper token ring, more tiles than workgroups
	add(("ffn_f_f8", 384, 512, True))
	# ---- tests/test_gpu_attn.py
	for h, hd in ((4, 32), (2, 64), (2, 128), (8, 64)):
		add(("attn", h, hd, True))
	for h, hd in ((2, 64), (2, 128), (8, 64), (4, 32), (4, 64)):
		add(("attn", h, hd, False))
	for h, hd, out in ((8, 64, BF16), (4, 32, BF16), (2, 128, BF16), (2, 64, INT8), (2, 64, BF16)):
		add(("attn_rows", h, hd, out, True))
	for h, hd in ((8, 64), (2, 128)):
		add(("attn_rows", h, hd, BF16, False))
	# ---- tests/test_gpu_attn_bwd.py
	for h, hd in ((8, 64), (2, 128), (4, 32), (2, 64)):
		add(("attn_d_q", h, hd, True))
	add(("attn_d_q", 8, 64, False))
	add(("attn_d_q", 16, 128, False))                    # bench.py
	for h, hd in ((8, 64), (2, 128), (4, 32), (2, 64)):
		add(("attn_d_kv", h, hd, True))
	add(("attn_d_kv", 8, 64, False))
	add(("attn_d_kv", 16, 128, False))                   # bench.py
	add(("attn_d_q", 4, 128, False))
	add(("attn_d_kv", 4, 128, False))
	add(("attn", 4, 128, False))
	for h, hd, cap in ((4, 32, 256), (4, 64, 256), (2, 128, 512), (2, 32, 4096), (2, 64, 4096)):
		add(("decode", h, hd, cap, True))
	for h, hd, cap, out in ((4, 64, 256, BF16), (2, 128, 512, BF16), (4, 32, 256, INT8)):
		add(("decode_rows", h, hd, cap, out, True))
	for d in (512, 2048, 4096):
		add(("rms_norm", d, E4M3))
		add(("rms_norm", d, BF16))
	# ---- __graft_entry__.smoke()
	add(("ffn_f", 512, 512, True, INT8))
	add(("ffn_y", 512, 256, True, INT8, INT8))
	# ---- bench.py
	for strict in (False, True):
		add(("ffn_f", 2048, 16384, strict, INT8))
		add(("ffn_y", 2048, 8192, strict, INT8, INT8))
		add(("attn", 32, 128, strict))
		add(("decode", 32, 128, 4096, strict))
	add(("ffn_f_f8", 4096, 32768, False))
	add(("ffn_y", 4096, 16384, False, E4M3, E4M3))
	add(("ffn_f_f8", 4096, 32768, True))                 # tests/test_gpu_fullsize.py: config 3, strict builds
	add(("ffn_y", 4096, 16384, True, E4M3, E4M3))
	add(("attn_q", 2048, 2048))
	add(("attn_kv", 2048, 4096, 128))
	add(("attn", 16, 128, False))
	add(("attn_y", 2048, 2048, False, E4M3))
	add(("ffn_f", 2048, 16384, False, E4M3))
	add(("ffn_y", 2048, 8192, False, E4M3, INT8))
	add(("attn", 8, 64, False))
	add(("attn_rows", 32, 128, BF16, False))
	add(("decode_rows", 32, 128, 4096, BF16, False))
	# ---- tests/test_gpu_fullsize.py (the strict ffn pair, attention and decode kernels are listed above)
	add(("attn", 16, 128, True))
	add(("attn_rows", 32, 128, BF16, True))
	add(("decode_rows", 32, 128, 4096, BF16, True))
	add(("acc_probe_full",))
	# ---- tests/test_gpu_refconfig.py: the reference's own configuration (64 heads of 32, widths 2048)
	add(("attn_kv", 2048, 4096, 32))
	add(("attn", 64, 32, True))
	add(("attn_y", 2048, 2048, True, E4M3))
	add(("ffn_f", 2048, 4096, True, E4M3))
	add(("ffn_y", 2048, 2048, True, E4M3, INT8))
	# ---- tests/test_gpu_gemm.py: run-time dequantisation scales, bf16 out
	for strict in (True, False):
		add(("dequant", 1024, 512, INT8, INT8, False, strict))
		add(("dequant", 1024, 512, INT8, INT8, True, strict))
	add(("dequant", 512, 256, E4M3, E4M3, False, True))
	# ---- tests/test_gpu_fullsize.py: benchmark config 2 in its literal form (per-token / per-channel scales)
	for strict in (True, False):                             # the speed builds are bench.py's
		add(("dequant", 2048, 16384, INT8, INT8, True, strict))
		add(("dequant", 8192, 2048, INT8, INT8, False, strict))
	# ---- x17ai_amd.block: benchmark config 4 (bench.py, tests/config4_chain.py) and the reference's own configuration
	for strict in (True, False):
		add(("block", 2048, 16, 128, 8192, BF16, strict))
		add(("attn_qkv", 2048, 2048, 4096, 128, strict))
	add(("block", 2048, 64, 32, 2048, None, True))
	add(("block", 512, 8, 32, 256, None, True))          # tests/test_gpu_files.py
	add(("attn_q", 128, 256))
	add(("attn_y", 128, 128, True, INT8))                # tests/test_gpu_gemm.py: the launcher's alias check
	return s


def _build_one(spec) -> str:
	kind = spec[0]
	if kind == "block":
		from .block import Block, BlockConfig
		Block(None, BlockConfig(spec[1], spec[2], spec[3], spec[4], 0, 1, spec[5], spec[6]))
		return f"block-d{spec[1]}-h{spec[2]}x{spec[3]}-f{spec[4]}-{'strict' if spec[6] else 'fast'}"
	if kind == "attn_q":
		return recipes.attn_q_kernel(None, spec[1], spec[2]).name
	if kind == "attn_q_norm":
		return recipes.attn_q_norm_kernel(None, spec[1], spec[2], spec[3], spec[4], True, spec[5] if len(spec) > 5 else 1.0).name
	if kind == "attn_qkv":
		return recipes.attn_qkv_kernel(None, spec[1], spec[2], spec[3], spec[4], spec[5]).name
	if kind == "ffn_f":
		return recipes.ffn_f_kernel(None, spec[1], spec[2], spec[3], spec[4]).name
	if kind == "attn_y":
		return recipes.attn_y_kernel(None, spec[1], spec[2], spec[3], spec[4]).name
	if kind == "attn_kv":
		return recipes.attn_kv_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "ffn_y":
		return recipes.ffn_y_kernel(None, spec[1], spec[2], spec[3], spec[4], spec[5]).name
	if kind == "mixed":
		return recipes.mixed_gemm_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "ffn_f_f8":
		return recipes.ffn_f_f8_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "attn":
		return recipes.attn_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "attn_d_q":
		return recipes.attn_d_q_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "attn_d_kv":
		return recipes.attn_d_kv_kernel(None, spec[1], spec[2], spec[3]).name
	if kind == "attn_rows":
		return recipes.attn_row_scaled_kernel(None, spec[1], spec[2], spec[3], spec[4]).name
	if kind == "decode":
		return recipes.attn_decode_kernel(None, spec[1], spec[2], spec[3], spec[4]).name
	if kind == "decode_rows":
		return recipes.attn_decode_row_scaled_kernel(None, spec[1], spec[2], spec[3], spec[4], spec[5]).name
	if kind == "rms_norm":
		return recipes.rms_norm_kernel(None, spec[1], spec[2]).name
	if kind == "dequant":
		return recipes.dequant_gemm_kernel(None, spec[1], spec[2], spec[3], spec[4], spec[5], spec[6]).name
	if kind == "acc_probe":
		k, n = 1024, 256
		cfg = GemmConfig(GemmInputConfig(INT8, k, None, False), GemmInputConfig(INT8, k, n, True), INT8)
		GemmKernel(None, f"acc_probe-k{k}-n{n}", cfg, ScaleConfig(1.0, 1.0))
		return GemmKernel(None, f"acc_probe2-k{k}-n{n}", cfg, ScaleConfig(1.0 / (k * 127.0), 1.0)).name
	if kind == "e4m3_range":
		cfg = GemmConfig(GemmInputConfig(INT8, 128, None, False), GemmInputConfig(INT8, 128, 256, True), E4M3)
		GemmKernel(None, "e4m3_range-strict", cfg, GeGluConfig(1.0 / 32.0, 1.0), True)
		return GemmKernel(None, "e4m3_range-fast", cfg, GeGluConfig(1.0 / 32.0, 1.0), False).name
	if kind == "acc_probe_full":
		k, n = 2048, 16384
		cfg = GemmConfig(GemmInputConfig(INT8, k, None, False), GemmInputConfig(INT8, k, n, True), INT8)
		return GemmKernel(None, f"acc_probe-k{k}-n{n}", cfg, ScaleConfig(1.0, 1.0)).name
	raise ValueError(spec)


def build_host_libraries() -> None:
	subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-j4"], check=True, stdout=subprocess.DEVNULL)


def build_all(workers: int = 8) -> list:
	build_host_libraries()
	specs = _specs()
	names = []
	with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
		for name in pool.map(_build_one, specs):
			names.append(name)
	return names


if __name__ == "__main__":
	import time
	t0 = time.time()
	built = build_all()
	print(f"built {len(built)} kernels in {time.time() - t0:.1f}s")
