"""Hand-written memory instructions (the direct-to-LDS tile requests are inline assembly with scalar operands) sit outside
the compiler's hazard bookkeeping: on gfx9-family hardware a scalar register written by the vector unit (v_readfirstlane,
v_readlane) must not be read by a memory instruction within the next five instructions.  The product sources never put
such a write in front of a request -- their addresses are scalar arithmetic -- and this test holds the built code objects
to that: it disassembles this repository's own kernels (never a shipped library) and scans every memory instruction.
A second rule of the same family: a scalar write of M0 needs one wait state before a direct-to-LDS load reads it (the
compiler inserts an s_nop for its own loads; the hand-written requests carry their own), so no instruction that writes
M0 may sit directly in front of a *_load_lds_* instruction.
A third rule is this pool's: packed single-precision arithmetic (v_pk_add_f32, v_pk_mul_f32, v_pk_fma_f32) is compiled out
(-target-feature -packed-fp32-ops) and never written by hand; the scan holds every built code object to it."""
import glob
import os
import re
import shutil
import subprocess

import pytest

from x17ai_amd import recipes

BUNDLER = "/opt/rocm/llvm/bin/clang-offload-bundler"
OBJDUMP = "/opt/rocm/llvm/bin/llvm-objdump"
MEMORY = re.compile(r"(global|buffer|flat|scratch)_(load|store|atomic)")
SCALAR_WRITE = re.compile(r"(v_readfirstlane_b32|v_readlane_b32)\s+s(\d+)")
SCALAR_PAIR = re.compile(r"s\[(\d+):(\d+)\]")
M0_WRITE = re.compile(r"s_\w+\s+m0\s*,")
LDS_DMA = re.compile(r"(global|buffer)_load_lds_\w+|buffer_load_\w+.*\blds\b")
PACKED_F32 = re.compile(r"v_pk_(add|mul|fma)_f32")


def _instructions(code_object, tmp_path):
	obj = os.path.join(tmp_path, "kernel.o")
	subprocess.run([BUNDLER, "--unbundle", "--type=o", "--input=" + code_object, "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
	                "--output=" + obj], check=True, capture_output=True)
	text = subprocess.run([OBJDUMP, "-d", obj], check=True, capture_output=True, text=True).stdout
	return [line.strip() for line in text.split("\n") if line.startswith("\t")]


def _hazards(ins):
	found = []
	for i, line in enumerate(ins):
		if not MEMORY.match(line):
			continue
		pair = SCALAR_PAIR.search(line)
		if not pair:
			continue
		lo, hi = int(pair.group(1)), int(pair.group(2))
		for j in range(max(0, i - 5), i):
			w = SCALAR_WRITE.match(ins[j])
			if w and lo <= int(w.group(2)) <= hi:
				found.append((ins[j], line, i - j))
	return found


def _m0_hazards(ins):
	return [(ins[i - 1], line) for i, line in enumerate(ins) if i > 0 and LDS_DMA.match(line) and M0_WRITE.match(ins[i - 1])]


@pytest.mark.skipif(not (os.path.exists(BUNDLER) and os.path.exists(OBJDUMP) and shutil.which("hipcc")), reason="needs the ROCm LLVM tools")
def test_no_memory_instruction_reads_a_scalar_register_the_vector_unit_has_just_written(tmp_path):
	kernels = [recipes.attn_kernel(None, h, hd, strict) for h, hd in ((4, 32), (2, 64), (2, 128)) for strict in (True, False)]
	kernels.append(recipes.attn_q_kernel(None, 128, 256))
	kernels.append(recipes.mixed_gemm_kernel(None, 512, 384, False))
	cache = os.path.join(os.path.dirname(os.path.abspath(recipes.__file__)), "cache", "kernels")
	scanned = 0
	for k in kernels:
		code_object = os.path.join(cache, k.name, "kernel.hsaco")
		assert os.path.exists(code_object), code_object
		ins = _instructions(code_object, str(tmp_path))
		assert any("global_load_lds" in line for line in ins), k.name          # the hand-written requests are in there
		assert _hazards(ins) == [], k.name
		assert _m0_hazards(ins) == [], k.name
		scanned += 1
	# and whatever else has been built into the cache
	for code_object in glob.glob(os.path.join(cache, "*", "kernel.hsaco")):
		ins = _instructions(code_object, str(tmp_path))
		assert _hazards(ins) == [], code_object
		assert _m0_hazards(ins) == [], code_object
		assert [line for line in ins if PACKED_F32.match(line)] == [], code_object
		scanned += 1
	assert scanned >= len(kernels)


def test_the_scan_sees_a_hazard_when_there_is_one():
	ins = ["v_readfirstlane_b32 s21, v117", "v_readfirstlane_b32 s20, v116", "s_mov_b32 m0, s8", "global_load_lds_dwordx4 v122, s[20:21]"]
	assert len(_hazards(ins)) == 2
	ins = ["v_readfirstlane_b32 s20, v116"] + ["s_nop 0"] * 5 + ["global_load_lds_dwordx4 v122, s[20:21]"]
	assert _hazards(ins) == []
	assert len(_m0_hazards(["s_add_i32 m0, s8, 0x1000", "global_load_lds_dwordx4 v122, s[20:21]"])) == 1
	assert len(_m0_hazards(["s_mov_b32 m0, s8", "global_load_lds_dwordx4 v122, s[20:21]"])) == 1
	assert _m0_hazards(["s_mov_b32 m0, s8", "s_nop 0", "global_load_lds_dwordx4 v122, s[20:21]"]) == []
	assert _m0_hazards(["s_add_i32 m0, s8, 0x1000", "v_add_u32_e32 v1, v2, v3", "global_load_lds_dwordx4 v122, s[20:21]"]) == []
