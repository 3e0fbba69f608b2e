"""Every prebuilt gfx950 code object keeps its working set in registers.

A kernel whose register allocation spills (or whose address arithmetic ends up in stack variables) still computes
the right numbers, so no parity test notices: it only runs several times slower.  The code object itself says so:
its metadata note carries the scratch bytes per lane and the spill counts the compiler recorded.
"""
import glob
import os
import struct

import msgpack
import pytest

KERNELS = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "x17ai_amd", "cache", "kernels")
BUNDLE_MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def device_elf(blob):
	"""The gfx950 ELF inside a clang offload bundle (or the blob itself when it is a bare ELF)."""
	if not blob.startswith(BUNDLE_MAGIC):
		return blob
	pos = len(BUNDLE_MAGIC)
	(count,) = struct.unpack_from("<Q", blob, pos)
	pos += 8
	for _ in range(count):
		offset, size, triple_len = struct.unpack_from("<QQQ", blob, pos)
		pos += 24
		triple = blob[pos:pos + triple_len].decode()
		pos += triple_len
		if "gfx950" in triple:
			return blob[offset:offset + size]
	raise AssertionError("no gfx950 entry in the bundle")


def kernel_metadata(elf):
	"""amdhsa.kernels of the NT_AMDGPU_METADATA note (ELF64 little endian)."""
	assert elf[:4] == b"\x7fELF" and elf[4] == 2 and elf[5] == 1
	shoff, = struct.unpack_from("<Q", elf, 0x28)
	shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
	for i in range(shnum):
		base = shoff + i * shentsize
		sh_type, = struct.unpack_from("<I", elf, base + 4)
		sh_offset, sh_size = struct.unpack_from("<QQ", elf, base + 0x18)
		if sh_type != 7:   # SHT_NOTE
			continue
		pos, end = sh_offset, sh_offset + sh_size
		while pos < end:
			namesz, descsz, ntype = struct.unpack_from("<III", elf, pos)
			pos += 12
			name = elf[pos:pos + namesz].rstrip(b"\0")
			pos += (namesz + 3) & ~3
			desc = elf[pos:pos + descsz]
			pos += (descsz + 3) & ~3
			if name == b"AMDGPU" and ntype == 32:
				return msgpack.unpackb(desc, raw=False)["amdhsa.kernels"]
	raise AssertionError("no AMDGPU metadata note")


def code_objects():
	return sorted(glob.glob(os.path.join(KERNELS, "*", "kernel.hsaco")))


def test_prebuilt_kernels_use_no_scratch_and_spill_no_vector_registers():
	paths = code_objects()
	if not paths:
		pytest.skip("no prebuilt code objects in the tree")
	bad = []
	for path in paths:
		with open(path, "rb") as f:
			kernels = kernel_metadata(device_elf(f.read()))
		assert len(kernels) == 1, path          # every code object exports the one entry `kernel`
		k = kernels[0]
		if k[".private_segment_fixed_size"] != 0 or k[".vgpr_spill_count"] != 0:
			bad.append((os.path.basename(os.path.dirname(path)), k[".private_segment_fixed_size"], k[".vgpr_spill_count"]))
	assert not bad, f"kernels with scratch bytes per lane / spilled vector registers: {bad}"
