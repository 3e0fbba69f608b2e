"""The kernel cache on the GPU.  The reference recompiles every kernel on every run (src/device/cuda/gemm.rs:408-416
renders the templates and calls nvcc unconditionally); here kernel_build keys each code object by a hash of everything
it is compiled from and skips the compiler on a match.  A cache hit must launch the identical code object, and any
change of a generated parameter must rebuild."""
import os

import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd import _ffi
from oracle import strict as S
from tests.gpu_common import i8_codes, rng_for

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


def _kernel(dev, name, inp_scale):
	k, n = 128, 256
	cfg = X.GemmConfig(X.GemmInputConfig(X.INT8, k, None, False), X.GemmInputConfig(X.INT8, k, n, True), X.INT8)
	return X.GemmKernel(dev, name, cfg, X.ScaleConfig(inp_scale, 8.0))


def test_cache_hit_launches_the_same_code_object_and_a_changed_parameter_rebuilds(dev, tmp_path, monkeypatch):
	monkeypatch.setenv("X17AI_KERNEL_CACHE", str(tmp_path))
	rng = rng_for("cache")
	m, k, n = 256, 128, 256
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	at, bt = X.Tensor.from_numpy(dev, a, X.INT8), X.Tensor.from_numpy(dev, b, X.INT8)
	kdir = tmp_path / "cache-probe"

	def run(kern):
		c = X.Tensor(dev, (m, n), X.INT8)
		kern.launch(at, bt, c)
		return c.download()

	k1 = _kernel(dev, "cache-probe", 1.0 / 64.0)                       # cold: compiled here, on the GPU box
	hsaco = kdir / "kernel.hsaco"
	assert hsaco.exists() and (kdir / "meta.json").exists() and (kdir / "build.key").exists()
	stamp, key, code = hsaco.stat().st_mtime_ns, (kdir / "build.key").read_text(), hsaco.read_bytes()
	out1 = run(k1)
	assert np.array_equal(out1, S.epilogue_scale(S.gemm_i32(a, b), 1.0 / 64.0, 8.0))

	k2 = _kernel(dev, "cache-probe", 1.0 / 64.0)                       # warm: nothing is compiled
	assert hsaco.stat().st_mtime_ns == stamp and (kdir / "build.key").read_text() == key and hsaco.read_bytes() == code
	assert np.array_equal(run(k2), out1)
	assert k2.metadata == k1.metadata

	k3 = _kernel(dev, "cache-probe", 1.0 / 32.0)                       # one generated parameter differs: rebuilt
	assert (kdir / "build.key").read_text() != key
	assert "1.56250000000000000e-02" not in (kdir / "common.h").read_text()
	out3 = run(k3)
	assert np.array_equal(out3, S.epilogue_scale(S.gemm_i32(a, b), 1.0 / 32.0, 8.0)) and not np.array_equal(out3, out1)
	# the first kernel object keeps the module it loaded: its launches are unaffected by the rebuild
	assert np.array_equal(run(k1), out1)

	# a damaged cache entry is not trusted
	hsaco.unlink()
	k4 = _kernel(dev, "cache-probe", 1.0 / 32.0)
	assert hsaco.exists() and np.array_equal(run(k4), out3)
	assert _ffi.kernel_cache_dir() == str(tmp_path) and sorted(os.listdir(tmp_path)) == ["cache-probe"]
