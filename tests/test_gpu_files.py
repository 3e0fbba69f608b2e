"""File -> device -> kernels -> file on the GPU: the path of the reference's block driver (src/main.rs:40-75 loads
nine `<name>_<tag>.safetensors` files with Tensor::from_safetensors_file, src/tensor.rs:155-179; :264-280 stores
eight with save_safetensors_file, src/tensor.rs:213-249) through x17ai_amd.block, checked against the CPU oracle.
"""
import math
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import x17ai_amd as X
from x17ai_amd import block as BL
from x17ai_amd import recipes
from x17ai_amd import tensor_files as TF
from oracle import strict as S
from tests.gpu_common import e4m3_compare, i8_codes, rng_for

pytestmark = pytest.mark.gpu

T, D, H, HD, F = 512, 512, 8, 32, 256


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


def _inputs():
	rng = rng_for("files-block")
	sk = rng.standard_normal((H, HD))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	return {
		"x": i8_codes(rng, (T, D)),
		"attn_q_weights": i8_codes(rng, (H * HD, D)),
		"attn_kv_weights": i8_codes(rng, (H, 2, HD, D)),            # rank 4 on disk, as new_block.py stores it
		"ffn_f_weights": i8_codes(rng, (2 * F, D)),
		"ffn_y_weights": i8_codes(rng, (2 * D, F)),
		"attn_y_weights": i8_codes(rng, (2 * D, H * HD)),
		"sinks_k": S.f32_to_fixedi8((sk * 8).astype(np.float32)),
		"sinks_v": i8_codes(rng, (H, HD), 1.3),
		"attn_temperature": (0.5 + rng.random((H, 1))).astype(np.float32),
	}


def test_block_driver_over_tensor_files(dev, tmp_path, capsys):
	inp = _inputs()
	src, dst = tmp_path / "block_torch", tmp_path / "block_hip"
	src.mkdir()
	for key, stem in BL.INPUT_FILES:
		save_file({key: torch.from_numpy(inp[key])}, str(src / (stem + ".safetensors")))
	# the driver itself, arguments as the reference's constants (src/main.rs:28-35)
	rc = BL.main(["--input", str(src), "--output", str(dst), "--head-dim", str(HD), "--n-heads", str(H), "--f-width", str(F)])
	assert rc == 0
	text = capsys.readouterr().out
	assert "attn_q in" in text and "ffn_y_f8 in" in text and "TFLOPS" in text      # src/main.rs:356-373
	got = {}
	for key, stem in BL.OUTPUT_FILES:
		back = load_file(str(dst / (stem + ".safetensors")))
		assert list(back) == ["tensor"]                                              # src/tensor.rs:236
		got[key] = back["tensor"]
	assert got["kv"].shape == (T, H, 2, HD) and got["kv"].dtype == torch.int8        # src/main.rs:266
	assert got["attn_y"].dtype == torch.float8_e4m3fn and got["attn_l"].shape == (H, T)
	np8 = lambda t: t.view(torch.uint8).numpy() if t.dtype == torch.float8_e4m3fn else t.numpy()
	x = inp["x"]
	inp_scale = 1.0 / math.sqrt(D) / 64.0
	q = S.epilogue_scale(S.gemm_i32(x, inp["attn_q_weights"]), inp_scale, 8.0)
	assert np.array_equal(np8(got["q"]), q)
	kv, rrms = S.epilogue_l2norm(S.gemm_i32(x, inp["attn_kv_weights"].reshape(2 * H * HD, D)), HD, recipes.L2_NORM_EPS, inp_scale, 8.0)
	assert np.array_equal(np8(got["kv"]).reshape(T, 2 * H * HD), kv)
	assert np.array_equal(np8(got["k_rrms"]).view(np.uint32), rrms.view(np.uint32))
	ao, al = S.attn_fwd_i8(q, kv, inp["sinks_k"], inp["sinks_v"], inp["attn_temperature"].reshape(-1), H, HD, 0)
	assert np.array_equal(np8(got["attn_out"]), ao)
	assert np.array_equal(np8(got["attn_l"]).view(np.uint32), al.view(np.uint32))
	ay = S.epilogue_residual(S.gemm_i32(ao, inp["attn_y_weights"]), x, 1.0 / math.sqrt(H * HD) / 64.0, 1.0, S.STORE_E4M3)
	assert np.array_equal(np8(got["attn_y"]), ay)
	ff = S.epilogue_geglu(S.gemm_i32(x, inp["ffn_f_weights"]), inp_scale, 1.0, S.STORE_E4M3)
	assert np.array_equal(np8(got["ffn_f"]), ff)
	fy = S.epilogue_residual(S.gemm_f32_seq(ff, True, inp["ffn_y_weights"], False), x, math.sqrt(recipes.GELU_VAR_FIX_2 / F) / 8.0,
	                         1.0, S.STORE_E4M3)
	frac, beyond = e4m3_compare(np8(got["ffn_y"]), fy)
	assert frac < 5e-3 and beyond == 0.0, (frac, beyond)


def test_file_conventions_on_the_device(dev, tmp_path):
	"""A raw `.bin` file and a `.safetensors` file of the same codes give the same device tensor and the same kernel
	output; the i8 code -128 (NaN on the host side, block_utils.py:118-124) reaches the kernel unchanged."""
	rng = rng_for("files-bin")
	m, k, n = 256, 128, 256
	a = i8_codes(rng, (m, k))
	a[3, 5] = -128
	b = i8_codes(rng, (n, k))
	a.tofile(str(tmp_path / "a_i8.bin"))
	save_file({"a": torch.from_numpy(a)}, str(tmp_path / "a_i8.safetensors"))
	save_file({"b": torch.from_numpy(b)}, str(tmp_path / "b_i8.safetensors"))
	t_bin = TF.load_tensor_file(str(tmp_path / "a_i8.bin"), dev, (m, k))
	t_st = TF.load_tensor_file(str(tmp_path / "a_i8.safetensors"), dev)
	assert np.array_equal(t_bin.download(), a) and np.array_equal(t_st.download(), a)
	assert np.isnan(TF.real_values(t_st.download(), X.INT8)[3, 5])
	bt = TF.load_tensor_file(str(tmp_path / "b_i8.safetensors"), dev)
	kern = recipes.attn_q_kernel(dev, k, n)
	outs = []
	for t in (t_bin, t_st):
		c = X.Tensor(dev, (m, n), X.INT8)
		kern.launch(t, bt, c)
		outs.append(c.download())
	want = S.epilogue_scale(S.gemm_i32(a, b), 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(outs[0], want) and np.array_equal(outs[1], want)
	# a device tensor cannot be saved directly (src/tensor.rs:213-219): to_cpu first
	with pytest.raises(X.X17Error):
		t_st.save_safetensors_file(str(tmp_path / "direct_i8.safetensors"))
	cpu = t_st.to_cpu()
	cpu.save_safetensors_file(str(tmp_path / "round_i8.safetensors"))
	assert np.array_equal(load_file(str(tmp_path / "round_i8.safetensors"))["tensor"].numpy(), a)
	assert os.path.getsize(str(tmp_path / "a_i8.bin")) == m * k
