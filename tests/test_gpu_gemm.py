"""GPU parity of the 8-bit GEMM family (gemm_b8 / gemm_f8 and their four fused epilogues).

Every call goes Python -> flat C ABI of the operator layer -> C-ABI device shim -> HIP kernel.
The checker is the CPU oracle (oracle/x17_oracle.c).  Bars:
  * int32 accumulators, Scale and L2-norm outputs, and everything built with strict_math:
    bit-exact;
  * hardware-transcendental builds (strict_math=False): at most one output code apart, in a
    stated small fraction of elements;
  * f32-accumulated GEMMs (any e4m3 operand): the summation order inside the matrix cores is
    not the oracle's, so outputs may differ by one output code in a stated small fraction.
"""
import math

import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd import recipes
from oracle import strict as S
from tests.gpu_common import e4m3_bytes, e4m3_compare, i8_codes, rng_for

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


def _up(dev, arr, dtype):
	return X.Tensor.from_numpy(dev, arr, dtype)


SHAPES = [(256, 128, 256), (512, 1024, 512), (256, 2048, 1024)]     # (M, K, N_raw)


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_scale_epilogue_bit_exact(dev, m, k, n):
	rng = rng_for("scale", m, k, n)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	kern = recipes.attn_q_kernel(dev, k, n)
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
	got = c.download()
	want = S.epilogue_scale(S.gemm_i32(a, b), 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(got, want)
	assert kern.n_ops(_up(dev, a, X.INT8), _up(dev, b, X.INT8)) == 2.0 * m * k * n


def test_int32_accumulators_bit_exact(dev):
	"""Reads raw accumulators out through a Scale epilogue with scale 1: sparse +-1/0 operands keep
	every |acc| <= 127, so the int8 output IS the accumulator."""
	m, k, n = 256, 1024, 256
	rng = rng_for("acc")
	a = (rng.integers(-1, 2, (m, k)) * (rng.random((m, k)) < 0.05)).astype(np.int8)
	b = (rng.integers(-1, 2, (n, k)) * (rng.random((n, k)) < 0.5)).astype(np.int8)
	cfg = X.GemmConfig(X.GemmInputConfig(X.INT8, k, None, False), X.GemmInputConfig(X.INT8, k, n, True), X.INT8)
	kern = X.GemmKernel(dev, f"acc_probe-k{k}-n{n}", cfg, X.ScaleConfig(1.0, 1.0))
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
	acc = a.astype(np.int64) @ b.astype(np.int64).T
	assert np.abs(acc).max() <= 127 and np.abs(acc).max() >= 8
	assert np.array_equal(c.download().astype(np.int64), acc)
	# and the other extreme: saturated operands, |acc| up to K * 127 * 127, read through a small scale
	a2 = np.where(rng.random((m, k)) < 0.5, 127, -127).astype(np.int8)
	b2 = np.where(rng.random((n, k)) < 0.5, 127, -127).astype(np.int8)
	a2[:8] = 127
	b2[:8] = 127
	kern2 = X.GemmKernel(dev, f"acc_probe2-k{k}-n{n}", cfg, X.ScaleConfig(1.0 / (k * 127.0), 1.0))
	kern2.launch(_up(dev, a2, X.INT8), _up(dev, b2, X.INT8), c)
	want = S.epilogue_scale(S.gemm_i32(a2, b2), 1.0 / (k * 127.0), 1.0)
	assert want.max() == 127
	assert np.array_equal(c.download(), want)


@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("m,k", [(256, 512), (512, 2048)])
def test_l2norm_epilogue_bit_exact(dev, hd, m, k):
	n = 512
	rng = rng_for("l2", hd, m, k)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	kern = recipes.attn_kv_kernel(dev, k, n, hd)
	c = X.Tensor(dev, (m, n), X.INT8)
	rrms = X.Tensor(dev, (m, n // (2 * hd)), X.F32)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, rrms)
	want_c, want_r = S.epilogue_l2norm(S.gemm_i32(a, b), hd, recipes.L2_NORM_EPS, 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(c.download(), want_c)
	assert np.array_equal(rrms.download().view(np.uint32), want_r.view(np.uint32))


@pytest.mark.parametrize("hd", [64, 128])
def test_l2norm_epilogue_on_a_walk_of_more_tiles_than_workgroups(dev, hd):
	"""2048 tokens x 2048 raw columns = 512 output tiles over the 256 persistent workgroups: every workgroup writes two
	tiles with the next tile's loads and the rrms stores in flight; heads of 64 and 128 columns."""
	m, k, n = 2048, 256, 2048
	rng = rng_for("l2-walk", hd)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	kern = recipes.attn_kv_kernel(dev, k, n, hd)
	c = X.Tensor(dev, (m, n), X.INT8)
	rrms = X.Tensor(dev, (m, n // (2 * hd)), X.F32)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, rrms)
	want_c, want_r = S.epilogue_l2norm(S.gemm_i32(a, b), hd, recipes.L2_NORM_EPS, 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(c.download(), want_c)
	assert np.array_equal(rrms.download().view(np.uint32), want_r.view(np.uint32))


def _bf16_bits(x: np.ndarray) -> np.ndarray:
	u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
	return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.parametrize("hd", [32, 64, 128])
def test_learned_scale_q_writer_bit_exact(dev, hd):
	"""cuda/qkvg_fwd_i8.cuh:145-219: every head L2-normalised, then a bf16 scale per column."""
	m, k, n = 512, 512, 512
	rng = rng_for("qnorm", hd)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	dyn = _bf16_bits(0.25 + 1.5 * rng.random(n))
	kern = recipes.attn_q_norm_kernel(dev, k, n, hd, 0.0)
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, _up(dev, dyn, X.BF16))
	want = S.epilogue_qnorm(S.gemm_i32(a, b), hd, 0.0, 8.0, dyn)
	got = c.download()
	assert np.array_equal(got, want)
	assert len(np.unique(got)) > 50                       # (not a constant, not saturated)
	# the learned scales are column-wise: wrong scale vector, wrong answer
	assert not np.array_equal(S.epilogue_qnorm(S.gemm_i32(a, b), hd, 0.0, 8.0, np.roll(dyn, 1)), want)


def test_learned_scale_q_writer_with_the_base_writer_scale(dev):
	"""The old writer's base class was built with SCALE = 1 / sqrt(MODEL_DIM) (cuda/qkvg_fwd_i8.cuh:151-159) and is
	gone from the reference tree; the live scaled writer's f32 overload applies its SCALE (cuda/gemm_b8.cuh:307-324).
	That reading is one constant away: post_scale = 1 / sqrt(K), one more f32 multiply before the conversion."""
	m, k, n, hd = 512, 512, 512, 64
	rng = rng_for("qnorm-post")
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	dyn = _bf16_bits(8.0 + 8.0 * rng.random(n))                 # (large learned scales keep the codes off zero)
	post = 1.0 / math.sqrt(k)
	kern = recipes.attn_q_norm_kernel(dev, k, n, hd, 0.0, True, post)
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, _up(dev, dyn, X.BF16))
	want = S.epilogue_qnorm(S.gemm_i32(a, b), hd, 0.0, 8.0, dyn, post_scale=post)
	got = c.download()
	assert np.array_equal(got, want)
	assert len(np.unique(got)) > 20
	assert not np.array_equal(want, S.epilogue_qnorm(S.gemm_i32(a, b), hd, 0.0, 8.0, dyn))


def test_learned_scale_q_writer_with_eps_at_a_full_width(dev):
	"""The hook that survives in the live header adds EPS (cuda/gemm_b8.cuh:808); 1024 columns = four column tiles."""
	m, k, n, hd = 512, 2048, 1024, 128
	rng = rng_for("qnorm-eps")
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	a[7] = 0                                                   # an all-zero token row: sum of squares 0, rsq(eps)
	dyn = _bf16_bits(0.5 + rng.random(n))
	kern = recipes.attn_q_norm_kernel(dev, k, n, hd, recipes.L2_NORM_EPS)
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, _up(dev, dyn, X.BF16))
	want = S.epilogue_qnorm(S.gemm_i32(a, b), hd, recipes.L2_NORM_EPS, 8.0, dyn)
	assert np.array_equal(c.download(), want)
	assert not c.download()[7].any()


@pytest.mark.parametrize("hd", [32, 64, 128])
def test_fused_q_kv_projection_equals_the_two_kernels(dev, hd):
	"""One launch for src/main.rs:387-493's two: q, kv and rrms bit for bit those of the oracle (and so of the separate
	kernels)."""
	m, k, nq, nkv = 512, 512, 256, 512
	rng = rng_for("qkv", hd)
	x, wq, wkv = i8_codes(rng, (m, k)), i8_codes(rng, (nq, k)), i8_codes(rng, (nkv, k))
	kern = recipes.attn_qkv_kernel(dev, k, nq, nkv, hd)
	q, kv = X.Tensor(dev, (m, nq), X.INT8), X.Tensor(dev, (m, nkv), X.INT8)
	rrms = X.Tensor(dev, (m, nkv // (2 * hd)), X.F32)
	kern.launch_qkv(_up(dev, x, X.INT8), _up(dev, wq, X.INT8), _up(dev, wkv, X.INT8), q, kv, rrms)
	inp = 1.0 / math.sqrt(k) / 64.0
	want_q = S.epilogue_scale(S.gemm_i32(x, wq), inp, 8.0)
	want_kv, want_r = S.epilogue_l2norm(S.gemm_i32(x, wkv), hd, recipes.L2_NORM_EPS, inp, 8.0)
	assert np.array_equal(q.download(), want_q)
	assert np.array_equal(kv.download(), want_kv)
	assert np.array_equal(rrms.download().view(np.uint32), want_r.view(np.uint32))
	# shape checks of the launcher
	with pytest.raises(X.X17Error):
		kern.launch_qkv(_up(dev, x, X.INT8), _up(dev, wkv, X.INT8), _up(dev, wq, X.INT8), q, kv, rrms)
	with pytest.raises(X.X17Error):
		kern.launch(_up(dev, x, X.INT8), _up(dev, wq, X.INT8), q, rrms)


def test_shapes_of_the_reference_that_are_not_whole_tiles(dev):
	"""src/device/cuda/gemm.rs:605-614 accepts rows % 64 == 0 and raw columns % 128 == 0; the tile here is 256 x 256.
	320 token rows x 384 raw columns (one full tile and an overhanging one in each direction) through every writer,
	against the oracle over the whole output; below one tile and off the 64 / 128 grid are errors."""
	m, k, n = 320, 512, 384
	rng = rng_for("tails")
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	acc = S.gemm_i32(a, b)
	inp = 1.0 / math.sqrt(k) / 64.0
	ta, tb = _up(dev, a, X.INT8), _up(dev, b, X.INT8)
	c = X.Tensor(dev, (m, n), X.INT8)
	recipes.attn_q_kernel(dev, k, n).launch(ta, tb, c)
	assert np.array_equal(c.download(), S.epilogue_scale(acc, inp, 8.0))
	ch = X.Tensor(dev, (m, n // 2), X.E4M3)
	recipes.ffn_f_kernel(dev, k, n, True, X.E4M3).launch(ta, tb, ch)
	assert np.array_equal(ch.download(), S.epilogue_geglu(acc, inp, 1.0, S.STORE_E4M3))
	res = i8_codes(rng, (m, n // 2))
	recipes.attn_y_kernel(dev, n // 2, k, True).launch(ta, tb, ch, _up(dev, res, X.INT8))
	assert np.array_equal(ch.download(), S.epilogue_residual(acc, res, inp, 1.0, S.STORE_E4M3))
	for hd in (32, 64):
		rrms = X.Tensor(dev, (m, n // (2 * hd)), X.F32)
		recipes.attn_kv_kernel(dev, k, n, hd).launch(ta, tb, c, rrms)
		want_c, want_r = S.epilogue_l2norm(acc, hd, recipes.L2_NORM_EPS, inp, 8.0)
		assert np.array_equal(c.download(), want_c)
		assert np.array_equal(rrms.download().view(np.uint32), want_r.view(np.uint32))
	# e4m3 activations x int8 weights (the four-wave form)
	ae = e4m3_bytes(rng, (m, k))
	recipes.mixed_gemm_kernel(dev, k, n, False).launch(_up(dev, ae, X.E4M3), tb, c)
	want = S.epilogue_scale(S.gemm_f32_seq(ae, True, b, False), 1.0 / math.sqrt(k) / 8.0, 8.0)
	assert np.abs(c.download().astype(np.int32) - want.astype(np.int32)).max() <= 1
	# what the reference rejects is rejected here too, and so is less than one tile
	kern = recipes.attn_q_kernel(dev, k, n)
	for rows in (288, 192):
		with pytest.raises(X.X17Error, match="divisible by \\[64, 128\\]"):
			kern.launch(_up(dev, a[:rows], X.INT8), tb, X.Tensor(dev, (rows, n), X.INT8))
	with pytest.raises(X.X17Error, match="multiple of 128"):
		recipes.attn_q_kernel(dev, k, 320)
	with pytest.raises(X.X17Error, match="at least one tile"):
		recipes.attn_q_kernel(dev, k, 128)


def test_more_writers_on_shapes_that_are_not_whole_tiles(dev):
	"""The remaining writers off the 256-grid, 320 token rows (a full tile and an overhanging one): the dequantising
	writer (row and column scale indexing) with and without GeGLU and the learned-scale Q writer on 384 raw columns,
	the fused q + kv kernel with 256 q columns + 384 kv columns (the moved-back column tile lies wholly on the kv
	side), and head_dim 128 -- kv alone and fused -- with overhanging rows."""
	m, k, n = 320, 512, 384
	rng = rng_for("tails-2")
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	acc = S.gemm_i32(a, b)
	inp = 1.0 / math.sqrt(k) / 64.0
	ta, tb = _up(dev, a, X.INT8), _up(dev, b, X.INT8)
	rs = (0.01 + 0.01 * rng.random(m)).astype(np.float32)
	cs = (0.01 + 0.01 * rng.random(n)).astype(np.float32)
	for geglu in (False, True):
		c = X.Tensor(dev, (m, n // 2 if geglu else n), X.BF16)
		recipes.dequant_gemm_kernel(dev, k, n, X.INT8, X.INT8, geglu, True).launch_dequant(ta, tb, c, _up(dev, rs, X.F32), _up(dev, cs, X.F32))
		assert np.array_equal(c.download(), S.epilogue_dequant(acc, rs, cs, geglu)), geglu
	dyn = _bf16_bits(0.25 + 1.5 * rng.random(n))
	c = X.Tensor(dev, (m, n), X.INT8)
	recipes.attn_q_norm_kernel(dev, k, n, 64, 0.0).launch(ta, tb, c, _up(dev, dyn, X.BF16))
	assert np.array_equal(c.download(), S.epilogue_qnorm(acc, 64, 0.0, 8.0, dyn))
	# fused q + kv: 256 + 384 raw columns, head_dim 64; then 256 + 512 with head_dim 128 (rows off the grid only)
	for nq, nkv, hd in ((256, 384, 64), (256, 512, 128)):
		wq, wkv = i8_codes(rng, (nq, k)), i8_codes(rng, (nkv, k))
		q, kv = X.Tensor(dev, (m, nq), X.INT8), X.Tensor(dev, (m, nkv), X.INT8)
		rrms = X.Tensor(dev, (m, nkv // (2 * hd)), X.F32)
		recipes.attn_qkv_kernel(dev, k, nq, nkv, hd).launch_qkv(ta, _up(dev, wq, X.INT8), _up(dev, wkv, X.INT8), q, kv, rrms)
		want_kv, want_r = S.epilogue_l2norm(S.gemm_i32(a, wkv), hd, recipes.L2_NORM_EPS, inp, 8.0)
		assert np.array_equal(q.download(), S.epilogue_scale(S.gemm_i32(a, wq), inp, 8.0)), (nq, nkv, hd)
		assert np.array_equal(kv.download(), want_kv), (nq, nkv, hd)
		assert np.array_equal(rrms.download().view(np.uint32), want_r.view(np.uint32)), (nq, nkv, hd)
		if hd == 128:
			kv2, rr2 = X.Tensor(dev, (m, nkv), X.INT8), X.Tensor(dev, (m, nkv // (2 * hd)), X.F32)
			recipes.attn_kv_kernel(dev, k, nkv, hd).launch(ta, _up(dev, wkv, X.INT8), kv2, rr2)
			assert np.array_equal(kv2.download(), want_kv)
			assert np.array_equal(rr2.download().view(np.uint32), want_r.view(np.uint32))


@pytest.mark.parametrize("store", [X.E4M3, X.INT8])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_geglu_epilogue(dev, m, k, n, store):
	rng = rng_for("geglu", m, k, n, store)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	acc = S.gemm_i32(a, b)
	inp = 1.0 / math.sqrt(k) / 64.0
	out_scale = 1.0 if store == X.E4M3 else 8.0
	want = S.epilogue_geglu(acc, inp, out_scale, S.STORE_E4M3 if store == X.E4M3 else S.STORE_I8)
	for strict in (True, False):
		kern = recipes.ffn_f_kernel(dev, k, n, strict, store)
		c = X.Tensor(dev, (m, n // 2), store)
		kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
		got = c.download()
		if strict:
			assert np.array_equal(got, want)
		elif store == X.E4M3:
			neq, beyond = e4m3_compare(got, want)
			assert neq < 2e-3 and beyond == 0.0, (neq, beyond)
		else:
			d = np.abs(got.astype(np.int32) - want.astype(np.int32))
			assert d.max() <= 1 and np.mean(d > 0) < 2e-3


@pytest.mark.parametrize("store", [X.E4M3, X.INT8])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_residual_epilogue(dev, m, k, n, store):
	rng = rng_for("residual", m, k, n, store)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	r = i8_codes(rng, (m, n // 2))
	acc = S.gemm_i32(a, b)
	inp = 1.0 / math.sqrt(k) / 64.0
	want = S.epilogue_residual(acc, r, inp, 1.0, S.STORE_E4M3 if store == X.E4M3 else S.STORE_I8)
	for strict in (True, False):
		kern = recipes.attn_y_kernel(dev, n // 2, k, strict, store)
		c = X.Tensor(dev, (m, n // 2), store)
		kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, _up(dev, r, X.INT8))
		got = c.download()
		if strict:
			assert np.array_equal(got, want)
		elif store == X.E4M3:
			neq, beyond = e4m3_compare(got, want)
			assert neq < 2e-3 and beyond == 0.0, (neq, beyond)
		else:
			d = np.abs(got.astype(np.int32) - want.astype(np.int32))
			assert d.max() <= 1 and np.mean(d > 0) < 2e-3


@pytest.mark.parametrize("m,k,n", [(256, 512, 256), (512, 2048, 512)])
def test_mixed_e4m3_i8_residual(dev, m, k, n):
	"""ffn_y_fwd_f8: e4m3 activations x int8 weights on the bf16 matrix cores, f32 accumulate."""
	rng = rng_for("mixed", m, k, n)
	a = e4m3_bytes(rng, (m, k), 0.6)
	b = i8_codes(rng, (n, k))
	r = i8_codes(rng, (m, n // 2))
	inp = math.sqrt(recipes.GELU_VAR_FIX_2 / k) / 8.0
	want = S.epilogue_residual(S.gemm_f32_seq(a, True, b, False), r, inp, 1.0, S.STORE_E4M3)
	kern = recipes.ffn_y_kernel(dev, n // 2, k, True)
	c = X.Tensor(dev, (m, n // 2), X.E4M3)
	kern.launch(_up(dev, a, X.E4M3), _up(dev, b, X.INT8), c, _up(dev, r, X.INT8))
	neq, beyond = e4m3_compare(c.download(), want)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)


@pytest.mark.parametrize("geglu", [False, True])
def test_mixed_e4m3_i8_scale_and_geglu(dev, geglu):
	"""The e4m3 x int8 operand mix under the Scale and GeGLU writers (K of eight steps: the paced rounds, fully unrolled)."""
	m, k, n = 512, 1024, 512
	rng = rng_for("mixed-writers", geglu)
	a = e4m3_bytes(rng, (m, k), 0.6)
	b = i8_codes(rng, (n, k))
	acc = S.gemm_f32_seq(a, True, b, False)
	inp = 1.0 / math.sqrt(k) / 8.0
	kern = recipes.mixed_gemm_kernel(dev, k, n, geglu, True)
	if geglu:
		want = S.epilogue_geglu(acc, inp, 1.0, S.STORE_E4M3)
		c = X.Tensor(dev, (m, n // 2), X.E4M3)
		kern.launch(_up(dev, a, X.E4M3), _up(dev, b, X.INT8), c)
		neq, beyond = e4m3_compare(c.download(), want)
		assert neq < 5e-3 and beyond == 0.0, (neq, beyond)
	else:
		want = S.epilogue_scale(acc, inp, 8.0)
		c = X.Tensor(dev, (m, n), X.INT8)
		kern.launch(_up(dev, a, X.E4M3), _up(dev, b, X.INT8), c)
		d = np.abs(c.download().astype(np.int32) - want.astype(np.int32))
		assert d.max() <= 1 and np.mean(d > 0) < 5e-3, (d.max(), np.mean(d > 0))


@pytest.mark.parametrize("m,k,n", [(256, 512, 256), (512, 4096, 512)])
def test_fp8_geglu(dev, m, k, n):
	"""All-fp8 ffn_f: e4m3 x e4m3 on the fp8 matrix cores, f32 accumulate, GeGLU -> e4m3."""
	rng = rng_for("fp8", m, k, n)
	a = e4m3_bytes(rng, (m, k))
	b = e4m3_bytes(rng, (n, k))
	want = S.epilogue_geglu(S.gemm_f32_seq(a, True, b, True), 1.0 / math.sqrt(k), 1.0, S.STORE_E4M3)
	kern = recipes.ffn_f_f8_kernel(dev, k, n, True)
	c = X.Tensor(dev, (m, n // 2), X.E4M3)
	kern.launch(_up(dev, a, X.E4M3), _up(dev, b, X.E4M3), c)
	neq, beyond = e4m3_compare(c.download(), want)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)


def test_e4m3_store_keeps_the_dialect_over_the_whole_range(dev):
	"""GeGLU outputs from far below the smallest e4m3 magnitude to far above 448.  The hardware-transcendental build
	stores through the gfx950 conversion instruction: it must still produce the reference's dialect (no subnormal
	codes, no negative zero, no NaN code, saturation at +-448) and sit within one grid step of the strict build,
	which equals the oracle bit for bit."""
	m, k, n = 256, 128, 256
	rng = rng_for("e4m3-range")
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	want = S.epilogue_geglu(S.gemm_i32(a, b), 1.0 / 32.0, 1.0, S.STORE_E4M3)
	assert np.mean((want & 0x7F) == 0x7E) > 0.01 and np.mean(want == 0) > 0.05
	cfg = X.GemmConfig(X.GemmInputConfig(X.INT8, k, None, False), X.GemmInputConfig(X.INT8, k, n, True), X.E4M3)
	got = {}
	for mode, strict in (("strict", True), ("fast", False)):
		kern = X.GemmKernel(dev, f"e4m3_range-{mode}", cfg, X.GeGluConfig(1.0 / 32.0, 1.0), strict)
		c = X.Tensor(dev, (m, n // 2), X.E4M3)
		kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
		got[mode] = c.download()
	assert np.array_equal(got["strict"], want)
	fast = got["fast"]
	assert not np.any((fast & 0x7F) == 0x7F)                                   # NaN code
	assert not np.any(((fast & 0x78) == 0) & (fast != 0))                      # subnormal codes and -0
	neq, beyond = e4m3_compare(fast, want)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)
	sat = (want & 0x7F) == 0x7E
	assert np.mean(fast[sat] != want[sat]) < 5e-3


def test_more_tiles_than_workgroups_with_the_shortest_ring_of_three(dev):
	"""K = 384 is three K steps: the first K the three-deep token ring is built for, where every request of a tile's
	last two steps already belongs to the workgroup's NEXT tile.  260 tiles on at most 256 persistent workgroups:
	four of them walk two tiles, the others end after one (their last requests go to a ring position nobody reads)."""
	m, k, n = 256 * 65, 384, 1024
	rng = rng_for("ring3", m, k, n)
	a, b = i8_codes(rng, (m, k)), i8_codes(rng, (n, k))
	kern = recipes.attn_q_kernel(dev, k, n)
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
	want = S.epilogue_scale(S.gemm_i32(a, b), 1.0 / math.sqrt(k) / 64.0, 8.0)
	assert np.array_equal(c.download(), want)
	# the same walk in the four-wave e4m3 form (130 x 2 tiles)
	m, n = 256 * 130, 512
	a8, b8 = e4m3_bytes(rng, (m, k)), e4m3_bytes(rng, (n, k))
	want = S.epilogue_geglu(S.gemm_f32_seq(a8, True, b8, True), 1.0 / math.sqrt(k), 1.0, S.STORE_E4M3)
	kern = recipes.ffn_f_f8_kernel(dev, k, n, True)
	c = X.Tensor(dev, (m, n // 2), X.E4M3)
	kern.launch(_up(dev, a8, X.E4M3), _up(dev, b8, X.E4M3), c)
	neq, beyond = e4m3_compare(c.download(), want)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)


def _absmax_quantize(x, axis):
	"""Symmetric int8 with scale = absmax / 127 along `axis` (f32 arithmetic)."""
	x = x.astype(np.float32)
	scale = (np.abs(x).max(axis=axis, keepdims=True) / np.float32(127.0)).astype(np.float32)
	codes = np.clip(np.rint(x / scale), -127, 127).astype(np.int8)
	return codes, scale.reshape(-1)


@pytest.mark.parametrize("geglu", [False, True])
def test_dequant_epilogue_per_row_per_channel_scales(dev, geglu):
	"""Run-time per-token x per-output-channel scales, bf16 out (no counterpart in the reference: defined by
	the oracle's two-multiply order).  Strict build bit-exact; speed build within bf16 ulps; and the
	dequantised product close to the float matmul it approximates."""
	m, k, n = 512, 1024, 512
	rng = rng_for("dequant", geglu)
	xf = rng.standard_normal((m, k), dtype=np.float32)
	wf = rng.standard_normal((n, k), dtype=np.float32) / np.float32(math.sqrt(k))
	a, rs = _absmax_quantize(xf, 1)
	b, cs = _absmax_quantize(wf, 1)
	acc = S.gemm_i32(a, b)
	want = S.epilogue_dequant(acc, rs, cs, geglu)
	outs = {}
	for strict in (True, False):
		kern = recipes.dequant_gemm_kernel(dev, k, n, X.INT8, X.INT8, geglu, strict)
		c = X.Tensor(dev, (m, n // 2 if geglu else n), X.BF16)
		kern.launch_dequant(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c, _up(dev, rs, X.F32), _up(dev, cs, X.F32))
		outs[strict] = c.download()
	assert np.array_equal(outs[True], want)
	d = np.abs(outs[False].astype(np.int32) - want.astype(np.int32))
	# one bf16 ulp, except where 1 + tanh cancels: there the two gelu formulations differ by several ulps of a
	# tiny value, bounded absolutely
	assert np.mean(d > 1) < 1e-3 and np.mean(d > 0) < 0.02, (d.max(), np.mean(d > 1), np.mean(d > 0))
	fast_f = (outs[False].astype(np.uint32) << 16).view(np.float32)
	want_f = (want.astype(np.uint32) << 16).view(np.float32)
	assert np.allclose(fast_f, want_f, rtol=2.0 ** -7, atol=float(np.abs(want_f).max()) * 1e-5)
	# what it approximates: x @ w^T (then GeGLU) in float64; int8 quantisation noise only
	got_f = (outs[True].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	ref = xf.astype(np.float64) @ wf.astype(np.float64).T
	if geglu:
		g, l = ref[:, 0::2], ref[:, 1::2]
		ref = 0.5 * g * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g ** 3))) * l
	rel_l2 = np.linalg.norm(got_f - ref) / np.linalg.norm(ref)
	assert rel_l2 < 0.03, rel_l2


def test_dequant_epilogue_fp8_per_tensor_scales(dev):
	"""e4m3 x e4m3 with per-tensor scales (constant scale vectors), f32 accumulate, bf16 out."""
	m, k, n = 256, 512, 256
	rng = rng_for("dequant-f8")
	a, b = e4m3_bytes(rng, (m, k)), e4m3_bytes(rng, (n, k))
	rs = np.full(m, 0.75, np.float32)
	cs = np.full(n, 1.0 / math.sqrt(k), np.float32)
	want = S.epilogue_dequant(S.gemm_f32_seq(a, True, b, True), rs, cs, False)
	kern = recipes.dequant_gemm_kernel(dev, k, n, X.E4M3, X.E4M3, False, True)
	c = X.Tensor(dev, (m, n), X.BF16)
	kern.launch_dequant(_up(dev, a, X.E4M3), _up(dev, b, X.E4M3), c, _up(dev, rs, X.F32), _up(dev, cs, X.F32))
	got_bits = c.download()
	got = (got_bits.astype(np.uint32) << 16).view(np.float32)
	ref = (want.astype(np.uint32) << 16).view(np.float32)
	# the matrix cores add the f32 products in another order than the oracle: one bf16 ulp, plus an absolute
	# slack of 1e-4 of the largest output for sums that cancel
	assert np.allclose(got, ref, rtol=2.0 ** -7, atol=float(np.abs(ref).max()) * 1e-4)
	assert np.mean(got_bits != want) < 0.05
	with pytest.raises(X.X17Error, match="row-scale and a column-scale"):
		kern.launch(_up(dev, a, X.E4M3), _up(dev, b, X.E4M3), c)


def test_launch_rejects_bad_arguments(dev):
	"""Shape / dtype / device checks of the launcher (src/device/cuda/tensor_check.rs, gemm.rs:591-616)."""
	k, n = 128, 256
	kern = recipes.attn_q_kernel(dev, k, n)
	a = X.Tensor(dev, (256, k), X.INT8)
	b = X.Tensor(dev, (n, k), X.INT8)
	c = X.Tensor(dev, (256, n), X.INT8)
	with pytest.raises(X.X17Error, match="has dtype e4m3, but should have i8"):
		kern.launch(X.Tensor(dev, (256, k), X.E4M3), b, c)
	with pytest.raises(X.X17Error, match="columns, but should have 128"):
		kern.launch(X.Tensor(dev, (256, 2 * k), X.INT8), b, c)
	with pytest.raises(X.X17Error, match="must be 2D"):
		kern.launch(X.Tensor(dev, (256, k, 1), X.INT8), b, c)
	with pytest.raises(X.X17Error, match="hold at least one 256 x 256 tile"):
		kern.launch(X.Tensor(dev, (64, k), X.INT8), b, X.Tensor(dev, (64, n), X.INT8))
	with pytest.raises(X.X17Error, match="hold at least one 256 x 256 tile"):
		kern.launch(X.Tensor(dev, (192, k), X.INT8), b, X.Tensor(dev, (192, n), X.INT8))     # divisible by 64, below a tile
	# an overhanging tile recomputes its neighbour's rows: an in-place gated residual would read what another
	# workgroup has already overwritten
	kr = recipes.attn_y_kernel(dev, n // 2, k, True, X.INT8)
	xr = X.Tensor(dev, (256, n // 2), X.INT8)
	with pytest.raises(X.X17Error, match="must not share memory with the residual"):
		kr.launch(a, b, xr, xr)
	# the fused q + kv entry point on a kernel that is not one
	with pytest.raises(X.X17Error, match="is not a fused q . kv kernel"):
		kern.launch_qkv(a, b, b, c, c, X.Tensor(dev, (256, 1), X.F32))
	with pytest.raises(X.X17Error, match="is not on device"):
		kern.launch(X.Tensor(None, (256, k), X.INT8), b, c)
	kern.launch(a, b, c)
	dev.synchronize()
