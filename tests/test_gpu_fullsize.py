"""GPU parity at the full benchmark sizes.

The CPU oracle cannot redo these workloads whole in test time, so each check uses a property that does
not depend on the size: a GEMM output row depends only on its own token row and the weights, an attention
head only on its own columns, a decoded (sequence, head) only on its own cache slice.  The kernels run at
full size (persistent grid, every tile / query block / workgroup exercised); a sample of rows / heads /
sequences is then recomputed by the oracle and compared to the strict builds bit for bit.
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


def _sample_rows(rng, m, count):
	# first and last rows, the rows around every 256-row tile edge of the first tiles, and random ones
	fixed = [0, 1, 255, 256, 257, m - 257, m - 256, m - 1]
	return np.unique(np.concatenate((np.array(fixed), rng.integers(0, m, count - len(fixed)))))


def test_config2_ffn_pair_sampled_rows(dev):
	"""benchmark config 2: tokens 8192, d_model 2048, d_ff 8192 -- ffn_f (GeGLU -> FixedI8) and the int8
	ffn_y (gated residual -> e4m3), strict builds, 96 sampled token rows of each against the oracle."""
	m, d, f = 8192, 2048, 8192
	rng = rng_for("full-config2")
	x, w1, w2 = i8_codes(rng, (m, d)), i8_codes(rng, (2 * f, d)), i8_codes(rng, (2 * d, f))
	k1 = recipes.ffn_f_kernel(dev, d, 2 * f, True, X.INT8)
	k2 = recipes.ffn_y_kernel(dev, d, f, True, X.INT8, X.INT8)
	xt = _up(dev, x, X.INT8)
	ft = X.Tensor(dev, (m, f), X.INT8)
	yt = X.Tensor(dev, (m, d), X.E4M3)
	k1.launch(xt, _up(dev, w1, X.INT8), ft)
	k2.launch(ft, _up(dev, w2, X.INT8), yt, xt)
	got_f, got_y = ft.download(), yt.download()
	rows = _sample_rows(rng, m, 96)
	want_f = S.epilogue_geglu(S.gemm_i32(x[rows], w1), 1.0 / math.sqrt(d) / 64.0, 8.0, S.STORE_I8)
	assert np.array_equal(got_f[rows], want_f)
	inp_y = math.sqrt(recipes.GELU_VAR_FIX_2 / f) / 64.0
	want_y = S.epilogue_residual(S.gemm_i32(got_f[rows], w2), x[rows], inp_y, 1.0, S.STORE_E4M3)
	assert np.array_equal(got_y[rows], want_y)
	# every tile wrote something plausible: no output row is left at the allocator's fill
	assert np.count_nonzero(np.abs(got_f.astype(np.int32)).sum(axis=1) == 0) == 0


def test_config3_fp8_ffn_pair_sampled_rows(dev):
	"""benchmark config 3: tokens 16384, d_model 4096, d_ff 16384, e4m3 x e4m3 with f32 accumulation (four waves of
	128 x 128 per workgroup, eight and four tiles per workgroup): ffn_f (GeGLU -> e4m3) and ffn_y (gated residual ->
	e4m3), strict builds, 48 sampled token rows of each against the oracle.  The matrix cores add the products of a
	K slice in their own order, the oracle one by one: outputs may sit one e4m3 step apart in under 0.5 % of the
	elements and never further."""
	m, d, f = 16384, 4096, 16384
	rng = rng_for("full-config3")
	x, w1, w2 = e4m3_bytes(rng, (m, d)), e4m3_bytes(rng, (2 * f, d)), e4m3_bytes(rng, (2 * d, f))
	res = i8_codes(rng, (m, d))
	k1 = recipes.ffn_f_f8_kernel(dev, d, 2 * f, True)
	k2 = recipes.ffn_y_kernel(dev, d, f, True, X.E4M3, X.E4M3)
	ft = X.Tensor(dev, (m, f), X.E4M3)
	yt = X.Tensor(dev, (m, d), X.E4M3)
	k1.launch(_up(dev, x, X.E4M3), _up(dev, w1, X.E4M3), ft)
	k2.launch(ft, _up(dev, w2, X.E4M3), yt, _up(dev, res, X.INT8))
	got_f, got_y = ft.download(), yt.download()
	rows = _sample_rows(rng, m, 48)
	want_f = S.epilogue_geglu(S.gemm_f32_seq(x[rows], True, w1, True), 1.0 / math.sqrt(d), 1.0, S.STORE_E4M3)
	neq, beyond = e4m3_compare(got_f[rows], want_f)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)
	inp_y = math.sqrt(recipes.GELU_VAR_FIX_2 / f)
	want_y = S.epilogue_residual(S.gemm_f32_seq(got_f[rows], True, w2, True), res[rows], inp_y, 1.0, S.STORE_E4M3)
	neq, beyond = e4m3_compare(got_y[rows], want_y)
	assert neq < 5e-3 and beyond == 0.0, (neq, beyond)
	# every tile wrote: no output row of f is all zero bytes
	assert np.count_nonzero((got_f != 0).sum(axis=1) == 0) == 0


def test_repeated_launches_give_the_same_bytes(dev):
	"""The LDS rings are recycled behind one barrier per K step and the tile requests run ahead across tile
	boundaries: an ordering mistake there would show as output that depends on timing.  Each arithmetic at a size
	where every workgroup walks eight tiles, launched eight times back to back: every output equals the first."""
	rng = rng_for("repeat")
	m = 8192
	cases = (
		("int8", recipes.ffn_f_kernel(dev, 2048, 16384, False, X.INT8), i8_codes(rng, (m, 2048)), X.INT8,
		 i8_codes(rng, (16384, 2048)), X.INT8, (m, 8192), X.INT8, None),
		("e4m3", recipes.ffn_f_f8_kernel(dev, 4096, 32768, False), e4m3_bytes(rng, (m, 4096)), X.E4M3,
		 e4m3_bytes(rng, (32768, 4096)), X.E4M3, (m, 16384), X.E4M3, None),
		("e4m3 x int8", recipes.ffn_y_kernel(dev, 2048, 8192, False), e4m3_bytes(rng, (m, 8192)), X.E4M3,
		 i8_codes(rng, (4096, 8192)), X.INT8, (m, 2048), X.E4M3, i8_codes(rng, (m, 2048))),
	)
	for name, kern, a, a_dt, b, b_dt, out_shape, out_dt, res in cases:
		at, bt = _up(dev, a, a_dt), _up(dev, b, b_dt)
		rt = None if res is None else _up(dev, res, X.INT8)
		outs = [X.Tensor(dev, out_shape, out_dt) for _ in range(8)]
		for o in outs:
			if rt is None:
				kern.launch(at, bt, o)
			else:
				kern.launch(at, bt, o, rt)
		first = outs[0].download()
		assert np.count_nonzero(first) > first.size // 2, name
		for i, o in enumerate(outs[1:], 1):
			assert np.array_equal(o.download(), first), (name, i)


def test_config2_literal_per_token_per_channel_scales(dev):
	"""benchmark config 2 as worded: x ~ N(0,1) per-token int8 (absmax / 127), W1 [2048 x 8192 (x2 gated)] and
	W2 [8192 x 2048] ~ N(0, 1/sqrt(fan_in)) per-output-channel int8, int32 accumulate, fused dequantisation +
	GeGLU, bf16 out; the bf16 activations are re-quantised per token for the second GEMM.  Sampled rows
	against the oracle, bit for bit, and the whole against the float64 computation it approximates."""
	m, d, f = 8192, 2048, 8192
	rng = rng_for("full-config2-literal")

	def quant(x):
		scale = (np.abs(x).max(axis=1, keepdims=True) / np.float32(127.0)).astype(np.float32)
		return np.clip(np.rint(x / scale), -127, 127).astype(np.int8), scale.reshape(-1)

	xf = rng.standard_normal((m, d), dtype=np.float32)
	w1f = rng.standard_normal((2 * f, d), dtype=np.float32) / np.float32(math.sqrt(d))
	w2f = rng.standard_normal((d, f), dtype=np.float32) / np.float32(math.sqrt(f))
	x, xs = quant(xf)
	w1, w1s = quant(w1f)
	w2, w2s = quant(w2f)
	k1 = recipes.dequant_gemm_kernel(dev, d, 2 * f, X.INT8, X.INT8, True, True)
	k2 = recipes.dequant_gemm_kernel(dev, f, d, X.INT8, X.INT8, False, True)
	h_t = X.Tensor(dev, (m, f), X.BF16)
	k1.launch_dequant(_up(dev, x, X.INT8), _up(dev, w1, X.INT8), h_t, _up(dev, xs, X.F32), _up(dev, w1s, X.F32))
	h_bits = h_t.download()
	hf = (h_bits.astype(np.uint32) << 16).view(np.float32)
	h, hs = quant(hf)                                       # host-side requantisation between the two GEMMs
	y_t = X.Tensor(dev, (m, d), X.BF16)
	k2.launch_dequant(_up(dev, h, X.INT8), _up(dev, w2, X.INT8), y_t, _up(dev, hs, X.F32), _up(dev, w2s, X.F32))
	y_bits = y_t.download()
	rows = _sample_rows(rng, m, 64)
	assert np.array_equal(h_bits[rows], S.epilogue_dequant(S.gemm_i32(x[rows], w1), xs[rows], w1s, True))
	assert np.array_equal(y_bits[rows], S.epilogue_dequant(S.gemm_i32(h[rows], w2), hs[rows], w2s, False))
	# dequantised outputs against the float computation on a row sample: relative L2 and max-abs error
	g = xf[rows].astype(np.float64) @ w1f.astype(np.float64).T
	gate, lin = g[:, 0::2], g[:, 1::2]
	h_ref = 0.5 * gate * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (gate + 0.044715 * gate ** 3))) * lin
	y_ref = h_ref @ w2f.astype(np.float64).T
	y_got = (y_bits[rows].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	rel_l2 = np.linalg.norm(y_got - y_ref) / np.linalg.norm(y_ref)
	assert rel_l2 < 0.05 and np.abs(y_got - y_ref).max() < 0.25, (rel_l2, np.abs(y_got - y_ref).max())


def test_config2_checksum_of_checksums(dev):
	"""Column sums of an int8 GEMM are linear in the token rows: sum_m C[m, n] = (sum_m A[m, :]) . B[n, :].
	With +-1/0 operands sparse enough that no accumulator leaves the FixedI8 range, a scale-1 epilogue
	returns the accumulators themselves, and the whole 8192 x 16384 output is checked through one vector."""
	m, k, n = 8192, 2048, 16384
	rng = rng_for("full-checksum")
	a = (rng.integers(-1, 2, (m, k)) * (rng.random((m, k)) < 0.02)).astype(np.int8)
	b = (rng.integers(-1, 2, (n, k)) * (rng.random((n, k)) < 0.3)).astype(np.int8)
	cfg = X.GemmConfig(X.GemmInputConfig(X.INT8, k, None, False), X.GemmInputConfig(X.INT8, k, n, True), X.INT8)
	kern = X.GemmKernel(dev, f"acc_probe-k{k}-n{n}", cfg, X.ScaleConfig(1.0, 1.0))
	c = X.Tensor(dev, (m, n), X.INT8)
	kern.launch(_up(dev, a, X.INT8), _up(dev, b, X.INT8), c)
	got = c.download().astype(np.int64)
	assert np.abs(got).max() < 127                      # nothing saturated, so got IS the accumulator
	col = a.astype(np.int64).sum(axis=0)
	assert np.array_equal(got.sum(axis=0), b.astype(np.int64) @ col)
	row = b.astype(np.int64).sum(axis=0)
	assert np.array_equal(got.sum(axis=1), a.astype(np.int64) @ row)


def _attn_inputs(rng, rows, h, hd):
	q = i8_codes(rng, (rows, h * hd))
	k = rng.standard_normal((rows, h, hd), dtype=np.float32)
	k /= np.sqrt((k * k).mean(-1, keepdims=True))
	v = rng.standard_normal((rows, h, hd), dtype=np.float32) * 1.3
	kv = S.f32_to_fixedi8((np.concatenate((k, v), axis=2).reshape(rows, 2 * h * hd) * 8).astype(np.float32))
	sk = rng.standard_normal((h, hd))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	return q, kv, S.f32_to_fixedi8((sk * 8).astype(np.float32)), i8_codes(rng, (h, hd), 1.3), (0.5 + rng.random(h)).astype(np.float32)


def _head_columns(arr, heads, width):
	return np.ascontiguousarray(np.concatenate([arr[:, h * width:(h + 1) * width] for h in heads], axis=1))


def test_config4_attention_sampled_heads(dev):
	"""benchmark config 4 attention: 4 sequences x 8192 tokens, 16 heads x 128, window 512.  Heads are
	independent, so three heads of two of the sequences are recomputed by the oracle (all 8192 queries)."""
	t, b, h, hd, w = 8192, 4, 16, 128, 512
	rng = rng_for("full-config4-attn")
	q, kv, sk, sv, temp = _attn_inputs(rng, t * b, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, True)
	out = X.Tensor(dev, q.shape, X.INT8)
	l = X.Tensor(dev, (h, t * b), X.F32)
	kern.launch(_up(dev, q, X.INT8), _up(dev, kv, X.INT8), _up(dev, sk, X.INT8), _up(dev, sv, X.INT8),
	            _up(dev, temp, X.F32), out, l, w, b)
	got, got_l = out.download(), l.download()
	heads = [0, 7, 15]
	for seq in (0, 3):
		rows = slice(seq * t, (seq + 1) * t)
		want, want_l = S.attn_fwd_i8(_head_columns(q[rows], heads, hd), _head_columns(kv[rows], heads, 2 * hd),
		                             sk[heads], sv[heads], temp[heads], len(heads), hd, w)
		assert np.array_equal(_head_columns(got[rows], heads, hd), want)
		assert np.array_equal(got_l[heads][:, rows].view(np.uint32), want_l.view(np.uint32))


def test_config5_prefill_sampled_heads(dev):
	"""benchmark config 5 prefill: one sequence of 65536 tokens, 32 heads x 128, window 4096; two heads
	recomputed by the oracle.  Also the speed build against the strict one over the whole output."""
	t, h, hd, w = 65536, 32, 128, 4096
	rng = rng_for("full-config5-attn")
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	qt, kvt = _up(dev, q, X.INT8), _up(dev, kv, X.INT8)
	skt, svt, tt = _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32)
	out = X.Tensor(dev, q.shape, X.INT8)
	l = X.Tensor(dev, (h, t), X.F32)
	recipes.attn_kernel(dev, h, hd, True).launch(qt, kvt, skt, svt, tt, out, l, w, 1)
	got, got_l = out.download(), l.download()
	heads = [3, 31]
	want, want_l = S.attn_fwd_i8(_head_columns(q, heads, hd), _head_columns(kv, heads, 2 * hd),
	                             sk[heads], sv[heads], temp[heads], len(heads), hd, w)
	assert np.array_equal(_head_columns(got, heads, hd), want)
	assert np.array_equal(got_l[heads].view(np.uint32), want_l.view(np.uint32))
	out_fast = X.Tensor(dev, q.shape, X.INT8)
	recipes.attn_kernel(dev, h, hd, False).launch(qt, kvt, skt, svt, tt, out_fast, None, w, 1)
	d = np.abs(out_fast.download().astype(np.int32) - got.astype(np.int32))
	assert d.max() <= 1 and np.mean(d > 0) < 0.02, (d.max(), np.mean(d > 0))


def test_config5_decode_sampled_sequences(dev):
	"""benchmark config 5 decode: 64 sequences against 4096 cached positions, 32 heads x 128.  Ragged
	lengths (0, 1, 15, 16, 17, ..., 4096); four heads of every sequence recomputed by the oracle."""
	s, cap, h, hd, w = 64, 4096, 32, 128, 4096
	rng = rng_for("full-config5-decode")
	q, _, sk, sv, temp = _attn_inputs(rng, s, h, hd)
	cache = np.empty((s, cap, 2 * h * hd), np.int8)
	for i in range(s):
		cache[i] = i8_codes(rng, (cap, 2 * h * hd))
	lens = rng.integers(1, cap + 1, s).astype(np.uint32)
	lens[:8] = [0, 1, 15, 16, 17, 4095, 4096, 2048]
	# flat score distributions for some sequences: nearly every 8-bit probability is then nonzero and every tile
	# moves the output (with Gaussian queries only about one key in a hundred keeps a nonzero probability)
	q[8:16] = q[8:16] // 16
	q[16] = 0
	lens[8:17] = [4096, 4096, 4001, 3000, 2049, 1000, 4096, 333, 4096]
	kern = recipes.attn_decode_kernel(dev, h, hd, cap, True)
	out = X.Tensor(dev, (s, h * hd), X.INT8)
	l = X.Tensor(dev, (s, h), X.F32)
	kern.launch(_up(dev, q, X.INT8), _up(dev, cache, X.INT8), _up(dev, lens.view(np.float32), X.F32),
	            _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32), out, l, w)
	got, got_l = out.download(), l.download()
	heads = [0, 5, 17, 31]
	sub_cache = np.ascontiguousarray(np.concatenate([cache[:, :, hh * 2 * hd:(hh + 1) * 2 * hd] for hh in heads], axis=2))
	want, want_l = S.attn_decode_i8(_head_columns(q, heads, hd), sub_cache, lens, sk[heads], sv[heads], temp[heads],
	                                len(heads), hd, w)
	assert np.array_equal(_head_columns(got, heads, hd), want)
	assert np.array_equal(got_l[:, heads].view(np.uint32), np.asarray(want_l).reshape(s, len(heads)).view(np.uint32))


def _scales(rng, shape):
	return (0.125 * (0.5 + rng.random(shape))).astype(np.float32)


def test_config5_row_scaled_prefill_and_decode_sampled_heads(dev):
	"""benchmark config 5 with one scale per (row, head) of q, k and v and bf16 output: the 65536-token
	prefill (one head recomputed by the oracle, all queries) and the 64-sequence decode against row-scaled
	caches with ragged lengths (three heads of every sequence)."""
	t, h, hd, w = 65536, 32, 128, 4096
	rng = rng_for("full-config5-rows")
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	qs, ks, vs = _scales(rng, (h, t)), _scales(rng, (h, t)), _scales(rng, (h, t))
	vw, sw, osc = recipes.attn_row_scale_operands(vs, X.BF16)
	out = X.Tensor(dev, q.shape, X.BF16)
	l = X.Tensor(dev, (h, t), X.F32)
	skt, svt, tt = _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32)
	recipes.attn_row_scaled_kernel(dev, h, hd, X.BF16, True).launch_row_scaled(
		_up(dev, q, X.INT8), _up(dev, kv, X.INT8), skt, svt, tt, out, l, w,
		_up(dev, qs, X.F32), _up(dev, ks, X.F32), _up(dev, vw, X.F32), _up(dev, sw, X.F32), _up(dev, osc, X.F32))
	got, got_l = out.download(), l.download()
	heads = [20]
	want, want_l = S.attn_fwd_i8_row_scaled(_head_columns(q, heads, hd), _head_columns(kv, heads, 2 * hd), sk[heads], sv[heads],
	                                        temp[heads], len(heads), hd, w, qs[heads], ks[heads], vw[heads], sw[heads], osc[heads],
	                                        out_bf16=True)
	assert np.array_equal(_head_columns(got, heads, hd), want)
	assert np.array_equal(got_l[heads].view(np.uint32), want_l.view(np.uint32))

	s, cap = 64, 4096
	qd = q[:s]
	cache = kv.reshape(t // cap, cap, 2 * h * hd)[np.arange(s) % (t // cap)]      # the prefill's kv rows, as 64 caches
	lens = rng.integers(1, cap + 1, s).astype(np.uint32)
	lens[:8] = [0, 1, 15, 16, 17, 4095, 4096, 2048]
	qsd, ksd, vsd = _scales(rng, (s, h)), _scales(rng, (s, h, cap)), _scales(rng, (s, h, cap))
	vwd, swd, oscd = recipes.attn_row_scale_operands(vsd, X.BF16)
	outd = X.Tensor(dev, (s, h * hd), X.BF16)
	ld = X.Tensor(dev, (s, h), X.F32)
	recipes.attn_decode_row_scaled_kernel(dev, h, hd, cap, X.BF16, True).launch_row_scaled(
		_up(dev, qd, X.INT8), _up(dev, cache, X.INT8), _up(dev, lens.view(np.float32), X.F32), skt, svt, tt, outd, ld, w,
		_up(dev, qsd, X.F32), _up(dev, ksd, X.F32), _up(dev, vwd, X.F32), _up(dev, swd, X.F32), _up(dev, oscd, X.F32))
	gotd, gotd_l = outd.download(), ld.download()
	heads = [1, 16, 30]
	sub_cache = np.ascontiguousarray(np.concatenate([cache[:, :, hh * 2 * hd:(hh + 1) * 2 * hd] for hh in heads], axis=2))
	wantd, wantd_l = S.attn_decode_i8_row_scaled(
		_head_columns(qd, heads, hd), sub_cache, lens, sk[heads], sv[heads], temp[heads], len(heads), hd, w,
		qsd[:, heads], ksd[:, heads], vwd[:, heads], swd[heads], oscd[heads], out_bf16=True)
	assert np.array_equal(_head_columns(gotd, heads, hd), wantd)
	assert np.array_equal(gotd_l[:, heads].view(np.uint32), np.asarray(wantd_l).reshape(s, len(heads)).view(np.uint32))


def test_config4_block_chain(dev):
	"""benchmark config 4 as one chain (tests/config4_chain.py): seeded bf16 residual stream [4 x 8192, 2048] through
	x17ai_amd.block.Block -- rms_norm, q, kv (head_dim 128, 4096 raw columns, a 16-tile-wide persistent walk),
	attention, attn_y, ffn_f -> e4m3, e4m3 x int8 ffn_y -- strict builds, each stage against the oracle on the GPU's
	own upstream output: sampled token rows bit for bit (ffn_y: one e4m3 code, < 0.5 %), three attention heads over
	all 8192 queries of their sequence.  Then the speed build of each stage against the strict one over the whole
	tensors, with the bounds the speed builds are documented to keep."""
	from tests import config4_chain as C
	inp = C.inputs()
	got = C.run_strict(dev, inp)
	C.check_strict(inp, got)
	rep = C.fast_vs_strict(dev, inp, got)
	# no approximate operation upstream of these stores
	assert rep["attn_q"]["mismatched"] == 0 and rep["attn_kv"]["mismatched"] == 0 and rep["attn_kv"]["rrms_bits_equal"]
	a = rep["attn_fwd_i8"]
	assert a["hist_abs_code_diff_0_1_2_3_more"][2:] == [0, 0, 0] and a["mismatched"] < 0.02 * a["elements"], a
	for name in ("attn_y", "ffn_f", "ffn_y_f8"):
		r = rep[name]
		assert r["frac_mismatched"] < 5e-3 and r["frac_beyond_one_code"] == 0.0, (name, r)
	# the q and kv projections as one launch (24 column tiles, the first 8 through the Scale writer): the same bytes
	fused = C.run_fused_qkv(dev, got)
	for name in ("q", "kv"):
		assert np.array_equal(fused[name], got[name]), name
	assert np.array_equal(fused["k_rrms"].view(np.uint32), got["k_rrms"].view(np.uint32))


def test_benched_speed_builds_against_strict_builds(dev):
	"""Every speed build bench.py times outside the config 4 chain, at the size it is timed at, against its strict build
	over ALL outputs (tests/fast_builds.py; the figures of one run are tests/golden/fast_builds_vs_strict.json): config 5
	decode with ragged lengths, flat-score sequences and the dense all-zero-query case, plain and row-scaled; the
	row-scaled bf16 prefill over all 65536 x 4096 outputs; the dequantising GEMM pair of config 2."""
	from tests import fast_builds as FB
	d = FB.decode(dev)
	assert d["hist_abs_code_diff_0_1_2_3_more"][2:] == [0, 0, 0] and d["mismatched"] < 0.02 * d["elements"], d
	assert d["l_max_abs"] < 1e-4 and d["dense_sequences_mismatched"] < 0.02 * 8 * 4096, d
	r = FB.decode_row_scaled(dev)
	assert r["frac_mismatched"] < 1e-3 and r["beyond_one_step_and_floor"] == 0 and r["l_max_abs"] < 1e-4, r
	p = FB.prefill_row_scaled(dev)
	# (bf16 patterns differ where a rounding flips: 5.6 % of them, by one bf16 step; 1.4e-5 of the outputs differ by
	# more than a step and more than the weight of one 8-bit probability step)
	assert p["frac_mismatched"] < 0.10 and p["beyond_one_step_and_floor"] < 1e-4 * p["elements"], p
	assert p["rel_l2"] < 3e-3 and p["max_abs"] <= 0.125 and p["l_max_abs"] < 1e-4, p
	q = FB.dequant_pair(dev)
	assert q["plain_bf16"]["mismatched"] == 0, q                   # no approximate operation upstream of the store
	g = q["geglu_bf16"]
	assert g["frac_mismatched"] < 1e-4 and g["beyond_one_step_and_floor"] == 0 and g["rel_l2"] < 1e-4, g
