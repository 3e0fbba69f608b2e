"""GPU parity of the int8 sliding-window attention (prefill), the single-token decode and rms_norm.

Checker: the CPU oracle's restatement of the reference's op sequence (oracle/x17_oracle.c), which
itself reproduces the CUDA side of the reference's golden report (tests/test_oracle_golden.py).
Bars: strict_math builds are bit-exact (int8 output codes and the f32 log-sum-exp bits);
hardware-exponent builds stay within one output code in a stated small fraction of elements.
"""
import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd import recipes
from oracle import strict as S
from tests.gpu_common import e4m3_bytes, i8_codes, rng_for

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


def _attn_inputs(rng, rows, h, hd):
	q = i8_codes(rng, (rows, h * hd))
	k = rng.standard_normal((rows, h, hd))
	k /= np.sqrt((k * k).mean(-1, keepdims=True))                  # K is RMS-normed upstream
	v = rng.standard_normal((rows, h, hd)) * 1.3
	kv = S.f32_to_fixedi8((np.concatenate((k, v), axis=2).reshape(rows, 2 * h * hd) * 8).astype(np.float32))
	sk = rng.standard_normal((h, hd))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	sink_k = S.f32_to_fixedi8((sk * 8).astype(np.float32))
	sink_v = i8_codes(rng, (h, hd), 1.3)
	temp = (0.5 + rng.random(h)).astype(np.float32)
	return q, kv, sink_k, sink_v, temp


def _run_attn(dev, kern, q, kv, sink_k, sink_v, temp, window, batch=1, want_l=True):
	h = sink_k.shape[0]
	out = X.Tensor(dev, q.shape, X.INT8)
	l = X.Tensor(dev, (h, q.shape[0]), X.F32) if want_l else None
	kern.launch(X.Tensor.from_numpy(dev, q, X.INT8), X.Tensor.from_numpy(dev, kv, X.INT8),
	            X.Tensor.from_numpy(dev, sink_k, X.INT8), X.Tensor.from_numpy(dev, sink_v, X.INT8),
	            X.Tensor.from_numpy(dev, temp, X.F32), out, l, window, batch)
	return out.download(), (l.download() if want_l else None)


# (T, H, hd, window)
CASES = [
	(256, 4, 32, 0), (256, 4, 32, 64), (384, 2, 64, 0), (512, 2, 64, 128), (512, 2, 64, 16),
	(384, 2, 128, 0), (640, 2, 128, 256), (1024, 8, 64, 256),          # the last one is benchmark config 1
]


@pytest.mark.parametrize("t,h,hd,w", CASES)
def test_attn_strict_bit_exact(dev, t, h, hd, w):
	rng = rng_for("attn", t, h, hd, w)
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, True)
	got, got_l = _run_attn(dev, kern, q, kv, sk, sv, temp, w)
	want, want_l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	assert np.array_equal(got, want)
	assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32))


@pytest.mark.parametrize("t,h,hd,w", [(512, 2, 64, 128), (640, 2, 128, 256), (1024, 8, 64, 256), (1536, 4, 32, 512), (1024, 2, 128, 0)])
def test_attn_fast_within_one_code(dev, t, h, hd, w):
	rng = rng_for("attn", t, h, hd, w)
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, False)
	got, got_l = _run_attn(dev, kern, q, kv, sk, sv, temp, w)
	want, want_l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	d = np.abs(got.astype(np.int32) - want.astype(np.int32))
	assert d.max() <= 1 and np.mean(d > 0) < 0.02, (d.max(), np.mean(d > 0))
	assert np.max(np.abs(got_l - want_l)) < 1e-4


@pytest.mark.parametrize("t,h,hd,w,strict", [(448, 2, 64, 128, True), (192, 4, 32, 0, True), (1088, 2, 128, 256, True),
                                             (1088, 2, 128, 256, False), (16384 + 64, 2, 128, 512, False),
                                             (128, 2, 64, 0, False), (192, 2, 128, 64, False)])
def test_attn_sequence_lengths_that_are_multiples_of_64_only(dev, t, h, hd, w, strict):
	"""src/device/cuda/attn.rs:398-404 accepts seq_len % 64 == 0; the query block here holds 128 queries.  The last
	block of such a sequence starts 64 queries early: every output against the oracle (strict builds bit for bit)."""
	rng = rng_for("attn-t64", t, h, hd, w)
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, strict)
	got, got_l = _run_attn(dev, kern, q, kv, sk, sv, temp, w)
	want, want_l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	if strict:
		assert np.array_equal(got, want)
		assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32))
	else:
		d = np.abs(got.astype(np.int32) - want.astype(np.int32))
		assert d.max() <= 1 and np.mean(d > 0) < 0.02, (d.max(), np.mean(d > 0))
		assert np.max(np.abs(got_l - want_l)) < 1e-4
	# two stacked sequences of such a length: the second one's rows start at an odd multiple of 64
	if t == 448:
		q2, kv2 = np.concatenate((q, q[::-1])), np.concatenate((kv, kv[::-1]))
		got2, _ = _run_attn(dev, kern, q2, kv2, sk, sv, temp, w, batch=2)
		assert np.array_equal(got2[:t], want)
		assert np.array_equal(got2[t:], S.attn_fwd_i8(q[::-1], kv[::-1], sk, sv, temp, h, hd, w)[0])


def test_attn_batched_sequences_and_no_l(dev):
	"""gridDim.z extension: stacked sequences are independent; L may be omitted (attn.rs:396)."""
	t, h, hd, w, b = 256, 2, 64, 64, 3
	rng = rng_for("attn-batch")
	q, kv, sk, sv, temp = _attn_inputs(rng, b * t, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, True)
	got, got_l = _run_attn(dev, kern, q, kv, sk, sv, temp, w, batch=b)
	got2, _ = _run_attn(dev, kern, q, kv, sk, sv, temp, w, batch=b, want_l=False)
	for i in range(b):
		want, want_l = S.attn_fwd_i8(q[i * t:(i + 1) * t], kv[i * t:(i + 1) * t], sk, sv, temp, h, hd, w)
		assert np.array_equal(got[i * t:(i + 1) * t], want)
		assert np.array_equal(got_l[:, i * t:(i + 1) * t].view(np.uint32), want_l.view(np.uint32))
	assert np.array_equal(got, got2)


def test_attn_special_cases(dev):
	"""Closed-form cases: query 0 sees only the sink; a window that covers the whole sequence equals
	no window; constant V comes back exactly when all scores are equal (q = 0: every probability is
	exactly 255) and within one code otherwise (the numerator sums rounded probabilities, the
	denominator unrounded ones)."""
	t, h, hd = 256, 2, 64
	rng = rng_for("attn-special")
	q, kv, sk, sv, temp = _attn_inputs(rng, t, h, hd)
	kern = recipes.attn_kernel(dev, h, hd, True)
	got, _ = _run_attn(dev, kern, q, kv, sk, sv, temp, 0)
	assert np.array_equal(got[0].reshape(h, hd), sv)
	got_w, _ = _run_attn(dev, kern, q, kv, sk, sv, temp, 256)
	assert np.array_equal(got, got_w)
	kv2 = kv.reshape(t, h, 2, hd).copy()
	kv2[:, :, 1, :] = 40
	sv2 = np.full_like(sv, 40)
	got_c, _ = _run_attn(dev, kern, np.zeros_like(q), kv2.reshape(t, -1), sk, sv2, temp, 64)
	assert np.all(got_c == 40)
	got_r, _ = _run_attn(dev, kern, q, kv2.reshape(t, -1), sk, sv2, temp, 64)
	assert np.all(np.abs(got_r.astype(np.int32) - 40) <= 1)
	want_r, _ = S.attn_fwd_i8(q, kv2.reshape(t, -1), sk, sv2, temp, h, hd, 64)
	assert np.array_equal(got_r, want_r)


def test_attn_fast_temperature_signs_and_closed_forms(dev):
	"""The speed build takes the row maximum over the scores' bits on fully visible tiles, which needs a positive head
	temperature; heads with a negative or zero temperature go through its masked path instead.  All three kinds of
	head in one launch against the oracle, and the closed forms: query 0 sees only the sink, constant V comes back
	exactly when every probability is 255 (q = 0, or temperature 0)."""
	t, h, hd, w = 768, 4, 64, 256
	rng = rng_for("attn-fast-signs")
	q, kv, sk, sv, _ = _attn_inputs(rng, t, h, hd)
	temp = np.array([0.8, -0.6, 0.0, 1.3], np.float32)
	kern = recipes.attn_kernel(dev, h, hd, False)
	got, got_l = _run_attn(dev, kern, q, kv, sk, sv, temp, w)
	want, want_l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	d = np.abs(got.astype(np.int32) - want.astype(np.int32))
	assert d.max() <= 1 and np.mean(d > 0) < 0.02, (d.max(), np.mean(d > 0))
	assert np.max(np.abs(got_l - want_l)) < 1e-4
	assert np.array_equal(got[0].reshape(h, hd), sv)
	kv2 = kv.reshape(t, h, 2, hd).copy()
	kv2[:, :, 1, :] = 40
	sv2 = np.full_like(sv, 40)
	got_c, _ = _run_attn(dev, kern, np.zeros_like(q), kv2.reshape(t, -1), sk, sv2, temp, w)
	assert np.all(got_c == 40)
	got_z, _ = _run_attn(dev, kern, q, kv2.reshape(t, -1), sk, sv2, temp, w)
	assert np.all(got_z.reshape(t, h, hd)[:, 2, :] == 40)          # the head with temperature 0
	assert np.all(np.abs(got_z.astype(np.int32) - 40) <= 1)


def test_attn_launch_rejects_bad_arguments(dev):
	h, hd = 2, 64
	kern = recipes.attn_kernel(dev, h, hd, True)
	rng = rng_for("attn-bad")
	q, kv, sk, sv, temp = _attn_inputs(rng, 256, h, hd)
	with pytest.raises(X.X17Error, match="window_size must be zero or divisible by 16"):
		_run_attn(dev, kern, q, kv, sk, sv, temp, 24)
	with pytest.raises(X.X17Error, match="at least one query block of 128"):
		_run_attn(dev, kern, q[:64], kv[:64], sk, sv, temp, 0)
	# a last block that overhangs recomputes its neighbour's queries from q: the output may not alias an input
	qt = X.Tensor.from_numpy(dev, q, X.INT8)
	with pytest.raises(X.X17Error, match="must not share memory with q or kv"):
		kern.launch(qt, X.Tensor.from_numpy(dev, kv, X.INT8), X.Tensor.from_numpy(dev, sk, X.INT8), X.Tensor.from_numpy(dev, sv, X.INT8),
		            X.Tensor.from_numpy(dev, temp, X.F32), qt, None, 0)
	with pytest.raises(X.X17Error, match="kv has 128 rows, but should have 256"):
		_run_attn(dev, kern, q, kv[:128], sk, sv, temp, 0)


# ---------------------------------------------------------------- decode

# (the last two cases have a cache large enough for the P.V partials to live in the free halves of the LDS slots)
@pytest.mark.parametrize("h,hd,cap,w", [(4, 32, 256, 0), (4, 64, 256, 64), (2, 128, 512, 128), (2, 128, 512, 0),
                                        (2, 32, 4096, 0), (2, 64, 4096, 2048)])
def test_decode_bit_exact_and_equals_prefill_row(dev, h, hd, cap, w):
	s = 6
	rng = rng_for("decode", h, hd, cap, w)
	q, kv, sk, sv, temp = _attn_inputs(rng, s * cap, h, hd)
	cache = kv.reshape(s, cap, 2 * h * hd)
	qd = q[:s]
	lens = np.array([0, 1, 17, cap // 2 + 5, cap - 1, cap], dtype=np.uint32)
	kern = recipes.attn_decode_kernel(dev, h, hd, cap, True)
	out = X.Tensor(dev, (s, h * hd), X.INT8)
	l = X.Tensor(dev, (s, h), X.F32)
	kern.launch(X.Tensor.from_numpy(dev, qd, X.INT8), X.Tensor.from_numpy(dev, cache, X.INT8),
	            X.Tensor.from_numpy(dev, lens.view(np.float32), X.F32), X.Tensor.from_numpy(dev, sk, X.INT8),
	            X.Tensor.from_numpy(dev, sv, X.INT8), X.Tensor.from_numpy(dev, temp, X.F32), out, l, w)
	got, got_l = out.download(), l.download()
	want, want_l = S.attn_decode_i8(qd, cache, lens, sk, sv, temp, h, hd, w)
	assert np.array_equal(got, want)
	assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32))
	# the definition: decoding at position p equals row p of a prefill over the first p+1 rows
	seq = 3
	p = int(lens[seq])
	rows = ((p + 1 + 127) // 128) * 128
	qq = np.zeros((rows, h * hd), np.int8)
	qq[p] = qd[seq]
	kk = np.zeros((rows, 2 * h * hd), np.int8)
	kk[:p] = cache[seq, :p]
	pre, pre_l = S.attn_fwd_i8(qq, kk, sk, sv, temp, h, hd, w)
	assert np.array_equal(pre[p], got[seq])
	assert np.array_equal(pre_l[:, p].view(np.uint32), got_l[seq].view(np.uint32))


# ---------------------------------------------------------------- rms_norm

@pytest.mark.parametrize("rows,d", [(8, 512), (64, 2048), (256, 4096)])
def test_rms_norm_bit_exact(dev, rows, d):
	rng = rng_for("rms", rows, d)
	x = e4m3_bytes(rng, (rows, d), 1.5)
	kern = recipes.rms_norm_kernel(dev, d, X.E4M3)
	out = X.Tensor(dev, (rows, d), X.INT8)
	kern.launch(X.Tensor.from_numpy(dev, x, X.E4M3), out)
	assert np.array_equal(out.download(), S.rms_norm(x, recipes.L2_NORM_EPS, "e4m3"))
	xb = (rng.standard_normal((rows, d)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
	kern_b = recipes.rms_norm_kernel(dev, d, X.BF16)
	kern_b.launch(X.Tensor.from_numpy(dev, xb, X.BF16), out)
	assert np.array_equal(out.download(), S.rms_norm(xb, recipes.L2_NORM_EPS, "bf16"))
	with pytest.raises(X.X17Error, match="rows must be divisible by 8"):
		kern.launch(X.Tensor(dev, (4, d), X.E4M3), X.Tensor(dev, (4, d), X.INT8))


# ---------------------------------------------------------------- row-scaled operands (own definition)

def _row_scaled_inputs(rng, rows, h, hd):
	"""q, k, v ~ N(0, 1) times a per-(row, head) magnitude, quantised per row to int8 at absmax / 127."""
	from oracle import dense as D
	spread = np.exp(rng.normal(0.0, 0.5, (3, rows, h, 1)))
	qc, qs = D.quantize_rows(rng.standard_normal((rows, h, hd)) * spread[0])
	kc, ks = D.quantize_rows(rng.standard_normal((rows, h, hd)) * spread[1])
	vc, vs = D.quantize_rows(rng.standard_normal((rows, h, hd)) * spread[2])
	kv = np.concatenate((kc, vc), axis=2).reshape(rows, 2 * h * hd)
	sink_k = i8_codes(rng, (h, hd))
	sink_v = i8_codes(rng, (h, hd), 1.3)
	temp = (0.5 + rng.random(h)).astype(np.float32)
	head_major = lambda a: np.ascontiguousarray(a.T)          # the scale matrices are [H, rows], like L
	return qc.reshape(rows, h * hd), kv, head_major(qs), head_major(ks), head_major(vs), sink_k, sink_v, temp


def _run_row_scaled(dev, kern, q, kv, sink_k, sink_v, temp, window, qs, ks, vw, sw, osc, batch=1):
	h = sink_k.shape[0]
	out = X.Tensor(dev, q.shape, kern.config.out_dtype)
	l = X.Tensor(dev, (h, q.shape[0]), X.F32)
	f32 = lambda a: X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32)
	kern.launch_row_scaled(X.Tensor.from_numpy(dev, q, X.INT8), X.Tensor.from_numpy(dev, kv, X.INT8),
	                       X.Tensor.from_numpy(dev, sink_k, X.INT8), X.Tensor.from_numpy(dev, sink_v, X.INT8),
	                       f32(temp), out, l, window, f32(qs), f32(ks), f32(vw), f32(sw), f32(osc), batch)
	return out.download(), l.download()


# the first case is benchmark config 1 as written: per-row absmax / 127 scales, bf16 output
@pytest.mark.parametrize("t,h,hd,w,out_dtype", [
	(1024, 8, 64, 256, X.BF16), (384, 4, 32, 0, X.BF16), (640, 2, 128, 256, X.BF16), (512, 2, 64, 48, X.INT8),
])
def test_attn_row_scaled_strict_bit_exact(dev, t, h, hd, w, out_dtype):
	rng = rng_for("attn-rows", t, h, hd, w)
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(rng, t, h, hd)
	vw, sw, osc = recipes.attn_row_scale_operands(vs, out_dtype)
	kern = recipes.attn_row_scaled_kernel(dev, h, hd, out_dtype, True)
	got, got_l = _run_row_scaled(dev, kern, q, kv, sk, sv, temp, w, qs, ks, vw, sw, osc)
	want, want_l = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, qs, ks, vw, sw, osc, out_bf16=out_dtype == X.BF16)
	assert np.array_equal(got, want)
	assert np.array_equal(got_l.view(np.uint32), want_l.view(np.uint32))


def test_attn_row_scaled_equals_plain_kernel_at_scale_one_eighth(dev):
	"""With every scale 1/8 and every weight 1 the row-scaled kernel IS the reference's arithmetic."""
	t, h, hd, w, b = 256, 2, 64, 64, 2
	rng = rng_for("attn-rows-eighth")
	q, kv, sk, sv, temp = _attn_inputs(rng, b * t, h, hd)
	plain, plain_l = _run_attn(dev, recipes.attn_kernel(dev, h, hd, True), q, kv, sk, sv, temp, w, batch=b)
	eighth = np.full((h, b * t), 0.125, np.float32)
	kern = recipes.attn_row_scaled_kernel(dev, h, hd, X.INT8, True)
	got, got_l = _run_row_scaled(dev, kern, q, kv, sk, sv, temp, w, eighth, eighth, np.ones((h, b * t)), np.ones(h), np.ones(h),
	                             batch=b)
	assert np.array_equal(got, plain)
	assert np.array_equal(got_l.view(np.uint32), plain_l.view(np.uint32))


@pytest.mark.parametrize("t,h,hd,w", [(1024, 8, 64, 256), (640, 2, 128, 256)])
def test_attn_row_scaled_fast_within_tolerance(dev, t, h, hd, w):
	"""Hardware-exponent build, bf16 output: relative L2 error against the strict definition below 2^-8
	and no element further off than 3 % of the largest output (a probability that rounds the other way
	moves one value row by one step)."""
	rng = rng_for("attn-rows", t, h, hd, w)
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(rng, t, h, hd)
	vw, sw, osc = recipes.attn_row_scale_operands(vs, X.BF16)
	kern = recipes.attn_row_scaled_kernel(dev, h, hd, X.BF16, False)
	got, got_l = _run_row_scaled(dev, kern, q, kv, sk, sv, temp, w, qs, ks, vw, sw, osc)
	want, want_l = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, qs, ks, vw, sw, osc, out_bf16=True)
	g = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	e = (want.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	rel_l2 = np.sqrt(np.sum((g - e) ** 2) / np.sum(e ** 2))
	max_abs = np.abs(g - e).max() / np.abs(e).max()
	assert rel_l2 < 2.0 ** -8 and max_abs < 0.03, (rel_l2, max_abs)
	assert np.max(np.abs(got_l - want_l)) < 1e-4


def test_attn_row_scaled_launch_checks(dev):
	t, h, hd = 128, 2, 64
	rng = rng_for("attn-rows-checks")
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(rng, t, h, hd)
	vw, sw, osc = recipes.attn_row_scale_operands(vs, X.BF16)
	kern = recipes.attn_row_scaled_kernel(dev, h, hd, X.BF16, True)
	with pytest.raises(X.X17Error):          # scale matrix of the wrong shape
		_run_row_scaled(dev, kern, q, kv, sk, sv, temp, 0, qs[:, :64], ks, vw, sw, osc)
	with pytest.raises(X.X17Error):          # a plain launch of a row-scaled kernel
		_run_attn(dev, kern, q, kv, sk, sv, temp, 0)
	with pytest.raises(X.X17Error):          # and scales handed to a plain kernel
		_run_row_scaled(dev, recipes.attn_kernel(dev, h, hd, True), q, kv, sk, sv, temp, 0, qs, ks, vw, sw, osc)
	with pytest.raises(X.X17Error):          # bf16 output exists only with row scales
		X.AttnKernel(None, "attn-bad-out", X.AttnKernelConfig(X.INT8, h, hd, h * hd, 2 * h * hd, h * hd, False, X.BF16))


@pytest.mark.parametrize("h,hd,cap,w,out_dtype", [(4, 64, 256, 64, X.BF16), (2, 128, 512, 0, X.BF16), (4, 32, 256, 0, X.INT8)])
def test_decode_row_scaled_bit_exact(dev, h, hd, cap, w, out_dtype):
	s = 6
	rng = rng_for("decode-rows", h, hd, cap, w)
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(rng, s * cap, h, hd)
	cache = kv.reshape(s, cap, 2 * h * hd)
	lens = np.array([0, 1, 17, cap // 2 + 5, cap - 1, cap], dtype=np.uint32)
	per_cache = lambda a: np.ascontiguousarray(a.reshape(h, s, cap).transpose(1, 0, 2))      # [S, H, cap]
	vw, sw, osc = recipes.attn_row_scale_operands(per_cache(vs), out_dtype)
	ks3 = per_cache(ks)
	for i, n in enumerate(lens):                    # rows past the cached length hold no scale worth reading
		ks3[i, :, n:] = np.nan
		vw[i, :, n:] = np.nan
	qd, qsd = q[:s], np.ascontiguousarray(qs[:, :s].T)
	kern = recipes.attn_decode_row_scaled_kernel(dev, h, hd, cap, out_dtype, True)
	out = X.Tensor(dev, (s, h * hd), out_dtype)
	l = X.Tensor(dev, (s, h), X.F32)
	f32 = lambda a: X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32)
	kern.launch_row_scaled(X.Tensor.from_numpy(dev, qd, X.INT8), X.Tensor.from_numpy(dev, cache, X.INT8),
	                       X.Tensor.from_numpy(dev, lens.view(np.float32), X.F32), X.Tensor.from_numpy(dev, sk, X.INT8),
	                       X.Tensor.from_numpy(dev, sv, X.INT8), f32(temp), out, l, w, f32(qsd), f32(ks3), f32(vw), f32(sw), f32(osc))
	want, want_l = S.attn_decode_i8_row_scaled(qd, cache, lens, sk, sv, temp, h, hd, w, qsd, ks3, vw, sw, osc,
	                                           out_bf16=out_dtype == X.BF16)
	assert np.array_equal(out.download(), want)
	assert np.array_equal(l.download().view(np.uint32), want_l.view(np.uint32))
	with pytest.raises(X.X17Error):                 # a plain launch of a row-scaled kernel
		kern.launch(X.Tensor.from_numpy(dev, qd, X.INT8), X.Tensor.from_numpy(dev, cache, X.INT8),
		            X.Tensor.from_numpy(dev, lens.view(np.float32), X.F32), X.Tensor.from_numpy(dev, sk, X.INT8),
		            X.Tensor.from_numpy(dev, sv, X.INT8), f32(temp), out, l, w)
