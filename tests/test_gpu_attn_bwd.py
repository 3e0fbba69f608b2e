"""GPU parity of the attention backward kernels (attn_d_q_i8.hip, attn_d_kv_i8.hip) against the dense float64
definition (oracle/backward.py, pinned by tests/test_oracle_backward.py).
dQ multiplies on the f16 matrix cores (dO rows scaled to [1, 2) and rounded to f16, dS rounded to f16) and writes bf16:
tolerance parity, with the tolerance written here -- relative L2 error below 4e-3 (one bf16 rounding of the output
alone is 2.3e-3 rms) and every element within 1.5 bf16 steps of its row's largest magnitude plus a 1e-2 relative term (and an absolute floor for rows
whose gradient cancels to zero).
dK / dV multiply on the bf16 matrix cores (P and dS rounded to bf16 as attn_d_kv.cuh:330-365 does) and write bf16:
relative L2 error below 4e-3 for each of dK and dV, and every element within 2^-8 of the sum of the magnitudes of its
terms (each term carries one bf16 rounding of P or dS, 2^-9 relative) plus one bf16 step of its own value."""
import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd import recipes
from oracle import backward as B
from oracle import strict as S
from tests.gpu_common import i8_codes, rng_for

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


def _bf16_bits(x):
	u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
	return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _bf16_value(bits):
	return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def _inputs(rng, rows, h, hd):
	q = i8_codes(rng, (rows, h * hd))
	k = rng.standard_normal((rows, h, hd), dtype=np.float32)
	k /= np.sqrt((k * k).mean(-1, keepdims=True))
	v = rng.standard_normal((rows, h, hd), dtype=np.float32) * 1.3
	kv = S.f32_to_fixedi8((np.concatenate((k, v), axis=2).reshape(rows, 2 * h * hd) * 8).astype(np.float32))
	sk = rng.standard_normal((h, hd))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	return q, kv, S.f32_to_fixedi8((sk * 8).astype(np.float32)), i8_codes(rng, (h, hd), 1.3), (0.5 + rng.random(h)).astype(np.float32)


def _run(dev, h, hd, t, batch, w, strict, d_o_bits, q, kv, sk, sv, temp):
	"""Forward (strict build) for out and L, then the backward kernel; returns everything as numpy."""
	rows = t * batch
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	tq, tkv, tsk, tsv, tt = up(q, X.INT8), up(kv, X.INT8), up(sk, X.INT8), up(sv, X.INT8), up(temp, X.F32)
	out, l = X.Tensor(dev, (rows, h * hd), X.INT8), X.Tensor(dev, (h, rows), X.F32)
	recipes.attn_kernel(dev, h, hd, True).launch(tq, tkv, tsk, tsv, tt, out, l, w, batch)
	dq, d = X.Tensor(dev, (rows, h * hd), X.BF16), X.Tensor(dev, (h, rows), X.F32)
	recipes.attn_d_q_kernel(dev, h, hd, strict).launch_d_q(tq, tkv, tsk, tsv, tt, out, up(d_o_bits, X.BF16), dq, l, d, w, batch)
	return out.download(), l.download(), dq.download(), d.download()


def _check(got_bits, got_d, want, want_d, d_o):
	got = _bf16_value(got_bits)
	rel_l2 = np.linalg.norm(got - want) / np.linalg.norm(want)
	assert rel_l2 < 4e-3, rel_l2
	row_max = np.abs(want).max(axis=1, keepdims=True)
	# (floor: a row whose probabilities are one-hot has dP - D = 0 exactly, and the kernel's f32 difference leaves
	# rounding noise of the order 2^-24 |D|; 1e-6 of the row's sum of |dO| is far above that and far below any gradient)
	floor = 1e-6 * np.abs(d_o).sum(axis=1, keepdims=True)
	assert np.all(np.abs(got - want) <= 1.5 * 2.0 ** -8 * row_max + 1e-2 * np.abs(want) + floor + 1e-30), float(np.abs(got - want).max())
	# D = dO . o with the stored output: f32 sums of f16-rounded dO
	scale = np.abs(d_o).sum(axis=1).max()
	assert np.abs(got_d - want_d).max() <= 2e-3 * scale, (float(np.abs(got_d - want_d).max()), scale)


@pytest.mark.parametrize("strict", [True, False])
def test_d_q_at_the_size_of_benchmark_config_1(dev, strict):
	"""T = 1024, 8 heads x 64, window 256 (two heads per workgroup), dO ~ N(0, 0.1^2) as bf16."""
	t, h, hd, w = 1024, 8, 64, 256
	rng = rng_for("attn-bwd-config1")
	q, kv, sk, sv, temp = _inputs(rng, t, h, hd)
	d_o_bits = _bf16_bits(rng.standard_normal((t, h * hd)) * 0.1)
	d_o = _bf16_value(d_o_bits)
	out, l, dq_bits, d = _run(dev, h, hd, t, 1, w, strict, d_o_bits, q, kv, sk, sv, temp)
	want, want_d = B.attn_d_q(q, kv, sk, sv, temp, h, hd, w, out, d_o, l.astype(np.float64))
	_check(dq_bits, d.astype(np.float64), want, want_d, d_o)
	assert np.abs(want).max() > 1e-3
	# query 0 of the sequence sees only the sink: no dependence on q
	assert not _bf16_value(dq_bits[0]).any()


@pytest.mark.parametrize("h,hd,t,batch,w", [(2, 128, 384, 1, 0), (2, 128, 320, 2, 48), (4, 32, 256, 3, 16), (2, 64, 192, 1, 64)])
def test_d_q_shapes_windows_batches_and_overhanging_blocks(dev, h, hd, t, batch, w):
	rng = rng_for("attn-bwd", h, hd, t, batch, w)
	rows = t * batch
	q, kv, sk, sv, temp = _inputs(rng, rows, h, hd)
	temp[0] = -0.7                                            # a negative head temperature
	# gradients of very different magnitudes from row to row (each row is scaled on its own), some rows all zero
	mag = 10.0 ** rng.uniform(-9, 1, (rows, 1))
	d_o_f = rng.standard_normal((rows, h * hd)) * mag
	d_o_f[5] = 0.0
	d_o_f[rows - 1, :hd] = 0.0
	d_o_bits = _bf16_bits(d_o_f)
	d_o = _bf16_value(d_o_bits)
	out, l, dq_bits, d = _run(dev, h, hd, t, batch, w, True, d_o_bits, q, kv, sk, sv, temp)
	got = _bf16_value(dq_bits)
	for b in range(batch):                                    # sequences are independent: one oracle call each
		r = slice(b * t, (b + 1) * t)
		want, want_d = B.attn_d_q(q[r], kv[r], sk, sv, temp, h, hd, w, out[r], d_o[r], l[:, r].astype(np.float64))
		for hh in range(h):                                   # per head: rows of different heads have different scales
			c = slice(hh * hd, (hh + 1) * hd)
			row_max = np.abs(want[:, c]).max(axis=1, keepdims=True)
			err = np.abs(got[r, c] - want[:, c])
			assert np.all(err <= 1.5 * 2.0 ** -8 * row_max + 1e-2 * np.abs(want[:, c]) + 1e-30), (b, hh, float(err.max()))
			dscale = np.abs(d_o[r, c]).sum(axis=1)
			assert np.all(np.abs(d[hh, r] - want_d[hh]) <= 2e-3 * dscale + 1e-30), (b, hh)
	assert not got[5].any()


def test_d_q_launch_rejects_bad_arguments(dev):
	h, hd, t = 2, 64, 256
	rng = rng_for("attn-bwd-bad")
	q, kv, sk, sv, temp = _inputs(rng, t, h, hd)
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	args = [up(q, X.INT8), up(kv, X.INT8), up(sk, X.INT8), up(sv, X.INT8), up(temp, X.F32)]
	out, l = X.Tensor(dev, (t, h * hd), X.INT8), X.Tensor(dev, (h, t), X.F32)
	d_o, dq = X.Tensor(dev, (t, h * hd), X.BF16), X.Tensor(dev, (t, h * hd), X.BF16)
	kern = recipes.attn_d_q_kernel(dev, h, hd, True)
	with pytest.raises(X.X17Error, match="is a backward kernel"):
		kern.launch(*args, out, l, 0)
	with pytest.raises(X.X17Error, match="is not a backward-with-respect-to-q kernel"):
		recipes.attn_kernel(dev, h, hd, True).launch_d_q(*args, out, d_o, dq, l, None, 0)
	with pytest.raises(X.X17Error, match="d_out has dtype i8, but should have bf16"):
		kern.launch_d_q(*args, out, out, dq, l, None, 0)
	with pytest.raises(X.X17Error, match="must not share memory"):
		kern.launch_d_q(*args, out, d_o, d_o, l, None, 0)
	kern.launch_d_q(*args, out, d_o, dq, l, None, 0)
	dev.synchronize()


# ---------------------------------------------------------------- dK, dV

def _run_kv(dev, h, hd, t, batch, w, strict, d_o_bits, q, kv, sk, sv, temp):
	"""Forward and dQ pass (strict builds) for out, L and D, then the dK/dV kernel; returns l, d, d_kv as numpy."""
	rows = t * batch
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	tq, tkv, tsk, tsv, tt = up(q, X.INT8), up(kv, X.INT8), up(sk, X.INT8), up(sv, X.INT8), up(temp, X.F32)
	out, l = X.Tensor(dev, (rows, h * hd), X.INT8), X.Tensor(dev, (h, rows), X.F32)
	recipes.attn_kernel(dev, h, hd, True).launch(tq, tkv, tsk, tsv, tt, out, l, w, batch)
	t_do = up(d_o_bits, X.BF16)
	dq, d = X.Tensor(dev, (rows, h * hd), X.BF16), X.Tensor(dev, (h, rows), X.F32)
	recipes.attn_d_q_kernel(dev, h, hd, True).launch_d_q(tq, tkv, tsk, tsv, tt, out, t_do, dq, l, d, w, batch)
	d_kv = X.Tensor.from_numpy(dev, np.full((rows, 2 * h * hd), 0x7FC0, np.uint16), X.BF16)        # NaN until written
	recipes.attn_d_kv_kernel(dev, h, hd, strict).launch_d_kv(tq, tkv, tt, t_do, l, d, d_kv, w, batch)
	return l.download(), d.download(), d_kv.download()


def _term_magnitudes(q, kv, sk, sv, temp, h, hd, w, d_o, l, d):
	"""Per element of d_kv, the sum of the magnitudes of its terms: |dS|^T |q| t for dK, P^T |dO| for dV (float64)."""
	t = q.shape[0]
	wr = 0 if w == 0 else ((w - 1) // 16 + 1) * 16
	out = np.empty((t, 2 * h * hd))
	for hh in range(h):
		qs, ks, vs = slice(hh * hd, (hh + 1) * hd), slice(2 * hh * hd, (2 * hh + 1) * hd), slice((2 * hh + 1) * hd, (2 * hh + 2) * hd)
		qr, kr, vr = q[:, qs] / 8.0, kv[:, ks] / 8.0, kv[:, vs] / 8.0
		ti = B.temperature(t, hd, wr, float(temp[hh]))
		prob = np.where(B.visible(t, wr)[:, 1:], np.exp2((qr @ kr.T) * ti - (l[hh][:, None] - B.LOG2_255)), 0.0)
		ds = np.log(2.0) * prob * np.abs(d_o[:, qs] @ vr.T - d[hh][:, None])
		out[:, ks] = (ds * np.abs(ti)).T @ np.abs(qr)
		out[:, vs] = prob.T @ np.abs(d_o[:, qs])
	return out


def _check_kv(got_bits, want, terms, h, hd):
	got = _bf16_value(got_bits)
	assert np.isfinite(got).all()                                       # every element was written
	for hh in range(h):
		for part in (slice(2 * hh * hd, (2 * hh + 1) * hd), slice((2 * hh + 1) * hd, (2 * hh + 2) * hd)):
			rel_l2 = np.linalg.norm(got[:, part] - want[:, part]) / np.linalg.norm(want[:, part])
			assert rel_l2 < 4e-3, (hh, part, rel_l2)
	err = np.abs(got - want)
	bound = 2.0 ** -8 * terms + 2.0 ** -8 * np.abs(want) + 1e-30
	assert np.all(err <= bound), (float((err / bound).max()), np.unravel_index(np.argmax(err / bound), err.shape))


@pytest.mark.parametrize("strict", [True, False])
def test_d_kv_at_the_size_of_benchmark_config_1(dev, strict):
	"""T = 1024, 8 heads x 64, window 256 (two heads per workgroup), dO ~ N(0, 0.1^2) as bf16."""
	t, h, hd, w = 1024, 8, 64, 256
	rng = rng_for("attn-bwd-kv-config1")
	q, kv, sk, sv, temp = _inputs(rng, t, h, hd)
	d_o_bits = _bf16_bits(rng.standard_normal((t, h * hd)) * 0.1)
	d_o = _bf16_value(d_o_bits)
	l, d, got = _run_kv(dev, h, hd, t, 1, w, strict, d_o_bits, q, kv, sk, sv, temp)
	l, d = l.astype(np.float64), d.astype(np.float64)
	want = B.attn_d_kv(q, kv, sk, sv, temp, h, hd, w, d_o, l, d)
	assert np.abs(want).max() > 1e-3
	_check_kv(got, want, _term_magnitudes(q, kv, sk, sv, temp, h, hd, w, d_o, l, d), h, hd)
	# the last key of the sequence is seen by no query
	assert not _bf16_value(got[t - 1]).any()


@pytest.mark.parametrize("h,hd,t,batch,w", [(2, 128, 384, 1, 0), (2, 128, 320, 2, 48), (4, 32, 256, 3, 16), (2, 64, 192, 1, 64),
                                            (2, 64, 128, 2, 0)])
def test_d_kv_shapes_windows_batches_and_overhanging_blocks(dev, h, hd, t, batch, w):
	rng = rng_for("attn-bwd-kv", h, hd, t, batch, w)
	rows = t * batch
	q, kv, sk, sv, temp = _inputs(rng, rows, h, hd)
	temp[0] = -0.7                                            # a negative head temperature
	# gradients of very different magnitudes from row to row (bf16 is used as it is), some rows all zero
	mag = 10.0 ** rng.uniform(-9, 1, (rows, 1))
	d_o_f = rng.standard_normal((rows, h * hd)) * mag
	d_o_f[5] = 0.0
	d_o_bits = _bf16_bits(d_o_f)
	d_o = _bf16_value(d_o_bits)
	l, d, got_bits = _run_kv(dev, h, hd, t, batch, w, True, d_o_bits, q, kv, sk, sv, temp)
	l, d = l.astype(np.float64), d.astype(np.float64)
	got = _bf16_value(got_bits)
	assert np.isfinite(got).all()
	for b in range(batch):                                    # sequences are independent: one oracle call each
		r = slice(b * t, (b + 1) * t)
		want = B.attn_d_kv(q[r], kv[r], sk, sv, temp, h, hd, w, d_o[r], l[:, r], d[:, r])
		terms = _term_magnitudes(q[r], kv[r], sk, sv, temp, h, hd, w, d_o[r], l[:, r], d[:, r])
		err = np.abs(got[r] - want)
		bound = 2.0 ** -8 * terms + 2.0 ** -8 * np.abs(want) + 1e-30
		assert np.all(err <= bound), (b, float((err / bound).max()))
		assert not got[r][t - 1].any()                        # a sequence's last key is seen by no query of it


def test_d_kv_launch_rejects_bad_arguments(dev):
	h, hd, t = 2, 64, 256
	rng = rng_for("attn-bwd-kv-bad")
	q, kv, sk, sv, temp = _inputs(rng, t, h, hd)
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	tq, tkv, tt = up(q, X.INT8), up(kv, X.INT8), up(temp, X.F32)
	l, d = X.Tensor.from_numpy(dev, np.zeros((h, t), np.float32), X.F32), X.Tensor.from_numpy(dev, np.zeros((h, t), np.float32), X.F32)
	d_o = X.Tensor.from_numpy(dev, np.zeros((t, h * hd), np.uint16), X.BF16)
	d_kv = X.Tensor(dev, (t, 2 * h * hd), X.BF16)
	kern = recipes.attn_d_kv_kernel(dev, h, hd, True)
	with pytest.raises(X.X17Error, match="is not a backward-with-respect-to-k-and-v kernel"):
		recipes.attn_d_q_kernel(dev, h, hd, True).launch_d_kv(tq, tkv, tt, d_o, l, d, d_kv, 0)
	with pytest.raises(X.X17Error, match="is a backward kernel"):
		kern.launch(tq, tkv, up(sk, X.INT8), up(sv, X.INT8), tt, X.Tensor(dev, (t, h * hd), X.INT8), None, 0)
	with pytest.raises(X.X17Error, match="d_kv"):
		kern.launch_d_kv(tq, tkv, tt, d_o, l, d, X.Tensor(dev, (t, h * hd), X.BF16), 0)      # the width of q, not of kv
	with pytest.raises(X.X17Error, match="window_size must be zero or divisible by 16"):
		kern.launch_d_kv(tq, tkv, tt, d_o, l, d, d_kv, 24)
	with pytest.raises(X.X17Error, match="at least one key block of 128"):
		kern.launch_d_kv(up(q[:64], X.INT8), up(kv[:64], X.INT8), tt, up(np.zeros((64, h * hd), np.uint16), X.BF16),
		                 up(np.zeros((h, 64), np.float32), X.F32), up(np.zeros((h, 64), np.float32), X.F32), X.Tensor(dev, (64, 2 * h * hd), X.BF16), 0)
	kern.launch_d_kv(tq, tkv, tt, d_o, l, d, d_kv, 0)
	dev.synchronize()
	assert not _bf16_value(d_kv.download()).any()                       # dO = 0, D = 0: no gradient


def test_backward_speed_builds_at_the_size_of_benchmark_config_4(dev):
	"""The attention shape of benchmark config 4 (32768 rows, 16 heads x 128, window 512; here 16 sequences of 2048) on
	the builds bench.py times.  Two size-independent checks: (sequence, head) pairs are independent, so three of them
	are recomputed whole by the dense oracle; and both kernels are homogeneous in dO -- with dO and D multiplied by 4
	every product, sum and rounding is the same up to the exponent, so every output must be exactly 4 times the first
	run's (a lost tile, a race or a stale LDS slot breaks the equality)."""
	t, batch, h, hd, w = 2048, 16, 16, 128, 512
	rows = t * batch
	rng = rng_for("attn-bwd-config4")
	q, kv, sk, sv, temp = _inputs(rng, rows, h, hd)
	d_o_bits = _bf16_bits(rng.standard_normal((rows, h * hd)) * 0.1)
	d_o = _bf16_value(d_o_bits)
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	tq, tkv, tsk, tsv, tt = up(q, X.INT8), up(kv, X.INT8), up(sk, X.INT8), up(sv, X.INT8), up(temp, X.F32)
	out, l = X.Tensor(dev, (rows, h * hd), X.INT8), X.Tensor(dev, (h, rows), X.F32)
	recipes.attn_kernel(dev, h, hd, False).launch(tq, tkv, tsk, tsv, tt, out, l, w, batch)
	k_q, k_kv = recipes.attn_d_q_kernel(dev, h, hd, False), recipes.attn_d_kv_kernel(dev, h, hd, False)
	results = []
	for factor in (1.0, 4.0):
		t_do = up(_bf16_bits(d_o * factor), X.BF16)
		dq, d, dkv = X.Tensor(dev, (rows, h * hd), X.BF16), X.Tensor(dev, (h, rows), X.F32), X.Tensor(dev, (rows, 2 * h * hd), X.BF16)
		k_q.launch_d_q(tq, tkv, tsk, tsv, tt, out, t_do, dq, l, d, w, batch)
		k_kv.launch_d_kv(tq, tkv, tt, t_do, l, d, dkv, w, batch)
		results.append((_bf16_value(dq.download()), d.download().astype(np.float64), _bf16_value(dkv.download())))
	(dq1, d1, dkv1), (dq4, d4, dkv4) = results
	assert np.array_equal(dq4, 4.0 * dq1) and np.array_equal(d4, 4.0 * d1) and np.array_equal(dkv4, 4.0 * dkv1)
	assert np.isfinite(dkv1).all() and np.abs(dkv1).max() > 1e-3
	out_h, l_h = out.download(), l.download().astype(np.float64)
	for seq, head in ((0, 0), (7, 9), (15, 15)):
		r = slice(seq * t, (seq + 1) * t)
		qc, kc = slice(head * hd, (head + 1) * hd), slice(2 * head * hd, 2 * (head + 1) * hd)
		one = (q[r][:, qc], kv[r][:, kc], sk[head:head + 1], sv[head:head + 1], temp[head:head + 1], 1, hd, w)
		want_q, want_d = B.attn_d_q(*one, out_h[r][:, qc], d_o[r][:, qc], l_h[head:head + 1, r])
		_check(_bf16_bits(dq1[r][:, qc]), d1[head:head + 1, r], want_q, want_d, d_o[r][:, qc])
		want_kv = B.attn_d_kv(*one, d_o[r][:, qc], l_h[head:head + 1, r], d1[head:head + 1, r])
		terms = _term_magnitudes(q[r][:, qc], kv[r][:, kc], sk[head:head + 1], sv[head:head + 1], temp[head:head + 1], 1, hd, w,
		                         d_o[r][:, qc], l_h[head:head + 1, r], d1[head:head + 1, r])
		_check_kv(_bf16_bits(dkv1[r][:, kc]), want_kv, terms, 1, hd)


def test_backward_launches_are_repeatable_and_long_walks_are_homogeneous(dev):
	"""One 16384-token sequence with a 4096-key window (the window of benchmark config 5: 133 query tiles per key block,
	129 key tiles per query block), 4 heads x 128, speed builds.  Launching twice gives the same bytes (overhanging
	blocks store the same values, no accumulation order depends on timing), and dO and D times 4 give exactly 4 times
	every output."""
	t, h, hd, w = 16384, 4, 128, 4096
	rng = rng_for("attn-bwd-long")
	q, kv, sk, sv, temp = _inputs(rng, t, h, hd)
	d_o = _bf16_value(_bf16_bits(rng.standard_normal((t, h * hd)) * 0.05))
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	tq, tkv, tsk, tsv, tt = up(q, X.INT8), up(kv, X.INT8), up(sk, X.INT8), up(sv, X.INT8), up(temp, X.F32)
	out, l = X.Tensor(dev, (t, h * hd), X.INT8), X.Tensor(dev, (h, t), X.F32)
	recipes.attn_kernel(dev, h, hd, False).launch(tq, tkv, tsk, tsv, tt, out, l, w, 1)
	k_q, k_kv = recipes.attn_d_q_kernel(dev, h, hd, False), recipes.attn_d_kv_kernel(dev, h, hd, False)
	runs = []
	for factor in (1.0, 1.0, 4.0):
		t_do = up(_bf16_bits(d_o * factor), X.BF16)
		dq, d, dkv = X.Tensor(dev, (t, h * hd), X.BF16), X.Tensor(dev, (h, t), X.F32), X.Tensor(dev, (t, 2 * h * hd), X.BF16)
		k_q.launch_d_q(tq, tkv, tsk, tsv, tt, out, t_do, dq, l, d, w, 1)
		k_kv.launch_d_kv(tq, tkv, tt, t_do, l, d, dkv, w, 1)
		runs.append((dq.download(), d.download(), dkv.download()))
	for a, b in zip(runs[0], runs[1]):
		assert np.array_equal(a, b)
	dq1, d1, dkv1 = _bf16_value(runs[0][0]), runs[0][1].astype(np.float64), _bf16_value(runs[0][2])
	dq4, d4, dkv4 = _bf16_value(runs[2][0]), runs[2][1].astype(np.float64), _bf16_value(runs[2][2])
	assert np.array_equal(dq4, 4.0 * dq1) and np.array_equal(d4, 4.0 * d1) and np.array_equal(dkv4, 4.0 * dkv1)
	assert np.isfinite(dkv1).all() and np.abs(dkv1).max() > 1e-4 and np.abs(dq1).max() > 1e-4
	assert not dq1[0].any() and not dkv1[t - 1].any()
