"""CPU pins of the oracle's building blocks (no GPU): conversions, the deterministic transcendental
definitions, the integer GEMM, every epilogue against the float64 closed forms of the reference's
torch oracle, the attention recurrence against the dense float64 softmax, decode and rms_norm."""
import math

import numpy as np
import pytest
import torch

from oracle import dense as D
from oracle import strict as S


def _rng(seed):
	return np.random.default_rng(seed)


# ---------------------------------------------------------------- conversions

def test_fixedi8_closed_form_and_ties():
	x = np.concatenate([_rng(1).standard_normal(200000) * 60, np.arange(-130, 131) + 0.5, np.arange(-130, 131.0),
	                    [1e9, -1e9, 126.5, 127.49, -127.5]]).astype(np.float32)
	want = np.clip(np.rint(x.astype(np.float64)), -127, 127).astype(np.int8)      # rint = round half to even
	assert np.array_equal(S.f32_to_fixedi8(x), want)


def test_e4m3_decode_matches_ocp_e4m3fn_for_every_code_the_reference_emits():
	codes = np.array([c for c in range(256) if (c & 0x7F) >= 0x08 and (c & 0x7F) != 0x7F] + [0], dtype=np.uint8)
	ours = S.e4m3_to_f32(codes)
	ocp = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
	assert np.array_equal(ours, ocp)
	assert np.array_equal(S.f32_to_e4m3(ours), codes)                              # round trip


def test_e4m3_encode_is_round_half_away_with_flush_and_saturation():
	x = (_rng(2).standard_normal(2_000_000) * np.exp(_rng(3).standard_normal(2_000_000) * 2)).astype(np.float32)
	ours = S.e4m3_to_f32(S.f32_to_e4m3(x))
	ftz = np.where(np.abs(x) < (1 + 15 / 16) * 2.0 ** -7, 0, x).astype(np.float32)
	rne = torch.from_numpy(np.clip(ftz, -448, 448)).to(torch.float8_e4m3fn).to(torch.float32).numpy()
	neq = ours != rne
	# they may differ only on exact ties, where ours is the neighbour further from zero
	assert np.mean(neq) < 1e-5
	assert np.all(np.abs(ours[neq]) > np.abs(rne[neq]))
	assert np.all(np.abs(np.abs(ours[neq]) - np.abs(x[neq])) == np.abs(np.abs(rne[neq]) - np.abs(x[neq])))
	# thresholds (cuda/utils_b8.cuh:636-647)
	edge = np.array([1.9375 * 2 ** -7, np.nextafter(np.float32(1.9375 * 2 ** -7), 0), 448.0, 449.0, 1e9, -1e9, -0.001], np.float32)
	assert S.f32_to_e4m3(edge).tolist() == [0x08, 0x00, 0x7E, 0x7E, 0x7E, 0xFE, 0x00]
	# hand-made ties round away from zero: 0.53125 is halfway between 0.5 and 0.5625
	assert S.e4m3_to_f32(S.f32_to_e4m3(np.array([0.53125, -0.53125], np.float32))).tolist() == [0.5625, -0.5625]
	# monotone over a fine sweep
	sweep = np.linspace(-500, 500, 400001).astype(np.float32)
	assert np.all(np.diff(S.e4m3_to_f32(S.f32_to_e4m3(sweep))) >= 0)


# ---------------------------------------------------------------- transcendental definitions

def _ulps(approx, exact):
	ulp = np.spacing(np.abs(exact.astype(np.float32))).astype(np.float64)
	return np.max(np.abs(approx.astype(np.float64) - exact) / ulp)


def test_sfu_definitions_against_libm():
	r = _rng(4)
	x = np.concatenate([-r.random(2_000_000) * 124.9, r.random(100_000) * 30, -r.random(500_000)]).astype(np.float32)
	assert _ulps(S.sfu("ex2", x), np.exp2(x.astype(np.float64))) < 1.0
	pos = np.clip(np.exp(r.standard_normal(2_000_000) * 15), 1e-30, 1e30).astype(np.float32)
	assert _ulps(S.sfu("lg2", pos), np.log2(pos.astype(np.float64))) < 2.0
	assert _ulps(S.sfu("rcp", pos), 1.0 / pos.astype(np.float64)) < 0.51
	assert _ulps(S.sfu("rsq", pos), 1.0 / np.sqrt(pos.astype(np.float64))) < 2.0
	t = (r.standard_normal(2_000_000) * 3).astype(np.float32)
	assert np.max(np.abs(S.sfu("tanh", t) - np.tanh(t.astype(np.float64)))) < 2e-7
	# exact special values the recurrences rely on
	assert S.sfu("ex2", np.array([0.0, -1.0, 3.0, -np.inf, -200.0], np.float32)).tolist() == [1.0, 0.5, 8.0, 0.0, 0.0]
	assert S.sfu("lg2", np.array([1.0, 2.0, 0.25, 1024.0], np.float32)).tolist() == [0.0, 1.0, -2.0, 10.0]
	assert S.sfu("tanh", np.array([0.0, 50.0, -50.0], np.float32)).tolist() == [0.0, 1.0, -1.0]


def test_constexpr_sqrt_is_the_correctly_rounded_one_where_it_matters():
	for v in (2.0, 2048.0, 32.0, 128.0, (1 / math.sqrt(2048) / 64) ** 2 * 2 / math.pi):
		assert abs(S.constexpr_sqrt(v) - math.sqrt(v)) <= np.spacing(math.sqrt(v))
		assert abs(S.constexpr_inv_sqrt(v) - 1 / math.sqrt(v)) <= np.spacing(1 / math.sqrt(v))
		assert np.float32(S.constexpr_inv_sqrt(v)) == np.float32(1 / math.sqrt(v))


# ---------------------------------------------------------------- GEMM + epilogues

def test_gemm_i32_against_int64_matmul_and_brute_force():
	r = _rng(5)
	a = r.integers(-127, 128, (37, 256), dtype=np.int8)
	b = r.integers(-127, 128, (29, 256), dtype=np.int8)
	assert np.array_equal(S.gemm_i32(a, b).astype(np.int64), a.astype(np.int64) @ b.astype(np.int64).T)
	tiny = S.gemm_i32(a[:2, :3].copy(), b[:2, :3].copy())
	for i in range(2):
		for j in range(2):
			assert tiny[i, j] == sum(int(a[i, k]) * int(b[j, k]) for k in range(3))


def _acc(seed, m, n, k=2048):
	r = _rng(seed)
	return (r.standard_normal((m, n)) * 64.0 * math.sqrt(k)).astype(np.int32)      # what N(0,1) operands give


def test_scale_epilogue_against_float64():
	acc = _acc(6, 128, 512)
	inp = 1 / math.sqrt(2048) / 64
	got = S.epilogue_scale(acc, inp, 8.0).astype(np.int32)
	want = D.quantize_i8_codes(acc.astype(np.float64) * inp)
	d = np.abs(got - want)
	assert d.max() <= 1 and np.mean(d > 0) < 1e-4


def test_geglu_epilogue_against_float64():
	acc = _acc(7, 256, 1024)
	inp = 1 / math.sqrt(2048) / 64
	got = S.e4m3_to_f32(S.epilogue_geglu(acc, inp, 1.0)).astype(np.float64)
	want = D.quantize_e4m3(D.geglu(acc.astype(np.float64) * inp))
	big = np.maximum(np.abs(got), np.abs(want))
	rel = np.abs(got - want) / np.where(big == 0, 1, big)
	assert np.mean(got != want) < 1e-3
	assert np.all((rel <= 0.126) | (big <= 2.0 ** -6))
	# FixedI8 store with out_scale 8 is the same value on the other grid
	got8 = S.epilogue_geglu(acc, inp, 8.0, S.STORE_I8).astype(np.int32)
	want8 = D.quantize_i8_codes(D.geglu(acc.astype(np.float64) * inp))
	assert np.abs(got8 - want8).max() <= 1 and np.mean(got8 != want8) < 1e-3


def test_dequant_epilogue_against_torch_bf16_and_tanh_gelu():
	"""The run-time-scale writer: bf16 rounding against torch's float32 -> bfloat16 cast (a library routine,
	round to nearest even), the plain form against the same products formed in float32 by torch, and the
	GeGLU form against torch's tanh-approximated gelu in float64 (within bf16 resolution)."""
	rng = np.random.default_rng(31)
	m, n = 48, 64
	acc = rng.integers(-200000, 200000, (m, n), dtype=np.int32)
	rs = (rng.random(m) * 1e-3 + 1e-4).astype(np.float32)
	cs = (rng.random(n) * 1e-2 + 1e-3).astype(np.float32)
	got = S.epilogue_dequant(acc, rs, cs, False)
	prod = (torch.from_numpy(acc).to(torch.float32) * torch.from_numpy(rs)[:, None]) * torch.from_numpy(cs)[None, :]
	want = prod.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
	assert np.array_equal(got, want)
	# exact ties round to even: 1 + 2^-8 -> 1.0, 1 + 3 * 2^-8 -> 1 + 2^-6
	ties = np.array([[1 << 24 | 1 << 16, 1 << 24 | 3 << 16]], dtype=np.int32)        # as integers: 2^24 + 2^16 k
	one = np.array([2.0 ** -24], np.float32)
	bits = S.epilogue_dequant(ties, one, np.ones(2, np.float32), False)
	assert bits.tolist() == [[0x3F80, 0x3F82]]
	gg = S.epilogue_dequant(acc, rs, cs, True)
	x = prod.to(torch.float64)
	ref = torch.nn.functional.gelu(x[:, 0::2], approximate="tanh") * x[:, 1::2]
	gg_f = (gg.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	assert np.allclose(gg_f, ref.numpy(), rtol=2.0 ** -7, atol=1e-6 * float(ref.abs().max()))


def test_residual_epilogue_against_float64_and_identities():
	acc = _acc(8, 256, 1024)
	r = _rng(9)
	res = S.f32_to_fixedi8((r.standard_normal((256, 512)) * 8).astype(np.float32))
	inp = 1 / math.sqrt(2048) / 64
	got = S.e4m3_to_f32(S.epilogue_residual(acc, res, inp, 1.0)).astype(np.float64)
	want = D.quantize_e4m3(D.gated_residual(res / 8.0, acc.astype(np.float64) * inp))
	big = np.maximum(np.abs(got), np.abs(want))
	rel = np.abs(got - want) / np.where(big == 0, 1, big)
	assert np.mean(got != want) < 2e-3
	assert np.all((rel <= 0.126) | (big <= 2.0 ** -6))
	# docs/design.md:6-7 -- at gate 0 both weights are one half: out = x/2 + y/2
	z = np.zeros((1, 2), np.int32)
	z[0, 1] = 12345
	one = S.e4m3_to_f32(S.epilogue_residual(z, np.array([[40]], np.int8), inp, 1.0))
	assert one[0, 0] == S.e4m3_to_f32(S.f32_to_e4m3(np.array([0.5 * 5.0 + 0.5 * 12345 * inp], np.float32)))[0]
	x = np.linspace(-6, 6, 1001)
	assert np.allclose(D.sigmoid_base4(x) + D.sigmoid_base4(-x), 1.0)
	assert np.allclose(D.softplus_base4(x) - D.softplus_base4(-x), x)
	assert np.allclose(D.gelu(x) - D.gelu(-x), x)


def test_l2norm_epilogue_against_float64_and_order():
	hd = 32
	acc = _acc(10, 128, 512)
	inp = 1 / math.sqrt(2048) / 64
	kv, rrms = S.epilogue_l2norm(acc, hd, 2.0 ** -70, inp, 8.0)
	raw = acc.astype(np.float64).reshape(128, 512 // (2 * hd), 2 * hd)
	k, rr = D.rms_norm(raw[..., :hd], 2.0 ** -70)
	want = D.quantize_i8_codes(np.concatenate((k, raw[..., hd:] * inp), axis=2)).reshape(128, 512)
	d = np.abs(kv.astype(np.int32) - want)
	assert d.max() <= 1 and np.mean(d > 0) < 1e-4
	assert np.allclose(rrms, rr[..., 0] * 8.0, rtol=3e-7)               # scale = 8 * sqrt(hd) / |acc|
	# invariant: sum of squares of the K codes is 64 * hd
	ks = kv.reshape(128, -1, 2, hd)[:, :, 0, :].astype(np.float64)
	assert np.allclose((ks ** 2).sum(-1), 64.0 * hd, rtol=0.05)
	# the summation order is part of the definition: four interleaved partial sums
	a = acc[0, :hd].astype(np.float32)
	s = [np.float32(0)] * 4
	for dd in range(hd):
		q = (dd % 8) // 2
		s[q] = np.float32(np.float64(a[dd]) * np.float64(a[dd]) + np.float64(s[q]))      # fma: one rounding
	total = np.float32(np.float32(s[0] + s[1]) + np.float32(s[2] + s[3])) + np.float32(2.0 ** -70)
	want_scale = S.sfu("rsq", np.array([total], np.float32))[0] * np.float32(8.0 * math.sqrt(hd))
	assert rrms[0, 0] == np.float32(want_scale)


@pytest.mark.parametrize("hd", [32, 64, 128])
def test_learned_scale_q_writer(hd):
	"""cuda/qkvg_fwd_i8.cuh:145-219: L2 norm over every head of q, then a bf16 scale per column.  Pinned by (i) reduction to
	the K halves of the L2-norm writer when every scale is 1 -- codes and rrms bit for bit --, (ii) the float64 closed form
	q = x / sqrt(mean(x^2)) * scale on the FixedI8 grid, (iii) the scales being column-wise and applied AFTER the norm."""
	m, n = 64, 512
	acc = _acc(11 + hd, m, n)
	ones = np.full(n, 0x3F80, np.uint16)                           # bf16 1.0
	q1, r1 = S.epilogue_qnorm(acc, hd, 2.0 ** -70, 8.0, ones, want_rrms=True)
	kvacc = np.zeros((m, 2 * n), np.int32)
	kvacc.reshape(m, n // hd, 2, hd)[:, :, 0, :] = acc.reshape(m, n // hd, hd)
	kv, rr = S.epilogue_l2norm(kvacc, hd, 2.0 ** -70, 1.0, 8.0)
	assert np.array_equal(kv.reshape(m, n // hd, 2, hd)[:, :, 0, :], q1.reshape(m, n // hd, hd))
	assert np.array_equal(rr.view(np.uint32), r1.view(np.uint32))
	# float64 closed form with scales that differ per column (exactly representable in bf16: multiples of 1/64 in [0.5, 1.5))
	rng = np.random.default_rng(5)
	scale = (32 + rng.integers(0, 64, n)) / 64.0
	dyn = (scale.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
	assert np.array_equal((dyn.astype(np.uint32) << 16).view(np.float32), scale.astype(np.float32))
	got = S.epilogue_qnorm(acc, hd, 0.0, 8.0, dyn)
	x = acc.astype(np.float64).reshape(m, n // hd, hd)
	want = (x / np.sqrt((x * x).mean(-1, keepdims=True))).reshape(m, n) * scale * 8.0
	want_codes = np.clip(np.rint(want), -127, 127)
	d = np.abs(got.astype(np.float64) - want_codes)
	assert d.max() <= 1 and np.mean(d > 0) < 1e-3
	assert np.abs(got - want).max() <= 0.5 + 1e-3                  # each code within half a step of the exact value
	# a rolled scale vector or scales applied per head instead of per column give another answer
	assert not np.array_equal(S.epilogue_qnorm(acc, hd, 0.0, 8.0, np.roll(dyn, 1)), got)
	per_head = np.repeat(dyn[::hd], hd)
	assert not np.array_equal(S.epilogue_qnorm(acc, hd, 0.0, 8.0, per_head), got)
	# eps only matters for an all-zero head: rsq(0) would be infinite, rsq(eps) * 0 is 0
	z = acc.copy()
	z[3, :hd] = 0
	assert not S.epilogue_qnorm(z, hd, 2.0 ** -70, 8.0, dyn)[3, :hd].any()
	# the factor of the old writer's vanished base class (1 / sqrt(MODEL_DIM), cuda/qkvg_fwd_i8.cuh:151-159) is an
	# explicit argument: post_scale = 1 is the default above; a power of two moves every unsaturated code exactly;
	# 1 / sqrt(K) follows the float64 closed form times that factor
	assert np.array_equal(S.epilogue_qnorm(acc, hd, 0.0, 8.0, dyn, post_scale=1.0), got)
	half = S.epilogue_qnorm(acc, hd, 0.0, 4.0, dyn)                      # out_scale 4 = out_scale 8 times 0.5 ...
	assert np.array_equal(S.epilogue_qnorm(acc, hd, 0.0, 8.0, dyn, post_scale=0.5)[np.abs(got) < 127], half[np.abs(got) < 127])
	ps = 1.0 / np.sqrt(np.float64(2048.0))
	scaled = S.epilogue_qnorm(acc, hd, 0.0, 8.0 * 32.0, dyn, post_scale=ps)   # (out_scale 256 keeps the codes off zero)
	want_s = want * 32.0 * ps
	assert np.abs(scaled - np.clip(want_s, -127, 127)).max() <= 0.5 + 1e-3
	assert len(np.unique(scaled)) > 20


def test_gemm_f32_seq_against_float64():
	r = _rng(11)
	a = S.f32_to_e4m3((r.standard_normal((32, 512)) * 0.7).astype(np.float32))
	b = r.integers(-127, 128, (48, 512), dtype=np.int8)
	got = S.gemm_f32_seq(a, True, b, False)
	want = S.e4m3_to_f32(a).astype(np.float64) @ b.astype(np.float64).T
	assert np.max(np.abs(got - want)) <= 512 * 2.0 ** -24 * np.max(np.abs(want)) * 4


# ---------------------------------------------------------------- attention, decode, rms_norm

def _attn_inputs(r, t, h, hd):
	q = S.f32_to_fixedi8((r.standard_normal((t, h * hd)) * 8).astype(np.float32))
	k = r.standard_normal((t, h, hd))
	k /= np.sqrt((k * k).mean(-1, keepdims=True))
	v = r.standard_normal((t, h, hd))
	kv = S.f32_to_fixedi8((np.concatenate((k, v), 2).reshape(t, -1) * 8).astype(np.float32))
	sk = S.f32_to_fixedi8((r.standard_normal((h, hd)) * 8).astype(np.float32))
	sv = S.f32_to_fixedi8((r.standard_normal((h, hd)) * 8).astype(np.float32))
	temp = (0.5 + r.random(h)).astype(np.float32)
	return q, kv, sk, sv, temp


@pytest.mark.parametrize("t,h,hd,w", [(256, 2, 32, 0), (320, 2, 64, 64), (256, 1, 128, 16)])
def test_attention_against_dense_float64(t, h, hd, w):
	q, kv, sk, sv, temp = _attn_inputs(_rng(12), t, h, hd)
	out, l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	kvr = kv.reshape(t, h, 2 * hd) / 8.0
	o, ld = D.attn(q.reshape(t, h, hd) / 8.0, kvr[..., :hd], kvr[..., hd:], sk / 8.0, sv / 8.0, temp.astype(np.float64), w, 255.0)
	d = np.abs(D.quantize_i8_codes(o).reshape(t, -1) - out.astype(np.int32))
	assert d.max() <= 1 and np.mean(d > 0) < 0.03           # same probabilities grid (1/255): rounding noise only
	assert np.max(np.abs(ld.T - l)) < 5e-5
	# against the reference oracle's own 1/8-step probabilities the picture of expected.txt:65-71 appears
	o8, _ = D.attn(q.reshape(t, h, hd) / 8.0, kvr[..., :hd], kvr[..., hd:], sk / 8.0, sv / 8.0, temp.astype(np.float64), w, 8.0)
	d8 = np.abs(D.quantize_i8_codes(o8).reshape(t, -1) - out.astype(np.int32))
	assert d8.max() <= 6 and 0.1 < np.mean(d8 > 0) < 0.5


def test_attention_closed_form_cases():
	t, h, hd = 128, 2, 32
	q, kv, sk, sv, temp = _attn_inputs(_rng(13), t, h, hd)
	out, l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, 0)
	# query 0 sees only the sink: output = sink_v, L = log2(255) + sink score
	assert np.array_equal(out[0].reshape(h, hd), sv)
	s_sink = (q[0].reshape(h, hd).astype(np.int64) * sk).sum(-1) * (1 / math.sqrt(hd) / 64) * math.log2(4.0) * temp
	assert np.allclose(l[:, 0], math.log2(255.0) + s_sink, atol=1e-4)
	# a window that covers everything is no window; windows are rounded up to multiples of 16
	assert np.array_equal(out, S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, 128)[0])
	assert np.array_equal(S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, 17)[0], S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, 32)[0])
	# constant V gives V back
	kv2 = kv.reshape(t, h, 2, hd).copy()
	kv2[:, :, 1] = 24
	outc, _ = S.attn_fwd_i8(q, kv2.reshape(t, -1), sk, np.full_like(sv, 24), temp, h, hd, 32)
	assert np.all(outc == 24)
	# zero head temperature: uniform weights over the sink and the min(i, W) visible keys
	w = 16
	outu, _ = S.attn_fwd_i8(q, kv, sk, sv, np.zeros(h, np.float32), h, hd, w)
	v = kv.reshape(t, h, 2, hd)[:, :, 1].astype(np.float64)
	for i in (0, 5, 40, 127):
		lo = max(0, i - w)
		mean = (sv + v[lo:i].sum(0)) / (1 + i - lo)
		assert np.abs(outu[i].reshape(h, hd) - mean).max() <= 0.5 + 1e-6


def test_decode_is_the_prefill_row():
	h, hd, cap, w = 2, 32, 64, 32
	q, kv, sk, sv, temp = _attn_inputs(_rng(14), 3 * cap, h, hd)
	cache = kv.reshape(3, cap, -1)
	lens = np.array([0, 37, cap], np.uint32)
	out, l = S.attn_decode_i8(q[:3], cache, lens, sk, sv, temp, h, hd, w)
	for s, p in enumerate(lens):
		p = int(p)
		qq = np.zeros((p + 1, h * hd), np.int8)
		qq[p] = q[s]
		kk = np.zeros((p + 1, 2 * h * hd), np.int8)
		kk[:p] = cache[s, :p]
		po, pl = S.attn_fwd_i8(qq, kk, sk, sv, temp, h, hd, w)
		assert np.array_equal(po[p], out[s]) and np.array_equal(pl[:, p], l[s])


def test_rms_norm_against_float64_and_legacy_known_answer():
	r = _rng(15)
	x = S.f32_to_e4m3((r.standard_normal((16, 1024)) * 2).astype(np.float32))
	got = S.rms_norm(x, 2.0 ** -70).astype(np.int32)
	xv = S.e4m3_to_f32(x).astype(np.float64)
	want = D.quantize_i8_codes(D.rms_norm(xv, 2.0 ** -70)[0])
	d = np.abs(got - want)
	assert d.max() <= 1 and np.mean(d > 0) < 1e-3
	# known answer of the reference's legacy unit test (src_old/nn/fragments/tests/test_rms_norm.rs:28-40)
	inp = np.array([[-1.2719, -0.6884, -0.6477, -1.3343, -1.7648], [-1.9440, 0.9989, 2.8260, -0.3503, -0.5406],
	                [0.1619, -0.9744, -0.6539, 1.9764, 0.7423], [0.0689, 1.1983, 0.0077, -0.6580, -0.4917]])
	exp = np.array([[-1.0451, -0.5656, -0.5322, -1.0963, -1.4501], [-1.1974, 0.6153, 1.7407, -0.2158, -0.3330],
	                [0.1495, -0.9000, -0.6040, 1.8255, 0.6856], [0.1059, 1.8422, 0.0118, -1.0116, -0.7559]])
	assert np.allclose(D.rms_norm(inp, 1e-5)[0], exp, atol=1e-4)


# ---------------------------------------------------------------- row-scaled attention (own definition)

def bf16_bits_to_f64(bits: np.ndarray) -> np.ndarray:
	return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def _row_scaled_inputs(r, t, h, hd):
	"""q, k, v ~ N(0, 1) with a per-(row, head) spread of magnitudes, int8 codes at scale absmax / 127."""
	spread = np.exp(r.normal(0.0, 0.7, (3, t, h, 1)))
	qc, qs = D.quantize_rows(r.standard_normal((t, h, hd)) * spread[0])
	kc, ks = D.quantize_rows(r.standard_normal((t, h, hd)) * spread[1])
	vc, vs = D.quantize_rows(r.standard_normal((t, h, hd)) * spread[2])
	sk = S.f32_to_fixedi8((r.standard_normal((h, hd)) * 8).astype(np.float32))
	sv = S.f32_to_fixedi8((r.standard_normal((h, hd)) * 8).astype(np.float32))
	temp = (0.5 + r.random(h)).astype(np.float32)
	kv = np.concatenate((kc, vc), axis=2).reshape(t, -1)
	head_major = lambda a: np.ascontiguousarray(a.T)          # the scale matrices are [H, T], like L
	return qc.reshape(t, -1), kv, head_major(qs), head_major(ks), head_major(vs), sk, sv, temp


def test_row_scaled_attention_reduces_to_the_reference_mode_at_scale_one_eighth():
	t, h, hd, w = 192, 2, 64, 48
	q, kv, sk, sv, temp = _attn_inputs(_rng(31), t, h, hd)
	ref_out, ref_l = S.attn_fwd_i8(q, kv, sk, sv, temp, h, hd, w)
	eighth = np.full((h, t), 0.125, np.float32)
	ones = np.ones((h, t), np.float32)
	out, l = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, eighth, eighth, ones, np.ones(h), np.ones(h))
	assert np.array_equal(out, ref_out) and np.array_equal(l, ref_l)
	# a power of two moves freely between the query scale and the head temperature (the key scale has no
	# such partner: the sink key keeps its fixed scale of 1/8)
	out2, l2 = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp * 4, h, hd, w, eighth / 4, eighth, ones, np.ones(h), np.ones(h))
	assert np.array_equal(out2, ref_out) and np.array_equal(l2, ref_l)
	# the bf16 store holds the same values before their rounding to codes
	outb, _ = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, eighth, eighth, ones, np.ones(h), np.full(h, 0.125),
	                                   out_bf16=True)
	unclamped = np.abs(ref_out) < 127
	assert np.all(np.abs(bf16_bits_to_f64(outb) * 8.0 - ref_out)[unclamped] <= 0.5 + 127 * 2.0 ** -8)


@pytest.mark.parametrize("t,h,hd,w", [(256, 2, 64, 64), (192, 3, 32, 0), (128, 1, 128, 32)])
def test_row_scaled_attention_against_dense_float64(t, h, hd, w):
	from x17ai_amd.recipes import attn_row_scale_operands
	from x17ai_amd.api import BF16
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(_rng(32), t, h, hd)
	v_weight, sink_w, out_scale = attn_row_scale_operands(vs, BF16)
	assert v_weight.max() == 1.0 and v_weight.min() > 0
	out, _ = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, qs, ks, v_weight, sink_w, out_scale, out_bf16=True)
	got = bf16_bits_to_f64(out).reshape(t, h, hd)
	kvr = kv.reshape(t, h, 2, hd)
	for hh in range(h):
		args = (q.reshape(t, h, hd)[:, hh], kvr[:, hh, 0], kvr[:, hh, 1], qs[hh], ks[hh], vs[hh],
		        sk[hh] / 8.0, sv[hh] / 8.0, float(temp[hh]), w)
		same_grid = D.attn_one_head_row_scaled(*args, quantize_p=True)
		exact = D.attn_one_head_row_scaled(*args, quantize_p=False)
		scale = np.abs(exact).max()
		# same probability grid: bf16 rounding of the output (2^-9 relative) everywhere, except where a
		# probability sits on a rounding boundary and goes the other way (one step of one value row)
		err = np.abs(got[:, hh] - same_grid) / scale
		assert np.mean(err > 2.0 ** -8) < 0.03 and err.max() < 0.03, (np.mean(err > 2.0 ** -8), err.max())
		# exact softmax: what 8-bit probabilities cost
		err = np.abs(got[:, hh] - exact) / scale
		assert np.sqrt(np.mean(err ** 2)) < 0.01 and err.max() < 0.06, (np.sqrt(np.mean(err ** 2)), err.max())


def test_row_scaled_decode_is_the_row_scaled_prefill_row():
	from x17ai_amd.recipes import attn_row_scale_operands
	from x17ai_amd.api import BF16
	t, h, hd, w = 128, 2, 64, 32
	q, kv, qs, ks, vs, sk, sv, temp = _row_scaled_inputs(_rng(33), t, h, hd)
	vw, sink_w, out_scale = attn_row_scale_operands(vs, BF16)
	pre, pre_l = S.attn_fwd_i8_row_scaled(q, kv, sk, sv, temp, h, hd, w, qs, ks, vw, sink_w, out_scale, out_bf16=True)
	for p in (0, 1, 17, 100):
		cap = 112                                   # rows from p on are never read: poison them
		cache = np.full((1, cap, 2 * h * hd), 99, np.int8)
		cache[0, :p] = kv[:p]
		kc = np.full((1, h, cap), np.nan, np.float32)
		kc[0, :, :p] = ks[:, :p]
		vc = np.full((1, h, cap), np.nan, np.float32)
		vc[0, :, :p] = vw[:, :p]
		out, l = S.attn_decode_i8_row_scaled(q[p:p + 1], cache, np.array([p], np.uint32), sk, sv, temp, h, hd, w,
		                                     qs[:, p][None, :], kc, vc, sink_w, out_scale, out_bf16=True)
		assert np.array_equal(out[0], pre[p]) and np.array_equal(l[0], pre_l[:, p])
