"""The speed builds bench.py times outside the config 4 chain, each against its strict build at the size it is timed at.

The strict builds of these shapes are held against the CPU oracle by tests/test_gpu_fullsize.py (sampled heads,
sequences and rows); here the hardware-transcendental builds run on the same inputs and every output element is
compared with the strict build's:
  decode()             config 5 decode, 64 sequences x 4096 cached positions, 32 heads x 128: ragged lengths, flat-score
                       sequences and the dense case (an all-zero query: every probability is 255), FixedI8 out + L
  decode_row_scaled()  the same cache with one scale per (row, head) of k and v, bf16 out
  prefill_row_scaled() config 5 prefill, 65536 tokens, window 4096, per-(row, head) scales, bf16 out, whole output
  dequant_pair()       config 2 in its literal form: per-token x per-channel scales, GeGLU, bf16 out (both GEMMs)
report() runs all four; tests/golden/make_fast_builds_report.py writes its result to
tests/golden/fast_builds_vs_strict.json and tests/test_gpu_fullsize.py asserts the bounds.
"""
from __future__ import annotations

import math

import numpy as np

import x17ai_amd as X
from x17ai_amd import recipes
from oracle import strict as S
from tests.config4_chain import _i8_diff
from tests.gpu_common import i8_codes, rng_for

T5, H5, HD5, W5 = 65536, 32, 128, 4096
S5, CAP5 = 64, 4096


def _up(dev, arr, dtype):
	return X.Tensor.from_numpy(dev, arr, dtype)


def bf16_diff(a, b, scale_rows=None):
	"""Two bf16 tensors (uint16 bit patterns) as real numbers: count of differing patterns, of elements further
	apart than one bf16 step of the larger magnitude AND than `floor` (1/255 of the tensor's rms: the weight of one
	8-bit probability step), max-abs and relative-L2 difference."""
	av = (a.reshape(-1).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	bv = (b.reshape(-1).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
	d = np.abs(av - bv)
	rms = math.sqrt(float(np.mean(bv * bv)))
	floor = rms / 255.0
	big = np.maximum(np.abs(av), np.abs(bv))
	beyond = (d > big * 2.0 ** -7) & (d > floor)
	return {"elements": int(av.size), "mismatched": int(np.count_nonzero(a.reshape(-1) != b.reshape(-1))),
	        "frac_mismatched": float(np.mean(a.reshape(-1) != b.reshape(-1))),
	        "beyond_one_step_and_floor": int(np.count_nonzero(beyond)), "rms": rms,
	        "max_abs": float(d.max()), "rel_l2": float(np.linalg.norm(av - bv) / np.linalg.norm(bv))}


def _attn_inputs(rng, rows, h, hd):
	q = i8_codes(rng, (rows, h * hd))
	k = rng.standard_normal((rows, h, hd), dtype=np.float32)
	k /= np.sqrt((k * k).mean(-1, keepdims=True))
	v = rng.standard_normal((rows, h, hd), dtype=np.float32) * 1.3
	kv = S.f32_to_fixedi8((np.concatenate((k, v), axis=2).reshape(rows, 2 * h * hd) * 8).astype(np.float32))
	sk = rng.standard_normal((h, hd))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	return q, kv, S.f32_to_fixedi8((sk * 8).astype(np.float32)), i8_codes(rng, (h, hd), 1.3), (0.5 + rng.random(h)).astype(np.float32)


def _scales(rng, shape):
	return (0.125 * (0.5 + rng.random(shape))).astype(np.float32)


def _decode_case(rng):
	q, _, sk, sv, temp = _attn_inputs(rng, S5, H5, HD5)
	cache = np.empty((S5, CAP5, 2 * H5 * HD5), np.int8)
	for i in range(S5):
		cache[i] = i8_codes(rng, (CAP5, 2 * H5 * HD5))
	lens = rng.integers(1, CAP5 + 1, S5).astype(np.uint32)
	lens[:8] = [0, 1, 15, 16, 17, 4095, 4096, 2048]
	q[8:16] = q[8:16] // 16                       # flat score distributions: nearly every probability is nonzero
	q[16:24] = 0                                  # the dense case: every probability is 255, every row is read
	lens[8:24] = [4096, 4096, 4001, 3000, 2049, 1000, 4096, 333, 4096, 4096, 4095, 4081, 17, 2048, 4096, 4096]
	return q, cache, lens, sk, sv, temp


def decode(dev):
	rng = rng_for("fast-builds-decode")
	q, cache, lens, sk, sv, temp = _decode_case(rng)
	args = (_up(dev, q, X.INT8), _up(dev, cache, X.INT8), _up(dev, lens.view(np.float32), X.F32),
	        _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32))
	got = {}
	for strict in (True, False):
		out, l = X.Tensor(dev, (S5, H5 * HD5), X.INT8), X.Tensor(dev, (S5, H5), X.F32)
		recipes.attn_decode_kernel(dev, H5, HD5, CAP5, strict).launch(*args, out, l, W5)
		got[strict] = (out.download(), l.download())
	rep = _i8_diff(got[False][0], got[True][0])
	rep["l_max_abs"] = float(np.abs(got[False][1].astype(np.float64) - got[True][1]).max())
	dense = _i8_diff(got[False][0][16:24], got[True][0][16:24])
	rep["dense_sequences_mismatched"] = dense["mismatched"]
	return rep


def decode_row_scaled(dev):
	rng = rng_for("fast-builds-decode-rows")
	q, cache, lens, sk, sv, temp = _decode_case(rng)
	qs, ks, vs = _scales(rng, (S5, H5)), _scales(rng, (S5, H5, CAP5)), _scales(rng, (S5, H5, CAP5))
	vw, sw, osc = recipes.attn_row_scale_operands(vs, X.BF16)
	args = (_up(dev, q, X.INT8), _up(dev, cache, X.INT8), _up(dev, lens.view(np.float32), X.F32),
	        _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32))
	sc = (_up(dev, qs, X.F32), _up(dev, ks, X.F32), _up(dev, vw, X.F32), _up(dev, sw, X.F32), _up(dev, osc, X.F32))
	got = {}
	for strict in (True, False):
		out, l = X.Tensor(dev, (S5, H5 * HD5), X.BF16), X.Tensor(dev, (S5, H5), X.F32)
		recipes.attn_decode_row_scaled_kernel(dev, H5, HD5, CAP5, X.BF16, strict).launch_row_scaled(*args, out, l, W5, *sc)
		got[strict] = (out.download(), l.download())
	rep = bf16_diff(got[False][0], got[True][0])
	rep["l_max_abs"] = float(np.abs(got[False][1].astype(np.float64) - got[True][1]).max())
	return rep


def prefill_row_scaled(dev):
	rng = rng_for("fast-builds-prefill-rows")
	q, kv, sk, sv, temp = _attn_inputs(rng, T5, H5, HD5)
	qs, ks, vs = _scales(rng, (H5, T5)), _scales(rng, (H5, T5)), _scales(rng, (H5, T5))
	vw, sw, osc = recipes.attn_row_scale_operands(vs, X.BF16)
	args = (_up(dev, q, X.INT8), _up(dev, kv, X.INT8), _up(dev, sk, X.INT8), _up(dev, sv, X.INT8), _up(dev, temp, X.F32))
	sc = (_up(dev, qs, X.F32), _up(dev, ks, X.F32), _up(dev, vw, X.F32), _up(dev, sw, X.F32), _up(dev, osc, X.F32))
	got = {}
	for strict in (True, False):
		out, l = X.Tensor(dev, (T5, H5 * HD5), X.BF16), X.Tensor(dev, (H5, T5), X.F32)
		recipes.attn_row_scaled_kernel(dev, H5, HD5, X.BF16, strict).launch_row_scaled(*args, out, l, W5, *sc)
		got[strict] = (out.download(), l.download())
	rep = bf16_diff(got[False][0], got[True][0])
	rep["l_max_abs"] = float(np.abs(got[False][1].astype(np.float64) - got[True][1]).max())
	return rep


def dequant_pair(dev):
	m, d, f = 8192, 2048, 8192
	rng = rng_for("fast-builds-dequant")
	x, w1, w2 = i8_codes(rng, (m, d)), i8_codes(rng, (2 * f, d)), i8_codes(rng, (d, f))
	h = i8_codes(rng, (m, f))
	rs = (0.01 + 0.01 * rng.random(m)).astype(np.float32)
	cs1 = (0.01 + 0.01 * rng.random(2 * f)).astype(np.float32)
	cs2 = (0.01 + 0.01 * rng.random(d)).astype(np.float32)
	xt, w1t, w2t, ht = _up(dev, x, X.INT8), _up(dev, w1, X.INT8), _up(dev, w2, X.INT8), _up(dev, h, X.INT8)
	rst, cs1t, cs2t = _up(dev, rs, X.F32), _up(dev, cs1, X.F32), _up(dev, cs2, X.F32)
	got = {}
	for strict in (True, False):
		o1, o2 = X.Tensor(dev, (m, f), X.BF16), X.Tensor(dev, (m, d), X.BF16)
		recipes.dequant_gemm_kernel(dev, d, 2 * f, X.INT8, X.INT8, True, strict).launch_dequant(xt, w1t, o1, rst, cs1t)
		recipes.dequant_gemm_kernel(dev, f, d, X.INT8, X.INT8, False, strict).launch_dequant(ht, w2t, o2, rst, cs2t)
		got[strict] = (o1.download(), o2.download())
	return {"geglu_bf16": bf16_diff(got[False][0], got[True][0]), "plain_bf16": bf16_diff(got[False][1], got[True][1])}


def report(dev):
	return {"config5_decode": decode(dev), "config5_decode_row_scaled_bf16": decode_row_scaled(dev),
	        "config5_prefill_row_scaled_bf16": prefill_row_scaled(dev), "config2_dequant_pair": dequant_pair(dev)}
