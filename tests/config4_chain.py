"""Benchmark config 4 as one chain on the GPU: 4 sequences x 8192 tokens of seeded bf16 residual stream through
rms_norm -> q / kv -> attention (16 heads x 128, window 512) -> attn_y, and ffn_f (d_ff 8192) -> ffn_y, every
stage of x17ai_amd.block.Block at its full shape (stage order and recipes of src/main.rs:193-280).

run_strict()        launches the strict builds and returns inputs, weights and every stage's output as numpy arrays
check_strict()      holds each stage against the CPU oracle ON THE GPU'S OWN UPSTREAM OUTPUT (sampled token rows
                    for the row-wise stages, sampled heads for the attention)
fast_vs_strict()    runs the hardware-transcendental build of each stage on the strict build's upstream output and
                    returns, per stage, the mismatch histogram, max-abs and relative-L2 difference
Used by tests/test_gpu_fullsize.py and by tests/golden/make_config4_report.py.
"""
from __future__ import annotations

import math

import numpy as np

import x17ai_amd as X
from x17ai_amd import recipes
from x17ai_amd.block import Block, BlockConfig
from oracle import strict as S
from tests.gpu_common import e4m3_compare, i8_codes, rng_for

T, B, D, H, HD, W, F = 8192, 4, 2048, 16, 128, 512, 8192
ROWS = T * B
INP = 1.0 / math.sqrt(D) / 64.0                       # src/main.rs:412-416, 461-469, 599-603
INP_ATTN_Y = 1.0 / math.sqrt(H * HD) / 64.0           # src/main.rs:548-557
INP_FFN_Y = math.sqrt(recipes.GELU_VAR_FIX_2 / F) / 8.0   # src/main.rs:650-660


def config(strict: bool, fused_qkv: bool = False) -> BlockConfig:
	return BlockConfig(D, H, HD, F, W, B, X.BF16, strict, fused_qkv)


def inputs():
	rng = rng_for("config4-chain")
	x = rng.standard_normal((ROWS, D), dtype=np.float32)
	x_bf16 = ((x.view(np.uint32) + 0x7FFF + ((x.view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)   # round to nearest even
	sk = rng.standard_normal((H, HD))
	sk /= np.sqrt((sk * sk).mean(-1, keepdims=True))
	wkv = rng.standard_normal((H, 2, HD, D)).astype(np.float32)
	wkv[:, 1] *= 1.3                                   # V_SCALE_FIX, new_block.py:27-52
	return {
		"x_bf16": x_bf16,
		"attn_q_weights": i8_codes(rng, (H * HD, D)),
		"attn_kv_weights": S.f32_to_fixedi8((wkv.reshape(2 * H * HD, D) * 8.0).astype(np.float32)),
		"attn_y_weights": i8_codes(rng, (2 * D, H * HD)),
		"ffn_f_weights": i8_codes(rng, (2 * F, D)),
		"ffn_y_weights": i8_codes(rng, (2 * D, F)),
		"sinks_k": S.f32_to_fixedi8((sk * 8).astype(np.float32)),
		"sinks_v": i8_codes(rng, (H, HD), 1.3),
		"attn_temperature": (0.5 + rng.random(H)).astype(np.float32),
	}


def _upload(dev, inp):
	w = {k: X.Tensor.from_numpy(dev, v, X.F32 if k == "attn_temperature" else X.INT8) for k, v in inp.items() if k != "x_bf16"}
	return X.Tensor.from_numpy(dev, inp["x_bf16"], X.BF16), w


def run_strict(dev, inp, fused_qkv: bool = False):
	"""Every stage's output of the strict build, downloaded."""
	x, w = _upload(dev, inp)
	block = Block(dev, config(True, fused_qkv))
	out = block.forward(x, w)
	return {k: t.download() for k, t in out.items()}


def run_fused_qkv(dev, got, strict: bool = True):
	"""q, kv and rrms of the fused projection kernel on the FixedI8 x of `got` (run_strict's result)."""
	inp = inputs()
	k = recipes.attn_qkv_kernel(dev, D, H * HD, 2 * H * HD, HD, strict)
	q = X.Tensor(dev, (ROWS, H * HD), X.INT8)
	kv = X.Tensor(dev, (ROWS, 2 * H * HD), X.INT8)
	rr = X.Tensor(dev, (ROWS, H), X.F32)
	k.launch_qkv(X.Tensor.from_numpy(dev, got["x"], X.INT8), X.Tensor.from_numpy(dev, inp["attn_q_weights"], X.INT8),
	             X.Tensor.from_numpy(dev, inp["attn_kv_weights"], X.INT8), q, kv, rr)
	return {"q": q.download(), "kv": kv.download(), "k_rrms": rr.download()}


def sample_rows(rng, count=96):
	# first / last rows, rows either side of 256-row tile edges and of sequence edges, random ones
	fixed = [0, 1, 255, 256, 257, T - 1, T, T + 1, 2 * T - 257, ROWS - 256, ROWS - 1]
	return np.unique(np.concatenate((np.array(fixed), rng.integers(0, ROWS, count - len(fixed)))))


def head_columns(arr, heads, width):
	return np.ascontiguousarray(np.concatenate([arr[:, h * width:(h + 1) * width] for h in heads], axis=1))


def check_strict(inp, got, rows=None, attn_cases=((1, (3, 12)), (2, (9,)))):
	"""Asserts every stage of `got` (run_strict's result) against the oracle on the GPU's own upstream output."""
	rng = rng_for("config4-chain-rows")
	rows = sample_rows(rng) if rows is None else rows
	x = got["x"]
	# rms_norm, bf16 in (rms_norm.cu:55-113)
	assert np.array_equal(x[rows], S.rms_norm(inp["x_bf16"][rows], recipes.L2_NORM_EPS, "bf16")), "rms_norm"
	# q: Scale writer
	assert np.array_equal(got["q"][rows], S.epilogue_scale(S.gemm_i32(x[rows], inp["attn_q_weights"]), INP, 8.0)), "attn_q"
	# kv + rrms: L2-norm writer, head_dim 128
	kv, rrms = S.epilogue_l2norm(S.gemm_i32(x[rows], inp["attn_kv_weights"]), HD, recipes.L2_NORM_EPS, INP, 8.0)
	assert np.array_equal(got["kv"][rows], kv), "attn_kv"
	assert np.array_equal(got["k_rrms"][rows].view(np.uint32), rrms.view(np.uint32)), "k_rrms"
	# attention: heads of a sequence are independent
	for seq, heads in attn_cases:
		heads = list(heads)
		r = slice(seq * T, (seq + 1) * T)
		want, want_l = S.attn_fwd_i8(head_columns(got["q"][r], heads, HD), head_columns(got["kv"][r], heads, 2 * HD),
		                             inp["sinks_k"][heads], inp["sinks_v"][heads], inp["attn_temperature"][heads], len(heads), HD, W)
		assert np.array_equal(head_columns(got["attn_out"][r], heads, HD), want), ("attn_out", seq, heads)
		assert np.array_equal(got["attn_l"][heads][:, r].view(np.uint32), want_l.view(np.uint32)), ("attn_l", seq, heads)
	# attn_y: gated residual -> e4m3
	acc = S.gemm_i32(got["attn_out"][rows], inp["attn_y_weights"])
	assert np.array_equal(got["attn_y"][rows], S.epilogue_residual(acc, x[rows], INP_ATTN_Y, 1.0, S.STORE_E4M3)), "attn_y"
	# ffn_f: GeGLU -> e4m3
	acc = S.gemm_i32(x[rows], inp["ffn_f_weights"])
	assert np.array_equal(got["ffn_f"][rows], S.epilogue_geglu(acc, INP, 1.0, S.STORE_E4M3)), "ffn_f"
	# ffn_y: e4m3 x int8, f32 sums in the matrix cores' order: one e4m3 code at most, rarely
	acc = S.gemm_f32_seq(got["ffn_f"][rows], True, inp["ffn_y_weights"], False)
	want = S.epilogue_residual(acc, x[rows], INP_FFN_Y, 1.0, S.STORE_E4M3)
	frac, beyond = e4m3_compare(got["ffn_y"][rows], want)
	assert frac < 5e-3 and beyond == 0.0, ("ffn_y_f8", frac, beyond)
	return {"rows": len(rows), "ffn_y_frac_one_code": frac}


def _i8_diff(a, b):
	d = np.abs(a.astype(np.int16) - b.astype(np.int16)).reshape(-1)
	hist = [int(np.count_nonzero(d == k)) for k in range(4)]
	hist.append(int(d.size - sum(hist)))                       # |diff| >= 4
	err2 = float(np.sum(d.astype(np.float32) ** 2, dtype=np.float64))
	ref2 = float(np.sum(b.reshape(-1).astype(np.float32) ** 2, dtype=np.float64))
	return {"elements": int(a.size), "mismatched": int(np.count_nonzero(d)), "hist_abs_code_diff_0_1_2_3_more": hist,
	        "max_abs": float(d.max()) / 8.0, "rel_l2": math.sqrt(err2 / ref2)}


def _e4m3_diff(a, b):
	a, b = a.reshape(-1), b.reshape(-1)
	neq = beyond = 0.0
	max_abs = err2 = ref2 = 0.0
	step = 1 << 24
	for i in range(0, a.size, step):                          # (chunks: the f tensor has 268 M elements)
		ca, cb = a[i:i + step], b[i:i + step]
		f, bey = e4m3_compare(ca, cb)
		neq += f * ca.size
		beyond += bey * ca.size
		av, bv = S.e4m3_to_f32(ca).astype(np.float64), S.e4m3_to_f32(cb).astype(np.float64)
		max_abs = max(max_abs, float(np.abs(av - bv).max()))
		err2 += float(np.sum((av - bv) ** 2))
		ref2 += float(np.sum(bv ** 2))
	return {"elements": int(a.size), "mismatched": int(round(neq)), "frac_mismatched": neq / a.size,
	        "frac_beyond_one_code": beyond / a.size, "max_abs": max_abs, "rel_l2": math.sqrt(err2 / ref2)}


def fast_vs_strict(dev, inp, got):
	"""The speed build of every stage on the strict build's upstream output, against the strict build's output."""
	_, w = _upload(dev, inp)
	up = lambda name, dt: X.Tensor.from_numpy(dev, got[name], dt)
	x = up("x", X.INT8)
	fast = Block(dev, config(False))
	rep = {}
	# stages without an approximate operation upstream of the store: identical bytes in both builds
	q = X.Tensor(dev, (ROWS, H * HD), X.INT8)
	fast.k_q.launch(x, w["attn_q_weights"], q)
	rep["attn_q"] = _i8_diff(q.download(), got["q"])
	kv = X.Tensor(dev, (ROWS, 2 * H * HD), X.INT8)
	rr = X.Tensor(dev, (ROWS, H), X.F32)
	fast.k_kv.launch(x, w["attn_kv_weights"], kv, rr)
	rep["attn_kv"] = _i8_diff(kv.download(), got["kv"])
	rep["attn_kv"]["rrms_bits_equal"] = bool(np.array_equal(rr.download().view(np.uint32), got["k_rrms"].view(np.uint32)))
	del q, kv, rr
	ao = X.Tensor(dev, (ROWS, H * HD), X.INT8)
	al = X.Tensor(dev, (H, ROWS), X.F32)
	fast.k_attn.launch(up("q", X.INT8), up("kv", X.INT8), w["sinks_k"], w["sinks_v"], w["attn_temperature"], ao, al, W, B)
	rep["attn_fwd_i8"] = _i8_diff(ao.download(), got["attn_out"])
	rep["attn_fwd_i8"]["l_max_abs"] = float(np.abs(al.download().astype(np.float64) - got["attn_l"]).max())
	del ao, al
	ay = X.Tensor(dev, (ROWS, D), X.E4M3)
	fast.k_attn_y.launch(up("attn_out", X.INT8), w["attn_y_weights"], ay, x)
	rep["attn_y"] = _e4m3_diff(ay.download(), got["attn_y"])
	del ay
	ff = X.Tensor(dev, (ROWS, F), X.E4M3)
	fast.k_ffn_f.launch(x, w["ffn_f_weights"], ff)
	rep["ffn_f"] = _e4m3_diff(ff.download(), got["ffn_f"])
	del ff
	fy = X.Tensor(dev, (ROWS, D), X.E4M3)
	fast.k_ffn_y.launch(up("ffn_f", X.E4M3), w["ffn_y_weights"], fy, x)
	rep["ffn_y_f8"] = _e4m3_diff(fy.download(), got["ffn_y"])
	return rep
