#!/usr/bin/env python3
"""Benchmark of the quantized block-forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--only KERNEL] [--copy-probe]

Headline (the JSON line's `value`): benchmark config 2, the int8 FFN GEMM pair
  ffn_f_fwd   x[8192, 2048] i8 . W1[16384, 2048]^T  -> GeGLU   -> f[8192, 8192] FixedI8
  ffn_y_fwd   f[8192, 8192] i8 . W2[4096, 8192]^T   -> gated residual with x -> y[8192, 2048] e4m3
One step = both launches over the 8192-token batch; inputs are resident in HBM before the timed
region.  value = (2*M*K*N_raw of both GEMMs) * steps / wall time, in TOPS.

`roofline` is for the dominant kernel (the ffn_f GEMM): algorithmic int8 ops per launch divided by
its mean launch duration, measured with HIP events on the launching stream inside the timed
region, against the MI355X dense int8 MFMA peak.  `cpu_baseline` is the CPU oracle (a port of the
reference's arithmetic) timed on a bounded row sample of the same workload on the host cores.
`extras` reports the other benchmark configurations (fp8 FFN, block forward, attention prefill,
decode, rms_norm), each as median-of-launches, next to the roofline that bounds it.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
	sys.path.insert(0, ROOT)

import numpy as np

PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, published
PEAK_FP8_TFLOPS = 5000.0     # dense fp8
PEAK_BF16_TFLOPS = 2500.0    # dense bf16
PEAK_HBM_GBS = 8000.0        # HBM3E

# HBM bytes per ffn_f launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/), or None
FFN_F_TRAFFIC_BYTES = int((198254 * 2.0 + 65536 * 1.0) * 1024)
# HBM bytes one decode launch of config 5 fetches (profiles/attn_decode_i8_config5.txt): all K rows plus the
# V rows with a nonzero 8-bit probability -- about half of the 2 GiB cache for the synthetic Gaussian codes
DECODE_TRAFFIC_BYTES = int(529500 * 2.0 * 1024)


def _rand_i8(rng, shape):
	return rng.integers(-127, 128, size=shape, dtype=np.int8)


def _rand_codes(rng, shape, sigma=1.0):
	# FixedI8 codes of N(0, sigma^2): cheap float32 path, same distribution as the tests use
	return np.clip(np.rint(rng.standard_normal(shape, dtype=np.float32) * (8.0 * sigma)), -127, 127).astype(np.int8)


def _median_launch(dev, X, fn, iters, warm):
	for _ in range(warm):
		fn()
	dev.synchronize()
	timers = [X.Timer(dev) for _ in range(iters)]
	for t in timers:
		t.start()
		fn()
		t.stop()
	dev.synchronize()
	ts = sorted(t.elapsed_seconds() for t in timers)
	return ts[len(ts) // 2], ts[0]


def headline(dev, X, recipes, steps, warmup):
	M, D, F = 8192, 2048, 8192
	rng = np.random.default_rng(2000)
	x = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
	w1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * F, D)), X.INT8)
	w2 = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, F)), X.INT8)
	f = X.Tensor(dev, (M, F), X.INT8)
	y = X.Tensor(dev, (M, D), X.E4M3)
	k1 = recipes.ffn_f_kernel(dev, D, 2 * F, False, X.INT8)
	k2 = recipes.ffn_y_kernel(dev, D, F, False, X.INT8, X.INT8)
	ops1 = k1.n_ops(x, w1)
	ops2 = k2.n_ops(f, w2)

	def step(timer=None):
		if timer is not None:
			timer.start()
		k1.launch(x, w1, f)
		if timer is not None:
			timer.stop()
		k2.launch(f, w2, y, x)

	for _ in range(warmup):
		step()
	timers = [X.Timer(dev) for _ in range(steps)]
	dev.synchronize()
	t0 = time.perf_counter()
	for t in timers:
		step(t)
	dev.synchronize()
	t1 = time.perf_counter()
	wall = t1 - t0
	k1_mean = sum(t.elapsed_seconds() for t in timers) / steps
	return {
		"wall_s": wall, "ops_per_step": ops1 + ops2, "k1_ops": ops1, "k1_mean_s": k1_mean,
		"shapes": {"tokens": M, "d_model": D, "d_ff": F},
	}


def cpu_baseline():
	"""The CPU oracle on config 2 (all 8192 token rows: about 12 s on 16 host threads)."""
	from oracle import strict as S
	M, D, F = 8192, 2048, 8192
	rng = np.random.default_rng(2001)
	x, w1, w2 = _rand_codes(rng, (M, D)), _rand_codes(rng, (2 * F, D)), _rand_codes(rng, (2 * D, F))
	t0 = time.perf_counter()
	f = S.epilogue_geglu(S.gemm_i32(x, w1), 1.0 / math.sqrt(D) / 64.0, 8.0, S.STORE_I8)
	gelu_var_fix_2 = 1.0 / ((1.0 / 3.0) + (0.5 / math.pi) * (1.0 / math.sqrt(3.0)))
	S.epilogue_residual(S.gemm_i32(f, w2), x, math.sqrt(gelu_var_fix_2 / F) / 64.0, 1.0, S.STORE_E4M3)
	dt = time.perf_counter() - t0
	ops = 2.0 * M * D * 2 * F + 2.0 * M * F * 2 * D
	return {"value": ops / dt / 1e12, "unit": "TOPS", "cores": S.num_threads(), "kind": "port",
	        "sample": f"{M} of 8192 token rows of config 2 (both GEMMs + epilogues), {dt:.1f} s of CPU time"}


def mfma_probe(dev, X):
	"""Loops of nothing but MFMAs on register operands, all-zero and Gaussian data: what the matrix cores of this
	machine sustain (the clock under dense MFMA load depends on how much the operands toggle)."""
	from x17ai_amd.api import MfmaProbe
	rng = np.random.default_rng(7)
	out = X.Tensor(dev, (256 * 512,), X.F32)
	result = {}
	for kind, name, peak in ((0, "int8", PEAK_INT8_TOPS), (1, "e4m3", PEAK_INT8_TOPS), (2, "f16", PEAK_INT8_TOPS / 2)):
		probe = MfmaProbe(dev, kind)
		if kind == 0:
			gauss = _rand_codes(rng, (12 * 512 * 16,))
		elif kind == 1:
			gauss = rng.integers(0x20, 0x50, 12 * 512 * 16).astype(np.uint8).view(np.int8)       # normal e4m3 codes
			gauss = np.where(rng.random(gauss.shape) < 0.5, gauss, gauss | np.int8(-128)).astype(np.int8)
		else:
			gauss = rng.standard_normal(12 * 512 * 8).astype(np.float16).view(np.int8)
		for data_name, data in (("zeros", np.zeros(12 * 512 * 16, np.int8)), ("gaussian", gauss)):
			operands = X.Tensor.from_numpy(dev, np.ascontiguousarray(data), X.INT8)
			ops = [0.0]

			def fn():
				ops[0] = probe.launch(operands, out, 4096)
			med, mn = _median_launch(dev, X, fn, 10, 3)
			result[f"{name}_{data_name}"] = {"median_us": med * 1e6, "tops": ops[0] / med / 1e12,
			                                 "frac_of_nominal_peak": ops[0] / med / 1e12 / peak}
	return result


def extras(dev, X, recipes):
	out = {}
	rng = np.random.default_rng(3000)

	def gemm_entry(kern, a, b, c, extra, peak, iters=20, warm=5):
		med, mn = _median_launch(dev, X, lambda: kern.launch(a, b, c, extra), iters, warm)
		ops = kern.n_ops(a, b)
		return {"median_us": med * 1e6, "min_us": mn * 1e6, "tops": ops / med / 1e12, "frac_of_peak": ops / med / 1e12 / peak}

	# ---- config 2 per kernel, both math builds
	M, D, F = 8192, 2048, 8192
	x = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
	w1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * F, D)), X.INT8)
	w2 = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, F)), X.INT8)
	f = X.Tensor(dev, (M, F), X.INT8)
	y = X.Tensor(dev, (M, D), X.E4M3)
	c2 = {}
	for strict in (False, True):
		tag = "strict" if strict else "fast"
		c2[f"ffn_f_{tag}"] = gemm_entry(recipes.ffn_f_kernel(dev, D, 2 * F, strict, X.INT8), x, w1, f, None, PEAK_INT8_TOPS)
		c2[f"ffn_y_{tag}"] = gemm_entry(recipes.ffn_y_kernel(dev, D, F, strict, X.INT8, X.INT8), f, w2, y, x, PEAK_INT8_TOPS)
	# the same pair in the literal form of the config text: per-token / per-output-channel scale vectors
	# applied in the epilogue, bf16 out (W2 ungated: N_raw = d_model)
	rs = X.Tensor.from_numpy(dev, (0.01 + 0.01 * rng.random(M)).astype(np.float32), X.F32)
	cs1 = X.Tensor.from_numpy(dev, (0.01 + 0.01 * rng.random(2 * F)).astype(np.float32), X.F32)
	cs2 = X.Tensor.from_numpy(dev, (0.01 + 0.01 * rng.random(D)).astype(np.float32), X.F32)
	w2l = X.Tensor.from_numpy(dev, _rand_codes(rng, (D, F)), X.INT8)
	hb = X.Tensor(dev, (M, F), X.BF16)
	yb = X.Tensor(dev, (M, D), X.BF16)
	kd1 = recipes.dequant_gemm_kernel(dev, D, 2 * F, X.INT8, X.INT8, True, False)
	kd2 = recipes.dequant_gemm_kernel(dev, F, D, X.INT8, X.INT8, False, False)
	for name, kern, a_, b_, c_, cs_ in (("dequant_geglu_bf16", kd1, x, w1, hb, cs1), ("dequant_bf16", kd2, f, w2l, yb, cs2)):
		med, mn = _median_launch(dev, X, lambda: kern.launch_dequant(a_, b_, c_, rs, cs_), 20, 5)
		ops = kern.n_ops(a_, b_)
		c2[name] = {"median_us": med * 1e6, "min_us": mn * 1e6, "tops": ops / med / 1e12, "frac_of_peak": ops / med / 1e12 / PEAK_INT8_TOPS}
	out["config2_int8_ffn"] = c2
	del rs, cs1, cs2, w2l, hb, yb
	del w1, w2, f, y

	# ---- config 3: all-fp8 FFN, tokens=16384, d_model=4096, d_ff=16384
	M3, D3, F3 = 16384, 4096, 16384
	def e4m3_rand(shape):
		return _rand_e4m3(rng, shape)
	x3 = X.Tensor.from_numpy(dev, e4m3_rand((M3, D3)), X.E4M3)
	w13 = X.Tensor.from_numpy(dev, e4m3_rand((2 * F3, D3)), X.E4M3)
	f3 = X.Tensor(dev, (M3, F3), X.E4M3)
	c3 = {"ffn_f_f8": gemm_entry(recipes.ffn_f_f8_kernel(dev, D3, 2 * F3, False), x3, w13, f3, None, PEAK_FP8_TFLOPS, 10, 3)}
	del w13
	w23 = X.Tensor.from_numpy(dev, e4m3_rand((2 * D3, F3)), X.E4M3)
	r3 = X.Tensor.from_numpy(dev, _rand_codes(rng, (M3, D3)), X.INT8)
	y3 = X.Tensor(dev, (M3, D3), X.E4M3)
	c3["ffn_y_f8"] = gemm_entry(recipes.ffn_y_kernel(dev, D3, F3, False, X.E4M3, X.E4M3), f3, w23, y3, r3, PEAK_FP8_TFLOPS, 10, 3)
	out["config3_fp8_ffn"] = c3
	del x3, w23, f3, r3, y3

	# ---- config 4: block forward, 4 x 8192 tokens, d_model 2048, 16 heads x 128, window 512, d_ff 8192
	T, B, H, HD, W = 8192, 4, 16, 128, 512
	rows = T * B
	xb = X.Tensor.from_numpy(dev, (rng.standard_normal((rows, D), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16), X.BF16)
	xi = X.Tensor(dev, (rows, D), X.INT8)
	wq = X.Tensor.from_numpy(dev, _rand_codes(rng, (H * HD, D)), X.INT8)
	wkv = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * H * HD, D)), X.INT8)
	wy = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, H * HD)), X.INT8)
	wf = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * F, D)), X.INT8)
	wfy = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, F)), X.INT8)
	sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
	sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
	temp = X.Tensor.from_numpy(dev, (0.5 + rng.random(H)).astype(np.float32), X.F32)
	q = X.Tensor(dev, (rows, H * HD), X.INT8)
	kv = X.Tensor(dev, (rows, 2 * H * HD), X.INT8)
	rrms = X.Tensor(dev, (rows, H), X.F32)
	ao = X.Tensor(dev, (rows, H * HD), X.INT8)
	al = X.Tensor(dev, (H, rows), X.F32)
	ay = X.Tensor(dev, (rows, D), X.E4M3)
	ff = X.Tensor(dev, (rows, F), X.E4M3)
	fy = X.Tensor(dev, (rows, D), X.E4M3)
	k_rms = recipes.rms_norm_kernel(dev, D, X.BF16)
	k_q = recipes.attn_q_kernel(dev, D, H * HD)
	k_kv = recipes.attn_kv_kernel(dev, D, 2 * H * HD, HD)
	k_at = recipes.attn_kernel(dev, H, HD, False)
	k_ay = recipes.attn_y_kernel(dev, D, H * HD, False)
	k_ff = recipes.ffn_f_kernel(dev, D, 2 * F, False)
	k_fy = recipes.ffn_y_kernel(dev, D, F, False)
	stages = [
		("rms_norm", lambda: k_rms.launch(xb, xi)),
		("attn_q", lambda: k_q.launch(xi, wq, q)),
		("attn_kv", lambda: k_kv.launch(xi, wkv, kv, rrms)),
		("attn_fwd_i8", lambda: k_at.launch(q, kv, sk, sv, temp, ao, al, W, B)),
		("attn_y", lambda: k_ay.launch(ao, wy, ay, xi)),
		("ffn_f", lambda: k_ff.launch(xi, wf, ff)),
		("ffn_y_f8", lambda: k_fy.launch(ff, wfy, fy, xi)),
	]
	c4 = {}
	total = 0.0
	for name, fn in stages:
		med, mn = _median_launch(dev, X, fn, 10, 3)
		c4[name + "_us"] = med * 1e6
		total += med
	pairs = W * (W - 1) // 2 + (T - W) * W
	attn_ops = 4.0 * HD * H * B * pairs
	c4["attn_tops"] = attn_ops / (c4["attn_fwd_i8_us"] * 1e-6) / 1e12
	c4["attn_frac_of_int8_peak"] = c4["attn_tops"] / PEAK_INT8_TOPS
	c4["rms_norm_gbs"] = rows * D * 3 / (c4["rms_norm_us"] * 1e-6) / 1e9
	c4["rms_norm_frac_of_hbm"] = c4["rms_norm_gbs"] / PEAK_HBM_GBS
	c4["ffn_y_f8_tflops"] = 2.0 * rows * F * 2 * D / (c4["ffn_y_f8_us"] * 1e-6) / 1e12
	c4["block_tokens_per_s"] = rows / total
	# end to end, back to back on the stream
	def block():
		for _, fn in stages:
			fn()
	med, _ = _median_launch(dev, X, block, 5, 2)
	c4["block_back_to_back_us"] = med * 1e6
	c4["block_tokens_per_s_back_to_back"] = rows / med
	out["config4_block"] = c4
	del xb, xi, wq, wkv, wy, wf, wfy, q, kv, rrms, ao, al, ay, ff, fy

	# ---- config 1: attention T=1024, H=8, hd=64, W=256
	T1, H1, HD1, W1 = 1024, 8, 64, 256
	q1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T1, H1 * HD1)), X.INT8)
	kv1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T1, 2 * H1 * HD1)), X.INT8)
	sk1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H1, HD1)), X.INT8)
	sv1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H1, HD1)), X.INT8)
	tp1 = X.Tensor.from_numpy(dev, np.ones(H1, np.float32), X.F32)
	o1 = X.Tensor(dev, (T1, H1 * HD1), X.INT8)
	k1 = recipes.attn_kernel(dev, H1, HD1, False)
	med, _ = _median_launch(dev, X, lambda: k1.launch(q1, kv1, sk1, sv1, tp1, o1, None, W1), 20, 5)
	p1 = W1 * (W1 - 1) // 2 + (T1 - W1) * W1
	out["config1_attn"] = {"median_us": med * 1e6, "gops": 4.0 * HD1 * H1 * p1 / 1e9, "tops": 4.0 * HD1 * H1 * p1 / med / 1e12}

	# the same shape as the configuration words it: one scale per (row, head) of q, k and v, bf16 output; the scales
	# vary around 1/8 so that the scores keep the spread they have in the fixed-scale runs
	def row_scale_tensors(rows, heads):
		scales = [(0.125 * (0.75 + 0.5 * rng.random((heads, rows)))).astype(np.float32) for _ in range(3)]
		vw, sw, osc = recipes.attn_row_scale_operands(scales[2], X.BF16)
		return [X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32) for a in (scales[0], scales[1], vw, sw, osc)]
	rs1 = row_scale_tensors(T1, H1)
	ob1 = X.Tensor(dev, (T1, H1 * HD1), X.BF16)
	k1r = recipes.attn_row_scaled_kernel(dev, H1, HD1, X.BF16, False)
	med, _ = _median_launch(dev, X, lambda: k1r.launch_row_scaled(q1, kv1, sk1, sv1, tp1, ob1, None, W1, *rs1), 20, 5)
	out["config1_attn_row_scaled_bf16"] = {"median_us": med * 1e6, "tops": 4.0 * HD1 * H1 * p1 / med / 1e12}

	# ---- config 5: prefill T=65536, H=32, hd=128, W=4096; decode 64 sequences x 4096 cached positions
	T5, H5, HD5, W5 = 65536, 32, 128, 4096
	q5 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T5, H5 * HD5)), X.INT8)
	kv5 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T5, 2 * H5 * HD5)), X.INT8)
	sk5 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H5, HD5)), X.INT8)
	sv5 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H5, HD5)), X.INT8)
	tp5 = X.Tensor.from_numpy(dev, np.ones(H5, np.float32), X.F32)
	o5 = X.Tensor(dev, (T5, H5 * HD5), X.INT8)
	c5 = {}
	for strict in (False, True):
		k5 = recipes.attn_kernel(dev, H5, HD5, strict)
		med, _ = _median_launch(dev, X, lambda: k5.launch(q5, kv5, sk5, sv5, tp5, o5, None, W5), 3, 1)
		p5 = W5 * (W5 - 1) // 2 + (T5 - W5) * W5
		tag = "strict" if strict else "fast"
		c5[f"prefill_{tag}_ms"] = med * 1e3
		c5[f"prefill_{tag}_tops"] = 4.0 * HD5 * H5 * p5 / med / 1e12
		c5[f"prefill_{tag}_frac_of_int8_peak"] = c5[f"prefill_{tag}_tops"] / PEAK_INT8_TOPS
	rs5 = row_scale_tensors(T5, H5)
	ob5 = X.Tensor(dev, (T5, H5 * HD5), X.BF16)
	k5r = recipes.attn_row_scaled_kernel(dev, H5, HD5, X.BF16, False)
	med, _ = _median_launch(dev, X, lambda: k5r.launch_row_scaled(q5, kv5, sk5, sv5, tp5, ob5, None, W5, *rs5), 3, 1)
	c5["prefill_row_scaled_bf16_ms"] = med * 1e3
	c5["prefill_row_scaled_bf16_tops"] = 4.0 * HD5 * H5 * p5 / med / 1e12
	del q5, kv5, o5, ob5, rs5
	S5, CAP = 64, 4096
	one = _rand_codes(rng, (1, CAP, 2 * H5 * HD5))
	cache = X.Tensor.from_numpy(dev, np.ascontiguousarray(np.broadcast_to(one, (S5, CAP, 2 * H5 * HD5))), X.INT8)
	qd = X.Tensor.from_numpy(dev, _rand_codes(rng, (S5, H5 * HD5)), X.INT8)
	lens = X.Tensor.from_numpy(dev, np.full(S5, CAP, np.uint32).view(np.float32), X.F32)
	od = X.Tensor(dev, (S5, H5 * HD5), X.INT8)
	for strict in (False, True):
		kd = recipes.attn_decode_kernel(dev, H5, HD5, CAP, strict)
		med, _ = _median_launch(dev, X, lambda: kd.launch(qd, cache, lens, sk5, sv5, tp5, od, None, W5), 10, 3)
		nbytes = S5 * CAP * 2 * H5 * HD5
		tag = "strict" if strict else "fast"
		c5[f"decode_{tag}_us"] = med * 1e6
		c5[f"decode_{tag}_cache_gbs"] = nbytes / med / 1e9            # whole cache / time: counts the V rows skipped
		c5[f"decode_{tag}_hbm_gbs"] = DECODE_TRAFFIC_BYTES / med / 1e9  # bytes actually fetched (rocprofv3) / time
		c5[f"decode_{tag}_frac_of_hbm"] = DECODE_TRAFFIC_BYTES / med / 1e9 / PEAK_HBM_GBS
	# the cache as a row-scaled prefill leaves it: one scale per (row, head) of k and v, bf16 output
	kd_rows = recipes.attn_decode_row_scaled_kernel(dev, H5, HD5, CAP, X.BF16, False)
	scale_one = [(0.125 * (0.75 + 0.5 * rng.random((1, H5, CAP)))).astype(np.float32) for _ in range(2)]
	vw5, sw5, os5 = recipes.attn_row_scale_operands(np.broadcast_to(scale_one[1], (S5, H5, CAP)), X.BF16)
	f32t = lambda a: X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32)
	rsd = [f32t(0.125 * (0.75 + 0.5 * rng.random((S5, H5)))), f32t(np.broadcast_to(scale_one[0], (S5, H5, CAP))), f32t(vw5), f32t(sw5), f32t(os5)]
	odb = X.Tensor(dev, (S5, H5 * HD5), X.BF16)
	med, _ = _median_launch(dev, X, lambda: kd_rows.launch_row_scaled(qd, cache, lens, sk5, sv5, tp5, odb, None, W5, *rsd), 10, 3)
	c5["decode_row_scaled_bf16_us"] = med * 1e6
	out["config5_long_context"] = c5
	# what the matrix cores sustain with no memory traffic at all, beside the nominal peaks used above
	out["mfma_probe"] = mfma_probe(dev, X)
	return out


def _rand_e4m3(rng, shape):
	"""valid reference-dialect e4m3 bytes with magnitudes in [0.25, 3.75]: exponent field 5..8"""
	b = (rng.integers(5, 9, size=shape, dtype=np.uint8) << 3) | rng.integers(0, 8, size=shape, dtype=np.uint8)
	return b | (rng.integers(0, 2, size=shape, dtype=np.uint8) << 7)


def single(dev, X, recipes, name, iters):
	"""One kernel of one benchmark workload, launched `iters` times: what the rocprofv3 summaries under
	profiles/ are taken from (every code object exports the entry `kernel`, so a profile of several
	kernels at once cannot tell them apart by name)."""
	rng = np.random.default_rng(3000)
	D, F = 2048, 8192
	if name == "ffn_f_config2":
		M = 8192
		a = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
		b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * F, D)), X.INT8)
		c = X.Tensor(dev, (M, F), X.INT8)
		k = recipes.ffn_f_kernel(dev, D, 2 * F, False, X.INT8)
		fn, work, unit = (lambda: k.launch(a, b, c)), k.n_ops(a, b) / 1e12, "TOPS"
	elif name == "ffn_f_f8_config3":
		M, D3, F3 = 16384, 4096, 16384
		a = X.Tensor.from_numpy(dev, _rand_e4m3(rng, (M, D3)), X.E4M3)
		b = X.Tensor.from_numpy(dev, _rand_e4m3(rng, (2 * F3, D3)), X.E4M3)
		c = X.Tensor(dev, (M, F3), X.E4M3)
		k = recipes.ffn_f_f8_kernel(dev, D3, 2 * F3, False)
		fn, work, unit = (lambda: k.launch(a, b, c)), k.n_ops(a, b) / 1e12, "TFLOP/s"
	elif name == "ffn_y_f8_config4":
		M = 32768
		a = X.Tensor.from_numpy(dev, rng.integers(0x20, 0x50, (M, F), dtype=np.uint8), X.E4M3)
		b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, F)), X.INT8)
		r = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
		c = X.Tensor(dev, (M, D), X.E4M3)
		k = recipes.ffn_y_kernel(dev, D, F, False)
		fn, work, unit = (lambda: k.launch(a, b, c, r)), k.n_ops(a, b) / 1e12, "TFLOP/s"
	elif name in ("attn_config4", "attn_config5"):
		T, B, H, HD, W = (8192, 4, 16, 128, 512) if name == "attn_config4" else (65536, 1, 32, 128, 4096)
		rows = T * B
		q = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, H * HD)), X.INT8)
		kv = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, 2 * H * HD)), X.INT8)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, (0.5 + rng.random(H)).astype(np.float32), X.F32)
		o = X.Tensor(dev, (rows, H * HD), X.INT8)
		l = X.Tensor(dev, (H, rows), X.F32)
		k = recipes.attn_kernel(dev, H, HD, False)
		pairs = W * (W - 1) // 2 + (T - W) * W
		fn, work, unit = (lambda: k.launch(q, kv, sk, sv, tp, o, l, W, B)), 4.0 * HD * H * B * pairs / 1e12, "TOPS"
	elif name == "decode_config5":
		S5, CAP, H, HD, W = 64, 4096, 32, 128, 4096
		one = _rand_codes(rng, (1, CAP, 2 * H * HD))
		cache = X.Tensor.from_numpy(dev, np.ascontiguousarray(np.broadcast_to(one, (S5, CAP, 2 * H * HD))), X.INT8)
		qd = X.Tensor.from_numpy(dev, _rand_codes(rng, (S5, H * HD)), X.INT8)
		lens = X.Tensor.from_numpy(dev, np.full(S5, CAP, np.uint32).view(np.float32), X.F32)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, np.ones(H, np.float32), X.F32)
		od = X.Tensor(dev, (S5, H * HD), X.INT8)
		k = recipes.attn_decode_kernel(dev, H, HD, CAP, False)
		fn, work, unit = (lambda: k.launch(qd, cache, lens, sk, sv, tp, od, None, W)), S5 * CAP * 2 * H * HD / 1e9, "GB/s of cache (rows with zero probability are not fetched)"
	elif name == "rms_norm_config4":
		rows = 32768
		xb = X.Tensor.from_numpy(dev, (rng.standard_normal((rows, D), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16), X.BF16)
		xi = X.Tensor(dev, (rows, D), X.INT8)
		k = recipes.rms_norm_kernel(dev, D, X.BF16)
		fn, work, unit = (lambda: k.launch(xb, xi)), rows * D * 3 / 1e9, "GB/s"
	else:
		raise SystemExit(f"bench.py: unknown --only target {name!r}")
	med, mn = _median_launch(dev, X, fn, iters, 3)
	print(json.dumps({"only": name, "launches": iters, "median_us": med * 1e6, "min_us": mn * 1e6,
	                  "rate": work / med, "unit": unit}))


ONLY_TARGETS = ("ffn_f_config2", "ffn_f_f8_config3", "ffn_y_f8_config4", "attn_config4", "attn_config5", "decode_config5", "rms_norm_config4")


def main():
	ap = argparse.ArgumentParser()
	ap.add_argument("--gpus", type=int, default=1)
	ap.add_argument("--steps", type=int, default=50)
	ap.add_argument("--warmup", type=int, default=10)
	ap.add_argument("--no-extras", action="store_true")
	ap.add_argument("--no-cpu", action="store_true")
	ap.add_argument("--copy-probe", action="store_true",
	                help="only run a 1 GiB device-to-device copy kernel (calibrates the HBM traffic counters)")
	ap.add_argument("--mfma-probe", action="store_true",
	                help="only run loops of nothing but MFMAs on register operands (all-zero and Gaussian data; int8, "
	                     "e4m3, f16): what the matrix cores of this machine sustain, beside the nominal peaks")
	ap.add_argument("--only", choices=ONLY_TARGETS,
	                help="launch one kernel of one workload --steps times and print its median (used for the profiles)")
	args = ap.parse_args()
	if args.gpus != 1:
		print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
		sys.exit(2)

	import x17ai_amd as X
	from x17ai_amd import recipes

	dev = X.Device(0)
	if args.copy_probe:
		from x17ai_amd.api import CopyProbe
		n = 1 << 30
		src = X.Tensor.from_numpy(dev, np.zeros(n, np.int8), X.INT8)
		dst = X.Tensor(dev, (n,), X.INT8)
		probe = CopyProbe(dev)
		for _ in range(5):
			probe.launch(src, dst)
		dev.synchronize()
		print(json.dumps({"copy_probe_bytes_read": n, "copy_probe_bytes_written": n, "launches": 5}))
		return
	if args.mfma_probe:
		print(json.dumps({"mfma_probe": mfma_probe(dev, X)}))
		return
	if args.only:
		single(dev, X, recipes, args.only, args.steps)
		return
	h = headline(dev, X, recipes, args.steps, args.warmup)
	value = h["ops_per_step"] * args.steps / h["wall_s"] / 1e12
	achieved = h["k1_ops"] / h["k1_mean_s"] / 1e12
	line = {
		"metric": "int8 TOPS at 1 MI355X (config 2: FFN GEMM pair ffn_f_fwd + ffn_y_fwd_i8); fp8 TOPS, block-fwd tokens/sec and % of MFMA/HBM roofline under extras",
		"value": value, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
		"ms_per_step": h["wall_s"] / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
		"vs_baseline": None, "dtype": "int8", "data": "synthetic",
		"config": {"workload": "config 2: int8 FFN GEMM pair, tokens=8192, d_model=2048, d_ff=8192 (gated layout: "
		                       "W1 [16384, 2048] GeGLU -> FixedI8, W2 [4096, 8192] gated residual -> e4m3)",
		           "math": "hardware transcendentals in the epilogues (strict build reported under extras)"},
		"roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_INT8_TOPS, "unit": "TFLOP/s",
		             "frac": achieved / PEAK_INT8_TOPS, "traffic": FFN_F_TRAFFIC_BYTES,
		             "kernel": "gemm_b8 (ffn_f_fwd: M=8192, K=2048, N_raw=16384, GeGLU epilogue)",
		             "mean_launch_us": h["k1_mean_s"] * 1e6},
	}
	if not args.no_cpu:
		line["cpu_baseline"] = cpu_baseline()
	if not args.no_extras:
		line["extras"] = extras(dev, X, recipes)
	dev.synchronize()
	print(json.dumps(line))


if __name__ == "__main__":
	main()
