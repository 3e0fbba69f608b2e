#!/usr/bin/env python3
"""Benchmark of the quantized block-forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--only KERNEL]

Headline (the JSON line's `value`): benchmark config 4, the full quantized block forward over
4 sequences x 8192 tokens, d_model 2048, 16 heads x 128, window 512, d_ff 8192:
  rms_norm (bf16 -> FixedI8 x) -> attn_q, attn_kv -> attn_fwd_i8 -> attn_y ; ffn_f -> ffn_y_f8
(x17ai_amd.block.Block: stage order and scale recipes of src/main.rs:193-280, 387-675).  One step = the
seven launches over the 32768-token batch; inputs and weights are resident in HBM before the timed
region.  value = 32768 * steps / wall time, in tokens per second.

`roofline` is for the dominant kernel of that block, the e4m3 x int8 ffn_y GEMM (44 % of the block's
time; both operands are widened exactly to f16 and multiplied on the f16 matrix cores): algorithmic flops
per launch divided by its mean launch duration, measured with HIP events on the launching stream inside
the timed region, against the MI355X dense f16 MFMA peak.  `roofline.traffic` is read from the rocprofv3
summary under profiles/ named in `roofline.traffic_source` (null when that file is absent).
`cpu_baseline` is the CPU oracle (a port of the reference's arithmetic) timed on a bounded token sample of
the same block on the host cores.  `extras` reports the other benchmark configurations (int8 and fp8 FFN
pairs in TOPS, attention prefill, decode, rms_norm), each as median-of-launches next to the roofline that
bounds it, with a bounded CPU figure per configuration.
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

PEAK_F16_TFLOPS = 2500.0     # dense f16
# launches per measurement, after the reference's own harnesses (attn_fwd_i8.cu:117-182, ffn_f_fwd_f8.cu:108-161):
# 50 warm-up launches, 100 timed (attention: 10 timed), median and minimum reported
GEMM_WARM, GEMM_TIMED = 50, 100
ATTN_WARM, ATTN_TIMED = 50, 10     # (attn_fwd_i8.cu:117: int warmup = 50)
DECODE_WARM, DECODE_TIMED = 50, 100


def profile_traffic(file_name, kernel_name):
	"""HBM bytes per launch as the rocprofv3 summary under profiles/ records them (the line
	`roofline.traffic: N bytes per launch`), with the content hash of the kernel build that summary was taken from
	(`roofline.kernel_key: HASH`, the kernel cache's build.key).  Returns (bytes, key) -- bytes is None when the file or
	the line is missing, or when the kernel being timed now was built from other sources or parameters than the
	profiled one (a summary of another build says nothing about this one)."""
	import re
	from x17ai_amd import _ffi
	try:
		with open(os.path.join(ROOT, "profiles", file_name)) as fh:
			text = fh.read()
	except OSError:
		return None, None
	m = re.search(r"^roofline\.traffic:\s*([0-9]+)\s*bytes per launch", text, re.M)
	k = re.search(r"^roofline\.kernel_key:\s*([0-9a-f]+)", text, re.M)
	try:
		with open(os.path.join(_ffi.kernel_cache_dir(), kernel_name, "build.key")) as fh:
			current = fh.read().strip()
	except OSError:
		current = None
	if not m or not k or current is None or k.group(1) != current:
		return None, current
	return int(m.group(1)), current


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


CONFIG4 = dict(T=8192, B=4, D=2048, H=16, HD=128, W=512, F=8192)


def config4_inputs(rng, rows):
	"""Synthetic block inputs of benchmark config 4 for `rows` token rows: the bf16 residual stream and FixedI8
	weights (N(0,1) codes; the 1/sqrt(fan_in) of the configuration is folded into the kernels' constants exactly as
	src/main.rs:412-421 folds it)."""
	c = CONFIG4
	D, H, HD, F = c["D"], c["H"], c["HD"], c["F"]
	return {
		"x_bf16": (rng.standard_normal((rows, D), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16),
		"attn_q_weights": _rand_codes(rng, (H * HD, D)),
		"attn_kv_weights": _rand_codes(rng, (2 * H * HD, D)),
		"attn_y_weights": _rand_codes(rng, (2 * D, H * HD)),
		"ffn_f_weights": _rand_codes(rng, (2 * F, D)),
		"ffn_y_weights": _rand_codes(rng, (2 * D, F)),
		"sinks_k": _rand_codes(rng, (H, HD)),
		"sinks_v": _rand_codes(rng, (H, HD)),
		"attn_temperature": (0.5 + rng.random(H)).astype(np.float32),
	}


def config4_block(dev, X, fused_qkv=False):
	from x17ai_amd.block import Block, BlockConfig
	c = CONFIG4
	cfg = BlockConfig(c["D"], c["H"], c["HD"], c["F"], c["W"], c["B"], X.BF16, False, fused_qkv)
	block = Block(dev, cfg)
	rows = c["T"] * c["B"]
	inp = config4_inputs(np.random.default_rng(4000), rows)
	w = {k: X.Tensor.from_numpy(dev, v, X.F32 if k == "attn_temperature" else X.INT8) for k, v in inp.items() if k != "x_bf16"}
	x = X.Tensor.from_numpy(dev, inp["x_bf16"], X.BF16)
	block.validate(rows, w)
	out = block.new_outputs(rows)
	return block, x, w, out, rows


def headline(dev, X, steps, warmup, fused_qkv=False):
	"""`steps` block forwards back to back on the stream; an event pair around the dominant launch of each."""
	block, x, w, out, rows = config4_block(dev, X, fused_qkv)
	stages = block.stages(x, w, out)
	dominant = "ffn_y_f8"

	def step(timer=None):
		for name, launch in stages:
			if timer is not None and name == dominant:
				timer.start()
				launch()
				timer.stop()
			else:
				launch()

	for _ in range(warmup):
		step()
	timers = [X.Timer(dev) for _ in range(steps)]
	dev.synchronize()
	t0 = time.perf_counter()
	for t in timers:
		step(t)
	dev.synchronize()
	wall = time.perf_counter() - t0
	ops = block.n_ops(rows)
	return {"wall_s": wall, "rows": rows, "dominant_ops": ops[dominant], "dominant_kernel_name": block.k_ffn_y.name,
	        "dominant_mean_s": sum(t.elapsed_seconds() for t in timers) / steps,
	        "stage_names": [name for name, _ in stages]}


def cpu_baseline():
	"""The CPU oracle over a bounded sample of the config 4 block: the first 4096 tokens of one sequence through all
	seven stages (attention: all 16 heads over those 4096 positions, window 512).  tokens / CPU seconds."""
	from oracle import strict as S
	from x17ai_amd import recipes
	c = CONFIG4
	D, H, HD, F, W = c["D"], c["H"], c["HD"], c["F"], c["W"]
	n = 4096
	inp = config4_inputs(np.random.default_rng(4000), n)
	inp_scale = 1.0 / math.sqrt(D) / 64.0
	t0 = time.perf_counter()
	x = S.rms_norm(inp["x_bf16"], recipes.L2_NORM_EPS, "bf16")
	q = S.epilogue_scale(S.gemm_i32(x, inp["attn_q_weights"]), inp_scale, 8.0)
	kv, _ = S.epilogue_l2norm(S.gemm_i32(x, inp["attn_kv_weights"]), HD, recipes.L2_NORM_EPS, inp_scale, 8.0)
	ao, _ = S.attn_fwd_i8(q, kv, inp["sinks_k"], inp["sinks_v"], inp["attn_temperature"], H, HD, W)
	S.epilogue_residual(S.gemm_i32(ao, inp["attn_y_weights"]), x, 1.0 / math.sqrt(H * HD) / 64.0, 1.0, S.STORE_E4M3)
	f = S.epilogue_geglu(S.gemm_i32(x, inp["ffn_f_weights"]), inp_scale, 1.0, S.STORE_E4M3)
	S.epilogue_residual(S.gemm_f32_seq(f, True, inp["ffn_y_weights"], False), x,
	                    math.sqrt(recipes.GELU_VAR_FIX_2 / F) / 8.0, 1.0, S.STORE_E4M3)
	dt = time.perf_counter() - t0
	return {"value": n / dt, "unit": "tokens/s", "cores": S.num_threads(), "kind": "port",
	        "sample": f"the first {n} tokens of one sequence of config 4 through all seven stages "
	                  f"(16 heads, window 512), {dt:.1f} s of CPU time"}


def cpu_extras():
	"""A bounded CPU figure per remaining configuration, in that configuration's unit."""
	from oracle import strict as S
	from oracle import dense
	from x17ai_amd import recipes
	out = {}
	rng = np.random.default_rng(5000)
	# config 1, the reference's CPU-runnable case: dense float64 attention (new_block.py:183-232 semantics), one head
	# at a time, T=1024, H=8, hd=64, W=256 -- and the strict C port on the same shape
	T1, H1, HD1, W1 = 1024, 8, 64, 256
	qc, kvc = _rand_codes(rng, (T1, H1 * HD1)), _rand_codes(rng, (T1, 2 * H1 * HD1))
	sk, sv = _rand_codes(rng, (H1, HD1)), _rand_codes(rng, (H1, HD1))
	ops1 = 4.0 * HD1 * H1 * (W1 * (W1 - 1) // 2 + (T1 - W1) * W1)
	# one convention for every CPU figure: the threads the strict C port uses (OMP_NUM_THREADS, else the host's cores);
	# numpy's BLAS is held to the same number for the dense figure
	from threadpoolctl import threadpool_limits
	t0 = time.perf_counter()
	with threadpool_limits(limits=S.num_threads()):
		for h in range(H1):
			kh = kvc[:, 2 * h * HD1:(2 * h + 1) * HD1].astype(np.float64) / 8
			vh = kvc[:, (2 * h + 1) * HD1:(2 * h + 2) * HD1].astype(np.float64) / 8
			dense.attn_one_head(qc[:, h * HD1:(h + 1) * HD1].astype(np.float64) / 8, kh, vh, sk[h].astype(np.float64) / 8,
			                    sv[h].astype(np.float64) / 8, 1.0, W1)
	dt = time.perf_counter() - t0
	out["config1_attn_dense_f64"] = {"value": ops1 / dt / 1e12, "unit": "TOPS", "cores": S.num_threads(), "kind": "port",
	                                 "sample": f"all of config 1 (numpy float64, dense [T, T+1] scores, BLAS threads = cores), {dt:.2f} s"}
	t0 = time.perf_counter()
	S.attn_fwd_i8(qc, kvc, sk, sv, np.ones(H1, np.float32), H1, HD1, W1)
	dt = time.perf_counter() - t0
	out["config1_attn_strict"] = {"value": ops1 / dt / 1e12, "unit": "TOPS", "cores": S.num_threads(), "kind": "port",
	                              "sample": f"all of config 1 (strict C port), {dt:.3f} s"}
	# config 2: the int8 FFN pair, 2048 of the 8192 token rows
	M, D, F = 2048, 2048, 8192
	x, w1, w2 = _rand_codes(rng, (M, D)), _rand_codes(rng, (2 * F, D)), _rand_codes(rng, (2 * D, F))
	t0 = time.perf_counter()
	f = S.epilogue_geglu(S.gemm_i32(x, w1), 1.0 / math.sqrt(D) / 64.0, 8.0, S.STORE_I8)
	S.epilogue_residual(S.gemm_i32(f, w2), x, math.sqrt(recipes.GELU_VAR_FIX_2 / F) / 64.0, 1.0, S.STORE_E4M3)
	dt = time.perf_counter() - t0
	out["config2_int8_ffn"] = {"value": (2.0 * M * D * 2 * F + 2.0 * M * F * 2 * D) / dt / 1e12, "unit": "TOPS",
	                           "cores": S.num_threads(), "kind": "port",
	                           "sample": f"{M} of 8192 token rows, both GEMMs + epilogues, {dt:.1f} s"}
	del x, w1, w2, f
	# config 3: the e4m3 FFN pair, 256 of the 16384 token rows (f32 sums in k order)
	M3, D3, F3 = 256, 4096, 16384
	x3, w13, w23 = _rand_e4m3(rng, (M3, D3)), _rand_e4m3(rng, (2 * F3, D3)), _rand_e4m3(rng, (2 * D3, F3))
	r3 = _rand_codes(rng, (M3, D3))
	t0 = time.perf_counter()
	f3 = S.epilogue_geglu(S.gemm_f32_seq(x3, True, w13, True), 1.0 / math.sqrt(D3), 1.0, S.STORE_E4M3)
	S.epilogue_residual(S.gemm_f32_seq(f3, True, w23, True), r3, math.sqrt(recipes.GELU_VAR_FIX_2 / F3), 1.0, S.STORE_E4M3)
	dt = time.perf_counter() - t0
	out["config3_fp8_ffn"] = {"value": (2.0 * M3 * D3 * 2 * F3 + 2.0 * M3 * F3 * 2 * D3) / dt / 1e12, "unit": "TFLOP/s",
	                          "cores": S.num_threads(), "kind": "port",
	                          "sample": f"{M3} of 16384 token rows, both GEMMs + epilogues, {dt:.1f} s"}
	del w13
	del x3, w23, f3
	# config 5: prefill over the first 8192 positions of 2 of the 32 heads; decode of 2 of the 64 sequences
	T5, H5, HD5, W5 = 8192, 8, 128, 4096
	q5, kv5 = _rand_codes(rng, (T5, H5 * HD5)), _rand_codes(rng, (T5, 2 * H5 * HD5))
	sk5, sv5 = _rand_codes(rng, (H5, HD5)), _rand_codes(rng, (H5, HD5))
	t0 = time.perf_counter()
	S.attn_fwd_i8(q5, kv5, sk5, sv5, np.ones(H5, np.float32), H5, HD5, W5, want_l=False)
	dt = time.perf_counter() - t0
	ops5 = 4.0 * HD5 * H5 * (W5 * (W5 - 1) // 2 + (T5 - W5) * W5)
	out["config5_prefill"] = {"value": ops5 / dt / 1e12, "unit": "TOPS", "cores": S.num_threads(), "kind": "port",
	                          "sample": f"positions 0..{T5 - 1} of {H5} of the 32 heads (window 4096), {dt:.1f} s"}
	SD, CAP, HDEC = 16, 4096, 32
	cache = _rand_codes(rng, (SD, CAP, 2 * HDEC * HD5))
	qd = _rand_codes(rng, (SD, HDEC * HD5))
	skd, svd = _rand_codes(rng, (HDEC, HD5)), _rand_codes(rng, (HDEC, HD5))
	t0 = time.perf_counter()
	S.attn_decode_i8(qd, cache, np.full(SD, CAP, np.uint32), skd, svd, np.ones(HDEC, np.float32), HDEC, HD5, W5)
	dt = time.perf_counter() - t0
	out["config5_decode"] = {"value": cache.nbytes / dt / 1e9, "unit": "GB/s of cache", "cores": S.num_threads(), "kind": "port",
	                         "sample": f"{SD} of the 64 sequences (4096 cached positions x 32 heads each), {dt:.2f} s"}
	return out


def extras(dev, X, recipes):
	out = {}
	rng = np.random.default_rng(3000)

	def gemm_entry(kern, a, b, c, extra, peak, iters=GEMM_TIMED, warm=GEMM_WARM):
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
	# both launches back to back, 50 steps after 10 (the headline of earlier versions of this benchmark)
	kf, ky = recipes.ffn_f_kernel(dev, D, 2 * F, False, X.INT8), recipes.ffn_y_kernel(dev, D, F, False, X.INT8, X.INT8)
	def pair():
		kf.launch(x, w1, f)
		ky.launch(f, w2, y, x)
	for _ in range(10):
		pair()
	dev.synchronize()
	t0 = time.perf_counter()
	for _ in range(50):
		pair()
	dev.synchronize()
	c2["pair_back_to_back_tops"] = (kf.n_ops(x, w1) + ky.n_ops(f, w2)) * 50 / (time.perf_counter() - t0) / 1e12
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
		med, mn = _median_launch(dev, X, lambda: kern.launch_dequant(a_, b_, c_, rs, cs_), GEMM_TIMED, GEMM_WARM)
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
	c3 = {"ffn_f_f8": gemm_entry(recipes.ffn_f_f8_kernel(dev, D3, 2 * F3, False), x3, w13, f3, None, PEAK_FP8_TFLOPS)}
	del w13
	w23 = X.Tensor.from_numpy(dev, e4m3_rand((2 * D3, F3)), X.E4M3)
	r3 = X.Tensor.from_numpy(dev, _rand_codes(rng, (M3, D3)), X.INT8)
	y3 = X.Tensor(dev, (M3, D3), X.E4M3)
	c3["ffn_y_f8"] = gemm_entry(recipes.ffn_y_kernel(dev, D3, F3, False, X.E4M3, X.E4M3), f3, w23, y3, r3, PEAK_FP8_TFLOPS)
	out["config3_fp8_ffn"] = c3
	del x3, w23, f3, r3, y3

	# ---- config 4 per stage (the headline's block): median of each stage launched alone, both projection forms
	c = CONFIG4
	T, B, H, HD, W, F4 = c["T"], c["B"], c["H"], c["HD"], c["W"], c["F"]
	c4 = {}
	for fused in (False, True) if hasattr(recipes, "attn_qkv_kernel") else (False,):
		block, xb, wts, outs, rows = config4_block(dev, X, fused)
		ops = block.n_ops(rows)
		total = 0.0
		for name, fn in block.stages(xb, wts, outs):
			if fused and name != "attn_qkv":
				continue
			iters, warm = (ATTN_TIMED, ATTN_WARM) if name == "attn_fwd_i8" else (GEMM_TIMED, GEMM_WARM)
			med, mn = _median_launch(dev, X, fn, iters, warm)
			c4[name + "_us"] = med * 1e6
			if name in ops:
				c4[name + "_tops"] = ops[name] / med / 1e12
			total += med
		if not fused:
			c4["sum_of_stage_medians_us"] = total * 1e6
		del block, xb, wts, outs
	pairs = W * (W - 1) // 2 + (T - W) * W
	c4["attn_fwd_i8_tops"] = 4.0 * HD * H * B * pairs / (c4["attn_fwd_i8_us"] * 1e-6) / 1e12     # visible (query, key) pairs only
	c4["attn_frac_of_int8_peak"] = c4["attn_fwd_i8_tops"] / PEAK_INT8_TOPS
	c4["rms_norm_gbs"] = rows * D * 3 / (c4["rms_norm_us"] * 1e-6) / 1e9
	c4["rms_norm_frac_of_hbm"] = c4["rms_norm_gbs"] / PEAK_HBM_GBS
	for name in ("attn_q", "attn_kv", "attn_qkv", "attn_y", "ffn_f"):
		if name + "_tops" in c4:
			c4[name + "_frac_of_int8_peak"] = c4[name + "_tops"] / PEAK_INT8_TOPS
	c4["ffn_y_f8_frac_of_f16_peak"] = c4["ffn_y_f8_tops"] / PEAK_F16_TFLOPS
	out["config4_block_stages"] = c4
	# the attention backward with respect to q at the same attention shape (first kernel of the backward path)
	rowsb = T * B
	qb_ = X.Tensor.from_numpy(dev, _rand_codes(rng, (rowsb, H * HD)), X.INT8)
	kvb = X.Tensor.from_numpy(dev, _rand_codes(rng, (rowsb, 2 * H * HD)), X.INT8)
	skb = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
	svb = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
	tpb = X.Tensor.from_numpy(dev, (0.5 + rng.random(H)).astype(np.float32), X.F32)
	ob, lb = X.Tensor(dev, (rowsb, H * HD), X.INT8), X.Tensor(dev, (H, rowsb), X.F32)
	recipes.attn_kernel(dev, H, HD, False).launch(qb_, kvb, skb, svb, tpb, ob, lb, W, B)
	dob = X.Tensor.from_numpy(dev, (rng.standard_normal((rowsb, H * HD), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16), X.BF16)
	dqb, ddb = X.Tensor(dev, (rowsb, H * HD), X.BF16), X.Tensor(dev, (H, rowsb), X.F32)
	kb_ = recipes.attn_d_q_kernel(dev, H, HD, False)
	med, _ = _median_launch(dev, X, lambda: kb_.launch_d_q(qb_, kvb, skb, svb, tpb, ob, dob, dqb, lb, ddb, W, B), ATTN_TIMED, ATTN_WARM)
	out["config4_attn_d_q"] = {"median_us": med * 1e6, "tops": 6.0 * HD * H * B * pairs / med / 1e12,
	                           "note": "QK on the int8 matrix cores, dP and dQ on the f16 cores: 6 hd multiply-adds per visible (query, key) pair"}
	# ... and with respect to k and v (consumes the D the dQ launch wrote)
	dkvb = X.Tensor(dev, (rowsb, 2 * H * HD), X.BF16)
	kkv = recipes.attn_d_kv_kernel(dev, H, HD, False)
	med, _ = _median_launch(dev, X, lambda: kkv.launch_d_kv(qb_, kvb, tpb, dob, lb, ddb, dkvb, W, B), ATTN_TIMED, ATTN_WARM)
	out["config4_attn_d_kv"] = {"median_us": med * 1e6, "tops": 8.0 * HD * H * B * pairs / med / 1e12,
	                            "note": "QK on the int8 matrix cores, dP, dV and dK on the bf16 cores: 8 hd multiply-adds per visible (query, key) pair"}
	del qb_, kvb, ob, lb, dob, dqb, ddb, dkvb

	# ---- config 1: attention T=1024, H=8, hd=64, W=256
	T1, H1, HD1, W1 = 1024, 8, 64, 256
	q1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T1, H1 * HD1)), X.INT8)
	kv1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (T1, 2 * H1 * HD1)), X.INT8)
	sk1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H1, HD1)), X.INT8)
	sv1 = X.Tensor.from_numpy(dev, _rand_codes(rng, (H1, HD1)), X.INT8)
	tp1 = X.Tensor.from_numpy(dev, np.ones(H1, np.float32), X.F32)
	o1 = X.Tensor(dev, (T1, H1 * HD1), X.INT8)
	k1 = recipes.attn_kernel(dev, H1, HD1, False)
	med, _ = _median_launch(dev, X, lambda: k1.launch(q1, kv1, sk1, sv1, tp1, o1, None, W1), 100, 50)
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
	med, _ = _median_launch(dev, X, lambda: k1r.launch_row_scaled(q1, kv1, sk1, sv1, tp1, ob1, None, W1, *rs1), 100, 50)
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
		med, _ = _median_launch(dev, X, lambda: k5.launch(q5, kv5, sk5, sv5, tp5, o5, None, W5), ATTN_TIMED, ATTN_WARM)
		p5 = W5 * (W5 - 1) // 2 + (T5 - W5) * W5
		tag = "strict" if strict else "fast"
		c5[f"prefill_{tag}_ms"] = med * 1e3
		c5[f"prefill_{tag}_tops"] = 4.0 * HD5 * H5 * p5 / med / 1e12
		c5[f"prefill_{tag}_frac_of_int8_peak"] = c5[f"prefill_{tag}_tops"] / PEAK_INT8_TOPS
	rs5 = row_scale_tensors(T5, H5)
	ob5 = X.Tensor(dev, (T5, H5 * HD5), X.BF16)
	k5r = recipes.attn_row_scaled_kernel(dev, H5, HD5, X.BF16, False)
	med, _ = _median_launch(dev, X, lambda: k5r.launch_row_scaled(q5, kv5, sk5, sv5, tp5, ob5, None, W5, *rs5), ATTN_TIMED, ATTN_WARM)
	c5["prefill_row_scaled_bf16_ms"] = med * 1e3
	c5["prefill_row_scaled_bf16_tops"] = 4.0 * HD5 * H5 * p5 / med / 1e12
	del q5, kv5, o5, ob5, rs5
	S5, CAP = 64, 4096
	one = _rand_codes(rng, (1, CAP, 2 * H5 * HD5))
	cache = X.Tensor.from_numpy(dev, np.ascontiguousarray(np.broadcast_to(one, (S5, CAP, 2 * H5 * HD5))), X.INT8)
	qd = X.Tensor.from_numpy(dev, _rand_codes(rng, (S5, H5 * HD5)), X.INT8)
	lens = X.Tensor.from_numpy(dev, np.full(S5, CAP, np.uint32).view(np.float32), X.F32)
	od = X.Tensor(dev, (S5, H5 * HD5), X.INT8)
	nbytes = S5 * CAP * 2 * H5 * HD5                  # the whole cache: what the recurrence reads when no probability rounds to 0
	q_flat = X.Tensor.from_numpy(dev, np.zeros((S5, H5 * HD5), np.int8), X.INT8)
	for strict in (False, True):
		kd = recipes.attn_decode_kernel(dev, H5, HD5, CAP, strict)
		tag = "strict" if strict else "fast"
		# dense case: an all-zero query gives every key the same score, so every 8-bit probability is 255 and every
		# K and V row of the window is read -- the roofline figure of the kernel
		med, _ = _median_launch(dev, X, lambda: kd.launch(q_flat, cache, lens, sk5, sv5, tp5, od, None, W5), DECODE_TIMED, DECODE_WARM)
		c5[f"decode_dense_{tag}_us"] = med * 1e6
		c5[f"decode_dense_{tag}_gbs"] = nbytes / med / 1e9
		c5[f"decode_dense_{tag}_frac_of_hbm"] = nbytes / med / 1e9 / PEAK_HBM_GBS
		# Gaussian queries and cache: about 99 % of the 8-bit probabilities are 0 and their V rows are not fetched.
		# The rate below divides the WHOLE cache by the time: work avoided, not bandwidth (it can exceed the HBM peak).
		med, _ = _median_launch(dev, X, lambda: kd.launch(qd, cache, lens, sk5, sv5, tp5, od, None, W5), DECODE_TIMED, DECODE_WARM)
		c5[f"decode_gaussian_{tag}_us"] = med * 1e6
		c5[f"decode_gaussian_{tag}_cache_gbs_work_avoided"] = nbytes / med / 1e9
	# the cache as a row-scaled prefill leaves it: one scale per (row, head) of k and v, bf16 output
	kd_rows = recipes.attn_decode_row_scaled_kernel(dev, H5, HD5, CAP, X.BF16, False)
	scale_one = [(0.125 * (0.75 + 0.5 * rng.random((1, H5, CAP)))).astype(np.float32) for _ in range(2)]
	vw5, sw5, os5 = recipes.attn_row_scale_operands(np.broadcast_to(scale_one[1], (S5, H5, CAP)), X.BF16)
	f32t = lambda a: X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32)
	rsd = [f32t(0.125 * (0.75 + 0.5 * rng.random((S5, H5)))), f32t(np.broadcast_to(scale_one[0], (S5, H5, CAP))), f32t(vw5), f32t(sw5), f32t(os5)]
	odb = X.Tensor(dev, (S5, H5 * HD5), X.BF16)
	med, _ = _median_launch(dev, X, lambda: kd_rows.launch_row_scaled(qd, cache, lens, sk5, sv5, tp5, odb, None, W5, *rsd), DECODE_TIMED, DECODE_WARM)
	c5["decode_row_scaled_bf16_us"] = med * 1e6
	out["config5_long_context"] = c5
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
	elif name == "attn_row_scaled_config5":
		T, H, HD, W = 65536, 32, 128, 4096
		q = X.Tensor.from_numpy(dev, _rand_codes(rng, (T, H * HD)), X.INT8)
		kv = X.Tensor.from_numpy(dev, _rand_codes(rng, (T, 2 * H * HD)), X.INT8)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, np.ones(H, np.float32), X.F32)
		scales = [(0.125 * (0.75 + 0.5 * rng.random((H, T)))).astype(np.float32) for _ in range(3)]
		vw, sw, osc = recipes.attn_row_scale_operands(scales[2], X.BF16)
		rs = [X.Tensor.from_numpy(dev, np.ascontiguousarray(a, dtype=np.float32), X.F32) for a in (scales[0], scales[1], vw, sw, osc)]
		o = X.Tensor(dev, (T, H * HD), X.BF16)
		k = recipes.attn_row_scaled_kernel(dev, H, HD, X.BF16, False)
		pairs = W * (W - 1) // 2 + (T - W) * W
		fn, work, unit = (lambda: k.launch_row_scaled(q, kv, sk, sv, tp, o, None, W, *rs)), 4.0 * HD * H * pairs / 1e12, "TOPS"
	elif name == "attn_d_q_config4":
		# the backward with respect to q at the attention shape of config 4 (QK + dP + dQ: 6 hd multiply-adds per pair)
		T, B, H, HD, W = 8192, 4, 16, 128, 512
		rows = T * B
		q = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, H * HD)), X.INT8)
		kv = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, 2 * H * HD)), X.INT8)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, (0.5 + rng.random(H)).astype(np.float32), X.F32)
		o = X.Tensor(dev, (rows, H * HD), X.INT8)
		l = X.Tensor(dev, (H, rows), X.F32)
		recipes.attn_kernel(dev, H, HD, False).launch(q, kv, sk, sv, tp, o, l, W, B)
		d_o = X.Tensor.from_numpy(dev, (rng.standard_normal((rows, H * HD), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16), X.BF16)
		dq = X.Tensor(dev, (rows, H * HD), X.BF16)
		dd = X.Tensor(dev, (H, rows), X.F32)
		k = recipes.attn_d_q_kernel(dev, H, HD, False)
		pairs = W * (W - 1) // 2 + (T - W) * W
		fn, work, unit = (lambda: k.launch_d_q(q, kv, sk, sv, tp, o, d_o, dq, l, dd, W, B)), 6.0 * HD * H * B * pairs / 1e12, "TOPS"
	elif name == "attn_d_kv_config4":
		# the backward with respect to k and v at the attention shape of config 4 (QK + dP + dV + dK: 8 hd multiply-adds per pair)
		T, B, H, HD, W = 8192, 4, 16, 128, 512
		rows = T * B
		q = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, H * HD)), X.INT8)
		kv = X.Tensor.from_numpy(dev, _rand_codes(rng, (rows, 2 * H * HD)), X.INT8)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, (0.5 + rng.random(H)).astype(np.float32), X.F32)
		o = X.Tensor(dev, (rows, H * HD), X.INT8)
		l = X.Tensor(dev, (H, rows), X.F32)
		recipes.attn_kernel(dev, H, HD, False).launch(q, kv, sk, sv, tp, o, l, W, B)
		d_o = X.Tensor.from_numpy(dev, (rng.standard_normal((rows, H * HD), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16), X.BF16)
		dq = X.Tensor(dev, (rows, H * HD), X.BF16)
		dd = X.Tensor(dev, (H, rows), X.F32)
		recipes.attn_d_q_kernel(dev, H, HD, False).launch_d_q(q, kv, sk, sv, tp, o, d_o, dq, l, dd, W, B)
		dkv = X.Tensor(dev, (rows, 2 * H * HD), X.BF16)
		k = recipes.attn_d_kv_kernel(dev, H, HD, False)
		pairs = W * (W - 1) // 2 + (T - W) * W
		fn, work, unit = (lambda: k.launch_d_kv(q, kv, tp, d_o, l, dd, dkv, W, B)), 8.0 * HD * H * B * pairs / 1e12, "TOPS"
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
	elif name == "decode_dense_config5":
		# an all-zero query: every key scores the same, every 8-bit probability is 255, every K and V row is read
		S5, CAP, H, HD, W = 64, 4096, 32, 128, 4096
		one = _rand_codes(rng, (1, CAP, 2 * H * HD))
		cache = X.Tensor.from_numpy(dev, np.ascontiguousarray(np.broadcast_to(one, (S5, CAP, 2 * H * HD))), X.INT8)
		qd = X.Tensor.from_numpy(dev, np.zeros((S5, H * HD), np.int8), X.INT8)
		lens = X.Tensor.from_numpy(dev, np.full(S5, CAP, np.uint32).view(np.float32), X.F32)
		sk = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		sv = X.Tensor.from_numpy(dev, _rand_codes(rng, (H, HD)), X.INT8)
		tp = X.Tensor.from_numpy(dev, np.ones(H, np.float32), X.F32)
		od = X.Tensor(dev, (S5, H * HD), X.INT8)
		k = recipes.attn_decode_kernel(dev, H, HD, CAP, False)
		fn, work, unit = (lambda: k.launch(qd, cache, lens, sk, sv, tp, od, None, W)), S5 * CAP * 2 * H * HD / 1e9, "GB/s"
	elif name in ("attn_kv_config4", "attn_qkv_config4", "ffn_f_config4", "attn_y_config4"):
		M, H, HD = 32768, 16, 128
		a = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
		if name == "attn_kv_config4":
			b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * H * HD, D)), X.INT8)
			c, rr = X.Tensor(dev, (M, 2 * H * HD), X.INT8), X.Tensor(dev, (M, H), X.F32)
			k = recipes.attn_kv_kernel(dev, D, 2 * H * HD, HD, False)
			fn, work = (lambda: k.launch(a, b, c, rr)), k.n_ops(a, b) / 1e12
		elif name == "attn_qkv_config4":
			bq = X.Tensor.from_numpy(dev, _rand_codes(rng, (H * HD, D)), X.INT8)
			b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * H * HD, D)), X.INT8)
			cq, c, rr = X.Tensor(dev, (M, H * HD), X.INT8), X.Tensor(dev, (M, 2 * H * HD), X.INT8), X.Tensor(dev, (M, H), X.F32)
			k = recipes.attn_qkv_kernel(dev, D, H * HD, 2 * H * HD, HD, False)
			fn, work = (lambda: k.launch_qkv(a, bq, b, cq, c, rr)), 2.0 * M * D * 3 * H * HD / 1e12
		elif name == "ffn_f_config4":
			b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * F, D)), X.INT8)
			c = X.Tensor(dev, (M, F), X.E4M3)
			k = recipes.ffn_f_kernel(dev, D, 2 * F, False)
			fn, work = (lambda: k.launch(a, b, c)), k.n_ops(a, b) / 1e12
		else:
			b = X.Tensor.from_numpy(dev, _rand_codes(rng, (2 * D, H * HD)), X.INT8)
			r = X.Tensor.from_numpy(dev, _rand_codes(rng, (M, D)), X.INT8)
			c = X.Tensor(dev, (M, D), X.E4M3)
			k = recipes.attn_y_kernel(dev, D, H * HD, False)
			fn, work = (lambda: k.launch(a, b, c, r)), k.n_ops(a, b) / 1e12
		unit = "TOPS"
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


ONLY_TARGETS = ("ffn_f_config2", "ffn_f_f8_config3", "ffn_y_f8_config4", "attn_config4", "attn_config5", "attn_row_scaled_config5",
                "attn_d_q_config4", "attn_d_kv_config4", "decode_config5",
                "decode_dense_config5", "attn_kv_config4", "attn_qkv_config4", "ffn_f_config4", "attn_y_config4", "rms_norm_config4")


def main():
	ap = argparse.ArgumentParser()
	ap.add_argument("--gpus", type=int, default=1)
	ap.add_argument("--steps", type=int, default=50)
	ap.add_argument("--warmup", type=int, default=10)
	ap.add_argument("--no-extras", action="store_true")
	ap.add_argument("--no-cpu", action="store_true")
	ap.add_argument("--separate-qkv", action="store_true",
	                help="headline block with the q and kv projections as two launches, as src/main.rs launches them "
	                     "(default: one launch that reads x once)")
	ap.add_argument("--only", choices=ONLY_TARGETS,
	                help="launch one kernel of one workload --steps times and print its median (used for the profiles)")
	args = ap.parse_args()
	if args.gpus != 1:
		print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
		sys.exit(2)

	import x17ai_amd as X
	from x17ai_amd import recipes

	dev = X.Device(0)
	if args.only:
		single(dev, X, recipes, args.only, args.steps)
		return
	h = headline(dev, X, args.steps, args.warmup, not args.separate_qkv)
	value = h["rows"] * args.steps / h["wall_s"]
	achieved = h["dominant_ops"] / h["dominant_mean_s"] / 1e12
	traffic_file = "gemm_b8_ffn_y_f8_config4.txt"
	traffic, kernel_key = profile_traffic(traffic_file, h["dominant_kernel_name"])
	c = CONFIG4
	line = {
		"metric": "block-fwd tokens/sec at 1 MI355X (config 4: full quantized block forward); int8/fp8 TOPS and % of "
		          "MFMA/HBM roofline per kernel under extras",
		"value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
		"ms_per_step": h["wall_s"] / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
		"vs_baseline": None, "dtype": "int8", "data": "synthetic",
		"config": {"workload": f"config 4: full quantized block forward, batch {c['B']} x seq {c['T']} tokens, d_model {c['D']}, "
		                       f"{c['H']} heads x {c['HD']}, window {c['W']}, d_ff {c['F']}; stages " + " -> ".join(h["stage_names"]),
		           "operands": "bf16 residual stream in; FixedI8 x, q, kv, attention out; int8 weights; e4m3 attn_y, ffn_f, ffn_y "
		                       "(int8 x int8 -> int32 on the int8 matrix cores; ffn_y e4m3 x int8 -> f32 on the f16 matrix cores)",
		           "math": "hardware transcendentals in the epilogues and the softmax (the bit-exact strict builds are the tests')"},
		"roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
		             "frac": achieved / PEAK_F16_TFLOPS, "traffic": traffic,
		             "traffic_source": "profiles/" + traffic_file if traffic is not None else None,
		             "kernel_key": kernel_key,
		             "kernel": "gemm_b8 (ffn_y_fwd_f8: M=32768, K=8192, N_raw=4096, e4m3 x int8 widened to f16, gated-residual epilogue)",
		             "mean_launch_us": h["dominant_mean_s"] * 1e6},
	}
	if not args.no_cpu:
		line["cpu_baseline"] = cpu_baseline()
	if not args.no_extras:
		line["extras"] = extras(dev, X, recipes)
		if not args.no_cpu:
			line["extras"]["cpu_baselines"] = cpu_extras()
	dev.synchronize()
	print(json.dumps(line))


if __name__ == "__main__":
	main()
