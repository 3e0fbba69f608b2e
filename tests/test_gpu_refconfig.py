"""The reference's own golden run (block.config.json:2-9: 16384 tokens, model width 2048, 64 heads of 32,
no window, FFN width 2048) through the HIP kernels.

The inputs are regenerated from torch's seed (tests/refconfig.py), every stage runs on the GPU in its
strict_math build, and the results are held against
  * the CPU oracle on the same inputs: bit for bit over the whole tensor for the int8 GEMM stages, over
    sampled heads for the attention (all 16384 queries of each), to one e4m3 code for the f32-accumulated stage,
  * the numbers of the reference's report (expected.txt, cited per assert) where the report's torch side
    or CUDA side pins them, and
  * the statistics the oracle produced for the whole attention output at this configuration
    (tests/golden/attn_refconfig_report.txt, a ten-minute CPU run): equal mean and variance over all
    33.5 M output codes, so the unsampled heads are covered as well.
"""
import json
import math
import os

import numpy as np
import pytest

import x17ai_amd as X
from x17ai_amd.block import Block, BlockConfig
from oracle import dense as D
from oracle import strict as S
from tests import refconfig as R
from tests.gpu_common import e4m3_compare

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
	d = X.Device(0)
	yield d
	d.synchronize()


@pytest.fixture(scope="module")
def ref():
	return R.inputs()


def _up(dev, arr, dtype):
	return X.Tensor.from_numpy(dev, np.ascontiguousarray(arr), dtype)


@pytest.fixture(scope="module")
def stages(dev, ref):
	"""q, kv (+ rrms), attention (+ L), attn_y, ffn_f, ffn_y of the reference run, computed on the GPU by the block
	object in main.rs's stage order (src/main.rs:193-263)."""
	block = Block(dev, BlockConfig(R.MODEL_DIM, R.N_HEADS, R.HEAD_DIM, R.F_WIDTH, 0, 1, None, True))
	w = {k: _up(dev, v, X.F32 if k == "attn_temperature" else X.INT8) for k, v in ref.items() if k != "x"}
	out = block.forward(_up(dev, ref["x"], X.INT8), w)
	names = {"q": "q", "kv": "kv", "k_rrms": "rrms", "attn_out": "attn_out", "attn_l": "attn_l", "attn_y": "attn_y",
	         "ffn_f": "ffn_f", "ffn_y": "ffn_y"}
	return {names[k]: t.download() for k, t in out.items()}


INP = 1.0 / math.sqrt(R.MODEL_DIM) / 64.0        # src/main.rs:412-416, 461-469, 599-603


def test_q_and_kv_projections(ref, stages):
	acc = R.acc_exact(ref["x"], ref["attn_q_weights"])
	assert np.array_equal(stages["q"], S.epilogue_scale(acc, INP, 8.0))
	mn, mx, mean, var = R.i8_stats(stages["q"])
	assert (mn, mx) == (-47, 44)                                                   # expected.txt:7-8
	assert f"{mean:.6e}" == "-7.706583e-04" and f"{var:.6e}" == "6.426495e+01"     # expected.txt:9-10 (A == B, :11)
	acc = R.acc_exact(ref["x"], ref["attn_kv_weights"])
	kv, rrms = S.epilogue_l2norm(acc, R.HEAD_DIM, R.L2_NORM_EPS, INP, 8.0)
	assert np.array_equal(stages["kv"], kv)
	assert np.array_equal(stages["rrms"].view(np.uint32), rrms.view(np.uint32))
	mn, mx, mean, var = R.i8_stats(stages["kv"])
	assert (mn, mx) == (-57, 56)                                                   # expected.txt:22-23
	assert abs(mean - (-1.544356e-03)) < 5e-7 and f"{var:.6e}" == "8.622969e+01"   # expected.txt:24 (CUDA side)


def test_attention_sampled_heads_and_whole_output_statistics(ref, stages):
	t, h, hd = R.SEQ_LEN, R.N_HEADS, R.HEAD_DIM
	heads = [0, 37, 63]
	cols = lambda a, w: np.ascontiguousarray(np.concatenate([a[:, i * w:(i + 1) * w] for i in heads], axis=1))
	want, want_l = S.attn_fwd_i8(cols(stages["q"], hd), cols(stages["kv"], 2 * hd), ref["sinks_k"][heads], ref["sinks_v"][heads],
	                             ref["attn_temperature"][heads], len(heads), hd, 0)
	assert np.array_equal(cols(stages["attn_out"], hd), want)
	assert np.array_equal(stages["attn_l"][heads].view(np.uint32), want_l.view(np.uint32))
	# all 64 heads: the oracle's statistics over the whole output, recorded by its full-size run
	path = os.path.join(os.path.dirname(__file__), "golden", "attn_refconfig_report.txt")
	text = open(path).read()
	report = json.loads(text[text.index("{"):])
	mn, mx, mean, var = R.i8_stats(stages["attn_out"])
	assert (mn, mx) == (-51, 53)                                                   # expected.txt:64
	assert mean == report["B_mean"] and var == report["B_var"]
	assert abs(var - 4.497738e+01) < 2e-3 and abs(mean - (-1.945496e-03)) < 2e-4  # expected.txt:66 (CUDA side)


def test_attn_y_and_ffn(ref, stages):
	x = ref["x"]
	# attn_y: int8 GEMM over the GPU's own attention output, gated residual, e4m3 store (src/main.rs:546)
	acc = R.acc_exact(stages["attn_out"], ref["attn_y_weights"])
	inp = 1.0 / math.sqrt(R.ATTN_WIDTH) / 64.0                                     # src/main.rs:548-557
	assert np.array_equal(stages["attn_y"], S.epilogue_residual(acc, x, inp, 1.0, S.STORE_E4M3))
	# ffn_f: GeGLU -> e4m3
	acc = R.acc_exact(x, ref["ffn_f_weights"])
	f_strict = S.epilogue_geglu(acc, INP, 1.0)
	assert np.array_equal(stages["ffn_f"], f_strict)
	f_pregate = (acc.astype(np.float64) / 64.0) * (1.0 / math.sqrt(float(R.MODEL_DIM)))
	f_dense = D.quantize_e4m3(D.geglu(f_pregate))                                  # new_block.py:134-140
	n_neq = int(np.count_nonzero(S.e4m3_to_f32(stages["ffn_f"]).astype(np.float64) != f_dense))
	assert n_neq <= 4000, n_neq                                                    # expected.txt:141: 1661 for the CUDA kernels
	# ffn_y: e4m3 x int8 with f32 accumulation inside the matrix cores: one e4m3 code at most, rarely
	rows = slice(0, 2048)
	acc = S.gemm_f32_seq(stages["ffn_f"][rows], True, ref["ffn_y_weights"], False)
	inp = math.sqrt(D.GELU_VAR_FIX_2 / R.F_WIDTH) / 8.0                            # src/main.rs:650-660
	y_strict = S.epilogue_residual(acc, x[rows], inp, 1.0, S.STORE_E4M3)
	frac, beyond = e4m3_compare(stages["ffn_y"][rows], y_strict)
	assert frac < 5e-3 and beyond == 0.0, (frac, beyond)
