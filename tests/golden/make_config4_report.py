"""Writes tests/golden/config4_fast_vs_strict.json on a machine with an MI355X: benchmark config 4 as one chain
(tests/config4_chain.py), the strict builds checked against the CPU oracle, then per stage the speed build against
the strict one -- mismatch histogram, max-abs and relative-L2 difference over the whole tensors.  The same
comparison for the FFN pairs of benchmark configs 2 (int8) and 3 (e4m3) at their full sizes is appended.

    python tests/golden/make_config4_report.py [output.json]
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import x17ai_amd as X
from tests import config4_chain as C


def ffn_pairs():
	"""Speed build against strict build over the whole outputs of the config 2 and config 3 FFN pairs (the strict
	builds of these shapes are held against the oracle on sampled rows by tests/test_gpu_fullsize.py)."""
	import numpy as np
	from x17ai_amd import recipes
	from tests.gpu_common import e4m3_bytes, i8_codes, rng_for
	dev = X.Device(0)
	up = lambda a, dt: X.Tensor.from_numpy(dev, a, dt)
	rep = {}
	# config 2: x i8 [8192, 2048], W1 [16384, 2048] -> GeGLU -> f FixedI8 [8192, 8192]; W2 [4096, 8192] -> residual -> e4m3
	m, d, f = 8192, 2048, 8192
	rng = rng_for("report-config2")
	x, w1, w2 = up(i8_codes(rng, (m, d)), X.INT8), up(i8_codes(rng, (2 * f, d)), X.INT8), up(i8_codes(rng, (2 * d, f)), X.INT8)
	out = {}
	for strict in (True, False):
		tf, ty = X.Tensor(dev, (m, f), X.INT8), X.Tensor(dev, (m, d), X.E4M3)
		recipes.ffn_f_kernel(dev, d, 2 * f, strict, X.INT8).launch(x, w1, tf)
		if strict:
			f_strict = tf
		recipes.ffn_y_kernel(dev, d, f, strict, X.INT8, X.INT8).launch(f_strict, w2, ty, x)      # both on the strict f
		out[strict] = (tf.download(), ty.download())
	rep["config2_ffn_f_i8"] = C._i8_diff(out[False][0], out[True][0])
	rep["config2_ffn_y_i8_to_e4m3"] = C._e4m3_diff(out[False][1], out[True][1])
	del x, w1, w2, out, f_strict
	# config 3: x e4m3 [16384, 4096], W1 [32768, 4096] -> GeGLU -> f e4m3 [16384, 16384]; W2 [8192, 16384] -> residual -> e4m3
	m, d, f = 16384, 4096, 16384
	rng = rng_for("report-config3")
	x, w1 = up(e4m3_bytes(rng, (m, d)), X.E4M3), up(e4m3_bytes(rng, (2 * f, d)), X.E4M3)
	fs = {}
	for strict in (True, False):
		tf = X.Tensor(dev, (m, f), X.E4M3)
		recipes.ffn_f_f8_kernel(dev, d, 2 * f, strict).launch(x, w1, tf)
		fs[strict] = tf
	rep["config3_ffn_f_f8"] = C._e4m3_diff(fs[False].download(), fs[True].download())
	del x, w1
	w2, r = up(e4m3_bytes(rng, (2 * d, f)), X.E4M3), up(i8_codes(rng, (m, d)), X.INT8)
	ys = {}
	for strict in (True, False):
		ty = X.Tensor(dev, (m, d), X.E4M3)
		recipes.ffn_y_kernel(dev, d, f, strict, X.E4M3, X.E4M3).launch(fs[True], w2, ty, r)
		ys[strict] = ty.download()
	rep["config3_ffn_y_f8"] = C._e4m3_diff(ys[False], ys[True])
	return rep


def main():
	out_path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "tests", "golden", "config4_fast_vs_strict.json")
	dev = X.Device(0)
	inp = C.inputs()
	got = C.run_strict(dev, inp)
	checked = C.check_strict(inp, got)
	rep = {"workload": f"config 4: {C.B} x {C.T} tokens, d_model {C.D}, {C.H} heads x {C.HD}, window {C.W}, d_ff {C.F}",
	       "device": dev.name, "strict_vs_oracle": checked, "fast_vs_strict": C.fast_vs_strict(dev, inp, got)}
	del got, inp
	rep["ffn_pairs_fast_vs_strict"] = ffn_pairs()
	with open(out_path, "w") as f:
		json.dump(rep, f, indent=1)
		f.write("\n")
	print(json.dumps(rep))


if __name__ == "__main__":
	main()
