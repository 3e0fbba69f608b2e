"""Dense float64 restatement of the reference's PyTorch-CPU oracle (new_block.py).

TEST INFRASTRUCTURE ONLY (same rules as oracle/strict.py).  This is the reference's
"CPU path": float64 everywhere, dense [T, T+1] score matrices, textbook formulas.
It is used (i) to pin the strict C oracle (which follows the CUDA op sequence instead)
through mismatch statistics of the kind the reference's own golden report
(expected.txt) accepts, and (ii) as a readable statement of what every stage means.
"""
from __future__ import annotations

import math

import numpy as np

FIXED_I8_SCALE = 8.0

# block_utils.py:32-36 == cuda/utils_core.cuh:414-418 == src/main.rs:650
GELU_VAR_FIX_2 = 1.0 / ((1.0 / 3.0) + (0.5 / math.pi) * (1.0 / math.sqrt(3.0)))
GELU_VAR_FIX = math.sqrt(GELU_VAR_FIX_2)


def quantize(a: np.ndarray) -> np.ndarray:
	"""new_block.py:12-13 -- FixedI8 grid, returned as real values (code / 8)."""
	return np.clip(np.rint(a * 8.0), -127.0, 127.0) / 8.0


def quantize_i8_codes(a: np.ndarray) -> np.ndarray:
	"""new_block.py:15-16"""
	return np.clip(np.rint(a * 8.0), -127.0, 127.0).astype(np.int32)


def store_i8_codes(a: np.ndarray) -> np.ndarray:
	"""block_utils.py:163-166 -- how a tensor is written to an *_i8 file: through float32."""
	w = np.asarray(a, dtype=np.float64).astype(np.float32)
	return np.clip(np.rint(w * np.float32(8.0)), -127.0, 127.0).astype(np.int32)


def e4m3_ftz(a: np.ndarray) -> np.ndarray:
	"""block_utils.py:126-137 -- flush what would not round up to the smallest normal."""
	threshold = (1.0 + 15.0 / 16.0) * 2.0 ** -7
	return np.where(np.abs(a) < threshold, 0.0, a)


def e4m3_rne(a: np.ndarray) -> np.ndarray:
	"""Round to the OCP e4m3fn grid, ties to even, saturating at +-448; what torch's
	.to(float8_e4m3fn) does for the non-subnormal range used by the reference
	(new_block.py:18-19): torch narrows float64 to float32 first, then rounds once more, and
	that double rounding is kept here.  Inputs are expected to be e4m3_ftz()'d already."""
	a = np.asarray(a, dtype=np.float64).astype(np.float32).astype(np.float64)
	out = np.zeros_like(a)
	nz = a != 0.0
	mag = np.abs(a[nz])
	e = np.floor(np.log2(mag))
	e = np.maximum(e, -6.0)                 # below 2^-6 the grid spacing stays 2^-9
	step = 2.0 ** (e - 3.0)
	r = np.rint(mag / step) * step
	r = np.minimum(r, 448.0)
	out[nz] = np.sign(a[nz]) * r
	return out


def quantize_e4m3(a: np.ndarray) -> np.ndarray:
	"""new_block.py:18-19"""
	return e4m3_rne(e4m3_ftz(a))


def rms_norm(x: np.ndarray, eps: float):
	"""new_block.py:83-85"""
	rrms = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
	return x * rrms, rrms


def gelu(x: np.ndarray) -> np.ndarray:
	"""new_block.py:87-91"""
	ck = math.sqrt(2.0 / math.pi)
	ck3 = 0.044715 * ck
	y = ck3 * x * x * x + ck * x
	return 0.5 * x * np.tanh(y) + 0.5 * x


def geglu(x: np.ndarray) -> np.ndarray:
	"""new_block.py:93-96 -- even columns gate, odd columns linear."""
	return gelu(x[..., 0::2]) * x[..., 1::2]


def sigmoid_base4(x: np.ndarray) -> np.ndarray:
	"""new_block.py:98-105"""
	return 1.0 / (1.0 + np.exp2(-2.0 * x))


def softplus_base4(x: np.ndarray) -> np.ndarray:
	"""new_block.py:107-108 (written overflow-safe)."""
	return np.maximum(x, 0.0) + np.log2(1.0 + np.exp2(-2.0 * np.abs(x))) / 2.0


def gated_residual(x: np.ndarray, y: np.ndarray) -> np.ndarray:
	"""new_block.py:110-116"""
	gate = y[..., 0::2]
	return sigmoid_base4(-gate) * x + softplus_base4(gate) * y[..., 1::2]


def ssmax_n(seq_len: int, window: int) -> np.ndarray:
	"""new_block.py:162-181"""
	i = np.arange(seq_len, dtype=np.float64)
	if window > 0:
		i = np.minimum(i, float(window))
	return (i + 4.0)[:, None]


def attn_one_head(q, k, v, sink_k, sink_v, temperature_scale: float, window: int,
                  prob_steps: float = 8.0, row_block: int = 2048):
	"""new_block.py:183-232.  q, k, v are real values on the FixedI8 grid, [T, hd].
	prob_steps = 8 reproduces the reference oracle (probabilities rounded to 1/8 steps,
	:225); prob_steps = 255 models the CUDA kernel's u8 probabilities instead.
	The dense [T, T+1] matrices are formed `row_block` query rows at a time (and only up to
	the last causally visible column), which changes nothing in the arithmetic of a row.
	Returns (o [T, hd], l [T]) with l in the kernel's convention log2(sum * 255) + max*log2e."""
	t, hd = q.shape
	k = np.concatenate((sink_k[None, :], k), axis=0)
	v = np.concatenate((sink_v[None, :], v), axis=0)
	temperature = math.sqrt(1.0 / hd) * np.log(ssmax_n(t, window)) * temperature_scale
	log2e = 1.0 / math.log(2.0)
	o = np.empty((t, hd), dtype=np.float64)
	l = np.empty((t,), dtype=np.float64)
	for r0 in range(0, t, row_block):
		r1 = min(t, r0 + row_block)
		ncol = r1 + 1                                   # sink + keys 0 .. r1-1
		s = q[r0:r1] @ k[:ncol].T
		rows = np.arange(r0, r1)[:, None]
		cols = np.arange(ncol - 1)[None, :]
		real_mask = cols >= rows
		if window > 0:
			real_mask |= cols < rows - window
		mask = np.zeros((r1 - r0, ncol), dtype=bool)
		mask[:, 1:] = real_mask
		s = np.where(mask, -np.inf, s)
		s = s * temperature[r0:r1]
		mx = s.max(axis=1, keepdims=True)
		p = np.exp(s - mx)
		total = p.sum(axis=1, keepdims=True)
		l[r0:r1] = (np.log(total) + mx)[:, 0] * log2e + math.log2(255.0)
		p[:, 1:] = np.rint(p[:, 1:] * prob_steps) / prob_steps   # p <= 1: quantize()'s clamp is idle
		o[r0:r1] = (p @ v[:ncol]) / total
	return o, l


def quantize_rows(a: np.ndarray):
	"""Symmetric int8 quantisation of the last axis: scale = absmax / 127 (1 for an all-zero row),
	codes = rint(a / scale).  Returns (codes int8, scale float32 without the last axis)."""
	absmax = np.abs(a).max(axis=-1)
	scale = np.where(absmax > 0, absmax / 127.0, 1.0).astype(np.float32)
	codes = np.clip(np.rint(a / scale[..., None].astype(np.float64)), -127, 127).astype(np.int8)
	return codes, scale


def attn_one_head_row_scaled(q_codes, k_codes, v_codes, q_scale, k_scale, v_scale, sink_k, sink_v,
                             temperature_scale: float, window: int, quantize_p: bool = True):
	"""The dense softmax of attn_one_head over operands given as int8 codes with one scale per row
	(real value = code * scale); sink_k, sink_v are real values.  With quantize_p the probability of
	key j enters the numerator as rint(255 p_j w_j) / (255 w_j), w_j = v_scale[j] / max(v_scale), which
	models u8 probabilities that carry the value row's relative scale; without it the softmax is exact.
	Returns o [T, hd] (real values)."""
	t, hd = q_codes.shape
	q = q_codes.astype(np.float64) * np.asarray(q_scale, dtype=np.float64)[:, None]
	k = k_codes.astype(np.float64) * np.asarray(k_scale, dtype=np.float64)[:, None]
	v_scale = np.asarray(v_scale, dtype=np.float32)
	v_ref = np.float32(v_scale.max())
	w = (v_scale / v_ref).astype(np.float64)                        # float32 quotient, as a caller would form it
	k = np.concatenate((sink_k[None, :], k), axis=0)
	temperature = math.sqrt(1.0 / hd) * np.log(ssmax_n(t, window)) * temperature_scale
	s = q @ k.T
	rows = np.arange(t)[:, None]
	cols = np.arange(t)[None, :]
	real_mask = cols >= rows
	if window > 0:
		real_mask |= cols < rows - window
	mask = np.zeros((t, t + 1), dtype=bool)
	mask[:, 1:] = real_mask
	s = np.where(mask, -np.inf, s) * temperature
	p = np.exp(s - s.max(axis=1, keepdims=True))
	total = p.sum(axis=1, keepdims=True)
	if quantize_p:
		pk = np.rint(p[:, 1:] * 255.0 * w[None, :]) * (float(v_ref) / 255.0)
		num = pk @ v_codes.astype(np.float64)
	else:
		num = p[:, 1:] @ (v_codes.astype(np.float64) * v_scale.astype(np.float64)[:, None])
	return (p[:, :1] * sink_v[None, :] + num) / total


def attn(q, k, v, sinks_k, sinks_v, attn_temperature, window: int, prob_steps: float = 8.0):
	"""new_block.py:234-258.  q, k, v: [T, H, hd]; sinks [H, hd]; attn_temperature [H]."""
	outs, ls = [], []
	for h in range(q.shape[1]):
		o, l = attn_one_head(q[:, h], k[:, h], v[:, h], sinks_k[h], sinks_v[h],
		                     float(attn_temperature[h]), window, prob_steps)
		outs.append(o)
		ls.append(l)
	return np.stack(outs, axis=1), np.stack(ls, axis=1)
