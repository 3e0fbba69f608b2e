"""Dense float64 definition of the attention backward (dQ, dK, dV), for the int8 generation of the path.

TEST INFRASTRUCTURE ONLY (same rules as oracle/strict.py and oracle/dense.py).

The reference's backward kernels (attn_d_q.cuh:1-410, attn_d_kv.cuh, ffn_d_*.cu) belong to its bf16 generation:
bf16 Q / K / V / O / dO tiles, a score-only sink with an output gate, e-based scalable softmax.  The int8 / e4m3
generation this build covers has no backward in the reference yet, so what "dQ of attn_fwd_i8" means is fixed here,
following the structure of attn_d_q.cuh (flash-attention backward: P recomputed from the forward's log-sum-exp L,
D = rowsum(dO * O), dS = P * (dP - D), dQ = dS . K) on the forward semantics of new_block.py:183-232 /
cuda/attn_fwd_i8.cuh:368-619:

  real operands   q = q_code / 8, k = k_code / 8, v = v_code / 8 (FixedI8), sink key / value likewise
  scores          s_ij = t_i * (q_i . k_j),  t_i = hd^-1/2 * log2(min(W', i) + 4) * head_temp      (base 2)
                  keys j in [max(0, i - W'), i - 1] plus the sink (a real key AND value here, unlike the bf16 sink)
  probabilities   P_ij = 2^(s_ij - (L_i - log2 255)) -- the forward's L is log2(255 * sum_j 2^s_ij); the backward
                  takes the exact probabilities (the forward's 8-bit rounding of P is treated as the identity)
  D_i             = dO_i . o_i with o_i = out_code_i / 8: the forward output AS STORED (attn_d_q.cuh:236-262 does the
                  same with its stored bf16 O)
  dS_ij           = ln 2 * P_ij * (dO_i . v_j - D_i)
  dq_i            = t_i * sum_j dS_ij * k_j          (gradient with respect to the REAL q; the quantisation of q is
                  treated as the identity as well)

  dk_j            = sum_i t_i * dS_ij * q_i          (structure of attn_d_kv.cuh:200-400: one block of keys walks the
  dv_j            = sum_i P_ij * dO_i                 queries that see it; D comes from the dQ pass; gradients with
                                                      respect to the REAL k and v of the sequence's own keys -- like
                                                      attn_d_kv.cuh, no gradient is formed for the sink or the temperature)

With the exact o and L of the dense forward this is the derivative of sum(dO * o) with respect to q, k and v
(tests/test_oracle_backward.py holds it against torch autograd in float64).  With the stored int8 output in D the
rows of dS no longer sum to exactly zero; the deviation is bounded by |dO_i| * |o_i - o_hat_i| and is part of the
definition (the same happens with a bf16 O in the reference, at a smaller scale).
"""
from __future__ import annotations

import math

import numpy as np

from . import dense

LOG2_255 = math.log2(255.0)


def temperature(seq_len: int, head_dim: int, window: int, head_temp: float) -> np.ndarray:
	"""t_i of the scores in base 2, [T, 1] (window already rounded up to 16 by the caller if it wants the kernel's W')."""
	return math.sqrt(1.0 / head_dim) * np.log2(dense.ssmax_n(seq_len, window)) * head_temp


def visible(seq_len: int, window: int) -> np.ndarray:
	"""[T, T + 1] boolean: column 0 is the sink (always visible), column 1 + j is key j: visible iff j < i and i - j <= W."""
	rows = np.arange(seq_len)[:, None]
	cols = np.arange(seq_len)[None, :]
	vis = cols < rows
	if window > 0:
		vis &= cols >= rows - window
	return np.concatenate((np.ones((seq_len, 1), dtype=bool), vis), axis=1)


def attn_fwd_one_head(q, k, v, sink_k, sink_v, head_temp: float, window: int):
	"""Exact dense forward (no probability rounding): (o [T, hd], l [T]) with l = log2(255 * sum 2^s)."""
	t, hd = q.shape
	ka = np.concatenate((sink_k[None, :], k), axis=0)
	va = np.concatenate((sink_v[None, :], v), axis=0)
	s = (q @ ka.T) * temperature(t, hd, window, head_temp)
	s = np.where(visible(t, window), s, -np.inf)
	mx = s.max(axis=1, keepdims=True)
	p = np.exp2(s - mx)
	total = p.sum(axis=1, keepdims=True)
	return (p @ va) / total, (np.log2(total) + mx)[:, 0] + LOG2_255


def attn_d_q_one_head(q, k, v, sink_k, sink_v, head_temp: float, window: int, o_stored, d_o, l):
	"""dq [T, hd] and D [T] for one head.  q, k, v, sink_k, sink_v, o_stored, d_o: real values (float64), l: the
	forward's log-sum-exp in its own convention."""
	t, hd = q.shape
	ka = np.concatenate((sink_k[None, :], k), axis=0)
	va = np.concatenate((sink_v[None, :], v), axis=0)
	ti = temperature(t, hd, window, head_temp)
	s = (q @ ka.T) * ti
	prob = np.where(visible(t, window), np.exp2(s - (np.asarray(l, dtype=np.float64)[:, None] - LOG2_255)), 0.0)
	dp = d_o @ va.T
	d = np.sum(d_o * o_stored, axis=1)
	ds = math.log(2.0) * prob * (dp - d[:, None])
	return ti * (ds @ ka), d


def attn_d_q(q_codes, kv_codes, sink_k_codes, sink_v_codes, head_temp, n_heads: int, head_dim: int, window: int,
             out_codes, d_out, l):
	"""The kernel's interface in float64: q_codes int8 [T, H*hd], kv_codes int8 [T, H*2*hd] (per head K then V), sinks
	int8 [H, hd], head_temp [H], out_codes int8 [T, H*hd] (the forward's output), d_out real [T, H*hd], l [H, T].
	The window is rounded up to a multiple of 16 as the forward does (cuda/attn_fwd_i8.cuh:408-412).
	Returns (dq float64 [T, H*hd], d float64 [H, T])."""
	t = q_codes.shape[0]
	w = 0 if window == 0 else ((window - 1) // 16 + 1) * 16
	dq = np.empty((t, n_heads * head_dim), dtype=np.float64)
	d = np.empty((n_heads, t), dtype=np.float64)
	for h in range(n_heads):
		sl = slice(h * head_dim, (h + 1) * head_dim)
		kc = kv_codes[:, 2 * h * head_dim:(2 * h + 1) * head_dim].astype(np.float64) / 8.0
		vc = kv_codes[:, (2 * h + 1) * head_dim:(2 * h + 2) * head_dim].astype(np.float64) / 8.0
		dq[:, sl], d[h] = attn_d_q_one_head(
			q_codes[:, sl].astype(np.float64) / 8.0, kc, vc, sink_k_codes[h].astype(np.float64) / 8.0,
			sink_v_codes[h].astype(np.float64) / 8.0, float(head_temp[h]), w,
			out_codes[:, sl].astype(np.float64) / 8.0, np.asarray(d_out, dtype=np.float64)[:, sl], l[h])
	return dq, d


def attn_d_kv_one_head(q, k, v, sink_k, sink_v, head_temp: float, window: int, d_o, l, d):
	"""(dk [T, hd], dv [T, hd], d_sink_k [hd], d_sink_v [hd]) for one head.  `d` is the D of the dQ pass (whatever
	output it was formed with); the sink's two gradients are returned for the tests' invariants only."""
	t, hd = q.shape
	ka = np.concatenate((sink_k[None, :], k), axis=0)
	va = np.concatenate((sink_v[None, :], v), axis=0)
	ti = temperature(t, hd, window, head_temp)
	s = (q @ ka.T) * ti
	prob = np.where(visible(t, window), np.exp2(s - (np.asarray(l, dtype=np.float64)[:, None] - LOG2_255)), 0.0)
	ds = math.log(2.0) * prob * (d_o @ va.T - np.asarray(d, dtype=np.float64)[:, None])
	dka = (ds * ti).T @ q
	dva = prob.T @ d_o
	return dka[1:], dva[1:], dka[0], dva[0]


def attn_d_kv(q_codes, kv_codes, sink_k_codes, sink_v_codes, head_temp, n_heads: int, head_dim: int, window: int,
              d_out, l, d):
	"""The kernel's interface in float64: operands as in attn_d_q, d [H, T] from the dQ pass.  Returns d_kv float64
	[T, H*2*hd] in the layout of kv (per head dK then dV)."""
	t = q_codes.shape[0]
	w = 0 if window == 0 else ((window - 1) // 16 + 1) * 16
	d_kv = np.empty((t, 2 * n_heads * head_dim), dtype=np.float64)
	for h in range(n_heads):
		sl = slice(h * head_dim, (h + 1) * head_dim)
		ks, vs = slice(2 * h * head_dim, (2 * h + 1) * head_dim), slice((2 * h + 1) * head_dim, (2 * h + 2) * head_dim)
		d_kv[:, ks], d_kv[:, vs], _, _ = attn_d_kv_one_head(
			q_codes[:, sl].astype(np.float64) / 8.0, kv_codes[:, ks].astype(np.float64) / 8.0,
			kv_codes[:, vs].astype(np.float64) / 8.0, sink_k_codes[h].astype(np.float64) / 8.0,
			sink_v_codes[h].astype(np.float64) / 8.0, float(head_temp[h]), w,
			np.asarray(d_out, dtype=np.float64)[:, sl], l[h], d[h])
	return d_kv
