"""Pins of the backward definition (oracle/backward.py): the int8 generation has no backward in the reference, so the
dense float64 formulas are held against what the mathematics fixes -- torch autograd over the same dense forward,
finite differences, and the invariants of a softmax gradient -- chosen so that a dropped term, a wrong sign, a missing
ln 2 or a mis-placed temperature fails one of them."""
import math

import numpy as np
import pytest
import torch

from oracle import backward as B
from oracle import dense


def _case(seed, t=96, hd=32, sigma=1.0):
	rng = np.random.default_rng(seed)
	q = dense.quantize(rng.standard_normal((t, hd)) * sigma)
	k = rng.standard_normal((t, hd))
	k = dense.quantize(k / np.sqrt((k * k).mean(-1, keepdims=True)))
	v = dense.quantize(rng.standard_normal((t, hd)) * 1.3)
	sk = rng.standard_normal(hd)
	sk = dense.quantize(sk / np.sqrt((sk * sk).mean()))
	sv = dense.quantize(rng.standard_normal(hd) * 1.3)
	d_o = rng.standard_normal((t, hd)) * 0.1
	return q, k, v, sk, sv, d_o


def _torch_forward(q, k, v, sk, sv, temp, window):
	"""The dense forward in torch float64, written independently of oracle/backward.py: natural-base softmax with
	ln(n) temperature (new_block.py:183-232), which is the same function as the base-2 form."""
	t, hd = q.shape
	ka = torch.cat((sk[None, :], k), 0)
	va = torch.cat((sv[None, :], v), 0)
	i = torch.arange(t, dtype=torch.float64)
	n = (torch.minimum(i, torch.tensor(float(window))) if window > 0 else i) + 4.0
	s = (q @ ka.T) * (math.sqrt(1.0 / hd) * torch.log(n)[:, None] * temp)
	rows, cols = torch.arange(t)[:, None], torch.arange(t)[None, :]
	vis = cols < rows
	if window > 0:
		vis = vis & (cols >= rows - window)
	vis = torch.cat((torch.ones(t, 1, dtype=torch.bool), vis), 1)
	s = torch.where(vis, s, torch.tensor(-float("inf"), dtype=torch.float64))
	return torch.softmax(s, dim=1) @ va


@pytest.mark.parametrize("window,temp", [(0, 1.0), (32, 0.7), (16, 1.4), (48, -0.8)])
def test_d_q_equals_torch_autograd(window, temp):
	q, k, v, sk, sv, d_o = _case(3 + window)
	o, l = B.attn_fwd_one_head(q, k, v, sk, sv, temp, window)
	dq, d = B.attn_d_q_one_head(q, k, v, sk, sv, temp, window, o, d_o, l)
	tq = torch.tensor(q, requires_grad=True)
	to = _torch_forward(tq, *(torch.tensor(a) for a in (k, v, sk, sv)), temp, window)
	assert np.abs(to.detach().numpy() - o).max() < 1e-12                        # the two forwards are one function
	(to * torch.tensor(d_o)).sum().backward()
	want = tq.grad.numpy()
	assert np.abs(dq - want).max() < 1e-12 * max(1.0, np.abs(want).max())
	assert np.abs(want).max() > 1e-3                                            # (not a comparison of zeros)
	assert np.abs(d - (d_o * o).sum(1)).max() < 1e-14
	# the forward's own log-sum-exp convention: the dense oracle of the forward path reports the same L
	# (that restatement masks before it scales, as new_block.py does, which only works for positive temperatures)
	if temp > 0:
		o2, l2 = dense.attn_one_head(q, k, v, sk, sv, temp, window, prob_steps=1e12)
		assert np.abs(l2 - l).max() < 1e-9 and np.abs(o2 - o).max() < 1e-9


def test_d_q_against_finite_differences_and_its_invariants():
	q, k, v, sk, sv, d_o = _case(11, t=48, hd=32)
	temp, window = 0.9, 16
	o, l = B.attn_fwd_one_head(q, k, v, sk, sv, temp, window)
	dq, _ = B.attn_d_q_one_head(q, k, v, sk, sv, temp, window, o, d_o, l)
	loss = lambda qq: float((B.attn_fwd_one_head(qq, k, v, sk, sv, temp, window)[0] * d_o).sum())
	rng = np.random.default_rng(5)
	for _ in range(6):
		i, c = int(rng.integers(0, 48)), int(rng.integers(0, 32))
		e = np.zeros_like(q)
		e[i, c] = 1e-5
		fd = (loss(q + e) - loss(q - e)) / 2e-5
		assert abs(fd - dq[i, c]) < 1e-7 * max(1.0, abs(fd)), (i, c, fd, dq[i, c])
	# query 0 sees only the sink: its output does not depend on q
	assert np.abs(dq[0]).max() < 1e-15
	# constant V (and sink value): the output is that constant whatever the scores
	vc = np.full_like(v, 0.625)
	oc, lc = B.attn_fwd_one_head(q, k, vc, sk, np.full_like(sv, 0.625), temp, window)
	dqc, _ = B.attn_d_q_one_head(q, k, vc, sk, np.full_like(sv, 0.625), temp, window, oc, d_o, lc)
	assert np.abs(dqc).max() < 1e-12
	# linear in dO; zero temperature: uniform weights, no dependence on q
	dq2, _ = B.attn_d_q_one_head(q, k, v, sk, sv, temp, window, o, 3.0 * d_o, l)
	assert np.abs(dq2 - 3.0 * dq).max() < 1e-12
	o0, l0 = B.attn_fwd_one_head(q, k, v, sk, sv, 0.0, window)
	assert np.abs(B.attn_d_q_one_head(q, k, v, sk, sv, 0.0, window, o0, d_o, l0)[0]).max() == 0.0


def test_stored_int8_output_in_d_is_a_bounded_deviation():
	"""D uses the forward output as stored (FixedI8 codes): the deviation from the exact gradient is the term
	ln 2 * t_i * (D_exact - D_stored) * sum_j P_ij k_j and nothing else."""
	q, k, v, sk, sv, d_o = _case(21, t=64, hd=32)
	temp, window = 1.0, 0
	o, l = B.attn_fwd_one_head(q, k, v, sk, sv, temp, window)
	o_hat = dense.quantize(o)
	exact, d_exact = B.attn_d_q_one_head(q, k, v, sk, sv, temp, window, o, d_o, l)
	stored, d_stored = B.attn_d_q_one_head(q, k, v, sk, sv, temp, window, o_hat, d_o, l)
	ka = np.concatenate((sk[None, :], k), 0)
	ti = B.temperature(64, 32, window, temp)
	prob = np.where(B.visible(64, window), np.exp2((q @ ka.T) * ti - (l[:, None] - B.LOG2_255)), 0.0)
	want = math.log(2.0) * ti * (d_exact - d_stored)[:, None] * (prob @ ka)
	assert np.abs((stored - exact) - want).max() < 1e-13
	assert np.abs(d_exact - d_stored).max() <= np.abs(d_o).sum(1).max() / 16.0 + 1e-12      # |o - o_hat| <= 1/16 per element


def test_multi_head_wrapper_slices_heads_and_rounds_the_window():
	rng = np.random.default_rng(2)
	t, h, hd = 64, 3, 32
	qc = np.clip(np.rint(rng.standard_normal((t, h * hd)) * 8), -127, 127).astype(np.int8)
	kvc = np.clip(np.rint(rng.standard_normal((t, 2 * h * hd)) * 8), -127, 127).astype(np.int8)
	skc = np.clip(np.rint(rng.standard_normal((h, hd)) * 8), -127, 127).astype(np.int8)
	svc = np.clip(np.rint(rng.standard_normal((h, hd)) * 8), -127, 127).astype(np.int8)
	temp = np.array([0.6, 1.0, 1.3])
	d_o = rng.standard_normal((t, h * hd)) * 0.1
	out = np.empty((t, h * hd), np.int8)
	l = np.empty((h, t))
	for hh in range(h):
		sl = slice(hh * hd, (hh + 1) * hd)
		o, l[hh] = B.attn_fwd_one_head(qc[:, sl] / 8.0, kvc[:, 2 * hh * hd:(2 * hh + 1) * hd] / 8.0, kvc[:, (2 * hh + 1) * hd:(2 * hh + 2) * hd] / 8.0,
		                               skc[hh] / 8.0, svc[hh] / 8.0, temp[hh], 32)
		out[:, sl] = np.clip(np.rint(o * 8), -127, 127)
	dq, d = B.attn_d_q(qc, kvc, skc, svc, temp, h, hd, 24, out, d_o, l)        # window 24 rounds up to 32
	hh = 1
	sl = slice(hh * hd, (hh + 1) * hd)
	want, want_d = B.attn_d_q_one_head(qc[:, sl] / 8.0, kvc[:, 2 * hd:3 * hd] / 8.0, kvc[:, 3 * hd:4 * hd] / 8.0, skc[1] / 8.0, svc[1] / 8.0,
	                                   1.0, 32, out[:, sl] / 8.0, d_o[:, sl], l[1])
	assert np.array_equal(dq[:, sl], want) and np.array_equal(d[1], want_d)



@pytest.mark.parametrize("window,temp", [(0, 1.0), (32, 0.7), (16, 1.4), (48, -0.8)])
def test_d_kv_equals_torch_autograd(window, temp):
	q, k, v, sk, sv, d_o = _case(103 + window)
	o, l = B.attn_fwd_one_head(q, k, v, sk, sv, temp, window)
	d = (d_o * o).sum(1)
	dk, dv, dsk, dsv = B.attn_d_kv_one_head(q, k, v, sk, sv, temp, window, d_o, l, d)
	tk, tv, tsk, tsv = (torch.tensor(a, requires_grad=True) for a in (k, v, sk, sv))
	(_torch_forward(torch.tensor(q), tk, tv, tsk, tsv, temp, window) * torch.tensor(d_o)).sum().backward()
	for got, want in ((dk, tk.grad), (dv, tv.grad), (dsk, tsk.grad), (dsv, tsv.grad)):
		want = want.numpy()
		assert np.abs(want).max() > 1e-3
		assert np.abs(got - want).max() < 1e-12 * max(1.0, np.abs(want).max())


def test_d_kv_against_finite_differences_and_its_invariants():
	q, k, v, sk, sv, d_o = _case(111, t=48, hd=32)
	temp, window = 0.9, 16
	o, l = B.attn_fwd_one_head(q, k, v, sk, sv, temp, window)
	d = (d_o * o).sum(1)
	dk, dv, dsk, dsv = B.attn_d_kv_one_head(q, k, v, sk, sv, temp, window, d_o, l, d)
	loss_k = lambda kk: float((B.attn_fwd_one_head(q, kk, v, sk, sv, temp, window)[0] * d_o).sum())
	loss_v = lambda vv: float((B.attn_fwd_one_head(q, k, vv, sk, sv, temp, window)[0] * d_o).sum())
	rng = np.random.default_rng(6)
	for _ in range(6):
		j, c = int(rng.integers(0, 47)), int(rng.integers(0, 32))
		e = np.zeros_like(k)
		e[j, c] = 1e-5
		for loss, grad in ((loss_k, dk), (loss_v, dv)):
			fd = (loss(k + e if grad is dk else v + e) - loss(k - e if grad is dk else v - e)) / 2e-5
			assert abs(fd - grad[j, c]) < 1e-7 * max(1.0, abs(fd)), (j, c, fd, grad[j, c])
	# the last key is seen by no query; key j is seen by at most `window` queries
	assert np.abs(dk[-1]).max() == 0.0 and np.abs(dv[-1]).max() == 0.0
	# probabilities of a row sum to one over the sink and the keys: the dv rows and the sink's sum to the dO rows' sum
	assert np.abs(dv.sum(0) + dsv - d_o.sum(0)).max() < 1e-12
	# rows of dS sum to zero with the exact D, so a shift of every key (sink included) by one vector changes nothing:
	# sum_j dk_j + d_sink_k = sum_i t_i (sum_j dS_ij) q_i = 0
	assert np.abs(dk.sum(0) + dsk).max() < 1e-12
	# linear in (dO, D) together; zero temperature: scores do not depend on k
	dk2, dv2, _, _ = B.attn_d_kv_one_head(q, k, v, sk, sv, temp, window, 3.0 * d_o, l, 3.0 * d)
	assert np.abs(dk2 - 3.0 * dk).max() < 1e-12 and np.abs(dv2 - 3.0 * dv).max() < 1e-12
	o0, l0 = B.attn_fwd_one_head(q, k, v, sk, sv, 0.0, window)
	assert np.abs(B.attn_d_kv_one_head(q, k, v, sk, sv, 0.0, window, d_o, l0, (d_o * o0).sum(1))[0]).max() == 0.0


def test_d_kv_multi_head_wrapper_uses_the_layout_of_kv():
	rng = np.random.default_rng(4)
	t, h, hd = 64, 2, 32
	qc = np.clip(np.rint(rng.standard_normal((t, h * hd)) * 8), -127, 127).astype(np.int8)
	kvc = np.clip(np.rint(rng.standard_normal((t, 2 * h * hd)) * 8), -127, 127).astype(np.int8)
	skc = np.clip(np.rint(rng.standard_normal((h, hd)) * 8), -127, 127).astype(np.int8)
	svc = np.clip(np.rint(rng.standard_normal((h, hd)) * 8), -127, 127).astype(np.int8)
	temp = np.array([0.6, 1.2])
	d_o = rng.standard_normal((t, h * hd)) * 0.1
	l, d = np.empty((h, t)), rng.standard_normal((h, t)) * 0.05
	for hh in range(h):
		_, l[hh] = B.attn_fwd_one_head(qc[:, hh * hd:(hh + 1) * hd] / 8.0, kvc[:, 2 * hh * hd:(2 * hh + 1) * hd] / 8.0,
		                               kvc[:, (2 * hh + 1) * hd:(2 * hh + 2) * hd] / 8.0, skc[hh] / 8.0, svc[hh] / 8.0, temp[hh], 32)
	got = B.attn_d_kv(qc, kvc, skc, svc, temp, h, hd, 24, d_o, l, d)            # window 24 rounds up to 32
	dk, dv, _, _ = B.attn_d_kv_one_head(qc[:, hd:] / 8.0, kvc[:, 2 * hd:3 * hd] / 8.0, kvc[:, 3 * hd:] / 8.0, skc[1] / 8.0, svc[1] / 8.0,
	                                    1.2, 32, d_o[:, hd:], l[1], d[1])
	assert np.array_equal(got[:, 2 * hd:3 * hd], dk) and np.array_equal(got[:, 3 * hd:], dv)
