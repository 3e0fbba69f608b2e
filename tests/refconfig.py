"""Inputs of the reference's own golden run, regenerated bit-for-bit.

The reference checks in no tensor data; its golden report (expected.txt) was produced from
tensors drawn by new_block.py:27-52 with torch's CPU generator, seed 42, float64, in a fixed
order, at the configuration of block.config.json:2-9.  The same draws are repeated here with
the installed torch, so the statistics printed in expected.txt can be checked directly.
"""
from __future__ import annotations

import functools

import numpy as np
import torch

SEQ_LEN = 16384
MODEL_DIM = 2048
HEAD_DIM = 32
N_HEADS = 64
F_WIDTH = 2048
ATTN_WIDTH = N_HEADS * HEAD_DIM
L2_NORM_EPS = 2.0 ** -70
V_SCALE_FIX = 1.3


def _codes(t: torch.Tensor) -> np.ndarray:
	"""block_utils.py:163-166 -- int8 storage goes through float32 first."""
	w = t.to(torch.float32)
	return torch.clamp(torch.round(w * 8.0), -127.0, 127.0).to(torch.int8).numpy()


@functools.lru_cache(maxsize=1)
def inputs() -> dict:
	old = torch.get_default_dtype()
	torch.set_default_dtype(torch.float64)
	try:
		g = torch.Generator(device="cpu")
		g.manual_seed(42)
		x = torch.randn((SEQ_LEN, MODEL_DIM), generator=g)
		sk = torch.randn((N_HEADS, HEAD_DIM), generator=g)
		sk = sk * torch.rsqrt(torch.mean(sk * sk, dim=-1, keepdim=True) + L2_NORM_EPS)
		sv = torch.randn((N_HEADS, HEAD_DIM), generator=g)
		temp = 0.5 + torch.rand((N_HEADS, 1), generator=g)
		wq = torch.randn((N_HEADS * HEAD_DIM, MODEL_DIM), generator=g)
		wkv = torch.randn((N_HEADS, 2, HEAD_DIM, MODEL_DIM), generator=g)
		wy_attn = torch.randn((2 * MODEL_DIM, ATTN_WIDTH), generator=g)
		wkv[:, 1, :, :] *= V_SCALE_FIX
		sv *= V_SCALE_FIX
		wf = torch.randn((2 * F_WIDTH, MODEL_DIM), generator=g)
		wy_ffn = torch.randn((2 * MODEL_DIM, F_WIDTH), generator=g)
		return {
			"x": _codes(x),
			"sinks_k": _codes(sk),
			"sinks_v": _codes(sv),
			"attn_temperature": temp.to(torch.float32).numpy().reshape(-1),
			"attn_q_weights": _codes(wq),
			"attn_kv_weights": _codes(wkv).reshape(2 * ATTN_WIDTH, MODEL_DIM),
			"attn_y_weights": _codes(wy_attn),
			"ffn_f_weights": _codes(wf),
			"ffn_y_weights": _codes(wy_ffn),
		}
	finally:
		torch.set_default_dtype(old)


def acc_exact(a_codes: np.ndarray, b_codes: np.ndarray) -> np.ndarray:
	"""Exact int32 accumulators through float64 BLAS (every partial sum is < 2**53)."""
	acc = a_codes.astype(np.float64) @ b_codes.astype(np.float64).T
	return acc.astype(np.int32)


def i8_stats(codes: np.ndarray):
	c = codes.astype(np.float64)
	return int(codes.min()), int(codes.max()), float(c.mean()), float(c.var())
