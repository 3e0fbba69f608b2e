"""ctypes front-end of the C oracle (oracle/x17_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  The shipped HIP path never imports this module.

All functions take and return numpy arrays; shapes follow the reference's layouts
(weights are [N_raw, K] row-major, "trans" in src/device/cuda/gemm.rs:463-468).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libx17_oracle.so")

STORE_I8 = 0
STORE_E4M3 = 1


def build(force: bool = False) -> str:
	"""Compile the oracle with the Makefile next to this file."""
	if force or not os.path.exists(_LIB_PATH):
		subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
		               stdout=subprocess.DEVNULL)
	return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
	global _lib
	if _lib is None:
		build()
		_lib = ctypes.CDLL(_LIB_PATH)
		_lib.x17o_constexpr_sqrt.restype = ctypes.c_double
		_lib.x17o_constexpr_sqrt.argtypes = [ctypes.c_double]
		_lib.x17o_constexpr_inv_sqrt.restype = ctypes.c_double
		_lib.x17o_constexpr_inv_sqrt.argtypes = [ctypes.c_double]
		_lib.x17o_num_threads.restype = ctypes.c_int
	return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
	assert a.flags["C_CONTIGUOUS"]
	return ctypes.c_void_p(a.ctypes.data)


def _sz(v: int) -> ctypes.c_size_t:
	return ctypes.c_size_t(int(v))


def num_threads() -> int:
	return int(lib().x17o_num_threads())


# ---------------------------------------------------------------- conversions / SFU

def f32_to_fixedi8(x: np.ndarray) -> np.ndarray:
	x = np.ascontiguousarray(x, dtype=np.float32)
	out = np.empty(x.shape, dtype=np.int8)
	lib().x17o_f32_to_fixedi8(_p(x), _p(out), _sz(x.size))
	return out


def f32_to_e4m3(x: np.ndarray) -> np.ndarray:
	x = np.ascontiguousarray(x, dtype=np.float32)
	out = np.empty(x.shape, dtype=np.uint8)
	lib().x17o_f32_to_e4m3(_p(x), _p(out), _sz(x.size))
	return out


def e4m3_to_f32(c: np.ndarray) -> np.ndarray:
	c = np.ascontiguousarray(c, dtype=np.uint8)
	out = np.empty(c.shape, dtype=np.float32)
	lib().x17o_e4m3_to_f32(_p(c), _p(out), _sz(c.size))
	return out


_SFU = {"ex2": 0, "lg2": 1, "rcp": 2, "rsq": 3, "tanh": 4}


def sfu(name: str, x: np.ndarray) -> np.ndarray:
	x = np.ascontiguousarray(x, dtype=np.float32)
	out = np.empty(x.shape, dtype=np.float32)
	lib().x17o_sfu(ctypes.c_int(_SFU[name]), _p(x), _p(out), _sz(x.size))
	return out


def constexpr_sqrt(x: float) -> float:
	return float(lib().x17o_constexpr_sqrt(ctypes.c_double(x)))


def constexpr_inv_sqrt(x: float) -> float:
	return float(lib().x17o_constexpr_inv_sqrt(ctypes.c_double(x)))


# ---------------------------------------------------------------- GEMM cores

def gemm_i32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
	"""acc[m, n] = sum_k a[m, k] * b[n, k] in int32 (a, b int8)."""
	a = np.ascontiguousarray(a, dtype=np.int8)
	b = np.ascontiguousarray(b, dtype=np.int8)
	m, k = a.shape
	n, k2 = b.shape
	assert k == k2
	acc = np.empty((m, n), dtype=np.int32)
	lib().x17o_gemm_i32(_p(a), _p(b), _p(acc), _sz(m), _sz(n), _sz(k))
	return acc


def gemm_f32_seq(a: np.ndarray, a_is_e4m3: bool, b: np.ndarray, b_is_e4m3: bool) -> np.ndarray:
	"""f32-accumulated GEMM over 8-bit operands (i8 codes or e4m3 bytes), k ascending."""
	a = np.ascontiguousarray(a).view(np.uint8)
	b = np.ascontiguousarray(b).view(np.uint8)
	m, k = a.shape
	n, k2 = b.shape
	assert k == k2
	acc = np.empty((m, n), dtype=np.float32)
	lib().x17o_gemm_f32_seq(_p(a), ctypes.c_int(int(a_is_e4m3)), _p(b), ctypes.c_int(int(b_is_e4m3)),
	                        _p(acc), _sz(m), _sz(n), _sz(k))
	return acc


# ---------------------------------------------------------------- epilogues

def _acc_args(acc: np.ndarray):
	if acc.dtype == np.int32:
		return np.ascontiguousarray(acc), 0
	if acc.dtype == np.float32:
		return np.ascontiguousarray(acc), 1
	raise TypeError(f"accumulators must be int32 or float32, got {acc.dtype}")


def _out(shape, store):
	return np.empty(shape, dtype=np.uint8 if store == STORE_E4M3 else np.int8)


def epilogue_scale(acc, inp_scale: float, out_scale: float, store: int = STORE_I8):
	acc, is_f32 = _acc_args(acc)
	m, n = acc.shape
	c = _out((m, n), store)
	lib().x17o_epilogue_scale(_p(acc), ctypes.c_int(is_f32), _p(c), _sz(m), _sz(n),
	                          ctypes.c_double(inp_scale), ctypes.c_double(out_scale), ctypes.c_int(store))
	return c


def epilogue_geglu(acc, inp_scale: float, out_scale: float, store: int = STORE_E4M3):
	acc, is_f32 = _acc_args(acc)
	m, n_raw = acc.shape
	assert n_raw % 2 == 0
	c = _out((m, n_raw // 2), store)
	lib().x17o_epilogue_geglu(_p(acc), ctypes.c_int(is_f32), _p(c), _sz(m), _sz(n_raw),
	                          ctypes.c_double(inp_scale), ctypes.c_double(out_scale), ctypes.c_int(store))
	return c


def epilogue_residual(acc, residual, inp_scale: float, out_scale: float, store: int = STORE_E4M3):
	acc, is_f32 = _acc_args(acc)
	m, n_raw = acc.shape
	assert n_raw % 2 == 0
	residual = np.ascontiguousarray(residual, dtype=np.int8)
	assert residual.shape == (m, n_raw // 2)
	c = _out((m, n_raw // 2), store)
	lib().x17o_epilogue_residual(_p(acc), ctypes.c_int(is_f32), _p(residual), _p(c), _sz(m), _sz(n_raw),
	                             ctypes.c_double(inp_scale), ctypes.c_double(out_scale), ctypes.c_int(store))
	return c


def epilogue_dequant(acc, row_scale, col_scale, geglu: bool = False) -> np.ndarray:
	"""bf16 bits (uint16) of (f32(acc) * row_scale[m]) * col_scale[n], optionally through GeGLU over column pairs."""
	acc, is_f32 = _acc_args(acc)
	m, n = acc.shape
	row_scale = np.ascontiguousarray(row_scale, dtype=np.float32).reshape(-1)
	col_scale = np.ascontiguousarray(col_scale, dtype=np.float32).reshape(-1)
	assert row_scale.shape == (m,) and col_scale.shape == (n,)
	out = np.empty((m, n // 2 if geglu else n), dtype=np.uint16)
	lib().x17o_epilogue_dequant(_p(acc), ctypes.c_int(is_f32), _p(row_scale), _p(col_scale), _p(out), _sz(m), _sz(n),
	                            ctypes.c_int(int(geglu)))
	return out


def epilogue_l2norm(acc, head_dim: int, eps: float, inp_scale: float, out_scale: float):
	"""Returns (kv codes int8 [M, N_raw], rrms float32 [M, N_raw / (2*head_dim)]).

	head_scale = out * sqrt(head_dim) and sep_scale = inp * out are formed in double exactly
	as src/device/cuda/gemm.rs:146,152 does before they are pasted into the kernel source."""
	acc = np.ascontiguousarray(acc, dtype=np.int32)
	m, n_raw = acc.shape
	assert n_raw % (2 * head_dim) == 0
	c = np.empty((m, n_raw), dtype=np.int8)
	rrms = np.empty((m, n_raw // (2 * head_dim)), dtype=np.float32)
	head_scale = out_scale * float(np.sqrt(np.float64(head_dim)))
	sep_scale = inp_scale * out_scale
	lib().x17o_epilogue_l2norm(_p(acc), _p(c), _p(rrms), _sz(m), _sz(n_raw), _sz(head_dim),
	                           ctypes.c_double(eps), ctypes.c_double(head_scale), ctypes.c_double(sep_scale))
	return c, rrms


def epilogue_qnorm(acc, head_dim: int, eps: float, out_scale: float, dyn_bf16, want_rrms: bool = False,
                   post_scale: float = 1.0):
	"""The learned-scale Q writer (cuda/qkvg_fwd_i8.cuh:145-219; hook cuda/gemm_b8.cuh:761-824): every head_dim raw
	columns are one head, L2-normalised like the K halves of epilogue_l2norm, then multiplied by a bf16 scale per
	column (dyn_bf16: uint16 bit patterns, [N_raw]) and, when post_scale != 1, by f32(post_scale) (the factor of the
	old writer's vanished base class, cuda/qkvg_fwd_i8.cuh:151-159).  Returns q codes int8 [M, N_raw] (and rrms
	[M, N_raw / head_dim])."""
	acc = np.ascontiguousarray(acc, dtype=np.int32)
	dyn = np.ascontiguousarray(dyn_bf16, dtype=np.uint16)
	m, n_raw = acc.shape
	assert n_raw % head_dim == 0 and dyn.shape == (n_raw,)
	c = np.empty((m, n_raw), dtype=np.int8)
	rrms = np.empty((m, n_raw // head_dim), dtype=np.float32) if want_rrms else None
	head_scale = out_scale * float(np.sqrt(np.float64(head_dim)))
	lib().x17o_epilogue_qnorm(_p(acc), _p(c), _p(rrms) if want_rrms else None, _p(dyn), _sz(m), _sz(n_raw), _sz(head_dim),
	                          ctypes.c_double(eps), ctypes.c_double(head_scale), ctypes.c_double(post_scale))
	return (c, rrms) if want_rrms else c


# ---------------------------------------------------------------- attention / decode / rms_norm

def attn_fwd_i8(q, kv, sink_k, sink_v, head_temp, n_heads: int, head_dim: int, window: int,
                want_l: bool = True, fast_exp: bool = False):
	"""q [T, H*hd] int8, kv [T, H*2*hd] int8 -> (out int8 [T, H*hd], L float32 [H, T] or None)."""
	q = np.ascontiguousarray(q, dtype=np.int8)
	kv = np.ascontiguousarray(kv, dtype=np.int8)
	sink_k = np.ascontiguousarray(sink_k, dtype=np.int8)
	sink_v = np.ascontiguousarray(sink_v, dtype=np.int8)
	head_temp = np.ascontiguousarray(head_temp, dtype=np.float32).reshape(-1)
	t = q.shape[0]
	assert q.shape == (t, n_heads * head_dim) and kv.shape == (t, 2 * n_heads * head_dim)
	assert sink_k.shape == (n_heads, head_dim) and sink_v.shape == (n_heads, head_dim)
	assert head_temp.shape == (n_heads,)
	out = np.empty_like(q)
	l = np.empty((n_heads, t), dtype=np.float32) if want_l else None
	rc = lib().x17o_attn_fwd_i8(_sz(t), _sz(n_heads), _sz(head_dim), _p(q), _p(kv), _p(sink_k), _p(sink_v),
	                            _p(head_temp), _p(out), _p(l) if want_l else None, _sz(window),
	                            ctypes.c_int(int(fast_exp)))
	assert rc == 0
	return out, l


def attn_fwd_i8_row_scaled(q, kv, sink_k, sink_v, head_temp, n_heads: int, head_dim: int, window: int,
                           q_scale, k_scale, v_weight, sink_v_weight, out_scale, out_bf16: bool = False,
                           want_l: bool = True, fast_exp: bool = False):
	"""attn_fwd_i8 over row-scaled operands: q_scale, k_scale, v_weight float32 [H, T]; sink_v_weight,
	out_scale float32 [H].  Returns (out, L): out int8 codes, or bf16 bit patterns (uint16) with out_bf16."""
	q = np.ascontiguousarray(q, dtype=np.int8)
	kv = np.ascontiguousarray(kv, dtype=np.int8)
	sink_k = np.ascontiguousarray(sink_k, dtype=np.int8)
	sink_v = np.ascontiguousarray(sink_v, dtype=np.int8)
	head_temp = np.ascontiguousarray(head_temp, dtype=np.float32).reshape(-1)
	t = q.shape[0]
	assert q.shape == (t, n_heads * head_dim) and kv.shape == (t, 2 * n_heads * head_dim)
	assert sink_k.shape == (n_heads, head_dim) and sink_v.shape == (n_heads, head_dim)
	rows = [np.ascontiguousarray(a, dtype=np.float32) for a in (q_scale, k_scale, v_weight)]
	heads = [np.ascontiguousarray(a, dtype=np.float32).reshape(-1) for a in (sink_v_weight, out_scale)]
	assert all(a.shape == (n_heads, t) for a in rows) and all(a.shape == (n_heads,) for a in heads)
	out = np.empty(q.shape, dtype=np.uint16 if out_bf16 else np.int8)
	l = np.empty((n_heads, t), dtype=np.float32) if want_l else None
	rc = lib().x17o_attn_fwd_i8_row_scaled(_sz(t), _sz(n_heads), _sz(head_dim), _p(q), _p(kv), _p(sink_k), _p(sink_v),
	                                       _p(head_temp), _p(out), _p(l) if want_l else None, _sz(window),
	                                       ctypes.c_int(int(fast_exp)), _p(rows[0]), _p(rows[1]), _p(rows[2]),
	                                       _p(heads[0]), _p(heads[1]), ctypes.c_int(int(out_bf16)))
	assert rc == 0
	return out, l


def attn_decode_i8(q, cache, cache_len, sink_k, sink_v, head_temp, n_heads: int, head_dim: int,
                   window: int, want_l: bool = True, fast_exp: bool = False):
	"""q [S, H*hd], cache [S, cap, H*2*hd], cache_len uint32 [S] -> (out [S, H*hd], L [S, H])."""
	q = np.ascontiguousarray(q, dtype=np.int8)
	cache = np.ascontiguousarray(cache, dtype=np.int8)
	cache_len = np.ascontiguousarray(cache_len, dtype=np.uint32)
	sink_k = np.ascontiguousarray(sink_k, dtype=np.int8)
	sink_v = np.ascontiguousarray(sink_v, dtype=np.int8)
	head_temp = np.ascontiguousarray(head_temp, dtype=np.float32).reshape(-1)
	s, cap, w = cache.shape
	assert w == 2 * n_heads * head_dim and q.shape == (s, n_heads * head_dim)
	out = np.empty_like(q)
	l = np.empty((s, n_heads), dtype=np.float32) if want_l else None
	rc = lib().x17o_attn_decode_i8(_sz(s), _sz(cap), _p(cache_len), _sz(n_heads), _sz(head_dim),
	                               _p(q), _p(cache), _p(sink_k), _p(sink_v), _p(head_temp),
	                               _p(out), _p(l) if want_l else None, _sz(window),
	                               ctypes.c_int(int(fast_exp)))
	assert rc == 0
	return out, l


def attn_decode_i8_row_scaled(q, cache, cache_len, sink_k, sink_v, head_temp, n_heads: int, head_dim: int, window: int,
                              q_scale, k_scale, v_weight, sink_v_weight, out_scale, out_bf16: bool = False,
                              want_l: bool = True, fast_exp: bool = False):
	"""attn_decode_i8 over row-scaled operands: q_scale float32 [S, H]; k_scale, v_weight [S, H, cap];
	sink_v_weight, out_scale [H].  out: int8 codes or (out_bf16) bf16 bit patterns."""
	q = np.ascontiguousarray(q, dtype=np.int8)
	cache = np.ascontiguousarray(cache, dtype=np.int8)
	cache_len = np.ascontiguousarray(cache_len, dtype=np.uint32)
	sink_k = np.ascontiguousarray(sink_k, dtype=np.int8)
	sink_v = np.ascontiguousarray(sink_v, dtype=np.int8)
	head_temp = np.ascontiguousarray(head_temp, dtype=np.float32).reshape(-1)
	s, cap, w = cache.shape
	assert w == 2 * n_heads * head_dim and q.shape == (s, n_heads * head_dim)
	q_scale = np.ascontiguousarray(q_scale, dtype=np.float32)
	k_scale = np.ascontiguousarray(k_scale, dtype=np.float32)
	v_weight = np.ascontiguousarray(v_weight, dtype=np.float32)
	heads = [np.ascontiguousarray(a, dtype=np.float32).reshape(-1) for a in (sink_v_weight, out_scale)]
	assert q_scale.shape == (s, n_heads) and k_scale.shape == (s, n_heads, cap) and v_weight.shape == (s, n_heads, cap)
	assert all(a.shape == (n_heads,) for a in heads)
	out = np.empty(q.shape, dtype=np.uint16 if out_bf16 else np.int8)
	l = np.empty((s, n_heads), dtype=np.float32) if want_l else None
	rc = lib().x17o_attn_decode_i8_row_scaled(_sz(s), _sz(cap), _p(cache_len), _sz(n_heads), _sz(head_dim),
	                                          _p(q), _p(cache), _p(sink_k), _p(sink_v), _p(head_temp),
	                                          _p(out), _p(l) if want_l else None, _sz(window), ctypes.c_int(int(fast_exp)),
	                                          _p(q_scale), _p(k_scale), _p(v_weight), _p(heads[0]), _p(heads[1]),
	                                          ctypes.c_int(int(out_bf16)))
	assert rc == 0
	return out, l


def rms_norm(inp: np.ndarray, eps: float, in_kind: str = "e4m3") -> np.ndarray:
	"""inp [T, D]: uint8 e4m3 bytes (in_kind 'e4m3') or uint16 bf16 bits (in_kind 'bf16')."""
	kind = {"e4m3": 1, "bf16": 2}[in_kind]
	inp = np.ascontiguousarray(inp, dtype=np.uint8 if kind == 1 else np.uint16)
	t, d = inp.shape
	out = np.empty((t, d), dtype=np.int8)
	rc = lib().x17o_rms_norm(_p(inp), ctypes.c_int(kind), _p(out), _sz(t), _sz(d), ctypes.c_double(eps))
	assert rc == 0, "rms_norm requires D % 512 == 0"
	return out
