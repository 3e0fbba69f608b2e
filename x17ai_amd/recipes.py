"""The block's kernels with the reference's scale recipes (src/main.rs:387-675).

Each function mirrors one create_*_kernel of the reference's block driver: same operand
dtypes, same epilogue, same scale expressions.  Kernel names carry the shape so that
several configurations can live side by side in the kernel cache.
"""
from __future__ import annotations

import math
from typing import Optional

from .api import (
	BF16, E4M3, INT8,
	AttnDecodeKernel, AttnKernel, AttnKernelConfig, Device, DequantConfig, GeGluConfig, GemmConfig, GemmInputConfig, GemmKernel,
	QkvConfig, QNormConfig, ResidualConfig, RMSNormConfig, RmsNormKernel, ScaleConfig,
)

FIXED_I8_SCALE = 8.0                     # src/main.rs:33
L2_NORM_EPS = 1.0 / 2.0 ** 70            # src/main.rs:35
# src/main.rs:650 == cuda/utils_core.cuh:414-418
GELU_VAR_FIX_2 = 1.0 / ((1.0 / 3.0) + (0.5 / math.pi) * (1.0 / math.sqrt(3.0)))


def _inv_sqrt(x: float) -> float:       # src/util.rs:20-24
	return 1.0 / math.sqrt(x)


def _mode(strict: bool) -> str:
	return "strict" if strict else "fast"


def _gemm(a_dtype, b_dtype, c_dtype, k, n_raw):
	return GemmConfig(GemmInputConfig(a_dtype, k, None, False), GemmInputConfig(b_dtype, k, n_raw, True), c_dtype)


def attn_q_kernel(device: Optional[Device], model_dim: int, q_proj_outputs: int, strict: bool = True) -> GemmKernel:
	"""src/main.rs:387-438 -- x[i8] . Wq[i8]^T with the Scale epilogue -> q[i8]."""
	cfg = ScaleConfig(_inv_sqrt(model_dim) / (FIXED_I8_SCALE * FIXED_I8_SCALE), FIXED_I8_SCALE)
	return GemmKernel(device, f"attn_q_fwd-k{model_dim}-n{q_proj_outputs}-{_mode(strict)}",
	                  _gemm(INT8, INT8, INT8, model_dim, q_proj_outputs), cfg, strict)


def attn_kv_kernel(device: Optional[Device], model_dim: int, kv_proj_outputs: int, head_dim: int,
                   strict: bool = True) -> GemmKernel:
	"""src/main.rs:440-493 -- x . Wkv^T with the L2-norm (RMSNorm) epilogue -> kv[i8], rrms[f32]."""
	cfg = RMSNormConfig(L2_NORM_EPS, head_dim, head_dim,
	                    _inv_sqrt(model_dim) / (FIXED_I8_SCALE * FIXED_I8_SCALE), FIXED_I8_SCALE)
	return GemmKernel(device, f"attn_kv_fwd-k{model_dim}-n{kv_proj_outputs}-hd{head_dim}-{_mode(strict)}",
	                  _gemm(INT8, INT8, INT8, model_dim, kv_proj_outputs), cfg, strict)


def attn_qkv_kernel(device: Optional[Device], model_dim: int, q_proj_outputs: int, kv_proj_outputs: int, head_dim: int,
                    strict: bool = True) -> GemmKernel:
	"""attn_q_kernel and attn_kv_kernel (src/main.rs:387-493) as one launch that reads x once: the first
	q_proj_outputs raw columns go through the Scale writer into q, the rest through the L2-norm writer into kv and
	rrms.  Launch with GemmKernel.launch_qkv; the outputs equal those of the two kernels bit for bit."""
	inp = _inv_sqrt(model_dim) / (FIXED_I8_SCALE * FIXED_I8_SCALE)
	cfg = QkvConfig(q_proj_outputs, ScaleConfig(inp, FIXED_I8_SCALE),
	                RMSNormConfig(L2_NORM_EPS, head_dim, head_dim, inp, FIXED_I8_SCALE))
	return GemmKernel(device, f"attn_qkv_fwd-k{model_dim}-q{q_proj_outputs}-kv{kv_proj_outputs}-hd{head_dim}-{_mode(strict)}",
	                  _gemm(INT8, INT8, INT8, model_dim, q_proj_outputs + kv_proj_outputs), cfg, strict)


def attn_q_norm_kernel(device: Optional[Device], model_dim: int, q_proj_outputs: int, head_dim: int,
                       eps: float = 0.0, strict: bool = True, post_scale: float = 1.0) -> GemmKernel:
	"""The reference's older Q projection with learned scales (attn_q_fwd_i8.cu:30-34 loads q_norm_scales.bin for
	it; writer cuda/qkvg_fwd_i8.cuh:145-219): x[i8] . Wq[i8]^T, every head L2-normalised to sqrt(head_dim) * 8 and
	multiplied by a bf16 scale per column (launch(x, wq, q, q_norm_scales)).  eps = 0 is the old writer; the hook
	that survives in cuda/gemm_b8.cuh:761-824 adds L2_NORM_EPS.  post_scale: the factor applied after the learned
	scales -- the old writer's base class (gone from the reference tree) was built with 1 / sqrt(model_dim),
	cuda/qkvg_fwd_i8.cuh:151-159; 1.0 stores the normalised values as they are."""
	cfg = QNormConfig(eps, head_dim, FIXED_I8_SCALE, post_scale)
	tag = "" if post_scale == 1.0 else f"-post{post_scale:.6g}"
	return GemmKernel(device, f"attn_q_norm_fwd-k{model_dim}-n{q_proj_outputs}-hd{head_dim}{tag}-{_mode(strict)}",
	                  _gemm(INT8, INT8, INT8, model_dim, q_proj_outputs), cfg, strict)


def attn_kernel(device: Optional[Device], n_heads: int, head_dim: int, strict: bool = True) -> AttnKernel:
	"""src/main.rs:495-523 -- int8 sliding-window attention; strides are the dense widths."""
	width = n_heads * head_dim
	cfg = AttnKernelConfig(INT8, n_heads, head_dim, width, 2 * width, width)
	return AttnKernel(device, f"attn_fwd_i8-h{n_heads}-hd{head_dim}-{_mode(strict)}", cfg, strict)


def attn_d_q_kernel(device: Optional[Device], n_heads: int, head_dim: int, strict: bool = True) -> AttnKernel:
	"""The backward of attn_kernel with respect to q (structure of the reference's attn_d_q.cuh:70-383 on the int8
	generation's forward): launch_d_q(q, kv, sink_k, sink_v, temperatures, out, d_out, d_q, l, d, window)."""
	w = n_heads * head_dim
	cfg = AttnKernelConfig(INT8, n_heads, head_dim, w, 2 * w, w, False, INT8, True)
	return AttnKernel(device, f"attn_d_q_i8-h{n_heads}-hd{head_dim}-{_mode(strict)}", cfg, strict)


def attn_d_kv_kernel(device: Optional[Device], n_heads: int, head_dim: int, strict: bool = True) -> AttnKernel:
	"""The backward of attn_kernel with respect to k and v (structure of the reference's attn_d_kv.cuh:200-400 on the
	int8 generation's forward): launch_d_kv(q, kv, temperatures, d_out, l, d, d_kv, window)."""
	w = n_heads * head_dim
	cfg = AttnKernelConfig(INT8, n_heads, head_dim, w, 2 * w, w, False, INT8, False, True)
	return AttnKernel(device, f"attn_d_kv_i8-h{n_heads}-hd{head_dim}-{_mode(strict)}", cfg, strict)


def attn_row_scaled_kernel(device: Optional[Device], n_heads: int, head_dim: int, out_dtype: int = BF16,
                           strict: bool = True) -> AttnKernel:
	"""The attention kernel over int8 codes with one scale per (row, head) -- symmetric absmax / 127
	quantisation of q, k and v -- writing bf16 real values or FixedI8 codes."""
	width = n_heads * head_dim
	cfg = AttnKernelConfig(INT8, n_heads, head_dim, width, 2 * width, width, True, out_dtype)
	tag = "bf16" if out_dtype == BF16 else "i8"
	return AttnKernel(device, f"attn_fwd_i8_rows-h{n_heads}-hd{head_dim}-o{tag}-{_mode(strict)}", cfg, strict)


def attn_y_kernel(device: Optional[Device], model_dim: int, attn_width: int, strict: bool = True,
                  c_dtype: int = E4M3) -> GemmKernel:
	"""src/main.rs:525-576 -- attn_out[i8] . Wy[i8]^T with the gated-residual epilogue -> e4m3."""
	cfg = ResidualConfig(_inv_sqrt(attn_width) / (FIXED_I8_SCALE * FIXED_I8_SCALE), 1.0)
	return GemmKernel(device, f"attn_y_fwd-k{attn_width}-n{2 * model_dim}-c{c_dtype}-{_mode(strict)}",
	                  _gemm(INT8, INT8, c_dtype, attn_width, 2 * model_dim), cfg, strict)


def ffn_f_kernel(device: Optional[Device], model_dim: int, ffn_f_proj_outputs: int, strict: bool = True,
                 c_dtype: int = E4M3) -> GemmKernel:
	"""src/main.rs:578-627 -- x[i8] . Wf[i8]^T with the GeGLU epilogue -> f[e4m3].
	c_dtype=INT8 emits f as FixedI8 instead (out_scale 8), the operand of an int8 ffn_y."""
	out_scale = 1.0 if c_dtype == E4M3 else FIXED_I8_SCALE
	cfg = GeGluConfig(_inv_sqrt(model_dim) / (FIXED_I8_SCALE * FIXED_I8_SCALE), out_scale)
	return GemmKernel(device, f"ffn_f_fwd-k{model_dim}-n{ffn_f_proj_outputs}-c{c_dtype}-{_mode(strict)}",
	                  _gemm(INT8, INT8, c_dtype, model_dim, ffn_f_proj_outputs), cfg, strict)


def ffn_y_kernel(device: Optional[Device], model_dim: int, f_width: int, strict: bool = True,
                 a_dtype: int = E4M3, b_dtype: int = INT8) -> GemmKernel:
	"""src/main.rs:629-678 -- f . Wy^T with the gated-residual epilogue -> e4m3.
	a_dtype=E4M3, b_dtype=INT8 is the reference's ffn_y_fwd_f8; INT8 x INT8 is the int8 variant
	(f in FixedI8 carries one more factor 8); E4M3 x E4M3 is the all-fp8 variant."""
	inp = math.sqrt(GELU_VAR_FIX_2 / f_width)
	if a_dtype == INT8:
		inp /= FIXED_I8_SCALE
	if b_dtype == INT8:
		inp /= FIXED_I8_SCALE
	cfg = ResidualConfig(inp, 1.0)
	return GemmKernel(device, f"ffn_y_fwd-a{a_dtype}b{b_dtype}-k{f_width}-n{2 * model_dim}-{_mode(strict)}",
	                  _gemm(a_dtype, b_dtype, E4M3, f_width, 2 * model_dim), cfg, strict)


def ffn_f_f8_kernel(device: Optional[Device], model_dim: int, ffn_f_proj_outputs: int, strict: bool = True) -> GemmKernel:
	"""All-fp8 ffn_f: x[e4m3] . Wf[e4m3]^T, f32 accumulate, GeGLU -> e4m3.  Operands are real values
	(no FixedI8 factor), so only the 1/sqrt(K) variance fix remains in inp_scale."""
	cfg = GeGluConfig(_inv_sqrt(model_dim), 1.0)
	return GemmKernel(device, f"ffn_f_fwd_f8-k{model_dim}-n{ffn_f_proj_outputs}-{_mode(strict)}",
	                  _gemm(E4M3, E4M3, E4M3, model_dim, ffn_f_proj_outputs), cfg, strict)


def mixed_gemm_kernel(device: Optional[Device], k: int, n_raw: int, geglu: bool, strict: bool = True) -> GemmKernel:
	"""e4m3 activations x int8 weights with the Scale writer (-> FixedI8) or the GeGLU writer (-> e4m3): the
	operand mix of ffn_y_fwd_f8 (cuda/gemm_b16.cuh:72-185) under the other two writers that accept f32 sums."""
	inp = _inv_sqrt(k) / FIXED_I8_SCALE
	if geglu:
		return GemmKernel(device, f"mixed_geglu-k{k}-n{n_raw}-{_mode(strict)}", _gemm(E4M3, INT8, E4M3, k, n_raw),
		                  GeGluConfig(inp, 1.0), strict)
	return GemmKernel(device, f"mixed_scale-k{k}-n{n_raw}-{_mode(strict)}", _gemm(E4M3, INT8, INT8, k, n_raw),
	                  ScaleConfig(inp, FIXED_I8_SCALE), strict)


def dequant_gemm_kernel(device: Optional[Device], k: int, n_raw: int, a_dtype: int = INT8, b_dtype: int = INT8,
                        geglu: bool = False, strict: bool = True) -> GemmKernel:
	"""No counterpart in src/main.rs: a[M, k] . b[n_raw, k]^T with run-time per-row and per-column f32
	dequantisation scales -> bf16 [M, n_raw] (or GeGLU over column pairs -> bf16 [M, n_raw / 2]).  This is
	the literal form of symmetric per-token / per-output-channel int8 (scale = absmax / 127) and of e4m3
	operands with per-tensor scales."""
	name = f"dequant_gemm-a{a_dtype}b{b_dtype}-k{k}-n{n_raw}-{'geglu' if geglu else 'plain'}-{_mode(strict)}"
	return GemmKernel(device, name, _gemm(a_dtype, b_dtype, BF16, k, n_raw), DequantConfig(geglu), strict)


def rms_norm_kernel(device: Optional[Device], model_dim: int, in_dtype: int = E4M3, eps: float = L2_NORM_EPS) -> RmsNormKernel:
	"""rms_norm.cu:55-113."""
	return RmsNormKernel(device, f"rms_norm-d{model_dim}-in{in_dtype}", in_dtype, model_dim, eps)


def attn_decode_kernel(device: Optional[Device], n_heads: int, head_dim: int, cache_capacity: int,
                       strict: bool = True) -> AttnDecodeKernel:
	return AttnDecodeKernel(device, f"attn_decode_i8-h{n_heads}-hd{head_dim}-cap{cache_capacity}-{_mode(strict)}",
	                        n_heads, head_dim, cache_capacity, strict)


def attn_decode_row_scaled_kernel(device: Optional[Device], n_heads: int, head_dim: int, cache_capacity: int,
                                  out_dtype: int = BF16, strict: bool = True) -> AttnDecodeKernel:
	"""The decode kernel over a cache of int8 codes with one scale per (row, head)."""
	tag = "bf16" if out_dtype == BF16 else "i8"
	return AttnDecodeKernel(device, f"attn_decode_i8_rows-h{n_heads}-hd{head_dim}-cap{cache_capacity}-o{tag}-{_mode(strict)}",
	                        n_heads, head_dim, cache_capacity, strict, True, out_dtype)


def attn_row_scale_operands(v_scale, out_dtype: int):
	"""Per-head operands of the row-scaled attention kernels from the value rows' scales.

	v_scale: float32 [n_heads, rows] (prefill) or [S, n_heads, capacity] (decode caches), real v = code * v_scale.
	Returns float32 arrays (v_weight shaped like v_scale, sink_v_weight [n_heads], out_scale [n_heads]): each
	head's largest value scale becomes its reference scale v_ref, a row's 8-bit probabilities are weighted by
	v_scale / v_ref <= 1, the sink value (a FixedI8 code, real = code / 8) enters at (1 / 8) / v_ref, and the
	result is brought back by v_ref (bf16 output, real values) or 8 * v_ref (FixedI8 output)."""
	import numpy as np
	v_scale = np.asarray(v_scale, dtype=np.float32)
	if v_scale.ndim not in (2, 3) or not np.all(np.isfinite(v_scale)) or not np.all(v_scale > 0):
		raise ValueError("v_scale must be a [n_heads, rows] or [S, n_heads, capacity] array of finite positive scales")
	v_ref = v_scale.max(axis=-1) if v_scale.ndim == 2 else v_scale.max(axis=(0, 2))
	v_weight = (v_scale / v_ref[:, None]).astype(np.float32)
	sink_v_weight = (np.float32(1.0 / FIXED_I8_SCALE) / v_ref).astype(np.float32)
	if out_dtype == BF16:
		out_scale = v_ref
	elif out_dtype == INT8:
		out_scale = (np.float32(FIXED_I8_SCALE) * v_ref).astype(np.float32)
	else:
		raise ValueError("row-scaled attention writes int8 or bf16")
	return v_weight, sink_v_weight, out_scale
