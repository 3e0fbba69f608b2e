"""The quantized transformer-block forward as one object: the stage order, the kernels and the files of the
reference's block driver (src/main.rs:37-385).

main.rs loads nine single-tensor files (x and the weights, block_utils.py:49-100 naming), builds six kernels
with the scale recipes of src/main.rs:387-675, launches q -> kv -> attention -> attn_y -> ffn_f -> ffn_y on
one stream with an event pair around each, and stores eight outputs.  `Block` owns exactly that; `main()` is
the driver (`python -m x17ai_amd.block --input tmp/block_torch --output tmp/block_hip`).

Two additions, both off by default so that the default object IS main.rs:
  * `rms_norm_input`: the residual stream arrives as bf16 (or e4m3) and rms_norm.cu:55-113 turns it into the
    FixedI8 x first (the inter-block step: rms_norm.cu reads the previous block's ffn_y);
  * `batch`: the token rows are `batch` independent sequences of equal length (grid.z of the attention launch).
q, kv and ffn_f all read the same x; attn_y and ffn_y each gate-mix their branch with x and are stored
separately, as in main.rs (no final sum).
"""
from __future__ import annotations

import argparse
import dataclasses
import os
import sys
from typing import Callable, Dict, List, Optional, Tuple

from . import recipes
from .api import BF16, E4M3, F32, INT8, Device, Tensor, Timer
from ._ffi import X17Error
from .tensor_files import load_tensor_file

# src/main.rs:40-75 -- (key, file stem) of the nine inputs, in load order
INPUT_FILES: Tuple[Tuple[str, str], ...] = (
	("x", "x_i8"),
	("attn_q_weights", "attn_q_weights_i8"),
	("attn_kv_weights", "attn_kv_weights_i8"),
	("ffn_f_weights", "ffn_f_weights_i8"),
	("ffn_y_weights", "ffn_y_weights_i8"),
	("attn_y_weights", "attn_y_weights_i8"),
	("sinks_k", "sinks_k_i8"),
	("sinks_v", "sinks_v_i8"),
	("attn_temperature", "attn_temperature_f32"),
)
# src/main.rs:273-280 -- (key, file stem) of the eight outputs, in store order
OUTPUT_FILES: Tuple[Tuple[str, str], ...] = (
	("q", "q_i8"),
	("kv", "kv_i8"),
	("k_rrms", "k_rrms_f32"),
	("attn_out", "attn_out_i8"),
	("attn_l", "attn_l_f32"),
	("attn_y", "attn_y_f8"),
	("ffn_f", "ffn_f_f8"),
	("ffn_y", "ffn_y_f8"),
)
# launch order, src/main.rs:193-263 (rms_norm first when the block is given the residual stream)
STAGE_ORDER: Tuple[str, ...] = ("rms_norm", "attn_q", "attn_kv", "attn_fwd_i8", "attn_y", "ffn_f", "ffn_y_f8")


@dataclasses.dataclass
class BlockConfig:
	"""The constants of src/main.rs:28-35 (block.config.json) as a value."""
	model_dim: int
	n_heads: int
	head_dim: int
	f_width: int
	window_size: int = 0
	batch: int = 1
	rms_norm_input: Optional[int] = None      # None: x is FixedI8 (main.rs); BF16 / E4M3: rms_norm runs first
	strict_math: bool = True
	# one launch for the q and kv projections (x read once), instead of main.rs's two
	fused_qkv: bool = False

	@property
	def attn_width(self) -> int:
		return self.n_heads * self.head_dim


def _expect(t: Tensor, name: str, dtype: int, shape) -> None:
	if t.dtype != dtype:
		raise X17Error(f"expected {name} dtype {dtype}, got {t.dtype}")
	if tuple(t.shape) != tuple(shape):
		raise X17Error(f"expected {name} shape {tuple(shape)}, got {tuple(t.shape)}")


class Block:
	"""The six (seven with rms_norm) kernels of one block and their launch order."""

	def __init__(self, device: Optional[Device], config: BlockConfig):
		c = config
		self.device = device
		self.config = c
		s = c.strict_math
		self.k_rms = None if c.rms_norm_input is None else recipes.rms_norm_kernel(device, c.model_dim, c.rms_norm_input)
		if c.fused_qkv:
			self.k_qkv = recipes.attn_qkv_kernel(device, c.model_dim, c.attn_width, 2 * c.attn_width, c.head_dim, s)
			self.k_q = self.k_kv = None
		else:
			self.k_qkv = None
			self.k_q = recipes.attn_q_kernel(device, c.model_dim, c.attn_width, s)
			self.k_kv = recipes.attn_kv_kernel(device, c.model_dim, 2 * c.attn_width, c.head_dim, s)
		self.k_attn = recipes.attn_kernel(device, c.n_heads, c.head_dim, s)
		self.k_attn_y = recipes.attn_y_kernel(device, c.model_dim, c.attn_width, s)
		self.k_ffn_f = recipes.ffn_f_kernel(device, c.model_dim, 2 * c.f_width, s)
		self.k_ffn_y = recipes.ffn_y_kernel(device, c.model_dim, c.f_width, s)

	# ------------------------------------------------------------ validation (src/main.rs:680-1060)
	def validate(self, n_inputs: int, w: Dict[str, Tensor]) -> None:
		c = self.config
		if n_inputs == 0 or n_inputs % c.batch != 0:
			raise X17Error(f"expected x rows to be a positive multiple of batch={c.batch}, got {n_inputs}")
		_expect(w["attn_q_weights"], "attn_q_weights", INT8, (c.attn_width, c.model_dim))
		kvw = w["attn_kv_weights"]
		if kvw.dtype != INT8:
			raise X17Error(f"expected attn_kv_weights dtype i8, got {kvw.dtype}")
		if len(kvw.shape) == 4:
			# src/main.rs:763-772: [heads, 2, head_dim, model_dim] is accepted and flattened
			if tuple(kvw.shape) != (c.n_heads, 2, c.head_dim, c.model_dim):
				raise X17Error(f"expected attn_kv_weights shape [{c.n_heads}, 2, {c.head_dim}, {c.model_dim}], got {list(kvw.shape)}")
			kvw.reshape((2 * c.attn_width, c.model_dim))
		_expect(kvw, "attn_kv_weights", INT8, (2 * c.attn_width, c.model_dim))
		_expect(w["attn_y_weights"], "attn_y_weights", INT8, (2 * c.model_dim, c.attn_width))
		_expect(w["ffn_f_weights"], "ffn_f_weights", INT8, (2 * c.f_width, c.model_dim))
		_expect(w["ffn_y_weights"], "ffn_y_weights", INT8, (2 * c.model_dim, c.f_width))
		_expect(w["sinks_k"], "sinks_k", INT8, (c.n_heads, c.head_dim))
		_expect(w["sinks_v"], "sinks_v", INT8, (c.n_heads, c.head_dim))
		t = w["attn_temperature"]
		if t.dtype != F32 or int(_numel(t.shape)) != c.n_heads:
			raise X17Error(f"expected attn_temperature to hold {c.n_heads} f32 values, got dtype {t.dtype} shape {list(t.shape)}")

	def new_outputs(self, n_inputs: int) -> Dict[str, Tensor]:
		"""src/main.rs:79-86."""
		c, dev = self.config, self.device
		out = {
			"q": Tensor(dev, (n_inputs, c.attn_width), INT8),
			"kv": Tensor(dev, (n_inputs, 2 * c.attn_width), INT8),
			"k_rrms": Tensor(dev, (n_inputs, c.n_heads), F32),
			"attn_out": Tensor(dev, (n_inputs, c.attn_width), INT8),
			"attn_l": Tensor(dev, (c.n_heads, n_inputs), F32),
			"attn_y": Tensor(dev, (n_inputs, c.model_dim), E4M3),
			"ffn_f": Tensor(dev, (n_inputs, c.f_width), E4M3),
			"ffn_y": Tensor(dev, (n_inputs, c.model_dim), E4M3),
		}
		if c.rms_norm_input is not None:
			out["x"] = Tensor(dev, (n_inputs, c.model_dim), INT8)
		return out

	def stages(self, x: Tensor, w: Dict[str, Tensor], out: Dict[str, Tensor]) -> List[Tuple[str, Callable[[], None]]]:
		"""(name, launch) of every stage in launch order.  `x` is the FixedI8 x, or the bf16 / e4m3 residual
		stream when the block was configured with rms_norm_input (the FixedI8 x is then out["x"])."""
		c = self.config
		n_inputs = x.shape[0]
		seq_len = n_inputs // c.batch
		st: List[Tuple[str, Callable[[], None]]] = []
		if self.k_rms is not None:
			_expect(x, "x", c.rms_norm_input, (n_inputs, c.model_dim))
			xi = out["x"]
			st.append(("rms_norm", lambda: self.k_rms.launch(x, xi)))
		else:
			_expect(x, "x", INT8, (n_inputs, c.model_dim))
			xi = x
		if self.k_qkv is not None:
			st.append(("attn_qkv", lambda: self.k_qkv.launch_qkv(xi, w["attn_q_weights"], w["attn_kv_weights"], out["q"],
			                                                    out["kv"], out["k_rrms"])))
		else:
			st.append(("attn_q", lambda: self.k_q.launch(xi, w["attn_q_weights"], out["q"])))
			st.append(("attn_kv", lambda: self.k_kv.launch(xi, w["attn_kv_weights"], out["kv"], out["k_rrms"])))
		st.append(("attn_fwd_i8", lambda: self.k_attn.launch(out["q"], out["kv"], w["sinks_k"], w["sinks_v"], w["attn_temperature"],
		                                                     out["attn_out"], out["attn_l"], c.window_size, c.batch)))
		st.append(("attn_y", lambda: self.k_attn_y.launch(out["attn_out"], w["attn_y_weights"], out["attn_y"], xi)))
		st.append(("ffn_f", lambda: self.k_ffn_f.launch(xi, w["ffn_f_weights"], out["ffn_f"])))
		st.append(("ffn_y_f8", lambda: self.k_ffn_y.launch(out["ffn_f"], w["ffn_y_weights"], out["ffn_y"], xi)))
		del seq_len
		return st

	def n_ops(self, n_inputs: int) -> Dict[str, float]:
		"""Operations per stage as main.rs prints them (gemm.rs:445-449, attn.rs:72-84)."""
		c = self.config
		g = lambda k, n: 2.0 * n_inputs * k * n
		return {
			"attn_q": g(c.model_dim, c.attn_width), "attn_kv": g(c.model_dim, 2 * c.attn_width),
			"attn_qkv": g(c.model_dim, 3 * c.attn_width),
			"attn_fwd_i8": c.batch * self.k_attn.n_ops(n_inputs // c.batch, c.window_size),
			"attn_y": g(c.attn_width, 2 * c.model_dim), "ffn_f": g(c.model_dim, 2 * c.f_width),
			"ffn_y_f8": g(c.f_width, 2 * c.model_dim),
		}

	def forward(self, x: Tensor, w: Dict[str, Tensor], out: Optional[Dict[str, Tensor]] = None,
	            timers: Optional[Dict[str, Timer]] = None) -> Dict[str, Tensor]:
		"""Launches every stage on the device's stream (nothing is synchronised).  With `timers` (a dict that is
		filled with one Timer per stage) each launch sits between an event pair, as in src/main.rs:193-263."""
		self.validate(x.shape[0], w)
		if out is None:
			out = self.new_outputs(x.shape[0])
		for name, launch in self.stages(x, w, out):
			if timers is not None:
				t = timers.get(name) or Timer(self.device)
				timers[name] = t
				t.start()
				launch()
				t.stop()
			else:
				launch()
		return out


def _numel(shape) -> int:
	n = 1
	for s in shape:
		n *= int(s)
	return n


def load_inputs(directory: str, device: Optional[Device]) -> Dict[str, Tensor]:
	"""The nine `<name>_<tag>.safetensors` files of src/main.rs:40-75."""
	return {key: load_tensor_file(os.path.join(directory, stem + ".safetensors"), device) for key, stem in INPUT_FILES}


def save_outputs(directory: str, out: Dict[str, Tensor], config: BlockConfig) -> List[str]:
	"""src/main.rs:264-280: download, synchronise, one file per tensor; kv is stored as [n, heads, 2, head_dim]."""
	os.makedirs(directory, exist_ok=True)
	paths = []
	for key, stem in OUTPUT_FILES:
		cpu = out[key].to_cpu()
		if key == "kv":
			cpu.reshape((cpu.shape[0], config.n_heads, 2, config.head_dim))
		path = os.path.join(directory, stem + ".safetensors")
		cpu.save_safetensors_file(path)
		paths.append(path)
	return paths


def main(argv=None) -> int:
	ap = argparse.ArgumentParser(description="block forward over the reference's tensor files (twin of src/main.rs)")
	ap.add_argument("--input", default=os.path.join("tmp", "block_torch"))
	ap.add_argument("--output", default=os.path.join("tmp", "block_hip"))
	ap.add_argument("--head-dim", type=int, default=32)          # src/main.rs:28-35
	ap.add_argument("--n-heads", type=int, default=64)
	ap.add_argument("--f-width", type=int, default=2048)
	ap.add_argument("--window-size", type=int, default=0)
	ap.add_argument("--batch", type=int, default=1)
	ap.add_argument("--fast-math", action="store_true", help="hardware transcendentals instead of the deterministic ones")
	ap.add_argument("--fused-qkv", action="store_true")
	args = ap.parse_args(argv)

	dev = Device(0)
	w = load_inputs(args.input, dev)
	x = w.pop("x")
	if len(x.shape) != 2:
		raise X17Error(f"expected x to be rank 2, got shape {list(x.shape)}")
	n_inputs, model_dim = x.shape
	cfg = BlockConfig(model_dim, args.n_heads, args.head_dim, args.f_width, args.window_size, args.batch, None,
	                  not args.fast_math, args.fused_qkv)
	block = Block(dev, cfg)
	timers: Dict[str, Timer] = {}
	out = block.forward(x, w, None, timers)
	paths = save_outputs(args.output, out, cfg)
	dev.synchronize()
	print("loaded:")
	for key, _ in INPUT_FILES:
		t = x if key == "x" else w[key]
		print(f"\t{key}: {list(t.shape)} dtype {t.dtype}, {t.nbytes} bytes")
	print("launched:")
	ops = block.n_ops(n_inputs)
	for name, t in timers.items():
		s = t.elapsed_seconds()
		print(f"\t{name} in {s * 1e3:.4f} ms, {ops[name] / s / 1e12:.3f} TFLOPS")
	print("stored:")
	for p in paths:
		print(f"\t{p}")
	return 0


if __name__ == "__main__":
	sys.exit(main())
