"""Shared helpers of the GPU parity tests: seeded inputs in the reference's number formats."""
from __future__ import annotations

import zlib

import numpy as np

from oracle import strict as S


def rng_for(*key) -> np.random.Generator:
	"""A generator seeded by the test's name and parameters: the same inputs in every run and on every machine
	(Python's own hash of a string changes from process to process)."""
	return np.random.default_rng(zlib.crc32(repr(tuple(key)).encode()))


def i8_codes(rng: np.random.Generator, shape, sigma: float = 1.0) -> np.ndarray:
	"""FixedI8 codes of N(0, sigma^2) reals: clamp(rne(8 x), +-127) (new_block.py:12-16)."""
	return S.f32_to_fixedi8((rng.standard_normal(shape) * (8.0 * sigma)).astype(np.float32))


def e4m3_bytes(rng: np.random.Generator, shape, sigma: float = 1.0) -> np.ndarray:
	"""e4m3 bytes of N(0, sigma^2) reals in the reference's dialect (cuda/utils_b8.cuh:636-647)."""
	return S.f32_to_e4m3((rng.standard_normal(shape) * sigma).astype(np.float32))


def e4m3_compare(a: np.ndarray, b: np.ndarray):
	"""(fraction of differing bytes, fraction differing by more than one grid step)."""
	av = S.e4m3_to_f32(a).astype(np.float64)
	bv = S.e4m3_to_f32(b).astype(np.float64)
	neq = a != b
	big = np.maximum(np.abs(av), np.abs(bv))
	rel = np.abs(av - bv) / np.where(big == 0, 1.0, big)
	# one step of the e4m3 grid is at most 12.5 % of the larger magnitude; flushes against 2^-6 count as one step
	beyond = neq & (rel > 0.126) & (big > 2.0 ** -6)
	return float(np.mean(neq)), float(np.mean(beyond))
