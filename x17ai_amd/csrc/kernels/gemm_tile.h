// gemm_tile.h -- tile geometry of the 8-bit GEMM kernel as plain constexprs.
//
// Included by the device code (gemm_b8.hip) and by the small host program that prints
// meta.json, so that the C++ constants stay the single source of truth for the launch
// geometry, as in the reference (templates/basic_gemm/meta.cu:10-17,
// src/device/cuda/gemm.rs:529-537).  Needs X17_A_KIND / X17_B_KIND from common.h.
#pragma once

namespace x17 { namespace gemm_tile {

constexpr unsigned WAVE = 64;
#ifndef X17_GEMM_WAVES_M
#define X17_GEMM_WAVES_M 4
#endif
// 4 x 2 waves (two per SIMD, 64 x 128 each: the second wave fills the first one's MFMA issue gaps)
// or 2 x 2 waves (one per SIMD, 128 x 128 each: fewest LDS reads per MFMA)
constexpr unsigned WAVES_M = X17_GEMM_WAVES_M;  // waves along the token (M) dimension
constexpr unsigned WAVES_N = 2;                 // waves along the output-column (N) dimension
constexpr unsigned THREADS_PER_BLOCK = WAVE * WAVES_M * WAVES_N;

constexpr unsigned WAVE_M = 256 / WAVES_M;      // tokens per wave
constexpr unsigned WAVE_N = 128;                // raw output columns per wave
constexpr unsigned M_PER_BLOCK = WAVE_M * WAVES_M;
constexpr unsigned N_PER_BLOCK = WAVE_N * WAVES_N;
constexpr unsigned K_STEP = 128;                // bytes of K staged per pipeline step
constexpr unsigned STAGES = 2;

constexpr unsigned SMEM_BYTES = STAGES * (M_PER_BLOCK + N_PER_BLOCK) * K_STEP;

}} // namespace x17::gemm_tile
