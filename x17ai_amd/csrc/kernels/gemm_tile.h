// gemm_tile.h -- tile geometry of the 8-bit GEMM kernel as plain constexprs.
//
// Included by the device code (gemm_b8.hip) and by the small host program that prints
// meta.json, so that the C++ constants stay the single source of truth for the launch
// geometry, as in the reference (templates/basic_gemm/meta.cu:10-17,
// src/device/cuda/gemm.rs:529-537).  Needs X17_A_KIND / X17_B_KIND from common.h.
//
// A build may override the geometry with -DX17_GEMM_M_PER_BLOCK (128 or 256 tokens per workgroup),
// -DX17_GEMM_WAVES_M / -DX17_GEMM_WAVES_N (wavefronts along the tokens / along the raw output columns),
// -DX17_GEMM_K_STEP (64 or 128 bytes of K per pipeline step), -DX17_GEMM_STAGES (LDS ring depth) and
// -DX17_GEMM_X_STAGES (ring depth of the token operand alone: STAGES or STAGES + 1).  Needs X17_A_COLS too.
#pragma once

namespace x17 { namespace gemm_tile {

constexpr unsigned WAVE = 64;

#ifndef X17_GEMM_M_PER_BLOCK
#define X17_GEMM_M_PER_BLOCK 256
#endif
#ifndef X17_GEMM_WAVES_M
#define X17_GEMM_WAVES_M 4
#endif
#ifndef X17_GEMM_WAVES_N
#define X17_GEMM_WAVES_N 2
#endif
#ifndef X17_GEMM_K_STEP
#define X17_GEMM_K_STEP 128
#endif
#ifndef X17_GEMM_STAGES
#define X17_GEMM_STAGES 2
#endif

constexpr unsigned M_PER_BLOCK = X17_GEMM_M_PER_BLOCK;   // tokens per workgroup
constexpr unsigned N_PER_BLOCK = 256;                    // raw output columns per workgroup
constexpr unsigned WAVES_M = X17_GEMM_WAVES_M;           // waves along the token (M) dimension
constexpr unsigned WAVES_N = X17_GEMM_WAVES_N;           // waves along the output-column (N) dimension
constexpr unsigned THREADS_PER_BLOCK = WAVE * WAVES_M * WAVES_N;

constexpr unsigned WAVE_M = M_PER_BLOCK / WAVES_M;       // tokens per wave (64 or 128)
constexpr unsigned WAVE_N = N_PER_BLOCK / WAVES_N;       // raw output columns per wave (128 or 64)
constexpr unsigned K_STEP = X17_GEMM_K_STEP;             // bytes of K staged per pipeline step
constexpr unsigned STAGES = X17_GEMM_STAGES;

// The token tiles may have a ring one deeper than the weight tiles: 3 x 32 KB + 2 x 32 KB fill the 160 KB of
// LDS of a compute unit exactly, and the token loads then have two steps to arrive, the weight loads one
// (with two stages of both, a step's 64 KB of loads have a single step -- about their own latency -- to land).
#ifndef X17_GEMM_X_STAGES
#define X17_GEMM_X_STAGES \
	((X17_GEMM_STAGES == 2 && X17_GEMM_K_STEP == 128 && X17_GEMM_M_PER_BLOCK == 256 && (X17_A_COLS) / 128 >= 3) ? 3 : X17_GEMM_STAGES)
#endif
constexpr unsigned X_STAGES = X17_GEMM_X_STAGES;
static_assert(X_STAGES == STAGES || X_STAGES == STAGES + 1, "the token ring is as deep as the weight ring or one deeper");

constexpr unsigned SMEM_BYTES = (X_STAGES * M_PER_BLOCK + STAGES * N_PER_BLOCK) * K_STEP;

// The kernel is persistent (a workgroup walks tiles g, g + G, ...): the launcher starts at most this
// many workgroups, one per compute unit of an MI355X.
constexpr unsigned MAX_BLOCKS = 256;

// Wavefronts per SIMD the register budget is sized for: waves of eight 32 x 32 blocks (64 x 128 or 128 x 64)
// keep their 128 accumulators and everything else within 256 registers so that two of them share a SIMD
// (two workgroups per compute unit when a workgroup has four waves); 128 x 128 waves need all 512.
constexpr unsigned WAVES_PER_SIMD = (WAVE_M / 32) * (WAVE_N / 32) <= 8 ? 2 : 1;

static_assert(M_PER_BLOCK == 128 || M_PER_BLOCK == 256, "tokens per workgroup: 128 or 256");
static_assert(WAVE_M == 64 || WAVE_M == 128, "a wave owns 64 or 128 tokens");
static_assert(WAVE_N == 128 || WAVE_N == 64, "a wave owns 128 or 64 raw output columns");
static_assert(K_STEP == 64 || K_STEP == 128, "K step: 64 or 128 bytes");
static_assert(STAGES >= 2 && STAGES <= 4, "2 to 4 stages");
static_assert(SMEM_BYTES <= 160 * 1024, "LDS ring does not fit");

}} // namespace x17::gemm_tile
