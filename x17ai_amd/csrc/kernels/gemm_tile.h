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

// ---- index arithmetic of the tile requests (global -> LDS, 16 bytes per lane).  The kernel calls these; so does the
// host-side audit (gemm_requests_audit.cpp), which enumerates every request of a launch on the CPU and checks that it
// stays inside its operand.
// LDS rows hold K_STEP bytes = CHUNKS chunks of 16; one 64-lane load fills UNIT_ROWS rows ("a load unit").
constexpr unsigned CHUNKS = K_STEP / 16;
constexpr unsigned SWZ_SHIFT = K_STEP == 128 ? 1 : 2;
constexpr unsigned UNIT_ROWS = 64 / CHUNKS;
// With eight waves, two per SIMD, only the first of each pair (waves 0 .. 3) requests tiles.
constexpr unsigned LOADER_WAVES = WAVES_M * WAVES_N == 8 ? 4 : WAVES_M * WAVES_N;
constexpr unsigned X_UNITS = M_PER_BLOCK / UNIT_ROWS / LOADER_WAVES;   // load units per loading wave, step and tile
constexpr unsigned W_UNITS = N_PER_BLOCK / UNIT_ROWS / LOADER_WAVES;
// The weight row that LDS weight row r0 (a multiple of UNIT_ROWS) starts from.  With WN = WAVE_N columns per wave, LDS
// weight row R = WN*wn + 32*bn + i holds weight row WN*wn + (WN/2)*((i/4)%2) + 16*bn + 4*(i/8) + i%4 (so that a lane
// collects consecutive output columns); the head-normalising writers keep the natural order.
constexpr unsigned w_unit_row(unsigned r0, bool natural) {
	return natural ? r0 : WAVE_N * (r0 / WAVE_N) + 16 * ((r0 % WAVE_N) / 32) + 4 * ((r0 % 32) / 8);
}
// Row inside its load unit, as an operand row offset, and 16-byte chunk of the K step that lane `lane` fetches
// (`odd`: parity of the unit, which shifts the swizzle phase).
constexpr unsigned x_lane_row(unsigned lane) { return lane / CHUNKS; }
constexpr unsigned w_lane_row(unsigned lane, bool natural) {
	unsigned const j = lane / CHUNKS;
	return natural ? j : (WAVE_N / 2) * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);
}
constexpr unsigned lane_chunk(unsigned lane, unsigned odd) {
	unsigned const j = lane / CHUNKS, p = lane % CHUNKS;
	return p ^ (((odd * UNIT_ROWS + j) >> SWZ_SHIFT) & (CHUNKS - 1));
}
// First token row and first raw column of tile `lin` of the persistent walk: each XCD (the hardware deals workgroups
// round-robin to 8 of them) gets a contiguous run of tiles, walked in bands of `band` token tiles; a last tile that
// would overhang the matrix is moved back to end at its edge.
struct TileOrigin { unsigned m, n; };
constexpr TileOrigin tile_origin(unsigned lin, unsigned a_rows, unsigned n_raw, unsigned band) {
	unsigned const tiles_m = (a_rows + M_PER_BLOCK - 1) / M_PER_BLOCK;
	unsigned const tiles_n = (n_raw + N_PER_BLOCK - 1) / N_PER_BLOCK;
	unsigned const total = tiles_m * tiles_n;
	if (total % 8 == 0) {
		lin = (lin % 8) * (total / 8) + lin / 8;
	}
	unsigned const band_tiles = band * tiles_n;
	unsigned const b = lin / band_tiles;
	unsigned const in_band = lin % band_tiles;
	unsigned const rows_in_band = (tiles_m - b * band) < band ? (tiles_m - b * band) : band;
	unsigned m = (b * band + in_band % rows_in_band) * M_PER_BLOCK;
	unsigned n = (in_band / rows_in_band) * N_PER_BLOCK;
	m = m + M_PER_BLOCK > a_rows ? a_rows - M_PER_BLOCK : m;
	n = n + N_PER_BLOCK > n_raw ? n_raw - N_PER_BLOCK : n;
	return TileOrigin{m, n};
}
#ifdef X17_GEMM_BAND
constexpr unsigned BAND = X17_GEMM_BAND;
#else
constexpr unsigned BAND = 2048 / M_PER_BLOCK;
#endif

static_assert(M_PER_BLOCK == 128 || M_PER_BLOCK == 256, "tokens per workgroup: 128 or 256");
static_assert(WAVE_M == 64 || WAVE_M == 128, "a wave owns 64 or 128 tokens");
static_assert(WAVE_N == 128 || WAVE_N == 64, "a wave owns 128 or 64 raw output columns");
static_assert(K_STEP == 64 || K_STEP == 128, "K step: 64 or 128 bytes");
static_assert(STAGES >= 2 && STAGES <= 4, "2 to 4 stages");
static_assert(SMEM_BYTES <= 160 * 1024, "LDS ring does not fit");

}} // namespace x17::gemm_tile
