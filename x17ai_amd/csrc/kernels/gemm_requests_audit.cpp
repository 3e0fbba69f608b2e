// Host-side audit of the GEMM kernel's tile requests.  Compiled with the kernel's own common.h and gemm_tile.h -- the
// index arithmetic below IS the kernel's (gemm_b8.hip calls the same functions) -- it enumerates, on the CPU, every
// 16-byte direct-to-LDS request a launch with `a_rows` token rows makes: every tile of the persistent walk, every K
// step, every loading wave, load unit and lane.  It checks that each request stays inside its operand and that the
// requests of one tile and step cover the tile's 16-byte chunks exactly once, and prints the extents as JSON.
//
//     gemm_requests_audit <a_rows> [rows the token operand really has, default a_rows]
//
// No GPU is involved; a kernel whose requests would leave an operand is found here, not on the device.
#include "common.h"
#include "gemm_tile.h"

#include <cstdio>
#include <cstdlib>
#include <vector>

namespace gt = x17::gemm_tile;

static int fail(char const *what, unsigned long long a, unsigned long long b) {
	std::printf("{\"ok\": false, \"error\": \"%s\", \"value\": %llu, \"limit\": %llu}\n", what, a, b);
	return 1;
}

int main(int argc, char **argv) {
	if (argc != 2 && argc != 3) {
		std::fprintf(stderr, "usage: %s <a_rows> [allocated rows]\n", argv[0]);
		return 2;
	}
	unsigned long long const a_rows_arg = std::strtoull(argv[1], nullptr, 10);
	unsigned long long const a_rows_allocated = argc == 3 ? std::strtoull(argv[2], nullptr, 10) : a_rows_arg;
	constexpr unsigned K = X17_A_COLS, N_RAW = X17_B_ROWS;
	constexpr bool NATURAL = X17_EPILOGUE == 3 || X17_EPILOGUE == 5 || X17_EPILOGUE == 6;
#if X17_EPILOGUE == 6
	constexpr unsigned Q_COLS = X17_Q_COLS;
#else
	constexpr unsigned Q_COLS = N_RAW;       // one weight matrix
#endif
	if (a_rows_arg < gt::M_PER_BLOCK || a_rows_arg % 64 != 0 || a_rows_arg > 0xFFFFFFFFull) {
		return fail("token rows must be a multiple of 64, at least one tile and fit 32 bits (the launcher rejects them)", a_rows_arg, gt::M_PER_BLOCK);
	}
	unsigned const a_rows = (unsigned)a_rows_arg;
	constexpr unsigned K_STEPS = K / gt::K_STEP;

	// the pattern of one tile and step, relative to the tile's origin: (row, chunk) of every lane of every load
	std::vector<unsigned> x_seen(gt::M_PER_BLOCK * gt::CHUNKS, 0), w_seen(gt::N_PER_BLOCK * gt::CHUNKS, 0);
	unsigned x_max_row = 0, w_max_row = 0, max_chunk = 0;
	unsigned long long per_step = 0;
	for (unsigned wave = 0; wave < gt::LOADER_WAVES; ++wave) {
		for (unsigned u = 0; u < gt::X_UNITS; ++u) {
			for (unsigned lane = 0; lane < 64; ++lane) {
				unsigned const row = (wave * gt::X_UNITS + u) * gt::UNIT_ROWS + gt::x_lane_row(lane);
				unsigned const chunk = gt::lane_chunk(lane, u & 1);
				if (row >= gt::M_PER_BLOCK) return fail("token row of a request outside its tile", row, gt::M_PER_BLOCK);
				if (chunk >= gt::CHUNKS) return fail("chunk of a request outside the K step", chunk, gt::CHUNKS);
				++x_seen[row * gt::CHUNKS + chunk];
				x_max_row = row > x_max_row ? row : x_max_row;
				max_chunk = chunk > max_chunk ? chunk : max_chunk;
				++per_step;
			}
		}
		for (unsigned u = 0; u < gt::W_UNITS; ++u) {
			for (unsigned lane = 0; lane < 64; ++lane) {
				unsigned const r0 = (wave * gt::W_UNITS + u) * gt::UNIT_ROWS;
				unsigned const row = gt::w_unit_row(r0, NATURAL) + gt::w_lane_row(lane, NATURAL);
				unsigned const chunk = gt::lane_chunk(lane, u & 1);
				if (row >= gt::N_PER_BLOCK) return fail("weight row of a request outside its tile", row, gt::N_PER_BLOCK);
				if (chunk >= gt::CHUNKS) return fail("chunk of a request outside the K step", chunk, gt::CHUNKS);
				++w_seen[row * gt::CHUNKS + chunk];
				w_max_row = row > w_max_row ? row : w_max_row;
				++per_step;
			}
		}
	}
	for (unsigned v : x_seen) if (v != 1) return fail("a token-tile chunk is not requested exactly once", v, 1);
	for (unsigned v : w_seen) if (v != 1) return fail("a weight-tile chunk is not requested exactly once", v, 1);

	// every tile of the walk (whatever the grid: workgroup g of G takes tiles g, g + G, ...), every K step
	unsigned const tiles_m = (a_rows + gt::M_PER_BLOCK - 1) / gt::M_PER_BLOCK;
	unsigned const tiles_n = (N_RAW + gt::N_PER_BLOCK - 1) / gt::N_PER_BLOCK;
	unsigned const total = tiles_m * tiles_n;
	unsigned long long a_extent = 0, bq_extent = 0, bkv_extent = 0;
	std::vector<unsigned char> tile_seen((size_t)tiles_m * tiles_n, 0);
	for (unsigned lin = 0; lin < total; ++lin) {
		gt::TileOrigin const o = gt::tile_origin(lin, a_rows, N_RAW, gt::BAND);
		if (o.m % 64 != 0 || o.m + gt::M_PER_BLOCK > a_rows) return fail("tile leaves the token rows", o.m + gt::M_PER_BLOCK, a_rows);
		if (o.n % 128 != 0 || o.n + gt::N_PER_BLOCK > N_RAW) return fail("tile leaves the raw columns", o.n + gt::N_PER_BLOCK, N_RAW);
		// (a moved-back tile keeps its place in the grid of tiles: the last tile row / column)
		unsigned const gm = (o.m + gt::M_PER_BLOCK - 1) / gt::M_PER_BLOCK, gn = (o.n + gt::N_PER_BLOCK - 1) / gt::N_PER_BLOCK;
		if (tile_seen[(size_t)gm * tiles_n + gn]++) return fail("a tile is walked twice", lin, total);
		bool const kv_side = o.n >= Q_COLS;
		if (!kv_side && o.n + gt::N_PER_BLOCK > Q_COLS) return fail("a tile straddles the q and kv weights", o.n + gt::N_PER_BLOCK, Q_COLS);
		unsigned const w_first = kv_side ? o.n - Q_COLS : o.n;
		unsigned const w_rows = kv_side ? N_RAW - Q_COLS : Q_COLS;
		for (unsigned ks = 0; ks < K_STEPS; ++ks) {
			unsigned long long const col_end = (unsigned long long)ks * gt::K_STEP + 16ull * max_chunk + 16;
			if (col_end > K) return fail("request leaves its operand row", col_end, K);
			unsigned long long const a_end = (unsigned long long)(o.m + x_max_row) * K + col_end;
			unsigned long long const w_end = (unsigned long long)(w_first + w_max_row) * K + col_end;
			if (a_end > a_rows_allocated * K) return fail("token request past the end of a", a_end, a_rows_allocated * K);
			if (w_end > (unsigned long long)w_rows * K) return fail("weight request past the end of b", w_end, (unsigned long long)w_rows * K);
			a_extent = a_end > a_extent ? a_end : a_extent;
			(kv_side ? bkv_extent : bq_extent) = w_end > (kv_side ? bkv_extent : bq_extent) ? w_end : (kv_side ? bkv_extent : bq_extent);
		}
	}
	std::printf("{\"ok\": true, \"tiles\": %u, \"requests\": %llu, \"a_extent\": %llu, \"a_bytes\": %llu, \"b_extent\": %llu, \"b_bytes\": %llu, "
	            "\"b_kv_extent\": %llu, \"b_kv_bytes\": %llu}\n",
	            total, per_step * K_STEPS * total, a_extent, a_rows_allocated * K, bq_extent, (unsigned long long)Q_COLS * K,
	            bkv_extent, (unsigned long long)(N_RAW - Q_COLS) * K);
	return 0;
}
