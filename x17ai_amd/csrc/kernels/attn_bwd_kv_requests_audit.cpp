// Host-side audit of the attention backward (dK, dV) kernel's tile requests and LDS addressing.  Compiled with the
// kernel's own common.h and attn_bwd_kv_tile.h -- the index arithmetic below IS the kernel's (attn_d_kv_i8.hip calls
// the same functions) -- it checks, on the CPU,
//   * that each LDS layout's request map is the inverse of the offset function its readers use, that the staging
//     threads' requests fill every 16-byte position of a tile exactly once and stay inside the head's columns, and
//     that every operand read (row reads, transposed reads, constants) stays inside its tile;
//   * for every workgroup of a launch (sequence, head, key block): that its walk over query tiles is not empty, stays
//     inside its own sequence, covers every query that sees one of a wavefront's keys, and that every request of every
//     step stays inside q, d_out and the [H, rows] matrices L and D.
//
//     attn_bwd_kv_requests_audit <seq_len> <batch> <window_size> [rows the operands really have, default seq_len * batch]
//
// No GPU is involved; a kernel whose requests would leave an operand is found here, not on the device.
#include "common.h"
#include "attn_bwd_kv_tile.h"

#include <cstdio>
#include <cstdlib>
#include <vector>

namespace at = x17::attn_tile;
namespace kt = x17::attn_bwd_kv_tile;

static int fail(char const *what, unsigned long long a, unsigned long long b) {
	std::printf("{\"ok\": false, \"error\": \"%s\", \"value\": %llu, \"limit\": %llu}\n", what, a, b);
	return 1;
}

int main(int argc, char **argv) {
	if (argc != 4 && argc != 5) {
		std::fprintf(stderr, "usage: %s <seq_len> <batch> <window_size> [allocated rows]\n", argv[0]);
		return 2;
	}
	unsigned long long const seq_len_arg = std::strtoull(argv[1], nullptr, 10), batch = std::strtoull(argv[2], nullptr, 10);
	unsigned const window_size = (unsigned)std::strtoull(argv[3], nullptr, 10);
	constexpr unsigned HD = X17_HEAD_DIM, H = X17_N_HEADS, Q_STRIDE = X17_Q_STRIDE, O_STRIDE = X17_O_STRIDE;
	constexpr unsigned CPR = kt::CPR, WIDE_CPR = kt::WIDE_CPR, ROWS = kt::Q_PER_STEP;
	if (seq_len_arg % 64 != 0 || seq_len_arg < kt::KEYS_PER_BLOCK || batch == 0 || seq_len_arg * batch > 0xFFFFFFFFull
	    || (window_size != 0 && window_size % 16 != 0)) {
		return fail("the launcher rejects this shape (seq_len % 64, at least one key block, window % 16)", seq_len_arg, kt::KEYS_PER_BLOCK);
	}
	unsigned const seq_len = (unsigned)seq_len_arg;
	unsigned long long const rows = argc == 5 ? std::strtoull(argv[4], nullptr, 10) : seq_len_arg * batch;
	unsigned long long const q_bytes = rows * Q_STRIDE, do_bytes = rows * O_STRIDE * 2ull;
	unsigned const wr = at::rounded_window(window_size);

	// ---- layouts: offset functions are bijections onto the tile, request maps are their inverses
	{
		std::vector<unsigned> seen(ROWS * CPR, 0);
		for (unsigned row = 0; row < ROWS; ++row) for (unsigned c = 0; c < CPR; ++c) {
			unsigned const off = kt::q_raw_offset(row, c);
			if (off % 16 != 0 || off + 16 > kt::Q_RAW_BYTES) return fail("raw Q offset leaves the tile", off + 16, kt::Q_RAW_BYTES);
			++seen[off / 16];
			if (kt::q_raw_source(off / 16, Q_STRIDE) != row * Q_STRIDE + c * 16) return fail("raw Q request map is not the inverse of its layout", off / 16, row * CPR + c);
		}
		for (unsigned v : seen) if (v != 1) return fail("raw Q layout is not a bijection", v, 1);
	}
	{
		std::vector<unsigned> seen_rows(ROWS * WIDE_CPR, 0), seen_tr(ROWS * WIDE_CPR, 0);
		for (unsigned row = 0; row < ROWS; ++row) for (unsigned c = 0; c < WIDE_CPR; ++c) {
			unsigned const off = kt::rows_offset(row, c);
			if (off % 16 != 0 || off + 16 > kt::WIDE_BYTES) return fail("row-layout offset leaves the tile", off + 16, kt::WIDE_BYTES);
			++seen_rows[off / 16];
			if (kt::rows_source(off / 16, O_STRIDE * 2) != row * O_STRIDE * 2 + c * 16) return fail("row-layout request map is not the inverse of its layout", off / 16, row * WIDE_CPR + c);
			unsigned const goff = kt::granule_offset(row, c / 2) + (c % 2) * 16;
			if (goff % 16 != 0 || goff + 16 > kt::WIDE_BYTES) return fail("granule-layout offset leaves the tile", goff + 16, kt::WIDE_BYTES);
			++seen_tr[goff / 16];
			if (kt::granule_source(goff / 16, O_STRIDE * 2) != row * O_STRIDE * 2 + c * 16) return fail("granule-layout request map is not the inverse of its layout", goff / 16, row * WIDE_CPR + c);
		}
		for (unsigned v : seen_rows) if (v != 1) return fail("row layout is not a bijection", v, 1);
		for (unsigned v : seen_tr) if (v != 1) return fail("granule layout is not a bijection", v, 1);
	}
	// ---- the requesting threads: whole wavefronts; their requests fill every position once and stay in the head's columns
	if (kt::Q_STAGERS % at::WAVE != 0 || kt::WIDE_STAGERS % at::WAVE != 0 || kt::WIDE_STAGERS > kt::THREADS_PER_BLOCK) {
		return fail("requesting threads are not whole wavefronts of the workgroup", kt::WIDE_STAGERS, kt::THREADS_PER_BLOCK);
	}
	{
		std::vector<unsigned> q_pos(ROWS * CPR, 0), wide_pos(ROWS * WIDE_CPR, 0), widened(ROWS * CPR * 2, 0);
		for (unsigned tid = 0; tid < kt::THREADS_PER_BLOCK; ++tid) {
			unsigned const wave = tid / at::WAVE, lane = tid % at::WAVE;
			// LDS destination of a request: (region offset) + wave * 1024 + lane * 16 must be position `tid`
			if (wave * 1024 + lane * 16 != tid * 16) return fail("a request's LDS destination is not its position", wave * 1024 + lane * 16, tid * 16);
			if (kt::is_q_stager(tid)) {
				if (tid >= ROWS * CPR) return fail("a Q request's position is behind the tile", tid, ROWS * CPR);
				++q_pos[tid];
				unsigned const qs = kt::q_raw_source(tid, Q_STRIDE);
				if (qs / Q_STRIDE >= ROWS || qs % Q_STRIDE + 16 > HD) return fail("a Q request leaves the tile's rows or the head's columns", qs, ROWS * Q_STRIDE);
			}
			if (kt::is_wide_stager(tid)) {
				if (tid >= ROWS * WIDE_CPR) return fail("a dO request's position is behind the tile", tid, ROWS * WIDE_CPR);
				++wide_pos[tid];
				for (unsigned src : {kt::rows_source(tid, O_STRIDE * 2), kt::granule_source(tid, O_STRIDE * 2)}) {
					if (src / (O_STRIDE * 2) >= ROWS || src % (O_STRIDE * 2) + 16 > HD * 2) return fail("a dO request leaves the tile's rows or the head's columns", src, ROWS * O_STRIDE * 2);
				}
			}
			if (kt::is_widener(tid)) {
				// reads the 8 bytes at tid * 8 of the raw tile (position tid / 2, requested by a thread of another wavefront:
				// the kernel widens only behind a barrier) and writes 16 bytes of the widened tile
				if (tid * 8 + 8 > kt::Q_RAW_BYTES) return fail("a widening read leaves the raw tile", tid * 8 + 8, kt::Q_RAW_BYTES);
				if (!kt::is_q_stager(tid / 2)) return fail("a widening thread reads a position nobody requested", tid / 2, kt::Q_STAGERS);
				unsigned const n = kt::q_raw_logical_chunk(tid / 2);
				unsigned const dst = kt::granule_offset(n / CPR, n % CPR) + 16 * (tid % 2);
				if (dst + 16 > kt::WIDE_BYTES) return fail("a widening write leaves the bf16 tile", dst + 16, kt::WIDE_BYTES);
				++widened[dst / 16];
			}
		}
		for (unsigned v : q_pos) if (v != 1) return fail("a raw Q position is not requested exactly once", v, 1);
		for (unsigned v : wide_pos) if (v != 1) return fail("a dO position is not requested exactly once", v, 1);
		for (unsigned v : widened) if (v != 1) return fail("a 16-byte piece of the widened Q tile is not written exactly once", v, 1);
	}
	// ---- operand reads of a wavefront inside the tile (the lane formulas of attn_d_kv_i8.hip)
	for (unsigned lane = 0; lane < at::WAVE; ++lane) {
		unsigned const group = lane / 16, klane = lane % 16;
		for (unsigned qt = 0; qt < ROWS / 16; ++qt) {
			for (unsigned s = 0; s < (HD + 63) / 64; ++s) {
				unsigned const off = kt::q_raw_offset(16 * qt + klane, 16 * group < HD ? 4 * s + group : 0);
				if (off + 16 > kt::Q_RAW_BYTES) return fail("an S operand read leaves the raw Q tile", off + 16, kt::Q_RAW_BYTES);
			}
			for (unsigned sl = 0; sl < HD / 32; ++sl) {
				unsigned const off = kt::rows_offset(16 * qt + klane, 4 * sl + group);
				if (off + 16 > kt::WIDE_BYTES) return fail("a dP operand read leaves the dO tile", off + 16, kt::WIDE_BYTES);
			}
		}
		for (unsigned dt = 0; dt < HD / 16; ++dt) {
			unsigned const lo = kt::granule_offset(4 * group + (klane >> 2), dt) + 8 * (klane & 3);
			unsigned const hi = lo + 16 * CPR * 32;
			if (lo + 8 > kt::WIDE_BYTES || hi + 8 > kt::WIDE_BYTES) return fail("a transposed read leaves its tile", hi + 8, kt::WIDE_BYTES);
			// the shortcut the kernel takes must name the row the layout function names
			if (hi != kt::granule_offset(16 + 4 * group + (klane >> 2), dt) + 8 * (klane & 3)) return fail("transposed read: 16 rows further is not a constant stride", hi, lo);
		}
		if ((2 * ROWS + 16 + 4 * group) * 4 + 16 > kt::CONST_BYTES_PER_WAVE) {
			return fail("a constant read leaves the wavefront's block", (2 * ROWS + 16 + 4 * group) * 4 + 16, kt::CONST_BYTES_PER_WAVE);
		}
	}
	// the 32 lanes a transposed read serves at a time (eight consecutive rows, one granule column) lie in eight different
	// 32-byte columns of the 256-byte bank window
	for (unsigned dt = 0; dt < HD / 16; ++dt) for (unsigned row0 = 0; row0 < ROWS; row0 += 8) {
		unsigned mask = 0;
		for (unsigned r = 0; r < 8; ++r) mask |= 1u << ((kt::granule_offset(row0 + r, dt) >> 5) & 7);
		if (mask != 0xFF) return fail("transposed reads of eight consecutive rows share a bank column", mask, 0xFF);
	}
	if (at::WAVE * 4 > kt::LD_BYTES_PER_WAVE) return fail("the L / D request is larger than its block", at::WAVE * 4, kt::LD_BYTES_PER_WAVE);
	if (kt::SMEM_BYTES > 160 * 1024) return fail("LDS map larger than a CU's LDS", kt::SMEM_BYTES, 160 * 1024);

	// ---- the walk of every workgroup
	unsigned long long requests = 0, q_extent = 0, do_extent = 0, ld_extent = 0, steps = 0;
	unsigned const key_blocks = (seq_len + kt::KEYS_PER_BLOCK - 1) / kt::KEYS_PER_BLOCK;
	for (unsigned long long seq = 0; seq < batch; ++seq) {
		unsigned long long const row_base = seq * seq_len;
		for (unsigned kb = 0; kb < key_blocks; ++kb) {
			unsigned const k0 = kt::block_first_key(kb, seq_len);
			if (k0 % 64 != 0 || k0 + kt::KEYS_PER_BLOCK > seq_len) return fail("key block leaves its sequence", k0 + kt::KEYS_PER_BLOCK, seq_len);
			unsigned const tile_begin = kt::first_query_tile(k0), tile_end = kt::end_query_tile(k0 + kt::KEYS_PER_BLOCK - 1, wr, seq_len);
			if (tile_end <= tile_begin) return fail("a workgroup walks no tile", tile_end, tile_begin);
			if ((unsigned long long)tile_end * ROWS > seq_len) return fail("the walk reaches behind its sequence", (unsigned long long)tile_end * ROWS, seq_len);
			for (unsigned w = 0; w < kt::KEY_WAVES; ++w) {
				unsigned const kw0 = k0 + w * kt::KEYS_PER_WAVE, kw1 = kw0 + kt::KEYS_PER_WAVE - 1;
				unsigned const first = kt::first_query_tile(kw0), last = kt::end_query_tile(kw1, wr, seq_len) - 1;
				if (first < tile_begin || last >= tile_end) return fail("a wavefront's tiles are outside its workgroup's walk", last, tile_end);
				// every query that sees one of the wavefront's keys: i in (j, min(j + W', seq_len - 1)], checked at the extremes
				unsigned const lowest = kw0 + 1 < seq_len ? kw0 + 1 : seq_len - 1;
				unsigned long long const reach = wr == 0xFFFFFFFFu ? seq_len - 1 : ((unsigned long long)kw1 + wr < seq_len - 1 ? (unsigned long long)kw1 + wr : seq_len - 1);
				if (lowest / ROWS < first) return fail("the first query that sees a key is before the wavefront's first tile", lowest / ROWS, first);
				if (reach / ROWS != last) return fail("the wavefront's last tile is not the tile of the last query that sees its keys", reach / ROWS, last);
			}
			for (unsigned tile = tile_begin; tile < tile_end; ++tile) {
				unsigned long long const first_row = row_base + (unsigned long long)tile * ROWS;
				unsigned long long const q_end = (first_row + ROWS - 1) * Q_STRIDE + (unsigned long long)(H - 1) * HD + HD;
				unsigned long long const do_end = ((first_row + ROWS - 1) * O_STRIDE + (unsigned long long)(H - 1) * HD + HD) * 2;
				if (q_end > q_bytes) return fail("Q request past the end of q", q_end, q_bytes);
				if (do_end > do_bytes) return fail("dO request past the end of d_out", do_end, do_bytes);
				if (first_row + ROWS > rows) return fail("L / D request past the end of a [H, rows] matrix", first_row + ROWS, rows);
				q_extent = q_end > q_extent ? q_end : q_extent;
				do_extent = do_end > do_extent ? do_end : do_extent;
				ld_extent = first_row + ROWS > ld_extent ? first_row + ROWS : ld_extent;
				requests += kt::Q_STAGERS + 2ull * kt::WIDE_STAGERS + kt::THREADS_PER_BLOCK;
				++steps;
			}
		}
	}
	std::printf("{\"ok\": true, \"workgroups\": %llu, \"steps\": %llu, \"requests\": %llu, \"q_extent\": %llu, \"q_bytes\": %llu, "
	            "\"d_out_extent\": %llu, \"d_out_bytes\": %llu, \"ld_extent_rows\": %llu, \"rows\": %llu}\n",
	            batch * key_blocks * (H / at::HEADS_PER_KERNEL), steps * H, requests * H, q_extent, q_bytes, do_extent, do_bytes, ld_extent, rows);
	return 0;
}
