// Host-side audit of the attention kernel's K/V tile requests.  Compiled with the kernel's own common.h and
// attn_tile.h -- the index arithmetic below IS the kernel's (attn_fwd_i8.hip calls the same functions) -- it walks, on
// the CPU, every workgroup of a launch (sequence, head, query block) through the request schedule of its build (the
// speed build asks for a tile in every step, past the end the last one again; the strict build stops asking) and
// checks that every 16-byte request, every 4-byte scale request of the row-scaled build and every query load stays
// inside its operand and inside the workgroup's own sequence, and that the requests of a tile cover its chunks once.
//
//     attn_requests_audit <seq_len> <batch> <window_size> [rows q / kv really have, default seq_len * batch]
//
// No GPU is involved; a kernel whose requests would leave an operand is found here, not on the device.
#include "common.h"
#include "attn_tile.h"

#include <cstdio>
#include <cstdlib>
#include <vector>

namespace at = x17::attn_tile;

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
	constexpr unsigned HD = X17_HEAD_DIM, H = X17_N_HEADS, Q_STRIDE = X17_Q_STRIDE, KV_STRIDE = X17_KV_STRIDE;
	constexpr unsigned CPR = at::CHUNKS_PER_ROW;
	constexpr bool SPEED = X17_STRICT_MATH == 0;
	if (seq_len_arg % 64 != 0 || seq_len_arg < at::Q_PER_BLOCK || batch == 0 || seq_len_arg * batch > 0xFFFFFFFFull
	    || (window_size != 0 && window_size % 16 != 0)) {
		return fail("the launcher rejects this shape (seq_len % 64, at least one query block, window % 16)", seq_len_arg, at::Q_PER_BLOCK);
	}
	unsigned const seq_len = (unsigned)seq_len_arg;
	unsigned long long const rows = argc == 5 ? std::strtoull(argv[4], nullptr, 10) : seq_len_arg * batch;
	unsigned long long const kv_bytes = rows * KV_STRIDE, q_bytes = rows * Q_STRIDE;
	unsigned const wr = at::rounded_window(window_size);

	// the lanes' offsets inside a tile: 32 key rows x CPR chunks, each exactly once, K inside [0, HD), V inside [HD, 2 HD)
	std::vector<unsigned> k_seen(at::KV_PER_STEP * CPR, 0), v_seen(at::KV_PER_STEP * CPR, 0);
	unsigned stagers = 0;
	for (unsigned tid = 0; tid < at::THREADS_PER_BLOCK; ++tid) {
		if (!at::is_stager(tid)) continue;
		++stagers;
		unsigned const ko = at::stage_k_offset(tid, KV_STRIDE), vo = at::stage_v_offset(tid, KV_STRIDE);
		unsigned const kr = ko / KV_STRIDE, kc = ko % KV_STRIDE, vr = vo / KV_STRIDE, vc = vo % KV_STRIDE;
		if (kr >= at::KV_PER_STEP || vr >= at::KV_PER_STEP) return fail("a staging thread's key row is outside the tile", kr > vr ? kr : vr, at::KV_PER_STEP);
		if (kc % 16 != 0 || kc + 16 > HD) return fail("a K chunk leaves the head's K columns", kc + 16, HD);
		if (vc % 16 != 0 || vc < HD || vc + 16 > 2 * HD) return fail("a V chunk leaves the head's V columns", vc + 16, 2 * HD);
		++k_seen[kr * CPR + kc / 16];
		++v_seen[vr * CPR + (vc - HD) / 16];
	}
	if (stagers != at::KV_PER_STEP * CPR) return fail("number of staging threads", stagers, at::KV_PER_STEP * CPR);
	for (unsigned v : k_seen) if (v != 1) return fail("a K-tile chunk is not requested exactly once", v, 1);
	for (unsigned v : v_seen) if (v != 1) return fail("a V-tile chunk is not requested exactly once", v, 1);

	unsigned long long requests = 0, kv_extent = 0, q_extent = 0, scale_extent = 0;
	unsigned const q_blocks = (seq_len + at::Q_PER_BLOCK - 1) / at::Q_PER_BLOCK;
	for (unsigned long long seq = 0; seq < batch; ++seq) {
		unsigned long long const row_base = seq * seq_len;
		for (unsigned qb = 0; qb < q_blocks; ++qb) {
			unsigned const q0 = at::block_first_query(qb, seq_len);
			if (q0 % 64 != 0 || q0 + at::Q_PER_BLOCK > seq_len) return fail("query block leaves its sequence", q0 + at::Q_PER_BLOCK, seq_len);
			unsigned const kb_begin = at::first_key_block(q0, wr), kb_end = at::end_key_block(q0);
			if (kb_end <= kb_begin || kb_end - kb_begin < at::RING) return fail("a workgroup walks fewer tiles than its ring holds", kb_end - kb_begin, at::RING);
			unsigned const n_steps = kb_end - kb_begin, last = n_steps - 1;
			// one requested tile: all of its key rows must be rows of THIS sequence
			auto tile = [&](unsigned t) -> int {
				if (t > last) return fail("request for a tile behind the walk's last", t, last);
				unsigned long long const first_key = (unsigned long long)(kb_begin + t) * at::KV_PER_STEP;
				if (first_key + at::KV_PER_STEP > seq_len) return fail("tile reaches behind its sequence", first_key + at::KV_PER_STEP, seq_len);
				for (unsigned head = 0; head < H; head += H - 1 ? H - 1 : 1) {       // first and last head bound the columns
					unsigned long long const end = (row_base + first_key + at::KV_PER_STEP - 1) * KV_STRIDE + (unsigned long long)head * 2 * HD + 2 * HD;
					if (end > kv_bytes) return fail("K/V request past the end of kv", end, kv_bytes);
					kv_extent = end > kv_extent ? end : kv_extent;
				}
				unsigned long long const sc_end = row_base + first_key + at::KV_PER_STEP;         // (scale matrices: [H, rows])
				scale_extent = sc_end > scale_extent ? sc_end : scale_extent;
				requests += 2ull * stagers;
				return 0;
			};
			if (SPEED) {
				// prologue: raw V tile 0, then K tiles 0..2 with V tiles 1..3; the source then stands at tile 3
				for (unsigned j = 0; j <= at::PREFETCH; ++j) if (int rc = tile(j)) return rc;
				unsigned src_tile = at::PREFETCH;
				for (unsigned s = 0; s < n_steps; ++s) {
					bool const more = at::further_tile_exists(s, n_steps);
					if (int rc = tile(src_tile)) return rc;                         // K (and the scales of the row-scaled build)
					if (int rc = tile(src_tile + (more ? 1 : 0))) return rc;        // raw V, one tile further while there is one
					src_tile += more ? 1 : 0;
				}
				if (src_tile != last) return fail("the source pointer does not end on the last tile", src_tile, last);
			} else {
				for (unsigned j = 0; j < at::PREFETCH && j < n_steps; ++j) if (int rc = tile(j)) return rc;
				for (unsigned i = 0; i + at::PREFETCH < n_steps; ++i) if (int rc = tile(i + at::PREFETCH)) return rc;
			}
			// the block's query rows (16-byte loads, 32 bytes of head_dim per lane and slice)
			unsigned long long const q_end = (row_base + q0 + at::Q_PER_BLOCK - 1) * Q_STRIDE + (unsigned long long)(H - 1) * HD + HD;
			if (q_end > q_bytes) return fail("query load past the end of q", q_end, q_bytes);
			q_extent = q_end > q_extent ? q_end : q_extent;
		}
	}
	if (scale_extent > rows) return fail("scale request past the end of a [H, rows] scale matrix", scale_extent, rows);
	std::printf("{\"ok\": true, \"workgroups\": %llu, \"requests\": %llu, \"kv_extent\": %llu, \"kv_bytes\": %llu, \"q_extent\": %llu, "
	            "\"q_bytes\": %llu, \"scale_extent_rows\": %llu, \"rows\": %llu}\n",
	            batch * q_blocks * (H / at::HEADS_PER_KERNEL), requests * H, kv_extent, kv_bytes, q_extent, q_bytes, scale_extent, rows);
	return 0;
}
