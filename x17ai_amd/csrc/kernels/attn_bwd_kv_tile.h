// attn_bwd_kv_tile.h -- tile geometry and index arithmetic of the attention backward-with-respect-to-k-and-v kernel
// (attn_d_kv_i8.hip) as plain constexprs, shared by the device code, the host program that prints its meta.json and the
// host-side audit of its tile requests (attn_bwd_kv_requests_audit.cpp).  Needs X17_HEAD_DIM from common.h.
// Structure of the reference's attn_d_kv.cuh:26-37: a workgroup owns a block of keys and walks the queries that see it.
#pragma once

#include "attn_tile.h"

namespace x17 { namespace attn_bwd_kv_tile {

namespace at = x17::attn_tile;

constexpr unsigned HEAD_DIM = at::HEAD_DIM;
constexpr unsigned KEY_WAVES = 8;
constexpr unsigned KEYS_PER_WAVE = 16;
constexpr unsigned KEYS_PER_BLOCK = KEY_WAVES * KEYS_PER_WAVE;        // 128 keys of one head per workgroup
constexpr unsigned Q_PER_STEP = 32;                                    // queries staged per pipeline step
constexpr unsigned THREADS_PER_BLOCK = at::WAVE * KEY_WAVES;
static_assert(KEYS_PER_BLOCK == at::Q_PER_BLOCK, "the launcher's grid and its smallest sequence are the forward's");
// tiles are requested PREFETCH steps ahead into rings of PREFETCH + 1 slots; one step before its use the int8 Q tile
// is widened to bf16
constexpr unsigned PREFETCH = 2;
constexpr unsigned RING = PREFETCH + 1;
// 16 keys per wavefront on the 16 x 16 matrix instructions: 64 accumulators (dK^T and dV^T of 16 keys x head_dim 128)
// and the keys' own K and V fragments leave room for two wavefronts per SIMD, which a lone wavefront's issue rate needs
constexpr unsigned WAVES_PER_SIMD = 2;

constexpr unsigned CPR = at::CHUNKS_PER_ROW;                // 16-byte chunks of an int8 row of the head
constexpr unsigned WIDE_CPR = 2 * CPR;                      // ... of a bf16 row
constexpr unsigned Q_STAGERS = Q_PER_STEP * CPR;            // threads that request the raw Q tile: 16-byte chunk t each
constexpr unsigned WIDE_STAGERS = Q_PER_STEP * WIDE_CPR;    // threads that request the dO tile: chunk t of each of its two layouts
static_assert(WIDE_STAGERS <= THREADS_PER_BLOCK && Q_STAGERS % at::WAVE == 0, "whole wavefronts request, one chunk per lane");
constexpr unsigned Q_RAW_BYTES = Q_PER_STEP * HEAD_DIM;     // int8 queries as they arrive
constexpr unsigned WIDE_BYTES = Q_PER_STEP * HEAD_DIM * 2;  // a bf16 tile (dO as it arrives, Q widened)
constexpr unsigned LD_BYTES_PER_WAVE = 2 * Q_PER_STEP * 4;  // the tile's L and D values (f32), one copy per wavefront
// one ring slot: raw Q | dO laid out for row reads | dO laid out for transposed reads | L and D (per wavefront)
constexpr unsigned Q_RAW_OFFSET = 0;
constexpr unsigned DO_ROWS_OFFSET = Q_RAW_OFFSET + Q_RAW_BYTES;
constexpr unsigned DO_TR_OFFSET = DO_ROWS_OFFSET + WIDE_BYTES;
constexpr unsigned LD_OFFSET = DO_TR_OFFSET + WIDE_BYTES;
constexpr unsigned SLOT_BYTES = LD_OFFSET + KEY_WAVES * LD_BYTES_PER_WAVE;
// behind the ring, with the slot numbering of the ring (so that one compile-time slot number addresses a step's
// operands everywhere): the bf16 Q tiles and, per wavefront, the per-query constants temperature | L - lg2(255) | D
constexpr unsigned Q_WIDE_OFFSET = RING * SLOT_BYTES;
constexpr unsigned CONST_BYTES_PER_WAVE = 3 * Q_PER_STEP * 4;
constexpr unsigned CONST_OFFSET = Q_WIDE_OFFSET + RING * WIDE_BYTES;
constexpr unsigned SMEM_BYTES = CONST_OFFSET + RING * KEY_WAVES * CONST_BYTES_PER_WAVE;

// ---- the walk.  Key blocks are placed like the forward's query blocks (a last block that would overhang starts
// earlier and recomputes some of its neighbour's keys, storing the same values).
constexpr unsigned block_first_key(unsigned key_block_index, unsigned seq_len) { return at::block_first_query(key_block_index, seq_len); }
// last query that sees a key of [.., last_key]: query i sees key j iff j < i <= j + W' (wr: the rounded window, 2^32 - 1 = none)
constexpr unsigned last_seeing_query(unsigned last_key, unsigned wr, unsigned seq_len) {
	return wr >= seq_len || wr >= seq_len - 1 - last_key ? seq_len - 1 : last_key + wr;
}
// query tiles (Q_PER_STEP queries) walked for the keys [first_key, last_key]: [first, end)
constexpr unsigned first_query_tile(unsigned first_key) { return first_key / Q_PER_STEP; }
constexpr unsigned end_query_tile(unsigned last_key, unsigned wr, unsigned seq_len) { return last_seeing_query(last_key, wr, seq_len) / Q_PER_STEP + 1; }

// ---- LDS layouts (byte offsets inside a tile) and the requests that fill them.  A request moves 16 bytes per lane to
// consecutive LDS addresses, so a layout is made by choosing which chunk of the source a lane asks for: position p
// (in 16-byte units) of a tile receives the source chunk the *_source function names.
constexpr bool is_q_stager(unsigned tid) { return tid < Q_STAGERS; }
constexpr bool is_wide_stager(unsigned tid) { return tid < WIDE_STAGERS; }
// raw int8 Q tile: the forward's K tile layout (linear chunk n = row * CPR + c in 128-byte line n / 8 at position
// (n % 8) ^ ((line >> 1) & 7)): one request per staging thread
constexpr unsigned q_raw_offset(unsigned row, unsigned c) {
	unsigned const n = row * CPR + c, line = n >> 3;
	return (line << 7) | (((n & 7) ^ ((line >> 1) & 7)) << 4);
}
constexpr unsigned q_raw_logical_chunk(unsigned p) {
	unsigned const line = p >> 3;
	return (line << 3) | ((p & 7) ^ ((line >> 1) & 7));
}
constexpr unsigned q_raw_source(unsigned p, unsigned row_stride_bytes) {
	unsigned const n = q_raw_logical_chunk(p);
	return (n / CPR) * row_stride_bytes + (n % CPR) * 16;
}
// bf16 tile read by rows (eight dims of one query per lane): a row is WIDE_CPR chunks of 16 bytes; 16 / WIDE_CPR rows
// share a 256-byte line and chunk c of a row sits at position c ^ line inside its row's part of the line
constexpr unsigned rows_offset(unsigned row, unsigned c) {
	constexpr unsigned RPL = 16 / WIDE_CPR;
	unsigned const line = row / RPL;
	return line * 256 + ((row % RPL) * WIDE_CPR + (c ^ (line & (WIDE_CPR - 1)))) * 16;
}
constexpr unsigned rows_source(unsigned p, unsigned row_stride_bytes) {
	constexpr unsigned RPL = 16 / WIDE_CPR;
	unsigned const line = p / 16, slot = p % 16;
	return (line * RPL + slot / WIDE_CPR) * row_stride_bytes + ((slot % WIDE_CPR) ^ (line & (WIDE_CPR - 1))) * 16;
}
// bf16 tile read transposed (eight queries of one dim per lane): 32-byte granule n = row * CPR + g (16 dims) in
// 256-byte line n / 8 at position (n % 8) ^ (line % CPR): the 32 lanes a ds_read_b64_tr_b16 serves at a time ask for
// granule g of eight consecutive rows, which then lie in eight different 32-byte columns
constexpr unsigned granule_offset(unsigned row, unsigned g) {
	unsigned const n = row * CPR + g, line = n >> 3;
	return (line << 8) | (((n & 7) ^ (line & (CPR - 1))) << 5);
}
constexpr unsigned granule_source(unsigned p, unsigned row_stride_bytes) {
	unsigned const gp = p / 2, line = gp / 8;
	unsigned const n = line * 8 + ((gp % 8) ^ (line & (CPR - 1)));
	return (n / CPR) * row_stride_bytes + (2 * (n % CPR) + p % 2) * 16;
}
// Q tile int8 -> bf16: thread t < 2 * Q_STAGERS widens half a chunk (eight codes) of raw position t / 2
constexpr bool is_widener(unsigned tid) { return tid < 2 * Q_STAGERS; }

}} // namespace x17::attn_bwd_kv_tile
