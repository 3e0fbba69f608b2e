// attn_tile.h -- tile geometry of the int8 sliding-window attention kernel as plain constexprs,
// shared by the device code (attn_fwd_i8.hip) and the host program that prints meta.json
// (reference: templates/attn/meta.cu:10-16).  Needs X17_HEAD_DIM from common.h.
#pragma once

#ifndef X17_ATTN_ROW_SCALES
#define X17_ATTN_ROW_SCALES 0      // 1: q/k/v codes carry one f32 scale per (row, head)
#endif
#ifndef X17_ATTN_OUT_BF16
#define X17_ATTN_OUT_BF16 0        // 1: the output is written as bf16 real values instead of FixedI8 codes
#endif

namespace x17 { namespace attn_tile {

constexpr unsigned HEAD_DIM = X17_HEAD_DIM;
// src/device/cuda/attn.rs:60-66 -- the launcher's grid.y counts groups of this many heads
constexpr unsigned HEADS_PER_KERNEL = (128 / HEAD_DIM) > 1 ? (128 / HEAD_DIM) : 1;

constexpr unsigned WAVE = 64;
constexpr unsigned Q_WAVES = 4;
constexpr unsigned Q_PER_WAVE = 32;
constexpr unsigned Q_PER_BLOCK = Q_WAVES * Q_PER_WAVE;      // 128 queries per workgroup
constexpr unsigned KV_PER_STEP = 32;                         // keys staged per pipeline step
constexpr unsigned THREADS_PER_BLOCK = WAVE * Q_WAVES;
// K/V tiles are fetched PREFETCH steps ahead of their use into rings of PREFETCH + 1 slots
constexpr unsigned PREFETCH = 3;
constexpr unsigned RING = PREFETCH + 1;
// Register budget: this many wavefronts (= workgroups) share a SIMD, so that one workgroup's waits for
// its K/V tiles and its barrier are covered by the others' arithmetic.
#ifndef X17_ATTN_WAVES_PER_SIMD
#define X17_ATTN_WAVES_PER_SIMD (X17_STRICT_MATH ? 2 : 3)   // the deterministic transcendentals need more registers
#endif
constexpr unsigned WAVES_PER_SIMD = X17_ATTN_WAVES_PER_SIMD;

constexpr unsigned K_TILE_BYTES = KV_PER_STEP * HEAD_DIM;        // int8 keys, row = one key
constexpr unsigned RAW_V_TILE_BYTES = KV_PER_STEP * HEAD_DIM;    // int8 values as they arrive
constexpr unsigned V_TILE_BYTES = KV_PER_STEP * HEAD_DIM * 2;    // values widened to f16
// row-scaled operands: per step the 32 keys' scales followed by the 32 value rows' weights (f32)
constexpr bool ROW_SCALES = X17_ATTN_ROW_SCALES != 0;
constexpr unsigned SCALE_TILE_BYTES = 2 * KV_PER_STEP * 4;
// LDS map: K ring | raw V ring | two f16 V tiles (the tile in use and the one being widened) | scale ring
constexpr unsigned K_RING_OFFSET = 0;
constexpr unsigned RAW_V_RING_OFFSET = RING * K_TILE_BYTES;
constexpr unsigned V_TILES_OFFSET = RAW_V_RING_OFFSET + RING * RAW_V_TILE_BYTES;
constexpr unsigned SCALE_RING_OFFSET = V_TILES_OFFSET + 2 * V_TILE_BYTES;
constexpr unsigned SMEM_BYTES = SCALE_RING_OFFSET + (ROW_SCALES ? RING * SCALE_TILE_BYTES : 0);

// ---- index arithmetic of the K/V tile requests (global -> LDS, 16 bytes per lane).  The kernel calls these; so does
// the host-side audit (attn_requests_audit.cpp), which enumerates every request of a launch on the CPU.
constexpr unsigned CHUNKS_PER_ROW = HEAD_DIM / 16;          // 16-byte chunks per key row
// cuda/attn_fwd_i8.cuh:408-412 -- window 0 means "no window"; otherwise rounded up to 16
constexpr unsigned rounded_window(unsigned window_size) {
	return window_size == 0 ? 0xFFFFFFFFu : ((window_size - 1) / 16 + 1) * 16;
}
// Position of a query block's first query.  A last block that would overhang the sequence (lengths are multiples of
// 64, src/device/cuda/attn.rs:398-404) starts earlier and recomputes some of its neighbour's queries.
constexpr unsigned block_first_query(unsigned q_block_index, unsigned seq_len) {
	return q_block_index * Q_PER_BLOCK + Q_PER_BLOCK > seq_len ? seq_len - Q_PER_BLOCK : q_block_index * Q_PER_BLOCK;
}
// Key blocks (KV_PER_STEP keys) a workgroup walks for queries [q0, q0 + Q_PER_BLOCK): [first, end)
constexpr unsigned first_key_block(unsigned q0, unsigned wr) { return (q0 - (q0 < wr ? q0 : wr)) / KV_PER_STEP; }
constexpr unsigned end_key_block(unsigned q_block0) { return q_block0 / KV_PER_STEP + Q_WAVES; }
// Threads that stage tiles: thread t fetches 16-byte chunk t of each 32-key tile
constexpr bool is_stager(unsigned tid) { return tid < KV_PER_STEP * CHUNKS_PER_ROW; }
// Byte offset, from the tile's first key row, of the chunk thread `tid` fetches: the K tile is stored swizzled (stored
// chunk `tid` holds logical chunk n), the V tile in order.
constexpr unsigned stage_k_offset(unsigned tid, unsigned kv_stride) {
	unsigned const line = tid >> 3;
	unsigned const n = (line << 3) | ((tid & 7) ^ ((line >> 1) & 7));
	return (n / CHUNKS_PER_ROW) * kv_stride + (n % CHUNKS_PER_ROW) * 16;
}
constexpr unsigned stage_v_offset(unsigned tid, unsigned kv_stride) {
	return (tid / CHUNKS_PER_ROW) * kv_stride + HEAD_DIM + (tid % CHUNKS_PER_ROW) * 16;
}
// Speed build: step s requests K tile min(s + PREFETCH, last) and raw V tile min(s + PREFETCH + 1, last); its source
// pointer moves on to the next tile exactly when that further tile exists.
constexpr bool further_tile_exists(unsigned s, unsigned n_steps) { return s + PREFETCH + 1 < n_steps; }

}} // namespace x17::attn_tile
