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

}} // namespace x17::attn_tile
