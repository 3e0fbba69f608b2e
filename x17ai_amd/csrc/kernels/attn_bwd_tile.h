// attn_bwd_tile.h -- tile geometry of the attention backward-with-respect-to-q kernel (attn_d_q_i8.hip) as plain
// constexprs, shared with the host program that prints its meta.json.  Needs X17_HEAD_DIM from common.h.
// The query blocking is the forward kernel's (attn_tile.h): 128 queries of one head per workgroup, a wavefront owns
// 32 queries, 32 keys per step.
#pragma once

#include "attn_tile.h"

namespace x17 { namespace attn_bwd_tile {

namespace at = x17::attn_tile;

constexpr unsigned THREADS_PER_BLOCK = at::THREADS_PER_BLOCK;
constexpr unsigned Q_PER_BLOCK = at::Q_PER_BLOCK;
// raw int8 K / V tiles are fetched PREFETCH steps ahead into rings of PREFETCH + 1 slots; one step before its use a
// tile is widened to f16 by the threads that fetched it, into one of two f16 tiles
constexpr unsigned PREFETCH = 2;
constexpr unsigned RING = PREFETCH + 1;
// 64 accumulators of dQ^T, the f16 dO fragments of all of head_dim and the forward's Q fragments stay in registers:
// two wavefronts per SIMD
constexpr unsigned WAVES_PER_SIMD = 2;

constexpr unsigned RAW_TILE_BYTES = at::KV_PER_STEP * at::HEAD_DIM;          // int8, as it arrives
constexpr unsigned F16_TILE_BYTES = at::KV_PER_STEP * at::HEAD_DIM * 2;
// LDS map: raw K ring | raw V ring | two f16 K tiles (granule layout, read transposed) | two f16 V tiles (row layout)
constexpr unsigned RAW_K_RING_OFFSET = 0;
constexpr unsigned RAW_V_RING_OFFSET = RING * RAW_TILE_BYTES;
constexpr unsigned K_F16_OFFSET = RAW_V_RING_OFFSET + RING * RAW_TILE_BYTES;
constexpr unsigned V_F16_OFFSET = K_F16_OFFSET + 2 * F16_TILE_BYTES;
constexpr unsigned SMEM_BYTES = V_F16_OFFSET + 2 * F16_TILE_BYTES;

}} // namespace x17::attn_bwd_tile
