// decode_tile.h -- launch geometry of the single-token decode kernel (shared with its meta program).
// Needs X17_HEAD_DIM and X17_CACHE_CAPACITY from common.h.
#pragma once

namespace x17 { namespace decode_tile {

constexpr unsigned HEAD_DIM = X17_HEAD_DIM;
constexpr unsigned CAPACITY = X17_CACHE_CAPACITY;       // cache rows per sequence, multiple of 16
constexpr unsigned THREADS_PER_BLOCK = 256;
constexpr unsigned HEADS_PER_BLOCK = 1;
constexpr unsigned MAX_TILES = CAPACITY / 16;           // 16-key tiles
constexpr unsigned CHUNK_TILES = 32;                    // tiles whose P.V partials are staged at once

// LDS: scores f32[CAPACITY], later reused for the P.V partials i32[CHUNK_TILES * HEAD_DIM]
//      | probabilities u8[CAPACITY] | quad sums f32[CAPACITY/4]
//      | per tile: max, rescale, running max f32[3 * MAX_TILES] | block maxima f32[256] | final partial sums f32[4]
constexpr unsigned SCORE_PV_BYTES =
	CAPACITY * 4 > CHUNK_TILES * HEAD_DIM * 4 ? CAPACITY * 4 : CHUNK_TILES * HEAD_DIM * 4;
//      | number of listed tiles u32[4] | listed tiles u16[MAX_TILES]
constexpr unsigned SMEM_BYTES = SCORE_PV_BYTES + CAPACITY + CAPACITY + 3 * MAX_TILES * 4 + 256 * 4 + 16 + 16 + MAX_TILES * 2;

}} // namespace x17::decode_tile
