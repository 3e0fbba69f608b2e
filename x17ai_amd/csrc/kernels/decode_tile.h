// decode_tile.h -- launch geometry of the single-token decode kernel (shared with its meta program).
// Needs X17_HEAD_DIM and X17_CACHE_CAPACITY from common.h.
#pragma once

namespace x17 { namespace decode_tile {

constexpr unsigned HEAD_DIM = X17_HEAD_DIM;
constexpr unsigned CAPACITY = X17_CACHE_CAPACITY;       // cache rows per sequence, multiple of 16
// Two wavefronts per (sequence, head): with at most 20 KB of LDS each, eight workgroups share a compute unit,
// so the 2048 workgroups of 64 sequences x 32 heads are all resident at once and stream their keys together.
constexpr unsigned THREADS_PER_BLOCK = 128;
constexpr unsigned HEADS_PER_BLOCK = 1;
constexpr unsigned MAX_TILES = CAPACITY / 16;           // 16-key tiles
// tiles whose P.V partials are staged at once: one thread per (tile, 16 dims)
constexpr unsigned CHUNK_TILES = THREADS_PER_BLOCK / (HEAD_DIM / 16);
constexpr unsigned PV_WORDS = CHUNK_TILES * HEAD_DIM;   // int32 partials of a chunk (2048 for every head_dim)

// LDS: one 16-byte slot per key quad.  It first holds the quad's four f32 scores; once the probabilities exist
// it holds {partial sum f32, four u8 probabilities, 8 free bytes}.  The P.V partials of a chunk live in the free
// halves of the slots when there are enough of them, otherwise in a region of their own.
constexpr unsigned SLOT_BYTES = CAPACITY * 4;
constexpr bool PV_IN_SLOTS = (CAPACITY / 4) * 2 >= PV_WORDS;
constexpr unsigned PV_OFFSET = SLOT_BYTES;                                   // used when !PV_IN_SLOTS
constexpr unsigned TILE_STATE_OFFSET = SLOT_BYTES + (PV_IN_SLOTS ? 0 : PV_WORDS * 4);
//      | per tile: running max (first the tile max) f32[MAX_TILES], rescale f32[MAX_TILES]
//      | wavefront maxima f32[4] | final partial sums f32[4] | number of listed tiles u32[4] | listed tiles u16[MAX_TILES]
constexpr unsigned SMEM_BYTES = TILE_STATE_OFFSET + 2 * MAX_TILES * 4 + 16 + 16 + 16 + MAX_TILES * 2;

}} // namespace x17::decode_tile
