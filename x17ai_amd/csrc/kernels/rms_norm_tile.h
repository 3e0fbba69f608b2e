// rms_norm_tile.h -- launch geometry of the rms_norm kernel (shared with its meta program).
#pragma once

namespace x17 { namespace rms_norm_tile {

constexpr unsigned LANES_PER_ROW = 32;          // the reference's summation order is defined over 32 lanes
constexpr unsigned ROWS_PER_BLOCK = 8;
constexpr unsigned THREADS_PER_BLOCK = LANES_PER_ROW * ROWS_PER_BLOCK;
constexpr unsigned VALUES_PER_LANE = 16;        // rms_norm.cu:12
constexpr unsigned VALUES_PER_STEP = LANES_PER_ROW * VALUES_PER_LANE;   // 512
constexpr unsigned SMEM_BYTES = 0;

}} // namespace x17::rms_norm_tile
