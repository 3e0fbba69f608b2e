// attn_tile.h -- tile geometry of the int8 sliding-window attention kernel as plain constexprs,
// shared by the device code (attn_fwd_i8.hip) and the host program that prints meta.json
// (reference: templates/attn/meta.cu:10-16).  Needs X17_HEAD_DIM from common.h.
#pragma once

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
constexpr unsigned STAGES = 2;

constexpr unsigned K_TILE_BYTES = KV_PER_STEP * HEAD_DIM;        // int8 keys, row = one key
constexpr unsigned V_TILE_BYTES = KV_PER_STEP * HEAD_DIM * 2;    // values widened to bf16
constexpr unsigned STAGE_BYTES = K_TILE_BYTES + V_TILE_BYTES;
constexpr unsigned SMEM_BYTES = STAGES * STAGE_BYTES;

}} // namespace x17::attn_tile
