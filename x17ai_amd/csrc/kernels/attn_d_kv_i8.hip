// attn_d_kv_i8.hip -- backward of the int8 sliding-window attention with respect to k and v, for gfx950.
//
// The reference's backward kernels (attn_d_kv.cuh:1-431) belong to its bf16 generation; its int8 / e4m3 generation has
// no backward yet.  This kernel keeps the structure of attn_d_kv.cuh:200-400 -- a workgroup owns a block of keys and
// walks the query tiles that see it; per tile S = Q . K^T, P from the forward's log-sum-exp L, dP = dO . V^T,
// dV += P^T . dO, dS = P * (dP - D) with D from the dQ pass, dK += dS^T . Q; P and dS are rounded to bf16 for their
// products as the reference does -- on the forward semantics of attn_fwd_i8.hip (cuda/attn_fwd_i8.cuh:368-619): FixedI8
// q / k / v codes (real = code / 8), scores in base 2 with the scalable-softmax temperature, causal sliding window.
// Per head, key j and the queries i that see it (j < i <= j + W'), t_i = hd^-1/2 * lg2(min(W', i) + 4) * head_temp[h]:
//   P_ij  = 2^(t_i (q_i . k_j) - (L_i - lg2 255))
//   dv_j  = sum_i P_ij dO_i
//   dS_ij = ln 2 * P_ij * (dO_i . v_j - D_i)
//   dk_j  = sum_i t_i dS_ij q_i                        (gradients with respect to the REAL k and v; bf16)
// Like attn_d_kv.cuh, no gradient is formed for the sink or the temperatures; the sink enters through L and D only.
//
// Design, MI355X-first:
//   * One workgroup = 8 wavefronts = 128 keys of one head; a wavefront owns 16 keys and works on the 16 x 16 matrix
//     instructions: its int8 K fragments, its V fragments widened to bf16 and the 2 x 32 accumulators of dK^T and dV^T
//     (dims x keys) stay in registers and leave room for two wavefronts per SIMD -- with a lone wavefront per SIMD
//     (32 keys, 32 x 32 instructions, 380 registers) no unit was busy more than a third of the time.
//   * Orientation: S and dP are (queries x keys), so a lane owns ONE key and 8 queries of the 32-query tile.  Their
//     MFMA results are then, packed to bf16, directly the "B" operand (contraction over the tile's 32 queries) of
//     dV^T += dO^T . P and dK^T += Q^T . dS; no lane exchange, no LDS round trip.
//   * S runs on v_mfma_i32_16x16x64_i8 from the raw int8 Q tile; dP, dV^T, dK^T on v_mfma_f32_16x16x32_bf16 (dO is bf16
//     in memory and is used as it is; int8 codes are exact in bf16): 28 matrix instructions per step for head_dim 128.
//   * Tiles of 32 queries arrive global -> LDS directly, two steps ahead: the raw Q rows, the dO rows twice -- once
//     laid out for row reads ("A" of dP: eight dims of one query) and once for ds_read_b64_tr_b16 ("A" of dV^T: eight
//     queries of one dim); a layout is chosen by which source chunk a lane requests, so neither copy costs an
//     LDS -> LDS pass -- and the tile's L and D values.  One step ahead the workgroup widens the Q tile to bf16 into
//     the transposed-read layout ("A" of dK^T) and every wavefront writes the tile's per-query constants
//     (temperature, L - lg2 255, D) for itself.
//
// common.h (generated per kernel) provides X17_N_HEADS, X17_HEAD_DIM, X17_Q_STRIDE, X17_KV_STRIDE, X17_O_STRIDE,
// X17_STRICT_MATH.  gridDim = (key blocks, head groups, sequences).

#include "common.h"
#include "x17_device.h"
#include "attn_bwd_kv_tile.h"

using namespace x17;
namespace at = x17::attn_tile;
namespace kt = x17::attn_bwd_kv_tile;

namespace {

constexpr u32 HD = X17_HEAD_DIM;
constexpr u32 N_HEADS = X17_N_HEADS;
constexpr u32 Q_STRIDE = X17_Q_STRIDE;
constexpr u32 KV_STRIDE = X17_KV_STRIDE;
constexpr u32 O_STRIDE = X17_O_STRIDE;
constexpr u32 HPK = at::HEADS_PER_KERNEL;
constexpr u32 K_SLICES = (HD + 63) / 64;   // 64 bytes of head_dim per QK MFMA (head_dim 32: the upper half is zero)
constexpr u32 D_SLICES = HD / 32;          // 32 dims per dP MFMA
constexpr u32 D_TILES = HD / 16;           // 16 output dims per dK^T / dV^T MFMA
constexpr u32 Q_TILES = kt::Q_PER_STEP / 16;   // S and dP: two 16-query tiles per step
constexpr u32 CPR = kt::CPR;

static_assert(HD == 32 || HD == 64 || HD == 128, "head_dim must be 32, 64 or 128");
static_assert(N_HEADS % HPK == 0, "n_heads must be divisible by heads_per_kernel");
static_assert(kt::PREFETCH == 2 && kt::RING == 3, "the pipeline below is written for a prefetch distance of 2");

constexpr f32 LOG2_PROB_SCALE = 7.9943534368588578f;                       // lg2(255): the forward's L carries it
constexpr f32 BASE_TEMPERATURE = f32(constexpr_inv_sqrt(f64(HD)) / 64.0);  // for dots of codes (8 q . 8 k)
// dk = t_real * ln 2 * sum_i w_i q_i with t_real = 64 * temperature (the temperature below is for dots of codes)
// and q = code / 8: 64 * ln 2 / 8
constexpr f32 EIGHT_LN2 = 5.5451774444795625f;

typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

// two int8 codes (bytes b and b + 1 of `biased` = word ^ 0x80808080) as two bf16, exact: byte -> f32, minus 128, the
// upper halves of the two floats
X17_DEV u32 bf16_pair(u32 biased, int b) {
	f32 const lo = f32((biased >> (8 * b)) & 0xFFu) - 128.0f;
	f32 const hi = f32((biased >> (8 * b + 8)) & 0xFFu) - 128.0f;
	return (f2u(lo) >> 16) | (f2u(hi) & 0xFFFF0000u);
}

X17_DEV v8bf transposed_fragment(u8 const *p0, u8 const *p1) {
	v4s const lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p0);
	v4s const hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p1);
	v8s const both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
	return __builtin_bit_cast(v8bf, both);
}

} // namespace

extern "C" __global__ __launch_bounds__(kt::THREADS_PER_BLOCK)
__attribute__((amdgpu_waves_per_eu(kt::WAVES_PER_SIMD, kt::WAVES_PER_SIMD)))
void kernel(
	u32 seq_len,
	i8 const *q,
	i8 const *kv,
	f32 const *attn_temperature,
	u16 const *d_out,            // bf16 [rows, O_STRIDE]: gradient with respect to the real output
	f32 const *l,                // the forward's log-sum-exp [H, rows]
	f32 const *d_rows,           // D [H, rows] of the dQ pass
	u16 *d_kv,                   // bf16 [rows, KV_STRIDE]: per head dK then dV, the layout of kv
	u32 window_size
) {
	extern __shared__ __attribute__((aligned(1024))) u8 smem[];

	u32 const tid = threadIdx.x;
	u32 const lane = tid % 64;
	u32 const wave = __builtin_amdgcn_readfirstlane(tid / 64);
	u32 const group = lane / 16;          // the lane's k-group in the operands, its row group in the results
	u32 const klane = lane % 16;          // its key in S, dP and the accumulators; its row or dim in the "A" operands

	u32 const pairs = gridDim.y * gridDim.z;
	u32 const lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
	u32 const pair = lin % pairs;
	u32 const key_block_index = lin / pairs;
	u32 const head_group = pair % gridDim.y;
	u32 const seq = pair / gridDim.y;
	size_t const row_base = (size_t)seq * seq_len;
	size_t const all_rows = (size_t)gridDim.z * seq_len;
	u32 const key_block0 = kt::block_first_key(key_block_index, seq_len);
	u32 const key_wave0 = key_block0 + wave * kt::KEYS_PER_WAVE;
	u32 const key = key_wave0 + klane;
	u32 const wr = at::rounded_window(window_size);
	u32 const vis_bound = wr - 1 < 0x7FFFFFFFu ? wr - 1 : 0x7FFFFFFFu;
	u32 const tile_begin = kt::first_query_tile(key_block0);
	u32 const tile_end = kt::end_query_tile(key_block0 + kt::KEYS_PER_BLOCK - 1, wr, seq_len);
	u32 const wave_tile_first = kt::first_query_tile(key_wave0);
	u32 const wave_tile_last = kt::end_query_tile(key_wave0 + kt::KEYS_PER_WAVE - 1, wr, seq_len) - 1;
	u32 const n_steps = tile_end - tile_begin;

	// ---- lane constants of the requests and of the operand reads
	bool const q_stager = kt::is_q_stager(tid), wide_stager = kt::is_wide_stager(tid), widener = kt::is_widener(tid);
	u32 const q_src = kt::q_raw_source(tid, Q_STRIDE);
	u32 const rows_src = kt::rows_source(tid, O_STRIDE * 2);
	u32 const tr_src = kt::granule_source(tid, O_STRIDE * 2);
	// stored chunk tid / 2 of the raw Q tile holds logical chunk n: query n / CPR, dims 16 * (n % CPR) .. + 15; this
	// thread widens its half tid % 2
	u32 const q_logical = kt::q_raw_logical_chunk(tid / 2);
	u32 const q_wide_dst = kt::granule_offset(q_logical / CPR, q_logical % CPR) + 16 * (tid % 2);
	// "A" of S: query 16 qt + klane, the 16 bytes 64 s + 16 group of its row (none for head_dim 32's upper half)
	bool const k_group_in_row = 16 * group < HD;
	u32 q_read_off[Q_TILES][K_SLICES];
	// "A" of dP: query 16 qt + klane, dims 32 sl + 8 group + 0..7
	u32 do_read_off[Q_TILES][D_SLICES];
	X17_UNROLL for (u32 qt = 0; qt < Q_TILES; ++qt) {
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) q_read_off[qt][s] = kt::q_raw_offset(16 * qt + klane, k_group_in_row ? 4 * s + group : 0);
		X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) do_read_off[qt][sl] = kt::rows_offset(16 * qt + klane, 4 * sl + group);
	}
	// transposed reads ("A" of dV^T and dK^T: dim 16 dt + klane, the 8 queries 4 group + 0..3 and 16 + 4 group + 0..3):
	// lane t of sixteen asks for eight bytes of query 4 group + t / 4; sixteen queries further is a constant stride
	u32 tr_lane_off[D_TILES];
	X17_UNROLL for (u32 dt = 0; dt < D_TILES; ++dt) {
		tr_lane_off[dt] = kt::granule_offset(4 * group + (klane >> 2), dt) + 8 * (klane & 3);
	}
	constexpr u32 TR_SIXTEEN_ROWS = 16 * CPR * 32;

	for (u32 hh = 0; hh < HPK; ++hh) {
		u32 const head = head_group * HPK + hh;
		i8 const *q_head = q + row_base * Q_STRIDE + (size_t)head * HD;
		i8 const *kv_head = kv + row_base * KV_STRIDE + (size_t)head * 2 * HD;
		u8 const *do_head = reinterpret_cast<u8 const *>(d_out) + (row_base * O_STRIDE + (size_t)head * HD) * 2;
		f32 const *l_head = l + (size_t)head * all_rows + row_base;
		f32 const *d_head = d_rows + (size_t)head * all_rows + row_base;
		f32 const head_temperature = attn_temperature[head];

		auto issue_loads = [&](u32 tile, u32 slot) {
			u8 *base = smem + slot * kt::SLOT_BYTES;
			if (q_stager) {
				i8 const *q_tile = q_head + (size_t)(tile * kt::Q_PER_STEP) * Q_STRIDE;
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(q_tile + q_src), X17_LDS_PTR(base + kt::Q_RAW_OFFSET + wave * 1024), 16, 0, 0);
			}
			if (wide_stager) {
				u8 const *do_tile = do_head + (size_t)(tile * kt::Q_PER_STEP) * (O_STRIDE * 2);
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(do_tile + rows_src), X17_LDS_PTR(base + kt::DO_ROWS_OFFSET + wave * 1024), 16, 0, 0);
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(do_tile + tr_src), X17_LDS_PTR(base + kt::DO_TR_OFFSET + wave * 1024), 16, 0, 0);
			}
			// every wavefront for itself: lanes 0..31 the tile's L, lanes 32..63 its D
			f32 const *ld_src = (lane < 32 ? l_head : d_head) + tile * kt::Q_PER_STEP + lane % 32;
			__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(ld_src), X17_LDS_PTR(base + kt::LD_OFFSET + wave * kt::LD_BYTES_PER_WAVE), 4, 0, 0);
		};
		// Q tile int8 -> bf16, half a chunk per thread -- a chunk some other wavefront requested: only called behind a
		// barrier that every thread passed after waiting for its own requests -- and this wavefront's per-query constants
		auto prepare = [&](u32 tile, u32 slot) {
			u8 const *base = smem + slot * kt::SLOT_BYTES;
			if (widener) {
				v2u const raw = *reinterpret_cast<v2u const *>(base + kt::Q_RAW_OFFSET + tid * 8);
				u32 const b0 = raw[0] ^ 0x80808080u, b1 = raw[1] ^ 0x80808080u;
				*reinterpret_cast<v4u *>(smem + kt::Q_WIDE_OFFSET + slot * kt::WIDE_BYTES + q_wide_dst) =
					v4u{bf16_pair(b0, 0), bf16_pair(b0, 2), bf16_pair(b1, 0), bf16_pair(b1, 2)};
			}
			f32 const landed = *reinterpret_cast<f32 const *>(base + kt::LD_OFFSET + wave * kt::LD_BYTES_PER_WAVE + lane * 4);
			f32 *cst = reinterpret_cast<f32 *>(smem + kt::CONST_OFFSET + (slot * kt::KEY_WAVES + wave) * kt::CONST_BYTES_PER_WAVE);
			cst[kt::Q_PER_STEP + lane] = lane < 32 ? landed - LOG2_PROB_SCALE : landed;       // L - lg2 255 | D
			if (lane < 32) {
				u32 const qi = tile * kt::Q_PER_STEP + lane;
				u32 const visible = qi < wr ? qi : wr;
				cst[lane] = (BASE_TEMPERATURE * sfu::lg2(f32(visible + 4u))) * head_temperature;
			}
		};

		// ---- the wavefront's own operands
		v4i kf[K_SLICES];                    // "B" of S: lane = key, the 16 bytes 64 s + 16 group of its row
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
			kf[s] = v4i{0, 0, 0, 0};
			if (k_group_in_row) kf[s] = *reinterpret_cast<v4i const *>(kv_head + (size_t)key * KV_STRIDE + 64 * s + 16 * group);
		}
		v8bf vfrag[D_SLICES];                // "B" of dP: lane = key, dims 32 sl + 8 group + 0..7 as bf16
		X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) {
			v2u const raw = *reinterpret_cast<v2u const *>(kv_head + (size_t)key * KV_STRIDE + HD + 32 * sl + 8 * group);
			u32 const b0 = raw[0] ^ 0x80808080u, b1 = raw[1] ^ 0x80808080u;
			v4u const words = {bf16_pair(b0, 0), bf16_pair(b0, 2), bf16_pair(b1, 0), bf16_pair(b1, 2)};
			vfrag[sl] = __builtin_bit_cast(v8bf, words);
		}
		v4f dk_acc[D_TILES], dv_acc[D_TILES];    // (dims x keys): lane = key, register r = dim 16 dt + 4 group + r
		X17_UNROLL for (u32 dt = 0; dt < D_TILES; ++dt) {
			dk_acc[dt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
			dv_acc[dt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
		}

		// ---- pipeline prologue
		__syncthreads();                      // the previous head's tiles are no longer read
		X17_UNROLL for (u32 j = 0; j < kt::PREFETCH; ++j) {
			if (j < n_steps) issue_loads(tile_begin + j, j);
		}
		__builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
		__builtin_amdgcn_s_barrier();         // everybody's requests for tile 0 have landed
		prepare(tile_begin, 0);

		// one pipeline step, common to all wavefronts of the workgroup
		auto advance = [&](u32 i, u32 slot) {
			u32 const tile = tile_begin + i;
			// this thread's requests for tile i + 1 have landed; its LDS traffic of step i - 1 is complete; after the
			// barrier so is everybody else's: tile i is visible, the slot of tile i - 1 (= of tile i + 2) is free
			__builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
			__builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
			__builtin_amdgcn_s_barrier();
			if (i + kt::PREFETCH < n_steps) {
				issue_loads(tile + kt::PREFETCH, (slot + kt::PREFETCH) % kt::RING);
			}
			if (i + 1 < n_steps) {
				prepare(tile + 1, (slot + 1) % kt::RING);
			}
		};
		// the step's arithmetic for this wavefront's 16 keys
		auto compute = [&](u32 i, u32 slot) {
			u32 const tile = tile_begin + i;
			u8 const *base = smem + slot * kt::SLOT_BYTES;
			u8 const *q_wide = smem + kt::Q_WIDE_OFFSET + slot * kt::WIDE_BYTES;
			f32 const *cst = reinterpret_cast<f32 const *>(smem + kt::CONST_OFFSET + (slot * kt::KEY_WAVES + wave) * kt::CONST_BYTES_PER_WAVE);
			u32 const q0 = tile * kt::Q_PER_STEP;
			bool const need_mask = !(key_wave0 + kt::KEYS_PER_WAVE - 1 < q0 && (q0 + kt::Q_PER_STEP - 1 - key_wave0) <= wr);
			u32 pw[2 * Q_TILES], ww[2 * Q_TILES];     // P and the dK weights as bf16 pairs: "B" operands, slots = this lane's 8 queries
			X17_UNROLL for (u32 qt = 0; qt < Q_TILES; ++qt) {
				// S and dP (times 8: v codes) blocks: rows = 16 queries of the tile, columns = this wave's 16 keys
				v4i s_acc = {0, 0, 0, 0};
				X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
					v4i qa = *reinterpret_cast<v4i const *>(base + kt::Q_RAW_OFFSET + q_read_off[qt][s]);
					if (!k_group_in_row) qa = v4i{0, 0, 0, 0};
					s_acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qa, kf[s], s_acc, 0, 0, 0);
				}
				v4f dp_acc = {0.0f, 0.0f, 0.0f, 0.0f};
				X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) {
					v8bf const da = *reinterpret_cast<v8bf const *>(base + kt::DO_ROWS_OFFSET + do_read_off[qt][sl]);
					dp_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(da, vfrag[sl], dp_acc, 0, 0, 0);
				}
				// register r belongs to query q0 + 16 qt + 4 group + r; key j is visible to query i iff the distance
				// i - 1 - j, as an unsigned number, is at most W' - 1
				u32 const first = q0 + 16 * qt + 4 * group - 1 - key;
				v4f const ct = *reinterpret_cast<v4f const *>(cst + 16 * qt + 4 * group);
				v4f const cl = *reinterpret_cast<v4f const *>(cst + kt::Q_PER_STEP + 16 * qt + 4 * group);
				v4f const cd = *reinterpret_cast<v4f const *>(cst + 2 * kt::Q_PER_STEP + 16 * qt + 4 * group);
				f32 p[4], w[4];
				X17_UNROLL for (u32 r = 0; r < 4; ++r) {
					f32 pe = sfu::ex2(fmaf32(f32(s_acc[r]), ct[r], -cl[r]));
					if (need_mask) {
						pe = first + r <= vis_bound ? pe : 0.0f;
					}
					p[r] = pe;
					w[r] = (pe * fmaf32(dp_acc[r], 0.125f, -cd[r])) * ct[r];
				}
				pw[2 * qt] = pack2_bf16_rne(p[0], p[1]);
				pw[2 * qt + 1] = pack2_bf16_rne(p[2], p[3]);
				ww[2 * qt] = pack2_bf16_rne(w[0], w[1]);
				ww[2 * qt + 1] = pack2_bf16_rne(w[2], w[3]);
			}
			static_assert(Q_TILES == 2, "one 16 x 16 x 32 instruction contracts over the step's 32 queries");
			v8bf const pfrag = __builtin_bit_cast(v8bf, (v4u{pw[0], pw[1], pw[2], pw[3]}));
			v8bf const wfrag = __builtin_bit_cast(v8bf, (v4u{ww[0], ww[1], ww[2], ww[3]}));
			X17_UNROLL for (u32 dt = 0; dt < D_TILES; ++dt) {
				u32 const lo = tr_lane_off[dt], hi = lo + TR_SIXTEEN_ROWS;
				dv_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
					transposed_fragment(base + kt::DO_TR_OFFSET + lo, base + kt::DO_TR_OFFSET + hi), pfrag, dv_acc[dt], 0, 0, 0);
				dk_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
					transposed_fragment(q_wide + lo, q_wide + hi), wfrag, dk_acc[dt], 0, 0, 0);
			}
		};
		// A wavefront's keys are seen by the tiles [wave_tile_first, wave_tile_last] of the workgroup's walk.  Plain loops
		// instead of one loop with a skip (around a skip the compiler moves the accumulators about once per step), and
		// the middle stretch runs three steps per trip so that the ring slot of every LDS address is an immediate; the
		// steps before it reaches a multiple of three, and the last ones, take the slot from i.
		u32 const lead = wave_tile_first - tile_begin;
		u32 const active_end = wave_tile_last + 1 - tile_begin < n_steps ? wave_tile_last + 1 - tile_begin : n_steps;
		u32 i = 0;
		for (; i < lead; ++i) advance(i, i % kt::RING);
		for (; i < active_end && i % kt::RING != 0; ++i) {
			advance(i, i % kt::RING);
			compute(i, i % kt::RING);
		}
		for (; i + kt::RING <= active_end; i += kt::RING) {
			X17_UNROLL for (u32 slot = 0; slot < kt::RING; ++slot) {
				advance(i + slot, slot);
				compute(i + slot, slot);
			}
		}
		for (; i < active_end; ++i) {
			advance(i, i % kt::RING);
			compute(i, i % kt::RING);
		}
		for (; i < n_steps; ++i) advance(i, i % kt::RING);

		// ---- output: dk = 8 ln 2 * dk_acc, dv = dv_acc
		u16 *dkv_row = d_kv + (row_base + key) * KV_STRIDE + (size_t)head * 2 * HD;
		X17_UNROLL for (u32 dt = 0; dt < D_TILES; ++dt) {
			v2u const k_pair = {pack2_bf16_rne(dk_acc[dt][0] * EIGHT_LN2, dk_acc[dt][1] * EIGHT_LN2),
			                    pack2_bf16_rne(dk_acc[dt][2] * EIGHT_LN2, dk_acc[dt][3] * EIGHT_LN2)};
			v2u const v_pair = {pack2_bf16_rne(dv_acc[dt][0], dv_acc[dt][1]), pack2_bf16_rne(dv_acc[dt][2], dv_acc[dt][3])};
			*reinterpret_cast<v2u *>(dkv_row + 16 * dt + 4 * group) = k_pair;
			*reinterpret_cast<v2u *>(dkv_row + HD + 16 * dt + 4 * group) = v_pair;
		}
	}
}
