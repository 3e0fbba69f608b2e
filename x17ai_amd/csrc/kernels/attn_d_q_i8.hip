// attn_d_q_i8.hip -- backward of the int8 sliding-window attention with respect to q, for gfx950.
//
// The reference's backward kernels (attn_d_q.cuh:1-410) belong to its bf16 generation; its int8 / e4m3 generation has
// no backward yet.  This kernel keeps the structure of attn_d_q.cuh -- probabilities recomputed from the forward's
// log-sum-exp L, D = rowsum(dO * O) written out for a later dK/dV kernel, dS = P * (dP - D), dQ = dS . K -- on the
// forward semantics of attn_fwd_i8.hip (cuda/attn_fwd_i8.cuh:368-619): FixedI8 q / k / v codes (real = code / 8), a
// sink key AND value per head, scores in base 2 with the scalable-softmax temperature, causal sliding window.
// Per head and query i (position inside its sequence), with t_i = hd^-1/2 * lg2(min(W', i) + 4) * head_temp[h]:
//   P_ij  = 2^(t_i (q_i . k_j) - (L_i - lg2 255))     for the keys j in [max(0, i - W'), i - 1] and the sink
//   D_i   = dO_i . o_i,  o_i = out_code_i / 8         (the forward output as stored)
//   dS_ij = ln 2 * P_ij * (dO_i . v_j - D_i)
//   dq_i  = t_i * sum_j dS_ij k_j                      (gradient with respect to the REAL q; bf16)
// The forward's 8-bit rounding of P and the quantisation of q are treated as the identity.
//
// Design, MI355X-first (the forward kernel's blocking, so that its index arithmetic and tile layouts carry over):
//   * One workgroup = 4 wavefronts = 128 queries of one head; a wavefront owns 32 queries; 32 keys per step.
//   * S^T = K . Q^T on v_mfma_i32_32x32x32_i8 exactly as in the forward (keys are the "A" operand: a lane owns one
//     query and 8 keys of each 16-key tile).
//   * dP^T = V . dO^T and dQ^T += K^T . dS^T run on v_mfma_f32_32x32x16_f16.  K and V arrive as int8 (global -> LDS
//     directly, two steps ahead) and are widened to f16 once per workgroup, LDS -> LDS, one step ahead, by the
//     threads that fetched them: K into the granule layout that ds_read_b64_tr_b16 reads transposed (the "A" operand
//     K^T needs eight keys of one dim per lane), V into swizzled rows (the "A" operand V needs eight dims of one key).
//   * dO is bf16 in memory.  Everything is linear in dO_i, so each query row is scaled by a power of two that brings
//     its largest element into [1, 2) before it is rounded to f16 (more significand bits than bf16 for every element
//     that matters, and no underflow however small the gradients are); dq_i and D_i are scaled back at the end.
//     A lane keeps the f16 fragments of its whole row in registers: they are the "B" operand of dP^T directly.
//   * dS stays in registers: packed to f16 it is the "B" operand of the dQ^T product, as P is in the forward.
//
// common.h (generated per kernel) provides X17_N_HEADS, X17_HEAD_DIM, X17_Q_STRIDE, X17_KV_STRIDE, X17_O_STRIDE,
// X17_STRICT_MATH.  gridDim = (query blocks, head groups, sequences), as for the forward.

#include "common.h"
#include "x17_device.h"
#include "attn_bwd_tile.h"

using namespace x17;
namespace at = x17::attn_tile;
namespace bt = x17::attn_bwd_tile;

namespace {

constexpr u32 HD = X17_HEAD_DIM;
constexpr u32 N_HEADS = X17_N_HEADS;
constexpr u32 Q_STRIDE = X17_Q_STRIDE;
constexpr u32 KV_STRIDE = X17_KV_STRIDE;
constexpr u32 O_STRIDE = X17_O_STRIDE;
constexpr u32 HPK = at::HEADS_PER_KERNEL;
constexpr u32 K_SLICES = HD / 32;      // 32 bytes of head_dim per QK MFMA
constexpr u32 D_SLICES = HD / 16;      // 16 dims per dP MFMA
constexpr u32 D_BLOCKS = HD / 32;      // 32 output dims per dQ MFMA
constexpr u32 CPR = at::CHUNKS_PER_ROW;

static_assert(HD == 32 || HD == 64 || HD == 128, "head_dim must be 32, 64 or 128");
static_assert(N_HEADS % HPK == 0, "n_heads must be divisible by heads_per_kernel");

constexpr f32 LOG2_PROB_SCALE = 7.9943534368588578f;                       // lg2(255): the forward's L carries it
constexpr f32 BASE_TEMPERATURE = f32(constexpr_inv_sqrt(f64(HD)) / 64.0);  // for dots of codes (8 q . 8 k)
// dq = t_real * ln 2 * sum_j w_j k_j with t_real = 64 * temperature (the temperature below is for dots of codes)
// and k = code / 8: 64 * ln 2 / 8
constexpr f32 EIGHT_LN2 = 5.5451774444795625f;

typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

X17_DEV f32 partner_f32(f32 x, u32 half) {
	u32 u = f2u(x);
	auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
	return u2f(half == 0 ? r[1] : r[0]);
}
X17_DEV i32 partner_i32(i32 x, u32 half) {
	auto r = __builtin_amdgcn_permlane32_swap((u32)x, (u32)x, false, false);
	return (i32)(half == 0 ? r[1] : r[0]);
}

// Raw K tile, as in the forward: linear 16-byte chunk n = key * CPR + c lives in 128-byte line n / 8 at position
// (n % 8) ^ ((line >> 1) & 7), so that the sixteen keys a ds_read_b128 serves at a time land in sixteen slots.
X17_DEV u32 k_chunk_offset(u32 key, u32 c) {
	u32 n = key * CPR + c;
	u32 line = n >> 3;
	return (line << 7) | (((n & 7) ^ ((line >> 1) & 7)) << 4);
}
// f16 K tile, the forward's f16 V layout: 32-byte granule n = key * CPR + c (16 dims) lives in 256-byte line n / 8 at
// position (n % 8) ^ ((line & 3) << 1); the transposed 8-byte reads of 32 lanes then cover all banks once.
X17_DEV u32 granule_offset(u32 key, u32 c) {
	u32 n = key * CPR + c;
	u32 line = n >> 3;
	return (line << 8) | (((n & 7) ^ ((line & 3) << 1)) << 5);
}
// f16 V tile, read by rows: a key row is HD / 8 chunks of 16 bytes (8 dims); 16 / (HD / 8) keys share a 256-byte
// line, and chunk c16 of a key is stored at position c16 ^ line inside its key's part of the line: the sixteen keys
// a ds_read_b128 serves at a time (same c16) land in sixteen different slots for head_dim 32, 64 and 128.
X17_DEV u32 vrow_offset(u32 key, u32 c16) {
	constexpr u32 R = HD / 8, KPL = 16 / R;
	u32 const line = key / KPL;
	u32 const slot = (key % KPL) * R + (c16 ^ (line & (R - 1)));
	return line * 256 + slot * 16;
}

// sixteen int8 (four words) -> sixteen f16 (eight words), exact: flip the sign bit (b + 128 as an unsigned byte u),
// splice u under the f16 exponent of 1024 (0x6400 | u == 1024 + u), subtract 1152
X17_DEV void widen16(v4u raw, u32 (&w)[8]) {
	v2h const bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
	X17_UNROLL for (int i = 0; i < 4; ++i) {
		u32 word = raw[i] ^ 0x80808080u;
		u32 lo = __builtin_amdgcn_perm(0x64646464u, word, 0x04010400u);
		u32 hi = __builtin_amdgcn_perm(0x64646464u, word, 0x04030402u);
		w[2 * i] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, lo) + bias);
		w[2 * i + 1] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, hi) + bias);
	}
}

X17_DEV f32 i8_of(u32 word, int b) { return f32((i32)(i8)((word >> (8 * b)) & 0xFFu)); }

} // namespace

extern "C" __global__ __launch_bounds__(bt::THREADS_PER_BLOCK)
__attribute__((amdgpu_waves_per_eu(bt::WAVES_PER_SIMD, bt::WAVES_PER_SIMD)))
void kernel(
	u32 seq_len,
	i8 const *q,
	i8 const *kv,
	i8 const *sink_k,
	i8 const *sink_v,
	f32 const *attn_temperature,
	i8 const *out,               // the forward's output codes [rows, O_STRIDE]
	u16 const *d_out,            // bf16 [rows, O_STRIDE]: gradient with respect to the real output
	u16 *d_q,                    // bf16 [rows, Q_STRIDE]: gradient with respect to the real q
	f32 const *l,                // the forward's log-sum-exp [H, rows]
	f32 *d_rows,                 // D [H, rows] (may be null)
	u32 window_size
) {
	extern __shared__ __attribute__((aligned(1024))) u8 smem[];

	u32 const tid = threadIdx.x;
	u32 const lane = tid % 64;
	u32 const wave = __builtin_amdgcn_readfirstlane(tid / 64);
	u32 const half = lane / 32;
	u32 const qlane = lane % 32;

	// the forward's workgroup order: the query block is the slowest index and runs from the last block to the first
	u32 const pairs = gridDim.y * gridDim.z;
	u32 const lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
	u32 const pair = lin % pairs;
	u32 const q_block_index = gridDim.x - 1 - lin / pairs;
	u32 const head_group = pair % gridDim.y;
	u32 const seq = pair / gridDim.y;
	size_t const row_base = (size_t)seq * seq_len;
	size_t const all_rows = (size_t)gridDim.z * seq_len;
	u32 const q_block0 = at::block_first_query(q_block_index, seq_len);
	u32 const q_wave0 = q_block0 + wave * at::Q_PER_WAVE;
	u32 const qi = q_wave0 + qlane;
	u32 const wr = at::rounded_window(window_size);
	u32 const vis_bound = wr - 1 < 0x7FFFFFFFu ? wr - 1 : 0x7FFFFFFFu;
	u32 const kb_begin = at::first_key_block(q_block0, wr);
	u32 const kb_end = at::end_key_block(q_block0);
	u32 const wave_kb_first = at::first_key_block(q_wave0, wr);
	u32 const wave_kb_last = q_wave0 / at::KV_PER_STEP;
	u32 const n_steps = kb_end - kb_begin;

	for (u32 hh = 0; hh < HPK; ++hh) {
		u32 const head = head_group * HPK + hh;
		i8 const *q_head = q + row_base * Q_STRIDE + (size_t)head * HD;
		i8 const *kv_head = kv + row_base * KV_STRIDE + (size_t)head * 2 * HD;

		// ---- staging: thread t fetches 16-byte chunk t of the K tile and of the V tile and later widens them
		bool const stager = at::is_stager(tid);
		u32 stage_k_src = 0, stage_v_src = 0, k_f16_dst = 0, v_f16_dst0 = 0, v_f16_dst1 = 0;
		if (stager) {
			stage_k_src = at::stage_k_offset(tid, KV_STRIDE);
			stage_v_src = at::stage_v_offset(tid, KV_STRIDE);
			// stored chunk `tid` of the raw K tile holds logical chunk n: key n / CPR, dims 16 * (n % CPR) .. + 15
			u32 const line = tid >> 3;
			u32 const n = (line << 3) | ((tid & 7) ^ ((line >> 1) & 7));
			k_f16_dst = granule_offset(n / CPR, n % CPR);
			v_f16_dst0 = vrow_offset(tid / CPR, 2 * (tid % CPR));
			v_f16_dst1 = vrow_offset(tid / CPR, 2 * (tid % CPR) + 1);
		}
		auto issue_kv_load = [&](u32 kb, u32 slot) {
			if (stager) {
				i8 const *src = kv_head + (size_t)(kb * at::KV_PER_STEP) * KV_STRIDE;
				u8 *k_dst = smem + bt::RAW_K_RING_OFFSET + slot * bt::RAW_TILE_BYTES + wave * 1024;
				u8 *v_dst = smem + bt::RAW_V_RING_OFFSET + slot * bt::RAW_TILE_BYTES + wave * 1024;
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(src + stage_k_src), X17_LDS_PTR(k_dst), 16, 0, 0);
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(src + stage_v_src), X17_LDS_PTR(v_dst), 16, 0, 0);
			}
		};
		auto widen = [&](u32 slot, u32 buf) {
			if (stager) {
				u32 w[8];
				widen16(*reinterpret_cast<v4u const *>(smem + bt::RAW_K_RING_OFFSET + slot * bt::RAW_TILE_BYTES + tid * 16), w);
				u8 *kd = smem + bt::K_F16_OFFSET + buf * bt::F16_TILE_BYTES + k_f16_dst;
				*reinterpret_cast<v4u *>(kd) = v4u{w[0], w[1], w[2], w[3]};
				*reinterpret_cast<v4u *>(kd + 16) = v4u{w[4], w[5], w[6], w[7]};
				widen16(*reinterpret_cast<v4u const *>(smem + bt::RAW_V_RING_OFFSET + slot * bt::RAW_TILE_BYTES + tid * 16), w);
				u8 *vd = smem + bt::V_F16_OFFSET + buf * bt::F16_TILE_BYTES;
				*reinterpret_cast<v4u *>(vd + v_f16_dst0) = v4u{w[0], w[1], w[2], w[3]};
				*reinterpret_cast<v4u *>(vd + v_f16_dst1) = v4u{w[4], w[5], w[6], w[7]};
			}
		};
		// two loads in flight per staging thread and prefetched step; they complete in issue order
		auto wait_steps_in_flight = [&](u32 steps) {
			if (steps >= 1) {
				__builtin_amdgcn_s_waitcnt(0x0F72);          // vmcnt(2)
			} else {
				__builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
			}
		};
		static_assert(bt::PREFETCH == 2, "the waits below are written for a prefetch distance of 2");

		// ---- per-query set-up
		v4i qf[K_SLICES];
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
			qf[s] = *reinterpret_cast<v4i const *>(q_head + (size_t)qi * Q_STRIDE + 32 * s + 16 * half);
		}
		u32 const visible = qi < wr ? qi : wr;
		f32 temperature = BASE_TEMPERATURE * strict::lg2(f32(visible + 4u));
		temperature = temperature * attn_temperature[head];
		f32 const l_hat = l[(size_t)head * all_rows + row_base + qi] - LOG2_PROB_SCALE;

		// dO row: this lane's half of every 16-dim slice (dims 16 sl + 8 half .. + 7), bf16 -> f32
		u16 const *do_row = d_out + (row_base + qi) * O_STRIDE + (size_t)head * HD;
		i8 const *o_row = out + (row_base + qi) * O_STRIDE + (size_t)head * HD;
		f32 dof[D_SLICES][8];
		f32 row_max = 0.0f;
		X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) {
			v4u const raw = *reinterpret_cast<v4u const *>(do_row + 16 * sl + 8 * half);
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				dof[sl][2 * w] = u2f(raw[w] << 16);
				dof[sl][2 * w + 1] = u2f(raw[w] & 0xFFFF0000u);
				row_max = __builtin_fmaxf(row_max, __builtin_fmaxf(__builtin_fabsf(dof[sl][2 * w]), __builtin_fabsf(dof[sl][2 * w + 1])));
			}
		}
		row_max = __builtin_fmaxf(row_max, partner_f32(row_max, half));
		// power of two that brings the row's largest magnitude into [1, 2) (1 for an all-zero, infinite or NaN row)
		u32 const max_exp = (f2u(row_max) >> 23) & 0xFFu;
		bool const scalable = max_exp != 0 && max_exp != 0xFFu;
		f32 const scale = scalable ? u2f((254u - max_exp) << 23) : 1.0f;
		f32 const inv_scale = scalable ? u2f(max_exp << 23) : 1.0f;
		v8h dofrag[D_SLICES];                 // "B" operand of dP^T: lane = query, slots = dims 16 sl + 8 half + 0..7
		f32 d_part = 0.0f, dps_part = 0.0f;   // partial sums of D' = dO' . o and of dO' . sink_v (this lane's dims)
		X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) {
			v2u const oc = *reinterpret_cast<v2u const *>(o_row + 16 * sl + 8 * half);
			v2u const sv = *reinterpret_cast<v2u const *>(sink_v + (size_t)head * HD + 16 * sl + 8 * half);
			X17_UNROLL for (int e = 0; e < 8; ++e) {
				_Float16 const hval = (_Float16)(dof[sl][e] * scale);       // round to nearest even
				dofrag[sl][e] = hval;
				f32 const back = (f32)hval;
				d_part = fmaf32(back, i8_of(oc[e / 4], e % 4), d_part);
				dps_part = fmaf32(back, i8_of(sv[e / 4], e % 4), dps_part);
			}
		}
		f32 const d_other = partner_f32(d_part, half), dps_other = partner_f32(dps_part, half);
		// (both in code units of o and v: 8 times the real dot products; the lower half's partial sum first)
		f32 const d8 = half == 0 ? d_part + d_other : d_other + d_part;
		f32 const dps8 = half == 0 ? dps_part + dps_other : dps_other + dps_part;

		// the sink: a key and a value every query sees
		i32 sink_dot = 0;
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
			v4i sk = *reinterpret_cast<v4i const *>(sink_k + (size_t)head * HD + 32 * s + 16 * half);
			X17_UNROLL for (int w = 0; w < 4; ++w) sink_dot = __builtin_amdgcn_sdot4(qf[s][w], sk[w], sink_dot, false);
		}
		sink_dot += partner_i32(sink_dot, half);
		f32 const p_sink = sfu::ex2(f32(sink_dot) * temperature - l_hat);
		f32 const w_sink = p_sink * ((dps8 - d8) * 0.125f);
		v16f dq_acc[D_BLOCKS];               // dQ^T: lane = query, register r = dim 32 db + 8 (r / 4) + 4 half + r % 4
		X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
			X17_UNROLL for (int r4 = 0; r4 < 4; ++r4) {
				u32 const word = *reinterpret_cast<u32 const *>(sink_k + (size_t)head * HD + 32 * db + 8 * r4 + 4 * half);
				X17_UNROLL for (int b = 0; b < 4; ++b) dq_acc[db][4 * r4 + b] = w_sink * i8_of(word, b);
			}
		}

		// lane offsets of the operand fragments (the forward's transposed-read addressing for K^T)
		u32 kt_lane_off[D_BLOCKS];
		[[maybe_unused]] u32 kt_lane_off8[D_BLOCKS];
		{
			u32 const t = lane % 16, dh = (lane / 16) % 2;
			X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
				kt_lane_off[db] = granule_offset(4 * half + (t >> 2), 2 * db + dh) + 8 * (t & 3);
				kt_lane_off8[db] = granule_offset(8 + 4 * half + (t >> 2), 2 * db + dh) + 8 * (t & 3);
			}
		}

		// ---- pipeline prologue
		__syncthreads();                      // previous head's tiles are no longer read
		X17_UNROLL for (u32 j = 0; j < bt::PREFETCH; ++j) {
			if (j < n_steps) issue_kv_load(kb_begin + j, j);
		}
		wait_steps_in_flight((n_steps < bt::PREFETCH ? n_steps : bt::PREFETCH) - 1);
		widen(0, 0);

		for (u32 i = 0; i < n_steps; ++i) {
			u32 const kb = kb_begin + i;
			u32 const slot = i % bt::RING;
			// raw tile i + 1 has landed (this thread's chunks); at most step i + 2's loads stay in flight after the issue below
			wait_steps_in_flight(0);
			__builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0): own LDS traffic of step i - 1 is complete
			__builtin_amdgcn_s_barrier();                // ... and so is everybody else's: tiles i are visible
			if (i + bt::PREFETCH < n_steps) {
				issue_kv_load(kb + bt::PREFETCH, (i + bt::PREFETCH) % bt::RING);
			}
			if (i + 1 < n_steps) {
				widen((i + 1) % bt::RING, (i + 1) & 1);
			}
			if (kb < wave_kb_first || kb > wave_kb_last) {
				continue;
			}
			u8 const *k_raw = smem + bt::RAW_K_RING_OFFSET + slot * bt::RAW_TILE_BYTES;
			u8 const *k_f16 = smem + bt::K_F16_OFFSET + (i & 1) * bt::F16_TILE_BYTES;
			u8 const *v_f16 = smem + bt::V_F16_OFFSET + (i & 1) * bt::F16_TILE_BYTES;

			// S^T block: rows = 32 keys, columns = this wave's 32 queries
			v16i s_acc = {0};
			X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
				v4i kf = *reinterpret_cast<v4i const *>(k_raw + k_chunk_offset(qlane, 2 * s + half));
				s_acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[s], s_acc, 0, 0, 0);
			}
			// dP'^T block (times 8: v codes): rows = the same 32 keys
			v16f dp_acc = {0};
			X17_UNROLL for (u32 sl = 0; sl < D_SLICES; ++sl) {
				v8h const vf = *reinterpret_cast<v8h const *>(v_f16 + vrow_offset(qlane, 2 * sl + half));
				dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, dofrag[sl], dp_acc, 0, 0, 0);
			}

			u32 const key0 = kb * at::KV_PER_STEP;
			bool const need_mask = !(key0 + 31 < q_wave0 && (q_wave0 + 31 - key0) <= wr);
			X17_UNROLL for (u32 tile = 0; tile < 2; ++tile) {
				// this lane's keys of the tile: 4 half + {0..3} and 8 + 4 half + {0..3}
				f32 w[8];
				u32 const first = qi - 1 - (key0 + 16 * tile + 4 * half);
				X17_UNROLL for (u32 r = 0; r < 8; ++r) {
					f32 const s = f32(s_acc[8 * tile + r]) * temperature;
					f32 p = sfu::ex2(s - l_hat);
					if (need_mask) {
						// key j is visible iff the distance qi - 1 - j, as an unsigned number, is at most W' - 1
						u32 const distance = first - (8 * (r / 4) + (r % 4));
						p = distance <= vis_bound ? p : 0.0f;
					}
					w[r] = p * ((dp_acc[8 * tile + r] - d8) * 0.125f);
				}
				v8h wfrag;
				X17_UNROLL for (u32 r = 0; r < 8; ++r) wfrag[r] = (_Float16)w[r];
				X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
					u8 const *p0 = k_f16 + kt_lane_off[db] + tile * (16 * CPR * 32);
					u8 const *p1 = CPR >= 4 ? p0 + 8 * CPR * 32 : k_f16 + kt_lane_off8[db] + tile * (16 * CPR * 32);
					v4s const lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p0);
					v4s const hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p1);
					v8s const both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
					dq_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, both), wfrag, dq_acc[db], 0, 0, 0);
				}
			}
		}

		// ---- output: dq = 8 ln 2 * temperature * dq_acc / scale, D = d8 / (8 scale)
		f32 const out_scale = (temperature * EIGHT_LN2) * inv_scale;
		u16 *dq_row = d_q + (row_base + qi) * Q_STRIDE + (size_t)head * HD;
		X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
			X17_UNROLL for (int g = 0; g < 4; ++g) {
				f32 b[4];
				X17_UNROLL for (int e = 0; e < 4; ++e) b[e] = dq_acc[db][4 * g + e] * out_scale;
				v2u const pair = {pack2_bf16_rne(b[0], b[1]), pack2_bf16_rne(b[2], b[3])};
				*reinterpret_cast<v2u *>(dq_row + 32 * db + 8 * g + 4 * half) = pair;
			}
		}
		if (d_rows != nullptr && half == 0) {
			d_rows[(size_t)head * all_rows + row_base + qi] = (d8 * 0.125f) * inv_scale;
		}
	}
}
