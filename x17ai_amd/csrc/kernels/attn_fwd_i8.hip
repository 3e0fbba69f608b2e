// attn_fwd_i8.hip -- int8 causal sliding-window flash-attention forward with a sink token and
// scalable-softmax temperature, for gfx950.
//
// Replaces the reference's AttnForward (cuda/attn_fwd_i8.cuh:30-620); the kernel entry and its
// parameters follow templates/attn/kernel.cu:9-33.  The arithmetic it reproduces, per head and
// query i (0-based position inside its sequence):
//   keys j in [max(0, i - W'), i - 1] plus one sink key/value; W' = window rounded up to 16
//   (0 = no window);  n = min(W', i) + 4;  temperature = f32(hd^-1/2 / 64) * lg2(n) * head_temp[h];
//   s_j = f32(q_i . k_j) * temperature (int32 dot);  running max starts at the sink score, the
//   partial sums at 4 x 63.75, O at 255 * sink_v;  per 16-key tile (ascending): rescale when the
//   max grows, p_j = ex2(s_j - max) * 255, four partial sums over key quads of the tile,
//   P_j = rne(p_j), O += f32(sum_j P_j v_j);  at the end sum = (s0+s1)+(s2+s3),
//   L = lg2(sum) + max, out = fixedi8(O / sum).
//
// Design, MI355X-first:
//   * One workgroup = 4 wavefronts = 128 queries of one head; a wavefront owns 32 queries.
//     Keys/values are staged 32 keys per step (two 16-key tiles) through rings in LDS.
//   * S^T = K . Q^T on v_mfma_i32_32x32x32_i8 with the KEYS as the MFMA "A" operand: a lane then
//     owns one query (lane % 32) and 8 keys of each 16-key tile; the other 8 keys sit in lane+32.
//     Row max needs one cross-lane exchange per tile; the four per-quad partial sums of the
//     reference fall two-and-two into the lane pair, so they need none until the very end.
//   * P stays in registers: packed to f16 it already IS the "B" operand of O^T = V^T . P^T.
//     PV runs on v_mfma_f32_32x32x16_f16: K = 16 is exactly one 16-key tile, P (0..255) and
//     int8 V are exact in f16 and every tile sum is below 2^24, so the f32 result equals the
//     reference's f32(int32 dot) bit for bit.  (CDNA4 has no unsigned x signed int8 MFMA; an
//     int8 PV would need two MFMAs per tile for the 8-bit probabilities.)
//   * K and V go global -> LDS directly, three 32-key steps ahead of their use.  V is widened to
//     f16 once per workgroup, LDS -> LDS, one step ahead (sign-bit flip, byte splice under the
//     exponent of 1024, subtract 1152: five instructions per four values) and fetched transposed
//     with ds_read_b64_tr_b16, so no register transposes.
//   * Three workgroups share a compute unit (register budget of 168 per lane), so one workgroup's
//     waits for its tiles and its barrier are covered by the others' arithmetic.
//   * X17_STRICT_MATH = 1: deterministic ex2 and one explicit f32 add per tile (parity build).
//     X17_STRICT_MATH = 0: v_exp_f32 with the factor 255 folded into the exponent, accumulation
//     inside the PV MFMA, and lazy rescaling of O (speed build; results stay within one output code).
//
// common.h (generated per kernel) provides X17_N_HEADS, X17_HEAD_DIM, X17_Q_STRIDE,
// X17_KV_STRIDE, X17_O_STRIDE, X17_STRICT_MATH.
//
// Extension over the reference ABI: gridDim.z = number of independent sequences stacked along
// the rows of q / kv / out (each `seq_len` rows, own causal origin); L is [H, gridDim.z * seq_len].
//
// X17_ATTN_ROW_SCALES = 1 (no counterpart in the reference, whose codes share the constant scale 1/8):
// five more parameters give one f32 scale per (head, row) for q and k, a weight <= 1 per (head, row)
// for v (all three laid out [H, rows] like L), and per head the weight of the sink value and the output
// scale.  The recurrence becomes
//   tq = ((f32(hd^-1/2) * lg2(n)) * head_temp[h]) * q_scale[h, i],  s_j = (f32(q_i . k_j) * k_scale[h, j]) * tq,
//   sink score = f32(q_i . sink_k) * (tq * 0.125),  P_j = rne(p_j * v_weight[h, j]),
//   O starts at f32(255 * sink_v) * sink_v_weight[h],  out = store((O * rcp(sum)) * out_scale[h])
// and produces the bits of the plain kernel when every scale is 1/8 and every weight and out_scale is 1.
// X17_ATTN_OUT_BF16 = 1 stores bf16 real values (round to nearest even) instead of FixedI8 codes.

#include "common.h"
#include "x17_device.h"
#include "attn_tile.h"

using namespace x17;
namespace at = x17::attn_tile;

namespace {

constexpr u32 HD = X17_HEAD_DIM;
constexpr u32 N_HEADS = X17_N_HEADS;
constexpr u32 Q_STRIDE = X17_Q_STRIDE;
constexpr u32 KV_STRIDE = X17_KV_STRIDE;
constexpr u32 O_STRIDE = X17_O_STRIDE;
constexpr u32 HPK = at::HEADS_PER_KERNEL;
constexpr u32 K_SLICES = HD / 32;      // 32 bytes of head_dim per QK MFMA
constexpr u32 D_BLOCKS = HD / 32;      // 32 output dims per PV MFMA
constexpr u32 CPR = HD / 16;           // 16-byte chunks per key row
constexpr bool STRICT = X17_STRICT_MATH != 0;
constexpr bool ROW_SCALES = at::ROW_SCALES;
constexpr bool OUT_BF16 = X17_ATTN_OUT_BF16 != 0;
static_assert(ROW_SCALES || !OUT_BF16, "the bf16 output needs the row-scaled build (it supplies out_scale)");

static_assert(HD == 32 || HD == 64 || HD == 128, "head_dim must be 32, 64 or 128");
static_assert(N_HEADS % HPK == 0, "n_heads must be divisible by heads_per_kernel");

constexpr f32 PROB_SCALE = 255.0f;                                  // cuda/attn_fwd_i8.cuh:206
constexpr f32 LOG2_PROB_SCALE = 7.9943534368588578f;                // lg2(255)
constexpr f32 MAX_LIFT = 32.0f;                                     // (1024 + 255) * 32 stays inside f16
constexpr f32 BASE_TEMPERATURE = ROW_SCALES ? f32(constexpr_inv_sqrt(f64(HD)))
                                            : f32(constexpr_inv_sqrt(f64(HD)) / 64.0);   // :47, :447-449

typedef short v4s __attribute__((ext_vector_type(4)));

// value of lane ^ 32
X17_DEV f32 partner_f32(f32 x, u32 half) {
	u32 u = f2u(x);
	auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
	return u2f(half == 0 ? r[1] : r[0]);
}
X17_DEV i32 partner_i32(i32 x, u32 half) {
	auto r = __builtin_amdgcn_permlane32_swap((u32)x, (u32)x, false, false);
	return (i32)(half == 0 ? r[1] : r[0]);
}

// K tile: linear 16-byte chunk n = key * CPR + c lives in 128-byte line n / 8 at position
// (n % 8) ^ ((line >> 1) & 7).  The LDS serves a ds_read_b128 sixteen lanes at a time out of 64
// four-byte banks; with this mapping the sixteen keys of such a group land in sixteen different
// 16-byte slots for every supported head_dim.
X17_DEV u32 k_chunk_offset(u32 key, u32 c) {
	u32 n = key * CPR + c;
	u32 line = n >> 3;
	return (line << 7) | (((n & 7) ^ ((line >> 1) & 7)) << 4);
}

// V tile (f16): linear 32-byte granule n = key * CPR + c (16 dims) lives in 256-byte line n / 8
// at position (n % 8) ^ ((line & 3) << 1): the 4 keys x 2 granules that 32 lanes of a transposed
// read touch then cover all 64 banks exactly once (checked exhaustively for head_dim 32/64/128).
X17_DEV u32 v_granule_offset(u32 key, u32 c) {
	u32 n = key * CPR + c;
	u32 line = n >> 3;
	return (line << 8) | (((n & 7) ^ ((line & 3) << 1)) << 5);
}

X17_DEV u32 pack_f16(f32 lo, f32 hi) {
	// both values are integers below 2048: exact in f16 whatever the rounding mode
	return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

// One 16-byte-per-lane direct-to-LDS load: LDS destination in M0 (wave-uniform; lane l lands 16 * l bytes further),
// global source = a uniform 64-bit base in scalar registers + a 32-bit offset per lane (the compiler's own selection
// forms a 64-bit address per lane with a 64-bit vector add in front of every load).
X17_DEV void load_to_lds_16(u8 *lds_uniform, i8 const *src_uniform, u32 lane_offset) {
	// (the address is the same in every lane; reading it from the first one tells the compiler so)
	u32 const lds = __builtin_amdgcn_readfirstlane((u32)(size_t)X17_LDS_PTR(lds_uniform));
	// (gfx9 family: a scalar write of M0 needs one wait state before a direct-to-LDS load reads it; the compiler
	// inserts it for its own loads and cannot see into this string)
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
	             :: "s"(lds), "v"(lane_offset), "s"(src_uniform) : "memory", "m0");
}

// Speed build: p + PACK_MAGIC rounds p in [0, 256) to the nearest integer P (ties to even, as rintf) and leaves
// the f16 bit pattern of 1024 + P in the low half of the sum: 12582912 = 1.5 * 2^23 has an ulp of 1 and the bits
// 0x4B400000; adding 0x6400 = 25600 puts the f16 exponent of 1024 above the eight integer bits.
constexpr f32 PACK_MAGIC = 12582912.0f + 25600.0f;

} // namespace

extern "C" __global__ __launch_bounds__(at::THREADS_PER_BLOCK)
__attribute__((amdgpu_waves_per_eu(at::WAVES_PER_SIMD, at::WAVES_PER_SIMD)))
void kernel(
	u32 seq_len,
	i8 const *q,
	i8 const *kv,
	i8 const *sink_k,
	i8 const *sink_v,
	f32 const *attn_temperature,
	i8 *out,
	f32 *l_out,
	u32 window_size
#if X17_ATTN_ROW_SCALES
	,
	f32 const *q_scale,          // [n_heads, rows]
	f32 const *k_scale,          // [n_heads, rows]
	f32 const *v_weight,         // [n_heads, rows]
	f32 const *sink_v_weight,    // [n_heads]
	f32 const *out_scale         // [n_heads]
#endif
) {
	extern __shared__ __attribute__((aligned(1024))) u8 smem[];

	u32 const tid = threadIdx.x;
	u32 const lane = tid % 64;
	u32 const wave = __builtin_amdgcn_readfirstlane(tid / 64);
	u32 const half = lane / 32;
	u32 const qlane = lane % 32;

	// Which (sequence, head group, query block) this workgroup takes.  The hardware starts workgroups in the order of
	// their linear index (and deals them round-robin to the 8 XCDs).  The query block is the slowest index of that
	// order and runs from the last block to the first: the workgroups in flight at one time are the same few query
	// blocks of every (sequence, head group) pair -- neighbouring blocks of a pair share most of their key/value
	// window in the L2 of the XCD the pair keeps landing on when the pairs are a multiple of 8 -- and the blocks with
	// the shortest windows (the first of each sequence) come last, where they fill the tail of the launch.
	// Measured against the other orders on both long workloads: 2-4 % faster than query blocks fastest
	// (4 x 8192 tokens, window 512), 7 % faster on 65536 tokens with a window of 4096.
	u32 const pairs = gridDim.y * gridDim.z;
	u32 const lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
	u32 const pair = lin % pairs;
	u32 const q_block_index = gridDim.x - 1 - lin / pairs;
	u32 const head_group = pair % gridDim.y;
	u32 const seq = pair / gridDim.y;
	size_t const row_base = (size_t)seq * seq_len;          // first row of this sequence
	// position of the block's first query; a last block that would overhang the sequence (lengths are multiples of 64,
	// src/device/cuda/attn.rs:398-404) starts earlier and recomputes some of its neighbour's queries
	u32 const q_block0 = at::block_first_query(q_block_index, seq_len);
	u32 const q_wave0 = q_block0 + wave * at::Q_PER_WAVE;
	u32 const qi = q_wave0 + qlane;                         // this lane's query position

	// cuda/attn_fwd_i8.cuh:408-412 -- window 0 means "no window"; otherwise rounded up to 16
	u32 const wr = at::rounded_window(window_size);
	u32 const vis_bound = wr - 1 < 0x7FFFFFFFu ? wr - 1 : 0x7FFFFFFFu;

	// key blocks (32 keys) the workgroup walks, and the sub-range this wave needs
	u32 const kb_begin = at::first_key_block(q_block0, wr);
	u32 const kb_end = at::end_key_block(q_block0);                          // exclusive
	u32 const wave_kb_first = at::first_key_block(q_wave0, wr);
	u32 const wave_kb_last = q_wave0 / at::KV_PER_STEP;                      // inclusive

	for (u32 hh = 0; hh < HPK; ++hh) {
		u32 const head = head_group * HPK + hh;
		i8 const *q_head = q + row_base * Q_STRIDE + (size_t)head * HD;
		i8 const *kv_head = kv + row_base * KV_STRIDE + (size_t)head * 2 * HD;

		// ---- staging helpers for one 32-key block.  Both K and V travel global -> LDS without passing
		// through registers (thread t fetches 16-byte chunk t of each tile), PREFETCH steps ahead; one step
		// before its use a V tile is widened LDS -> LDS by the threads that fetched it.
		bool const stager = at::is_stager(tid);
		u32 stage_k_src = 0, stage_v_src = 0, widen_dst = 0;
		if (stager) {
			// lane `tid` fills stored chunk `tid` of the K tile (attn_tile.h finds which logical chunk lives there)
			stage_k_src = at::stage_k_offset(tid, KV_STRIDE);
			stage_v_src = at::stage_v_offset(tid, KV_STRIDE);
			widen_dst = v_granule_offset(tid / CPR, tid % CPR);
		}
		u32 const stage_lds = wave * 1024;                // wave-uniform part of the direct-to-LDS address
		auto issue_kv_load = [&](u32 kb, u32 slot) {
			if (stager) {
				i8 const *src = kv_head + (size_t)(kb * at::KV_PER_STEP) * KV_STRIDE;
				u8 *k_dst = smem + at::K_RING_OFFSET + slot * at::K_TILE_BYTES + stage_lds;
				u8 *v_dst = smem + at::RAW_V_RING_OFFSET + slot * at::RAW_V_TILE_BYTES + stage_lds;
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(src + stage_k_src), X17_LDS_PTR(k_dst), 16, 0, 0);
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(src + stage_v_src), X17_LDS_PTR(v_dst), 16, 0, 0);
			}
#if X17_ATTN_ROW_SCALES
			if (wave == 0) {
				// lanes 0..31 fetch the keys' scales, lanes 32..63 the value rows' weights: 4 bytes per lane
				f32 const *base = half == 0 ? k_scale : v_weight;
				f32 const *src = base + (size_t)head * ((size_t)gridDim.z * seq_len) + row_base + (size_t)kb * at::KV_PER_STEP + qlane;
				u8 *dst = smem + at::SCALE_RING_OFFSET + slot * at::SCALE_TILE_BYTES;
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(src), X17_LDS_PTR(dst), 4, 0, 0);
			}
#endif
		};
		auto widen_v = [&](u32 slot, u32 tile) {
			if (CPR == 8 || stager) {          // (head_dim 128: every thread stages)
				v4u raw = *reinterpret_cast<v4u const *>(smem + at::RAW_V_RING_OFFSET + slot * at::RAW_V_TILE_BYTES + tid * 16);
				// int8 -> f16: b + 128 as an unsigned byte u, 0x6400 | u == 1024 + u, minus 1152
				v2h const bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
				u32 w[8];
				X17_UNROLL for (int i = 0; i < 4; ++i) {
					u32 word = raw[i] ^ 0x80808080u;
					u32 l = __builtin_amdgcn_perm(0x64646464u, word, 0x04010400u);
					u32 h = __builtin_amdgcn_perm(0x64646464u, word, 0x04030402u);
					w[2 * i] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, l) + bias);
					w[2 * i + 1] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, h) + bias);
				}
				u8 *dst = smem + at::V_TILES_OFFSET + tile * at::V_TILE_BYTES + widen_dst;
				*reinterpret_cast<v4u *>(dst) = v4u{w[0], w[1], w[2], w[3]};
				*reinterpret_cast<v4u *>(dst + 16) = v4u{w[4], w[5], w[6], w[7]};
			}
		};
		// each staging thread has two loads in flight per prefetched step (three in the first wavefront of
		// the row-scaled build); they complete in issue order
		auto wait_steps_in_flight = [&](u32 steps) {
			if (ROW_SCALES && wave == 0) {
				if (steps >= 2) {
					__builtin_amdgcn_s_waitcnt(0x0F76);          // vmcnt(6)
				} else if (steps == 1) {
					__builtin_amdgcn_s_waitcnt(0x0F73);          // vmcnt(3)
				} else {
					__builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
				}
			} else if (steps >= 2) {
				__builtin_amdgcn_s_waitcnt(0x0F74);          // vmcnt(4)
			} else if (steps == 1) {
				__builtin_amdgcn_s_waitcnt(0x0F72);          // vmcnt(2)
			} else {
				__builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
			}
		};
		static_assert(at::PREFETCH == 3, "the waits below are written for a prefetch distance of 3");

		// ---- per-query setup (cuda/attn_fwd_i8.cuh:444-517)
		v4i qf[K_SLICES];
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
			qf[s] = *reinterpret_cast<v4i const *>(q_head + (size_t)qi * Q_STRIDE + 32 * s + 16 * half);
		}
		u32 const visible = qi < wr ? qi : wr;
		f32 temperature = BASE_TEMPERATURE * strict::lg2(f32(visible + 4u));
		temperature = temperature * attn_temperature[head];
#if X17_ATTN_ROW_SCALES
		temperature = temperature * q_scale[(size_t)head * ((size_t)gridDim.z * seq_len) + row_base + qi];
#endif
		// (the sign is the head's: lg2(visible + 4) >= 2)
		bool const positive_temperature = __builtin_amdgcn_readfirstlane(f2u(attn_temperature[head])) - 1u < 0x7F7FFFFFu;

		i32 sink_dot = 0;
		X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
			v4i sk = *reinterpret_cast<v4i const *>(sink_k + (size_t)head * HD + 32 * s + 16 * half);
			X17_UNROLL for (int w = 0; w < 4; ++w) sink_dot = __builtin_amdgcn_sdot4(qf[s][w], sk[w], sink_dot, false);
		}
		sink_dot += partner_i32(sink_dot, half);

		f32 m = ROW_SCALES ? f32(sink_dot) * (temperature * 0.125f) : f32(sink_dot) * temperature;
		f32 m_ref = m;                       // speed build: the maximum O's scale refers to, and 2^(m - m_ref)
		f32 lift = 1.0f;
		v2h lift2 = {(_Float16)1.0f, (_Float16)1.0f};
		f32 sum_lo = 0.25f * PROB_SCALE;     // partial sum of key quad `half` of every tile
		f32 sum_hi = 0.25f * PROB_SCALE;     // partial sum of key quad `2 + half`
		// (the lane pair holds the reference's four partial sums two-and-two; each starts at 63.75)
		v16f o_acc[D_BLOCKS];                // O^T: lane = query, register r = dim 32*db + 8*(r/4) + 4*half + r%4
		if constexpr (!STRICT && !ROW_SCALES) {
			// Speed build: O starts at 255 * sink_v at the scale 2^-12 its accumulation starts from (see below), and the
			// matrix cores compute that as the outer product (sink_v) x (255 * 2^-12): key slot 0 of the V^T operand
			// holds the sink value of the lane's dim, key slot 0 of the P^T operand the constant, every other slot is
			// zero -- one product per element, exact.  (A few instructions per 32 dims instead of a conversion, a fused
			// multiply-add and a multiplication per element.)
			typedef short v8s __attribute__((ext_vector_type(8)));
			_Float16 const p0 = half == 0 ? (_Float16)(PROB_SCALE / 4096.0f) : (_Float16)0.0f;
			v8s pz = {0, 0, 0, 0, 0, 0, 0, 0};
			pz[0] = __builtin_bit_cast(short, p0);
			X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
				_Float16 const v0 = half == 0 ? (_Float16)(f32)(i32)sink_v[(size_t)head * HD + 32 * db + qlane] : (_Float16)0.0f;
				v8s vz = {0, 0, 0, 0, 0, 0, 0, 0};
				vz[0] = __builtin_bit_cast(short, v0);
				v16f const zero = {0};
				o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, vz), __builtin_bit_cast(v8h, pz), zero, 0, 0, 0);
			}
		} else
		X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
			X17_UNROLL for (int r4 = 0; r4 < 4; ++r4) {
				// 255 * v for the int8 byte v, through the unsigned byte v + 128 (one conversion and one fma per value, all exact)
				u32 const word = *reinterpret_cast<u32 const *>(sink_v + (size_t)head * HD + 32 * db + 8 * r4 + 4 * half) ^ 0x80808080u;
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					o_acc[db][4 * r4 + b] = fmaf32(f32((word >> (8 * b)) & 0xFFu), 255.0f, -32640.0f);
				}
			}
		}
#if X17_ATTN_ROW_SCALES
		{
			f32 const sink_weight = sink_v_weight[head];
			X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
				X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] * sink_weight;
			}
		}
#endif

		u32 const n_steps = kb_end - kb_begin;
		if constexpr (!STRICT) {
			// ---- speed build.  The same recurrence, rebuilt around what the kernel turned out to be bound by: the
			// number of instructions of ANY kind a SIMD has to issue per step (scalar bookkeeping and waits count like
			// vector arithmetic; with three wavefronts per SIMD an instruction costs 1.5-2.5 ns of SIMD time whatever it does).
			//  * A wave's steps fall into runs -- nothing to do, masked (the window's edge), fully visible, the diagonal,
			//    nothing to do -- and each run is its own loop.  Every step requests a tile (past the end the last one
			//    again, into a slot nobody reads any more), so the waits are constants.
			//  * The long run (fully visible steps) is unrolled over the four phases of the tile ring: every LDS address
			//    is a register plus an immediate, and the ring arithmetic disappears from the scalar unit.
			//  * The tile requests take a scalar base and a lane offset; M0 is set by one scalar addition.
			//  * The 8-bit probabilities are rounded and turned into f16 by one fused multiply-add and one byte shuffle per
			//    pair (PACK_MAGIC); the lift and the removal of the 1024 are one packed fma.
			//  * O and the partial sums live at the scale of a reference maximum kept HEADROOM above the running one
			//    whenever it is set: the lift of new probabilities then starts at 2^-12 (8-bit integers times it are still
			//    exact f16 values), a moving maximum costs one exponential, and O has to be brought down only after the
			//    maximum has grown by 17 (Gaussian scores move it by that much a few times per query block, not per tile).
			//  * The score accumulators start at the bits of 1.5 * 2^23 instead of zero: the int32 sum 0x4B400000 + dot,
			//    read as a float, is 12582912 + dot exactly (|dot| < 2^22), so no score is ever converted.  What refers to
			//    a maximum lives in that biased domain: `ext` is the running extreme of sgn * (12582912 + dot) (exact) and
			//    `mb` the subtrahend of the exponent, ext * |temperature| - lg2 255 rounded to a float.  That rounding (an
			//    ulp of 12582912 * temperature) would move the maximum the probabilities are rounded against; its exact
			//    remainder is therefore taken and 2^-remainder (`fine`) multiplies every probability inside operations that
			//    are needed anyway (the rounding addition is the fused multiply-add above, the sums' lift carries it).
			//  * The row maximum of a tile needs the partner lane's eight keys only when it moves: both lanes hold the same
			//    `ext`, and the tile's maximum exceeds it exactly when one of the two halves does.
			//  * Row-scaled build: a key's scale is not monotone in the dot product and the 16 registers of the bias words are
			//    not there to spend (they cost spills inside the loop), so the accumulators start at zero and
			//    z = f32(dot) * k_scale (a conversion and a multiplication per score); the
			//    extremes are taken over z as floats, and -- z being small -- the subtrahend ext * |t| - lg2 255 rounds to
			//    within 4e-6 of its value: no remainder is carried (`fine` is 1) and the value row's weight takes its place
			//    in the rounding fused multiply-add, P = rne(p * v_weight).  The first wavefront requests the step's 32 key
			//    scales and 32 value weights with the K tile (one more load in flight per prefetched step: its waits count
			//    three loads per step).  Scales are taken to be non-negative (absmax / 127): the sign of a query's
			//    temperature is then the head's.
			constexpr f32 HEADROOM = 12.0f, LIFT0 = 1.0f / 4096.0f, DOT_BIAS = 12582912.0f;
			v16i s_bias;
			X17_UNROLL for (int r = 0; r < 16; ++r) s_bias[r] = ROW_SCALES ? 0 : 0x4B400000;
			if constexpr (!ROW_SCALES) {
				asm volatile("" : "+v"(s_bias));      // (kept in registers: rebuilding it per step would cost what it saves)
			}
			f32 const abs_t = __builtin_fabsf(temperature);
			f32 const sgn = positive_temperature ? 1.0f : -1.0f;
			f32 ext = ROW_SCALES ? (f32(sink_dot) * 0.125f) * sgn : (f32(sink_dot) + DOT_BIAS) * sgn;
			f32 mb, fine;
			auto set_subtrahend = [&]() {
				if constexpr (ROW_SCALES) {
					mb = fmaf32(ext, abs_t, -LOG2_PROB_SCALE);
					fine = 1.0f;
				} else {
					// ext * |t| as a rounded product and its exact remainder; prod - mb is exact (neighbouring floats)
					f32 const prod = ext * abs_t;
					f32 const low = fmaf32(ext, abs_t, -prod);
					mb = prod - LOG2_PROB_SCALE;
					fine = hw::ex2(-(((prod - mb) - LOG2_PROB_SCALE) + low));          // 2^-(what mb leaves over): close to 1
				}
			};
			set_subtrahend();
			f32 ext_ref = ext;                        // O and the sums refer to the maximum HEADROOM above this extreme's score
			lift = LIFT0;
			f32 sum_lift = LIFT0 * fine;
			lift2 = v2h{(_Float16)LIFT0, (_Float16)LIFT0};
			v2h neg_bias2 = {(_Float16)(-1024.0f * LIFT0), (_Float16)(-1024.0f * LIFT0)};      // -1024 * lift2
			sum_lo = sum_lo * LIFT0;
			sum_hi = sum_hi * LIFT0;
			if constexpr (ROW_SCALES) {
				X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
					X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] * LIFT0;
				}
			}
			u32 const first_active = wave_kb_first - kb_begin;
			u32 const diagonal = wave_kb_last - kb_begin;
			// first block that lies inside the window of all 32 queries: q_wave0 + 31 - 32 kb <= wr
			u32 const inside_kb = q_wave0 + 31 > wr ? (q_wave0 + 62 - wr) / 32 : 0;
			u32 const inside_clamped = inside_kb < wave_kb_first ? wave_kb_first : (inside_kb > wave_kb_last ? wave_kb_last : inside_kb);
			// (the fully visible steps take the row maximum over the scores' bits, which needs a positive temperature;
			// with any other temperature every step goes the way of the masked ones)
			u32 const first_full = (positive_temperature ? inside_clamped : wave_kb_last) - kb_begin;

			// Tile requests.  Step s asks for K tile s + 3 and raw V tile s + 4, into the ring slots that K tile s - 1 and raw
			// V tile s have just left (a V tile is widened -- by the thread that fetched it -- during the step before its
			// use, so its slot is free one step earlier than a K slot): both tiles are on their way for three whole steps
			// before anything waits for them.  The requests of a thread complete in the order V0, (K0, V1), (K1, V2), ...;
			// step s needs the pair (K s, V s + 1), which leaves the two pairs behind it in flight.
			// `src` is the address of tile min(s + 3, last) when step s makes its requests; V tile s + 4 is one tile further
			// through a second lane offset, or the last tile again once the sequence ends.
			// SLOT: the step's position in the tile rings (s % RING) as a compile-time number, or -1 for "compute it".
			constexpr u32 TILE_STEP_BYTES = at::KV_PER_STEP * KV_STRIDE;
			i8 const *src = kv_head + (size_t)(kb_begin * at::KV_PER_STEP) * KV_STRIDE;
			u32 const stage_v_next = stage_v_src + TILE_STEP_BYTES;
			u32 const lds_wave = (u32)(size_t)X17_LDS_PTR(smem) + stage_lds;
			// SLOT >= 0 also says that tiles s + 3 and s + 4 both exist (the caller's loop bound)
			// row-scaled build, first wavefront: lane l < 32 fetches the scale of key l of the K tile being requested, lane
			// 32 + l the weight of its value row (4 bytes per lane, one 256-byte slot of the scale ring)
			[[maybe_unused]] f32 const *sc_src = nullptr;
#if X17_ATTN_ROW_SCALES
			sc_src = (half == 0 ? k_scale : v_weight) + (size_t)head * ((size_t)gridDim.z * seq_len) + row_base
			         + (size_t)kb_begin * at::KV_PER_STEP + qlane;
#endif
#define X17_REQUEST_SCALES(ring_slot) \
			if (wave == 0) { \
				__builtin_amdgcn_global_load_lds(X17_GLOBAL_PTR(sc_src), X17_LDS_PTR(smem + at::SCALE_RING_OFFSET + (ring_slot) * at::SCALE_TILE_BYTES), 4, 0, 0); \
			}
			auto request_tiles = [&]<int SLOT>(u32 s) __attribute__((always_inline)) {
				if constexpr (SLOT >= 0) {
					if constexpr (ROW_SCALES) {
						X17_REQUEST_SCALES((SLOT + 3) % 4)
						sc_src += at::KV_PER_STEP;
					}
					if (CPR == 8 || stager) {
						asm volatile("s_add_i32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
						             :: "s"(lds_wave), "i"(at::K_RING_OFFSET + ((SLOT + 3) % 4) * at::K_TILE_BYTES), "v"(stage_k_src), "s"(src) : "memory", "m0", "scc");
						asm volatile("s_add_i32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
						             :: "s"(lds_wave), "i"(at::RAW_V_RING_OFFSET + SLOT * at::RAW_V_TILE_BYTES), "v"(stage_v_next), "s"(src) : "memory", "m0", "scc");
					}
					src += TILE_STEP_BYTES;
				} else {
					bool const more = at::further_tile_exists(s, n_steps);
					if constexpr (ROW_SCALES) {
						X17_REQUEST_SCALES((s + 3) % at::RING)
						sc_src += __builtin_amdgcn_readfirstlane(more ? at::KV_PER_STEP : 0u);
					}
					if (CPR == 8 || stager) {
						load_to_lds_16(smem + at::K_RING_OFFSET + ((s + 3) % at::RING) * at::K_TILE_BYTES + stage_lds, src, stage_k_src);
						load_to_lds_16(smem + at::RAW_V_RING_OFFSET + (s % at::RING) * at::RAW_V_TILE_BYTES + stage_lds, src, more ? stage_v_next : stage_v_src);
					}
					if (more) {
						src += TILE_STEP_BYTES;
					}
				}
			};
			auto stage = [&]<int SLOT>(u32 i) __attribute__((always_inline)) {
				if (ROW_SCALES && wave == 0) {
					__builtin_amdgcn_s_waitcnt(0x0F76);      // vmcnt(6): three loads per step in the first wavefront
				} else {
					__builtin_amdgcn_s_waitcnt(0x0F74);      // vmcnt(4): K tile i and raw V tile i + 1 have landed
				}
				__builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0): own LDS traffic of step i-1 is complete
				__builtin_amdgcn_s_barrier();                // ... and so is everybody else's: tiles i are visible
				request_tiles.template operator()<SLOT>(i);
			};
			// raw V tile of step i + 1 -> f16 tile (i + 1) % 2
			auto widen_next = [&]<int SLOT>(u32 i) __attribute__((always_inline)) {
				if constexpr (SLOT >= 0) {
					widen_v((SLOT + 1) % at::RING, (SLOT + 1) & 1);
				} else {
					widen_v((i + 1) % at::RING, (i + 1) & 1);
				}
			};
			// maximum of a lane pair's two values, in both lanes
			auto pair_max_i32 = [](i32 x) {
				auto const r = __builtin_amdgcn_permlane32_swap((u32)x, (u32)x, false, false);
				return (i32)r[0] > (i32)r[1] ? (i32)r[0] : (i32)r[1];
			};

			// V^T operand of the 32 dims of block db: lane = dim 32 * db + lane % 32, slots = keys 16 * tile + {4 * half .. + 3,
			// 8 + 4 * half .. + 3}.  The lane's part of the address is the same for both tiles and both key groups
			// (they differ by whole 256-byte lines: 4096 bytes per tile, 2048 per group of 8 keys).
			// A key's granules fill CPR * 32 bytes; 16 keys further is always a whole number of 4-line groups further
			// (the swizzle key repeats), 8 keys further is one only when a key row has at least four granules.
			u32 v_lane_off[D_BLOCKS];
			[[maybe_unused]] u32 v_lane_off8[D_BLOCKS];
			{
				u32 const t = lane % 16, dh = (lane / 16) % 2;
				X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
					v_lane_off[db] = v_granule_offset(4 * half + (t >> 2), 2 * db + dh) + 8 * (t & 3);
					v_lane_off8[db] = v_granule_offset(8 + 4 * half + (t >> 2), 2 * db + dh) + 8 * (t & 3);
				}
			}
			u32 k_lane_off[K_SLICES];
			X17_UNROLL for (u32 sl = 0; sl < K_SLICES; ++sl) k_lane_off[sl] = k_chunk_offset(qlane, 2 * sl + half);

			auto compute = [&]<bool MASKED, int SLOT>(u32 i) __attribute__((always_inline)) {
				u32 const k_slot = SLOT >= 0 ? (u32)SLOT : i % at::RING;
				u32 const v_slot = SLOT >= 0 ? (u32)SLOT & 1u : i & 1u;
				u8 const *k_tile = smem + at::K_RING_OFFSET + k_slot * at::K_TILE_BYTES;
				u8 const *v_tile = smem + at::V_TILES_OFFSET + v_slot * at::V_TILE_BYTES;
				v16i s_acc = s_bias;
				X17_UNROLL for (u32 sl = 0; sl < K_SLICES; ++sl) {
					v4i kf = *reinterpret_cast<v4i const *>(k_tile + k_lane_off[sl]);
					s_acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[sl], s_acc, 0, 0, 0);
				}
				widen_next.template operator()<SLOT>(i);      // (behind the matrix instructions, whose results are not ready yet)
				X17_UNROLL for (u32 tile = 0; tile < 2; ++tile) {
					f32 y[8];
					[[maybe_unused]] bool vis[8];
					f32 tmax;
					// row-scaled build: this lane's 8 keys of the tile are 4 * half + {0..3} and 8 + 4 * half + {0..3}
					[[maybe_unused]] f32 const *sc = nullptr;
					[[maybe_unused]] f32 z[8];
					if constexpr (ROW_SCALES) {
						sc = reinterpret_cast<f32 const *>(smem + at::SCALE_RING_OFFSET + k_slot * at::SCALE_TILE_BYTES) + 16 * tile + 4 * half;
						v4f const k0 = *reinterpret_cast<v4f const *>(sc), k1 = *reinterpret_cast<v4f const *>(sc + 8);
						X17_UNROLL for (u32 r = 0; r < 4; ++r) {
							z[r] = f32(s_acc[8 * tile + r]) * k0[r];
							z[4 + r] = f32(s_acc[8 * tile + 4 + r]) * k1[r];
						}
					}
					if constexpr (!MASKED && ROW_SCALES) {
						// (non-negative temperature: sgn = 1)
						X17_UNROLL for (u32 r = 0; r < 8; ++r) y[r] = z[r];
						tmax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(y[0], y[1]), __builtin_fmaxf(y[2], y[3])),
						                       __builtin_fmaxf(__builtin_fmaxf(y[4], y[5]), __builtin_fmaxf(y[6], y[7])));
					} else if constexpr (!MASKED) {
						// (positive temperature: sgn = 1; the biased scores are positive floats: their order is the order
						// of their bits as integers)
						X17_UNROLL for (u32 r = 0; r < 8; ++r) y[r] = u2f((u32)s_acc[8 * tile + r]);
						i32 const *a = reinterpret_cast<i32 const *>(&s_acc) + 8 * tile;
						auto mx = [](i32 x, i32 y) { return x > y ? x : y; };
						i32 const imax = mx(mx(mx(mx(mx(mx(mx(a[0], a[1]), a[2]), a[3]), a[4]), a[5]), a[6]), a[7]);     // four max3-type operations
						tmax = u2f((u32)imax);
					} else {
						u32 const key0 = (kb_begin + i) * at::KV_PER_STEP;
						u32 const first = qi - 1 - (key0 + 16 * tile + 4 * half);
						f32 ym[8];
						X17_UNROLL for (u32 r = 0; r < 8; ++r) {
							u32 const distance = first - (8 * (r / 4) + (r % 4));
							vis[r] = distance <= vis_bound;
							y[r] = ROW_SCALES ? z[r] * sgn : u2f((u32)s_acc[8 * tile + r]) * sgn;
							ym[r] = vis[r] ? y[r] : -__builtin_inff();
						}
						tmax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(ym[0], ym[1]), __builtin_fmaxf(ym[2], ym[3])),
						                       __builtin_fmaxf(__builtin_fmaxf(ym[4], ym[5]), __builtin_fmaxf(ym[6], ym[7])));
					}
					if (__any(tmax > ext)) {
						if constexpr (!MASKED && !ROW_SCALES) {
							tmax = u2f((u32)pair_max_i32((i32)f2u(tmax)));
						} else {
							tmax = __builtin_fmaxf(tmax, partner_f32(tmax, half));
						}
						ext = tmax > ext ? tmax : ext;
						set_subtrahend();
						lift = hw::ex2(fmaf32(ext - ext_ref, abs_t, -HEADROOM));      // (the difference is exact)
						if (__any(lift > MAX_LIFT)) {
							// O and the partial sums come down to the scale of the new maximum
							f32 const down = hw::rcp(lift) * LIFT0;
							X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
								X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] * down;
							}
							sum_lo = sum_lo * down;
							sum_hi = sum_hi * down;
							ext_ref = ext;
							lift = LIFT0;
						}
						lift2 = v2h{(_Float16)lift, (_Float16)lift};      // round to nearest
						neg_bias2 = lift2 * v2h{(_Float16)-1024.0f, (_Float16)-1024.0f};     // exact
						sum_lift = lift * fine;
					}
					f32 p[8];
					X17_UNROLL for (u32 r = 0; r < 8; ++r) {
						f32 const arg = fmaf32(y[r], abs_t, -mb);       // lg2 of 255 * 2^(score - maximum)
						if constexpr (!MASKED) {
							p[r] = hw::ex2(arg);
						} else {
							p[r] = hw::ex2(vis[r] ? arg : -__builtin_inff());
						}
					}
					sum_lo = fmaf32((p[0] + p[1]) + (p[2] + p[3]), sum_lift, sum_lo);
					sum_hi = fmaf32((p[4] + p[5]) + (p[6] + p[7]), sum_lift, sum_hi);
					v4u pp;
					[[maybe_unused]] f32 vw[8];
					if constexpr (ROW_SCALES) {
						v4f const w0 = *reinterpret_cast<v4f const *>(sc + 32), w1 = *reinterpret_cast<v4f const *>(sc + 40);
						X17_UNROLL for (u32 r = 0; r < 4; ++r) { vw[r] = w0[r]; vw[4 + r] = w1[r]; }
					}
					X17_UNROLL for (int w = 0; w < 4; ++w) {
						f32 const f_lo = ROW_SCALES ? vw[2 * w] : fine, f_hi = ROW_SCALES ? vw[2 * w + 1] : fine;
						u32 const lo16 = f2u(fmaf32(p[2 * w], f_lo, PACK_MAGIC)), hi16 = f2u(fmaf32(p[2 * w + 1], f_hi, PACK_MAGIC));
						u32 const pair = __builtin_amdgcn_perm(hi16, lo16, 0x05040100u);           // f16 (1024 + P) twice
						pp[w] = __builtin_bit_cast(u32, __builtin_elementwise_fma(__builtin_bit_cast(v2h, pair), lift2, neg_bias2));
					}
					v8h const pfrag = __builtin_bit_cast(v8h, pp);
					X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
						// (a key's granules fill whole lines of CPR * 32 bytes: 16 keys = one tile further, 8 keys = the other group)
						u8 const *p0 = v_tile + v_lane_off[db] + tile * (16 * CPR * 32);
						u8 const *p1 = CPR >= 4 ? p0 + 8 * CPR * 32 : v_tile + v_lane_off8[db] + tile * (16 * CPR * 32);
						v4s const lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p0);
						v4s const hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p1);
						typedef short v8s __attribute__((ext_vector_type(8)));
						v8s const both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
						o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, both), pfrag, o_acc[db], 0, 0, 0);
					}
				}
			};
			auto step = [&]<bool MASKED, int SLOT>(u32 i) __attribute__((always_inline)) {
				stage.template operator()<SLOT>(i);
				compute.template operator()<MASKED, SLOT>(i);
			};
			auto idle_step = [&](u32 i) __attribute__((always_inline)) {
				stage.template operator()<-1>(i);
				widen_next.template operator()<-1>(i);
			};

			__syncthreads();                      // previous head's tiles are no longer read
			// (every workgroup walks at least four tiles: 0 .. 3 exist)
			if (CPR == 8 || stager) {
				load_to_lds_16(smem + at::RAW_V_RING_OFFSET + stage_lds, src, stage_v_src);
				X17_UNROLL for (u32 j = 0; j < 3; ++j) {
					if constexpr (ROW_SCALES) {
						X17_REQUEST_SCALES(j)
						sc_src += at::KV_PER_STEP;
					}
					load_to_lds_16(smem + at::K_RING_OFFSET + j * at::K_TILE_BYTES + stage_lds, src + j * TILE_STEP_BYTES, stage_k_src);
					load_to_lds_16(smem + at::RAW_V_RING_OFFSET + (j + 1) * at::RAW_V_TILE_BYTES + stage_lds, src + j * TILE_STEP_BYTES, stage_v_next);
				}
			}
			src += 3 * TILE_STEP_BYTES;
			if (ROW_SCALES && wave == 0) {
				__builtin_amdgcn_s_waitcnt(0x0F79);   // vmcnt(9): raw V tile 0 has landed (three loads per later tile)
			} else {
				__builtin_amdgcn_s_waitcnt(0x0F76);   // vmcnt(6): raw V tile 0 has landed
			}
			widen_v(0, 0);
			u32 i = 0;
			for (; i < first_active; ++i) idle_step(i);
			for (; i < first_full; ++i) step.template operator()<true, -1>(i);
			// the fully visible run: single steps up to a multiple of the ring, whole rings, single steps again
			for (; i < diagonal && i % at::RING != 0; ++i) step.template operator()<false, -1>(i);
			static_assert(at::RING == 4 && at::PREFETCH == 3, "the run below and the requests are written out for rings of four");
			for (; i + at::RING <= diagonal && i + 2 * at::RING <= n_steps; i += at::RING) {
				step.template operator()<false, 0>(i);
				step.template operator()<false, 1>(i + 1);
				step.template operator()<false, 2>(i + 2);
				step.template operator()<false, 3>(i + 3);
			}
			for (; i < diagonal; ++i) step.template operator()<false, -1>(i);
			step.template operator()<true, -1>(i);
			for (++i; i < n_steps; ++i) idle_step(i);
			__builtin_amdgcn_s_waitcnt(0x0F70);   // the last requests write LDS: they land before the tiles are reused
			// the partial sums are at the scale of the maximum HEADROOM above ext_ref's score: the common ending below
			// takes them as if that were the maximum (sgn * ext_ref - 12582912 is that extreme's dot product, exactly)
			m = ROW_SCALES ? fmaf32(ext_ref * sgn, temperature, HEADROOM) : fmaf32(fmaf32(ext_ref, sgn, -DOT_BIAS), temperature, HEADROOM);
			lift = 1.0f;
		} else {
		// ---- pipeline prologue
		__syncthreads();                      // previous head's tiles are no longer read
		X17_UNROLL for (u32 j = 0; j < at::PREFETCH; ++j) {
			if (j < n_steps) issue_kv_load(kb_begin + j, j);
		}
		wait_steps_in_flight((n_steps < at::PREFETCH ? n_steps : at::PREFETCH) - 1);
		widen_v(0, 0);

		for (u32 i = 0; i < n_steps; ++i) {
			u32 const kb = kb_begin + i;
			u32 const slot = i % at::RING;
			// K tile i and raw V tile i+1 have landed (this thread's chunks), at most step i+2 stays in flight
			wait_steps_in_flight(i + 2 < n_steps ? 1 : 0);
			__builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0): own LDS traffic of step i-1 is complete
			__builtin_amdgcn_s_barrier();                // ... and so is everybody else's: tiles i are visible
			if (i + at::PREFETCH < n_steps) {
				issue_kv_load(kb + at::PREFETCH, (i + at::PREFETCH) % at::RING);
			}
			if (i + 1 < n_steps) {
				widen_v((i + 1) % at::RING, (i + 1) & 1);
			}

			if (kb >= wave_kb_first && kb <= wave_kb_last) {
				u8 const *k_tile = smem + at::K_RING_OFFSET + slot * at::K_TILE_BYTES;
				u8 const *v_tile = smem + at::V_TILES_OFFSET + (i & 1) * at::V_TILE_BYTES;

				// S^T block: rows = 32 keys, columns = this wave's 32 queries
				v16i s_acc = {0};
				X17_UNROLL for (u32 s = 0; s < K_SLICES; ++s) {
					v4i kf = *reinterpret_cast<v4i const *>(k_tile + k_chunk_offset(qlane, 2 * s + half));
					s_acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[s], s_acc, 0, 0, 0);
				}

				u32 const key0 = kb * at::KV_PER_STEP;
				// fully visible for all 32 queries of the wave?  (cuda/attn_fwd_i8.cuh:540-567)
				bool const need_mask = !(key0 + 31 < q_wave0 && (q_wave0 + 31 - key0) <= wr);

				X17_UNROLL for (u32 tile = 0; tile < 2; ++tile) {
					// Speed build, tile fully visible, positive temperature: the row maximum is taken over the
					// integer dots (the scaling is monotone, so f32(max) * temperature IS the maximum score) and
					// the scaling is fused into the exponent's subtraction further down.
					bool const int_path = !STRICT && !ROW_SCALES && !need_mask && positive_temperature;
					f32 s[8];
					f32 tmax;
					// row-scaled build: this lane's 8 keys of the tile are 4 * half + {0..3} and 8 + 4 * half + {0..3}
					[[maybe_unused]] f32 key_scale[8];
					[[maybe_unused]] f32 value_weight[8];
					if constexpr (ROW_SCALES) {
						f32 const *sc = reinterpret_cast<f32 const *>(smem + at::SCALE_RING_OFFSET + slot * at::SCALE_TILE_BYTES)
						                + 16 * tile + 4 * half;
						v4f k0 = *reinterpret_cast<v4f const *>(sc), k1 = *reinterpret_cast<v4f const *>(sc + 8);
						v4f w0 = *reinterpret_cast<v4f const *>(sc + 32), w1 = *reinterpret_cast<v4f const *>(sc + 40);
						X17_UNROLL for (int r = 0; r < 4; ++r) {
							key_scale[r] = k0[r]; key_scale[4 + r] = k1[r];
							value_weight[r] = w0[r]; value_weight[4 + r] = w1[r];
						}
					}
					if (int_path) {
						i32 const *a = reinterpret_cast<i32 const *>(&s_acc) + 8 * tile;
						auto mx = [](i32 x, i32 y) { return x > y ? x : y; };     // pairs of these become v_max3_i32
						i32 imax = mx(mx(mx(a[0], a[1]), mx(a[2], a[3])), mx(mx(a[4], a[5]), mx(a[6], a[7])));
						i32 other = partner_i32(imax, half);
						imax = imax > other ? imax : other;
						tmax = f32(imax) * temperature;
					} else {
						if constexpr (ROW_SCALES) {
							X17_UNROLL for (u32 r = 0; r < 8; ++r) s[r] = (f32(s_acc[8 * tile + r]) * key_scale[r]) * temperature;
						} else {
							X17_UNROLL for (u32 r = 0; r < 8; ++r) s[r] = f32(s_acc[8 * tile + r]) * temperature;
						}
						if (need_mask) {
							// key j is visible iff j < qi and qi - j <= wr, i.e. iff the distance qi - 1 - j, taken as an
							// unsigned number, is at most wr - 1 (a key at or behind the query wraps to a huge distance;
							// the bound is capped at 2^31 - 1 so that an unlimited window cannot meet it)
							u32 const first = qi - 1 - (key0 + 16 * tile + 4 * half);
							X17_UNROLL for (u32 r = 0; r < 8; ++r) {
								u32 const distance = first - (8 * (r / 4) + (r % 4));
								s[r] = distance <= vis_bound ? s[r] : -__builtin_inff();
							}
						}
						f32 lmax = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(s[0], s[1]), __builtin_fmaxf(s[2], s[3])),
						                           __builtin_fmaxf(__builtin_fmaxf(s[4], s[5]), __builtin_fmaxf(s[6], s[7])));
						tmax = __builtin_fmaxf(lmax, partner_f32(lmax, half));
					}

					// cuda/attn_fwd_i8.cuh:233-256 -- rescale only when some row's max grew
					f32 resc = 1.0f;
					if (__any(tmax > m)) {
						f32 new_m = __builtin_fmaxf(tmax, m);
						resc = sfu::ex2(m - new_m);      // exactly 1 for rows whose max did not move
						m = new_m;
						if constexpr (STRICT) {
							X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
								X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] * resc;
							}
						} else {
							// Speed build: O stays at the scale of an older maximum m_ref and the new probabilities are
							// lifted to that scale instead (8 values instead of the 2 * head_dim / 4 accumulators);
							// O is brought down only when the lift factor 2^(m - m_ref) of some query passes 64.
							lift = sfu::ex2(m - m_ref);
							if (__any(lift > MAX_LIFT)) {
								f32 const down = sfu::rcp(lift);
								X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
									X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] * down;
								}
								m_ref = m;
								lift = 1.0f;
							}
							lift2 = v2h{(_Float16)lift, (_Float16)lift};      // round to nearest
						}
					}

					// :265-290 -- p = ex2(s - max) * 255; partial sums over key quads; P = rne(p)
					f32 p[8];
					if constexpr (STRICT) {
						X17_UNROLL for (u32 r = 0; r < 8; ++r) p[r] = sfu::ex2(s[r] - m) * PROB_SCALE;
					} else {
						f32 const shift = m - LOG2_PROB_SCALE;        // 255 * 2^(s - m) = 2^(s - (m - lg2 255))
						if (int_path) {
							X17_UNROLL for (u32 r = 0; r < 8; ++r) {
								p[r] = sfu::ex2(fmaf32(f32(s_acc[8 * tile + r]), temperature, -shift));
							}
						} else {
							X17_UNROLL for (u32 r = 0; r < 8; ++r) p[r] = sfu::ex2(s[r] - shift);
						}
					}
					f32 add_lo = (p[0] + p[1]) + (p[2] + p[3]);
					f32 add_hi = (p[4] + p[5]) + (p[6] + p[7]);
					sum_lo = fmaf32(sum_lo, resc, add_lo);
					sum_hi = fmaf32(sum_hi, resc, add_hi);

					if constexpr (ROW_SCALES) {
						// the numerator takes the probabilities at the value rows' relative scales
						X17_UNROLL for (u32 r = 0; r < 8; ++r) p[r] = p[r] * value_weight[r];
					}
					v4u pp;
					X17_UNROLL for (int w = 0; w < 4; ++w) {
						u32 word = pack_f16(__builtin_rintf(p[2 * w]), __builtin_rintf(p[2 * w + 1]));
						if constexpr (!STRICT) {
							// integers up to 255 times a factor up to 64: in range, rounded to 11 bits
							// (bit-casting a vector ELEMENT in place reads element 0, hence the scalar temporary)
							word = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, word) * lift2);
						}
						pp[w] = word;
					}
					v8h const pfrag = __builtin_bit_cast(v8h, pp);

					// :588-605 -- O += f32(P . V) for this 16-key tile
					X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
						// V^T operand: lane = dim 32*db + lane%32, slots = keys 16*tile + {4*half..+3, 8+4*half..+3}
						u32 t = lane % 16;
						u32 dh = (lane / 16) % 2;
						v4s lo4, hi4;
						{
							u32 key = 16 * tile + 4 * half + (t >> 2);
							u8 const *p0 = v_tile + v_granule_offset(key, 2 * db + dh) + 8 * (t & 3);
							u8 const *p1 = v_tile + v_granule_offset(key + 8, 2 * db + dh) + 8 * (t & 3);
							lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p0);
							hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p1);
						}
						typedef short v8s __attribute__((ext_vector_type(8)));
						v8s both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
						v8h const vfrag = __builtin_bit_cast(v8h, both);
						if constexpr (STRICT) {
							v16f zero = {0};
							v16f pv = __builtin_amdgcn_mfma_f32_32x32x16_f16(vfrag, pfrag, zero, 0, 0, 0);
							X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = o_acc[db][r] + pv[r];
						} else {
							o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vfrag, pfrag, o_acc[db], 0, 0, 0);
						}
					}
				}
			}

		}
		}

		// ---- finish (cuda/attn_fwd_i8.cuh:293-351): the lane pair holds partial sums (s0, s2) and (s1, s3)
		f32 other_lo = partner_f32(sum_lo, half);
		f32 other_hi = partner_f32(sum_hi, half);
		f32 s0 = half == 0 ? sum_lo : other_lo;
		f32 s1 = half == 0 ? other_lo : sum_lo;
		f32 s2 = half == 0 ? sum_hi : other_hi;
		f32 s3 = half == 0 ? other_hi : sum_hi;
		f32 total = (s0 + s1) + (s2 + s3);
		if (l_out != nullptr && half == 0) {
			l_out[(size_t)head * ((size_t)gridDim.z * seq_len) + row_base + qi] = sfu::lg2(total) + m;
		}
		f32 inv = sfu::rcp(total);
		if constexpr (!STRICT) {
			inv = inv * sfu::rcp(lift);
		}
#if X17_ATTN_ROW_SCALES
		f32 const head_out_scale = out_scale[head];
		if constexpr (OUT_BF16) {
			u16 *o_row = reinterpret_cast<u16 *>(out) + (row_base + qi) * O_STRIDE + (size_t)head * HD;
			X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
				X17_UNROLL for (int g = 0; g < 4; ++g) {
					f32 b[4];
					X17_UNROLL for (int e = 0; e < 4; ++e) b[e] = (o_acc[db][4 * g + e] * inv) * head_out_scale;
					v2u pair = {pack2_bf16_rne(b[0], b[1]), pack2_bf16_rne(b[2], b[3])};
					*reinterpret_cast<v2u *>(o_row + 32 * db + 8 * g + 4 * half) = pair;
				}
			}
			continue;
		}
		X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
			X17_UNROLL for (int r = 0; r < 16; ++r) o_acc[db][r] = (o_acc[db][r] * inv) * head_out_scale;
		}
		inv = 1.0f;          // exact: the stores below multiply by it once more
#endif
		i8 *o_row = out + (row_base + qi) * O_STRIDE + (size_t)head * HD;
		X17_UNROLL for (u32 db = 0; db < D_BLOCKS; ++db) {
			// word g of this lane = dims 32*db + 8*g + 4*half .. +3
			u32 word[4];
			X17_UNROLL for (int g = 0; g < 4; ++g) {
				if constexpr (STRICT) {
					word[g] = pack4_fixedi8(o_acc[db][4 * g] * inv, o_acc[db][4 * g + 1] * inv,
					                        o_acc[db][4 * g + 2] * inv, o_acc[db][4 * g + 3] * inv);
				} else {
					// the scaling rides in the rounding addition; clamping the rounded value gives what rounding the
					// clamped one gives
					constexpr f32 MAGIC = 12582912.0f;
					u32 u[4];
					X17_UNROLL for (int e = 0; e < 4; ++e) {
						u[e] = f2u(__builtin_amdgcn_fmed3f(fmaf32(o_acc[db][4 * g + e], inv, MAGIC), MAGIC - 127.0f, MAGIC + 127.0f));
					}
					word[g] = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u) | __builtin_amdgcn_perm(u[3], u[2], 0x04000c0cu);
				}
			}
			// The lane pair (lane, lane + 32) holds the 32 bytes of this block interleaved word by word; two
			// cross-half swaps give the lower lane bytes 0..15 and the upper lane bytes 16..31, so that each
			// lane writes one 16-byte vector.
			auto a = __builtin_amdgcn_permlane32_swap(word[0], word[2], false, false);
			auto b = __builtin_amdgcn_permlane32_swap(word[1], word[3], false, false);
			v4u vec = {a[0], a[1], b[0], b[1]};
			*reinterpret_cast<v4u *>(o_row + 32 * db + 16 * half) = vec;
		}
	}
}
