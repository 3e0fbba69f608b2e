// attn_decode_i8.hip -- single-token attention against an int8 KV cache, for gfx950.
//
// The reference has no int8 decode kernel (its TODO.md:10-12 defers ragged tails to "the
// incremental kernel"; attn_incremental.cu is the bf16 precedent for queries appended to a
// longer KV).  This kernel is DEFINED as the prefill recurrence of cuda/attn_fwd_i8.cuh:368-619
// for ONE query per sequence, at position cache_len[s], against cache rows [0, cache_len[s]):
// same window rounding, same n = min(W', p) + 4, same 16-key tiles aligned at absolute
// positions, same per-tile max / rescale / u8 probabilities / four partial sums / one f32 add
// of the int32 P.V per tile.  So appending a token and decoding it gives bit for bit what a
// prefill over the longer sequence gives for that row.
//
// The work is bandwidth: every cached K byte is read exactly once, and so is every V row whose
// 8-bit probability is not zero (rows with probability 0 contribute nothing and are not fetched).  One workgroup
// of two wavefronts per (sequence, head), small enough in registers and LDS that eight share a compute unit:
// all workgroups of 64 sequences x 32 heads are then resident together and the key stream runs without a
// second, half-empty round.  The recurrence is cut into phases so that only two cheap scans remain
// sequential:
//   1  scores: HD/16 lanes per key row (16-byte coalesced loads), v_dot4 + lane reduction
//   2  per-tile max, prefix max over tiles (exact), rescale factors, probabilities, quad sums
//   3  four partial-sum chains (4 lanes)
//   4  P.V partials per tile in int32 (every lane, 16 dims x 16 keys), then one lane per output
//      dim runs the O = O * rescale + f32(partial) chain over the tiles
//
// common.h provides X17_N_HEADS, X17_HEAD_DIM, X17_CACHE_CAPACITY, X17_STRICT_MATH.
// Layouts: q, out [S, H*hd]; cache [S, CAPACITY, H*2*hd] (per head K then V, as kv of the
// prefill kernel); cache_len u32 [S]; L [S, H] or null.
//
// X17_ATTN_ROW_SCALES = 1: the row-scaled recurrence of attn_fwd_i8.hip for the one query -- q_scale
// [S, H], k_scale and v_weight [S, H, CAPACITY], sink_v_weight and out_scale [H]; X17_ATTN_OUT_BF16 = 1
// writes bf16 real values.  Only visible rows' scales are read (the rest of a cache may be uninitialised).

#include "common.h"
#include "x17_device.h"
#include "decode_tile.h"

using namespace x17;
namespace dt = x17::decode_tile;

namespace {
constexpr u32 HD = X17_HEAD_DIM;
constexpr u32 N_HEADS = X17_N_HEADS;
constexpr u32 CAP = X17_CACHE_CAPACITY;
constexpr u32 CPR = HD / 16;                         // lanes per key row
constexpr u32 ROW = 2 * N_HEADS * HD;                // bytes per cache row
constexpr u32 KEYS_PER_PASS = dt::THREADS_PER_BLOCK / CPR;
#ifndef X17_ATTN_ROW_SCALES
#define X17_ATTN_ROW_SCALES 0
#endif
#ifndef X17_ATTN_OUT_BF16
#define X17_ATTN_OUT_BF16 0
#endif
constexpr bool ROW_SCALES = X17_ATTN_ROW_SCALES != 0;
constexpr bool OUT_BF16 = X17_ATTN_OUT_BF16 != 0;
static_assert(ROW_SCALES || !OUT_BF16, "the bf16 output needs the row-scaled build (it supplies out_scale)");
constexpr f32 BASE_TEMPERATURE = ROW_SCALES ? f32(constexpr_inv_sqrt(f64(HD))) : f32(constexpr_inv_sqrt(f64(HD)) / 64.0);
static_assert(HD == 32 || HD == 64 || HD == 128, "head_dim must be 32, 64 or 128");
static_assert(CAP % 16 == 0, "cache capacity must be a multiple of 16");
static_assert(dt::CHUNK_TILES * CPR == dt::THREADS_PER_BLOCK, "one thread per (tile, 16-dim group) of a chunk");
static_assert(HD <= dt::THREADS_PER_BLOCK, "one thread per output dimension");

// LDS slot of key quad `quad` (16 bytes): four f32 scores, later {partial sum, packed probabilities, free, free}
X17_DEV u8 *quad_slot(u8 *smem, u32 quad) { return smem + 16 * quad; }
// int32 P.V partial of (chunk tile tl, dim d): in the free half of a slot, or in a region of its own.  Word e lives
// in slot e / 2; the slots of one 16-dim group are permuted by the group's index so that the group-wise writes of
// a wavefront spread over the LDS banks.
X17_DEV i32 *pv_word(u8 *smem, u32 tl, u32 d) {
	if constexpr (dt::PV_IN_SLOTS) {
		u32 const group = d >> 4;
		u32 const slot = tl * (HD / 2) + 8 * group + (((d >> 1) & 7) ^ (group & 7));
		return reinterpret_cast<i32 *>(smem + 16 * slot + 8 + 4 * (d & 1));
	} else {
		return reinterpret_cast<i32 *>(smem + dt::PV_OFFSET) + tl * HD + d;
	}
}
}

extern "C" __global__ __launch_bounds__(dt::THREADS_PER_BLOCK)
void kernel(
	i8 const *q, i8 const *cache, u32 const *cache_len,
	i8 const *sink_k, i8 const *sink_v, f32 const *attn_temperature,
	i8 *out, f32 *l_out, u32 window_size
#if X17_ATTN_ROW_SCALES
	,
	f32 const *q_scale, f32 const *k_scale, f32 const *v_weight, f32 const *sink_v_weight, f32 const *out_scale
#endif
) {
	extern __shared__ __attribute__((aligned(16))) u8 smem[];
	f32 *s_score = reinterpret_cast<f32 *>(smem);                               // [CAP], quad slots (see quad_slot)
	f32 *s_mrun = reinterpret_cast<f32 *>(smem + dt::TILE_STATE_OFFSET);         // [MAX_TILES] tile max, then running max
	f32 *s_tmax = s_mrun;
	f32 *s_resc = s_mrun + dt::MAX_TILES;                                        // [MAX_TILES]
	f32 *s_bmax = s_resc + dt::MAX_TILES;                                        // [4] one per wavefront
	f32 *s_sum = s_bmax + 4;                                                     // [4]
	u32 *s_nact = reinterpret_cast<u32 *>(s_sum + 4);                            // [4] (one used)
	u16 *s_act = reinterpret_cast<u16 *>(s_nact + 4);                            // [MAX_TILES] tiles that move O

	u32 const tid = threadIdx.x;
	u32 const head = blockIdx.x;
	u32 const seq = blockIdx.y;
	u32 const pos_raw = cache_len[seq];                  // the query's position; keys are rows < pos
	u32 const pos = pos_raw < CAP ? pos_raw : CAP;       // never read past the cache
	u32 const wr = window_size == 0 ? 0xFFFFFFFFu : ((window_size - 1) / 16 + 1) * 16;
	u32 const visible = pos < wr ? pos : wr;
	u32 const j_lo = pos - visible;
	u32 const t0 = j_lo / 16;
	u32 const n_tiles = visible == 0 ? 0 : (pos - 1) / 16 - t0 + 1;

	i8 const *kv_head = cache + (size_t)seq * CAP * ROW + (size_t)head * 2 * HD;
	i8 const *q_head = q + (size_t)seq * N_HEADS * HD + (size_t)head * HD;

	f32 temperature = BASE_TEMPERATURE * strict::lg2(f32(visible + 4u));
	temperature = temperature * attn_temperature[head];
#if X17_ATTN_ROW_SCALES
	temperature = temperature * q_scale[(size_t)seq * N_HEADS + head];
	f32 const *k_scale_head = k_scale + ((size_t)seq * N_HEADS + head) * CAP;     // indexed by cache row
	f32 const *v_weight_head = v_weight + ((size_t)seq * N_HEADS + head) * CAP;
#endif

	// this lane's 16 bytes of the query (chunk tid % CPR)
	u32 const c = tid % CPR;
	v4i const qc = *reinterpret_cast<v4i const *>(q_head + 16 * c);

	// sink score (every group of CPR lanes computes it)
	i32 sink_dot = 0;
	{
		v4i sk = *reinterpret_cast<v4i const *>(sink_k + (size_t)head * HD + 16 * c);
		X17_UNROLL for (int w = 0; w < 4; ++w) sink_dot = __builtin_amdgcn_sdot4(qc[w], sk[w], sink_dot, false);
		X17_UNROLL for (u32 mask = 1; mask < CPR; mask <<= 1) sink_dot += __shfl_xor(sink_dot, (int)mask, 64);
	}
	f32 const m0 = ROW_SCALES ? f32(sink_dot) * (temperature * 0.125f) : f32(sink_dot) * temperature;

	// ---- phase 1: scores of all keys of the walked tiles.  A thread keeps BATCH independent 16-byte
	// loads in flight (a load per pass would leave the kernel waiting on memory latency).
	u32 const n_keys = n_tiles * 16;
	// Few loads per thread and many resident workgroups: the workgroups of one sequence then walk its rows nearly
	// in step, which the DRAM pages like (measured: 2 loads in flight per thread beat 1, 4, 8 and 16).
#ifndef X17_DECODE_BATCH
#define X17_DECODE_BATCH 2
#endif
	constexpr u32 BATCH = X17_DECODE_BATCH;
	for (u32 base = 0; base < n_keys; base += KEYS_PER_PASS * BATCH) {
		v4i kc[BATCH];
		X17_UNROLL for (u32 bb = 0; bb < BATCH; ++bb) {
			u32 kidx = base + bb * KEYS_PER_PASS + tid / CPR;
			u32 j = t0 * 16 + kidx;
			bool vis = kidx < n_keys && j >= j_lo && j < pos;
			u32 j_safe = vis ? j : pos - 1;                   // a row that exists (n_tiles > 0 means pos >= 1)
			// every cache byte is read once: streaming (non-temporal) loads
			kc[bb] = __builtin_nontemporal_load(reinterpret_cast<v4i const *>(kv_head + (size_t)j_safe * ROW + 16 * c));
		}
		X17_UNROLL for (u32 bb = 0; bb < BATCH; ++bb) {
			u32 kidx = base + bb * KEYS_PER_PASS + tid / CPR;
			u32 j = t0 * 16 + kidx;
			bool in_range = kidx < n_keys;
			bool vis = in_range && j >= j_lo && j < pos;
			i32 dot = 0;
			X17_UNROLL for (int w = 0; w < 4; ++w) dot = __builtin_amdgcn_sdot4(qc[w], kc[bb][w], dot, false);
			X17_UNROLL for (u32 mask = 1; mask < CPR; mask <<= 1) dot += __shfl_xor(dot, (int)mask, 64);
			if (in_range && c == 0) {
				// (row-scaled build: the key's scale and the temperature are applied in a pass of their own below)
				f32 const score = ROW_SCALES ? f32(dot) : f32(dot) * temperature;
				s_score[kidx] = vis ? score : -__builtin_inff();
			}
		}
	}
	__syncthreads();
#if X17_ATTN_ROW_SCALES
	// the keys' scales, four per 16-byte load; masked keys keep -inf whatever their (possibly never written) scale
	for (u32 quad = tid; quad < n_tiles * 4; quad += dt::THREADS_PER_BLOCK) {
		v4f const ks = __builtin_nontemporal_load(reinterpret_cast<v4f const *>(k_scale_head + t0 * 16 + quad * 4));
		v4f sc = *reinterpret_cast<v4f const *>(s_score + quad * 4);
		X17_UNROLL for (int i = 0; i < 4; ++i) sc[i] = sc[i] == -__builtin_inff() ? sc[i] : (sc[i] * ks[i]) * temperature;
		*reinterpret_cast<v4f *>(s_score + quad * 4) = sc;
	}
	__syncthreads();
#endif

	// ---- phase 2a: per-tile max; each thread owns TPT consecutive tiles
	constexpr u32 TPT = (dt::MAX_TILES + dt::THREADS_PER_BLOCK - 1) / dt::THREADS_PER_BLOCK;
	f32 block_max = -__builtin_inff();
	X17_UNROLL for (u32 i = 0; i < TPT; ++i) {
		u32 t = tid * TPT + i;
		if (t < n_tiles) {
			f32 mx = -__builtin_inff();
			X17_UNROLL for (int k = 0; k < 16; k += 4) {
				v4f v = *reinterpret_cast<v4f const *>(s_score + t * 16 + k);
				mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fmaxf(v[0], v[1]), __builtin_fmaxf(v[2], v[3])));
			}
			s_tmax[t] = mx;
			block_max = __builtin_fmaxf(block_max, mx);
		}
	}
	// ---- phase 2b: running max before each thread's tiles (max is exact, so any grouping works): an
	// exclusive prefix maximum over the threads -- a shuffle scan inside each wavefront, the wavefront totals
	// through LDS -- then running max and rescale factor of every tile (cuda/attn_fwd_i8.cuh:233-256)
	f32 m_before;
	{
		u32 const lane = tid % 64;
		f32 incl = block_max;
		X17_UNROLL for (int d = 1; d < 64; d <<= 1) {
			f32 up = __shfl_up(incl, d, 64);
			if ((int)lane >= d) incl = __builtin_fmaxf(incl, up);
		}
		if (lane == 63) s_bmax[tid / 64] = incl;                  // this wavefront's maximum
		f32 excl = __shfl_up(incl, 1, 64);
		m_before = lane == 0 ? -__builtin_inff() : excl;
	}
	__syncthreads();
	{
		f32 m_prev = __builtin_fmaxf(m0, m_before);
		for (u32 w = 0; w < tid / 64; ++w) m_prev = __builtin_fmaxf(m_prev, s_bmax[w]);
		X17_UNROLL for (u32 i = 0; i < TPT; ++i) {
			u32 t = tid * TPT + i;
			if (t < n_tiles) {
				f32 tm = s_tmax[t];
				f32 resc = 1.0f;
				if (tm > m_prev) {
					resc = sfu::ex2(m_prev - tm);
					m_prev = tm;
				}
				s_mrun[t] = m_prev;
				s_resc[t] = resc;
			}
		}
	}
	__syncthreads();

	// ---- phase 2c: probabilities and quad sums (:265-290); one key quad per thread per pass
	for (u32 quad = tid; quad < n_tiles * 4; quad += dt::THREADS_PER_BLOCK) {
		f32 m = s_mrun[quad / 4];
		v4f s = *reinterpret_cast<v4f const *>(s_score + quad * 4);
		f32 p0 = sfu::ex2(s[0] - m) * 255.0f;
		f32 p1 = sfu::ex2(s[1] - m) * 255.0f;
		f32 p2 = sfu::ex2(s[2] - m) * 255.0f;
		f32 p3 = sfu::ex2(s[3] - m) * 255.0f;
		f32 const quad_sum = (p0 + p1) + (p2 + p3);
#if X17_ATTN_ROW_SCALES
		{
			// the numerator takes the probabilities at the value rows' relative scales; masked keys keep 0
			u32 const j = t0 * 16 + quad * 4;
			// (rows of a partly visible quad are inside the cache: its capacity is a multiple of 16)
			v4f const vw = __builtin_nontemporal_load(reinterpret_cast<v4f const *>(v_weight_head + j));
			p0 = s[0] == -__builtin_inff() ? 0.0f : p0 * vw[0];
			p1 = s[1] == -__builtin_inff() ? 0.0f : p1 * vw[1];
			p2 = s[2] == -__builtin_inff() ? 0.0f : p2 * vw[2];
			p3 = s[3] == -__builtin_inff() ? 0.0f : p3 * vw[3];
		}
#endif
		u32 packed = (u32)(i32)__builtin_rintf(p0) | ((u32)(i32)__builtin_rintf(p1) << 8)
			| ((u32)(i32)__builtin_rintf(p2) << 16) | ((u32)(i32)__builtin_rintf(p3) << 24);
		// in place: this thread has read its quad's scores, nobody else touches the slot
		*reinterpret_cast<v2u *>(quad_slot(smem, quad)) = v2u{f2u(quad_sum), packed};
	}
	__syncthreads();

	// ---- phase 3: the four partial-sum chains, one per lane of the first four, while the last wavefront lists the
	// tiles for phase 4.  The chain is serial; what costs time is fetching its operands from LDS, so they are
	// fetched 32 tiles at a time (the registers are free at this point) and the chain waits once per 32 steps.
	if (tid < 4) {
		constexpr u32 STEPS = 32;
		f32 sum = 63.75f;
		u32 t = 0;
		for (; t + STEPS <= n_tiles; t += STEPS) {
			v4f r[STEPS / 4];
			f32 a[STEPS];
			X17_UNROLL for (u32 i = 0; i < STEPS / 4; ++i) r[i] = *reinterpret_cast<v4f const *>(s_resc + t + 4 * i);
			X17_UNROLL for (u32 i = 0; i < STEPS; ++i) a[i] = *reinterpret_cast<f32 const *>(quad_slot(smem, (t + i) * 4 + tid));
			X17_UNROLL for (u32 i = 0; i < STEPS; ++i) sum = fmaf32(sum, r[i / 4][i % 4], a[i]);
		}
		for (; t < n_tiles; ++t) sum = fmaf32(sum, s_resc[t], *reinterpret_cast<f32 const *>(quad_slot(smem, t * 4 + tid)));
		s_sum[tid] = sum;
	}

	// ---- phase 4: O chains.  Lane d < HD owns output dim d.
	// A tile whose sixteen probabilities all rounded to zero and whose rescale factor is exactly 1 leaves O
	// untouched (O * 1 + 0), and after the first few tiles that is most of them: the last wave lists the
	// other tiles, in order, and only those are walked.
	if (tid >= dt::THREADS_PER_BLOCK - 64) {
		u32 const lane = tid % 64;
		u32 count = 0;
		for (u32 base = 0; base < n_tiles; base += 64) {
			u32 t = base + lane;
			bool active = false;
			if (t < n_tiles) {
				u32 any = 0;
				X17_UNROLL for (u32 k = 0; k < 4; ++k) any |= *reinterpret_cast<u32 const *>(quad_slot(smem, t * 4 + k) + 4);
				active = any != 0 || s_resc[t] != 1.0f;
			}
			unsigned long long const mask = __ballot(active);
			if (active) {
				s_act[count + __builtin_popcountll(mask & ((1ull << lane) - 1ull))] = (u16)t;
			}
			count += (u32)__builtin_popcountll(mask);
		}
		if (lane == 0) {
			s_nact[0] = count;
		}
	}
	__syncthreads();
	u32 const n_act = s_nact[0];

	f32 o = 0.0f;
	if (tid < HD) {
		o = f32((i32)sink_v[(size_t)head * HD + tid] * 255);
#if X17_ATTN_ROW_SCALES
		o = o * sink_v_weight[head];
#endif
	}
	// 4a: int32 P.V of one tile x 16 dims per thread.  The value rows of a chunk are requested (only rows with a
	// nonzero probability: masked keys have p == 0 and may lie outside the cache) while the previous chunk's chain
	// runs, so that a workgroup with many listed tiles waits for memory once, not once per chunk.
	u32 const tl = tid / CPR;
	u32 probs[4] = {0, 0, 0, 0};
	v4i vv[16];
	auto request_rows = [&](u32 chunk) {
		u32 const tiles_here = n_act - chunk < dt::CHUNK_TILES ? n_act - chunk : dt::CHUNK_TILES;
		if (tl < tiles_here) {
			u32 const t = s_act[chunk + tl];
			X17_UNROLL for (u32 k = 0; k < 4; ++k) probs[k] = *reinterpret_cast<u32 const *>(quad_slot(smem, t * 4 + k) + 4);
			X17_UNROLL for (int k = 0; k < 16; ++k) {
				u32 p = (probs[k / 4] >> (8 * (k % 4))) & 0xFFu;
				u32 j = (t0 + t) * 16 + k;
				vv[k] = v4i{0, 0, 0, 0};
				if (p != 0) {
					vv[k] = __builtin_nontemporal_load(reinterpret_cast<v4i const *>(kv_head + (size_t)j * ROW + HD + 16 * c));
				}
			}
		}
	};
	if (n_act > 0) {
		request_rows(0);
	}
	for (u32 chunk = 0; chunk < n_act; chunk += dt::CHUNK_TILES) {
		u32 const tiles_here = n_act - chunk < dt::CHUNK_TILES ? n_act - chunk : dt::CHUNK_TILES;
		if (tl < tiles_here) {
			i32 acc[16];
			X17_UNROLL for (int i = 0; i < 16; ++i) acc[i] = 0;
			X17_UNROLL for (int k = 0; k < 16; ++k) {
				i32 p = (i32)((probs[k / 4] >> (8 * (k % 4))) & 0xFFu);
				if (p != 0) {     // after the 8-bit quantisation most keys far below the maximum carry no weight
					X17_UNROLL for (int i = 0; i < 16; ++i) {
						acc[i] += p * (i32)(i8)(((u32)vv[k][i / 4] >> (8 * (i % 4))) & 0xFFu);
					}
				}
			}
			X17_UNROLL for (int i = 0; i < 16; i += 2) {
				*reinterpret_cast<v2i *>(pv_word(smem, tl, 16 * c + i)) = v2i{acc[i], acc[i + 1]};
			}
		}
		__syncthreads();
		if (chunk + dt::CHUNK_TILES < n_act) {
			request_rows(chunk + dt::CHUNK_TILES);
		}
		// 4b: one f32 multiply (rescale) and one f32 add per tile (:247-252, :588-605)
		if (tid < HD) {
			u32 tl2 = 0;
			for (; tl2 + 8 <= tiles_here; tl2 += 8) {
				f32 r[8];
				i32 a[8];
				X17_UNROLL for (int i = 0; i < 8; ++i) { r[i] = s_resc[s_act[chunk + tl2 + i]]; a[i] = *pv_word(smem, tl2 + i, tid); }
				X17_UNROLL for (int i = 0; i < 8; ++i) {
					o = o * r[i];
					o = o + f32(a[i]);
				}
			}
			for (; tl2 < tiles_here; ++tl2) {
				o = o * s_resc[s_act[chunk + tl2]];
				o = o + f32(*pv_word(smem, tl2, tid));
			}
		}
		__syncthreads();
	}

	// ---- finish (:293-351)
	__syncthreads();
	f32 const total = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
	f32 const m_final = n_tiles == 0 ? m0 : s_mrun[n_tiles - 1];
	if (tid == 0 && l_out != nullptr) {
		l_out[(size_t)seq * N_HEADS + head] = strict::lg2(total) + m_final;
	}
	if (tid < HD) {
		size_t const idx = (size_t)seq * N_HEADS * HD + (size_t)head * HD + tid;
#if X17_ATTN_ROW_SCALES
		f32 const value = (o * strict::rcp(total)) * out_scale[head];
		if constexpr (OUT_BF16) {
			reinterpret_cast<u16 *>(out)[idx] = (u16)f32_to_bf16_rne(value);
		} else {
			out[idx] = (i8)f32_to_fixedi8(value);
		}
#else
		out[idx] = (i8)f32_to_fixedi8(o * strict::rcp(total));
#endif
	}
}
