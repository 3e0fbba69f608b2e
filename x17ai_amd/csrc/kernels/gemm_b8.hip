// gemm_b8.hip -- C[M, N] = epilogue(A[M, K] . B[N_raw, K]^T) for 8-bit operands on gfx950.
//
// Replaces the reference's b8::Gemm (cuda/gemm_b8.cuh:624-755: i8 x i8 -> i32) and b16::Gemm
// (cuda/gemm_b16.cuh:436-567: any e4m3 operand, f32 accumulate) together with their four fused
// writers (Scaled :291-339, GeGlu :341-441, Residual :443-622, L2Norm :861-949).  The kernel
// entry and its parameters follow templates/basic_gemm/kernel.cu:9-32.
//
// Design, MI355X-first (nothing here is derived from the SM80 kernel):
//   * One workgroup = a 256 (tokens) x 256 (raw columns) output tile, by default 8 wavefronts of
//     64 x 128 (two per SIMD; gemm_tile.h can also build 4 wavefronts of 128 x 128); in the 4-wave form each
//     wavefront owns 128 x 128 as a 4 x 4 grid of 32x32 MFMA blocks (256 accumulator
//     registers per lane, one wavefront per SIMD).
//   * The WEIGHTS are the MFMA "A" operand and the TOKENS the "B" operand, i.e. the matrix
//     cores compute C^T.  A lane then owns one token and, per MFMA block, 16 output columns;
//     weight rows are permuted on their way into LDS so that those are 64 CONSECUTIVE
//     columns across the four blocks.  Gate/value pairs, whole K|V heads and 16-byte output
//     vectors all live inside one lane: the epilogues need no cross-lane shuffles (the SM80
//     code needs a 4x4 shuffle transpose per 32x32 tile, cuda/gemm_b8.cuh:411, 570, 592).
//   * Global -> LDS goes through the gfx950 16-byte direct-to-LDS load (no register staging),
//     K_STEP = 128 bytes per step, two stages, one barrier per step.  Rows are 128 bytes;
//     16-byte chunks are XOR-swizzled with the row-pair index so ds_read_b128 is conflict-free.
//   * int8: v_mfma_i32_32x32x32_i8.  e4m3 x e4m3: v_mfma_f32_32x32x64_f8f6f4.  Mixed
//     e4m3 x int8: both widened exactly to bf16 in registers, v_mfma_f32_32x32x16_bf16
//     (int8 codes need 7 significand bits, e4m3 has 4).
//   * Workgroup ids are remapped so that each XCD (own L2) works on a compact block of tiles.
//
// common.h (generated per kernel by the host-side kernel builder) provides:
//   X17_A_COLS (K), X17_B_ROWS (N_raw), X17_A_KIND / X17_B_KIND (0 = int8, 1 = e4m3),
//   X17_EPILOGUE (0 scale, 1 geglu, 2 residual, 3 l2norm), X17_STORE (0 FixedI8, 1 e4m3),
//   X17_INP_SCALE, X17_OUT_SCALE, and for l2norm X17_HEAD_DIM, X17_EPS, X17_HEAD_SCALE,
//   X17_SEP_SCALE (doubles), X17_STRICT_MATH.

#include "common.h"
#include "x17_device.h"
#include "gemm_tile.h"

using namespace x17;
namespace gt = x17::gemm_tile;

namespace {

constexpr u32 K_TOTAL = X17_A_COLS;
constexpr u32 N_RAW = X17_B_ROWS;
constexpr int A_KIND = X17_A_KIND;
constexpr int B_KIND = X17_B_KIND;
constexpr int EPILOGUE = X17_EPILOGUE;
constexpr int STORE = X17_STORE;

// 0: int8 MFMA, 1: fp8 MFMA, 2: bf16 MFMA after widening
constexpr int MMA = (A_KIND == 0 && B_KIND == 0) ? 0 : ((A_KIND == 1 && B_KIND == 1) ? 1 : 2);
constexpr bool ACC_F32 = MMA != 0;

static_assert(K_TOTAL % gt::K_STEP == 0, "K must be a multiple of 128");
static_assert(N_RAW % gt::N_PER_BLOCK == 0, "raw output columns must be a multiple of 256");

constexpr u32 ROW_BYTES = gt::K_STEP;                       // one LDS row = 128 bytes of K
constexpr u32 X_TILE_BYTES = gt::M_PER_BLOCK * ROW_BYTES;   // tokens
constexpr u32 W_TILE_BYTES = gt::N_PER_BLOCK * ROW_BYTES;   // weights
constexpr u32 STAGE_BYTES = X_TILE_BYTES + W_TILE_BYTES;
constexpr u32 K_STEPS = K_TOTAL / gt::K_STEP;

constexpr int BM = gt::WAVE_M / 32;                         // 32-token MFMA blocks per wave
constexpr u32 WAVES = gt::WAVES_M * gt::WAVES_N;
constexpr u32 ROWS_PER_WAVE = 256 / WAVES;                  // rows of each tile a wave copies per stage
constexpr u32 UNITS = ROWS_PER_WAVE / 8;                    // 8-row direct-to-LDS loads per wave and tile

using Acc = __attribute__((ext_vector_type(16))) int;       // raw 16 registers; reinterpreted as f32 when ACC_F32

// ------------------------------------------------------------------ epilogues
// Each receives, for ONE token row, 64 accumulators of 64 consecutive raw columns starting at
// raw column `n`, already converted to f32 (i32 -> f32 is the reference's implicit RNE cast).

// ScaledMatrixWriter, cuda/gemm_b8.cuh:291-339
struct ScaleEpilogue {
	static constexpr f64 SCALE = f64(X17_INP_SCALE) * f64(X17_OUT_SCALE);
	static constexpr u32 OUT_COLS = N_RAW;
	X17_DEV static void run(f32 const (&x)[64], u8 *c, u32 row, u32 n, void const *) {
		u8 *dst = c + (size_t)row * OUT_COLS + n;
		X17_UNROLL for (int v = 0; v < 4; ++v) {
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				u32 word = 0;
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					word |= store_convert<STORE>(x[16 * v + 4 * w + b] * f32(SCALE)) << (8 * b);
				}
				pack[w] = word;
			}
			*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
		}
	}
};

// GeGluMatrixWriter, cuda/gemm_b8.cuh:341-441 with math::fast::gelu, cuda/utils_core.cuh:426-448
struct GeGluEpilogue {
	static constexpr f64 I = X17_INP_SCALE;
	static constexpr f64 O = X17_OUT_SCALE;
	static constexpr f64 INP2 = I * I;
	static constexpr f64 OUT2 = INP2 * (O * O);
	static constexpr f64 KK = constexpr_sqrt(INP2);
	static constexpr f64 CK = constexpr_sqrt(INP2 * 2.0 * INV_PI);
	static constexpr f64 CK3 = 0.044715 * CK * INP2;
	static constexpr f64 Y = 0.5 * constexpr_sqrt(OUT2 * 1.0) * KK;
	static constexpr u32 OUT_COLS = N_RAW / 2;

	X17_DEV static f32 gate(f32 x) {
		f32 x2 = x * x;
		f32 s = fmaf32(f32(CK3) * x, x2, f32(CK) * x);
		f32 t = sfu::tanh(s);
		return fmaf32(f32(Y) * x, t, f32(Y) * x);
	}
	X17_DEV static void run(f32 const (&x)[64], u8 *c, u32 row, u32 n, void const *) {
		u8 *dst = c + (size_t)row * OUT_COLS + n / 2;
		X17_UNROLL for (int v = 0; v < 2; ++v) {
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				u32 word = 0;
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					int j = 16 * v + 4 * w + b;
					word |= store_convert<STORE>(gate(x[2 * j]) * x[2 * j + 1]) << (8 * b);
				}
				pack[w] = word;
			}
			*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
		}
	}
};

// ResidualMatrixWriter, cuda/gemm_b8.cuh:443-622; sigmoid_base4 / imprecise_softplus_base4,
// cuda/utils_core.cuh:397-405, 468-483
struct ResidualEpilogue {
	static constexpr f64 I = X17_INP_SCALE;
	static constexpr f64 O = X17_OUT_SCALE;
	static constexpr f64 SG_HALF = 0.5 * (1.0 / 8.0);
	static constexpr f64 SG_IN = LN2 * (-I);
	static constexpr f64 SP_INP = I;
	static constexpr f64 SP_OUT = I * O;
	static constexpr f32 SP_INP_SCALE = f32(SP_INP * 2.0);
	static constexpr f32 SP_OUT_SCALE = f32(SP_OUT / 2.0);
	static constexpr f32 SP_LINE = f32(SP_INP * SP_OUT);
	static constexpr u32 OUT_COLS = N_RAW / 2;

	X17_DEV static f32 mix(f32 g, f32 v, f32 r) {
		f32 old_w = fmaf32(f32(SG_HALF), sfu::tanh(f32(SG_IN) * g), f32(SG_HALF));
		f32 line = __builtin_fmaxf(0.0f, g);
		if constexpr (SP_LINE != 1.0f) {
			line = line * SP_LINE;
		}
		f32 new_w = fmaf32(sfu::lg2(1.0f + sfu::ex2(-__builtin_fabsf(g * SP_INP_SCALE))), SP_OUT_SCALE, line);
		return fmaf32(new_w, v, old_w * r);
	}
	X17_DEV static void run(f32 const (&x)[64], u8 *c, u32 row, u32 n, void const *extra) {
		size_t off = (size_t)row * OUT_COLS + n / 2;
		i8 const *res = reinterpret_cast<i8 const *>(extra) + off;
		u8 *dst = c + off;
		X17_UNROLL for (int v = 0; v < 2; ++v) {
			v4u rv = *reinterpret_cast<v4u const *>(res + 16 * v);
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				u32 word = 0;
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					int j = 16 * v + 4 * w + b;
					f32 r = f32((i32)(i8)((rv[w] >> (8 * b)) & 0xFFu));
					word |= store_convert<STORE>(mix(x[2 * j], x[2 * j + 1], r)) << (8 * b);
				}
				pack[w] = word;
			}
			*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
		}
	}
};

// The l2norm epilogue needs more than one lane for head_dim > 64 and is handled in the kernel body.
#if X17_EPILOGUE == 3
constexpr u32 HEAD_DIM = X17_HEAD_DIM;
static_assert(HEAD_DIM == 32 || HEAD_DIM == 64 || HEAD_DIM == 128, "head_dim must be 32, 64 or 128");
#endif

// ------------------------------------------------------------------ tile loads

// LDS rows are 128 bytes = 8 chunks of 16; logical chunk c of row r is stored at position
// c ^ ((r >> 1) & 7).  The LDS has 64 four-byte banks and serves a ds_read_b128 sixteen lanes at a
// time, so sixteen consecutive rows (two per 256-byte bank line) must land in sixteen different
// 16-byte slots: the row PAIR index is what has to be mixed in.
struct LaneOffsets {
	u32 x_src[2];   // per-lane byte offset into A for a direct-to-LDS load (even / odd 8-row unit)
	u32 w_src[2];   // per-lane byte offset into B
	u32 frag_row;   // (lane % 32) * ROW_BYTES
	u32 half;       // lane / 32
	u32 swz;        // (lane >> 1) & 7
};

X17_DEV void issue_stage_loads(
	u8 const *a_tile, u8 const *b_tile, u8 *stage, u32 k0, u32 wave, LaneOffsets const &lo
) {
	// Wave w copies token rows and LDS weight rows [ROWS_PER_WAVE * w, +ROWS_PER_WAVE), 8 rows per load.
	u8 *x_lds = stage + wave * ROWS_PER_WAVE * ROW_BYTES;
	u8 *w_lds = stage + X_TILE_BYTES + wave * ROWS_PER_WAVE * ROW_BYTES;
	u8 const *x_src = a_tile + (size_t)(wave * ROWS_PER_WAVE) * K_TOTAL + k0;
	X17_UNROLL for (u32 u = 0; u < UNITS; ++u) {
		__builtin_amdgcn_global_load_lds(
			X17_GLOBAL_PTR(x_src + (size_t)(u * 8) * K_TOTAL + lo.x_src[u & 1]),
			X17_LDS_PTR(x_lds + u * 8 * ROW_BYTES), 16, 0, 0);
	}
	// LDS weight row R = 128*wn + 32*bn + i holds weight row 128*wn + 64*((i/4)%2) + 16*bn + 4*(i/8) + i%4
	// (see the header comment); for the 8 rows of one load the lane-dependent part is constant.
	X17_UNROLL for (u32 u = 0; u < UNITS; ++u) {
		u32 r0 = wave * ROWS_PER_WAVE + u * 8;
		u32 n_uniform = 128 * (r0 / 128) + 16 * ((r0 % 128) / 32) + 4 * ((r0 % 32) / 8);
		__builtin_amdgcn_global_load_lds(
			X17_GLOBAL_PTR(b_tile + (size_t)n_uniform * K_TOTAL + k0 + lo.w_src[u & 1]),
			X17_LDS_PTR(w_lds + u * 8 * ROW_BYTES), 16, 0, 0);
	}
}

// One 16-byte operand chunk: row `row_off` (bytes), logical chunk `kc` of the 128-byte row.
X17_DEV v4i lds_chunk(u8 const *tile, u32 row_off, u32 kc, u32 swz) {
	return *reinterpret_cast<v4i const *>(tile + row_off + ((kc ^ swz) << 4));
}

X17_DEV v8bf widen8(u32 lo, u32 hi, int kind) {
	// eight 8-bit values -> eight bf16 (exact for int8 codes and for e4m3)
	u32 w[2] = {lo, hi};
	u32 out[4];
	X17_UNROLL for (int i = 0; i < 4; ++i) {
		u32 b0 = (w[i / 2] >> (16 * (i % 2))) & 0xFFu;
		u32 b1 = (w[i / 2] >> (16 * (i % 2) + 8)) & 0xFFu;
		u32 h0, h1;
		if (kind == 1) {
			h0 = e4m3_to_bf16_bits(b0);
			h1 = e4m3_to_bf16_bits(b1);
		} else {
			h0 = f2u(f32((i32)(i8)b0)) >> 16;
			h1 = f2u(f32((i32)(i8)b1)) >> 16;
		}
		out[i] = h0 | (h1 << 16);
	}
	v4u packed = {out[0], out[1], out[2], out[3]};
	return __builtin_bit_cast(v8bf, packed);
}

} // namespace

extern "C" __global__ __launch_bounds__(gt::THREADS_PER_BLOCK)
void kernel(
	u8 const *a, u32 a_rows,
	u8 const *b, u32 b_rows,
	u8 *c
#if X17_EPILOGUE == 3
	, f32 *rrms
#elif X17_EPILOGUE == 2
	, i8 const *residual
#endif
) {
	extern __shared__ __attribute__((aligned(1024))) u8 smem[];
	(void)a_rows;
	(void)b_rows;   // known at compile time, as in templates/basic_gemm/kernel.cu:18-21

	// ---- which tile: remap the linear workgroup id so each XCD gets a compact block of tiles
	u32 const tiles_m = gridDim.x;
	u32 const tiles_n = gridDim.y;
	u32 const total = tiles_m * tiles_n;
	u32 lin = blockIdx.x + blockIdx.y * tiles_m;
	if (total % 8 == 0) {
		lin = (lin % 8) * (total / 8) + lin / 8;      // hardware deals workgroups round-robin to 8 XCDs
	}
	// walk tiles in bands of 8 token-tiles so co-resident tiles share weight and token panels
	constexpr u32 BAND = 8;
	u32 tile_m, tile_n;
	{
		u32 band_tiles = BAND * tiles_n;
		u32 band = lin / band_tiles;
		u32 in_band = lin % band_tiles;
		u32 rows_in_band = (tiles_m - band * BAND) < BAND ? (tiles_m - band * BAND) : BAND;
		tile_m = band * BAND + in_band % rows_in_band;
		tile_n = in_band / rows_in_band;
	}

	u32 const tid = threadIdx.x;
	u32 const lane = tid % 64;
	u32 const wave = __builtin_amdgcn_readfirstlane(tid / 64);
	u32 const wm = wave / gt::WAVES_N;
	u32 const wn = wave % gt::WAVES_N;

	LaneOffsets lo;
	{
		u32 r = lane >> 3, p = lane & 7;
		X17_UNROLL for (u32 odd = 0; odd < 2; ++odd) {
			// the 8 rows of a load unit start at a multiple of 8: row pair index & 7 = 4 * (unit & 1) + r / 2
			u32 chunk = p ^ (4 * odd + (r >> 1));
			lo.x_src[odd] = r * K_TOTAL + 16 * chunk;
			lo.w_src[odd] = (64 * ((lane >> 5) & 1) + ((lane >> 3) & 3)) * K_TOTAL + 16 * chunk;
		}
		lo.frag_row = (lane % 32) * ROW_BYTES;
		lo.half = lane / 32;
		lo.swz = (lane >> 1) & 7;
	}

	u8 const *a_tile = a + (size_t)(tile_m * gt::M_PER_BLOCK) * K_TOTAL;
	u8 const *b_tile = b + (size_t)(tile_n * gt::N_PER_BLOCK) * K_TOTAL;

	Acc acc[4][BM];   // [bn][bm]
	X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
		X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
			X17_UNROLL for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0;
		}
	}

	issue_stage_loads(a_tile, b_tile, smem, 0, wave, lo);

	for (u32 ks = 0; ks < K_STEPS; ++ks) {
		__builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this step's tiles are in LDS
		__syncthreads();                      // ... for every wave, and step ks-1 is fully consumed
		if (ks + 1 < K_STEPS) {
			issue_stage_loads(a_tile, b_tile, smem + ((ks + 1) % gt::STAGES) * STAGE_BYTES,
			                  (ks + 1) * gt::K_STEP, wave, lo);
		}
		u8 const *x_tile = smem + (ks % gt::STAGES) * STAGE_BYTES + wm * gt::WAVE_M * ROW_BYTES + lo.frag_row;
		u8 const *w_tile = smem + (ks % gt::STAGES) * STAGE_BYTES + X_TILE_BYTES + wn * 128 * ROW_BYTES + lo.frag_row;

		if constexpr (MMA == 0) {
			// 32 bytes of K per MFMA; operand fragments of slice s+1 are fetched before the
			// MFMAs of slice s are issued, so LDS latency hides under matrix-core time
			v4i wf[2][4], xf[2][BM];
			X17_UNROLL for (int bn = 0; bn < 4; ++bn) wf[0][bn] = lds_chunk(w_tile, bn * 32 * ROW_BYTES, lo.half, lo.swz);
			X17_UNROLL for (int bm = 0; bm < BM; ++bm) xf[0][bm] = lds_chunk(x_tile, bm * 32 * ROW_BYTES, lo.half, lo.swz);
			X17_UNROLL for (u32 s = 0; s < 4; ++s) {
				if (s + 1 < 4) {
					u32 kc = 2 * (s + 1) + lo.half;
					X17_UNROLL for (int bn = 0; bn < 4; ++bn) wf[(s + 1) & 1][bn] = lds_chunk(w_tile, bn * 32 * ROW_BYTES, kc, lo.swz);
					X17_UNROLL for (int bm = 0; bm < BM; ++bm) xf[(s + 1) & 1][bm] = lds_chunk(x_tile, bm * 32 * ROW_BYTES, kc, lo.swz);
				}
				X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
					X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
						acc[bn][bm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[s & 1][bn], xf[s & 1][bm], acc[bn][bm], 0, 0, 0);
					}
				}
				// pin the issue order: two MFMAs, then one of the eight LDS reads of the next slice
				if (s + 1 < 4) {
					X17_UNROLL for (int i = 0; i < 4 + BM; ++i) {
						__builtin_amdgcn_sched_group_barrier(0x008, (4 * BM) / (4 + BM), 0);
						__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
					}
				} else {
					__builtin_amdgcn_sched_group_barrier(0x008, 4 * BM, 0);
				}
			}
		} else if constexpr (MMA == 1) {
			X17_UNROLL for (u32 s = 0; s < 2; ++s) {            // 64 bytes of K per MFMA
				v8i wf[4], xf[BM];
				u32 kc = 4 * s + 2 * lo.half;
				X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
					v4i lo4 = lds_chunk(w_tile, bn * 32 * ROW_BYTES, kc, lo.swz);
					v4i hi4 = lds_chunk(w_tile, bn * 32 * ROW_BYTES, kc + 1, lo.swz);
					wf[bn] = v8i{lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
				}
				X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
					v4i lo4 = lds_chunk(x_tile, bm * 32 * ROW_BYTES, kc, lo.swz);
					v4i hi4 = lds_chunk(x_tile, bm * 32 * ROW_BYTES, kc + 1, lo.swz);
					xf[bm] = v8i{lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
				}
				X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
					X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
						v16f r = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
							wf[bn], xf[bm], __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0, 0, 0, 0);
						acc[bn][bm] = __builtin_bit_cast(Acc, r);
					}
				}
			}
		} else {
			X17_UNROLL for (u32 s = 0; s < 4; ++s) {            // 32 bytes of K = two bf16 MFMAs of 16
				u32 kc = 2 * s + lo.half;
				v4i wraw[4], xraw[BM];
				X17_UNROLL for (int bn = 0; bn < 4; ++bn) wraw[bn] = lds_chunk(w_tile, bn * 32 * ROW_BYTES, kc, lo.swz);
				X17_UNROLL for (int bm = 0; bm < BM; ++bm) xraw[bm] = lds_chunk(x_tile, bm * 32 * ROW_BYTES, kc, lo.swz);
				X17_UNROLL for (int h = 0; h < 2; ++h) {
					v8bf wf[4], xf[BM];
					X17_UNROLL for (int bn = 0; bn < 4; ++bn) wf[bn] = widen8(wraw[bn][2 * h], wraw[bn][2 * h + 1], B_KIND);
					X17_UNROLL for (int bm = 0; bm < BM; ++bm) xf[bm] = widen8(xraw[bm][2 * h], xraw[bm][2 * h + 1], A_KIND);
					X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
						X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
							v16f r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
								wf[bn], xf[bm], __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0);
							acc[bn][bm] = __builtin_bit_cast(Acc, r);
						}
					}
				}
			}
		}
	}

	// ---- epilogue.  Lane owns token (32*bm + lane%32) of its wave and raw columns
	// 64*(lane/32) + 16*bn + r of its wave, r = accumulator register index.
	u32 const row0 = tile_m * gt::M_PER_BLOCK + wm * gt::WAVE_M + lane % 32;
	u32 const n0 = tile_n * gt::N_PER_BLOCK + wn * 128 + 64 * lo.half;

	X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
		u32 row = row0 + 32 * bm;
		f32 x[64];
		X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
			// (bit-casting a single vector element in place reads element 0; cast the whole vector first)
			v16f const as_f32 = __builtin_bit_cast(v16f, acc[bn][bm]);
			X17_UNROLL for (int r = 0; r < 16; ++r) {
				if constexpr (ACC_F32) {
					x[16 * bn + r] = as_f32[r];
				} else {
					x[16 * bn + r] = f32(acc[bn][bm][r]);
				}
			}
		}
#if X17_EPILOGUE == 0
		ScaleEpilogue::run(x, c, row, n0, nullptr);
#elif X17_EPILOGUE == 1
		GeGluEpilogue::run(x, c, row, n0, nullptr);
#elif X17_EPILOGUE == 2
		ResidualEpilogue::run(x, c, row, n0, residual);
#else
		// L2NormMatrixWriter, cuda/gemm_b8.cuh:861-949 with kv_helpers::l2_norm :767-830.
		// Per head the columns are [K (hd) | V (hd)].  Sum of squares of the K half: four partial
		// sums, partial q owns columns with (col % 8) / 2 == q in increasing column order, total
		// (s0+s1)+(s2+s3).  A lane holds 64 consecutive columns, so a 128-wide K half is summed by
		// the lower-half lane first and continued by lane+32.
		constexpr f32 EPS = f32(f64(X17_EPS));
		constexpr f32 HEAD_SCALE = f32(f64(X17_HEAD_SCALE));
		constexpr f32 SEP_SCALE = f32(f64(X17_SEP_SCALE));
		constexpr u32 HEADS_TOTAL = N_RAW / (2 * HEAD_DIM);
		u8 *dst = c + (size_t)row * N_RAW + n0;
		auto sumsq = [&](int first, int count, f32 (&s)[4]) {
			X17_UNROLL for (int d = 0; d < count; ++d) {
				int q = (d % 8) / 2;
				s[q] = fmaf32(x[first + d], x[first + d], s[q]);
			}
		};
		auto emit = [&](int first, int count, f32 scale, bool dyn) {
			(void)dyn;
			X17_UNROLL for (int v = 0; v < count / 16; ++v) {
				v4u pack;
				X17_UNROLL for (int w = 0; w < 4; ++w) {
					u32 word = 0;
					X17_UNROLL for (int bb = 0; bb < 4; ++bb) {
						int d = first + 16 * v + 4 * w + bb;
						word |= ((u32)f32_to_fixedi8(x[d] * scale) & 0xFFu) << (8 * bb);
					}
					pack[w] = word;
				}
				*reinterpret_cast<v4u *>(dst + first + 16 * v) = pack;
			}
		};
		if constexpr (HEAD_DIM == 32) {
			// a lane holds one whole head: K = x[0..32), V = x[32..64)
			f32 s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
			sumsq(0, 32, s);
			f32 scale = strict::rsq(((s[0] + s[1]) + (s[2] + s[3])) + EPS) * HEAD_SCALE;
			emit(0, 32, scale, true);
			emit(32, 32, SEP_SCALE, false);
			rrms[(size_t)row * HEADS_TOTAL + n0 / 64] = scale;
		} else if constexpr (HEAD_DIM == 64) {
			// lower-half lanes hold K, upper-half lanes hold V of the same head
			f32 s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
			sumsq(0, 64, s);
			f32 scale = strict::rsq(((s[0] + s[1]) + (s[2] + s[3])) + EPS) * HEAD_SCALE;
			if (lo.half == 0) {
				emit(0, 64, scale, true);
				rrms[(size_t)row * HEADS_TOTAL + n0 / 128] = scale;
			} else {
				emit(0, 64, SEP_SCALE, false);
			}
		} else {
			// a wave's 128 columns are the K half (even wn) or the V half (odd wn) of one head
			f32 s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
			if (wn % 2 == 0) {
				f32 t[4] = {0.0f, 0.0f, 0.0f, 0.0f};
				sumsq(0, 64, t);                                   // columns 0..63 (valid in lower lanes)
				X17_UNROLL for (int q = 0; q < 4; ++q) {
					f32 from_low = __shfl(t[q], lane % 32, 64);     // lower lane's partial sums
					s[q] = lo.half == 0 ? 0.0f : from_low;
				}
				if (lo.half != 0) {
					sumsq(0, 64, s);                               // continue with columns 64..127
				}
				X17_UNROLL for (int q = 0; q < 4; ++q) {
					s[q] = __shfl(s[q], 32 + lane % 32, 64);       // the finished sums live in the upper lanes
				}
				f32 scale = strict::rsq(((s[0] + s[1]) + (s[2] + s[3])) + EPS) * HEAD_SCALE;
				emit(0, 64, scale, true);
				if (lo.half == 0) {
					rrms[(size_t)row * HEADS_TOTAL + (tile_n * gt::N_PER_BLOCK + wn * 128) / 256] = scale;
				}
			} else {
				emit(0, 64, SEP_SCALE, false);
			}
		}
#endif
	}
}
