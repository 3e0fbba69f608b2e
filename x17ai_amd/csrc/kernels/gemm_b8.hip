// gemm_b8.hip -- C[M, N] = epilogue(A[M, K] . B[N_raw, K]^T) for 8-bit operands on gfx950.
//
// Replaces the reference's b8::Gemm (cuda/gemm_b8.cuh:624-755: i8 x i8 -> i32) and b16::Gemm
// (cuda/gemm_b16.cuh:436-567: any e4m3 operand, f32 accumulate) together with their four fused
// writers (Scaled :291-339, GeGlu :341-441, Residual :443-622, L2Norm :861-949).  The kernel
// entry and its parameters follow templates/basic_gemm/kernel.cu:9-32.
//
// Design, MI355X-first (nothing here is derived from the SM80 kernel):
//   * One workgroup = a 256 (tokens) x 256 (raw columns) output tile, by default 8 wavefronts of
//     64 x 128 (two per SIMD); gemm_tile.h can also build 8 wavefronts of 128 x 64 or 4 wavefronts of 128 x 128
//     (a 4 x 4 grid of 32x32 MFMA blocks, 256 accumulator registers per lane, one wavefront per SIMD: what the
//     host picks whenever an operand is e4m3).
//   * The WEIGHTS are the MFMA "A" operand and the TOKENS the "B" operand, i.e. the matrix
//     cores compute C^T.  A lane then owns one token and, per MFMA block, 16 output columns;
//     weight rows are permuted on their way into LDS so that those are 64 (32 for 64-column waves)
//     CONSECUTIVE columns across the blocks.  Gate/value pairs, whole K|V heads and 16-byte output
//     vectors all live inside one lane: the epilogues need no cross-lane shuffles (the SM80
//     code needs a 4x4 shuffle transpose per 32x32 tile, cuda/gemm_b8.cuh:411, 570, 592).
//   * Global -> LDS goes through the gfx950 16-byte direct-to-LDS load (no register staging) into
//     rings of LDS tiles (gemm_tile.h: K_STEP bytes of K per step; by default three token tiles and two
//     weight tiles of 32 KB, which is all 160 KB of a compute unit), one barrier per step;
//     16-byte chunks are XOR-swizzled so that ds_read_b128 is conflict-free.  In the int8 and e4m3 kernels the
//     issue order of a K step is pinned: each MFMA is followed by its share of the LDS reads and tile requests
//     (and, in the mixed arithmetic, of the next round's conversions to f16).
//   * int8: v_mfma_i32_32x32x32_i8.  e4m3 x e4m3: v_mfma_f32_32x32x64_f8f6f4.  Mixed
//     e4m3 x int8: both widened exactly to f16 in registers, v_mfma_f32_32x32x16_f16
//     (int8 codes need 7 significand bits, e4m3 has 4; every e4m3 value is a normal f16).
//   * Workgroup ids are remapped so that each XCD (own L2) works on a compact block of tiles.
//
// common.h (generated per kernel by the host-side kernel builder) provides:
//   X17_A_COLS (K), X17_B_ROWS (N_raw), X17_A_KIND / X17_B_KIND (0 = int8, 1 = e4m3),
//   X17_EPILOGUE (0 scale, 1 geglu, 2 residual, 3 l2norm, 4 dequant, 5 qnorm, 6 fused q + kv), X17_STORE
//   (0 FixedI8, 1 e4m3; dequant always stores bf16), X17_DEQ_GEGLU (dequant only: 0 plain, 1 GeGLU over column
//   pairs), X17_INP_SCALE, X17_OUT_SCALE, for l2norm / qnorm / fused X17_HEAD_DIM, X17_EPS, X17_HEAD_SCALE,
//   X17_SEP_SCALE (doubles), for fused X17_Q_COLS (the first raw columns belong to q) and X17_Q_SCALE,
//   X17_STRICT_MATH.
//
// Epilogue 5 (qnorm) is the reference's older Q writer with learned scales (cuda/qkvg_fwd_i8.cuh:145-219; the
// hook is still in the live header: kv_helpers::l2_norm<USE_DYN_SCALE>, cuda/gemm_b8.cuh:761-824): every head_dim
// raw columns are L2-normalised like the K halves of epilogue 3 and multiplied by a bf16 scale per column.
// Epilogue 6 computes the q and the kv projection of src/main.rs:387-493 in ONE launch over the same token tiles
// (raw columns [0, X17_Q_COLS) from the q weights through the Scale writer into q, the rest from the kv weights
// through the L2-norm writer into kv and rrms): the writer is chosen per output tile, x is read once.

#include "common.h"
#include "x17_device.h"
#include "gemm_tile.h"

using namespace x17;
namespace gt = x17::gemm_tile;

// The compiler fully unrolls a K loop of up to 8 steps and then runs out of registers; longer loops it
// unrolls by a small factor on its own, which measures 5 % faster than a rolled loop.
#if (X17_A_COLS / X17_GEMM_K_STEP) <= 8
#define X17_K_LOOP_PRAGMA _Pragma("clang loop unroll(disable)")
#else
#define X17_K_LOOP_PRAGMA
#endif

namespace {

constexpr u32 K_TOTAL = X17_A_COLS;
constexpr u32 N_RAW = X17_B_ROWS;
constexpr int A_KIND = X17_A_KIND;
constexpr int B_KIND = X17_B_KIND;
constexpr int STORE = X17_STORE;

// The writers that normalise whole heads (and the fused q + kv kernel, which contains one) keep the weight rows in
// their natural order: a lane then owns, of every 32-column block, the columns whose (column % 8) / 4 equals
// lane / 32 -- exactly two of the reference's four partial sums of squares (cuda/gemm_b8.cuh:789-801), so a head's
// sum needs one exchange between the lanes of a pair whatever its width.  Every other writer takes 64 consecutive
// columns per lane (pairs and 16-byte output vectors stay inside a lane).
constexpr bool NATURAL_COLS = X17_EPILOGUE == 3 || X17_EPILOGUE == 5 || X17_EPILOGUE == 6;

// 0: int8 MFMA, 1: fp8 MFMA, 2: f16 MFMA after widening
constexpr int MMA = (A_KIND == 0 && B_KIND == 0) ? 0 : ((A_KIND == 1 && B_KIND == 1) ? 1 : 2);
constexpr bool ACC_F32 = MMA != 0;

static_assert(K_TOTAL % gt::K_STEP == 0, "K must be a multiple of 128");
static_assert(N_RAW % 128 == 0 && N_RAW >= gt::N_PER_BLOCK, "raw output columns: a multiple of 128, at least one tile");

constexpr u32 ROW_BYTES = gt::K_STEP;                       // one LDS row = one step of K
constexpr u32 X_TILE_BYTES = gt::M_PER_BLOCK * ROW_BYTES;   // tokens
constexpr u32 W_TILE_BYTES = gt::N_PER_BLOCK * ROW_BYTES;   // weights
constexpr u32 XS = gt::X_STAGES;                             // ring depth of the token tiles
constexpr u32 WS = gt::STAGES;                               // ring depth of the weight tiles
constexpr u32 W_RING_OFFSET = XS * X_TILE_BYTES;             // LDS: XS token tiles, then WS weight tiles
constexpr u32 K_STEPS = K_TOTAL / gt::K_STEP;

constexpr int BM = gt::WAVE_M / 32;                         // 32-token MFMA blocks per wave
constexpr u32 WAVES = gt::WAVES_M * gt::WAVES_N;

using Acc = __attribute__((ext_vector_type(16))) int;       // raw 16 registers; reinterpreted as f32 when ACC_F32

// ------------------------------------------------------------------ epilogues
// Each receives, for ONE token row, the accumulators of LANE_COLS (64, or 32 for 64-column waves)
// consecutive raw columns starting at raw column `n`, already converted to f32 (i32 -> f32 is the
// reference's implicit RNE cast).
constexpr int BN = gt::WAVE_N / 32;                         // 32-column MFMA blocks per wave
constexpr int LANE_COLS = 16 * BN;                          // consecutive raw columns a lane ends up with

// ScaledMatrixWriter, cuda/gemm_b8.cuh:291-339
struct ScaleEpilogue {
	static constexpr f64 SCALE = f64(X17_INP_SCALE) * f64(X17_OUT_SCALE);
	static constexpr u32 OUT_COLS = N_RAW;
	X17_DEV static void run(f32 const (&x)[LANE_COLS], u8 *c, u32 row, u32 n, void const *) {
		u8 *dst = c + (size_t)row * OUT_COLS + n;
		X17_UNROLL for (int v = 0; v < LANE_COLS / 16; ++v) {
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				f32 y[4];
				X17_UNROLL for (int b = 0; b < 4; ++b) y[b] = x[16 * v + 4 * w + b] * f32(SCALE);
				pack[w] = pack4_store<STORE>(y[0], y[1], y[2], y[3]);
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
	// gate(g) * v.  The speed build uses 1 + tanh(s) = 2 / (1 + 2^(-2 s lg e)) and folds the constants:
	// g * v / (c + c * 2^(g * (A1 + A3 g^2))), c = 1 / (2 Y) -- two transcendentals and seven plain
	// operations; an overflowing exponential gives +inf and a quotient of zero, the right limit.
	static constexpr f64 LOG2E = 1.4426950408889634;
	X17_DEV static f32 gated(f32 g, f32 v) {
		if constexpr (X17_STRICT_MATH != 0) {
			return gate(g) * v;
		} else {
			f32 g2 = g * g;
			f32 t = fmaf32(g2, f32(-2.0 * LOG2E * CK3), f32(-2.0 * LOG2E * CK));
			f32 e = hw::ex2(t * g);
			f32 d = fmaf32(e, f32(0.5 / Y), f32(0.5 / Y));
			return (g * v) * hw::rcp(d);
		}
	}
	X17_DEV static void run(f32 const (&x)[LANE_COLS], u8 *c, u32 row, u32 n, void const *) {
		u8 *dst = c + (size_t)row * OUT_COLS + n / 2;
		X17_UNROLL for (int v = 0; v < LANE_COLS / 32; ++v) {
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				f32 y[4];
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					int j = 16 * v + 4 * w + b;
					y[b] = gated(x[2 * j], x[2 * j + 1]);
				}
				pack[w] = pack4_store<STORE>(y[0], y[1], y[2], y[3]);
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
		if constexpr (X17_STRICT_MATH == 0) {
			// Speed build: both weights from one exponential.  With u = 2 I g and E = 2^-|u|:
			//   1 + tanh(-I ln2 g) = 2 / (1 + 2^u) = 2 (u >= 0 ? E : 1) / (1 + E)       -> old_w
			//   lg2(1 + 2^-|u|)    = lg2(1 + E)                                          -> new_w
			// three transcendentals (ex2, rcp, lg2) instead of four.
			f32 const u = g * SP_INP_SCALE;
			f32 const e = hw::ex2(-__builtin_fabsf(u));
			f32 const d = 1.0f + e;
			f32 const old_w = (f32(2.0 * SG_HALF) * hw::rcp(d)) * (u >= 0.0f ? e : 1.0f);
			f32 line = __builtin_fmaxf(0.0f, g);
			if constexpr (SP_LINE != 1.0f) {
				line = line * SP_LINE;
			}
			f32 const new_w = fmaf32(hw::lg2(d), SP_OUT_SCALE, line);
			return fmaf32(new_w, v, old_w * r);
		}
		f32 old_w = fmaf32(f32(SG_HALF), sfu::tanh(f32(SG_IN) * g), f32(SG_HALF));
		f32 line = __builtin_fmaxf(0.0f, g);
		if constexpr (SP_LINE != 1.0f) {
			line = line * SP_LINE;
		}
		f32 new_w = fmaf32(sfu::lg2(1.0f + sfu::ex2(-__builtin_fabsf(g * SP_INP_SCALE))), SP_OUT_SCALE, line);
		return fmaf32(new_w, v, old_w * r);
	}
	X17_DEV static void run(f32 const (&x)[LANE_COLS], u8 *c, u32 row, u32 n, void const *extra) {
		size_t off = (size_t)row * OUT_COLS + n / 2;
		i8 const *res = reinterpret_cast<i8 const *>(extra) + off;
		u8 *dst = c + off;
		X17_UNROLL for (int v = 0; v < LANE_COLS / 32; ++v) {
			v4u rv = *reinterpret_cast<v4u const *>(res + 16 * v);
			v4u pack;
			X17_UNROLL for (int w = 0; w < 4; ++w) {
				f32 y[4];
				X17_UNROLL for (int b = 0; b < 4; ++b) {
					int j = 16 * v + 4 * w + b;
					f32 r = f32((i32)(i8)((rv[w] >> (8 * b)) & 0xFFu));
					y[b] = mix(x[2 * j], x[2 * j + 1], r);
				}
				pack[w] = pack4_store<STORE>(y[0], y[1], y[2], y[3]);
			}
			*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
		}
	}
};

// Dequantising writer: per-row (token) and per-column (output channel) f32 scales, bf16 output, optional
// GeGLU over column pairs.  The reference folds its scales into compile-time constants; this is the
// run-time-scale superset for symmetric per-row / per-channel int8 quantisation (bf16 store precedent:
// cuda/gemm_b16.cuh:264-294).  t = (x * row_scale) * col_scale, two f32 multiplies in that order.
#if X17_EPILOGUE == 4
static_assert(LANE_COLS == 64, "the dequantising writer is written for 128-column waves");
struct DequantEpilogue {
	static constexpr bool GEGLU = X17_DEQ_GEGLU != 0;
	static constexpr u32 OUT_COLS = GEGLU ? N_RAW / 2 : N_RAW;
	X17_DEV static void run(f32 const (&x)[64], u8 *c, u32 row, u32 n, f32 const *row_scale, f32 const *col_scale) {
		f32 const rs = row_scale[row];
		f32 t[64];
		X17_UNROLL for (int v = 0; v < 16; ++v) {
			v4f cs = *reinterpret_cast<v4f const *>(col_scale + n + 4 * v);
			X17_UNROLL for (int i = 0; i < 4; ++i) t[4 * v + i] = (x[4 * v + i] * rs) * cs[i];
		}
		if constexpr (GEGLU) {
			u8 *dst = c + ((size_t)row * OUT_COLS + n / 2) * 2;
			X17_UNROLL for (int v = 0; v < 4; ++v) {
				v4u pack;
				X17_UNROLL for (int w = 0; w < 4; ++w) {
					int j = 8 * v + 2 * w;
					pack[w] = pack2_bf16_rne(GeGluEpilogue::gated(t[2 * j], t[2 * j + 1]), GeGluEpilogue::gated(t[2 * j + 2], t[2 * j + 3]));
				}
				*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
			}
		} else {
			u8 *dst = c + ((size_t)row * OUT_COLS + n) * 2;
			X17_UNROLL for (int v = 0; v < 8; ++v) {
				v4u pack;
				X17_UNROLL for (int w = 0; w < 4; ++w) {
					int j = 8 * v + 2 * w;
					pack[w] = pack2_bf16_rne(t[j], t[j + 1]);
				}
				*reinterpret_cast<v4u *>(dst + 16 * v) = pack;
			}
		}
	}
};
#endif

// ---- writers over the natural column order (l2norm, qnorm and the fused q + kv kernel).
// For ONE token row a lane holds x[16 * b + r] = raw column 32 * b + 8 * (r / 4) + 4 * (lane / 32) + r % 4 of its
// wave's 128 columns (b = 32-column block, r = accumulator register).
#if X17_EPILOGUE == 3 || X17_EPILOGUE == 5 || X17_EPILOGUE == 6
static_assert(LANE_COLS == 64, "the head-normalising writers are written for 128-column waves");
constexpr u32 HEAD_DIM = X17_HEAD_DIM;
static_assert(HEAD_DIM == 32 || HEAD_DIM == 64 || HEAD_DIM == 128, "head_dim must be 32, 64 or 128");
struct NaturalWriters {
	static constexpr f32 EPS = f32(f64(X17_EPS));
	static constexpr f32 HEAD_SCALE = f32(f64(X17_HEAD_SCALE));
	static constexpr int HB = HEAD_DIM / 32;                    // 32-column blocks per head

	// value of lane ^ 32
	X17_DEV static f32 partner(f32 v, u32 half) {
		u32 const u = f2u(v);
		auto const r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
		return u2f(half == 0 ? r[1] : r[0]);
	}
	// The lane pair (lane, lane + 32) holds the 32 output bytes of a block interleaved word by word (word g of a lane
	// = columns 8 g + 4 half .. + 3); two cross-half swaps give the lower lane bytes 0..15 and the upper lane bytes
	// 16..31, so that each lane writes one 16-byte vector.
	X17_DEV static void store_block(u8 *block, u32 const (&w)[4], u32 half) {
		auto const a = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
		auto const b = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
		*reinterpret_cast<v4u *>(block + 16 * half) = v4u{a[0], a[1], b[0], b[1]};
	}
	// kv_helpers::l2_norm, cuda/gemm_b8.cuh:767-830: the sum of squares of the head made of blocks [B0, B0 + HB).
	// The reference's partial sum q owns the columns with (column % 8) / 2 == q in increasing order; the lower lane
	// of a pair runs the chains of q = 0 and 1, the upper lane those of 2 and 3, total (s0 + s1) + (s2 + s3).
	template <int B0>
	X17_DEV static f32 head_scale(f32 const (&x)[64], u32 half) {
		f32 p0 = 0.0f, p1 = 0.0f;
		X17_UNROLL for (int b = B0; b < B0 + HB; ++b) {
			X17_UNROLL for (int g = 0; g < 4; ++g) {
				p0 = fmaf32(x[16 * b + 4 * g], x[16 * b + 4 * g], p0);
				p0 = fmaf32(x[16 * b + 4 * g + 1], x[16 * b + 4 * g + 1], p0);
				p1 = fmaf32(x[16 * b + 4 * g + 2], x[16 * b + 4 * g + 2], p1);
				p1 = fmaf32(x[16 * b + 4 * g + 3], x[16 * b + 4 * g + 3], p1);
			}
		}
		f32 const mine = p0 + p1;
		f32 const other = partner(mine, half);
		f32 const total = half == 0 ? mine + other : other + mine;
		return strict::rsq(total + EPS) * HEAD_SCALE;
	}
	// block b of the row times `scale` (and, with learned scales, times the bf16 scale of each column, in that order:
	// cuda/gemm_b8.cuh:819-820) -> FixedI8, 16 bytes per lane.  `dst` and `dyn` point at the wave's first column.
	template <bool DYN>
	X17_DEV static void emit_block(f32 const (&x)[64], int b, f32 scale, u8 *dst, u16 const *dyn, u32 half) {
		u32 w[4];
		X17_UNROLL for (int g = 0; g < 4; ++g) {
			f32 y[4];
			X17_UNROLL for (int e = 0; e < 4; ++e) y[e] = x[16 * b + 4 * g + e] * scale;
			if constexpr (DYN) {
				v2u const d = *reinterpret_cast<v2u const *>(dyn + 32 * b + 8 * g + 4 * half);
				y[0] = y[0] * u2f(d[0] << 16);
				y[1] = y[1] * u2f(d[0] & 0xFFFF0000u);
				y[2] = y[2] * u2f(d[1] << 16);
				y[3] = y[3] * u2f(d[1] & 0xFFFF0000u);
				// The old writer hands its f32 values to a base writer built with SCALE = 1 / sqrt(MODEL_DIM)
				// (cuda/qkvg_fwd_i8.cuh:151-159); that base class is gone from the tree, and the live scaled writer's f32
				// overload multiplies by its SCALE unless it is 1 (cuda/gemm_b8.cuh:307-324).  X17_INP_SCALE carries that
				// factor (1.0: stored as is).
				if constexpr (f32(f64(X17_INP_SCALE)) != 1.0f) {
					X17_UNROLL for (int e = 0; e < 4; ++e) y[e] = y[e] * f32(f64(X17_INP_SCALE));
				}
			}
			w[g] = pack4_fixedi8(y[0], y[1], y[2], y[3]);
		}
		store_block(dst + 32 * b, w, half);
	}
#if X17_EPILOGUE == 3 || X17_EPILOGUE == 6
	// L2NormMatrixWriter, cuda/gemm_b8.cuh:861-949: per head the columns are [K (hd) | V (hd)]; K is normalised,
	// V only scaled, rrms[row, head] = the K scale.  `col0` = the wave's first raw column of the kv matrix.
	static constexpr f32 SEP_SCALE = f32(f64(X17_SEP_SCALE));
	X17_DEV static void l2norm_row(f32 const (&x)[64], u8 *c, f32 *rrms, u32 row, u32 col0, u32 kv_cols, u32 half) {
		u8 *dst = c + (size_t)row * kv_cols + col0;
		f32 *rr = rrms + (size_t)row * (kv_cols / (2 * HEAD_DIM));
		if constexpr (HEAD_DIM == 32) {
			f32 const scale0 = head_scale<0>(x, half);
			emit_block<false>(x, 0, scale0, dst, nullptr, half);
			emit_block<false>(x, 1, SEP_SCALE, dst, nullptr, half);
			f32 const scale1 = head_scale<2>(x, half);
			emit_block<false>(x, 2, scale1, dst, nullptr, half);
			emit_block<false>(x, 3, SEP_SCALE, dst, nullptr, half);
			if (half == 0) {
				rr[col0 / 64] = scale0;
				rr[col0 / 64 + 1] = scale1;
			}
		} else if constexpr (HEAD_DIM == 64) {
			f32 const scale = head_scale<0>(x, half);
			emit_block<false>(x, 0, scale, dst, nullptr, half);
			emit_block<false>(x, 1, scale, dst, nullptr, half);
			emit_block<false>(x, 2, SEP_SCALE, dst, nullptr, half);
			emit_block<false>(x, 3, SEP_SCALE, dst, nullptr, half);
			if (half == 0) rr[col0 / 128] = scale;
		} else {
			// the wave's 128 columns are the K half or the V half of one head
			if ((col0 / 128) % 2 == 0) {
				f32 const scale = head_scale<0>(x, half);
				X17_UNROLL for (int b = 0; b < 4; ++b) emit_block<false>(x, b, scale, dst, nullptr, half);
				if (half == 0) rr[col0 / 256] = scale;
			} else {
				X17_UNROLL for (int b = 0; b < 4; ++b) emit_block<false>(x, b, SEP_SCALE, dst, nullptr, half);
			}
		}
	}
#endif
#if X17_EPILOGUE == 5
	// QMatrixWriter, cuda/qkvg_fwd_i8.cuh:145-219: every head_dim columns are one normalised head
	template <int B0>
	X17_DEV static void qnorm_heads(f32 const (&x)[64], u8 *dst, u16 const *dyn, u32 half) {
		if constexpr (B0 < 4) {
			f32 const scale = head_scale<B0>(x, half);
			X17_UNROLL for (int b = B0; b < B0 + HB; ++b) emit_block<true>(x, b, scale, dst, dyn, half);
			qnorm_heads<B0 + HB>(x, dst, dyn, half);
		}
	}
	X17_DEV static void qnorm_row(f32 const (&x)[64], u8 *c, u16 const *dyn, u32 row, u32 col0, u32 half) {
		qnorm_heads<0>(x, c + (size_t)row * N_RAW + col0, dyn + col0, half);
	}
#endif
#if X17_EPILOGUE == 6
	// ScaledMatrixWriter (cuda/gemm_b8.cuh:291-339) over the natural column order, for the q columns
	X17_DEV static void scale_row(f32 const (&x)[64], u8 *c, u32 row, u32 col0, u32 q_cols, u32 half) {
		u8 *dst = c + (size_t)row * q_cols + col0;
		X17_UNROLL for (int b = 0; b < 4; ++b) emit_block<false>(x, b, f32(f64(X17_Q_SCALE)), dst, nullptr, half);
	}
#endif
};
#endif

// ------------------------------------------------------------------ tile loads

// LDS rows hold K_STEP bytes = CHUNKS chunks of 16; logical chunk c of row r is stored at position
// c ^ ((r >> SWZ_SHIFT) & (CHUNKS - 1)).  The LDS has 64 four-byte banks (256 bytes per bank line)
// and serves a ds_read_b128 sixteen lanes at a time, so sixteen consecutive rows must land in sixteen
// different 16-byte slots of the bank line: with 128-byte rows two rows share a bank line and the row
// PAIR index has to be mixed in, with 64-byte rows the row QUAD index.
constexpr u32 CHUNKS = gt::CHUNKS;
constexpr u32 SWZ_SHIFT = gt::SWZ_SHIFT;
constexpr u32 UNIT_ROWS = gt::UNIT_ROWS;                    // rows one 64-lane x 16-byte direct-to-LDS load fills
// With eight waves, two per SIMD, only the first of each pair (waves 0 .. 3) requests tiles.  The arbiter serves
// that wave first: with the loads shared evenly it ended its step early and sat at the barrier while its partner,
// the same loads to issue between its MFMAs, finished alone.  (Splitting the weight units 6:2, 4:4, 2:6 or 0:8
// between the two measured the same as 8:0.)
constexpr u32 LOADER_WAVES = gt::LOADER_WAVES;            // (a four-wave workgroup has one wave per SIMD)
constexpr u32 X_UNITS = gt::X_UNITS;                      // such loads per loading wave, step and tile
constexpr u32 W_UNITS = gt::W_UNITS;
constexpr u32 LOADS_PER_STAGE = X_UNITS + W_UNITS;
static_assert((X_UNITS * UNIT_ROWS) % 16 == 0 && (W_UNITS * UNIT_ROWS) % 16 == 0, "a wave's share must keep the swizzle phase");

// A wave that has a SIMD to itself has registers to spare: it keeps one lane offset per load unit, the unit's
// own row offset included, and all loads of a tile share ONE scalar base (no scalar add per load, two scalar
// register pairs instead of sixteen).
constexpr bool LANE_UNIT_OFFSETS = gt::WAVES_PER_SIMD == 1;
constexpr u32 X_OFFSETS = LANE_UNIT_OFFSETS ? X_UNITS : 2;
constexpr u32 W_OFFSETS = LANE_UNIT_OFFSETS ? W_UNITS : 2;
X17_DEV constexpr u32 w_unit_row(u32 r0) {   // weight row that LDS weight row r0 (a multiple of the unit) starts from
	return gt::w_unit_row(r0, NATURAL_COLS);
}
struct LaneOffsets {
	u32 x_src[X_OFFSETS];   // per-lane byte offset into A for a direct-to-LDS load (even / odd load unit, or per unit)
	u32 w_src[W_OFFSETS];   // per-lane byte offset into B
	u32 frag_row;   // (lane % 32) * ROW_BYTES
	u32 half;       // lane / 32
	u32 swz;        // swizzle key of the fragment row this lane reads
};

// Direct-to-LDS loads of a loading wave's share of one token tile / one weight tile: loading wave w copies
// token rows [X_UNITS * UNIT_ROWS * w, +X_UNITS * UNIT_ROWS) and as many LDS weight rows.
// With WN = WAVE_N columns per wave, LDS weight row R = WN*wn + 32*bn + i holds weight row
// WN*wn + (WN/2)*((i/4)%2) + 16*bn + 4*(i/8) + i%4: the MFMA hands output row i = 8*(r/4) + 4*(lane/32) + r%4
// to register r, so a lane collects columns (WN/2)*(lane/32) + 16*bn + r.  For the rows of one load unit the
// lane-dependent part is constant.
// One 16-byte-per-lane direct-to-LDS load: LDS destination in M0 (wave-uniform; lane l lands 16 * l bytes further),
// global source = uniform 64-bit base in scalar registers + a 32-bit offset per lane.  Written out because the
// compiler's own selection forms a 64-bit address per lane in ONE vector register pair for every load: a 64-bit
// vector add per load, each waiting until the previous load has read the pair (measured 3-5 % of the kernel).
X17_DEV void load_to_lds_16(u8 *lds_uniform, u8 const *src_uniform, u32 lane_offset) {
	// (gfx9 family: a scalar write of M0 needs one wait state before a direct-to-LDS load reads it; the compiler
	// inserts it for its own loads and cannot see into this string)
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
	             :: "s"((u32)(size_t)X17_LDS_PTR(lds_uniform)), "v"(lane_offset), "s"(src_uniform) : "memory", "m0");
}

template <u32 U>
X17_DEV void issue_x_load(u8 const *a_tile, u8 *x_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	u8 *x_lds = x_tile + (wave * X_UNITS + U) * UNIT_ROWS * ROW_BYTES;
	if constexpr (LANE_UNIT_OFFSETS) {
		load_to_lds_16(x_lds, a_tile + (size_t)(wave * X_UNITS * UNIT_ROWS) * K_TOTAL + k0, lo.x_src[U]);
	} else {
		u8 const *x_src = a_tile + (size_t)((wave * X_UNITS + U) * UNIT_ROWS) * K_TOTAL + k0;
		load_to_lds_16(x_lds, x_src, lo.x_src[U & 1]);
	}
}
template <u32 U>
X17_DEV void issue_w_load(u8 const *b_tile, u8 *w_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	u32 r0 = (wave * W_UNITS + U) * UNIT_ROWS;
	u8 *w_lds = w_tile + r0 * ROW_BYTES;
	if constexpr (LANE_UNIT_OFFSETS) {
		load_to_lds_16(w_lds, b_tile + (size_t)w_unit_row(wave * W_UNITS * UNIT_ROWS) * K_TOTAL + k0, lo.w_src[U]);
	} else {
		u8 const *w_src = b_tile + (size_t)w_unit_row(r0) * K_TOTAL + k0;
		load_to_lds_16(w_lds, w_src, lo.w_src[U & 1]);
	}
}
// this wave's share of one token tile / one weight tile of one step
template <u32 FIRST = 0, u32 LAST = X_UNITS>
X17_DEV void issue_x_units(u8 const *a_tile, u8 *x_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	if constexpr (FIRST < LAST) {
		issue_x_load<FIRST>(a_tile, x_tile, k0, wave, lo);
		issue_x_units<FIRST + 1, LAST>(a_tile, x_tile, k0, wave, lo);
	}
}
template <u32 FIRST = 0>
X17_DEV void issue_w_units(u8 const *b_tile, u8 *w_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	if constexpr (FIRST < W_UNITS) {
		issue_w_load<FIRST>(b_tile, w_tile, k0, wave, lo);
		issue_w_units<FIRST + 1>(b_tile, w_tile, k0, wave, lo);
	}
}
// (the other waves have nothing in flight: their waits on the load counter fall through)
X17_DEV void issue_x_loads(u8 const *a_tile, u8 *x_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	if (wave < LOADER_WAVES) {
		issue_x_units(a_tile, x_tile, k0, wave, lo);
	}
}
X17_DEV void issue_w_loads(u8 const *b_tile, u8 *w_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	if (wave < LOADER_WAVES) {
		issue_w_units(b_tile, w_tile, k0, wave, lo);
	}
}

// s_waitcnt vmcnt(N) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <u32 N>
X17_DEV void wait_vmcnt() {
	static_assert(N < 64);
	__builtin_amdgcn_s_waitcnt((N & 15u) | ((N >> 4) << 14) | 0x0F70u);
}
// Loads complete in issue order.  Behind every barrier a wave issues its share of one weight tile (step + WS)
// and then of one token tile (step + XS).  The tiles of step ks+1 are awaited with everything issued after
// the weight tile of that step still allowed in flight: the token tile issued with it when the token ring
// is the deeper one, and `later` whole steps.
X17_DEV void wait_step(u32 later, bool token_tile_behind) {
	if constexpr (WS >= 4) {
		if (later >= 2) {
			if (XS > WS && token_tile_behind) { wait_vmcnt<2 * LOADS_PER_STAGE + X_UNITS>(); } else { wait_vmcnt<2 * LOADS_PER_STAGE>(); }
			return;
		}
	}
	if constexpr (WS >= 3) {
		if (later >= 1) {
			if (XS > WS && token_tile_behind) { wait_vmcnt<LOADS_PER_STAGE + X_UNITS>(); } else { wait_vmcnt<LOADS_PER_STAGE>(); }
			return;
		}
	}
	if (XS > WS && token_tile_behind) { wait_vmcnt<X_UNITS>(); } else { wait_vmcnt<0>(); }
}

// One 16-byte operand chunk: row `row_off` (bytes), logical chunk `kc` of the row.
X17_DEV v4i lds_chunk(u8 const *tile, u32 row_off, u32 kc, u32 swz) {
	return *reinterpret_cast<v4i const *>(tile + row_off + ((kc ^ swz) << 4));
}

// Eight 8-bit values (two registers) -> eight f16, exact for both kinds.
//   e4m3: the gfx950 packed fp8 -> f16 conversion (scale 1).  It reads OCP e4m3; the codes the
//         reference's encoder produces (no subnormals, no NaN, no -0) mean the same in both.
//   int8: flip the sign bit (b + 128 as an unsigned byte u), splice u under the f16 exponent of 1024
//         (0x6400 | u == 1024 + u) and subtract 1152 -- five instructions per four bytes.
[[maybe_unused]] X17_DEV v8h widen8(u32 lo, u32 hi, int kind) {
	v2h p[4];
	if (kind == 1) {
		p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
		p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
		p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
		p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
	} else {
		v2h const bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
		u32 w[2] = {lo ^ 0x80808080u, hi ^ 0x80808080u};
		X17_UNROLL for (int i = 0; i < 2; ++i) {
			u32 l = __builtin_amdgcn_perm(0x64646464u, w[i], 0x04010400u);
			u32 h = __builtin_amdgcn_perm(0x64646464u, w[i], 0x04030402u);
			p[2 * i] = __builtin_bit_cast(v2h, l) + bias;
			p[2 * i + 1] = __builtin_bit_cast(v2h, h) + bias;
		}
	}
	return v8h{p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
}

// Operand fragments of one K slice (what one round of 4 x BM MFMA blocks consumes) and the MFMAs
// themselves, per arithmetic: 32 bytes of K for int8 and for the f16-widened mix, 64 for e4m3.
constexpr u32 SLICE_BYTES = MMA == 1 ? 64 : 32;
constexpr u32 SLICES = gt::K_STEP / SLICE_BYTES;
constexpr u32 CHUNKS_PER_FRAG = SLICE_BYTES / 32;           // 16-byte chunks a lane fetches per operand row
static_assert(SLICES % 2 == 0, "the fragment double buffer needs an even number of slices per step");

struct Frags {
	v4i w[BN][CHUNKS_PER_FRAG];
	v4i x[BM][CHUNKS_PER_FRAG];
};

X17_DEV void load_frags(Frags &f, u8 const *w_tile, u8 const *x_tile, u32 s, LaneOffsets const &lo) {
	// in the order the MFMAs of a slice want them: w0, every x, then the other w
	u32 const kc0 = CHUNKS_PER_FRAG * (2 * s + lo.half);
	X17_UNROLL for (u32 c = 0; c < CHUNKS_PER_FRAG; ++c) f.w[0][c] = lds_chunk(w_tile, 0, kc0 + c, lo.swz);
	X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
		X17_UNROLL for (u32 c = 0; c < CHUNKS_PER_FRAG; ++c) f.x[bm][c] = lds_chunk(x_tile, bm * 32 * ROW_BYTES, kc0 + c, lo.swz);
	}
	X17_UNROLL for (int bn = 1; bn < BN; ++bn) {
		X17_UNROLL for (u32 c = 0; c < CHUNKS_PER_FRAG; ++c) f.w[bn][c] = lds_chunk(w_tile, bn * 32 * ROW_BYTES, kc0 + c, lo.swz);
	}
}

X17_DEV void mma_slice(Frags const &f, Acc (&acc)[BN][BM]) {
	if constexpr (MMA == 0) {
		X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
			X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
				acc[bn][bm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[bn][0], f.x[bm][0], acc[bn][bm], 0, 0, 0);
			}
		}
	} else if constexpr (MMA == 1) {
		v8i wf[BN], xf[BM];
		X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
			v4i l = f.w[bn][0], h = f.w[bn][CHUNKS_PER_FRAG - 1];
			wf[bn] = v8i{l[0], l[1], l[2], l[3], h[0], h[1], h[2], h[3]};
		}
		X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
			v4i l = f.x[bm][0], h = f.x[bm][CHUNKS_PER_FRAG - 1];
			xf[bm] = v8i{l[0], l[1], l[2], l[3], h[0], h[1], h[2], h[3]};
		}
		X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
			X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
				v16f r = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
					wf[bn], xf[bm], __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0, 0, 0, 0);
				acc[bn][bm] = __builtin_bit_cast(Acc, r);
			}
		}
	} else {
		X17_UNROLL for (int h = 0; h < 2; ++h) {                // two f16 MFMAs of K = 16
			v8h wf[BN], xf[BM];
			X17_UNROLL for (int bn = 0; bn < BN; ++bn) wf[bn] = widen8(f.w[bn][0][2 * h], f.w[bn][0][2 * h + 1], B_KIND);
			X17_UNROLL for (int bm = 0; bm < BM; ++bm) xf[bm] = widen8(f.x[bm][0][2 * h], f.x[bm][0][2 * h + 1], A_KIND);
			X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
				X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
					v16f r = __builtin_amdgcn_mfma_f32_32x32x16_f16(
						wf[bn], xf[bm], __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0);
					acc[bn][bm] = __builtin_bit_cast(Acc, r);
				}
			}
		}
	}
}

// Pin the issue order of one slice: the LDS reads of the next fragments and this slice's share of the
// next stage's global loads are spread evenly between the MFMAs.  LDS latency then hides under
// matrix-core time, and a wave never sits in a burst of loads waiting for the memory pipeline to
// accept them (instructions issue in order: a queued load would hold back the MFMAs behind it).
template <u32 N_LOADS>
X17_DEV void interleave_slice(bool with_reads) {
	if constexpr (MMA != 2) {
		constexpr int READS = (BN + BM) * CHUNKS_PER_FRAG;
		constexpr int MFMAS = BN * BM;
		constexpr int GROUPS = MFMAS < READS ? MFMAS : READS;
		if (with_reads) {
			X17_UNROLL for (int i = 0; i < GROUPS; ++i) {
				__builtin_amdgcn_sched_group_barrier(0x008, MFMAS / GROUPS, 0);
				__builtin_amdgcn_sched_group_barrier(0x100, READS / GROUPS, 0);
				if (i < (int)N_LOADS) {
					__builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
				}
			}
		} else {
			__builtin_amdgcn_sched_group_barrier(0x008, MFMAS, 0);
		}
	}
}

// ---- the paced form of a slice (int8 and e4m3 arithmetic): every MFMA is followed by its share of the next
// fragments' LDS reads and of the tile requests, and nothing may move across the group boundaries, so a
// wave that has a SIMD to itself for a while keeps the matrix core fed instead of issuing requests in a burst.
constexpr int MFMAS_PER_SLICE = BN * BM;
constexpr int READS_PER_SLICE = (BN + BM) * (int)CHUNKS_PER_FRAG;

template <int I>
X17_DEV void mma_one(Frags const &f, Acc (&acc)[BN][BM]) {
	constexpr int bn = I / BM, bm = I % BM;
	if constexpr (MMA == 0) {
		acc[bn][bm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[bn][0], f.x[bm][0], acc[bn][bm], 0, 0, 0);
	} else {
		v4i wl = f.w[bn][0], wh = f.w[bn][CHUNKS_PER_FRAG - 1];
		v4i xl = f.x[bm][0], xh = f.x[bm][CHUNKS_PER_FRAG - 1];
		v8i wf = v8i{wl[0], wl[1], wl[2], wl[3], wh[0], wh[1], wh[2], wh[3]};
		v8i xf = v8i{xl[0], xl[1], xl[2], xl[3], xh[0], xh[1], xh[2], xh[3]};
		v16f r = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, xf, __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0, 0, 0, 0);
		acc[bn][bm] = __builtin_bit_cast(Acc, r);
	}
}
// read number J of a slice's fragments, in the order the MFMAs want them: w0, every x, then the other w
template <int J>
X17_DEV void read_one(Frags &f, u8 const *w_tile, u8 const *x_tile, u32 s, LaneOffsets const &lo) {
	constexpr int q = J / (int)CHUNKS_PER_FRAG;
	constexpr u32 c = J % CHUNKS_PER_FRAG;
	u32 const kc = CHUNKS_PER_FRAG * (2 * s + lo.half) + c;
	if constexpr (q == 0) {
		f.w[0][c] = lds_chunk(w_tile, 0, kc, lo.swz);
	} else if constexpr (q <= BM) {
		f.x[q - 1][c] = lds_chunk(x_tile, (q - 1) * 32 * ROW_BYTES, kc, lo.swz);
	} else {
		f.w[q - BM][c] = lds_chunk(w_tile, (q - BM) * 32 * ROW_BYTES, kc, lo.swz);
	}
}
template <int FIRST, int LAST>
X17_DEV void read_range(Frags &f, u8 const *w_tile, u8 const *x_tile, u32 s, LaneOffsets const &lo) {
	if constexpr (FIRST < LAST) {
		read_one<FIRST>(f, w_tile, x_tile, s, lo);
		read_range<FIRST + 1, LAST>(f, w_tile, x_tile, s, lo);
	}
}
template <u32 FIRST, u32 LAST>
X17_DEV void issue_w_range(u8 const *b_tile, u8 *w_tile, u32 k0, u32 wave, LaneOffsets const &lo) {
	if constexpr (FIRST < LAST) {
		issue_w_load<FIRST>(b_tile, w_tile, k0, wave, lo);
		issue_w_range<FIRST + 1, LAST>(b_tile, w_tile, k0, wave, lo);
	}
}
// KIND 0: no requests, 1: token units [FIRST, FIRST + COUNT), 2: weight units [FIRST, FIRST + COUNT)
template <int I, bool READS, int KIND, u32 FIRST, u32 COUNT>
X17_DEV void paced_slice(Frags const &cur, Frags &next, u8 const *nw, u8 const *nx, u32 ns, LaneOffsets const &lo,
                         Acc (&acc)[BN][BM], u8 const *src, u8 *dst, u32 k0, u32 wave) {
	if constexpr (I < MFMAS_PER_SLICE) {
		mma_one<I>(cur, acc);
		if constexpr (READS) {
			constexpr int R0 = I * READS_PER_SLICE / MFMAS_PER_SLICE, R1 = (I + 1) * READS_PER_SLICE / MFMAS_PER_SLICE;
			read_range<R0, R1>(next, nw, nx, ns, lo);
		}
		constexpr u32 L0 = FIRST + I * COUNT / MFMAS_PER_SLICE, L1 = FIRST + (I + 1) * COUNT / MFMAS_PER_SLICE;
		if constexpr (KIND == 1) {
			issue_x_units<L0, L1>(src, dst, k0, wave, lo);
		} else if constexpr (KIND == 2) {
			issue_w_range<L0, L1>(src, dst, k0, wave, lo);
		}
		__builtin_amdgcn_sched_barrier(0);
		paced_slice<I + 1, READS, KIND, FIRST, COUNT>(cur, next, nw, nx, ns, lo, acc, src, dst, k0, wave);
	}
}

// ---- the paced form for the mixed arithmetic (e4m3 x int8 widened to f16; one wave per SIMD).  A slice of 32 bytes
// of K is two rounds of BN x BM f16 MFMAs (K = 16 each).  The operands of a round are widened one round ahead, a
// piece of four bytes behind each MFMA, so the conversions run in the shadow of the matrix core instead of in
// front of it; the raw fragments of the next slice are read during the first round, tiles requested in the second.
struct Wide {
	v8h w[BN];
	v8h x[BM];
};
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

// four 8-bit values -> four f16, exact (see widen8)
X17_DEV v4h widen4(u32 word, int kind) {
	v2h lo2, hi2;
	if (kind == 1) {
		lo2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, 1.0f, false);
		hi2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, 1.0f, true);
	} else {
		v2h const bias = {(_Float16)-1152.0f, (_Float16)-1152.0f};
		u32 const u = word ^ 0x80808080u;
		lo2 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) + bias;
		hi2 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) + bias;
	}
	return v4h{lo2[0], lo2[1], hi2[0], hi2[1]};
}
constexpr int WIDEN_PIECES = 2 * (BN + BM);      // per round: every fragment in two pieces of four bytes
// piece P of the operands of round H (0 / 1: bytes 0..7 / 8..15 of the lane's 16) of the raw fragments `f`,
// fragments in the order the MFMAs want them: w0, every x, then the other w
template <int P, int H>
X17_DEV void widen_piece(Wide &wd, Frags const &f) {
	constexpr int q = P / 2, p = P % 2, dw = 2 * H + p;
	if constexpr (q == 0 || q > BM) {
		constexpr int bn = q == 0 ? 0 : q - BM;
		v4h const r = widen4((u32)f.w[bn][0][dw], B_KIND);
		X17_UNROLL for (int i = 0; i < 4; ++i) wd.w[bn][4 * p + i] = r[i];
	} else {
		v4h const r = widen4((u32)f.x[q - 1][0][dw], A_KIND);
		X17_UNROLL for (int i = 0; i < 4; ++i) wd.x[q - 1][4 * p + i] = r[i];
	}
}
template <int FIRST, int LAST, int H>
X17_DEV void widen_range(Wide &wd, Frags const &f) {
	if constexpr (FIRST < LAST) {
		widen_piece<FIRST, H>(wd, f);
		widen_range<FIRST + 1, LAST, H>(wd, f);
	}
}
// One round.  NEXT_H < 0: nothing to widen (the tile's last round); else the next round's operands are round NEXT_H
// of `raw`.  READS: the raw fragments `rd` of slice `ns` of tiles (nw, nx) are read behind the first MFMAs.
// KIND / FIRST / COUNT: tile requests as in paced_slice.
template <int I, int NEXT_H, bool READS, int KIND, u32 FIRST, u32 COUNT>
X17_DEV void mixed_round(Wide const &cur, Wide &nxt, Frags const &raw, Frags &rd, u8 const *nw, u8 const *nx, u32 ns,
                         LaneOffsets const &lo, Acc (&acc)[BN][BM], u8 const *src, u8 *dst, u32 k0, u32 wave) {
	if constexpr (I < MFMAS_PER_SLICE) {
		constexpr int bn = I / BM, bm = I % BM;
		v16f const r = __builtin_amdgcn_mfma_f32_32x32x16_f16(cur.w[bn], cur.x[bm], __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0);
		acc[bn][bm] = __builtin_bit_cast(Acc, r);
		if constexpr (NEXT_H >= 0) {
			widen_range<I * WIDEN_PIECES / MFMAS_PER_SLICE, (I + 1) * WIDEN_PIECES / MFMAS_PER_SLICE, NEXT_H>(nxt, raw);
		}
		if constexpr (READS) {
			constexpr int R0 = I * READS_PER_SLICE / MFMAS_PER_SLICE, R1 = (I + 1) * READS_PER_SLICE / MFMAS_PER_SLICE;
			read_range<R0, R1>(rd, nw, nx, ns, lo);
		}
		constexpr u32 L0 = FIRST + I * COUNT / MFMAS_PER_SLICE, L1 = FIRST + (I + 1) * COUNT / MFMAS_PER_SLICE;
		if constexpr (KIND == 1) {
			issue_x_units<L0, L1>(src, dst, k0, wave, lo);
		} else if constexpr (KIND == 2) {
			issue_w_range<L0, L1>(src, dst, k0, wave, lo);
		}
		__builtin_amdgcn_sched_barrier(0);
		mixed_round<I + 1, NEXT_H, READS, KIND, FIRST, COUNT>(cur, nxt, raw, rd, nw, nx, ns, lo, acc, src, dst, k0, wave);
	}
}

} // namespace

extern "C" __global__ __launch_bounds__(gt::THREADS_PER_BLOCK)
__attribute__((amdgpu_waves_per_eu(gt::WAVES_PER_SIMD, gt::WAVES_PER_SIMD)))
void kernel(
	u8 const *a, u32 a_rows,
	u8 const *b, u32 b_rows,
	u8 *c
#if X17_EPILOGUE == 3
	, f32 *rrms
#elif X17_EPILOGUE == 2
	, i8 const *residual
#elif X17_EPILOGUE == 4
	, f32 const *row_scale, f32 const *col_scale
#elif X17_EPILOGUE == 5
	, u16 const *q_norm_scales          // bf16 [N_raw]
#elif X17_EPILOGUE == 6
	// a, b = q weights [X17_Q_COLS, K], c = q [M, X17_Q_COLS]; then:
	, f32 *rrms, u8 const *b_kv /* [N_raw - X17_Q_COLS, K] */, u8 *c_kv /* [M, N_raw - X17_Q_COLS] */
#endif
) {
	extern __shared__ __attribute__((aligned(1024))) u8 smem[];
	(void)b_rows;   // known at compile time, as in templates/basic_gemm/kernel.cu:18-21

	// ---- which tiles.  The kernel is persistent: workgroup g of G works on tiles g, g + G, ... and
	// any grid shape is accepted (with one workgroup per tile, as the reference launches it, every
	// workgroup runs the loop once).  The linear tile id is remapped so that each XCD (own L2) gets a
	// compact block of tiles -- the hardware deals workgroups round-robin to the 8 XCDs -- and tiles
	// are walked in bands of token-tiles so that co-resident tiles share weight and token panels.
	// A shape that is not a whole number of tiles (src/device/cuda/gemm.rs:605-614 accepts rows % 64 == 0 and raw
	// columns % 128 == 0) is covered by moving the last tile of a row or column of tiles back until it ends at the
	// matrix edge: it recomputes a few rows or columns of its neighbour and stores the same bytes again, and nothing
	// in the kernel needs a predicate.  (tile_coords hands out a tile's first row and first raw column.)
	u32 const tiles_m = (a_rows + gt::M_PER_BLOCK - 1) / gt::M_PER_BLOCK;
	constexpr u32 tiles_n = (N_RAW + gt::N_PER_BLOCK - 1) / gt::N_PER_BLOCK;
	u32 const total = tiles_m * tiles_n;
	u32 const n_groups = gridDim.x * gridDim.y * gridDim.z;
	u32 const group = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
	auto tile_coords = [&](u32 lin, u32 &tile_m, u32 &tile_n) {
		gt::TileOrigin const o = gt::tile_origin(lin, a_rows, N_RAW, gt::BAND);
		tile_m = o.m;
		tile_n = o.n;
	};
	if (group >= total) {
		return;
	}

	u32 const tid = threadIdx.x;
	u32 const lane = tid % 64;
	u32 const wave = __builtin_amdgcn_readfirstlane(tid / 64);
	u32 const wm = wave / gt::WAVES_N;
	u32 const wn = wave % gt::WAVES_N;

	LaneOffsets lo;
	{
		// (row inside a load unit and logical chunk of the stored chunk position: gemm_tile.h)
		u32 even_odd_x[2], even_odd_w[2];
		X17_UNROLL for (u32 odd = 0; odd < 2; ++odd) {
			u32 const chunk = gt::lane_chunk(lane, odd);
			even_odd_x[odd] = gt::x_lane_row(lane) * K_TOTAL + 16 * chunk;
			even_odd_w[odd] = gt::w_lane_row(lane, NATURAL_COLS) * K_TOTAL + 16 * chunk;
		}
		if constexpr (LANE_UNIT_OFFSETS) {
			u32 const w_first = wave * W_UNITS * UNIT_ROWS;
			X17_UNROLL for (u32 u = 0; u < X_UNITS; ++u) lo.x_src[u] = even_odd_x[u & 1] + u * UNIT_ROWS * K_TOTAL;
			X17_UNROLL for (u32 u = 0; u < W_UNITS; ++u) {
				lo.w_src[u] = even_odd_w[u & 1] + (w_unit_row(w_first + u * UNIT_ROWS) - w_unit_row(w_first)) * K_TOTAL;
			}
		} else {
			X17_UNROLL for (u32 odd = 0; odd < 2; ++odd) {
				lo.x_src[odd] = even_odd_x[odd];
				lo.w_src[odd] = even_odd_w[odd];
			}
		}
		lo.frag_row = (lane % 32) * ROW_BYTES;
		lo.half = lane / 32;
		lo.swz = ((lane % 32) >> SWZ_SHIFT) & (CHUNKS - 1);
	}

	// ---- main loop.  Rings of XS token tiles and WS weight tiles in LDS; step ks consumes ring positions
	// ks % XS and ks % WS while the tiles of the following steps are in flight.  The one barrier per step sits
	// before the last slice's MFMAs, when every wave holds the last fragments of the step in registers: behind
	// it both positions are free, so the weight tile of step ks+WS and the token tile of step ks+XS are
	// requested there, and the first fragments of step ks+1 are fetched, so LDS latency is covered by
	// matrix-core time across the step boundary too.  The load stream runs across tile boundaries: the last
	// steps of a tile already fetch the first steps of the workgroup's next tile, which land while the epilogue
	// runs.  (a K shorter than the ring cannot prefetch across tiles: each tile then starts with its own prologue)
	static_assert(XS == WS || WS == 2, "a deeper token ring is supported on top of a two-deep weight ring");
	constexpr bool CROSS_TILE = K_STEPS >= XS;
	// Paced form: a step requests its token tile (step + XS - 1, into the position the PREVIOUS step's barrier
	// freed) during its first slices and its weight tile (step + WS) behind its own barrier, every request behind
	// an MFMA.  The pattern is the same in every step of every tile -- where nothing is left to fetch the request
	// is repeated from the tile's start into a position that no step reads again -- so no branch sits between
	// the MFMAs and the wait before a barrier is always "all but the token tile just requested".
	// (e4m3 fragments are twice the size: two such waves per SIMD do not fit the pinned order into 256 registers)
	constexpr bool PACED = WS == 2 && XS == 3 && CROSS_TILE && SLICES >= 2 && (MMA == 0 || gt::WAVES_PER_SIMD == 1);
	u32 const x_off = wm * gt::WAVE_M * ROW_BYTES + lo.frag_row;
	u32 const w_off = W_RING_OFFSET + wn * gt::WAVE_N * ROW_BYTES + lo.frag_row;

	// the weight rows of the tile whose first raw column is `col`: one matrix, or (fused q + kv) the q weights
	// followed by the kv weights
	auto weight_tile = [&](u32 col) -> u8 const * {
#if X17_EPILOGUE == 6
		static_assert(X17_Q_COLS % gt::N_PER_BLOCK == 0 && N_RAW - X17_Q_COLS >= gt::N_PER_BLOCK, "q and kv parts are whole tiles / at least a tile");
		return col < X17_Q_COLS ? b + (size_t)col * K_TOTAL : b_kv + (size_t)(col - X17_Q_COLS) * K_TOTAL;
#else
		return b + (size_t)col * K_TOTAL;
#endif
	};
	u32 tile_m, tile_n;
	tile_coords(group, tile_m, tile_n);
	u8 const *a_tile = a + (size_t)tile_m * K_TOTAL;
	u8 const *b_tile = weight_tile(tile_n);
	// the first steps of a tile nobody prefetched, in the order the waits of the main loop assume
	// (token tile s, weight tile s, ..., then the extra token tile of a deeper token ring)
	auto prologue = [&]() __attribute__((always_inline)) {
		X17_UNROLL for (u32 s = 0; s < WS; ++s) {
			if (s < K_STEPS) {
				issue_x_loads(a_tile, smem + s * X_TILE_BYTES, s * gt::K_STEP, wave, lo);
				issue_w_loads(b_tile, smem + W_RING_OFFSET + s * W_TILE_BYTES, s * gt::K_STEP, wave, lo);
			}
		}
		if constexpr (XS > WS && CROSS_TILE && !PACED) {
			issue_x_loads(a_tile, smem + WS * X_TILE_BYTES, WS * gt::K_STEP, wave, lo);
		}
		wait_vmcnt<0>();
		__builtin_amdgcn_s_barrier();
	};
	prologue();

	u32 xb = 0, wb = 0;                            // ring positions of the step being consumed
	for (u32 lin = group; lin < total; lin += n_groups) {
		bool const first_tile = lin == group;
		bool const more_tiles = lin + n_groups < total;
		bool const has_next = CROSS_TILE && more_tiles;      // prefetch the next tile's first steps
		u32 next_m = 0, next_n = 0;
		if (more_tiles) {
			tile_coords(lin + n_groups, next_m, next_n);
		}
		u8 const *a_next = a + (size_t)next_m * K_TOTAL;
		u8 const *b_next = weight_tile(next_n);
		if constexpr (!CROSS_TILE) {
			if (!first_tile) {
				__builtin_amdgcn_s_waitcnt(0xC07F);        // lgkmcnt(0)
				__builtin_amdgcn_s_barrier();              // nobody still reads the previous tile's buffers
				xb = 0;
				wb = 0;
				prologue();
			}
		}

		Acc acc[BN][BM];   // [bn][bm]
		X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
			X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
				X17_UNROLL for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0;
			}
		}

		// (step 0 of this tile is visible: the wait and the barrier were the previous tile's last ones)
		Frags frags[2];
		load_frags(frags[0], smem + wb * W_TILE_BYTES + w_off, smem + xb * X_TILE_BYTES + x_off, 0, lo);
		[[maybe_unused]] Wide wide[2];
		if constexpr (PACED && MMA == 2) {
			widen_range<0, WIDEN_PIECES, 0>(wide[0], frags[0]);      // (the only conversions of a tile no MFMA covers)
		}

		auto paced_k_loop = [&]<bool LOADER>() __attribute__((always_inline)) {
			constexpr u32 X_SLICES = SLICES >= 4 ? 2 : 1;                 // slices that carry token requests
			constexpr u32 X_PER_SLICE = X_UNITS / X_SLICES;
			// (values, not the captured variables: a choice between two captured pointers would keep them in memory)
			u8 const *const at = a_tile, *const an = a_next, *const bt = b_tile, *const bnx = b_next;
			bool const hn = has_next;
			// (no unroll pragma here: with the issue order pinned, unrolling a short loop completely costs no registers,
			// and the rolled form of this loop spills)
			for (u32 ks = 0; ks < K_STEPS; ++ks) {
				u32 const next_xb = xb + 1 == XS ? 0 : xb + 1;
				u32 const next_wb = wb + 1 == WS ? 0 : wb + 1;
				u32 const prev_xb = xb == 0 ? XS - 1 : xb - 1;
				u32 const x_step = ks + XS - 1, w_step = ks + WS;
				bool const x_here = x_step < K_STEPS, w_here = w_step < K_STEPS;
				u8 const *lx = (x_here || !hn) ? at : an;
				u8 const *lw = (w_here || !hn) ? bt : bnx;
				u32 const x_k0 = (x_here ? x_step : (hn ? x_step - K_STEPS : 0)) * gt::K_STEP;
				u32 const w_k0 = (w_here ? w_step : (hn ? w_step - K_STEPS : 0)) * gt::K_STEP;
				u8 *x_dst = smem + prev_xb * X_TILE_BYTES;
				u8 *w_dst = smem + W_RING_OFFSET + wb * W_TILE_BYTES;
				u8 const *w_tile = smem + wb * W_TILE_BYTES + w_off;
				u8 const *x_tile = smem + xb * X_TILE_BYTES + x_off;
				u8 const *nw_tile = smem + next_wb * W_TILE_BYTES + w_off;
				u8 const *nx_tile = smem + next_xb * X_TILE_BYTES + x_off;
				auto slices = [&]<u32 S>(auto &&self) __attribute__((always_inline)) {
					if constexpr (MMA == 2) {
						// first round: the operands of the second round are widened from the same raw fragments, the
						// next slice's raw fragments are read (behind the step's barrier when they belong to the next
						// step); second round: the next slice's first operands are widened, tiles are requested
						constexpr bool LAST = S + 1 == SLICES;
						constexpr int KIND = !LOADER ? 0 : (LAST ? 2 : (S < X_SLICES ? 1 : 0));
						constexpr u32 FIRST = LAST ? 0 : S * X_PER_SLICE, COUNT = LAST ? W_UNITS : X_PER_SLICE;
						u8 const *src = LAST ? lw : lx;
						u8 *dst = LAST ? w_dst : x_dst;
						u32 const k0 = LAST ? w_k0 : x_k0;
						if constexpr (LAST) {
							wait_vmcnt<X_UNITS>();
							__builtin_amdgcn_s_waitcnt(0xC07F);
							__builtin_amdgcn_s_barrier();
							// (the same code in a tile's last step, where what it reads and widens is never used: two
							// copies of the rounds would have to agree on where 256 accumulators live when they meet)
							mixed_round<0, 1, true, 0, 0, 0>(wide[0], wide[1], frags[S & 1], frags[(S + 1) & 1], nw_tile, nx_tile, 0, lo, acc, src, dst, k0, wave);
							mixed_round<0, 0, false, KIND, FIRST, COUNT>(wide[1], wide[0], frags[(S + 1) & 1], frags[S & 1], nw_tile, nx_tile, 0, lo, acc, src, dst, k0, wave);
						} else {
							mixed_round<0, 1, true, 0, 0, 0>(wide[0], wide[1], frags[S & 1], frags[(S + 1) & 1], w_tile, x_tile, S + 1, lo, acc, src, dst, k0, wave);
							mixed_round<0, 0, false, KIND, FIRST, COUNT>(wide[1], wide[0], frags[(S + 1) & 1], frags[S & 1], w_tile, x_tile, S + 1, lo, acc, src, dst, k0, wave);
							self.template operator()<S + 1>(self);
						}
					} else if constexpr (S + 1 < SLICES) {
						constexpr int KIND = LOADER && S < X_SLICES ? 1 : 0;
						paced_slice<0, true, KIND, S * X_PER_SLICE, X_PER_SLICE>(
							frags[S & 1], frags[(S + 1) & 1], w_tile, x_tile, S + 1, lo, acc, lx, x_dst, x_k0, wave);
						self.template operator()<S + 1>(self);
					} else {
						// the next step's tiles have landed once all but the token tile just requested have;
						// this wave is done reading this step's tiles
						wait_vmcnt<X_UNITS>();
						__builtin_amdgcn_s_waitcnt(0xC07F);
						__builtin_amdgcn_s_barrier();
						constexpr int KIND = LOADER ? 2 : 0;
						if (ks + 1 < K_STEPS) {
							paced_slice<0, true, KIND, 0, W_UNITS>(
								frags[S & 1], frags[(S + 1) & 1], nw_tile, nx_tile, 0, lo, acc, lw, w_dst, w_k0, wave);
						} else {
							paced_slice<0, false, KIND, 0, W_UNITS>(
								frags[S & 1], frags[(S + 1) & 1], nw_tile, nx_tile, 0, lo, acc, lw, w_dst, w_k0, wave);
						}
					}
				};
				slices.template operator()<0>(slices);
				xb = next_xb;
				wb = next_wb;
			}
		};
		if constexpr (PACED) {
			if (WAVES == LOADER_WAVES || wave < LOADER_WAVES) {
				paced_k_loop.template operator()<true>();
			} else {
				paced_k_loop.template operator()<false>();
			}
		} else {
		X17_K_LOOP_PRAGMA
		for (u32 ks = 0; ks < K_STEPS; ++ks) {
			u32 const next_xb = xb + 1 == XS ? 0 : xb + 1;
			u32 const next_wb = wb + 1 == WS ? 0 : wb + 1;
			// the tiles requested behind this step's barrier: weight step ks+WS, token step ks+XS (of this
			// output tile or of the workgroup's next one)
			u32 const w_step = ks + WS, x_step = ks + XS;
			bool const w_here = w_step < K_STEPS, x_here = x_step < K_STEPS;
			u8 const *lw = w_here ? b_tile : b_next;
			u8 const *lx = x_here ? a_tile : a_next;
			u32 const w_k0 = (w_here ? w_step : w_step - K_STEPS) * gt::K_STEP;
			u32 const x_k0 = (x_here ? x_step : x_step - K_STEPS) * gt::K_STEP;
			u8 const *w_tile = smem + wb * W_TILE_BYTES + w_off;
			u8 const *x_tile = smem + xb * X_TILE_BYTES + x_off;
			X17_UNROLL for (u32 s = 0; s < SLICES; ++s) {
				bool reads = true;
				if (s + 1 < SLICES) {
					load_frags(frags[(s + 1) & 1], w_tile, x_tile, s + 1, lo);
				} else if (ks + 1 < K_STEPS || has_next) {
					// Step ks+1 (or the next tile's step 0) must have landed; what was requested after its weight
					// tile may stay in flight: the token tile of step ks+2 when the token ring is the deeper one,
					// and up to WS-2 whole steps.  After an epilogue its stores share the counter with the loads:
					// wait for everything then.
					u32 const later_steps = has_next ? WS - 2 : (K_STEPS - 2 - ks < WS - 2 ? K_STEPS - 2 - ks : WS - 2);
					bool const token_tile_behind = has_next || ks + 2 < K_STEPS;
					bool const stores_pending = !first_tile && ks + 1 < WS;
					if (stores_pending) {
						wait_vmcnt<0>();
					} else {
						wait_step(later_steps, token_tile_behind);
					}
					__builtin_amdgcn_s_waitcnt(0xC07F);    // lgkmcnt(0): this wave is done reading this step's tiles
					__builtin_amdgcn_s_barrier();
					if (w_here || has_next) {
						issue_w_loads(lw, smem + W_RING_OFFSET + wb * W_TILE_BYTES, w_k0, wave, lo);
					}
					if (x_here || has_next) {
						issue_x_loads(lx, smem + xb * X_TILE_BYTES, x_k0, wave, lo);
					}
					if (ks + 1 < K_STEPS) {
						load_frags(frags[(s + 1) & 1], smem + next_wb * W_TILE_BYTES + w_off, smem + next_xb * X_TILE_BYTES + x_off, 0, lo);
					} else {
						reads = false;
					}
				} else {
					reads = false;
				}
				mma_slice(frags[s & 1], acc);
				if (s + 1 < SLICES) {
					interleave_slice<0>(reads);
				} else {
					interleave_slice<LOADS_PER_STAGE>(reads);
				}
			}
			xb = next_xb;
			wb = next_wb;
		}
		}

	// ---- epilogue.  Lane owns token (32*bm + lane%32) of its wave and raw columns
	// LANE_COLS*(lane/32) + 16*bn + r of its wave, r = accumulator register index.
	u32 const row0 = tile_m + wm * gt::WAVE_M + lane % 32;
	u32 const n0 = tile_n + wn * gt::WAVE_N + LANE_COLS * lo.half;

	X17_UNROLL for (int bm = 0; bm < BM; ++bm) {
		if constexpr (gt::WAVES_PER_SIMD == 1) {
			// Accumulators in the second half of the register file (where the vector ALU cannot read them) are copied
			// out row by row: pinning the later rows where they are keeps the register allocator from copying all
			// 256 out at once behind the K loop, which leaves no register for anything else.
			X17_UNROLL for (int later = bm + 1; later < BM; ++later) {
				X17_UNROLL for (int bn = 0; bn < BN; ++bn) asm volatile("" : "+a"(acc[bn][later]));
			}
		}
		u32 row = row0 + 32 * bm;
		f32 x[LANE_COLS];
		X17_UNROLL for (int bn = 0; bn < BN; ++bn) {
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
#elif X17_EPILOGUE == 4
		DequantEpilogue::run(x, c, row, n0, row_scale, col_scale);
#elif X17_EPILOGUE == 3
		NaturalWriters::l2norm_row(x, c, rrms, row, tile_n + wn * gt::WAVE_N, N_RAW, lo.half);
#elif X17_EPILOGUE == 5
		NaturalWriters::qnorm_row(x, c, q_norm_scales, row, tile_n + wn * gt::WAVE_N, lo.half);
#else
		{
			constexpr u32 Q_COLS = X17_Q_COLS;
			u32 const col0 = tile_n + wn * gt::WAVE_N;
			if (col0 < Q_COLS) {
				NaturalWriters::scale_row(x, c, row, col0, Q_COLS, lo.half);
			} else {
				NaturalWriters::l2norm_row(x, c_kv, rrms, row, col0 - Q_COLS, N_RAW - Q_COLS, lo.half);
			}
		}
#endif
	}

		tile_m = next_m;
		tile_n = next_n;
		a_tile = a_next;
		b_tile = b_next;
	}
	// the paced form's last requests go nowhere useful, but they write LDS: they must land before the workgroup ends
	wait_vmcnt<0>();
}
