// x17_device.h -- device-side basics shared by every gfx950 kernel of this library:
// fixed-width types, the 8-bit number formats of the reference, and the scalar math the
// epilogues and the softmax are built from.
//
// Number formats (reference: cuda/utils_b8.cuh:7-10, 629-657):
//   FixedI8  int8 with 3 fractional bits (real = code / 8), clamped to +-127
//   E4m3     OCP e4m3fn restricted to what the reference emits: no subnormals, no NaN,
//            no -0, magnitude <= 448, rounding half away from zero
//
// Transcendentals come in two builds, selected by X17_STRICT_MATH:
//   1  small deterministic f32 algorithms (fma/add/mul/integer ops only), bit-reproducible
//      on any IEEE-754 machine; the build parity tests run
//   0  the CDNA transcendental instructions (v_exp_f32, v_log_f32, v_rcp_f32, v_rsq_f32),
//      1 ulp class, for speed; outputs may differ from the strict build by one code
// The reference has the same switch for the same reason (X17_PRECISE_MATH,
// cuda/utils_core.cuh:30-32, 259-385).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef X17_STRICT_MATH
#define X17_STRICT_MATH 1
#endif

typedef uint8_t u8;
typedef int8_t i8;
typedef uint16_t u16;
typedef uint32_t u32;
typedef int32_t i32;
typedef uint64_t u64;
typedef float f32;
typedef double f64;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

#define X17_DEV __device__ __forceinline__
#define X17_UNROLL _Pragma("unroll")

#define X17_GLOBAL_PTR(p) ((const void __attribute__((address_space(1))) *)(p))
#define X17_LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))

namespace x17 {

X17_DEV u32 f2u(f32 f) { return __builtin_bit_cast(u32, f); }
X17_DEV f32 u2f(u32 u) { return __builtin_bit_cast(f32, u); }
X17_DEV f32 fmaf32(f32 a, f32 b, f32 c) { return __builtin_fmaf(a, b, c); }

// ------------------------------------------------------------------ conversions

// cuda/utils_b8.cuh:629-632
X17_DEV i32 f32_to_fixedi8(f32 v) {
	f32 c = __builtin_fmaxf(-127.0f, __builtin_fminf(127.0f, v));
	return (i32)__builtin_rintf(c);
}

// cuda/utils_b8.cuh:636-647
X17_DEV u32 f32_to_e4m3(f32 v) {
	u32 tmp = f2u(v);
	u32 sign = (tmp >> 24) & 0x80u;
	u32 rest = tmp & 0x7FFFFFFFu;
	constexpr u32 mn = (120u << 23) + (0xfu << 19);
	constexpr u32 mx = (135u << 23) + (0xcu << 19);
	u32 rounded = (rest + ((1u << 19) - (120u << 23))) >> 20;
	u32 clamped = rest > mx ? 0x7eu : rounded;
	return rest < mn ? 0u : (sign | clamped);
}

// cuda/utils_b8.cuh:652-657, widened to f32
X17_DEV f32 e4m3_to_f32(u32 c) {
	u32 sign = (c & 0x80u) << 24;
	u32 rest = (c & 0x7Fu) << 20;
	return rest == 0 ? 0.0f : u2f((sign | rest) + (120u << 23));
}

// e4m3 byte -> bf16 bits (exact): used to feed the bf16 matrix cores
X17_DEV u32 e4m3_to_bf16_bits(u32 c) {
	u32 sign = (c & 0x80u) << 8;
	u32 rest = (c & 0x7Fu) << 4;
	return rest == 0 ? 0u : ((sign | rest) + (120u << 7));
}

// f32 -> bf16 bits, round to nearest even (finite inputs)
X17_DEV u32 f32_to_bf16_rne(f32 v) {
	u32 b = f2u(v);
	return (b + 0x7FFFu + ((b >> 16) & 1u)) >> 16;
}
// Two of them packed into one word, `lo` in the low half: the gfx950 packed conversion (one instruction for the
// pair; round to nearest even like the above).
X17_DEV u32 pack2_bf16_rne(f32 lo, f32 hi) {
	typedef float pair_f32 __attribute__((ext_vector_type(2)));
	typedef __bf16 pair_bf16 __attribute__((ext_vector_type(2)));
	return __builtin_bit_cast(u32, __builtin_convertvector(pair_f32{lo, hi}, pair_bf16));
}

// Four FixedI8 codes packed into one word (a in the low byte).  Same values as f32_to_fixedi8:
// clamp, then add 1.5 * 2^23 -- the add rounds to an integer, ties to even, exactly like rint, and
// leaves the two's-complement code in the low byte of the float -- then gather the four low bytes.
X17_DEV u32 pack4_fixedi8(f32 a, f32 b, f32 c, f32 d) {
	constexpr f32 MAGIC = 12582912.0f;
	u32 ua = f2u(__builtin_amdgcn_fmed3f(a, -127.0f, 127.0f) + MAGIC);
	u32 ub = f2u(__builtin_amdgcn_fmed3f(b, -127.0f, 127.0f) + MAGIC);
	u32 uc = f2u(__builtin_amdgcn_fmed3f(c, -127.0f, 127.0f) + MAGIC);
	u32 ud = f2u(__builtin_amdgcn_fmed3f(d, -127.0f, 127.0f) + MAGIC);
	u32 lo = __builtin_amdgcn_perm(ub, ua, 0x0c0c0400u);     // bytes: a0, b0, 0, 0
	u32 hi = __builtin_amdgcn_perm(ud, uc, 0x04000c0cu);     // bytes: 0, 0, c0, d0
	return lo | hi;
}

// The same encoder on the gfx950 conversion instruction, for the hardware-transcendental builds: magnitudes below
// the reference's threshold (1.9375 * 2^-7) are zeroed first (the instruction would produce subnormal codes, the
// reference's dialect has none), the rest is clamped to +-448 (the instruction answers overflow with NaN) and
// converted two at a time.  One difference remains: a value exactly half way between two e4m3 neighbours goes to
// the even one here and away from zero in the reference's encoder (one f32 in 2^20 of a binade).
X17_DEV f32 e4m3_flush_clamp(f32 v) {
	f32 const kept = __builtin_fabsf(v) < 0.01513671875f ? 0.0f : v;          // 1.9375 * 2^-7 (bits 0x3C780000)
	return __builtin_amdgcn_fmed3f(kept, -448.0f, 448.0f);
}
X17_DEV u32 pack4_e4m3_hw(f32 a, f32 b, f32 c, f32 d) {
	int w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_flush_clamp(a), e4m3_flush_clamp(b), 0, false);
	w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_flush_clamp(c), e4m3_flush_clamp(d), w, true);
	return (u32)w;
}

template<int STORE> X17_DEV u32 pack4_store(f32 a, f32 b, f32 c, f32 d) {
	if constexpr (STORE == 1) {
#if defined(X17_STRICT_MATH) && !X17_STRICT_MATH
		return pack4_e4m3_hw(a, b, c, d);
#else
		return f32_to_e4m3(a) | (f32_to_e4m3(b) << 8) | (f32_to_e4m3(c) << 16) | (f32_to_e4m3(d) << 24);
#endif
	} else {
		return pack4_fixedi8(a, b, c, d);
	}
}

template<int STORE> X17_DEV u32 store_convert(f32 v) {
	if constexpr (STORE == 1) {
		return f32_to_e4m3(v);
	} else {
		return (u32)f32_to_fixedi8(v) & 0xFFu;
	}
}

// ------------------------------------------------------------------ deterministic scalar math
// Same algorithms, constants and operation order as the CPU checker uses; see the header note.

namespace strict {
	// 2^x; results below 2^-125 flush to zero
	X17_DEV f32 ex2(f32 x) {
		if (!(x >= -125.0f)) return 0.0f;
		x = __builtin_fminf(x, 126.0f);
		f32 n = __builtin_rintf(x);
		f32 f = x - n;
		f32 p = 0.00015453163359779865f;
		p = fmaf32(p, f, 0.0013390863314270973f);
		p = fmaf32(p, f, 0.009618083015084267f);
		p = fmaf32(p, f, 0.055503569543361664f);
		p = fmaf32(p, f, 0.24022650718688965f);
		p = fmaf32(p, f, 0.6931471824645996f);
		p = fmaf32(p, f, 1.0f);
		i32 ni = (i32)n;
		return u2f(f2u(p) + ((u32)ni << 23));
	}

	// log2(x), x positive normal finite
	X17_DEV f32 lg2(f32 x) {
		u32 b = f2u(x);
		i32 e = (i32)(b >> 23) - 127;
		f32 m = u2f((b & 0x007FFFFFu) | 0x3F800000u);
		if (m > 1.41421354f) { m = m * 0.5f; e += 1; }
		f32 t = m - 1.0f;
		f32 q = -0.10749789327383041f;
		q = fmaf32(q, t, 0.18476033210754395f);
		q = fmaf32(q, t, -0.19138838350772858f);
		q = fmaf32(q, t, 0.20485764741897583f);
		q = fmaf32(q, t, -0.23960812389850616f);
		q = fmaf32(q, t, 0.28855255246162415f);
		q = fmaf32(q, t, -0.36069655418395996f);
		q = fmaf32(q, t, 0.48089852929115295f);
		q = fmaf32(q, t, -0.7213473320007324f);
		q = fmaf32(q, t, 1.4426950216293335f);
		return fmaf32(t, q, (f32)e);
	}

	// 1/x, x positive normal finite
	X17_DEV f32 rcp(f32 x) {
		f32 r = u2f(0x7EF311C7u - f2u(x));
		X17_UNROLL for (int i = 0; i < 4; ++i) {
			f32 e = fmaf32(-x, r, 1.0f);
			r = fmaf32(r, e, r);
		}
		return r;
	}

	// 1/sqrt(x), x positive normal finite
	X17_DEV f32 rsq(f32 x) {
		f32 y = u2f(0x5F3759DFu - (f2u(x) >> 1));
		f32 hx = 0.5f * x;
		X17_UNROLL for (int i = 0; i < 4; ++i) {
			f32 t = hx * y;
			t = fmaf32(-t, y, 1.5f);
			y = y * t;
		}
		return y;
	}

	X17_DEV f32 tanh(f32 x) {
		f32 a = __builtin_fminf(__builtin_fabsf(x), 10.0f);
		f32 e = ex2(a * 2.8853900432586670f);
		f32 r = rcp(e + 1.0f);
		f32 t = fmaf32(-2.0f, r, 1.0f);
		return __builtin_copysignf(t, x);
	}
}

namespace hw {
	X17_DEV f32 ex2(f32 x) { return __builtin_amdgcn_exp2f(x); }
	X17_DEV f32 lg2(f32 x) { return __builtin_amdgcn_logf(x); }
	X17_DEV f32 rcp(f32 x) { return __builtin_amdgcn_rcpf(x); }
	X17_DEV f32 rsq(f32 x) { return __builtin_amdgcn_rsqf(x); }
	X17_DEV f32 tanh(f32 x) {
		f32 a = __builtin_fminf(__builtin_fabsf(x), 10.0f);
		f32 e = ex2(a * 2.8853900432586670f);
		f32 r = rcp(e + 1.0f);
		f32 t = fmaf32(-2.0f, r, 1.0f);
		return __builtin_copysignf(t, x);
	}
}

#if X17_STRICT_MATH
namespace sfu = strict;
#else
namespace sfu = hw;
#endif

// ------------------------------------------------------------------ compile-time constants
// The reference derives epilogue constants in double with its own bisection square root
// (cuda/utils_core.cuh:151-210); the f32 rounding of a constant can hinge on the last bit of
// the double, so the same routine is used here.

constexpr f64 constexpr_sqrt(f64 x) {
	if (x < 0.0 || x != x) return __builtin_nan("");
	if (x == 0.0) return 0.0;
	if (x == __builtin_inf()) return x;
	f64 above = x > 1.0 ? x : 1.0;
	f64 below = 0.0;
	bool stop = false;
	while (!stop) {
		f64 v = (0.5 * above) + (0.5 * below);
		f64 t = x / v;
		f64 new_above = t <= v ? v : above;
		f64 new_below = t >= v ? v : below;
		stop = (new_above == above) && (new_below == below);
		above = new_above;
		below = new_below;
	}
	f64 above_err = (above * above) - x;
	f64 below_err = x - (below * below);
	return above_err > below_err ? below : above;
}

constexpr f64 constexpr_inv_sqrt(f64 x) {
	if (x < 0.0 || x != x) return __builtin_nan("");
	if (x == 0.0) return __builtin_inf();
	if (x == __builtin_inf()) return 0.0;
	f64 above = 2.0 / constexpr_sqrt(x);
	f64 below = 0.0;
	bool stop = false;
	while (!stop) {
		f64 v = (0.5 * above) + (0.5 * below);
		f64 t = (x * v) * v;
		f64 new_above = t >= 1.0 ? v : above;
		f64 new_below = t <= 1.0 ? v : below;
		stop = (new_above == above) && (new_below == below);
		above = new_above;
		below = new_below;
	}
	f64 above_err = ((x * above) * above) - 1.0;
	f64 below_err = 1.0 - ((x * below) * below);
	return above_err > below_err ? below : above;
}

constexpr f64 INV_PI = 0.318309886183790671537767526745028724;
constexpr f64 LN2 = 0.693147180559945309417232121458176568;

} // namespace x17
