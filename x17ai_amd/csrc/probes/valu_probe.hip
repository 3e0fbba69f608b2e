// valu_probe.hip -- what a SIMD of the machine at hand issues.  Measurement aid only.
//  * X17_PROBE_OP < 100: loops of ONE instruction on sixteen independent registers -- how fast a SIMD issues it, as a
//    function of the wavefronts that share it.  The figures are not what the 4-cycles-per-instruction rule of thumb gives.
//  * X17_PROBE_OP >= 100: composite loops without memory traffic: matrix instructions next to vector instructions
//    (how much vector work hides behind one), and the instruction mix of one 32-key step of the attention kernel's
//    speed build in the kernel's order -- the time that mix needs when nothing waits for memory or a barrier.
//
// common.h provides X17_PROBE_OP, an index into the table below.  One workgroup = one wavefront; the host
// launches 1024 * w of them for w wavefronts per SIMD.
#include "common.h"
#include "x17_device.h"

using namespace x17;

#if X17_PROBE_OP == 0
#define X17_OP "v_fma_f32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 1
#define X17_OP "v_add_f32 %0, %0, %0"
#elif X17_PROBE_OP == 2
#define X17_OP "v_mul_f32 %0, %0, %0"
#elif X17_PROBE_OP == 3
#define X17_OP "v_xor_b32 %0, 0x80808080, %0"
#elif X17_PROBE_OP == 4
#define X17_OP "v_add_u32 %0, %0, %0"
#elif X17_PROBE_OP == 5
#define X17_OP "v_cvt_f32_i32 %0, %0"
#elif X17_PROBE_OP == 6
#define X17_OP "v_rndne_f32 %0, %0"
#elif X17_PROBE_OP == 7
#define X17_OP "v_max_f32 %0, %0, %0"
#elif X17_PROBE_OP == 8
#define X17_OP "v_max3_i32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 9
#define X17_OP "v_perm_b32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 10
#define X17_OP "v_cvt_pkrtz_f16_f32 %0, %0, %0"
#elif X17_PROBE_OP == 11
#define X17_OP "v_pk_mul_f16 %0, %0, %0"
#elif X17_PROBE_OP == 12
#define X17_OP "v_pk_fma_f16 %0, %0, %0, %0"
#elif X17_PROBE_OP == 13
#define X17_OP "v_pk_add_f16 %0, %0, %0"
#elif X17_PROBE_OP == 14
#define X17_OP "v_med3_f32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 15
#define X17_OP "v_exp_f32 %0, %0"
#elif X17_PROBE_OP == 16
#define X17_OP "v_rcp_f32 %0, %0"
#elif X17_PROBE_OP == 17
#define X17_OP "v_log_f32 %0, %0"
#elif X17_PROBE_OP == 18
#define X17_OP "v_permlane32_swap_b32 %0, %0"
#elif X17_PROBE_OP == 19
#define X17_OP "s_add_u32 %1, %1, 3"
#elif X17_PROBE_OP == 20
#define X17_OP "v_lshl_add_u32 %0, %0, 16, %0"
#elif X17_PROBE_OP == 21
#define X17_OP "v_add3_u32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 22
#define X17_OP "v_pack_b32_f16 %0, %0, %0"
#elif X17_PROBE_OP == 23
#define X17_OP "v_and_or_b32 %0, %0, %0, %0"
#elif X17_PROBE_OP == 24
#define X17_OP "v_cndmask_b32 %0, %0, %0, vcc"
#elif X17_PROBE_OP == 25
#define X17_OP "v_cmp_lt_f32 vcc, %0, %0"
#elif X17_PROBE_OP == 26
#define X17_OP "v_fmaak_f32 %0, %0, %0, 0x4b406400"
#elif X17_PROBE_OP == 27
#define X17_OP "v_mov_b32 %0, %0"
#elif X17_PROBE_OP >= 100 && X17_PROBE_OP < 110
#define X17_COMPOSITE 1
#else
#error "unknown X17_PROBE_OP"
#endif

#ifndef X17_COMPOSITE
extern "C" __global__ __launch_bounds__(64)
void kernel(f32 const *src, u32 iterations, f32 *out) {
	f32 r[16];
	X17_UNROLL for (int i = 0; i < 16; ++i) r[i] = src[threadIdx.x + i];
	u32 s = iterations;
	for (u32 it = 0; it < iterations; ++it) {
		X17_UNROLL for (int i = 0; i < 16; ++i) asm volatile(X17_OP : "+v"(r[i]), "+s"(s) : : "scc", "vcc");
	}
	f32 sum = f32(s);
	X17_UNROLL for (int i = 0; i < 16; ++i) sum += r[i];
	out[(size_t)blockIdx.x * 64 + threadIdx.x] = sum;
}
#else
// Every instruction is a volatile asm statement, so the order below is the order issued.  No vector instruction touches an
// accumulator of a matrix instruction; the sums written at the end only keep the loop alive.
#define A_OP(i) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(r[(i) % 16]))
#define B_OP(i) asm volatile("v_perm_b32 %0, %0, %0, %0" : "+v"(r[(i) % 16]))
#define C_OP(i) asm volatile("v_exp_f32 %0, %0" : "+v"(r[(i) % 16]))
#define S_OP() asm volatile("s_add_u32 %0, %0, 3" : "+s"(sc) : : "scc")
#define W_OP() asm volatile("s_waitcnt lgkmcnt(0)")
#define L_OP(i) asm volatile("ds_read_b128 %0, %1" : "=v"(lv[(i) % 2]) : "v"(laddr))
#define SM() asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(sacc) : "v"(a), "v"(b))
#define PM(j) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(oacc[j]) : "v"(ha), "v"(hb))

extern "C" __global__ __launch_bounds__(64)
void kernel(f32 const *src, u32 iterations, f32 *out) {
	__shared__ v4i lds[64];
	f32 r[16];
	X17_UNROLL for (int i = 0; i < 16; ++i) r[i] = src[threadIdx.x + i];
	v4i a = {1, 2, 3, 4}, b = {5, 6, 7, 8};
	v4i lv[2] = {a, b};
	v8h ha = {1, 2, 3, 4, 5, 6, 7, 8}, hb = {1, 1, 1, 1, 1, 1, 1, 1};
	v16i sacc;
	v16f oacc[4];
	X17_UNROLL for (int e = 0; e < 16; ++e) {
		sacc[e] = 0;
		X17_UNROLL for (int j = 0; j < 4; ++j) oacc[j][e] = 0.0f;
	}
	lds[threadIdx.x] = a;
	__syncthreads();
	u32 const laddr = threadIdx.x * 16;
	u32 sc = iterations;
	for (u32 it = 0; it < iterations; ++it) {
#if X17_PROBE_OP == 100          // four f16 matrix instructions on four accumulators
		PM(0); PM(1); PM(2); PM(3);
#elif X17_PROBE_OP == 101        // ... + 8 fused multiply-adds
		SM();
		X17_UNROLL for (int i = 0; i < 8; ++i) A_OP(i);
#elif X17_PROBE_OP == 102        // ... + 8 byte shuffles
		SM();
		X17_UNROLL for (int i = 0; i < 8; ++i) B_OP(i);
#elif X17_PROBE_OP == 103        // ... + 8 exponentials
		SM();
		X17_UNROLL for (int i = 0; i < 8; ++i) C_OP(i);
#elif X17_PROBE_OP == 104        // one int8 matrix instruction alone (a dependent chain)
		SM();
#elif X17_PROBE_OP == 105 || X17_PROBE_OP == 106
		// one 32-key step of the attention speed build (head_dim 128): 105 = vector + matrix instructions only,
		// 106 = with the scalar bookkeeping, the waits and the LDS reads
		constexpr bool FULL = X17_PROBE_OP == 106;
		if (FULL) { W_OP(); W_OP(); X17_UNROLL for (int i = 0; i < 8; ++i) S_OP(); }
		// scores: 4 dependent matrix instructions, their K fragments, the widening of V in between
		X17_UNROLL for (int m = 0; m < 4; ++m) {
			if (FULL) { L_OP(m); W_OP(); }
			SM();
			A_OP(m); B_OP(4 + m); B_OP(8 + m); B_OP(12 + m); B_OP(m + 1); A_OP(m + 2);
		}
		if (FULL) { L_OP(0); L_OP(1); L_OP(0); }
		X17_UNROLL for (int t = 0; t < 2; ++t) {
			X17_UNROLL for (int i = 0; i < 4; ++i) B_OP(i);          // row maximum
			A_OP(5);                                                  // compare
			if (FULL) S_OP();                                         // branch
			X17_UNROLL for (int i = 0; i < 8; ++i) { A_OP(i); C_OP(i); }       // exponent's argument, exponential
			X17_UNROLL for (int i = 0; i < 8; ++i) A_OP(8 + i);       // partial sums
			X17_UNROLL for (int i = 0; i < 8; ++i) A_OP(i);           // rounding
			X17_UNROLL for (int i = 0; i < 4; ++i) { B_OP(i); B_OP(4 + i); }   // byte shuffle, packed fma
			X17_UNROLL for (int j = 0; j < 4; ++j) {
				if (FULL) { L_OP(0); L_OP(1); W_OP(); }
				PM(j);
			}
		}
		if (FULL) { X17_UNROLL for (int i = 0; i < 4; ++i) S_OP(); }
#else
#error "unknown composite X17_PROBE_OP"
#endif
	}
	f32 sum = f32(sc);
	X17_UNROLL for (int i = 0; i < 16; ++i) sum += r[i];
	X17_UNROLL for (int e = 0; e < 16; ++e) {
		sum += f32(sacc[e]);
		X17_UNROLL for (int j = 0; j < 4; ++j) sum += oacc[j][e];
	}
	sum += f32(lv[0][0] + lv[1][1]);
	out[(size_t)blockIdx.x * 64 + threadIdx.x] = sum;
}
#endif
