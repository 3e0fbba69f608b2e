// valu_probe.hip -- loops of ONE vector instruction on sixteen independent registers.  Measurement aid only: how
// fast a SIMD of the machine at hand issues a given instruction, as a function of the wavefronts that share it.
// The attention kernel is bounded by exactly this (its softmax is a fixed mix of such instructions per score),
// and the figures are not what the 4-cycles-per-instruction rule of thumb gives.
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
#else
#error "unknown X17_PROBE_OP"
#endif

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
