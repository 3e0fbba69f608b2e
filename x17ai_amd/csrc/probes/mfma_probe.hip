// mfma_probe.hip -- a loop of nothing but matrix-core instructions on register operands.  Measurement aid
// only: what the matrix cores of the machine at hand sustain on given operand DATA (the clock a gfx950 holds
// under dense MFMA load depends on how much the operands toggle), with no memory traffic, no LDS and no
// barrier in the loop.  The GEMM kernels are read against this figure as well as against the nominal peak.
//
// common.h provides X17_PROBE_KIND: 0 = v_mfma_i32_32x32x32_i8, 1 = v_mfma_f32_32x32x64_f8f6f4 (e4m3),
// 2 = v_mfma_f32_32x32x16_f16.  Geometry as in gemm_b8.hip: 8 wavefronts per workgroup, two per SIMD, each with
// 4 x 2 accumulator blocks; per iteration a wavefront issues 8 MFMAs on 4 + 2 operand fragments.
#include "common.h"
#include "x17_device.h"

using namespace x17;

extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void kernel(v4i const *operands, u32 iterations, i32 *out) {
	u32 const tid = threadIdx.x;
	// twelve 16-byte operand chunks per lane (enough for the widest fragments), different for every lane
	v4i f[12];
	X17_UNROLL for (int i = 0; i < 12; ++i) f[i] = operands[(size_t)i * 512 + tid];
	v16i acc[4][2];
	X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
		X17_UNROLL for (int bm = 0; bm < 2; ++bm) {
			X17_UNROLL for (int r = 0; r < 16; ++r) acc[bn][bm][r] = 0;
		}
	}
	for (u32 it = 0; it < iterations; ++it) {
		X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
			X17_UNROLL for (int bm = 0; bm < 2; ++bm) {
#if X17_PROBE_KIND == 0
				acc[bn][bm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[bn], f[4 + bm], acc[bn][bm], 0, 0, 0);
#elif X17_PROBE_KIND == 1
				v8i const w = {f[bn][0], f[bn][1], f[bn][2], f[bn][3], f[6 + bn][0], f[6 + bn][1], f[6 + bn][2], f[6 + bn][3]};
				v8i const x = {f[4 + bm][0], f[4 + bm][1], f[4 + bm][2], f[4 + bm][3], f[10 + bm][0], f[10 + bm][1], f[10 + bm][2], f[10 + bm][3]};
				v16f const r = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0, 0, 0, 0);
				acc[bn][bm] = __builtin_bit_cast(v16i, r);
#else
				v16f const r = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, f[bn]), __builtin_bit_cast(v8h, f[4 + bm]),
				                                                      __builtin_bit_cast(v16f, acc[bn][bm]), 0, 0, 0);
				acc[bn][bm] = __builtin_bit_cast(v16i, r);
#endif
			}
		}
	}
	i32 sum = 0;
	X17_UNROLL for (int bn = 0; bn < 4; ++bn) {
		X17_UNROLL for (int bm = 0; bm < 2; ++bm) {
			X17_UNROLL for (int r = 0; r < 16; ++r) sum ^= acc[bn][bm][r];
		}
	}
	out[(size_t)blockIdx.x * 512 + tid] = sum;
}
