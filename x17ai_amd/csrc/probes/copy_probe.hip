// copy_probe.hip -- a plain device-to-device copy of known size.  Measurement aid only: hardware
// counters for HBM traffic are calibrated against what they read for this kernel.
#include "common.h"
#include "x17_device.h"

extern "C" __global__ __launch_bounds__(256)
void kernel(v4u const *src, u32 n_vec, v4u *dst) {
	u32 stride = gridDim.x * blockDim.x;
	for (u32 i = blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) {
		dst[i] = src[i];
	}
}
