// Launch geometry of the matrix-core probe as JSON: operations per MFMA instruction depend on the kind.
#include "common.h"
#include <cstdio>
int main() {
	// multiply-adds x 2 of one MFMA: 32 x 32 outputs, K = 32 (int8), 64 (e4m3) or 16 (f16)
	unsigned const k = X17_PROBE_KIND == 0 ? 32 : (X17_PROBE_KIND == 1 ? 64 : 16);
	std::printf("{\n\t\"THREADS_PER_BLOCK\": 512,\n\t\"SMEM_BYTES\": 0,\n\t\"BLOCKS\": 256,\n\t\"MFMAS_PER_ITERATION\": 8,\n\t\"OPS_PER_MFMA\": %u\n}\n",
	            2u * 32u * 32u * k);
}
