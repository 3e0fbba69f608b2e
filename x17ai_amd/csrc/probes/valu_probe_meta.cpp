// Launch geometry of the issue probe as JSON.  An iteration of a single-instruction loop holds 16 copies of the
// instruction; an iteration of a composite loop is one group (four matrix instructions for op 100).
#include "common.h"
#include <cstdio>
int main() {
	int const per_iteration = X17_PROBE_OP < 100 ? 16 : (X17_PROBE_OP == 100 ? 4 : 1);
	std::printf("{\n\t\"THREADS_PER_BLOCK\": 64,\n\t\"SMEM_BYTES\": 0,\n\t\"BLOCKS_PER_WAVE_PER_SIMD\": 1024,\n\t\"INSTRUCTIONS_PER_ITERATION\": %d\n}\n", per_iteration);
}
