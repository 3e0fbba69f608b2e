// Launch geometry of the vector-issue probe as JSON.
#include <cstdio>
int main() {
	std::printf("{\n\t\"THREADS_PER_BLOCK\": 64,\n\t\"SMEM_BYTES\": 0,\n\t\"BLOCKS_PER_WAVE_PER_SIMD\": 1024,\n\t\"INSTRUCTIONS_PER_ITERATION\": 16\n}\n");
}
