// Launch geometry of the copy probe as JSON.
#include <cstdio>
int main() {
	std::printf("{\n\t\"THREADS_PER_BLOCK\": 256,\n\t\"SMEM_BYTES\": 0,\n\t\"BLOCKS\": 4096\n}\n");
}
