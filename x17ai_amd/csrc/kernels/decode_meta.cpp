// Prints the launch geometry of the decode kernel as JSON.
#include "common.h"
#include "decode_tile.h"
#include <cstdio>

int main() {
	namespace dt = x17::decode_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", dt::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", dt::SMEM_BYTES);
	std::printf("\t\"HEADS_PER_BLOCK\": %u\n", dt::HEADS_PER_BLOCK);
	std::printf("}\n");
}
