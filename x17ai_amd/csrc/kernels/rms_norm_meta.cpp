// Prints the launch geometry of the rms_norm kernel as JSON.
#include "common.h"
#include "rms_norm_tile.h"
#include <cstdio>

int main() {
	namespace rt = x17::rms_norm_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", rt::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", rt::SMEM_BYTES);
	std::printf("\t\"ROWS_PER_BLOCK\": %u\n", rt::ROWS_PER_BLOCK);
	std::printf("}\n");
}
