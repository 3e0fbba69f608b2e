// Prints the launch geometry of the attention kernel configured by common.h as JSON
// (reference: templates/attn/meta.cu).
#include "common.h"
#include "attn_tile.h"
#include <cstdio>

int main() {
	namespace at = x17::attn_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", at::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", at::SMEM_BYTES);
	std::printf("\t\"Q_PER_BLOCK\": %u\n", at::Q_PER_BLOCK);
	std::printf("}\n");
}
