// Prints the launch geometry of the GEMM kernel configured by common.h as JSON; the host
// layer reads it back instead of mirroring the constants (reference: templates/basic_gemm/meta.cu).
#include "common.h"
#include "gemm_tile.h"
#include <cstdio>

int main() {
	namespace gt = x17::gemm_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", gt::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", gt::SMEM_BYTES);
	std::printf("\t\"M_PER_BLOCK\": %u,\n", gt::M_PER_BLOCK);
	std::printf("\t\"N_PER_BLOCK\": %u,\n", gt::N_PER_BLOCK);
	std::printf("\t\"MAX_BLOCKS\": %u\n", gt::MAX_BLOCKS);
	std::printf("}\n");
}
