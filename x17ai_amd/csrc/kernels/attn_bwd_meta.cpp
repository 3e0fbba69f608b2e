// Prints the launch geometry of the attention backward (dQ) kernel configured by common.h as JSON, with the keys the
// attention launcher reads (reference: templates/attn/meta.cu).
#include "common.h"
#include "attn_bwd_tile.h"
#include <cstdio>

int main() {
	namespace bt = x17::attn_bwd_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", bt::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", bt::SMEM_BYTES);
	std::printf("\t\"Q_PER_BLOCK\": %u\n", bt::Q_PER_BLOCK);
	std::printf("}\n");
}
