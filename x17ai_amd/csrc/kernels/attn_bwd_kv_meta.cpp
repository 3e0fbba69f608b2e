// Prints the launch geometry of the attention backward (dK, dV) kernel configured by common.h as JSON, with the keys
// the attention launcher reads (reference: templates/attn/meta.cu); Q_PER_BLOCK is the key block here.
#include "common.h"
#include "attn_bwd_kv_tile.h"
#include <cstdio>

int main() {
	namespace kt = x17::attn_bwd_kv_tile;
	std::printf("{\n");
	std::printf("\t\"THREADS_PER_BLOCK\": %u,\n", kt::THREADS_PER_BLOCK);
	std::printf("\t\"SMEM_BYTES\": %u,\n", kt::SMEM_BYTES);
	std::printf("\t\"Q_PER_BLOCK\": %u\n", kt::KEYS_PER_BLOCK);
	std::printf("}\n");
}
