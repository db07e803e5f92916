// Host-only sanitizer run: builds every registered program on the code-generation backend (emit + hiprtc check).
#include <cstdio>
#include <cstdint>
#include <initializer_list>
#include <string>
#include "tfhost.h"
int main() {
	const char* names[] = {"mlp","nbody","radix_sort","reductions","prefix_sum","radix_sort_ir","reductions_ir","softmax_ir","ops","radix_scatter_pass","dense_layer","dense_tanh","batched_matmul","indexing","broadcast_loops","atomics","group_reverse","tile_indices","lowered_idioms","tiled_matmul_ir","wave_eq"};
	if (tfhost_initialize(1 /* codegen */, "")) { printf("init failed: %s\n", tfhost_last_error()); return 1; }
	int bad = 0;
	for (const char* n : names) {
		const bool takes_rank = std::string(n) == "indexing";  // this one's parameter is the tensor rank: 3 or 4
		for (int64_t arg : {(int64_t)(takes_rank ? 3 : 0), (int64_t)(takes_rank ? 4 : 1), (int64_t)2}) {
			tfhost_program_t p = nullptr;
			int rc = tfhost_program_create(n, &arg, 1, &p);
			if (rc) { printf("%s(%ld): %s\n", n, (long)arg, tfhost_last_error()); bad += arg != 2; continue; }
			size_t count = 0;
			tfhost_program_kernel_count(p, &count);
			for (size_t i = 0; i < count; i++) {
				const char *src, *map; int threads; size_t id;
				tfhost_program_kernel_info(p, i, &src, &map, &threads, &id);
			}
			printf("%s(%ld): %zu kernels\n", n, (long)arg, count);
			tfhost_program_destroy(p);
		}
	}
	tfhost_shutdown();
	return bad ? 1 : 0;
}
