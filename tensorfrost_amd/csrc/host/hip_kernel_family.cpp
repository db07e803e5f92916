// A kernel and the further kernels its dispatch may need, emitted together; and the table entry the kernel manager
// dispatches each of them by. Shared by this repository's own GenerateCode (tf_backend.cpp) and by the generator arm a
// TensorFrost checkout reaches through GenerateKernel (Backend/CodeGen/Generators.cpp:9-23).
#include "hip_generator.h"
#include "sort_composition.h"

namespace tfhost {

std::vector<Kernel*> GenerateHIPKernelFamily(Program* program, Kernel* kernel, const std::function<void(Kernel*)>& give_id) {
	std::vector<Kernel*> family{kernel};
	AnalyzeSortFeatures(kernel);
	GenerateHIPKernel(program, kernel);
	if (kernel->wants_dense_variant) {
		Kernel* dense = CloneKernel(program, kernel);
		dense->serial_loops = true;
		give_id(dense);
		GenerateHIPKernel(program, dense);
		kernel->dense_variant = dense;
		family.push_back(dense);
	}
	MatchKernelIdiom(kernel);
	if (kernel->match.kind == IdiomMatch::Matmul && kernel->match.op == "tail") {
		// A matmul loop with an element-wise tail of its own: the kernel without the loop becomes a second
		// kernel that reads the product of the matmul primitive.
		Kernel* tail = MakeMatmulTailKernel(program, kernel, kernel->match.accumulator, kernel->match.loop);
		give_id(tail);
		GenerateHIPKernel(program, tail);
		kernel->tail_kernel = tail;
		family.push_back(tail);
	}
	return family;
}

// What the emitter decided for a kernel, as the table the kernel manager dispatches by.
HipKernelInfo MakeKernelInfo(const Kernel* kernel) {
	HipKernelInfo info;
	info.kernel_id = kernel->kernel_id_;
	info.tensor_count = kernel->read_write_memory.size() + kernel->read_only_memory.size();
	info.variable_count = kernel->variables.size();
	info.group_size = kernel->group_size;
	info.idiom = kernel->idiom;
	info.hip_threads = kernel->hip_threads;
	info.groups_per_hip_block = kernel->groups_per_hip_block;
	info.hip_blocks_per_tile = kernel->hip_blocks_per_tile;
	info.lanes_per_thread = kernel->lanes_per_thread;
	info.threads_per_lane_group = kernel->threads_per_lane_group;
	info.serial_load_loops = kernel->serial_load_loops;
	info.slabs = kernel->slabs;
	info.slab_trips = kernel->slab_trips;
	info.slab_words_per_thread = kernel->slab_words_per_thread;
	info.scalar_entry = kernel->scalar_entry;
	info.scalar_hip_threads = kernel->scalar_hip_threads;
	info.scalar_groups_per_hip_block = kernel->scalar_groups_per_hip_block;
	info.batch_entry = kernel->batch_entry;
	info.batch_capacity = kernel->batch_capacity;
	info.batch_call_bytes = kernel->batch_call_bytes;
	info.read_write_count = kernel->read_write_memory.size();
	info.primitive = kernel->primitive;
	info.primitive_tensors = kernel->primitive_tensors;
	info.primitive_variables = kernel->primitive_variables;
	info.match = kernel->match;  // the part of the match that does not refer to the tree
	info.sort = kernel->sort;
	info.has_tail_kernel = kernel->tail_kernel != nullptr;
	info.tail_kernel_id = kernel->tail_kernel ? kernel->tail_kernel->kernel_id_ : 0;
	info.has_dense_variant = kernel->dense_variant != nullptr;
	info.dense_variant_id = kernel->dense_variant ? kernel->dense_variant->kernel_id_ : 0;
	return info;
}

}  // namespace tfhost
