// Kernel registry base class of a backend.
#pragma once

#include <unordered_map>
#include <unordered_set>

#include "tf_ir.h"
#include "tf_memory.h"

namespace tfhost {

// Mirrors TensorFrost/Backend/KernelManager.h:16-30.
class KernelManager {
	std::unordered_set<Program*> programs;
	std::unordered_map<size_t, Kernel*> kernel_map;
	size_t global_kernel_id = 0;

 public:
	KernelManager() = default;
	virtual ~KernelManager() = default;
	virtual void DispatchKernel(TFDispatchInfo info) = 0;
	void AddKernelID(Program* program, Kernel* kernel);
	void RemoveProgram(Program* program);
	Kernel* GetKernel(size_t kernel_id) {
		auto it = kernel_map.find(kernel_id);
		return it == kernel_map.end() ? nullptr : it->second;
	}
};

extern KernelManager* global_kernel_manager;

}  // namespace tfhost
