#include "registry.h"

#include <chrono>

namespace tfhost {

std::map<std::string, ProgramFactory>& ProgramRegistry() {
	static std::map<std::string, ProgramFactory> registry;
	return registry;
}

Program* CreateProgram(const std::string& name, const std::vector<int64_t>& params) {
	auto it = ProgramRegistry().find(name);
	if (it == ProgramRegistry().end()) throw std::runtime_error("Unknown program: " + name);
	if (current_backend == BackendType::NotInitialized) throw std::runtime_error("Backend not initialized");
	Program* program = new Program();
	program->program_name = name;
	using Clock = std::chrono::steady_clock;
	auto seconds = [](Clock::time_point a, Clock::time_point b) { return std::chrono::duration<float>(b - a).count(); };
	try {
		const Clock::time_point t0 = Clock::now();
		it->second(program, params);
		if (!program->host_code) throw std::runtime_error("Program " + name + " has no host code (HostBuilder::Finish was not called)");
		const Clock::time_point t1 = Clock::now();
		GenerateCode(program);
		const Clock::time_point t2 = Clock::now();
		CompileKernels(program);  // sets shader_compile_time (milliseconds, as Backend.cpp:75-94)
		program->trace_time = seconds(t0, t1);
		program->codegen_time = seconds(t1, t2);
	} catch (...) {
		if (global_kernel_manager) global_kernel_manager->RemoveProgram(program);
		delete program;
		throw;
	}
	return program;
}

void DestroyProgram(Program* program) {
	if (!program) return;
	if (global_kernel_manager) {
		if (auto* hip = dynamic_cast<HipKernelManager*>(global_kernel_manager))
			for (auto& k : program->kernels_) hip->FreeKernel(k->kernel_id_);
		global_kernel_manager->RemoveProgram(program);
	}
	delete program;
}

}  // namespace tfhost
