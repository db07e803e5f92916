// Registry of programs that stand in for what `tf.compile(fn)` would hand the backend: the tree of the traced
// function after every pass -- its kernels in post-lowering form and the host nodes around them
// (TensorFrost/Tensor/TensorProgram.cpp:7-57 is the driver this replaces for the test programs).
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "../tf_backend.h"
#include "../host_program.h"
#include "../tf_ir.h"

namespace tfhost {

// Builds the IR of a program (kernels with KernelBuilder, the host part with HostBuilder); params are program-specific integers.
using ProgramFactory = std::function<void(Program* program, const std::vector<int64_t>& params)>;

std::map<std::string, ProgramFactory>& ProgramRegistry();

struct ProgramRegistrar {
	ProgramRegistrar(const char* name, ProgramFactory f) { ProgramRegistry()[name] = std::move(f); }
};

// trace -> (IR already lowered) -> GenerateCode -> CompileKernels, as TensorProgram::CreateProgram.
Program* CreateProgram(const std::string& name, const std::vector<int64_t>& params);
void DestroyProgram(Program* program);

}  // namespace tfhost
