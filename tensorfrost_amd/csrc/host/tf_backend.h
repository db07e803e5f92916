// Backend selection, kernel registry / dispatch, the six runtime callbacks and program execution.
//
// Restates the backend-independent parts of TensorFrost/Backend/Backend.{h,cpp} and
// TensorFrost/Backend/KernelManager.{h,cpp} and adds the HIP arms a patched TensorFrost tree would gain:
//   BackendType::HIP / CodeGenLang::HIP enum values            (Backend.h:22-35)
//   InitializeBackend: tfhip_init + HipMemoryManager + HipKernelManager   (Backend.cpp:49-68)
//   CompileKernels: HipKernelManager::CompileKernel per kernel  (Backend.cpp:75-94)
//   Region: roctx ranges                                        (Backend.cpp:125-133)
//   HipKernelManager::DispatchKernel                            (cf. Backends/OpenGL/KernelManager.h:105-159)
#pragma once

#include <exception>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "shim/HIP.h"
#include "tf_ir.h"
#include "tf_kernel_manager.h"
#include "tf_memory.h"
#include "tfhip.h"

namespace tfhost {

enum class BackendType { CPU, Vulkan, OpenGL, CodeGen, HIP, NotInitialized };
enum class CodeGenLang { CPP, HLSL, GLSL, HIP, None };

extern BackendType current_backend;
extern CodeGenLang current_kernel_lang;
extern std::string kernelCompileOptions;

// GenerateKernel's language switch (Generators.cpp:9-23) with the HIP arm.
void GenerateKernel(Program* program, Kernel* kernel);
// Registers every kernel of the program, generates its source and compiles it (the kernel half of
// GenerateCode, CPP.cpp:564-638, followed by CompileKernels, Backend.cpp:75-94).
void GenerateCode(Program* program);
void CompileKernels(Program* program);

void InitializeBackend(BackendType type, const std::string& compiler_options = "", CodeGenLang kernel_lang = CodeGenLang::None);
void StopBackend();
void Finish();

// The callbacks handed to generated host programs (Backend.cpp:96-133).
TFRuntime GetRuntimeCallbacks();

// Backend.cpp:137-185: arity check, copies tensor headers, runs the program's `main`.
std::vector<TFTensor*> ExecuteProgram(Program* program, std::vector<TFTensor*> inputs);

// One or more executions of a program on fixed buffers, recorded as a HIP graph. The reference has no
// counterpart: every call of a program walks the host path again (Definitions/TensorProgram.cpp:67-150 marshals
// the arguments, the emitted host code re-allocates and re-dispatches, CPP.cpp:482-518).
struct RecordedProgram {
	tfhip_graph_t graph = nullptr;
	std::vector<TFBuffer*> buffers;  // every buffer the recorded executions allocated, kept out of the pool
	std::vector<TFTensor*> outputs;  // of the last recorded execution; they live in `buffers`
	size_t nodes = 0;
};
// Runs the program once as usual (so that modules are loaded and scratch and pool have their sizes), then records
// `repeat` executions. `feedback` is empty or has one entry per input: the index of the output that becomes this
// input in the next execution, or -1 for an input that stays what it is. With feedback the graph ends by copying
// the last outputs into the buffers of the inputs they feed, so that every replay continues from the previous
// one. A program that reads a tensor back while it runs cannot be recorded.
RecordedProgram* RecordProgram(Program* program, std::vector<TFTensor*> inputs, size_t repeat, const std::vector<int>& feedback);
void ReplayProgram(RecordedProgram* recorded);
void DestroyRecordedProgram(RecordedProgram* recorded);

}  // namespace tfhost
