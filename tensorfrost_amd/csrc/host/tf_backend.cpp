#include "tf_backend.h"

#include <chrono>
#include <iostream>
#include <unordered_set>

#include "hip_generator.h"
#include "sort_composition.h"

namespace tfhost {

BackendType current_backend = BackendType::NotInitialized;
CodeGenLang current_kernel_lang = CodeGenLang::CPP;
std::string kernelCompileOptions;
KernelManager* global_kernel_manager = nullptr;

static void Check(int status, const std::string& what) {
	if (status != TFHIP_OK) throw std::runtime_error(what + ": " + tfhip_last_error());
}

// ---- kernel registry ----------------------------------------------------------------------------------

void KernelManager::AddKernelID(Program* program, Kernel* kernel) {
	programs.insert(program);
	kernel->kernel_id_ = global_kernel_id++;
	kernel_map[kernel->kernel_id_] = kernel;
}

void KernelManager::RemoveProgram(Program* program) {
	programs.erase(program);
	for (auto& k : program->kernels_) kernel_map.erase(k->kernel_id_);
}

// ---- code generation and compilation ---------------------------------------------------------------------

void GenerateKernel(Program* program, Kernel* kernel) {
	switch (current_kernel_lang) {
		case CodeGenLang::HIP:
			GenerateHIPKernel(program, kernel);
			return;
		default:
			throw std::runtime_error("Code generation for this language is not implemented yet");
	}
}

void GenerateCode(Program* program) {
	if (global_kernel_manager == nullptr) throw std::runtime_error("Backend not initialized");
	auto give_id = [program](Kernel* kernel) {
		global_kernel_manager->AddKernelID(program, kernel);
		kernel->kernel_name_ = "kernel_" + std::to_string(kernel->kernel_id_);
	};
	const size_t count = program->kernels_.size();  // dense variants and tail kernels are appended while this runs
	for (size_t i = 0; i < count; i++) {
		Kernel* kernel = program->kernels_[i].get();
		give_id(kernel);
		if (!kernel->primitive.empty()) continue;
		if (current_kernel_lang == CodeGenLang::HIP)
			GenerateHIPKernelFamily(program, kernel, give_id);
		else
			GenerateKernel(program, kernel);
	}
	if (auto* hip = dynamic_cast<HipKernelManager*>(global_kernel_manager))
		for (auto& kernel : program->kernels_) hip->SetKernelInfo(MakeKernelInfo(kernel.get()));
}

void CompileKernels(Program* program) {
	auto start = std::chrono::high_resolution_clock::now();
	for (auto& kernel : program->kernels_) {
		switch (current_backend) {
			case BackendType::HIP:
			case BackendType::CodeGen:  // no device: hiprtc still checks that the source builds for gfx950
				((HipKernelManager*)global_kernel_manager)->CompileKernel(kernel.get());
				break;
			default:
				throw std::runtime_error("Backend not implemented");
		}
	}
	auto end = std::chrono::high_resolution_clock::now();
	program->shader_compile_time = std::chrono::duration<float, std::milli>(end - start).count();
}

// ---- backend lifetime ---------------------------------------------------------------------------------

void StopBackend() {
	if (current_backend == BackendType::NotInitialized) return;
	delete global_kernel_manager;
	global_kernel_manager = nullptr;
	delete global_memory_manager;
	global_memory_manager = nullptr;
	if (current_backend == BackendType::HIP) tfhip_shutdown();
	current_backend = BackendType::NotInitialized;
}

void InitializeBackend(BackendType type, const std::string& compiler_options, CodeGenLang kernel_lang) {
	if (current_backend != BackendType::NotInitialized) {
		std::cout << "Warning: Backend already initialized, stopping current backend\n" << std::endl;
		StopBackend();
	}
	kernelCompileOptions = compiler_options;  // non-CPU backends default to no extra options (Backend.cpp:27-37)
	switch (type) {
		case BackendType::HIP:
			Check(tfhip_init(0), "Failed to initialize the HIP backend");
			current_kernel_lang = CodeGenLang::HIP;
			global_memory_manager = new HipMemoryManager();
			global_kernel_manager = new HipKernelManager();
			((HipKernelManager*)global_kernel_manager)->compile_options = kernelCompileOptions;
			break;
		case BackendType::CodeGen:
			// Emits and hiprtc-checks source without a device; programs cannot be executed.
			current_kernel_lang = CodeGenLang::HIP;
			global_memory_manager = nullptr;
			global_kernel_manager = new HipKernelManager();
			((HipKernelManager*)global_kernel_manager)->compile_options = kernelCompileOptions;
			break;
		default:
			throw std::runtime_error("Backend not implemented");
	}
	current_backend = type;
	if (kernel_lang != CodeGenLang::None) current_kernel_lang = kernel_lang;
}

void Finish() {
	if (current_backend == BackendType::HIP) Check(tfhip_sync(), "Failed to synchronize");
}

// ---- runtime callbacks (Backend.cpp:96-133) ---------------------------------------------------------------

static TFTensor Allocator(const char* name, const size_t* a, size_t dim, TFDataFormat format, void*) {
	try {
		std::vector<size_t> shape(a, a + dim);
		return *global_memory_manager->AllocateTensor(shape, format, name);
	} catch (const std::exception& e) {
		size_t size = 1;
		for (size_t i = 0; i < dim; i++) size *= a[i];
		throw std::runtime_error("Error allocating tensor " + std::string(name) + ": " + e.what() + ", requested size: " + std::to_string(size));
	}
}

static HipKernelManager* HipManager() { return current_backend == BackendType::HIP ? (HipKernelManager*)global_kernel_manager : nullptr; }

static void Deallocator(TFTensor a, void*) {
	HipKernelManager* km = HipManager();
	if (km && km->HasDeferredWork())
		km->DeferFree(a);  // a dispatch that is held back may still name this buffer
	else
		global_memory_manager->DeallocateTensor(a);
}
static uint32_t Readback(TFTensor a, size_t index, void*) {
	if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	return global_memory_manager->ReadbackValue(&a, index);
}
static void Writeback(TFTensor a, size_t index, uint32_t value, void*) {
	if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	global_memory_manager->WritebackValue(&a, index, value);
}
static void Dispatch(TFDispatchInfo info, void*) { global_kernel_manager->DispatchKernel(info); }
static void Region(const char* name, bool begin, void*) {
	if (current_backend == BackendType::HIP) {
		((HipKernelManager*)global_kernel_manager)->OnRegion(name, begin);
		if (begin)
			tfhip_range_push(name);
		else
			tfhip_range_pop();
	}
}

TFRuntime GetRuntimeCallbacks() { return TFRuntime{Allocator, Deallocator, Readback, Writeback, Dispatch, Region, nullptr}; }

std::vector<TFTensor*> ExecuteProgram(Program* program, std::vector<TFTensor*> inputs) {
	if (current_backend == BackendType::CodeGen) throw std::runtime_error("Cannot execute program with code generation backend");
	if (current_backend == BackendType::NotInitialized) throw std::runtime_error("Backend not initialized");
	if ((size_t)program->input_count != inputs.size())
		throw std::runtime_error("Invalid number of inputs for TensorProgram. Expected " + std::to_string(program->input_count) + ", got " + std::to_string(inputs.size()));

	std::vector<TFTensor> input_tensors;
	for (TFTensor* t : inputs) input_tensors.push_back(*t);
	TFTensor* out = new TFTensor[program->output_count];  // kept alive for the wrappers of the outputs
	try {
		if (HipKernelManager* km = HipManager()) km->RefreshOptions();
		program->execute_callback(input_tensors.data(), out, GetRuntimeCallbacks());
		if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	} catch (const std::exception& e) {
		delete[] out;
		try {
			if (HipKernelManager* km = HipManager()) km->FlushDeferred();
		} catch (...) {
		}
		throw std::runtime_error("Error executing program " + program->program_name + ": " + e.what());
	}
	std::vector<TFTensor*> outputs(program->output_count);
	for (int i = 0; i < program->output_count; i++) outputs[i] = &out[i];
	return outputs;
}

// ---- recorded programs ----------------------------------------------------------------------------------------

static void* DevicePointer(const TFTensor* t) { return ((TFHipBuffer*)t->buffer)->GetNative(); }

RecordedProgram* RecordProgram(Program* program, std::vector<TFTensor*> inputs, size_t repeat, const std::vector<int>& feedback) {
	if (current_backend != BackendType::HIP) throw std::runtime_error("Programs can only be recorded on the HIP backend");
	if (repeat == 0) throw std::runtime_error("Cannot record zero executions");
	if (repeat > 1 && feedback.empty()) throw std::runtime_error("Recording more than one execution needs feedback (outputs feeding the next inputs)");
	if (!feedback.empty() && feedback.size() != inputs.size())
		throw std::runtime_error("Feedback has " + std::to_string(feedback.size()) + " entries for " + std::to_string(inputs.size()) + " inputs");
	for (int f : feedback)
		if (f < -1 || f >= program->output_count) throw std::runtime_error("Feedback names output " + std::to_string(f) + " of " + std::to_string(program->output_count));

	// The ordinary run: loads modules, sizes the scratch buffer and fills the pool with buffers of the right sizes.
	std::vector<TFTensor*> first = ExecuteProgram(program, inputs);
	auto is_input = [&](const TFTensor* t) {
		for (TFTensor* in : inputs)
			if (in->buffer == t->buffer) return true;
		return false;
	};
	auto release_all = [&](const std::vector<TFTensor*>& tensors, const std::vector<TFTensor*>& keep) {
		std::unordered_set<TFBuffer*> done;
		for (TFTensor* t : keep) done.insert(t->buffer);
		for (TFTensor* t : tensors) {
			if (is_input(t) || !done.insert(t->buffer).second) continue;
			global_memory_manager->DeallocateTensor(*t);
		}
	};
	for (size_t i = 0; i < feedback.size(); i++) {
		if (feedback[i] < 0) continue;
		const TFTensor* from = first[feedback[i]];
		if (GetShape(from) != GetShape(inputs[i]) || from->format.type != inputs[i]->format.type) {
			release_all(first, {});
			throw std::runtime_error("Feedback: output " + std::to_string(feedback[i]) + " and input " + std::to_string(i) + " differ in shape or type");
		}
	}
	release_all(first, {});

	RecordedProgram* recorded = new RecordedProgram();
	global_memory_manager->BeginHold();
	bool recording = false;
	try {
		Check(tfhip_graph_begin(), "Failed to start recording");
		recording = true;
		std::vector<TFTensor*> current = inputs, out;
		for (size_t r = 0; r < repeat; r++) {
			std::vector<TFTensor*> previous = out;
			out = ExecuteProgram(program, current);
			// The previous execution's outputs have been consumed; the stream's order makes their reuse safe.
			release_all(previous, out);
			for (size_t i = 0; i < feedback.size(); i++)
				if (feedback[i] >= 0) current[i] = out[feedback[i]];
		}
		for (size_t i = 0; i < feedback.size(); i++) {
			if (feedback[i] < 0 || out[feedback[i]]->buffer == inputs[i]->buffer) continue;
			Check(tfhip_d2d(DevicePointer(inputs[i]), DevicePointer(out[feedback[i]]), GetSize(inputs[i])), "Failed to record the feedback copy");
		}
		recording = false;
		Check(tfhip_graph_end(&recorded->graph), "Failed to finish recording");
		recorded->outputs = out;
	} catch (...) {
		if (recording) tfhip_graph_end(nullptr);
		global_memory_manager->EndHold(false);
		delete recorded;
		throw;
	}
	recorded->buffers = global_memory_manager->EndHold(true);
	tfhip_graph_node_count(recorded->graph, &recorded->nodes);
	return recorded;
}

void ReplayProgram(RecordedProgram* recorded) { Check(tfhip_graph_launch(recorded->graph), "Failed to replay"); }

void DestroyRecordedProgram(RecordedProgram* recorded) {
	if (!recorded) return;
	tfhip_graph_destroy(recorded->graph);  // waits for the stream
	if (global_memory_manager) global_memory_manager->Unreserve(recorded->buffers);
	delete recorded;
}

}  // namespace tfhost
