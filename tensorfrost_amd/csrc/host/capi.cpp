#include <dlfcn.h>

#include <cstring>
#include <string>

#include "programs/registry.h"
#include "tf_backend.h"
#include "tfhost.h"

using namespace tfhost;

struct tfhost_program {
	Program* program;
};

struct tfhost_tensor {
	TFTensor* tensor;  // header owned by the memory manager's allocation (never freed, as in the reference)
	bool owns_buffer;  // false for aliases of an input returned as an output
};

struct tfhost_graph {
	RecordedProgram* recorded;
};

static thread_local std::string g_error;

template <class F>
static int Guard(F&& f) {
	try {
		f();
		return 0;
	} catch (const std::exception& e) {
		g_error = e.what();
		return -1;
	} catch (...) {
		g_error = "unknown error";
		return -1;
	}
}

static void RequireMemory() {
	if (global_memory_manager == nullptr) throw std::runtime_error("Backend not initialized (or it has no device memory)");
}

extern "C" {

const char* tfhost_last_error(void) { return g_error.c_str(); }

int tfhost_initialize(int backend, const char* options) {
	return Guard([&] {
		BackendType type = backend == TFHOST_BACKEND_HIP ? BackendType::HIP : backend == TFHOST_BACKEND_CODEGEN ? BackendType::CodeGen : BackendType::NotInitialized;
		if (type == BackendType::NotInitialized) throw std::runtime_error("Backend not implemented");
		InitializeBackend(type, options ? options : "");
	});
}

int tfhost_shutdown(void) {
	return Guard([] { StopBackend(); });
}

int tfhost_sync(void) {
	return Guard([] { Finish(); });
}

int tfhost_program_create(const char* name, const int64_t* params, size_t n_params, tfhost_program_t* out) {
	return Guard([&] {
		if (!name || !out) throw std::runtime_error("null argument");
		std::vector<int64_t> p(params, params + (params ? n_params : 0));
		*out = new tfhost_program{CreateProgram(name, p)};
	});
}

int tfhost_program_destroy(tfhost_program_t program) {
	return Guard([&] {
		if (!program) return;
		DestroyProgram(program->program);
		delete program;
	});
}

int tfhost_program_kernel_count(tfhost_program_t program, size_t* count) {
	return Guard([&] {
		if (!program || !count) throw std::runtime_error("null argument");
		*count = program->program->kernels_.size();
	});
}

int tfhost_program_kernel_info(tfhost_program_t program, size_t index, const char** source, const char** mapping, int* hip_threads, size_t* kernel_id) {
	return Guard([&] {
		if (!program) throw std::runtime_error("null argument");
		auto& kernels = program->program->kernels_;
		if (index >= kernels.size()) throw std::runtime_error("kernel index out of range");
		Kernel* k = kernels[index].get();
		if (source) *source = k->full_generated_code_.c_str();
		if (mapping) {
			static thread_local std::string text;
			static const char* kinds[] = {"", "+reduce", "+scan", "+matmul", "+expsum", "+normalise", "+expdiff", "+dividerows"};
			text = k->idiom + kinds[(int)k->match.kind];
			*mapping = text.c_str();
		}
		if (hip_threads) *hip_threads = k->hip_threads;
		if (kernel_id) *kernel_id = k->kernel_id_;
	});
}

int tfhost_program_host_code(tfhost_program_t program, const char** listing) {
	return Guard([&] {
		if (!program || !listing) throw std::runtime_error("null argument");
		if (!program->program->host_code) throw std::runtime_error("the program has no host code");
		static thread_local std::string text;
		text = PrintHostCode(*program->program->host_code);
		*listing = text.c_str();
	});
}

int tfhost_program_compile_times(tfhost_program_t program, float* trace_s, float* codegen_s, float* kernel_compile_s) {
	return Guard([&] {
		if (!program) throw std::runtime_error("null argument");
		if (trace_s) *trace_s = program->program->trace_time;
		if (codegen_s) *codegen_s = program->program->codegen_time;
		if (kernel_compile_s) *kernel_compile_s = program->program->shader_compile_time / 1000.0f;
	});
}

int tfhost_load_programs(const char* library_path) {
	return Guard([&] {
		if (!library_path) throw std::runtime_error("null argument");
		// The library's static ProgramRegistrar objects add its programs to the registry while it loads.
		if (!dlopen(library_path, RTLD_NOW | RTLD_GLOBAL)) throw std::runtime_error(std::string("cannot load program library: ") + dlerror());
	});
}

int tfhost_program_execute(tfhost_program_t program, const tfhost_tensor_t* inputs, size_t n_inputs, tfhost_tensor_t* outputs, size_t max_outputs, size_t* n_outputs) {
	return Guard([&] {
		if (!program || !n_outputs) throw std::runtime_error("null argument");
		std::vector<TFTensor*> in;
		for (size_t i = 0; i < n_inputs; i++) {
			if (!inputs[i]) throw std::runtime_error("input " + std::to_string(i) + " is null");
			in.push_back(inputs[i]->tensor);
		}
		std::vector<TFTensor*> out = ExecuteProgram(program->program, in);
		if (out.size() > max_outputs) throw std::runtime_error("program returns " + std::to_string(out.size()) + " tensors, room for " + std::to_string(max_outputs));
		for (size_t i = 0; i < out.size(); i++) {
			// An output that is one of the inputs shares its buffer: only one handle may return it to the pool
			// (Definitions/TensorProgram.cpp:118-148 aliases the Python objects in that case).
			bool alias = false;
			for (TFTensor* t : in) alias |= (t->buffer == out[i]->buffer);
			outputs[i] = new tfhost_tensor{out[i], !alias};
		}
		*n_outputs = out.size();
	});
}

int tfhost_program_record(tfhost_program_t program, const tfhost_tensor_t* inputs, size_t n_inputs, size_t repeat, const int* feedback,
                          tfhost_tensor_t* outputs, size_t max_outputs, size_t* n_outputs, tfhost_graph_t* graph) {
	return Guard([&] {
		RequireMemory();
		if (!program || !n_outputs || !graph) throw std::runtime_error("null argument");
		std::vector<TFTensor*> in;
		for (size_t i = 0; i < n_inputs; i++) {
			if (!inputs[i]) throw std::runtime_error("input " + std::to_string(i) + " is null");
			in.push_back(inputs[i]->tensor);
		}
		if ((size_t)program->program->output_count > max_outputs)
			throw std::runtime_error("program returns " + std::to_string(program->program->output_count) + " tensors, room for " + std::to_string(max_outputs));
		RecordedProgram* recorded = RecordProgram(program->program, in, repeat, feedback ? std::vector<int>(feedback, feedback + n_inputs) : std::vector<int>());
		// The graph owns the output buffers: these handles never return them to the pool.
		for (size_t i = 0; i < recorded->outputs.size(); i++) outputs[i] = new tfhost_tensor{recorded->outputs[i], false};
		*n_outputs = recorded->outputs.size();
		*graph = new tfhost_graph{recorded};
	});
}

int tfhost_graph_replay(tfhost_graph_t graph) {
	return Guard([&] {
		if (!graph) throw std::runtime_error("null argument");
		ReplayProgram(graph->recorded);
	});
}

int tfhost_graph_node_count(tfhost_graph_t graph, size_t* nodes) {
	return Guard([&] {
		if (!graph || !nodes) throw std::runtime_error("null argument");
		*nodes = graph->recorded->nodes;
	});
}

int tfhost_graph_destroy(tfhost_graph_t graph) {
	return Guard([&] {
		if (!graph) return;
		DestroyRecordedProgram(graph->recorded);
		delete graph;
	});
}

int tfhost_tensor_create(const size_t* shape, size_t dim, int type, const uint32_t* data, tfhost_tensor_t* out) {
	return Guard([&] {
		RequireMemory();
		if (!shape || !out) throw std::runtime_error("null argument");
		if (type < 0 || type > 3) throw std::runtime_error("invalid tensor type");
		std::vector<size_t> s(shape, shape + dim);
		TFDataFormat format{(TFType)type, 32};
		TFTensor* t;
		if (data) {
			std::vector<uint32_t> words(data, data + GetLinearSize(s));
			t = global_memory_manager->AllocateTensorWithData(s, words, format);
		} else {
			t = global_memory_manager->AllocateTensor(s, format);
		}
		*out = new tfhost_tensor{t, true};
	});
}

int tfhost_tensor_info(tfhost_tensor_t tensor, size_t* shape, size_t shape_capacity, size_t* dim, int* type, size_t* words) {
	return Guard([&] {
		if (!tensor) throw std::runtime_error("null argument");
		const TFTensor* t = tensor->tensor;
		if (dim) *dim = t->dim;
		if (type) *type = (int)t->format.type;
		if (words) *words = GetSize(t);
		if (shape) {
			if (shape_capacity < t->dim) throw std::runtime_error("shape buffer too small");
			for (size_t i = 0; i < t->dim; i++) shape[i] = t->shape[i];
		}
	});
}

int tfhost_tensor_read(tfhost_tensor_t tensor, uint32_t* dst, size_t n_words) {
	return Guard([&] {
		RequireMemory();
		if (!tensor || !dst) throw std::runtime_error("null argument");
		if (n_words > GetSize(tensor->tensor)) throw std::runtime_error("read past the end of the tensor");
		((TFBufferTemplate*)tensor->tensor->buffer)->GetDataAtOffset(0, n_words, dst);
	});
}

int tfhost_tensor_write(tfhost_tensor_t tensor, const uint32_t* src, size_t n_words) {
	return Guard([&] {
		RequireMemory();
		if (!tensor || !src) throw std::runtime_error("null argument");
		if (n_words > GetSize(tensor->tensor)) throw std::runtime_error("write past the end of the tensor");
		((TFBufferTemplate*)tensor->tensor->buffer)->SetDataAtOffset(0, std::vector<uint32_t>(src, src + n_words));
	});
}

int tfhost_tensor_device_pointer(tfhost_tensor_t tensor, void** ptr) {
	return Guard([&] {
		if (!tensor || !ptr) throw std::runtime_error("null argument");
		*ptr = ((TFHipBuffer*)tensor->tensor->buffer)->GetNative();
	});
}

int tfhost_tensor_release(tfhost_tensor_t tensor) {
	return Guard([&] {
		if (!tensor) return;
		if (tensor->owns_buffer && global_memory_manager) global_memory_manager->DeallocateTensor(*tensor->tensor);
		delete tensor;
	});
}

int tfhost_memory_stats(size_t* allocated_words, size_t* unused_words, size_t* buffers_created, size_t* buffers_removed) {
	return Guard([&] {
		RequireMemory();
		if (allocated_words) *allocated_words = global_memory_manager->GetAllocatedSize();
		if (unused_words) *unused_words = global_memory_manager->GetUnusedAllocatedSize();
		if (buffers_created) *buffers_created = global_memory_manager->GetBuffersCreated();
		if (buffers_removed) *buffers_removed = global_memory_manager->GetBuffersRemoved();
	});
}

int tfhost_dispatch_stats(size_t* dispatches, size_t* served_by_primitives) {
	return Guard([&] {
		if (global_kernel_manager == nullptr) throw std::runtime_error("Backend not initialized");
		auto* km = (HipKernelManager*)global_kernel_manager;
		if (dispatches) *dispatches = km->dispatch_count;
		if (served_by_primitives) *served_by_primitives = km->idiom_dispatch_count;
	});
}

int tfhost_batched_launch_stats(size_t* launches, size_t* dispatches) {
	return Guard([&] {
		if (global_kernel_manager == nullptr) throw std::runtime_error("Backend not initialized");
		auto* km = (HipKernelManager*)global_kernel_manager;
		if (launches) *launches = km->batched_launch_count;
		if (dispatches) *dispatches = km->batched_dispatch_count;
	});
}

int tfhost_fused_chain_count(size_t* chains) {
	return Guard([&] {
		if (global_kernel_manager == nullptr) throw std::runtime_error("Backend not initialized");
		if (chains) *chains = ((HipKernelManager*)global_kernel_manager)->fused_chain_count;
	});
}

}  // extern "C"
