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

#include "tf_ir.h"
#include "tf_memory.h"
#include "tfhip.h"

namespace tfhost {

enum class BackendType { CPU, Vulkan, OpenGL, CodeGen, HIP, NotInitialized };
enum class CodeGenLang { CPP, HLSL, GLSL, HIP, None };

extern BackendType current_backend;
extern CodeGenLang current_kernel_lang;
extern std::string kernelCompileOptions;

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

class HipKernelManager : public KernelManager {
	std::unordered_map<size_t, tfhip_kernel_t> kernel_handles;
	std::unordered_map<size_t, tfhip_kernel_t> scalar_handles;  // one-thread-at-a-time entry points of four-wide kernels
	int compute_units = 0;

 public:
	~HipKernelManager() override { FreeAllKernels(); }
	// hiprtc-compiles kernel->full_generated_code_; throws with the compiler log and the source on failure.
	void CompileKernel(Kernel* kernel);
	// Follows chains of dispatches that together are one primitive (see DispatchChain); everything else goes
	// straight to DispatchNow.
	void DispatchKernel(TFDispatchInfo info) override;
	// Runs one dispatch: the primitive a kernel stands for, the primitive its idiom matches, or the emitted kernel.
	void DispatchNow(TFDispatchInfo info);
	// While dispatches are held back the buffers they name must not return to the pool: the runtime's deallocator
	// hands its tensors here instead.
	bool HasDeferredWork() const { return chain.stage != 0 || sort.state != SortRegion::Idle; }
	void DeferFree(TFTensor tensor);
	// Runs what is held back, in order, then the frees. Called before anything that is not the chain's next
	// dispatch: another dispatch, a readback or writeback, the end of the program.
	void FlushDeferred();
	// Region begin / end as the host program announces them (Backend.cpp:125-133). The `Radix sort` region of
	// tf.sort.radix (Python/TensorFrost/sort.py:74,176) is followed dispatch by dispatch, see SortRegion below.
	void OnRegion(const char* name, bool begin);
	// Reads the options that may change between executions (TFHIP_NO_IDIOMS); called once per program execution.
	void RefreshOptions();
	bool idioms_enabled = true;
	void FreeKernel(size_t kernel_id);
	void FreeAllKernels();
	size_t dispatch_count = 0;
	size_t idiom_dispatch_count = 0;  // dispatches of emitted kernels that a primitive served instead
	size_t fused_chain_count = 0;     // chains of dispatches that one primitive call served

 private:
	// The lowered row softmax (tests/autograd_test.py:29-31: m = max(x), e = exp(x - m), y = e / sum(e)) reaches the
	// backend as three kernels, or five when Optimization.cpp:469-510 has split the reductions:
	//   [chunk maxima ->] row maxima -> [chunk sums of exp(x - max) ->] row sums -> y = exp(x - max) / sum
	// A reduction that Optimization.cpp:469-510 has split is, likewise, two kernels: chunk (slab) results, then the same
	// operation over those. Once the program releases the chunk tensor, one call of the reduction primitive on the
	// original matrix serves both.
	// A dispatch that can open or continue such a sequence on the same tensors is held back instead of run. When the
	// last kernel arrives, one call of the fused primitive writes y, the row maxima and the row sums (the program may
	// read both later) and the chunk tensors, which the program has already released, are never written. Anything
	// else flushes: the dispatches held back run as they would have, in their order.
	struct Deferred {
		TFDispatchInfo info;
		std::vector<TFTensor> tensors;
		std::vector<uint32_t> variables;
	};
	struct DispatchChain {
		// 0 idle, 1 first stage of a split reduction held (chunks of rows, or slabs down the columns), 2 row maxima held,
		// 3 chunk sums of exp held, 4 row sums of exp held, 5 both stages of a split reduction held (not row maxima)
		int stage = 0;
		std::string op;     // stages 1 and 5: the reduction
		bool down = false;  // stages 1 and 5: down the columns
		// x: the matrix; chunk_max / row_max: results of the first / second stage of the (max) reduction
		TFBuffer *x = nullptr, *chunk_max = nullptr, *row_max = nullptr, *chunk_sum = nullptr, *row_sum = nullptr;
		long rows = 0, cols = 0, chunks = 0;  // of x; chunks (slabs) of the first stage
		long sum_chunks = 0;                  // chunks of the split sum of exp(x - max)
		std::vector<Deferred> dispatches;
		std::vector<TFTensor> frees;
	} chain;
	// tf.sort.radix brackets its work with region_begin('Radix sort') / region_end('Radix sort'). Between the two, every
	// dispatch is checked against the composition of sort.py:76-176 -- the copy (+ key map) kernels, then six passes of
	// {packed histogram, unpack, chunk sums, chunk scan, scan in chunks, digit totals, scatter} on ping-pong buffers, each
	// kernel structurally the one sort_composition.cpp builds, each dispatch with the buffers and scalars the data flow of
	// sort.py prescribes -- and held back, as are the deallocations. When the region ends complete and the program has
	// released every intermediate tensor and both ping-pong partners, ONE call of the onesweep sort reads the caller's
	// keys and values and leaves in the region's key / value buffers what the 44 kernels would have left. Any deviation
	// (another kernel, other scalars, a different buffer, a readback, a tensor that stays alive) runs what is held, in
	// order, as dispatched.
	struct SortRegion {
		enum State { Idle, Following, Closed } state = Idle;  // Closed: ended complete, waiting for the ping-pong partners' release
		int passes = 0;      // complete passes
		int iterations = 0;  // 'Radix sort iteration' regions begun
		bool in_iteration = false;
		int step = 0;        // dispatches of the current pass already seen
		bool has_values = true;
		long N = 0, G = 0, chunks = 0;
		struct Copy {
			TFBuffer *dst, *src;
			int role;
		};
		std::vector<Copy> copies;
		TFBuffer* keys[2] = {nullptr, nullptr};    // [0]: written by the prologue, holds the result; [1]: its ping-pong partner
		TFBuffer* values[2] = {nullptr, nullptr};
		TFBuffer *packed = nullptr, *hist = nullptr, *sums = nullptr, *sums_scanned = nullptr, *scan = nullptr, *total = nullptr;
		std::vector<TFBuffer*> intermediates;
		std::vector<Deferred> dispatches;
		std::vector<TFTensor> frees;
	} sort;
	bool FollowSortDispatch(const Kernel* kernel, const TFDispatchInfo& info);  // true: fits and is held
	bool SortRegionReleased() const;
	void RunSortRegion();     // the onesweep call, then the frees
	void AbandonSortRegion(); // what is held runs as dispatched, then the frees
	void HoldInto(std::vector<Deferred>& list, const TFDispatchInfo& info);
	void RunHeld(std::vector<Deferred>& dispatches, std::vector<TFTensor>& frees, std::exception_ptr error);
	bool AdvanceChain(const Kernel* kernel, const TFDispatchInfo& info);
	bool RunSplitReductionWhole();
	bool RunSoftmaxStatistics();
	void Hold(const TFDispatchInfo& info);
};

extern KernelManager* global_kernel_manager;

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
