// The HIP backend's three classes, written against TensorFrost's backend base classes only:
//   TFHipBuffer       : TFBufferTemplate        (Backend/TensorMemory.h:74-88;   cf. Backends/CPU/Memory.h:18-47)
//   HipMemoryManager  : TensorMemoryManager     (Backend/TensorMemory.h:118-125; cf. Backends/CPU/Memory.h:49-59)
//   HipKernelManager  : KernelManager           (Backend/KernelManager.h:16-30;  cf. Backends/OpenGL/KernelManager.h:105-159)
// "hip_shim_base.h" is the only tree-specific file: it includes the headers that define those base classes (and
// Kernel with its kernel_id_ / kernel_name_ / full_generated_code_ members) and names the namespace they live in.
// Everything else the classes use is the C ABI of libtfhip (tfhip.h) and the per-kernel table of hip_kernel_info.h.
#pragma once

#include <exception>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "hip_kernel_info.h"
#include "hip_shim_base.h"
#include "tfhip.h"

namespace TFSHIM_NAMESPACE {

using tfhip::HipKernelInfo;
using tfhip::IdiomMatchInfo;

// A hipMalloc-backed buffer of `size` 32-bit words.
class TFHipBuffer : public TFBufferTemplate {
 public:
	void* device = nullptr;
	explicit TFHipBuffer(size_t size);
	~TFHipBuffer();
	void UpdateName(const char* new_name) override {
		if (new_name != nullptr) name = new_name;
	}
	void SetDataAtOffset(size_t offset, const std::vector<uint32_t>& data) override;
	void GetDataAtOffset(size_t offset, size_t size, uint32_t* data) override;  // blocks until the stream has drained
	void* GetNative() const { return device; }
};

class HipMemoryManager : public TensorMemoryManager {
	// The base class keeps its buffer lists private, so the device allocations still alive when the manager goes
	// are found through this set.
	std::unordered_set<TFHipBuffer*> owned;

 public:
	~HipMemoryManager();

 protected:
	TFBuffer* CreateBuffer(size_t size) override;
	void DeleteBuffer(TFBuffer* buffer) override;
};

class HipKernelManager : public KernelManager {
	std::unordered_map<size_t, tfhip_kernel_t> kernel_handles;
	std::unordered_map<size_t, tfhip_kernel_t> scalar_handles;  // one-thread-at-a-time entry points of four-wide kernels
	std::unordered_map<size_t, tfhip_kernel_t> batch_handles;   // entry points that run several small dispatches in one launch
	std::unordered_map<size_t, HipKernelInfo> kernel_infos;
	int compute_units = 0;
	// Ticket counters of dispatches that share a loop among HIP groups (one word per group of 64 threads; zero between
	// launches: the group that takes the last ticket clears its counter).
	static constexpr size_t kSlabTicketWords = 4096;
	void* slab_tickets = nullptr;

 public:
	~HipKernelManager() { FreeAllKernels(); }
	// What the HIP code generator decided for a kernel; has to precede CompileKernel and any dispatch of that id.
	void SetKernelInfo(const HipKernelInfo& info) { kernel_infos[info.kernel_id] = info; }
	const HipKernelInfo* FindKernelInfo(size_t kernel_id) const {
		auto it = kernel_infos.find(kernel_id);
		return it == kernel_infos.end() ? nullptr : &it->second;
	}
	// hiprtc-compiles kernel->full_generated_code_ with these options; throws with the compiler log and the source on failure.
	void CompileKernel(Kernel* kernel);
	std::string compile_options;
	// Follows chains of dispatches that together are one primitive (see DispatchChain); everything else goes
	// straight to DispatchNow.
	void DispatchKernel(TFDispatchInfo info) override;
	// Runs one dispatch: the primitive a kernel stands for, the primitive its idiom matches, or the emitted kernel.
	void DispatchNow(TFDispatchInfo info);
	// While dispatches are held back the buffers they name must not return to the pool: the runtime's deallocator
	// hands its tensors here instead.
	bool HasDeferredWork() const { return chain.stage != 0 || sort.state != SortRegion::Idle || batch.calls != 0; }
	void DeferFree(TFTensor tensor);
	// Runs everything that is held back, in order, then the frees: before a readback or writeback and at the end of
	// the program.
	void FlushDeferred();
	// The same for the chains and the sort region only; gathered small dispatches (see Batch) stay gathered unless
	// buffers are about to return to the pool. Called before a dispatch that is not the chain's next one.
	void FlushChain();
	// Launches the small dispatches gathered so far (see Batch below), then returns the buffers released meanwhile.
	void FlushBatch();
	// Region begin / end as the host program announces them (Backend.cpp:125-133). The `Radix sort` region of
	// tf.sort.radix (Python/TensorFrost/sort.py:74,176) is followed dispatch by dispatch, see SortRegion below.
	void OnRegion(const char* name, bool begin);
	// Reads the options that may change between executions (TFHIP_NO_IDIOMS, TFHIP_NO_GATHER, TFHIP_TRACE_CHAINS); called
	// once per program execution.
	void RefreshOptions();
	bool idioms_enabled = true;
	bool gather_enabled = true;  // TFHIP_NO_GATHER: every dispatch leaves as its own launch (for a host that does not pass written tensors first)
	bool trace_chains = false;  // TFHIP_TRACE_CHAINS: one line on stderr per step of a chain of dispatches and per flush
	void FreeKernel(size_t kernel_id);
	void FreeAllKernels();
	size_t dispatch_count = 0;
	size_t idiom_dispatch_count = 0;  // dispatches of emitted kernels that a primitive served instead
	size_t fused_chain_count = 0;     // chains of dispatches that one primitive call served
	size_t batched_launch_count = 0;  // launches that carried more than one dispatch
	size_t batched_dispatch_count = 0;  // dispatches those launches carried

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
		// 3 chunk sums of exp held, 4 row sums of exp held, 5 both stages of a split reduction held (not row maxima),
		// 6 a weight-gradient product X^T dY held (x = dY [rows, cols]; a, c, m: X [rows, m] and the result [m, cols])
		// 7 E = exp(x - max) held as a tensor of its own, 8 chunk sums of E held, 9 row sums of E held, 10 Y = E / sums held
		// (complete: waits for the release of E), 11 whole column sums held (x = dY, row_sum = the sums: a bias gradient
		// dispatched before its weight gradient)
		int stage = 0;
		std::string op;     // stages 1 and 5: the reduction
		bool down = false;  // stages 1 and 5: down the columns
		// x: the matrix; chunk_max / row_max: results of the first / second stage of the (max) reduction
		TFBuffer *x = nullptr, *chunk_max = nullptr, *row_max = nullptr, *chunk_sum = nullptr, *row_sum = nullptr;
		long rows = 0, cols = 0, chunks = 0;  // of x; chunks (slabs) of the first stage
		long sum_chunks = 0;                  // chunks of the split sum of exp(x - max)
		TFBuffer *a = nullptr, *c = nullptr;  // stage 6
		TFBuffer *e = nullptr, *y = nullptr;  // stages 7-10
		long m = 0;
		std::vector<Deferred> dispatches;
		std::vector<TFTensor> frees;
	} chain;
	// tf.sort.radix brackets its work with region_begin('Radix sort') / region_end('Radix sort') and every pass with
	// 'Radix sort iteration' (Python/TensorFrost/sort.py:74,103,171,176). Between the outer two, every dispatch of an
	// emitted kernel is held back, as are the deallocations, together with the iteration it belongs to. When the region
	// ends, what was held is checked as a whole (ValidateSortRegion) by data flow and by what its kernels compute
	// (SortFeatures), not by how the compiler cut the work into kernels:
	//   * before the first iteration only element-wise copies run, and they make the first pass's keys (values) from
	//     buffers the region never writes: the caller's, through the identity or an order-preserving key map;
	//   * every iteration ends with the scatter kernel; pass p scatters by digit (key >> p*b) & (2^b - 1), reads what pass
	//     p - 1 wrote and writes the other buffer of a ping-pong pair; passes * b covers the 32 bits of a key;
	//   * every other kernel of an iteration reads only that pass's keys / values and buffers written earlier in the same
	//     iteration, writes only buffers outside the key / value chain, and one of them takes the pass's digit of the keys.
	// Then the region computes the stable ascending order of the whole (mapped) key, whatever its kernels look like, and
	// once the program has released every buffer the region wrote except the last pass's results, ONE call of the
	// onesweep sort leaves in those what the held kernels would have left. Anything else -- a primitive, a readback, a
	// kernel that reads or writes outside that pattern, shifts that do not cover the key, a buffer that stays alive --
	// runs what is held, in order, as dispatched.
	struct SortRegion {
		enum State { Idle, Following, Closed } state = Idle;  // Closed: ended and validated, waiting for the releases
		int iterations = 0;  // 'Radix sort iteration' regions begun
		bool in_iteration = false;
		std::vector<Deferred> dispatches;
		std::vector<int> iteration_of;                 // per held dispatch: -1 before the first iteration, else its iteration
		std::vector<const HipKernelInfo*> kernel_of;   // per held dispatch
		std::vector<TFTensor> frees;
		// What ValidateSortRegion found.
		long N = 0;
		int key_kind = 0;    // TFHIP_KEY_*
		bool has_values = true;
		TFBuffer *source_keys = nullptr, *source_values = nullptr;
		TFBuffer *result_keys = nullptr, *result_values = nullptr;  // written by the last pass
		TFBuffer *other_keys = nullptr, *other_values = nullptr;    // their ping-pong partners
		std::vector<TFBuffer*> intermediates;                       // everything else the region wrote
	} sort;
	bool FollowSortDispatch(const HipKernelInfo* kernel, const TFDispatchInfo& info);  // true: held
	bool ValidateSortRegion();  // fills the second half of `sort`
	bool SortRegionReleased() const;
	void RunSortRegion();     // the onesweep call, then the frees
	void AbandonSortRegion(); // what is held runs as dispatched, then the frees
	void HoldInto(std::vector<Deferred>& list, const TFDispatchInfo& info);
	void RunHeld(std::vector<Deferred>& dispatches, std::vector<TFTensor>& frees, std::exception_ptr error);
	bool AdvanceChain(const HipKernelInfo* kernel, const TFDispatchInfo& info);
	bool RunSplitReductionWhole();
	bool RunSoftmaxStatistics();
	bool RunSeparateExpSoftmax();
	// The backward pass of a dense layer dispatches dW = X^T dY and then db = the column sums of dY: the product is held
	// back for one dispatch, and when the sums of the same dY follow, one call computes both from one read of dY.
	bool HoldWeightGradient(const HipKernelInfo* kernel, const TFDispatchInfo& info);
	bool CompleteGradientPair(const HipKernelInfo* kernel, const TFDispatchInfo& info);
	bool CompleteGradientPairReversed(const HipKernelInfo* kernel, const TFDispatchInfo& info);
	void Hold(const TFDispatchInfo& info);
	void FinishChain();
	// Consecutive small dispatches of the same emitted kernel that touch disjoint buffers (the per-parameter updates of an
	// optimizer: Python/TensorFrost/optimizers.py:104-167 issues one kernel per parameter tensor) are gathered and leave
	// as one launch whose grid.y picks the dispatch: each of them alone runs about as long as a launch costs. A buffer
	// counts as written when it is among the kernel's read-write bindings. Anything else that reaches the stream, or
	// a different kernel, a full argument array or an overlap with a gathered dispatch, launches what is gathered
	// first; buffers released meanwhile return to the pool after that launch.
	struct Batch {
		size_t kernel_id = 0;
		const HipKernelInfo* kernel = nullptr;
		unsigned calls = 0;
		uint32_t grid = 0, threads = 0;
		std::vector<unsigned char> arguments;
		struct Range {
			const char *begin, *end;  // device bytes a gathered dispatch touches
			bool written;
		};
		std::vector<Range> buffers;
		std::vector<TFTensor> frees;
	} batch;
	bool Batchable(const HipKernelInfo* kernel, const TFDispatchInfo& info) const;
	void Gather(const HipKernelInfo* kernel, void* const* buffers, const size_t* buffer_bytes, size_t n_buffers, const uint32_t* vars, size_t n_vars, uint32_t grid, uint32_t threads);
};

}  // namespace TFSHIM_NAMESPACE
