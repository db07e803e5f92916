// TEST INFRASTRUCTURE -- drives a tensor memory pool through a trace of allocations and releases and reports, step by
// step, which buffer served each request and which buffers were evicted.
//
// Compiled twice from this one file:
//   -DPOOL_REFERENCE  against TensorFrost/Backend/TensorMemory.h and linked with the reference's own, unmodified
//                     Backend/TensorMemory.cpp (recipe: oracle/ref/Makefile -> oracle/_ref/libref_pool.so);
//   otherwise         against this repository's restatement of that pool (tensorfrost_amd/csrc/host/tf_memory.{h,cpp}),
//                     compiled by tests/test_pool_against_reference.py.
// Both pools keep their buffers in std::unordered_set<TFBuffer*> and take "the last unused buffer the set's iteration
// yields" (TensorMemory.cpp:199-206), so which buffer serves a request depends on the buffers' ADDRESSES. The driver
// therefore places every buffer it creates at `arena + ordinal * stride`, ordinal counting the pool's CreateBuffer
// calls: two pools that make the same decisions on the same arena see the same addresses, hence the same iteration
// orders, and can be compared buffer for buffer. Nothing here is part of the product.
#include <cstddef>
#include <cstdint>
#include <new>
#include <stdexcept>
#include <vector>

#ifdef POOL_REFERENCE
#include "Backend/TensorMemory.h"
namespace pool = TensorFrost;
#else
#include "tf_memory.h"
namespace pool = tfhost;
#endif

namespace {

using namespace pool;

struct ArenaBuffer : TFBufferTemplate {
	long ordinal;
	ArenaBuffer(size_t size, long ordinal) : TFBufferTemplate(size), ordinal(ordinal) {}
	void UpdateName(const char* new_name) override { name = new_name; }
};

struct ArenaPool : TensorMemoryManager {
	char* arena;
	size_t stride, slots;
	long created = 0;
	std::vector<long> evicted;  // since the last call
	ArenaPool(void* arena, size_t stride, size_t slots) : arena((char*)arena), stride(stride), slots(slots) {
		if (stride < sizeof(ArenaBuffer)) throw std::runtime_error("arena stride too small");
	}
	TFBuffer* CreateBuffer(size_t size) override {
		if ((size_t)created >= slots) throw std::runtime_error("arena exhausted");
		ArenaBuffer* b = new (arena + (size_t)created * stride) ArenaBuffer(size, created);
		created++;
		return b;
	}
	void DeleteBuffer(TFBuffer* buffer) override {
		ArenaBuffer* b = static_cast<ArenaBuffer*>(buffer);
		evicted.push_back(b->ordinal);
		b->~ArenaBuffer();
	}
	ArenaBuffer* At(long ordinal) { return reinterpret_cast<ArenaBuffer*>(arena + (size_t)ordinal * stride); }
};

}  // namespace

extern "C" {

// The pool object is never destroyed: the reference's destructor calls the virtual DeleteBuffer from the base class
// (TensorMemory.cpp:226-232), which only a subclass still alive can answer. The arena belongs to the caller.
void* pool_create(void* arena, size_t stride, size_t slots) {
	try {
		return new ArenaPool(arena, stride, slots);
	} catch (...) {
		return nullptr;
	}
}

// Allocates `words` 32-bit words; returns the ordinal of the buffer that serves the request (negative on error), writes
// 1 to *created_new if the pool created it for this request, and the ordinals of the buffers evicted during the call to
// evicted[0 .. *n_evicted) (capacity cap).
long pool_alloc(void* handle, size_t words, int* created_new, long* evicted, size_t cap, size_t* n_evicted) {
	ArenaPool* p = (ArenaPool*)handle;
	try {
		p->evicted.clear();
		const long before = p->created;
		TFTensor* t = p->AllocateTensor({words}, TFDataFormat{(TFType)0, 32}, "trace");
		const long ordinal = static_cast<ArenaBuffer*>(t->buffer)->ordinal;
		*created_new = p->created != before;
		*n_evicted = p->evicted.size();
		for (size_t i = 0; i < p->evicted.size() && i < cap; i++) evicted[i] = p->evicted[i];
		return ordinal;
	} catch (...) {
		return -1;
	}
}

void pool_free(void* handle, long ordinal) {
	ArenaPool* p = (ArenaPool*)handle;
	TFTensor t{};
	t.buffer = p->At(ordinal);
	p->DeallocateTensor(t);
}

// The public fields of a live buffer as the pool left them.
void pool_buffer(void* handle, long ordinal, size_t* size, size_t* used_size, size_t* time_since_used) {
	ArenaBuffer* b = ((ArenaPool*)handle)->At(ordinal);
	*size = b->size;
	*used_size = b->used_size;
	*time_since_used = b->time_since_used;
}

size_t pool_allocated_words(void* handle) { return ((ArenaPool*)handle)->GetAllocatedSize(); }
size_t pool_unused_words(void* handle) { return ((ArenaPool*)handle)->GetUnusedAllocatedSize(); }
size_t pool_buffer_stride(void) { return (sizeof(ArenaBuffer) + 63) / 64 * 64; }

}  // extern "C"
