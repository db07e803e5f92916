// Tensor memory: the pooling allocator the generated host programs allocate from, and its HIP buffers.
//
// TensorMemoryManager / TFBufferTemplate restate the backend-independent part of
// TensorFrost/Backend/TensorMemory.{h,cpp} (class layout :74-141, pool logic .cpp:29-55,104-118,145-224):
// first-fit reuse of an unused buffer whose capacity lies in [n, 16n], a tick per allocation, eviction of
// buffers left unused for longer than the adaptive delay of their size class. The HIP subclasses live in
// shim/HIP.h and depend on nothing but the two base classes here, so that they compile unchanged against the
// TensorFrost tree's own header (cf. Backends/CPU/Memory.h:18-59, Backends/OpenGL/Memory.h:16-116).
#pragma once

#include <map>
#include <stdexcept>
#include <unordered_set>
#include <vector>

#include "tf_abi.h"

namespace tfhost {

class TFBufferTemplate : public TFBuffer {
 public:
	explicit TFBufferTemplate(size_t size) : TFBuffer{size, 0, 0, false, false, nullptr} {}
	virtual ~TFBufferTemplate() = default;
	virtual void UpdateName(const char*) { throw std::runtime_error("UpdateName not implemented"); }
	virtual void SetDataAtOffset(size_t, const std::vector<uint32_t>&) { throw std::runtime_error("SetDataAtOffset not implemented"); }
	virtual void GetDataAtOffset(size_t, size_t, uint32_t*) { throw std::runtime_error("GetDataAtOffset not implemented"); }
};

size_t GetLinearSize(const std::vector<size_t>& shape);
std::vector<size_t> GetShape(const TFTensor* tensor);
size_t GetSize(const TFTensor* tensor);

class TensorMemoryManager {
 private:
	size_t tick = 0;
	size_t buffers_created = 0;
	size_t buffers_removed = 0;
	static constexpr size_t DEFAULT_MAX_UNUSED_TIME = 128;
	static constexpr size_t MAX_POSSIBLE_UNUSED_TIME = 32768;
	std::map<size_t, std::unordered_set<TFBuffer*>> allocated_buffers;
	std::map<size_t, size_t> allocation_history;  // last tick at which a buffer of this size was created
	std::map<size_t, size_t> allocation_delay;    // unused ticks a buffer of this size survives
	std::unordered_set<TFBuffer*> unused_buffers;
	// Recording a graph (no counterpart in the reference): buffers handed out while `holding` are collected in
	// `held`; when recording ends they become `reserved`, i.e. they belong to the graph and stay out of the pool
	// until the graph is destroyed. Nothing is evicted while holding.
	bool holding = false;
	std::unordered_set<TFBuffer*> held;
	std::unordered_set<TFBuffer*> reserved;

	static TFTensor* MakeTensor(const std::vector<size_t>& shape, TFBuffer* buf, TFDataFormat type);
	void UpdateTick();
	size_t GetDeallocationDelay(size_t size) const;
	TFBuffer* AllocateBuffer(size_t size);
	TFBuffer* TryAllocateBuffer(size_t size);
	void DeallocateBuffer(TFBuffer* buffer);
	void RemoveBuffer(TFBuffer* buffer);

 protected:
	virtual TFBuffer* CreateBuffer(size_t) { throw std::runtime_error("CreateBuffer not implemented"); }
	virtual void DeleteBuffer(TFBuffer*) { throw std::runtime_error("DeleteBuffer not implemented"); }
	// Subclasses call this from their destructor while their DeleteBuffer is still reachable.
	void ReleaseAll();

 public:
	virtual std::vector<uint32_t> Readback(const TFTensor* memory);
	virtual uint32_t ReadbackValue(const TFTensor* memory, size_t index);
	virtual void Writeback(const TFTensor* memory, const std::vector<uint32_t>& data);
	virtual void WritebackValue(const TFTensor* memory, size_t index, uint32_t value);

	TFTensor* AllocateTensor(const std::vector<size_t>& shape, TFDataFormat type, const char* name = nullptr);
	TFTensor* AllocateTensorWithData(const std::vector<size_t>& shape, const std::vector<uint32_t>& data, TFDataFormat type,
	                                 bool read_only = false, const char* name = nullptr);
	void DeallocateTensor(TFTensor tensor);

	void BeginHold();
	// reserve = true: the held buffers leave the pool and are returned to the caller, who owns them until
	// Unreserve. reserve = false (recording failed): held buffers still handed out go back to the pool.
	std::vector<TFBuffer*> EndHold(bool reserve);
	void Unreserve(const std::vector<TFBuffer*>& buffers);

	size_t GetAllocatedSize() const;
	size_t GetUnusedAllocatedSize() const;
	size_t GetBuffersCreated() const { return buffers_created; }
	size_t GetBuffersRemoved() const { return buffers_removed; }

	virtual ~TensorMemoryManager();
};

extern TensorMemoryManager* global_memory_manager;

}  // namespace tfhost
