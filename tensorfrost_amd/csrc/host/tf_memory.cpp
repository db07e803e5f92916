#include "tf_memory.h"

#include <algorithm>
#include <string>

#include "tfhip.h"

namespace tfhost {

TensorMemoryManager* global_memory_manager = nullptr;

size_t GetLinearSize(const std::vector<size_t>& shape) {
	size_t size = 1;
	for (size_t d : shape) size *= d;
	return size;
}

std::vector<size_t> GetShape(const TFTensor* tensor) { return std::vector<size_t>(tensor->shape, tensor->shape + tensor->dim); }

size_t GetSize(const TFTensor* tensor) {
	size_t size = 1;
	for (size_t i = 0; i < tensor->dim; i++) size *= tensor->shape[i];
	return size;
}

// ---- pool (TensorMemory.cpp:29-55,104-118,145-224) -------------------------------------------------

TFBuffer* TensorMemoryManager::AllocateBuffer(size_t size) {
	TFBuffer* buffer = CreateBuffer(size);
	auto seen = allocation_history.find(size);
	if (seen != allocation_history.end()) {
		// A size that keeps being re-created is kept alive longer next time.
		size_t since_last = tick - seen->second;
		allocation_delay[size] = std::min(std::max(GetDeallocationDelay(size), since_last), MAX_POSSIBLE_UNUSED_TIME);
	} else {
		allocation_delay[size] = DEFAULT_MAX_UNUSED_TIME;
	}
	buffers_created++;
	allocated_buffers[size].insert(buffer);
	allocation_history[size] = tick;
	return buffer;
}

TFBuffer* TensorMemoryManager::TryAllocateBuffer(size_t size) {
	// Smallest size class in [size, 16*size] that has an unused buffer wins.
	TFBuffer* found = nullptr;
	const size_t max_size = 16 * size;
	for (auto it = allocated_buffers.lower_bound(size); it != allocated_buffers.end() && it->first <= max_size; ++it) {
		for (TFBuffer* candidate : it->second) {
			if (unused_buffers.count(candidate)) found = candidate;
		}
		if (found) break;
	}
	if (found)
		unused_buffers.erase(found);
	else
		found = AllocateBuffer(size);
	found->used_size = size;
	found->time_since_used = 0;
	if (holding) held.insert(found);
	UpdateTick();
	return found;
}

void TensorMemoryManager::UpdateTick() {
	std::vector<TFBuffer*> expired;
	if (holding) {  // recorded work refers to buffers that look unused
		tick++;
		return;
	}
	for (TFBuffer* buffer : unused_buffers) {
		if (buffer->time_since_used > GetDeallocationDelay(buffer->size))
			expired.push_back(buffer);
		else
			buffer->time_since_used++;
	}
	for (TFBuffer* buffer : expired) RemoveBuffer(buffer);
	tick++;
}

size_t TensorMemoryManager::GetDeallocationDelay(size_t size) const {
	auto it = allocation_delay.find(size);
	return it == allocation_delay.end() ? DEFAULT_MAX_UNUSED_TIME : it->second;
}

void TensorMemoryManager::DeallocateBuffer(TFBuffer* buffer) {
	if (reserved.count(buffer)) return;  // owned by a recorded graph
	unused_buffers.insert(buffer);
	buffer->time_since_used = 0;
	buffer->used_size = 0;
	buffer->up_to_date = false;
	buffer->name = "none";
}

void TensorMemoryManager::BeginHold() {
	if (holding) throw std::runtime_error("a graph is already being recorded");
	holding = true;
	held.clear();
}

std::vector<TFBuffer*> TensorMemoryManager::EndHold(bool reserve) {
	holding = false;
	std::vector<TFBuffer*> buffers(held.begin(), held.end());
	held.clear();
	for (TFBuffer* buffer : buffers) {
		if (reserve) {
			unused_buffers.erase(buffer);
			reserved.insert(buffer);
		} else if (!unused_buffers.count(buffer)) {
			DeallocateBuffer(buffer);
		}
	}
	return buffers;
}

void TensorMemoryManager::Unreserve(const std::vector<TFBuffer*>& buffers) {
	for (TFBuffer* buffer : buffers) {
		if (reserved.erase(buffer)) DeallocateBuffer(buffer);
	}
}

void TensorMemoryManager::RemoveBuffer(TFBuffer* buffer) {
	allocated_buffers[buffer->size].erase(buffer);
	unused_buffers.erase(buffer);
	DeleteBuffer(buffer);
	buffers_removed++;
}

TFTensor* TensorMemoryManager::MakeTensor(const std::vector<size_t>& shape, TFBuffer* buf, TFDataFormat type) {
	// Tensor headers and their shape arrays live for the rest of the process, as in the reference
	// (TensorMemory.cpp:69-82): generated programs keep returning them by value.
	size_t* shape_arr = new size_t[shape.size()];
	std::copy(shape.begin(), shape.end(), shape_arr);
	TFTensor* tensor = new TFTensor();
	tensor->buffer = buf;
	tensor->format = type;
	tensor->dim = shape.size();
	tensor->shape = shape_arr;
	return tensor;
}

TFTensor* TensorMemoryManager::AllocateTensor(const std::vector<size_t>& shape, TFDataFormat type, const char* name) {
	size_t size = GetLinearSize(shape);
	if (size == 0) throw std::invalid_argument("Trying to allocate a tensor with size 0");
	TFBuffer* buf = TryAllocateBuffer(size);
	buf->read_only = false;
	((TFBufferTemplate*)buf)->UpdateName(name);
	return MakeTensor(shape, buf, type);
}

TFTensor* TensorMemoryManager::AllocateTensorWithData(const std::vector<size_t>& shape, const std::vector<uint32_t>& data, TFDataFormat type,
                                                      bool read_only, const char* name) {
	TFTensor* tensor = AllocateTensor(shape, type, name);
	tensor->buffer->read_only = read_only;
	((TFBufferTemplate*)tensor->buffer)->SetDataAtOffset(0, data);
	return tensor;
}

void TensorMemoryManager::DeallocateTensor(TFTensor tensor) { DeallocateBuffer(tensor.buffer); }

std::vector<uint32_t> TensorMemoryManager::Readback(const TFTensor* memory) {
	std::vector<uint32_t> data(GetSize(memory));
	((TFBufferTemplate*)memory->buffer)->GetDataAtOffset(0, data.size(), data.data());
	return data;
}

uint32_t TensorMemoryManager::ReadbackValue(const TFTensor* memory, size_t index) {
	uint32_t value;
	((TFBufferTemplate*)memory->buffer)->GetDataAtOffset(index, 1, &value);
	return value;
}

void TensorMemoryManager::Writeback(const TFTensor* memory, const std::vector<uint32_t>& data) {
	((TFBufferTemplate*)memory->buffer)->SetDataAtOffset(0, data);
}

void TensorMemoryManager::WritebackValue(const TFTensor* memory, size_t index, uint32_t value) {
	((TFBufferTemplate*)memory->buffer)->SetDataAtOffset(index, {value});
}

size_t TensorMemoryManager::GetAllocatedSize() const {
	size_t total = 0;
	for (auto& [size, buffers] : allocated_buffers) total += size * buffers.size();
	return total;
}

size_t TensorMemoryManager::GetUnusedAllocatedSize() const {
	size_t total = 0;
	for (TFBuffer* buffer : unused_buffers) total += buffer->size;
	return total;
}

void TensorMemoryManager::ReleaseAll() {
	for (auto& [size, buffers] : allocated_buffers)
		for (TFBuffer* buffer : buffers) DeleteBuffer(buffer);
	allocated_buffers.clear();
	unused_buffers.clear();
}

TensorMemoryManager::~TensorMemoryManager() {}

}  // namespace tfhost
