#include "tf_context.h"

#include <stdexcept>
#include <vector>

namespace tfhost {

static const char* TypeLabel(TFType t) {
	switch (t) {
		case TFType_Float: return "Float";
		case TFType_Uint: return "Uint";
		case TFType_Int: return "Int";
		case TFType_Bool: return "Bool";
		default: return "None";
	}
}

TFContext::TFContext(TFRuntime runtime) : runtime(runtime) {}

size_t TFContext::compute_size(const size_t* shape, size_t dim) {
	size_t size = 1;
	for (size_t i = 0; i < dim; i++) size *= shape[i];
	return size;
}

TFTensor TFContext::allocate(std::string name, std::initializer_list<size_t> shape, TFDataFormat type) {
	const size_t* shape_arr = shape.begin();
	size_t dim = shape.size();
	for (size_t i = 0; i < dim; i++) {
		if (shape_arr[i] < 1)
			throw std::runtime_error("Invalid shape on dimension " + std::to_string(i) + " for " + name + ". Expected positive integer, got " + std::to_string(shape_arr[i]));
	}
	return runtime.alloc(name.c_str(), shape_arr, dim, type, runtime.custom_data);
}

void TFContext::deallocate(TFTensor tensor) { runtime.dealloc(tensor, runtime.custom_data); }

void TFContext::check_tensor(TFTensor tensor, std::string name, std::initializer_list<size_t> target_shape, TFDataFormat target_format) {
	const size_t* target = target_shape.begin();
	if (tensor.format != target_format)
		throw std::runtime_error("Invalid type for " + name + ". Expected " + TypeLabel(target_format.type) + ", got " + TypeLabel(tensor.format.type));
	if (tensor.dim != target_shape.size())
		throw std::runtime_error("Invalid number of dimensions for " + name + ". Expected " + std::to_string(target_shape.size()) + ", got " + std::to_string(tensor.dim));
	for (size_t i = 0; i < tensor.dim; i++) {
		if (tensor.shape[i] != target[i] || target[i] < 1)
			throw std::runtime_error("Invalid shape for dimension " + std::to_string(i) + " in " + name + ". Expected " + std::to_string(target[i]) + ", got " + std::to_string(tensor.shape[i]));
	}
}

TFTensor TFContext::reshape(TFTensor tensor, std::string name, std::initializer_list<size_t> shape, TFDataFormat type) {
	size_t* new_shape = new size_t[shape.size()];
	std::copy(shape.begin(), shape.end(), new_shape);
	TFTensor result = {tensor.buffer, type, shape.size(), new_shape};
	size_t old_size = compute_size(tensor.shape, tensor.dim);
	size_t new_size = compute_size(result.shape, result.dim);
	if (old_size != new_size)
		throw std::runtime_error("Cannot reshape " + name + ", expected " + std::to_string(new_size) + " elements, while input has " + std::to_string(old_size));
	return result;
}

TFTensor TFContext::assert_tensor(TFTensor tensor, std::string name, std::initializer_list<size_t> target_shape, TFDataFormat target_type) {
	check_tensor(tensor, name, target_shape, target_type);
	return tensor;
}

uint32_t TFContext::read(TFTensor tensor, size_t index) { return runtime.readback(tensor, index, runtime.custom_data); }
void TFContext::write(TFTensor tensor, size_t index, uint32_t value) { runtime.writeback(tensor, index, value, runtime.custom_data); }

void TFContext::dispatch(size_t kernel_id, std::initializer_list<TFTensor> read_write, std::initializer_list<TFTensor> read_only,
                         std::initializer_list<uint32_t> var, std::initializer_list<size_t> shape, std::initializer_list<size_t> group) {
	// All tensors travel in the read-write list, read-write ones first; one extra variable word carries the
	// group index offset (always 0 here).
	std::vector<TFTensor> all_tensors(read_write.begin(), read_write.end());
	all_tensors.insert(all_tensors.end(), read_only.begin(), read_only.end());
	std::vector<uint32_t> all_vars(var.begin(), var.end());
	all_vars.push_back(0);
	TFDispatchInfo info = {kernel_id, all_tensors.size(), all_tensors.data(), 0, nullptr, all_vars.size(), all_vars.data(), 0};
	for (const TFTensor& t : read_write) t.buffer->up_to_date = false;

	// Outer dimensions multiply; the last group.size() dimensions are divided (rounding up) by the group
	// size, group[i] pairing with shape[dim-1-i].
	const size_t* shape_arr = shape.begin();
	const size_t* group_arr = group.begin();
	size_t dispatch_dim = shape.size(), group_dim = group.size();
	size_t work_group_count = 1;
	for (size_t i = 0; i < dispatch_dim - group_dim; i++) work_group_count *= shape_arr[i];
	for (size_t i = 0; i < group_dim; i++) {
		size_t dim = shape_arr[dispatch_dim - i - 1];
		work_group_count *= (dim + group_arr[i] - 1) / group_arr[i];
	}
	info.work_group_count = work_group_count;
	runtime.dispatch(info, runtime.custom_data);
}

void TFContext::region_begin(std::string name) {
	if (runtime.region) runtime.region(name.c_str(), true, runtime.custom_data);
}
void TFContext::region_end(std::string name) {
	if (runtime.region) runtime.region(name.c_str(), false, runtime.custom_data);
}
void TFContext::assert_value(std::string name, bool condition) {
	if (!condition) throw std::runtime_error("Assertion failed: " + name);
}

}  // namespace tfhost
