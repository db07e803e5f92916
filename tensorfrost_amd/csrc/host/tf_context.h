// Host-side runtime object of a TensorFrost program.
//
// Generated host programs carry a textual copy of this class (declaration
// TensorFrost/Backend/CodeGen/Langs/CPP.cpp:364-384, definitions :390-551) and reach the backend only
// through the TFRuntime callback table. The host programs in programs/ are written in the same emitted
// form (cf. GenerateMain, CPP.cpp:678-718) against this restatement, so that they exercise the backend
// through exactly the calls a JIT-compiled TensorFrost program makes.
#pragma once

#include <initializer_list>
#include <string>

#include "tf_abi.h"

namespace tfhost {

inline bool operator==(const TFDataFormat& a, const TFDataFormat& b) { return a.type == b.type && a.size == b.size; }
inline bool operator!=(const TFDataFormat& a, const TFDataFormat& b) { return !(a == b); }

#define TFTypeNone TFDataFormat{TFType_None, 0}
#define TFTypeBool32 TFDataFormat{TFType_Bool, 32}
#define TFTypeFloat32 TFDataFormat{TFType_Float, 32}
#define TFTypeInt32 TFDataFormat{TFType_Int, 32}
#define TFTypeUint32 TFDataFormat{TFType_Uint, 32}

inline uint32_t asuint(float x) {
	uint32_t u;
	__builtin_memcpy(&u, &x, 4);
	return u;
}
inline uint32_t asuint(double x) { return asuint((float)x); }
inline uint32_t asuint(int x) { return (uint32_t)x; }
inline uint32_t asuint(uint32_t x) { return x; }
inline float asfloat(uint32_t x) {
	float f;
	__builtin_memcpy(&f, &x, 4);
	return f;
}
inline int asint(uint32_t x) { return (int)x; }

class TFContext {
 public:
	TFRuntime runtime;

	explicit TFContext(TFRuntime runtime);
	size_t compute_size(const size_t* shape, size_t dim);
	TFTensor allocate(std::string name, std::initializer_list<size_t> shape, TFDataFormat type);
	void deallocate(TFTensor tensor);
	void check_tensor(TFTensor tensor, std::string name, std::initializer_list<size_t> target_shape, TFDataFormat target_type);
	TFTensor reshape(TFTensor tensor, std::string name, std::initializer_list<size_t> shape, TFDataFormat type);
	TFTensor assert_tensor(TFTensor tensor, std::string name, std::initializer_list<size_t> target_shape, TFDataFormat target_type);
	uint32_t read(TFTensor tensor, size_t index);
	void write(TFTensor tensor, size_t index, uint32_t value);
	void dispatch(size_t kernel_id, std::initializer_list<TFTensor> read_write, std::initializer_list<TFTensor> read_only,
	              std::initializer_list<uint32_t> var, std::initializer_list<size_t> shape, std::initializer_list<size_t> group);
	void region_begin(std::string name);
	void region_end(std::string name);
	void assert_value(std::string name, bool condition);
};

}  // namespace tfhost
