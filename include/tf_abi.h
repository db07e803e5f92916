/*
 * tf_abi.h -- binary interface between a TensorFrost host program and a backend runtime.
 *
 * Every TensorFrost program is a JIT-compiled C++ shared object whose entry symbol "main" receives
 * input/output tensor arrays and a table of six callbacks (TFRuntime). The structs below are a
 * restatement of that interface; a backend that fills the table with its own functions is a drop-in.
 *
 * Replaces nothing -- it must stay byte-compatible with:
 *   TensorFrost/Backend/TensorMemory.h:19-72           (runtime side)
 *   TensorFrost/Backend/CodeGen/Langs/CPP.cpp:273-362  (copy embedded in every generated program)
 *   TensorFrost/Compiler/Operations.h (TFType / TFDataFormat)
 * The static_asserts pin the layout on LP64.
 */
#ifndef TF_ABI_H
#define TF_ABI_H

#include <stddef.h>
#include <stdint.h>
#ifndef __cplusplus
#include <stdbool.h>
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Element kinds. All storage is 32-bit words; the kind only steers reinterpretation. */
typedef enum TFType { TFType_Float = 0, TFType_Uint = 1, TFType_Int = 2, TFType_Bool = 3, TFType_None = 4 } TFType;

typedef struct TFDataFormat {
	TFType type;  /* 4 bytes + 4 padding */
	size_t size;  /* bit width, always 32 (0 for None) */
} TFDataFormat;

/* Header shared by every backend's buffer object; backends append their own fields behind it. */
typedef struct TFBuffer {
	size_t size;            /* capacity in 32-bit words */
	size_t used_size;       /* words handed out by the last allocation */
	size_t time_since_used; /* pool ticks since release */
	bool up_to_date;        /* host-cache hint, cleared by dispatch on read-write tensors */
	bool read_only;
	const char* name;
} TFBuffer;

typedef struct TFTensor {
	TFBuffer* buffer;
	TFDataFormat format;
	size_t dim;
	const size_t* shape; /* outermost first */
} TFTensor;

typedef struct TFTensorList {
	size_t count;
	const TFTensor* tensors;
} TFTensorList;

typedef struct TFDispatchInfo {
	size_t kernel_id;
	size_t read_write_count;             /* generated hosts put ALL tensors here (rw first, then ro) */
	const TFTensor* read_write_tensors;
	size_t read_only_count;              /* always 0 from generated hosts */
	const TFTensor* read_only_tensors;
	size_t variable_count;               /* user scalars + trailing block offset word */
	const uint32_t* variables;
	size_t work_group_count;             /* 1-D grid */
} TFDispatchInfo;

typedef TFTensor tf_alloc_func(const char* name, const size_t* shape, size_t dim, TFDataFormat format, void* user);
typedef void tf_dealloc_func(TFTensor tensor, void* user);
typedef uint32_t tf_readback_func(TFTensor tensor, size_t index, void* user);
typedef void tf_writeback_func(TFTensor tensor, size_t index, uint32_t value, void* user);
typedef void tf_dispatch_func(TFDispatchInfo info, void* user);
typedef void tf_region_func(const char* name, bool begin, void* user);

typedef struct TFRuntime {
	tf_alloc_func* alloc;
	tf_dealloc_func* dealloc;
	tf_readback_func* readback;
	tf_writeback_func* writeback;
	tf_dispatch_func* dispatch;
	tf_region_func* region;
	void* custom_data;
} TFRuntime;

/* Entry point of a JIT-compiled host program (symbol "main"). */
typedef int tf_main_func(TFTensor* in, TFTensor* out, TFRuntime runtime);

#ifdef __cplusplus
}  /* extern "C" */

static_assert(sizeof(TFDataFormat) == 16, "TFDataFormat layout");
static_assert(sizeof(TFBuffer) == 40, "TFBuffer layout");
static_assert(offsetof(TFBuffer, up_to_date) == 24 && offsetof(TFBuffer, read_only) == 25 && offsetof(TFBuffer, name) == 32, "TFBuffer layout");
static_assert(sizeof(TFTensor) == 40, "TFTensor layout");
static_assert(offsetof(TFTensor, format) == 8 && offsetof(TFTensor, dim) == 24 && offsetof(TFTensor, shape) == 32, "TFTensor layout");
static_assert(sizeof(TFDispatchInfo) == 64, "TFDispatchInfo layout");
static_assert(sizeof(TFRuntime) == 56, "TFRuntime layout");
#endif

#endif /* TF_ABI_H */
