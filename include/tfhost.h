/*
 * tfhost.h -- C driver surface of libtfhost.so, the C++ host side of the HIP backend (memory pool,
 * kernel manager, HIP emitter, program execution). It stands where TensorFrost's pybind11 module stands
 * for a Python user and exists so that tests and benchmarks can drive the backend through the same
 * sequence of calls:
 *   tf.initialize(backend, options)   TensorFrost/Frontend/Python/PybindModule.cpp:112-115
 *   tf.compile(fn)                    Frontend/Python/Definitions/TensorProgram.cpp:12-65
 *   program(*inputs)                  Frontend/Python/Definitions/TensorProgram.cpp:67-150
 *   tf.tensor(array) / tensor.numpy   Frontend/Python/Definitions/TensorMemory.cpp:24-29, PyTensorMemory.h:29-45
 *   tf.allocated_memory / unused      Frontend/Python/Definitions/TensorMemory.cpp:65-69
 * Programs are chosen by name from a built-in registry (the Python tracer is outside the backend).
 * Every call returns 0 or a negative status with tfhost_last_error() set; C++ exceptions (the reference's
 * error channel, surfaced to Python as RuntimeError) never cross this boundary.
 */
#ifndef TFHOST_H
#define TFHOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tfhost_program* tfhost_program_t;
typedef struct tfhost_tensor* tfhost_tensor_t;
typedef struct tfhost_graph* tfhost_graph_t;

#define TFHOST_BACKEND_HIP 0
#define TFHOST_BACKEND_CODEGEN 1 /* emit + compile source, never execute (the reference's tf.codegen) */

int tfhost_initialize(int backend, const char* kernel_compile_options);
int tfhost_shutdown(void);
const char* tfhost_last_error(void);
int tfhost_sync(void);

/* tf.compile: builds the named program's kernels, emits HIP for each, compiles them. */
int tfhost_program_create(const char* name, const int64_t* params, size_t n_params, tfhost_program_t* out);
int tfhost_program_destroy(tfhost_program_t program);
int tfhost_program_kernel_count(tfhost_program_t program, size_t* count);
/* Borrowed strings, valid until the program is destroyed: emitted source, how the emitter mapped the
 * kernel onto the GPU ("flat", "group", "reduction:wave", "primitive:<name>"), threads per HIP group. */
int tfhost_program_kernel_info(tfhost_program_t program, size_t index, const char** source, const char** mapping, int* hip_threads, size_t* kernel_id);
/* The program's host code -- input checks, allocations, host scalars, dispatches, regions, host loops -- as the
 * instruction list the host interpreter runs, one per line (borrowed string, valid until the next call on this
 * thread). It stands where the reference's generated C++ `main` stands (GenerateMain,
 * Backend/CodeGen/Langs/CPP.cpp:678-718), which the reference compiles with the system compiler
 * (Backends/CPU/KernelCompiler.cpp:94-220); here it is interpreted, so tf.compile needs no host compiler. */
int tfhost_program_host_code(tfhost_program_t program, const char** listing);
/* Seconds tf.compile spent on this program: building the tree, generating kernel source and host code, compiling
 * the kernels (the reference prints the last two as "Host Compile time" / "Shader compile time",
 * Frontend/Python/Definitions/TensorProgram.cpp:40-60). Any pointer may be NULL. */
int tfhost_program_compile_times(tfhost_program_t program, float* trace_s, float* codegen_s, float* kernel_compile_s);
/* Adds the programs of a shared library (static ProgramRegistrar objects, csrc/host/programs/registry.h) to the
 * registry tf.compile chooses from; the test suite keeps its op-by-op programs in such a library. */
int tfhost_load_programs(const char* library_path);
/* program(*inputs): outputs[0..*n_outputs) receive new tensor handles (capacity max_outputs). */
int tfhost_program_execute(tfhost_program_t program, const tfhost_tensor_t* inputs, size_t n_inputs, tfhost_tensor_t* outputs, size_t max_outputs, size_t* n_outputs);

/* Records `repeat` executions of the program on these inputs as one HIP graph (after one ordinary execution that
 * loads modules and sizes the pool) and returns handles of the last execution's outputs. Nothing recorded has run
 * yet: tfhost_graph_replay enqueues it, as often as wanted, always on the same buffers. The caller changes the
 * inputs between replays by writing into the input tensors, which must outlive the graph. feedback is NULL or
 * holds n_inputs entries: feedback[i] is the index of the output that becomes input i in the next execution (same
 * shape and type), or -1 for an input that stays as it is. With feedback the graph ends by copying the last
 * outputs into the inputs they feed, so each replay advances an iteration by `repeat` steps. The reference
 * has no counterpart; this replaces calling program(*inputs) again and again
 * (Frontend/Python/Definitions/TensorProgram.cpp:67-150) where the per-call host work matters. A program that
 * reads values back while it runs (Readback callback, Backend.cpp:108-111) cannot be recorded.
 * The output handles stay valid until tfhost_graph_destroy, which returns every buffer of the graph to the pool;
 * releasing them earlier only drops the handle. */
int tfhost_program_record(tfhost_program_t program, const tfhost_tensor_t* inputs, size_t n_inputs, size_t repeat, const int* feedback,
                          tfhost_tensor_t* outputs, size_t max_outputs, size_t* n_outputs, tfhost_graph_t* graph);
int tfhost_graph_replay(tfhost_graph_t graph);
int tfhost_graph_node_count(tfhost_graph_t graph, size_t* nodes);
int tfhost_graph_destroy(tfhost_graph_t graph);

/* tf.tensor(array): type is a TFType value (0 float, 1 uint, 2 int, 3 bool); data holds prod(shape) words. */
int tfhost_tensor_create(const size_t* shape, size_t dim, int type, const uint32_t* data, tfhost_tensor_t* out);
int tfhost_tensor_info(tfhost_tensor_t tensor, size_t* shape, size_t shape_capacity, size_t* dim, int* type, size_t* words);
int tfhost_tensor_read(tfhost_tensor_t tensor, uint32_t* dst, size_t n_words); /* tensor.numpy; blocks */
/* Overwrites the first n_words of the tensor's buffer (TFBufferTemplate::SetDataAtOffset, Backend/TensorMemory.h:74-88);
 * blocks until the copy is done. This is how the inputs of a recorded graph are changed between replays. */
int tfhost_tensor_write(tfhost_tensor_t tensor, const uint32_t* src, size_t n_words);
int tfhost_tensor_device_pointer(tfhost_tensor_t tensor, void** ptr);
/* Drops the handle and returns its buffer to the pool (what the Python wrapper's destructor does). */
int tfhost_tensor_release(tfhost_tensor_t tensor);

/* Pool statistics in 32-bit words / buffer counts. */
int tfhost_memory_stats(size_t* allocated_words, size_t* unused_words, size_t* buffers_created, size_t* buffers_removed);

/* Dispatches since initialisation, and how many of those were emitted kernels recognised as one reduction /
   prefix-sum / matmul loop (Compiler/Implementations.cpp:243-359,560-646) that a primitive served instead. */
int tfhost_dispatch_stats(size_t* dispatches, size_t* served_by_primitives);
/* How many times a whole sequence of dispatches was served by one primitive call: the three or five kernels of a
   lowered row softmax (max, sum of exp(x - max), normalise; tests/autograd_test.py:29-31, reductions split by
   Compiler/Steps/Optimization.cpp:469-510). Their dispatches also count in tfhost_dispatch_stats. */
int tfhost_fused_chain_count(size_t* chains);
/* Launches that carried more than one dispatch, and how many dispatches they carried: consecutive small dispatches of
   one emitted kernel on disjoint buffers (the per-parameter kernels of Python/TensorFrost/optimizers.py:104-167) leave
   as one launch. Their dispatches also count in tfhost_dispatch_stats. */
int tfhost_batched_launch_stats(size_t* launches, size_t* dispatches);

#ifdef __cplusplus
}
#endif
#endif /* TFHOST_H */
