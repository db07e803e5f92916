// Kernel-level intermediate representation consumed by the HIP emitter.
//
// The emitter's real input is TensorFrost's own IR after all passes have run: a tree of nodes under a
// "kernel" node whose memory accesses already carry flat addresses and whose thread indices are already
// expressed through block_id / block_thread_id (TensorFrost/Compiler/Graph/Node.h,
// Compiler/KernelGen.h:17-46 `Kernel`, :48-71 `Program`; index finalisation
// Compiler/Steps/GraphOps.cpp:1091-1186). That tree cannot be built in this repository (the frontend and
// passes are outside the backend), so this header restates the part of it a code generator reads:
// the op table of post-lowering operations (Compiler/Operations.cpp:23-179, everything that is not
// Algorithm/Gradient/host-only), node arguments by kind (input / index / memory), constants, debug
// names, the Modified flag, and children of scope nodes. `KernelBuilder` produces trees in exactly the
// shape the reference's passes leave behind, including its lowered idioms (reduction / scan / matmul
// loops, Compiler/Implementations.cpp:243-359,560-646).
#pragma once

#include <cstdint>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "tf_abi.h"

namespace tfhost {

enum class OpClass { Operator, UnaryOperator, Function, Copy, Keyword, DimensionIndex, Variable, TypeCast, TypeReinterpret, Constant, TernaryOperator, Special, Memory, Set };

struct OpInfo {
	const char* name;
	const char* code;  // operator token / function name
	OpClass cls;
};

// Looks an operation up by name; throws "IR Operation not defined: <name>" for unknown names
// (same failure as Compiler/Operations.cpp:206-217).
const OpInfo& FindOperation(const std::string& name);

struct Node {
	const OpInfo* op = nullptr;
	TFType type = TFType_None;
	std::vector<Node*> inputs;  // ArgType::Input, in order
	Node* index = nullptr;      // ArgType::Index: flat word address of a memory op (nullptr = 0)
	Node* memory = nullptr;     // ArgType::Memory: buffer / array of a memory op, or the target of `set`
	uint32_t data = 0;          // constant bits, block_thread_id dimension, array length
	std::string debug_name;
	std::string var_name;       // assigned by the generator
	bool modified = false;      // target of a `set`: never inlined into its users
	bool local_memory_op = false;  // memory op on a local_memory / group_memory array
	int use_count = 0;          // number of argument slots that reference this node
	std::vector<Node*> children;  // body of loop / if / kernel / host
	Node* parent = nullptr;
	// Host-side nodes only (the part of the tree outside kernels, Compiler/Operations.cpp:25-48):
	std::vector<Node*> shape;      // ArgType::Shape of memory / reshape / assert / kernel nodes, INNERMOST FIRST
	int input_index = -1;          // memory: NodeProp::InputMemory; input_shape: NodeProp::InputShapeMemory
	int input_dim = -1;            // input_shape: NodeProp::InputShapeDim
	int dispatch = -1;             // host `kernel` node: index into Program::dispatches

	const std::string& name() const;
};

// One kernel argument that is a scalar of the host program (shape values, host-side constants ...).
struct KernelVariable {
	Node* node;
	std::string name;
	TFType type;
};

// DimExpr, IdiomMatchInfo (a whole kernel recognised as one of the lowered algorithm loops,
// Compiler/Implementations.cpp:243-359,560-646), SortRole, HipKernelInfo: what the kernel manager reads at dispatch.
}  // namespace tfhost
#include "shim/hip_kernel_info.h"
namespace tfhost {
using tfhip::DimExpr;
using tfhip::HipKernelInfo;
using tfhip::IdiomMatchInfo;
using tfhip::kSortGroup;
using tfhip::kSortScanChunk;
using tfhip::SortRole;

struct IdiomMatch : IdiomMatchInfo {
	TFType type = TFType_Float;
	// Matmul with op "tail": the accumulator and the loop, so that the kernel without its loop can be built.
	const Node* accumulator = nullptr;
	const Node* loop = nullptr;
};

// Mirrors Compiler/KernelGen.h:17-46.
struct Kernel {
	Node* root = nullptr;
	std::vector<KernelVariable> variables;       // binding order
	std::vector<Node*> read_write_memory;        // binding order
	std::vector<Node*> read_only_memory;         // bound after the read-write ones
	std::vector<Node*> group_memory;
	std::vector<int> group_size;                 // innermost first: Node::group_size of the kernel node
	int dim = 1;                                 // dimensionality of the kernel shape: the number of its Shape arguments
	// Not members of the reference's Kernel but found in its tree (DeriveKernelGeometry; KernelBuilder records them as
	// it builds): thread-index nodes (index_0 .. index_{dim-1}) and the extents they are guarded against, innermost
	// first: inside `if (is_inside_dispatch)` the emitter may rely on 0 <= index_k < shape_k, shape_k >= 1.
	std::vector<Node*> index_nodes;
	std::vector<Node*> shape_nodes;
	Node* dispatch_guard = nullptr;              // the `if (is_inside_dispatch)` node

	size_t kernel_id_ = 0;
	std::string kernel_name_;
	std::string full_generated_code_;
	std::string generated_header_;
	std::string generated_bindings_;
	std::string generated_main_;
	std::vector<std::string> var_names;
	std::vector<std::string> var_types;

	// What the emitter decided (read by the kernel manager at dispatch time).
	int hip_threads = 0;           // threads of one HIP group
	int groups_per_hip_block = 1;  // IR thread-groups covered by one tile
	int hip_blocks_per_tile = 1;   // HIP groups that share one tile (row slabs of the four-wide mapping)
	int lanes_per_thread = 64;     // "reduction:wave": lanes that share one logical thread (64, 32, 16 or 8)
	int threads_per_lane_group = 1;  // "reduction:wave": logical threads a group of lanes works through, one after the other
	bool serial_load_loops = false;  // "flat" / "flat:vec4": a thread walks a loop of global loads by itself
	// "reduction:block" with one loop down the columns: several HIP groups may share a group of 64 threads, one slab of
	// the loop each (two more pointer parameters behind the tensors, one more variable word `_slabs`); the loop's trip
	// count for a dispatch, and the words a thread leaves per slab.
	bool slabs = false;
	DimExpr slab_trips;
	int slab_words_per_thread = 0;
	// "flat" / "flat:vec4": entry point that runs several small dispatches in one launch (empty if there is none), how many
	// dispatches its argument array holds and the bytes of one element (pointers, variable words, HIP group count).
	std::string batch_entry;
	int batch_capacity = 0, batch_call_bytes = 0;
	std::string idiom;             // "flat", "flat:vec4", "group", "reduction:wave"
	// Second, one-logical-thread-at-a-time entry point of a four-wide kernel (empty if there is none).
	std::string primitive;         // non-empty: dispatched to this libtfhip primitive, nothing is emitted
	size_t primitive_tensors = 0, primitive_variables = 0;
	IdiomMatch match;              // whole-kernel idiom the dispatcher may serve with a primitive instead
	tfhip::SortFeatures sort;      // what the kernel does, in the terms a `Radix sort` region is followed by (sort_features.cpp)
	// A matmul loop followed by an element-wise tail that is none of the fixed fused forms: the same kernel
	// without the loop, reading the product from one more read-only buffer (bound last). The dispatcher runs the
	// matmul primitive into a temporary and then this kernel.
	Kernel* tail_kernel = nullptr;
	// Accumulation loops whose loads are shared by the lanes along the innermost thread index (not by all threads):
	// split among the lanes of a wave they fill the chip from few threads; walked thread by thread they cost less
	// once there are enough threads. Both forms are emitted, this kernel cooperative, `dense_variant` (a copy with
	// `serial_loops` set) thread-serial, and the dispatch picks by the number of threads.
	Kernel* dense_variant = nullptr;
	bool serial_loops = false;
	// Every operation is printed as the tree holds it: no clamp or remainder is dropped or simplified because the
	// ranges of the thread indices make it the identity. For comparing emitted text with text the reference printed.
	bool verbatim = false;
	bool wants_dense_variant = false;  // set by the emitter on the cooperative form
	std::string scalar_entry;
	int scalar_hip_threads = 0;
	int scalar_groups_per_hip_block = 1;

	std::vector<Node*> MemoryBindings() const {
		std::vector<Node*> all(read_write_memory);
		all.insert(all.end(), read_only_memory.begin(), read_only_memory.end());
		return all;
	}
};

struct HostCode;  // host_program.h

// What a host `kernel` node dispatches: the kernel and, in binding order, the host tensors and host scalars it
// receives (the per-kernel maps of Compiler/KernelGen.h:17-46 seen from the host side; the dispatch shape is the
// node's Shape arguments).
struct DispatchBinding {
	Kernel* kernel = nullptr;
	std::vector<Node*> read_write, read_only, variables;
	std::vector<int> group;  // sizes the group count is computed with, innermost first
};

class Program {
 public:
	std::string program_name = "TensorProgram";
	std::vector<std::unique_ptr<Kernel>> kernels_;
	std::function<tf_main_func> execute_callback;
	int input_count = 0;
	int output_count = 0;
	float shader_compile_time = 0.0f;

	// All nodes are owned here.
	std::vector<std::unique_ptr<Node>> nodes;

	// The host part of the program's tree (what Program::ir_->root holds outside the kernel nodes,
	// Compiler/KernelGen.h:48-71): input checks, allocations, host scalars, dispatches, regions, host loops.
	// Built by HostBuilder; HostBuilder::Finish turns it into `host_code` and points execute_callback at
	// the interpreter, which stands where the reference's JIT-compiled `main` stands.
	Node* host_root = nullptr;
	std::vector<Node*> input_nodes;   // input_memory_map
	std::vector<Node*> output_nodes;  // output_memory_map
	std::vector<DispatchBinding> dispatches;
	std::shared_ptr<HostCode> host_code;
	// Seconds spent by tf.compile on this program: building the IR, emitting kernels + host code, compiling kernels.
	float trace_time = 0.0f, codegen_time = 0.0f;

	// Adds a kernel that is not emitted but served by a hand-written primitive of libtfhip (what the idiom
	// matcher substitutes for a recognised reduction / scan / matmul / sort subtree). `name` is one of
	// sgemm_nn|sgemm_nt|sgemm_tn {C | A, B} (M, N, K); with a fused tail, sgemm_<layout>_bias|_bias_relu {C | A, B, bias[N]}
	// and sgemm_<layout>_mask_positive {C | A, B, mask[M,N]}; reduce_rows_<op>|reduce_cols_<op> {out | x} (rows, cols);
	// softmax_rows {y | x} (rows, cols); scan_u32|scan_i32|scan_f32 {out | x} (n);
	// radix_sort_kv_u32|_i32|_f32 {keys_out, vals_out, keys_tmp, vals_tmp | keys_in, vals_in} (n).
	Kernel* AddPrimitive(const std::string& name, size_t n_tensors, size_t n_variables);
};

// A deep copy of the kernel's IR as a new kernel of `program` (nothing generated yet); mapping: original node -> copy.
Kernel* CloneKernel(Program* program, const Kernel* kernel, std::unordered_map<const Node*, Node*>* mapping = nullptr);

// Builds, as a new kernel of `program`, a copy of `kernel` in which the matmul loop is gone and the accumulator is
// a load of product[index_1 * shape_0 + index_0] from an extra read-only buffer bound after all others.
Kernel* MakeMatmulTailKernel(Program* program, const Kernel* kernel, const Node* accumulator, const Node* loop);

// Finds the thread indices, the extents they are guarded against and the `if (is_inside_dispatch)` node by walking
// the kernel's tree (they are ordinary nodes that Compiler/Steps/GraphOps.cpp:1091-1186 puts first among the kernel's
// children; TensorFrost's Kernel, Compiler/KernelGen.h:17-46, does not name them), and fills `index_nodes`,
// `shape_nodes`, `dispatch_guard`, `dim` (when it is 0) and `group_size` (when it is empty). A `dim` or `group_size`
// already set, as read from the kernel node's Shape arguments and Node::group_size, must agree with the tree.
void DeriveKernelGeometry(Kernel* kernel);

// ---- building kernels in the post-lowering form ---------------------------------------------------

class NodeBuilder;

// Value handle with operators, so kernels and host programs read like the reference's Python frontend.
struct V {
	Node* n = nullptr;
	NodeBuilder* b = nullptr;
	V() = default;
	V(Node* n, NodeBuilder* b) : n(n), b(b) {}
	TFType type() const { return n->type; }
};

// What building a scope of the tree needs, whether the scope lies in a kernel or in the host program:
// constants, operations of the table, `set`, loops and conditionals.
class NodeBuilder {
 public:
	// Constants.
	V Const(float v);
	V Const(int v);
	V ConstU(uint32_t v);
	V ConstB(bool v);

	// Generic operation by table name.
	V Op(const std::string& name, std::vector<V> inputs, TFType type);
	V Named(V v, const std::string& debug_name);

	void Set(V target, V value);  // marks target Modified
	void Keyword(const std::string& name);  // break / continue / discard

	// Scopes.
	void Loop(V begin, V end, V step, const std::function<void(V)>& body);
	void If(V cond, const std::function<void()>& body);

	// A constant flagged Modified: the target of later `set`s. In kernels this is how the reference's lowered
	// idioms start (Implementations.cpp: an accumulator named "sum" | "max" | "min" | "prod" | "prefix_sum" |
	// "matmul", then a loop); on the host it is a scalar the program updates (`x.val = ...`).
	V Accumulator(const std::string& idiom_name, TFType type, uint32_t init_bits);

	V Clamp(V x, V lo, V hi);

	Program* program() { return program_; }

 protected:
	explicit NodeBuilder(Program* program) : program_(program) {}
	Node* NewNode(const std::string& op, TFType type);
	void Append(Node* n);
	void Use(Node* user, V v);

	Program* program_;
	std::vector<Node*> scope_stack_;
};

class KernelBuilder : public NodeBuilder {
 public:
	// shape_dim: dimensionality of the dispatch; group: innermost-first group sizes ({} = the defaults
	// 256 / 16x16 / 8x8x8 of GraphOps.cpp:1143-1166).
	KernelBuilder(Program* program, int shape_dim, std::vector<int> group = {});

	// Kernel arguments.
	V Buffer(const std::string& name, bool read_only);  // a `memory` node bound to the kernel
	V Var(const std::string& name, TFType type);         // a host scalar passed in the variable block
	V GroupMemory(const std::string& name, TFType type, int size);
	V LocalMemory(const std::string& name, TFType type, int size);

	// Thread indices exactly as LinearBlockModeIndices / ComputeIndicesFromBlockIndex leave them:
	// emits block_id, block_thread_id<k>, blocks_shape_<k>, index_<k> and opens
	// `if (is_inside_dispatch)`. shape[k] is the extent of kernel dimension k, INNERMOST FIRST.
	// Returns index_0 .. index_{dim-1}. Everything built afterwards goes inside the `if`.
	std::vector<V> ThreadIndices(const std::vector<V>& shape_innermost_first);
	// The same guard around index arithmetic that the caller has built node by node (another version of the
	// reference computes it in another order): opens `if (inside)` as the dispatch guard and records that inside
	// it 0 <= indices[k] < shape[k], index k being the one that moves with block_thread_id<k>.
	void OpenDispatchGuard(V inside, const std::vector<V>& indices_innermost_first, const std::vector<V>& shape_innermost_first);
	V BlockId();
	V BlockThreadId(int k);

	// Memory operations on flat word addresses.
	V Load(V memory, V address, TFType type);
	void Store(V memory, V address, V value);
	V Atomic(const std::string& op, V memory, V address, V value, bool returns_previous = false);
	void Barrier();

	// C-order flat index from indices / extents given OUTERMOST FIRST (Tensor::FlatIndex).
	V FlatIndex(const std::vector<V>& indices, const std::vector<V>& shape);

	// Finishes the kernel and appends it to the program.
	Kernel* Finish();

 private:
	std::unique_ptr<Kernel> kernel_;
};

// One extent of a host tensor: a host scalar, a constant, or (inputs only) "whatever the caller passes" (-1),
// which becomes an input_shape node as `tf.input([-1, ...])` does.
struct Dim {
	V v;
	long constant = -1;
	Dim(V v) : v(v) {}
	Dim(int c) : constant(c) {}
	Dim(long c) : constant(c) {}
	Dim(size_t c) : constant((long)c) {}
};

// Builds the host part of a program's tree in the shape the reference's passes leave it (what GenerateMain,
// Backend/CodeGen/Langs/CPP.cpp:678-718, walks): per input the input_shape nodes of its unknown extents and the
// input `memory` node (emitted as tf.check_tensor), `memory` nodes that allocate, `deallocate`, host scalar
// arithmetic on shape values, `kernel` nodes (tf.dispatch), `region_begin/end`, host `load`/`store` (tf.read /
// tf.write), `reshape` / `assert`, host `loop` / `if`. Python-level loops of a traced function are unrolled by
// tracing, so a builder function unrolls them the same way with C++ loops around these calls.
// Shapes are given OUTERMOST FIRST, as in Python.
class HostBuilder : public NodeBuilder {
 public:
	explicit HostBuilder(Program* program);

	// tf.input(shape, type): the next input of the program.
	V Input(const std::string& name, const std::vector<Dim>& shape, TFType type);
	// The extents of a host tensor as host scalars (Int), outermost first.
	std::vector<V> Shape(V tensor);

	V Allocate(const std::string& name, const std::vector<Dim>& shape, TFType type);
	void Deallocate(V tensor);
	V Reshape(V tensor, const std::string& name, const std::vector<Dim>& shape, TFType type);
	V AssertTensor(V tensor, const std::string& name, const std::vector<Dim>& shape, TFType type);

	// tf.read / tf.write: one word of a tensor, read back by the host / written from it.
	V Read(V tensor, V index, TFType type);
	void Write(V tensor, V index, V value);

	// tf.dispatch of a kernel on host tensors (read-write ones first, then read-only, in the kernel's binding
	// order), host scalars for its variable block, and the dispatch shape. The group sizes the group count is
	// computed with are the kernel's own; a primitive-backed kernel has none and takes `group`, or the defaults.
	void Dispatch(Kernel* kernel, const std::vector<V>& read_write, const std::vector<V>& read_only, const std::vector<V>& variables,
	              const std::vector<Dim>& shape, std::vector<int> group = {});

	void RegionBegin(const std::string& name);
	void RegionEnd(const std::string& name);
	void AssertValue(const std::string& name, V condition);
	void PrintValue(const std::string& name, V value);

	// The next output of the program.
	void Output(V tensor);

	// Emits the host code (host_program.h) and makes it the program's execute_callback.
	void Finish();

 private:
	V DimValue(const Dim& d);
	void SetShape(Node* n, const std::vector<Dim>& shape);
	Node* TensorNode(const std::string& op, V source, const std::string& name, const std::vector<Dim>& shape, TFType type);
};

// Operators on V (typed like the op table: arithmetic keeps the operand type, comparisons give Bool).
V operator+(V a, V b);
V operator-(V a, V b);
V operator*(V a, V b);
V operator/(V a, V b);
V operator%(V a, V b);
V operator<<(V a, V b);
V operator>>(V a, V b);
V operator&(V a, V b);
V operator|(V a, V b);
V operator^(V a, V b);
V operator&&(V a, V b);
V operator||(V a, V b);
V operator<(V a, V b);
V operator<=(V a, V b);
V operator>(V a, V b);
V operator>=(V a, V b);
V operator==(V a, V b);
V operator!=(V a, V b);
V operator-(V a);
V operator!(V a);
V operator~(V a);
V Select(V cond, V a, V b);  // ternary
V ToFloat(V a);
V ToInt(V a);
V ToUint(V a);
V AsFloat(V a);
V AsUint(V a);
V AsInt(V a);
V Fn(const std::string& name, V a);            // unary function of the table (sin, exp, sqrt, abs, ...)
V Fn(const std::string& name, V a, V b);       // min, max, pow, atan2, modf, step
V Fn(const std::string& name, V a, V b, V c);  // clamp, lerp, fma

inline uint32_t FloatBits(float f) {
	uint32_t u;
	std::memcpy(&u, &f, 4);
	return u;
}

}  // namespace tfhost
