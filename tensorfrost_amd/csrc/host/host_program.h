// The host program of a TensorFrost program, run from its IR.
//
// The reference turns the host part of a program's tree into C++ text (GenerateMain,
// TensorFrost/Backend/CodeGen/Langs/CPP.cpp:678-718, statement forms Backend/CodeGen/Generators.cpp:333-385,
// 441-462), appends a textual copy of its TFContext class (CPP.cpp:364-551), writes both to a temporary file and
// runs the system C++ compiler on it (Backend/Backends/CPU/KernelCompiler.cpp:94-220; about 1.5 s per tf.compile)
// to obtain the `main(TFTensor* in, TFTensor* out, TFRuntime)` it calls for every program(*inputs).
//
// Here the same tree is lowered once, at tf.compile time, into a flat list of instructions over numbered value
// slots (32-bit words for host scalars, TFTensor headers for tensors), and `RunHostCode` walks that list. It
// reaches the backend only through the six TFRuntime callbacks, exactly as the compiled `main` does, so it is a
// drop-in for it: Program::execute_callback is bound to it by HostBuilder::Finish. Lowering takes microseconds,
// needs no compiler on the machine and leaves nothing in /tmp; a step costs a few tens of nanoseconds per host
// node, and a dispatch fills tensor / variable arrays sized when the code was lowered instead of heap temporaries.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "tf_abi.h"
#include "tf_ir.h"

namespace tfhost {

// Evaluates one scalar operation of the op table on 32-bit words, with the semantics the generated C++ has
// (operators of the operand type; the helper functions of the generated prelude, CPP.cpp:31-271).
using ScalarFn = uint32_t (*)(uint32_t a, uint32_t b, uint32_t c);
// The evaluator of `op` on operands of type `operand` (the type of the first input; casts: the source type)
// producing `result`; nullptr if the host cannot evaluate it.
ScalarFn FindScalarFn(const std::string& op, TFType operand, TFType result);

struct HostInstr {
	enum Code : uint8_t {
		Const,         // s[dst] = imm
		Scalar,        // s[dst] = fn(s[a], s[b], s[c])
		Copy,          // s[dst] = s[a]                                       (`set`, copy)
		InputShape,    // s[dst] = in[input].shape[dim]; checks in[input].dim == expected
		CheckInput,    // t[dst] = in[input]; tf.check_tensor(t[dst], name, shape, type)
		Allocate,      // t[dst] = tf.allocate(name, shape, type)
		Deallocate,    // tf.deallocate(t[a])
		Reshape,       // t[dst] = tf.reshape(t[a], name, shape, type)
		AssertTensor,  // t[dst] = tf.assert_tensor(t[a], name, shape, type)
		Read,          // s[dst] = tf.read(t[a], s[b])
		Write,         // tf.write(t[a], s[b], s[c])
		Dispatch,      // tf.dispatch(kernel, tensors, variables, shape, group)
		RegionBegin,
		RegionEnd,
		AssertValue,   // tf.assert_value(name, s[a])
		PrintValue,    // tf.print_value(name, s[a])
		LoopEnter,     // s[dst] = s[a]; if the range is empty jump
		LoopNext,      // s[dst] += s[c]; if still inside jump back to the body
		JumpIfNot,     // if (!s[a]) jump
		Jump,
		Output,        // out[imm] = t[a]
	} code;
	TFType type = TFType_None;     // result type (Allocate / Reshape / CheckInput: element type)
	int dst = -1, a = -1, b = -1, c = -1;
	uint32_t imm = 0;
	int jump = -1;
	ScalarFn fn = nullptr;
	int input = -1, dim = -1, expected_dims = -1;
	std::string name;
	std::vector<int> shape;        // scalar slots, OUTERMOST FIRST
	std::vector<int> tensors;      // Dispatch: tensor slots, read-write first
	size_t read_write = 0;         // Dispatch: how many of `tensors` are written
	std::vector<int> variables;    // Dispatch: scalar slots
	std::vector<int> group;        // Dispatch: group sizes, innermost first
	const Kernel* kernel = nullptr;
};

struct HostCode {
	std::vector<HostInstr> instrs;
	int scalar_slots = 0, tensor_slots = 0;
	size_t max_tensors = 0, max_variables = 0, max_dims = 0;
	int inputs = 0, outputs = 0;
	std::string program_name;
};

// Lowers program->host_root (inputs / outputs as recorded by HostBuilder). Throws on a tree the host cannot run
// (an operation with no scalar evaluator, a value used outside the scope that defines it).
std::shared_ptr<HostCode> LowerHostProgram(const Program* program);

// One execution: the role of the generated `main` (CPP.cpp:623-650). Errors are C++ exceptions with the
// messages of the reference's TFContext (CPP.cpp:390-551).
int RunHostCode(const HostCode& code, TFTensor* in, TFTensor* out, TFRuntime runtime);

// The host code as text, one instruction per line in the shape of the reference's generated C++ (for inspection
// and tests).
std::string PrintHostCode(const HostCode& code);

}  // namespace tfhost
