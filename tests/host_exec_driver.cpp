// CPU-only driver for the host interpreter: runs host programs against a TFRuntime whose six callbacks only keep
// a log (tensors are small host arrays), and evaluates single scalar operations. tests/test_host_exec.py reads what
// it prints. Linked against libtfhost.so; nothing here touches a GPU.
//
//   driver scalar            lines "op operand_type result_type a b c" (types f|i|u|b, words in hex) on stdin,
//                            one hex result (or "none") per line on stdout
//   driver run <scenario>    prints the callback log of one scenario
#include <cstdio>
#include <cstring>
#include <iostream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "host_program.h"
#include "programs/registry.h"
#include "tf_backend.h"

using namespace tfhost;

namespace {

struct MockBuffer : TFBuffer {
	std::string label;
	std::vector<uint32_t> words;
};

std::vector<std::string> g_log;

const char* TypeName(TFType t) { return t == TFType_Float ? "Float" : t == TFType_Uint ? "Uint" : t == TFType_Int ? "Int" : t == TFType_Bool ? "Bool" : "None"; }

std::string ShapeText(const size_t* shape, size_t dim) {
	std::string s = "[";
	for (size_t i = 0; i < dim; i++) s += (i ? "," : "") + std::to_string(shape[i]);
	return s + "]";
}

TFTensor MakeTensor(const std::string& name, const std::vector<size_t>& shape, TFType type) {
	size_t n = 1;
	for (size_t e : shape) n *= e;
	MockBuffer* b = new MockBuffer();
	b->size = n;
	b->used_size = n;
	b->time_since_used = 0;
	b->up_to_date = true;
	b->read_only = false;
	b->name = nullptr;
	b->label = name;
	b->words.assign(n, 0);
	size_t* kept = new size_t[shape.size() ? shape.size() : 1];
	for (size_t i = 0; i < shape.size(); i++) kept[i] = shape[i];
	return TFTensor{b, TFDataFormat{type, 32}, shape.size(), kept};
}

const std::string& Label(const TFTensor& t) { return static_cast<MockBuffer*>(t.buffer)->label; }

TFTensor Alloc(const char* name, const size_t* shape, size_t dim, TFDataFormat format, void*) {
	g_log.push_back(std::string("alloc ") + name + " " + ShapeText(shape, dim) + " " + TypeName(format.type));
	return MakeTensor(name, std::vector<size_t>(shape, shape + dim), format.type);
}
void Dealloc(TFTensor t, void*) { g_log.push_back("dealloc " + Label(t)); }
uint32_t Readback(TFTensor t, size_t index, void*) {
	g_log.push_back("read " + Label(t) + " " + std::to_string(index));
	return static_cast<MockBuffer*>(t.buffer)->words.at(index);
}
void Writeback(TFTensor t, size_t index, uint32_t value, void*) {
	g_log.push_back("write " + Label(t) + " " + std::to_string(index) + " " + std::to_string(value));
	static_cast<MockBuffer*>(t.buffer)->words.at(index) = value;
}
std::map<size_t, int> g_kernel_ordinal;  // kernel id -> position in the program
void Dispatch(TFDispatchInfo info, void*) {
	std::ostringstream o;
	o << "dispatch k" << g_kernel_ordinal.at(info.kernel_id) << " tensors";
	for (size_t i = 0; i < info.read_write_count; i++) o << " " << Label(info.read_write_tensors[i]) << (info.read_write_tensors[i].buffer->up_to_date ? "" : "*");
	o << " ro=" << info.read_only_count << " vars";
	for (size_t i = 0; i < info.variable_count; i++) o << " " << info.variables[i];
	o << " groups " << info.work_group_count;
	g_log.push_back(o.str());
	// so that the mark shows what THIS dispatch declared as written
	for (size_t i = 0; i < info.read_write_count; i++) info.read_write_tensors[i].buffer->up_to_date = true;
}
void Region(const char* name, bool begin, void*) { g_log.push_back(std::string(begin ? "begin " : "end ") + name); }

TFRuntime MockRuntime() { return TFRuntime{Alloc, Dealloc, Readback, Writeback, Dispatch, Region, nullptr}; }

void RunAndPrint(Program* program, std::vector<TFTensor> inputs) {
	g_kernel_ordinal.clear();
	for (size_t i = 0; i < program->kernels_.size(); i++) g_kernel_ordinal[program->kernels_[i]->kernel_id_] = (int)i;
	std::vector<TFTensor> out((size_t)program->output_count);
	g_log.clear();
	try {
		program->execute_callback(inputs.data(), out.data(), MockRuntime());
		for (const std::string& l : g_log) printf("%s\n", l.c_str());
		for (size_t i = 0; i < out.size(); i++) printf("out %zu %s %s %s\n", i, Label(out[i]).c_str(), ShapeText(out[i].shape, out[i].dim).c_str(), TypeName(out[i].format.type));
	} catch (const std::exception& e) {
		for (const std::string& l : g_log) printf("%s\n", l.c_str());
		printf("error %s\n", e.what());
	}
}

float AsFloat(uint32_t w) {
	float f;
	memcpy(&f, &w, 4);
	return f;
}

// A host program that uses what the benchmark programs do not: a host loop with break and continue, a host `if`,
// a scalar updated by `set`, tf.read / tf.write, reshape, assert_tensor, assert_value, float host arithmetic.
void BuildHostControlFlow(Program* program, const std::vector<int64_t>&) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("out", false);
	V n = kb.Var("n", TFType_Int), scale = kb.Var("scale", TFType_Float);
	V i = kb.ThreadIndices({n})[0];
	kb.Store(out, i, ToFloat(i) * scale);
	Kernel* kernel = kb.Finish();

	HostBuilder h(program);
	V counts = h.Input("counts", {-1}, TFType_Int);
	V len = h.Shape(counts)[0];
	V limit = h.Read(counts, h.Const(0), TFType_Int);  // counts[0]: how many loop trips at most
	V total = h.Accumulator("total", TFType_Int, 0u);
	h.Loop(h.Const(1), len, h.Const(1), [&](V k) {
		h.If(k > limit, [&] { h.Keyword("break"); });
		V c = h.Read(counts, k, TFType_Int);
		h.If(c < h.Const(0), [&] { h.Keyword("continue"); });
		h.Set(total, total + c);
		V t = h.Allocate("step", {c}, TFType_Float);
		h.Dispatch(kernel, {t}, {}, {c, ToFloat(k) * h.Const(0.5f)}, {c});
		h.Deallocate(t);
	});
	h.AssertValue("total is positive", total > h.Const(0));
	h.Write(counts, h.Const(0), AsUint(total));
	V grid = h.Allocate("grid", {total, 2}, TFType_Float);
	V flat = h.Reshape(grid, "flat", {total * h.Const(2)}, TFType_Float);
	V checked = h.AssertTensor(flat, "flat", {total + total}, TFType_Float);
	h.Dispatch(kernel, {checked}, {}, {total * h.Const(2), h.Const(1.0f) / ToFloat(total)}, {total * h.Const(2)});
	h.Output(grid);
	h.Output(checked);
	h.Finish();
}
ProgramRegistrar reg_control("host_control_flow", BuildHostControlFlow);

int RunScenario(const std::string& scenario) {
	InitializeBackend(BackendType::CodeGen, "");
	auto make = [](const char* name, std::vector<int64_t> params = {}) { return CreateProgram(name, params); };
	if (scenario == "wave_eq" || scenario == "wave_eq_bad_shape" || scenario == "wave_eq_bad_type" || scenario == "wave_eq_bad_dims") {
		Program* p = make("wave_eq");
		TFTensor u = MakeTensor("u", scenario == "wave_eq_bad_dims" ? std::vector<size_t>{100} : std::vector<size_t>{100, 37}, TFType_Float);
		TFTensor v = MakeTensor("v", scenario == "wave_eq_bad_shape" ? std::vector<size_t>{100, 38} : std::vector<size_t>{100, 37}, scenario == "wave_eq_bad_type" ? TFType_Int : TFType_Float);
		RunAndPrint(p, {u, v});
	} else if (scenario == "nbody") {
		Program* p = make("nbody");
		TFTensor dt = MakeTensor("dt", {1}, TFType_Float), eps = MakeTensor("eps", {1}, TFType_Float);
		const float dt_value = 0.25f, eps_value = 3.0f;
		memcpy(&static_cast<MockBuffer*>(dt.buffer)->words[0], &dt_value, 4);
		memcpy(&static_cast<MockBuffer*>(eps.buffer)->words[0], &eps_value, 4);
		RunAndPrint(p, {MakeTensor("X", {1000, 3}, TFType_Float), MakeTensor("V", {1000, 3}, TFType_Float), MakeTensor("M", {1000}, TFType_Float), dt, eps});
	} else if (scenario == "broadcast_loops") {
		Program* p = make("broadcast_loops");
		TFTensor first = MakeTensor("first", {1}, TFType_Int);
		static_cast<MockBuffer*>(first.buffer)->words[0] = 7;
		RunAndPrint(p, {MakeTensor("x", {500}, TFType_Float), MakeTensor("a", {500}, TFType_Int), MakeTensor("table", {40}, TFType_Float), MakeTensor("itable", {40}, TFType_Int), first});
	} else if (scenario == "radix_sort_ir") {
		Program* p = make("radix_sort_ir");
		RunAndPrint(p, {MakeTensor("keys", {1000}, TFType_Uint), MakeTensor("values", {1000}, TFType_Uint)});
	} else if (scenario == "indexing4") {
		Program* p = make("indexing", {4});
		RunAndPrint(p, {MakeTensor("data", {3, 9, 10, 17}, TFType_Float)});
	} else if (scenario == "tiled_bad") {
		Program* p = make("tiled_matmul_ir");
		RunAndPrint(p, {MakeTensor("A", {128, 64}, TFType_Float), MakeTensor("B", {64, 100}, TFType_Float)});
	} else if (scenario == "control" || scenario == "control_assert") {
		Program* p = make("host_control_flow");
		const char* listing_marker = "listing\n";
		TFTensor counts = MakeTensor("counts", {6}, TFType_Int);
		std::vector<int32_t> values = scenario == "control" ? std::vector<int32_t>{3, 5, -2, 300, 7, 9} : std::vector<int32_t>{2, -1, -1, 4, 4, 4};
		for (size_t i = 0; i < values.size(); i++) static_cast<MockBuffer*>(counts.buffer)->words[i] = (uint32_t)values[i];
		RunAndPrint(p, {counts});
		printf("%s%s", listing_marker, PrintHostCode(*p->host_code).c_str());
	} else if (scenario == "listing") {
		Program* p = make("wave_eq");
		printf("%s", PrintHostCode(*p->host_code).c_str());
	} else {
		fprintf(stderr, "unknown scenario %s\n", scenario.c_str());
		return 2;
	}
	(void)AsFloat;
	return 0;
}

TFType TypeOf(const std::string& letter) { return letter == "f" ? TFType_Float : letter == "i" ? TFType_Int : letter == "u" ? TFType_Uint : letter == "b" ? TFType_Bool : TFType_None; }

int RunScalar() {
	std::string op, operand, result;
	uint32_t a, b, c;
	while (std::cin >> op >> operand >> result >> std::hex >> a >> b >> c) {
		ScalarFn fn = FindScalarFn(op, TypeOf(operand), TypeOf(result));
		if (!fn) {
			printf("none\n");
			continue;
		}
		try {
			printf("%08x\n", fn(a, b, c));
		} catch (const std::exception& e) {
			printf("error %s\n", e.what());
		}
	}
	return 0;
}

}  // namespace

int main(int argc, char** argv) {
	try {
		if (argc >= 2 && std::string(argv[1]) == "scalar") return RunScalar();
		if (argc >= 3 && std::string(argv[1]) == "run") return RunScenario(argv[2]);
	} catch (const std::exception& e) {
		printf("fatal %s\n", e.what());
		return 1;
	}
	fprintf(stderr, "usage: driver scalar | driver run <scenario>\n");
	return 2;
}
