// Kernel text printed by the reference -> the kernel's tree -> the HIP emitter's text.
//
// The reference keeps, in a few notebooks, kernels as its own generator printed them after all passes (the GLSL
// dialect of Backend/CodeGen/Langs/GLSL.cpp; statement forms Backend/CodeGen/Generators.cpp:319-540). Every line of
// such a body is one node of the kernel's tree: `T name = expression;` a named value, `name = expression;` a `set`,
// `X_mem[address] = asuint(value);` a store, `for (int v = a; v < b; v += s)` a loop, `if (c)`, `break;`, `continue;`,
// `barrier();`, atomics; whatever is nested inside an expression is an unnamed node that the generator inlined. This
// file parses that text back into nodes (with KernelBuilder, i.e. into the form the emitter consumes from any
// program) and lets the HIP emitter print the kernel. A test then requires the emitted statements to equal the printed
// ones, statement for statement; if the tree lacked an operation or a statement form of the reference, or the emitter
// inlined, named or parenthesised differently, that comparison fails.
//
//   tftest_emit_kernel_text(body, group sizes, shared declarations) -> emitted HIP source of the kernel
#include <cctype>
#include <cstring>
#include <map>
#include <set>
#include <sstream>

#include "registry.h"
#include "hip_generator.h"

namespace tfhost {

namespace {

struct Token {
	enum Kind { Ident, Number, Punct, End } kind = End;
	std::string text;
};

std::vector<Token> Tokenize(const std::string& s) {
	std::vector<Token> out;
	size_t i = 0;
	static const char* three[] = {"<<=", ">>="};
	static const char* two[] = {"<<", ">>", "<=", ">=", "==", "!=", "&&", "||", "+=", "-="};
	while (i < s.size()) {
		const char c = s[i];
		if (std::isspace((unsigned char)c)) {
			i++;
			continue;
		}
		if (std::isalpha((unsigned char)c) || c == '_') {
			size_t j = i;
			while (j < s.size() && (std::isalnum((unsigned char)s[j]) || s[j] == '_')) j++;
			out.push_back({Token::Ident, s.substr(i, j - i)});
			i = j;
			continue;
		}
		if (std::isdigit((unsigned char)c) || (c == '.' && i + 1 < s.size() && std::isdigit((unsigned char)s[i + 1]))) {
			size_t j = i;
			if (c == '0' && j + 1 < s.size() && (s[j + 1] == 'x' || s[j + 1] == 'X')) {
				j += 2;
				while (j < s.size() && std::isxdigit((unsigned char)s[j])) j++;
			} else {
				while (j < s.size() && (std::isdigit((unsigned char)s[j]) || s[j] == '.')) j++;
				if (j < s.size() && (s[j] == 'e' || s[j] == 'E')) {
					j++;
					if (j < s.size() && (s[j] == '+' || s[j] == '-')) j++;
					while (j < s.size() && std::isdigit((unsigned char)s[j])) j++;
				}
			}
			if (j < s.size() && (s[j] == 'f' || s[j] == 'u')) j++;
			out.push_back({Token::Number, s.substr(i, j - i)});
			i = j;
			continue;
		}
		bool matched = false;
		for (const char* t : three)
			if (s.compare(i, 3, t) == 0) {
				out.push_back({Token::Punct, t});
				i += 3;
				matched = true;
				break;
			}
		if (matched) continue;
		for (const char* t : two)
			if (s.compare(i, 2, t) == 0) {
				out.push_back({Token::Punct, t});
				i += 2;
				matched = true;
				break;
			}
		if (matched) continue;
		out.push_back({Token::Punct, std::string(1, c)});
		i++;
	}
	out.push_back({Token::End, ""});
	return out;
}

TFType TypeOf(const std::string& name) {
	if (name == "float") return TFType_Float;
	if (name == "int") return TFType_Int;
	if (name == "uint") return TFType_Uint;
	if (name == "bool") return TFType_Bool;
	return TFType_None;
}

// GLSL spelling -> operation of the table (the inverse of GLSL.cpp:9-17's name map)
const std::map<std::string, std::string>& FunctionOps() {
	static const std::map<std::string, std::string> m = {{"mod", "modf"}, {"mix", "lerp"}, {"bitfieldReverse", "reversebits"}, {"fract", "frac"}, {"inversesqrt", "rsqrt"}};
	return m;
}

const std::map<std::string, std::string>& AtomicOps() {
	static const std::map<std::string, std::string> m = {{"atomicAdd", "InterlockedAdd"}, {"atomicMin", "InterlockedMin"}, {"atomicMax", "InterlockedMax"},
	                                                     {"atomicAnd", "InterlockedAnd"}, {"atomicOr", "InterlockedOr"},   {"atomicXor", "InterlockedXor"}};
	return m;
}

class KernelTextParser {
 public:
	KernelTextParser(Program* program, const std::vector<std::string>& lines, std::vector<int> group, const std::vector<std::string>& shared)
	    : lines_(lines), shared_(shared) {
		// dimensionality: the conjuncts of is_inside_dispatch
		int dims = 1;
		for (const std::string& l : lines_)
			if (l.find("bool is_inside_dispatch") != std::string::npos) {
				dims = 1;
				for (size_t p = l.find("&&"); p != std::string::npos; p = l.find("&&", p + 2)) dims++;
			}
		while ((int)group.size() > dims) group.pop_back();
		kb_ = std::make_unique<KernelBuilder>(program, dims, group);
		// buffers: written (or used by an atomic) = read-write, bound first
		std::vector<std::string> order;
		std::set<std::string> written;
		for (const std::string& l : lines_) {
			std::vector<Token> t = Tokenize(StripComment(l));
			for (size_t i = 0; i < t.size(); i++) {
				if (t[i].kind != Token::Ident || !IsBufferName(t[i].text)) continue;
				const std::string name = t[i].text.substr(0, t[i].text.size() - 4);
				if (std::find(order.begin(), order.end(), name) == order.end()) order.push_back(name);
				if (i == 0 || (i >= 2 && t[i - 1].text == "(" && AtomicOps().count(t[i - 2].text))) written.insert(name);
			}
			if (!t.empty() && t[0].kind == Token::Ident && t[0].text.rfind("atomicAdd_", 0) == 0) written.insert(t[0].text.substr(10, t[0].text.size() - 14));
		}
		for (const std::string& n : order)
			if (written.count(n)) buffers_[n] = kb_->Buffer(n, false);
		for (const std::string& n : order)
			if (!written.count(n)) buffers_[n] = kb_->Buffer(n, true);
	}

	Kernel* Parse() {
		ParseBlock(false);
		if (line_ != lines_.size()) Fail("unbalanced braces");
		Kernel* k = kb_->Finish();
		k->serial_loops = true;  // every loop as the thread-serial statement it is in the text
		k->verbatim = true;
		return k;
	}

 private:
	std::vector<std::string> lines_, shared_;
	size_t line_ = 0;
	std::unique_ptr<KernelBuilder> kb_;
	std::map<std::string, V> values_, buffers_, variables_, arrays_;
	std::vector<Token> tok_;
	size_t pos_ = 0;

	static bool IsBufferName(const std::string& s) { return s.size() > 4 && s.compare(s.size() - 4, 4, "_mem") == 0; }

	static std::string StripComment(const std::string& l) {
		const size_t p = l.find("//");
		return p == std::string::npos ? l : l.substr(0, p);
	}

	[[noreturn]] void Fail(const std::string& what) const {
		throw std::runtime_error("kernel text, line " + std::to_string(line_ + 1) + " (" + (line_ < lines_.size() ? lines_[line_] : std::string("end")) + "): " + what);
	}

	const Token& Peek(size_t ahead = 0) const { return tok_[std::min(pos_ + ahead, tok_.size() - 1)]; }
	Token Next() { return tok_[std::min(pos_++, tok_.size() - 1)]; }
	bool Accept(const std::string& text) {
		if (Peek().kind != Token::End && Peek().text == text) {
			pos_++;
			return true;
		}
		return false;
	}
	void Expect(const std::string& text) {
		if (!Accept(text)) Fail("expected '" + text + "' before '" + Peek().text + "'");
	}

	// ---- statements ------------------------------------------------------------------------------------------
	void ParseBlock(bool braced) {
		while (line_ < lines_.size()) {
			std::string raw = lines_[line_];
			std::string trimmed = raw;
			trimmed.erase(0, trimmed.find_first_not_of(" \t"));
			if (trimmed == "}") {
				if (!braced) Fail("unexpected '}'");
				line_++;
				return;
			}
			if (trimmed.rfind("//", 0) == 0) {  // `//float name[size]`: where the tree holds the group array
				std::vector<Token> t = Tokenize(trimmed.substr(2));
				if (t.size() >= 5 && TypeOf(t[0].text) != TFType_None && t[2].text == "[") {
					const std::string decl = "shared " + t[0].text + " " + t[1].text + "[" + t[3].text + "];";
					const bool shared = std::find(shared_.begin(), shared_.end(), decl) != shared_.end();
					arrays_[t[1].text] = shared ? kb_->GroupMemory(t[1].text, TypeOf(t[0].text), std::stoi(t[3].text)) : kb_->LocalMemory(t[1].text, TypeOf(t[0].text), std::stoi(t[3].text));
				}
				line_++;
				continue;
			}
			tok_ = Tokenize(StripComment(raw));
			pos_ = 0;
			ParseStatement();
		}
		if (braced) Fail("missing '}'");
	}

	void OpenBody(const std::function<void()>& build) {
		line_++;
		std::string open = line_ < lines_.size() ? lines_[line_] : "";
		open.erase(0, open.find_first_not_of(" \t"));
		if (open != "{") Fail("expected '{'");
		line_++;
		build();
	}

	void ParseStatement() {
		const Token first = Peek();
		if (first.kind == Token::Ident && first.text == "for") {
			// for (int v = a; v < b; v += s)
			Next();
			Expect("(");
			Expect("int");
			const std::string var = Next().text;
			Expect("=");
			V begin = Expression();
			Expect(";");
			if (Next().text != var) Fail("loop test on another variable");
			Expect("<");
			V end = Expression();
			Expect(";");
			if (Next().text != var) Fail("loop step on another variable");
			Expect("+=");
			V step = Expression();
			Expect(")");
			OpenBody([&] {
				kb_->Loop(begin, end, step, [&](V v) {
					kb_->Named(v, var);
					values_[var] = v;
					ParseBlock(true);
				});
			});
			return;
		}
		if (first.kind == Token::Ident && first.text == "if") {
			Next();
			Expect("(");
			V cond = Expression();
			Expect(")");
			if (cond.n->debug_name == "is_inside_dispatch") {
				OpenBody([&] {
					OpenGuard(cond);
					ParseBlock(true);
				});
			} else {
				OpenBody([&] { kb_->If(cond, [&] { ParseBlock(true); }); });
			}
			return;
		}
		if (first.kind == Token::Ident && (first.text == "break" || first.text == "continue" || first.text == "discard")) {
			kb_->Keyword(first.text);
			line_++;
			return;
		}
		if (first.kind == Token::Ident && first.text == "barrier") {
			kb_->Barrier();
			line_++;
			return;
		}
		if (first.kind == Token::Ident && TypeOf(first.text) != TFType_None && Peek(1).kind == Token::Ident && Peek(2).text == "=") {
			// T name = expression;
			const TFType type = TypeOf(Next().text);
			const std::string name = Next().text;
			Expect("=");
			V v = Expression(type);
			Expect(";");
			if (!v.n->debug_name.empty() || v.n->op->cls == OpClass::Variable || v.n->op->cls == OpClass::DimensionIndex || v.n->op->name == std::string("variable"))
				v = kb_->Op("copy", {v}, v.type());  // `int tx = block_thread_id1;`: a copy node with a name of its own
			if (v.type() != type) Fail("declared " + std::string(first.text) + ", expression has another type");
			// v<operation>[_n] is the name the generator gives a node without one (RegenerateNodeName): the node stays
			// unnamed, and the emitter decides by its own count what to call it if it keeps a line of its own
			const std::string automatic = "v" + std::string(v.n->op->name);
			const bool unnamed = name == automatic || (name.rfind(automatic + "_", 0) == 0 && name.find_first_not_of("0123456789", automatic.size() + 1) == std::string::npos);
			if (!unnamed) kb_->Named(v, name);
			values_[name] = v;
			line_++;
			return;
		}
		if (first.kind == Token::Ident && (AtomicOps().count(first.text) || first.text.rfind("atomicAdd_", 0) == 0)) {
			ParseAtomic(false);
			Expect(";");
			line_++;
			return;
		}
		if (first.kind == Token::Ident && Peek(1).text == "[") {
			// X_mem[address] = asuint(value);   array[address] = value;
			const std::string name = Next().text;
			Expect("[");
			V address = Expression();
			Expect("]");
			Expect("=");
			V value = Expression();
			Expect(";");
			if (IsBufferName(name)) {
				// the word written is asuint(value): the store holds the value itself
				if (value.n->op->name == std::string("asuint") && value.n->debug_name.empty()) value = Unwrap(value);
				kb_->Store(Buffer(name), address, value);
			} else {
				if (!arrays_.count(name)) Fail("unknown array " + name);
				kb_->Store(arrays_[name], address, value);
			}
			line_++;
			return;
		}
		if (first.kind == Token::Ident && Peek(1).text == "=") {
			const std::string name = Next().text;
			Expect("=");
			if (!values_.count(name)) Fail("assignment to an unknown name " + name);
			V value = Expression(values_[name].type());
			Expect(";");
			kb_->Set(values_[name], value);
			line_++;
			return;
		}
		Fail("statement form not recognised");
	}

	// Takes a single-use wrapper node out of the tree again (the argument stays).
	V Unwrap(V wrapper) {
		Node* inner = wrapper.n->inputs[0];
		inner->use_count--;
		Node* scope = wrapper.n->parent;
		scope->children.erase(std::find(scope->children.begin(), scope->children.end(), wrapper.n));
		return V(inner, kb_.get());
	}

	void OpenGuard(V cond) {
		// index k = the named value computed from block_thread_id<k>; its extent = the other side of its `<` in the guard
		std::vector<const Node*> conjuncts;
		std::function<void(const Node*)> split = [&](const Node* n) {
			if (n->op->name == std::string("and") && n->type == TFType_Bool && n->debug_name.empty()) {
				split(n->inputs[0]);
				split(n->inputs[1]);
			} else {
				conjuncts.push_back(n);
			}
		};
		const Node* root = cond.n;
		if (root->op->name == std::string("and")) {
			split(root->inputs[0]);
			split(root->inputs[1]);
		} else {
			conjuncts.push_back(root);
		}
		std::function<bool(const Node*, uint32_t)> moves_with = [&](const Node* n, uint32_t k) {
			if (n->op->name == std::string("block_thread_id")) return n->data == k;
			for (const Node* in : n->inputs)
				if (moves_with(in, k)) return true;
			return false;
		};
		std::vector<V> indices, shape;
		for (uint32_t k = 0; k < conjuncts.size(); k++) {
			bool found = false;
			for (const Node* c : conjuncts) {
				if (c->op->name != std::string("lt")) Fail("the dispatch guard is not a conjunction of index < extent");
				if (moves_with(c->inputs[0], k)) {
					indices.push_back(V(c->inputs[0], kb_.get()));
					shape.push_back(V(c->inputs[1], kb_.get()));
					found = true;
					break;
				}
			}
			if (!found) {
				// a dimension without a thread-group axis (kernel dimensions beyond the group's): in order of appearance
				for (const Node* c : conjuncts) {
					bool taken = false;
					for (V& i : indices) taken |= i.n == c->inputs[0];
					bool grouped = false;
					for (uint32_t g = 0; g < 3; g++) grouped |= moves_with(c->inputs[0], g);
					if (!taken && !grouped) {
						indices.push_back(V(c->inputs[0], kb_.get()));
						shape.push_back(V(c->inputs[1], kb_.get()));
						found = true;
						break;
					}
				}
			}
			if (!found) Fail("no index of the dispatch guard moves with block_thread_id" + std::to_string(k));
		}
		kb_->OpenDispatchGuard(cond, indices, shape);
	}

	V Buffer(const std::string& name_mem) {
		const std::string name = name_mem.substr(0, name_mem.size() - 4);
		if (!buffers_.count(name)) Fail("unknown buffer " + name);
		return buffers_[name];
	}

	V ParseAtomic(bool returns) {
		const std::string fn = Next().text;
		Expect("(");
		if (AtomicOps().count(fn)) {
			// atomicOp(X_mem[address], uint(input))   (GLSL.cpp:24-50)
			const std::string mem = Next().text;
			Expect("[");
			V address = Expression();
			Expect("]");
			Expect(",");
			Expect("uint");
			Expect("(");
			V input = Expression();
			Expect(")");
			Expect(")");
			std::string op = AtomicOps().at(fn);
			if (returns) op += "_Prev";
			return kb_->Atomic(op, Buffer(mem), address, input, returns);
		}
		// atomicAdd_<buffer>_mem(address, input): float add
		const std::string mem = fn.substr(10);
		V address = Expression();
		Expect(",");
		V input = Expression();
		Expect(")");
		return kb_->Atomic(returns ? "InterlockedAdd_Prev" : "InterlockedAdd", Buffer(mem), address, input, returns);
	}

	// ---- expressions (C precedence; every operator and call is one node) ----------------------------------------
	V Expression(TFType want = TFType_None) { return Ternary(want); }

	V Ternary(TFType want) {
		V c = Binary(0, want);
		if (Accept("?")) {
			V a = Ternary(want);
			Expect(":");
			V b = Ternary(want);
			return kb_->Op("ternary", {c, a, b}, a.type());
		}
		return c;
	}

	struct BinOp {
		const char* token;
		const char* op;
		int level;
		bool compare;
	};
	static const std::vector<BinOp>& BinOps() {
		static const std::vector<BinOp> ops = {{"||", "or", 0, true},  {"&&", "and", 1, true}, {"|", "or", 2, false},     {"^", "xor", 3, false},    {"&", "and", 4, false},
		                                       {"==", "eq", 5, true},  {"!=", "neq", 5, true}, {"<", "lt", 6, true},      {"<=", "lte", 6, true},    {">", "gt", 6, true},
		                                       {">=", "gte", 6, true}, {"<<", "lshift", 7, false}, {">>", "rshift", 7, false}, {"+", "add", 8, false}, {"-", "sub", 8, false},
		                                       {"*", "mul", 9, false}, {"/", "div", 9, false}, {"%", "mod", 9, false}};
		return ops;
	}

	V Binary(int level, TFType want) {
		if (level > 9) return Unary(want);
		V left = Binary(level + 1, want);
		while (true) {
			const BinOp* found = nullptr;
			if (Peek().kind == Token::Punct)
				for (const BinOp& b : BinOps())
					if (b.level == level && Peek().text == b.token) found = &b;
			if (!found) return left;
			Next();
			V right = Binary(level + 1, found->compare ? TFType_None : left.type());
			left = kb_->Op(found->op, {left, right}, found->compare ? TFType_Bool : left.type());
		}
	}

	V Unary(TFType want) {
		if (Peek().kind == Token::Punct && Peek().text == "-") {
			Next();
			if (Peek().kind == Token::Number) return Number(Next().text, true, want);  // a negative constant
			V x = Unary(want);
			return kb_->Op("neg", {x}, x.type());
		}
		if (Accept("!")) {
			V x = Unary(TFType_Bool);
			return kb_->Op("notb", {x}, TFType_Bool);
		}
		if (Accept("~")) {
			V x = Unary(want);
			return kb_->Op("not", {x}, x.type());
		}
		return Primary(want);
	}

	V Number(const std::string& text, bool negative, TFType want) {
		const char last = text.back();
		const bool is_hex = text.size() > 2 && text[1] == 'x';
		if (!is_hex && (last == 'f' || text.find('.') != std::string::npos || text.find('e') != std::string::npos)) {
			const float f = std::strtof(text.c_str(), nullptr);
			return kb_->Const(negative ? -f : f);
		}
		if (last == 'u') {
			const uint32_t u = (uint32_t)std::strtoul(text.c_str(), nullptr, 0);
			return kb_->ConstU(negative ? (uint32_t)(-(int64_t)u) : u);
		}
		const long long v = std::strtoll(text.c_str(), nullptr, 0);
		(void)want;  // a constant has the type it is printed with: 22 is an int also next to a uint
		return kb_->Const((int)(negative ? -v : v));
	}

	V Primary(TFType want) {
		const Token t = Next();
		if (t.kind == Token::Number) return Number(t.text, false, want);
		if (t.kind == Token::Punct && t.text == "(") {
			V v = Expression(want);
			Expect(")");
			return v;
		}
		if (t.kind != Token::Ident) Fail("unexpected '" + t.text + "'");
		const std::string& name = t.text;
		if (name == "true" || name == "false") return kb_->ConstB(name == "true");
		if (name == "var") {
			Expect(".");
			const std::string field = Next().text;
			if (!variables_.count(field)) variables_[field] = kb_->Var(field, TFType_Int);
			return variables_[field];
		}
		if (name == "block_id") return kb_->BlockId();
		if (name.rfind("block_thread_id", 0) == 0 && name.size() == 16) return kb_->BlockThreadId(name[15] - '0');
		if (Peek().text == "[") {
			Next();
			V address = Expression();
			Expect("]");
			if (IsBufferName(name)) return kb_->Load(Buffer(name), address, TFType_Uint);
			if (!arrays_.count(name)) Fail("unknown array " + name);
			return kb_->Load(arrays_[name], address, arrays_[name].type());
		}
		if (Peek().text == "(") {
			if (AtomicOps().count(name) || name.rfind("atomicAdd_", 0) == 0) {
				pos_--;
				return ParseAtomic(true);
			}
			Next();
			const TFType cast = TypeOf(name);
			if (cast != TFType_None) {
				// T(atomicOp(...)) is how a value-returning atomic is printed (GLSL.cpp:33-38)
				if (Peek().kind == Token::Ident && (AtomicOps().count(Peek().text) || Peek().text.rfind("atomicAdd_", 0) == 0)) {
					V a = ParseAtomic(true);
					Expect(")");
					return a;
				}
				V x = Expression();
				Expect(")");
				return kb_->Op(name, {x}, cast);
			}
			if (name == "asfloat" || name == "asint" || name == "asuint" || name == "asbool") {
				const TFType to = TypeOf(name.substr(2));
				// as<T>(X_mem[address]) is a load of type T, one node
				if (Peek().kind == Token::Ident && IsBufferName(Peek().text) && Peek(1).text == "[") {
					const std::string mem = Next().text;
					Next();
					V address = Expression();
					Expect("]");
					Expect(")");
					return kb_->Load(Buffer(mem), address, to);
				}
				V x = Expression();
				Expect(")");
				return kb_->Op(name, {x}, to);
			}
			std::vector<V> args;
			if (!Accept(")")) {
				do args.push_back(Expression(args.empty() ? want : args[0].type()));
				while (Accept(","));
				Expect(")");
			}
			std::string op = FunctionOps().count(name) ? FunctionOps().at(name) : name;
			if (op == "atan" && args.size() == 2) op = "atan2";
			TFType type = args.empty() ? TFType_None : args[0].type();
			if (op == "pcg") type = TFType_Uint;
			if (op == "pcgf") type = TFType_Float;
			return kb_->Op(op, args, type);  // throws for a name that is not in the op table
		}
		if (!values_.count(name)) Fail("unknown name " + name);
		return values_[name];
	}
};

// The kernel text the "kernel_text" program is built from (set by tftest_set_kernel_text before tf.compile).
struct PendingKernelText {
	std::string body, shared;
	int group[3] = {1, 1, 1};
} g_pending;

std::vector<std::string> SplitLines(const char* text) {
	std::vector<std::string> out;
	std::istringstream in(text ? text : "");
	for (std::string l; std::getline(in, l);)
		if (l.find_first_not_of(" \t\r") != std::string::npos) out.push_back(l);
	return out;
}

// A program around one kernel parsed from printed text, so that the kernel can be run: every buffer of the kernel is an
// input tensor (read-write ones first, in the kernel's binding order, written in place), the kernel's variables and
// the dispatch shape are constants of the host program.
//   params: flags (bit 0: emit as any program's kernel would be, not verbatim), number of dispatch dimensions, the
//           dispatch shape outermost first, then the value of every kernel variable in binding order.
//   output: one word that nothing writes (a program has at least one output).
void BuildKernelTextProgram(Program* program, const std::vector<int64_t>& params) {
	if (params.size() < 2) throw std::runtime_error("kernel_text: parameters are flags, dimension count, shape, variable values");
	const bool as_any_kernel = params[0] & 1;
	const size_t dims = (size_t)params[1];
	if (params.size() < 2 + dims) throw std::runtime_error("kernel_text: dispatch shape missing");
	std::vector<int> group = {g_pending.group[0], g_pending.group[1], g_pending.group[2]};
	KernelTextParser parser(program, SplitLines(g_pending.body.c_str()), group, SplitLines(g_pending.shared.c_str()));
	Kernel* kernel = parser.Parse();
	if (as_any_kernel) {
		kernel->serial_loops = false;
		kernel->verbatim = false;
	}
	if (params.size() != 2 + dims + kernel->variables.size())
		throw std::runtime_error("kernel_text: the kernel has " + std::to_string(kernel->variables.size()) + " variables, " + std::to_string(params.size() - 2 - dims) + " values given");
	HostBuilder h(program);
	std::vector<V> read_write, read_only, variables;
	for (Node* m : kernel->read_write_memory) read_write.push_back(h.Input(m->debug_name, {-1}, TFType_Uint));
	for (Node* m : kernel->read_only_memory) read_only.push_back(h.Input(m->debug_name, {-1}, TFType_Uint));
	for (size_t i = 0; i < kernel->variables.size(); i++) variables.push_back(h.Const((int)params[2 + dims + i]));
	std::vector<Dim> shape;
	for (size_t i = 0; i < dims; i++) shape.push_back(Dim((long)params[2 + i]));
	h.Dispatch(kernel, read_write, read_only, variables, shape);
	h.Output(h.Allocate("nothing", {1}, TFType_Uint));
	h.Finish();
}

ProgramRegistrar reg_kernel_text("kernel_text", BuildKernelTextProgram);

}  // namespace

}  // namespace tfhost

// Sets the text the next tf.compile("kernel_text", ...) is built from, and reports the kernel's buffers (in the order
// the program takes them as inputs) and variables (in the order their values are passed) as "b0,b1,...|v0,v1,...".
extern "C" long tftest_set_kernel_text(const char* body, const int* group, const char* shared, char* out, size_t cap) {
	using namespace tfhost;
	std::string result;
	long status = 0;
	try {
		g_pending.body = body ? body : "";
		g_pending.shared = shared ? shared : "";
		for (int i = 0; i < 3; i++) g_pending.group[i] = group[i];
		Program program;
		KernelTextParser parser(&program, SplitLines(body), {group[0], group[1], group[2]}, SplitLines(shared));
		Kernel* kernel = parser.Parse();
		for (Node* m : kernel->MemoryBindings()) result += (result.empty() ? "" : ",") + m->debug_name;
		result += "|";
		for (size_t i = 0; i < kernel->variables.size(); i++) result += (i ? "," : "") + kernel->variables[i].name;
		status = (long)result.size();
	} catch (const std::exception& e) {
		result = e.what();
		status = -1;
	}
	if (cap) {
		const size_t n = std::min(cap - 1, result.size());
		std::memcpy(out, result.data(), n);
		out[n] = 0;
	}
	return status;
}

// body: the statements of the printed kernel after the block_id / block_thread_id lines, one per line; group: the
// three local sizes; shared: the `shared T name[n];` declarations printed above the kernel, one per line.
// Writes the whole HIP source the emitter generates for that kernel (prelude, variable block, kernel_0) to out (NUL-terminated, truncated to cap) and returns
// its full length, or -1 with the reason in out.
extern "C" long tftest_emit_kernel_text(const char* body, const int* group, const char* shared, char* out, size_t cap) {
	using namespace tfhost;
	std::string result;
	long status = 0;
	try {
		Program program;
		std::vector<int> g = {group[0], group[1], group[2]};
		KernelTextParser parser(&program, SplitLines(body), g, SplitLines(shared));
		Kernel* kernel = parser.Parse();
		kernel->kernel_name_ = "kernel_0";
		GenerateHIPKernel(&program, kernel);
		result = kernel->full_generated_code_;
		status = (long)result.size();
	} catch (const std::exception& e) {
		result = e.what();
		status = -1;
	}
	if (cap) {
		const size_t n = std::min(cap - 1, result.size());
		std::memcpy(out, result.data(), n);
		out[n] = 0;
	}
	return status;
}

// import_roundtrip.cpp
std::string ImportRoundTripOf(tfhost::Program* program, tfhost::Kernel* kernel, const std::string& label);

// The kernel parsed from printed text, sent through the mirror of the compiler's classes and the kernel importer and
// emitted from there: "" in out and 0, or -1 with the first difference. verbatim as tftest_emit_kernel_text emits it.
extern "C" long tftest_roundtrip_kernel_text(const char* body, const int* group, const char* shared, int verbatim, char* out, size_t cap) {
	using namespace tfhost;
	std::string result;
	long status = 0;
	try {
		Program program;
		std::vector<int> g = {group[0], group[1], group[2]};
		KernelTextParser parser(&program, SplitLines(body), g, SplitLines(shared));
		Kernel* kernel = parser.Parse();
		kernel->verbatim = verbatim != 0;
		result = ImportRoundTripOf(&program, kernel, "printed kernel");
		status = result.empty() ? 0 : -1;
	} catch (const std::exception& e) {
		result = std::string("exception: ") + e.what();
		status = -1;
	}
	if (cap) {
		const size_t n = std::min(cap - 1, result.size());
		std::memcpy(out, result.data(), n);
		out[n] = 0;
	}
	return status;
}
