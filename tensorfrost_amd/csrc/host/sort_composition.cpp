#include "sort_composition.h"

#include <unordered_map>

namespace tfhost {

namespace {

struct Digits {
	int bits, hist;  // bits per pass, histogram bins (sort.py:90-91)
	unsigned variant = 0;
};

// GetBits (sort.py:93-94). `pass` is the pass index, or with kSortShiftVariable the shift itself (pass * bits_per_pass
// evaluated on the host, where the loop variable lives).
V GetBits(KernelBuilder& kb, const Digits& dg, V key, V pass) {
	V shift = dg.variant & kSortShiftVariable ? pass : pass * kb.Const(dg.bits);
	return (key >> ToUint(shift)) & kb.ConstU((uint32_t)dg.hist - 1u);
}

// keys = tf.copy(keys), alone or fused with one of the order-preserving maps between float / int keys and uints
Kernel* BuildMap(Program* program, SortRole role) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("mapped", false), in = kb.Buffer("keys", true);
	V N = kb.Var("N", TFType_Int);
	V i = kb.ThreadIndices({N})[0];
	V x = kb.Named(kb.Load(in, i, TFType_Uint), "ux");
	V sign_bit = kb.ConstU(0x80000000u), ones = kb.ConstU(0xFFFFFFFFu);
	V y = x;
	if (role == SortRole::MapFloat) y = x ^ Select((x >> kb.ConstU(31u)) == kb.ConstU(1u), ones, sign_bit);
	if (role == SortRole::UnmapFloat) y = x ^ Select((x >> kb.ConstU(31u)) == kb.ConstU(0u), ones, sign_bit);
	if (role == SortRole::MapInt || role == SortRole::UnmapInt) y = x ^ sign_bit;
	kb.Store(out, i, y);
	return kb.Finish();
}

// keys = tf.copy(keys) [+ map] and values = tf.copy(values) in ONE kernel: what kernel fusion makes of them when both
// tensors have the same shape node (Compiler/Graph/Scope.cpp:165-188), e.g. values declared with keys.shape
Kernel* BuildFusedCopies(Program* program, SortRole key_role) {
	KernelBuilder kb(program, 1);
	V keys_out = kb.Buffer("mapped", false), values_out = kb.Buffer("values_copy", false), keys = kb.Buffer("keys", true), values = kb.Buffer("values", true);
	V N = kb.Var("N", TFType_Int);
	V i = kb.ThreadIndices({N})[0];
	V x = kb.Named(kb.Load(keys, i, TFType_Uint), "ux");
	V sign_bit = kb.ConstU(0x80000000u), ones = kb.ConstU(0xFFFFFFFFu);
	V y = x;
	if (key_role == SortRole::MapFloat) y = x ^ Select((x >> kb.ConstU(31u)) == kb.ConstU(1u), ones, sign_bit);
	if (key_role == SortRole::MapInt) y = x ^ sign_bit;
	kb.Store(keys_out, i, y);
	kb.Store(values_out, i, kb.Load(values, i, TFType_Uint));
	return kb.Finish();
}

// digits[e] = GetBits(keys_in[e], pass) as a tensor of its own (the value sort.py calls GetBits(keys_in, iter), kept
// in memory instead of being recomputed by the kernel that loads it)
Kernel* BuildDigits(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 1);
	V digits = kb.Buffer("digits", false), keys = kb.Buffer("keys_in", true);
	V N = kb.Var("N", TFType_Int), pass = kb.Var(dg.variant & kSortShiftVariable ? "shift" : "pass", TFType_Int);
	V i = kb.ThreadIndices({N})[0];
	kb.Store(digits, i, GetBits(kb, dg, kb.Load(keys, i, TFType_Uint), pass));
	return kb.Finish();
}

// group_histogram_packed[g, i] = sum_e packed_is_bit(g, e, i): kernel shape [G, hist / 4], the sum lowered to a loop over e
Kernel* BuildPackedHistogram(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 2);
	const bool from_digits = dg.variant & kSortDigitsBuffer;
	V packed = kb.Buffer("group_histogram_packed", false), keys = kb.Buffer(from_digits ? "digits" : "keys_in", true);
	V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int);
	V pass = from_digits ? V() : kb.Var(dg.variant & kSortShiftVariable ? "shift" : "pass", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(dg.hist / 4), G});
	V i = idx[0], g = idx[1];
	V acc = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(kSortGroup), kb.Const(1), [&](V e) {
		V element = kb.Named(g * kb.Const(kSortGroup) + e, "element");
		// grouped = split_dim(GetBits(keys_in, iter), 128): out-of-bounds elements read as 0
		V oob = kb.Named(kb.ConstB(false) || ((element < kb.Const(0)) || (element >= N)), "out_of_bounds");
		V key = kb.Load(keys, kb.Clamp(element, kb.Const(0), N - kb.Const(1)), TFType_Uint);
		V this_key = kb.Named(Select(oob, kb.ConstU(0u), from_digits ? key : GetBits(kb, dg, key, pass)), "this_key");
		auto is = [&](int k) { return ToUint(Select(this_key == ToUint(kb.Const(4) * i + kb.Const(k)), kb.Const(1), kb.Const(0))); };
		V bits = kb.Named(is(0) + (is(1) << kb.ConstU(8u)) + (is(2) << kb.ConstU(16u)) + (is(3) << kb.ConstU(24u)), "packed_is_bit");
		kb.Set(acc, acc + Select(element < N, bits, kb.ConstU(0u)));
	});
	kb.Store(packed, g * kb.Const(dg.hist / 4) + i, acc);
	return kb.Finish();
}

// group_histogram[g, i] computed where it is used instead of loaded (what load fusion makes of an element-wise value)
V Unpacked(KernelBuilder& kb, const Digits& dg, V packed, V g, V i) {
	V word = kb.Load(packed, g * kb.Const(dg.hist / 4) + i / kb.Const(4), TFType_Uint);
	return (word >> ToUint(kb.Const(8) * (i % kb.Const(4)))) & kb.ConstU(0xFFu);
}

// group_histogram[g, i] = (packed[g, i / 4] >> 8 * (i % 4)) & 0xFF: kernel shape [G, hist]
Kernel* BuildUnpack(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 2);
	V hist = kb.Buffer("group_histogram", false), packed = kb.Buffer("group_histogram_packed", true);
	V G = kb.Var("G", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(dg.hist), G});
	V i = idx[0], g = idx[1];
	V word = kb.Load(packed, g * kb.Const(dg.hist / 4) + i / kb.Const(4), TFType_Uint);
	kb.Store(hist, g * kb.Const(dg.hist) + i, (word >> ToUint(kb.Const(8) * (i % kb.Const(4)))) & kb.ConstU(0xFFu));
	return kb.Finish();
}

// prefix_sum_grouped, step 1: chunk_sum[c, i] = sum_{e < 64} hist[c*64 + e, i] (zero beyond G): kernel shape [chunks, hist]
Kernel* BuildChunkSums(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 2);
	const bool inlined = dg.variant & kSortInlinedUnpack;
	V sums = kb.Buffer("chunk_scan", false), hist = kb.Buffer(inlined ? "group_histogram_packed" : "group_histogram", true);
	V G = kb.Var("G", TFType_Int), chunks = kb.Var("chunks", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(dg.hist), chunks});
	V i = idx[0], c = idx[1];
	V acc = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(kSortScanChunk), kb.Const(1), [&](V e) {
		V g = kb.Named(c * kb.Const(kSortScanChunk) + e, "group");
		V oob = kb.Named(kb.ConstB(false) || ((g < kb.Const(0)) || (g >= G)), "out_of_bounds");
		V row = kb.Clamp(g, kb.Const(0), G - kb.Const(1));
		V x = inlined ? Unpacked(kb, dg, hist, row, i) : kb.Load(hist, row * kb.Const(dg.hist) + i, TFType_Uint);
		kb.Set(acc, acc + Select(oob, kb.ConstU(0u), x));
	});
	kb.Store(sums, c * kb.Const(dg.hist) + i, acc);
	return kb.Finish();
}

// step 2: inclusive prefix over the chunks, one thread per digit: kernel shape [hist]
Kernel* BuildChunkScan(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("chunk_scan_out", false), in = kb.Buffer("chunk_scan", true);
	V chunks = kb.Var("chunks", TFType_Int);
	V i = kb.ThreadIndices({kb.Const(dg.hist)})[0];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), chunks, kb.Const(1), [&](V c) {
		kb.Set(acc, acc + kb.Load(in, c * kb.Const(dg.hist) + i, TFType_Uint));
		kb.Store(out, c * kb.Const(dg.hist) + i, acc);
	});
	return kb.Finish();
}

// step 3: scan inside every chunk, the first element seeded with the previous chunk's running total; merge_dim drops
// the padded tail: kernel shape [chunks, hist]
Kernel* BuildScanInChunks(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 2);
	const bool inlined = dg.variant & kSortInlinedUnpack;
	V scan = kb.Buffer("group_histogram_scan", false), hist = kb.Buffer(inlined ? "group_histogram_packed" : "group_histogram", true), chunk_scan = kb.Buffer("chunk_scan_out", true);
	V G = kb.Var("G", TFType_Int), chunks = kb.Var("chunks", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(dg.hist), chunks});
	V i = idx[0], c = idx[1];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(kSortScanChunk), kb.Const(1), [&](V e) {
		V g = kb.Named(c * kb.Const(kSortScanChunk) + e, "group");
		kb.If(g < G, [&] {
			V seed = Select((c == kb.Const(0)) || (e != kb.Const(0)), kb.ConstU(0u),
			                kb.Load(chunk_scan, kb.Clamp(c - kb.Const(1), kb.Const(0), chunks - kb.Const(1)) * kb.Const(dg.hist) + i, TFType_Uint));
			V x = inlined ? Unpacked(kb, dg, hist, g, i) : kb.Load(hist, g * kb.Const(dg.hist) + i, TFType_Uint);
			kb.Set(acc, acc + x + seed);
			kb.Store(scan, g * kb.Const(dg.hist) + i, acc);
		});
	});
	return kb.Finish();
}

// total_bit_histogram = prefix_sum(group_histogram_scan[G - 1, :]): a single thread walks the digits
Kernel* BuildTotals(Program* program, const Digits& dg) {
	KernelBuilder kb(program, 1);
	V total = kb.Buffer("total_bit_histogram", false), scan = kb.Buffer("group_histogram_scan", true);
	V G = kb.Var("G", TFType_Int);
	V t = kb.ThreadIndices({kb.Const(1)})[0];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(dg.hist), kb.Const(1), [&](V k) {
		kb.Set(acc, acc + kb.Load(scan, (G - kb.Const(1)) * kb.Const(dg.hist) + k + t, TFType_Uint));
		kb.Store(total, k + t, acc);
	});
	return kb.Finish();
}

// The scatter kernel, group-buffer branch (sort.py:133-169): kernel shape [G, 128], group {128}
Kernel* BuildScatter(Program* program, const Digits& dg, bool has_values) {
	KernelBuilder kb(program, 2, {kSortGroup});
	V keys_out = kb.Buffer("keys_out", false);
	V values_out = has_values ? kb.Buffer("values_out", false) : V();
	V keys_in = kb.Buffer("keys_in", true);
	V values_in = has_values ? kb.Buffer("values_in", true) : V();
	V scan = kb.Buffer("group_histogram_scan", true), total = kb.Buffer("total_bit_histogram", true);
	V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int), pass = kb.Var(dg.variant & kSortShiftVariable ? "shift" : "pass", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kSortGroup), G});
	V e = idx[0], g = idx[1];
	V temp = kb.GroupMemory("temp", TFType_Uint, kSortGroup);
	V half_count = kb.GroupMemory("half_count", TFType_Uint, dg.hist);
	V gtid = kb.BlockThreadId(0);
	// initialize counters: a Python loop at trace time, so one guarded store per 128 bins (sort.py:139-143)
	for (int r = 0; r < (dg.hist + kSortGroup - 1) / kSortGroup; r++) {
		V index = r == 0 ? gtid : gtid + kb.Const(r * kSortGroup);
		kb.If(index < kb.Const(dg.hist), [&] { kb.Store(half_count, index, kb.ConstU(0u)); });
	}
	kb.Barrier();
	V element = kb.Named(g * kb.Const(kSortGroup) + e, "element");
	kb.If(element < N, [&] {
		V old_key = kb.Named(kb.Load(keys_in, element, TFType_Uint), "old_key");
		V bit = kb.Named(GetBits(kb, dg, old_key, pass), "bit");
		V ibit = kb.Named(ToInt(bit), "ibit");
		kb.Store(temp, gtid, bit);
		V quarter = kb.Named(e / kb.Const(kSortGroup / 4), "quarter_index");
		kb.If(quarter < kb.Const(3), [&] {
			auto flag = [&](int q) { return ToUint(Select(quarter < kb.Const(q), kb.Const(1), kb.Const(0))); };
			kb.Atomic("InterlockedAdd", half_count, ibit, flag(1) | (flag(2) << kb.ConstU(8u)) | (flag(3) << kb.ConstU(16u)));
		});
		kb.Barrier();
		V old_val = has_values ? kb.Named(kb.Load(values_in, element, TFType_Uint), "old_val") : V();
		V before_groups = Select(g == kb.Const(0), kb.ConstU(0u), kb.Load(scan, kb.Clamp(g - kb.Const(1), kb.Const(0), G - kb.Const(1)) * kb.Const(dg.hist) + ibit, TFType_Uint));
		V before_digits = Select(ibit == kb.Const(0), kb.ConstU(0u), kb.Load(total, kb.Clamp(ibit - kb.Const(1), kb.Const(0), kb.Const(dg.hist - 1)), TFType_Uint));
		V in_quarters = Select(quarter > kb.Const(0), (kb.Load(half_count, ibit, TFType_Uint) >> ToUint(kb.Const(8) * (quarter - kb.Const(1)))) & kb.ConstU(0xFFu), kb.ConstU(0u));
		V offset = kb.Accumulator("total_offset", TFType_Uint, 0u);
		kb.Set(offset, before_groups + before_digits + in_quarters);
		kb.Loop(quarter * kb.Const(kSortGroup / 4), e, kb.Const(1), [&](V j) { kb.Set(offset, offset + Select(kb.Load(temp, j, TFType_Uint) == bit, kb.ConstU(1u), kb.ConstU(0u))); });
		V dst = kb.Named(ToInt(offset), "dst");
		kb.Store(keys_out, dst, old_key);
		if (has_values) kb.Store(values_out, dst, old_val);
	});
	return kb.Finish();
}

}  // namespace

Kernel* BuildFusedCopyKernel(Program* program, SortRole key_role) { return BuildFusedCopies(program, key_role); }

Kernel* BuildDigitsKernel(Program* program, int bits, unsigned variant) { return BuildDigits(program, Digits{bits, 1 << bits, variant}); }

Kernel* BuildSortKernel(Program* program, SortRole role, int bits, unsigned variant) {
	if (bits < 2 || bits > 8) throw std::runtime_error("radix sort: bits per pass must lie in 2..8 (four 8-bit counters share a word of the packed histogram)");
	const Digits dg{bits, 1 << bits, variant};
	switch (role) {
		case SortRole::Copy:
		case SortRole::MapFloat:
		case SortRole::MapInt:
		case SortRole::UnmapFloat:
		case SortRole::UnmapInt: return BuildMap(program, role);
		case SortRole::Histogram: return BuildPackedHistogram(program, dg);
		case SortRole::Unpack: return BuildUnpack(program, dg);
		case SortRole::ChunkSums: return BuildChunkSums(program, dg);
		case SortRole::ChunkScan: return BuildChunkScan(program, dg);
		case SortRole::ScanInChunks: return BuildScanInChunks(program, dg);
		case SortRole::Totals: return BuildTotals(program, dg);
		case SortRole::Scatter: return BuildScatter(program, dg, true);
		case SortRole::ScatterKeys: return BuildScatter(program, dg, false);
		default: throw std::runtime_error("radix sort: no kernel for this role");
	}
}

// ---- structural identity --------------------------------------------------------------------------------------

namespace {

struct Hasher {
	uint64_t h = 1469598103934665603ull;
	void Word(uint64_t v) {
		for (int i = 0; i < 8; i++) {
			h ^= (v >> (8 * i)) & 0xFF;
			h *= 1099511628211ull;
		}
	}
	void Text(const char* s) {
		for (; *s; s++) {
			h ^= (unsigned char)*s;
			h *= 1099511628211ull;
		}
		Word(0x5eedull);
	}
};

struct Fingerprinter {
	const Kernel* kernel;
	Hasher hash;
	std::unordered_map<const Node*, uint64_t> ordinal;  // order of first appearance

	// Kernel arguments are identified by where they are bound, everything else by when it first appears.
	uint64_t Ref(const Node* n) {
		if (!n) return 0;
		auto it = ordinal.find(n);
		if (it != ordinal.end()) return it->second;
		// a value that is no statement of a scope (never the case for trees the builder makes): hashed where it is first used
		Visit(n);
		return ordinal.at(n);
	}

	void Visit(const Node* n) {
		if (ordinal.count(n)) return;
		const uint64_t id = ordinal.size() + 16;
		ordinal[n] = id;
		hash.Word(id);
		hash.Text(n->op->name);
		hash.Word((uint64_t)n->type);
		hash.Word(n->data);
		hash.Word((n->modified ? 1u : 0u) | (n->local_memory_op ? 2u : 0u));
		hash.Word(n->inputs.size());
		for (const Node* x : n->inputs) hash.Word(Ref(x));
		hash.Word(Ref(n->index));
		hash.Word(Ref(n->memory));
		hash.Word(n->children.size());
		for (const Node* c : n->children) Visit(c);
		hash.Word(0xE0D0ull);
	}
};

}  // namespace

uint64_t KernelFingerprint(const Kernel* kernel) {
	Fingerprinter f{kernel, {}, {}};
	f.hash.Word((uint64_t)kernel->dim);
	f.hash.Word(kernel->group_size.size());
	for (int g : kernel->group_size) f.hash.Word((uint64_t)g);
	// bound arguments first, so that a use of one hashes as its position
	f.hash.Word(kernel->read_write_memory.size());
	f.hash.Word(kernel->read_only_memory.size());
	for (const Node* m : kernel->MemoryBindings()) f.Visit(m);
	f.hash.Word(kernel->variables.size());
	for (const KernelVariable& v : kernel->variables) {
		f.hash.Word((uint64_t)v.type);
		f.Visit(v.node);
	}
	if (kernel->root) f.Visit(kernel->root);
	return f.hash.h;
}

}  // namespace tfhost
