// tf.sort.radix as the reference itself composes it (Python/TensorFrost/sort.py:38-187), kernel by kernel in lowered IR
// form, for a backend that is not tf.cpu (so the scatter kernel is the group-buffer branch, :133-169). Nothing here
// names a primitive: the whole sort runs on emitted kernels, which is what an unchanged TensorFrost program gets
// from this backend today (the hand-written onesweep sort is reached through the `radix_sort` program instead).
//
//   6 passes of 6 bits, groups of 128 keys, 64 histogram bins                                   (:89-91)
//   per pass: packed group histogram [G, 16] = sum over the group of four 8-bit counters/uint    (:105-112)
//             unpack to [G, 64]                                                                 (:114-115)
//             prefix_sum_grouped over groups: chunk sums of 64 groups, serial scan over chunks,
//             scan inside every chunk seeded with the previous chunk's total                    (:39-50,117)
//             prefix sum of the last row over the digits                                        (:118-119)
//             scatter kernel with group buffers                                                 (:133-169)
//   keys of type float / int go through the order-preserving maps to uint and back               (:52-72,82-87,178-182)
//
//   params[0] = TFType of the keys (default uint).  inputs keys[N], values[N] (uint).  outputs sorted keys, values.
#include "registry.h"

namespace tfhost {

namespace {

constexpr int kBits = 6, kHist = 64, kGroup = 128;

V GetBits(KernelBuilder& kb, V key, V pass) { return (key >> ToUint(pass * kb.Const(kBits))) & kb.ConstU((uint32_t)kHist - 1u); }

// keys = tf.copy(keys) fused with the map to uint (mode 0: copy, 1: float -> uint, 2: int -> uint, 3: uint -> float, 4: uint -> int)
Kernel* BuildMap(Program* program, int mode) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("mapped", false), in = kb.Buffer("keys", true);
	V N = kb.Var("N", TFType_Int);
	V i = kb.ThreadIndices({N})[0];
	V x = kb.Named(kb.Load(in, i, TFType_Uint), "ux");
	V sign_bit = kb.ConstU(0x80000000u), ones = kb.ConstU(0xFFFFFFFFu);
	V y = x;
	if (mode == 1) y = x ^ Select((x >> kb.ConstU(31u)) == kb.ConstU(1u), ones, sign_bit);
	if (mode == 3) y = x ^ Select((x >> kb.ConstU(31u)) == kb.ConstU(0u), ones, sign_bit);
	if (mode == 2 || mode == 4) y = x ^ sign_bit;
	kb.Store(out, i, y);
	return kb.Finish();
}

// group_histogram_packed[g, i] = sum_e packed_is_bit(g, e, i): kernel shape [G, 16], the sum lowered to a loop over e
Kernel* BuildPackedHistogram(Program* program) {
	KernelBuilder kb(program, 2);
	V packed = kb.Buffer("group_histogram_packed", false), keys = kb.Buffer("keys_in", true);
	V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int), pass = kb.Var("pass", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kHist / 4), G});
	V i = idx[0], g = idx[1];
	V acc = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(kGroup), kb.Const(1), [&](V e) {
		V element = kb.Named(g * kb.Const(kGroup) + e, "element");
		// grouped = split_dim(GetBits(keys_in, iter), 128): out-of-bounds elements read as 0
		V oob = kb.Named(kb.ConstB(false) || ((element < kb.Const(0)) || (element >= N)), "out_of_bounds");
		V key = kb.Load(keys, kb.Clamp(element, kb.Const(0), N - kb.Const(1)), TFType_Uint);
		V this_key = kb.Named(Select(oob, kb.ConstU(0u), GetBits(kb, key, pass)), "this_key");
		auto is = [&](int k) { return ToUint(Select(this_key == ToUint(kb.Const(4) * i + kb.Const(k)), kb.Const(1), kb.Const(0))); };
		V bits = kb.Named(is(0) + (is(1) << kb.ConstU(8u)) + (is(2) << kb.ConstU(16u)) + (is(3) << kb.ConstU(24u)), "packed_is_bit");
		kb.Set(acc, acc + Select(element < N, bits, kb.ConstU(0u)));
	});
	kb.Store(packed, g * kb.Const(kHist / 4) + i, acc);
	return kb.Finish();
}

// group_histogram[g, i] = (packed[g, i / 4] >> 8 * (i % 4)) & 0xFF: kernel shape [G, 64]
Kernel* BuildUnpack(Program* program) {
	KernelBuilder kb(program, 2);
	V hist = kb.Buffer("group_histogram", false), packed = kb.Buffer("group_histogram_packed", true);
	V G = kb.Var("G", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kHist), G});
	V i = idx[0], g = idx[1];
	V word = kb.Load(packed, g * kb.Const(kHist / 4) + i / kb.Const(4), TFType_Uint);
	kb.Store(hist, g * kb.Const(kHist) + i, (word >> ToUint(kb.Const(8) * (i % kb.Const(4)))) & kb.ConstU(0xFFu));
	return kb.Finish();
}

// prefix_sum_grouped, step 1: chunk_sum[c, i] = sum_{e < 64} hist[c*64 + e, i] (zero beyond G): kernel shape [chunks, 64]
Kernel* BuildChunkSums(Program* program) {
	KernelBuilder kb(program, 2);
	V sums = kb.Buffer("chunk_scan", false), hist = kb.Buffer("group_histogram", true);
	V G = kb.Var("G", TFType_Int), chunks = kb.Var("chunks", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kHist), chunks});
	V i = idx[0], c = idx[1];
	V acc = kb.Accumulator("sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(64), kb.Const(1), [&](V e) {
		V g = kb.Named(c * kb.Const(64) + e, "group");
		V oob = kb.Named(kb.ConstB(false) || ((g < kb.Const(0)) || (g >= G)), "out_of_bounds");
		V x = kb.Load(hist, kb.Clamp(g, kb.Const(0), G - kb.Const(1)) * kb.Const(kHist) + i, TFType_Uint);
		kb.Set(acc, acc + Select(oob, kb.ConstU(0u), x));
	});
	kb.Store(sums, c * kb.Const(kHist) + i, acc);
	return kb.Finish();
}

// step 2: inclusive prefix over the chunks, one thread per digit: kernel shape [64]
Kernel* BuildChunkScan(Program* program) {
	KernelBuilder kb(program, 1);
	V out = kb.Buffer("chunk_scan_out", false), in = kb.Buffer("chunk_scan", true);
	V chunks = kb.Var("chunks", TFType_Int);
	V i = kb.ThreadIndices({kb.Const(kHist)})[0];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), chunks, kb.Const(1), [&](V c) {
		kb.Set(acc, acc + kb.Load(in, c * kb.Const(kHist) + i, TFType_Uint));
		kb.Store(out, c * kb.Const(kHist) + i, acc);
	});
	return kb.Finish();
}

// step 3: scan inside every chunk, the first element seeded with the previous chunk's running total; merge_dim drops
// the padded tail: kernel shape [chunks, 64]
Kernel* BuildScanInChunks(Program* program) {
	KernelBuilder kb(program, 2);
	V scan = kb.Buffer("group_histogram_scan", false), hist = kb.Buffer("group_histogram", true), chunk_scan = kb.Buffer("chunk_scan_out", true);
	V G = kb.Var("G", TFType_Int), chunks = kb.Var("chunks", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kHist), chunks});
	V i = idx[0], c = idx[1];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(64), kb.Const(1), [&](V e) {
		V g = kb.Named(c * kb.Const(64) + e, "group");
		kb.If(g < G, [&] {
			V seed = Select((c == kb.Const(0)) || (e != kb.Const(0)), kb.ConstU(0u),
			                kb.Load(chunk_scan, kb.Clamp(c - kb.Const(1), kb.Const(0), chunks - kb.Const(1)) * kb.Const(kHist) + i, TFType_Uint));
			kb.Set(acc, acc + kb.Load(hist, g * kb.Const(kHist) + i, TFType_Uint) + seed);
			kb.Store(scan, g * kb.Const(kHist) + i, acc);
		});
	});
	return kb.Finish();
}

// total_bit_histogram = prefix_sum(group_histogram_scan[G - 1, :]): a single thread walks the 64 digits
Kernel* BuildTotals(Program* program) {
	KernelBuilder kb(program, 1);
	V total = kb.Buffer("total_bit_histogram", false), scan = kb.Buffer("group_histogram_scan", true);
	V G = kb.Var("G", TFType_Int);
	V t = kb.ThreadIndices({kb.Const(1)})[0];
	V acc = kb.Accumulator("prefix_sum", TFType_Uint, 0u);
	kb.Loop(kb.Const(0), kb.Const(kHist), kb.Const(1), [&](V k) {
		kb.Set(acc, acc + kb.Load(scan, (G - kb.Const(1)) * kb.Const(kHist) + k + t, TFType_Uint));
		kb.Store(total, k + t, acc);
	});
	return kb.Finish();
}

// The scatter kernel, group-buffer branch (sort.py:133-169): kernel shape [G, 128], group {128}
Kernel* BuildScatter(Program* program) {
	KernelBuilder kb(program, 2, {kGroup});
	V keys_out = kb.Buffer("keys_out", false), values_out = kb.Buffer("values_out", false);
	V keys_in = kb.Buffer("keys_in", true), values_in = kb.Buffer("values_in", true), scan = kb.Buffer("group_histogram_scan", true),
	  total = kb.Buffer("total_bit_histogram", true);
	V N = kb.Var("N", TFType_Int), G = kb.Var("G", TFType_Int), pass = kb.Var("pass", TFType_Int);
	std::vector<V> idx = kb.ThreadIndices({kb.Const(kGroup), G});
	V e = idx[0], g = idx[1];
	V temp = kb.GroupMemory("temp", TFType_Uint, kGroup);
	V half_count = kb.GroupMemory("half_count", TFType_Uint, kHist);
	V gtid = kb.BlockThreadId(0);
	kb.If(gtid < kb.Const(kHist), [&] { kb.Store(half_count, gtid, kb.ConstU(0u)); });
	kb.Barrier();
	V element = kb.Named(g * kb.Const(kGroup) + e, "element");
	kb.If(element < N, [&] {
		V old_key = kb.Named(kb.Load(keys_in, element, TFType_Uint), "old_key");
		V bit = kb.Named(GetBits(kb, old_key, pass), "bit");
		V ibit = kb.Named(ToInt(bit), "ibit");
		kb.Store(temp, gtid, bit);
		V quarter = kb.Named(e / kb.Const(kGroup / 4), "quarter_index");
		kb.If(quarter < kb.Const(3), [&] {
			auto flag = [&](int q) { return ToUint(Select(quarter < kb.Const(q), kb.Const(1), kb.Const(0))); };
			kb.Atomic("InterlockedAdd", half_count, ibit, flag(1) | (flag(2) << kb.ConstU(8u)) | (flag(3) << kb.ConstU(16u)));
		});
		kb.Barrier();
		V old_val = kb.Named(kb.Load(values_in, element, TFType_Uint), "old_val");
		V before_groups = Select(g == kb.Const(0), kb.ConstU(0u), kb.Load(scan, kb.Clamp(g - kb.Const(1), kb.Const(0), G - kb.Const(1)) * kb.Const(kHist) + ibit, TFType_Uint));
		V before_digits = Select(ibit == kb.Const(0), kb.ConstU(0u), kb.Load(total, kb.Clamp(ibit - kb.Const(1), kb.Const(0), kb.Const(kHist - 1)), TFType_Uint));
		V in_quarters = Select(quarter > kb.Const(0), (kb.Load(half_count, ibit, TFType_Uint) >> ToUint(kb.Const(8) * (quarter - kb.Const(1)))) & kb.ConstU(0xFFu), kb.ConstU(0u));
		V offset = kb.Accumulator("total_offset", TFType_Uint, 0u);
		kb.Set(offset, before_groups + before_digits + in_quarters);
		kb.Loop(quarter * kb.Const(kGroup / 4), e, kb.Const(1), [&](V j) { kb.Set(offset, offset + Select(kb.Load(temp, j, TFType_Uint) == bit, kb.ConstU(1u), kb.ConstU(0u))); });
		V dst = kb.Named(ToInt(offset), "dst");
		kb.Store(keys_out, dst, old_key);
		kb.Store(values_out, dst, old_val);
	});
	return kb.Finish();
}

}  // namespace

static void BuildRadixSortIr(Program* program, const std::vector<int64_t>& params) {
	const int key_type = params.empty() ? TFType_Uint : (int)params[0];
	Kernel* copy = BuildMap(program, 0);
	Kernel* map_in = BuildMap(program, key_type == TFType_Float ? 1 : key_type == TFType_Int ? 2 : 0);
	Kernel* map_out = BuildMap(program, key_type == TFType_Float ? 3 : key_type == TFType_Int ? 4 : 0);
	Kernel* histogram = BuildPackedHistogram(program);
	Kernel* unpack = BuildUnpack(program);
	Kernel* chunk_sums = BuildChunkSums(program);
	Kernel* chunk_scan = BuildChunkScan(program);
	Kernel* scan_in_chunks = BuildScanInChunks(program);
	Kernel* totals = BuildTotals(program);
	Kernel* scatter = BuildScatter(program);
	program->input_count = 2;
	program->output_count = 2;
	program->execute_callback = [=](TFTensor* in, TFTensor* out, TFRuntime runtime) -> int {
		TFContext tf(runtime);
		const TFDataFormat key_format{(TFType)key_type, 32};
		tf.region_begin("Radix sort");
		if (in[0].dim != 1) throw std::runtime_error("Invalid number of dimensions for keys. Expected 1, got " + std::to_string(in[0].dim));
		const size_t N = in[0].shape[0];
		const int n = (int)N;
		tf.check_tensor(in[0], "keys", {N}, key_format);
		tf.check_tensor(in[1], "values", {N}, TFTypeUint32);
		const size_t G = (N + kGroup - 1) / kGroup, chunks = (G + 63) / 64;
		// keys = tf.copy(keys) (+ map to uint); values = tf.copy(values)
		TFTensor keys = tf.allocate("keys", {N}, TFTypeUint32), values = tf.allocate("values", {N}, TFTypeUint32);
		tf.dispatch(map_in->kernel_id_, {keys}, {in[0]}, {asuint(n)}, {N}, {256});
		tf.dispatch(copy->kernel_id_, {values}, {in[1]}, {asuint(n)}, {N}, {256});
		TFTensor keys1 = tf.allocate("keys1", {N}, TFTypeUint32), values1 = tf.allocate("values1", {N}, TFTypeUint32);
		const int iters = (32 + kBits - 1) / kBits;
		for (int pass = 0; pass < iters / 2 * 2; pass++) {
			tf.region_begin("Radix sort iteration");
			TFTensor k_in = (pass & 1) ? keys1 : keys, k_out = (pass & 1) ? keys : keys1;
			TFTensor v_in = (pass & 1) ? values1 : values, v_out = (pass & 1) ? values : values1;
			TFTensor packed = tf.allocate("group_histogram_packed", {G, (size_t)kHist / 4}, TFTypeUint32);
			tf.dispatch(histogram->kernel_id_, {packed}, {k_in}, {asuint(n), asuint((int)G), asuint(pass)}, {G, (size_t)kHist / 4}, {16, 16});
			TFTensor hist = tf.allocate("group_histogram", {G, (size_t)kHist}, TFTypeUint32);
			tf.dispatch(unpack->kernel_id_, {hist}, {packed}, {asuint((int)G)}, {G, (size_t)kHist}, {16, 16});
			tf.deallocate(packed);
			TFTensor sums = tf.allocate("chunk_scan", {chunks, (size_t)kHist}, TFTypeUint32);
			tf.dispatch(chunk_sums->kernel_id_, {sums}, {hist}, {asuint((int)G), asuint((int)chunks)}, {chunks, (size_t)kHist}, {16, 16});
			TFTensor sums_scanned = tf.allocate("chunk_scan_out", {chunks, (size_t)kHist}, TFTypeUint32);
			tf.dispatch(chunk_scan->kernel_id_, {sums_scanned}, {sums}, {asuint((int)chunks)}, {(size_t)kHist}, {256});
			tf.deallocate(sums);
			TFTensor scan = tf.allocate("group_histogram_scan", {G, (size_t)kHist}, TFTypeUint32);
			tf.dispatch(scan_in_chunks->kernel_id_, {scan}, {hist, sums_scanned}, {asuint((int)G), asuint((int)chunks)}, {chunks, (size_t)kHist}, {16, 16});
			tf.deallocate(hist);
			tf.deallocate(sums_scanned);
			TFTensor total = tf.allocate("total_bit_histogram", {(size_t)kHist}, TFTypeUint32);
			tf.dispatch(totals->kernel_id_, {total}, {scan}, {asuint((int)G)}, {1}, {256});
			tf.dispatch(scatter->kernel_id_, {k_out, v_out}, {k_in, v_in, scan, total}, {asuint(n), asuint((int)G), asuint(pass)}, {G, (size_t)kGroup}, {(size_t)kGroup});
			tf.deallocate(scan);
			tf.deallocate(total);
			tf.region_end("Radix sort iteration");
		}
		tf.deallocate(keys1);
		tf.deallocate(values1);
		tf.region_end("Radix sort");
		TFTensor keys_sorted = tf.allocate("keys_sorted", {N}, key_format);
		tf.dispatch(map_out->kernel_id_, {keys_sorted}, {keys}, {asuint(n)}, {N}, {256});
		tf.deallocate(keys);
		out[0] = keys_sorted;
		out[1] = values;
		return 0;
	};
}

static ProgramRegistrar reg_radix_sort_ir("radix_sort_ir", BuildRadixSortIr);

}  // namespace tfhost
