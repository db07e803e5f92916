// tf.sort.radix as the reference itself composes it (Python/TensorFrost/sort.py:38-187), kernel by kernel in lowered IR
// form, for a backend that is not tf.cpu (so the scatter kernel is the group-buffer branch, :133-169). Nothing here
// names a primitive: the program dispatches the kernels of sort_composition.cpp inside the `Radix sort` region, which is
// what an unchanged TensorFrost program hands the backend. The kernel manager serves the region with the onesweep sort
// when it is exactly that composition (sort_region.cpp) and runs the kernels as emitted otherwise.
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
//   params[0] = TFType of the keys (default uint); params[1] = bits per pass (sort.py's bits_per_pass, default 6);
//   params[2] = 1: one more dispatch inside the region that sort.py does not have (a copy into values1, which pass 0
//   overwrites), so that the region is no longer the composition the kernel manager knows.
//   inputs keys[N], values[N] (uint).  outputs sorted keys, values.
#include "../sort_composition.h"
#include "registry.h"

namespace tfhost {

static void BuildRadixSortIr(Program* program, const std::vector<int64_t>& params) {
	const int key_type = params.empty() ? TFType_Uint : (int)params[0];
	const int kBits = params.size() > 1 && params[1] > 0 ? (int)params[1] : 6;
	const bool extra_dispatch = params.size() > 2 && params[2] == 1;
	const int kHist = 1 << kBits, kGroup = kSortGroup;
	Kernel* copy = BuildSortKernel(program, SortRole::Copy);
	Kernel* map_in = BuildSortKernel(program, key_type == TFType_Float ? SortRole::MapFloat : key_type == TFType_Int ? SortRole::MapInt : SortRole::Copy);
	Kernel* map_out = BuildSortKernel(program, key_type == TFType_Float ? SortRole::UnmapFloat : key_type == TFType_Int ? SortRole::UnmapInt : SortRole::Copy);
	Kernel* histogram = BuildSortKernel(program, SortRole::Histogram, kBits);
	Kernel* unpack = BuildSortKernel(program, SortRole::Unpack, kBits);
	Kernel* chunk_sums = BuildSortKernel(program, SortRole::ChunkSums, kBits);
	Kernel* chunk_scan = BuildSortKernel(program, SortRole::ChunkScan, kBits);
	Kernel* scan_in_chunks = BuildSortKernel(program, SortRole::ScanInChunks, kBits);
	Kernel* totals = BuildSortKernel(program, SortRole::Totals, kBits);
	Kernel* scatter = BuildSortKernel(program, SortRole::Scatter, kBits);
	// The host part as tracing sort.py:74-187 leaves it: the pass loop is a Python loop, so every pass has its own nodes.
	HostBuilder h(program);
	const TFType key_format = (TFType)key_type;
	h.RegionBegin("Radix sort");
	V keys_in = h.Input("keys", {-1}, key_format);
	V n = h.Shape(keys_in)[0];
	V values_in = h.Input("values", {n}, TFType_Uint);
	V G = (n + h.Const(kGroup - 1)) / h.Const(kGroup), chunks = (G + h.Const(63)) / h.Const(64);
	// keys = tf.copy(keys) (+ map to uint); values = tf.copy(values)
	V keys = h.Allocate("keys", {n}, TFType_Uint), values = h.Allocate("values", {n}, TFType_Uint);
	h.Dispatch(map_in, {keys}, {keys_in}, {n}, {n});
	h.Dispatch(copy, {values}, {values_in}, {n}, {n});
	V keys1 = h.Allocate("keys1", {n}, TFType_Uint), values1 = h.Allocate("values1", {n}, TFType_Uint);
	if (extra_dispatch) h.Dispatch(copy, {values1}, {values_in}, {n}, {n});
	const int iters = (32 + kBits - 1) / kBits;
	for (int pass = 0; pass < iters / 2 * 2; pass++) {
		h.RegionBegin("Radix sort iteration");
		V k_in = (pass & 1) ? keys1 : keys, k_out = (pass & 1) ? keys : keys1;
		V v_in = (pass & 1) ? values1 : values, v_out = (pass & 1) ? values : values1;
		V pass_index = h.Const(pass);
		V packed = h.Allocate("group_histogram_packed", {G, kHist / 4}, TFType_Uint);
		h.Dispatch(histogram, {packed}, {k_in}, {n, G, pass_index}, {G, kHist / 4});
		V hist = h.Allocate("group_histogram", {G, kHist}, TFType_Uint);
		h.Dispatch(unpack, {hist}, {packed}, {G}, {G, kHist});
		h.Deallocate(packed);
		V sums = h.Allocate("chunk_scan", {chunks, kHist}, TFType_Uint);
		h.Dispatch(chunk_sums, {sums}, {hist}, {G, chunks}, {chunks, kHist});
		V sums_scanned = h.Allocate("chunk_scan_out", {chunks, kHist}, TFType_Uint);
		h.Dispatch(chunk_scan, {sums_scanned}, {sums}, {chunks}, {kHist});
		h.Deallocate(sums);
		V scan = h.Allocate("group_histogram_scan", {G, kHist}, TFType_Uint);
		h.Dispatch(scan_in_chunks, {scan}, {hist, sums_scanned}, {G, chunks}, {chunks, kHist});
		h.Deallocate(hist);
		h.Deallocate(sums_scanned);
		V total = h.Allocate("total_bit_histogram", {kHist}, TFType_Uint);
		h.Dispatch(totals, {total}, {scan}, {G}, {1});
		h.Dispatch(scatter, {k_out, v_out}, {k_in, v_in, scan, total}, {n, G, pass_index}, {G, kGroup});
		h.Deallocate(scan);
		h.Deallocate(total);
		h.RegionEnd("Radix sort iteration");
	}
	h.Deallocate(keys1);
	h.Deallocate(values1);
	h.RegionEnd("Radix sort");
	V keys_sorted = h.Allocate("keys_sorted", {n}, key_format);
	h.Dispatch(map_out, {keys_sorted}, {keys}, {n}, {n});
	h.Deallocate(keys);
	h.Output(keys_sorted);
	h.Output(values);
	h.Finish();
}

static ProgramRegistrar reg_radix_sort_ir("radix_sort_ir", BuildRadixSortIr);

}  // namespace tfhost
