// tf.sort.radix as the reference itself composes it (Python/TensorFrost/sort.py:38-187), kernel by kernel in lowered IR
// form, for a backend that is not tf.cpu (so the scatter kernel is the group-buffer branch, :133-169). Nothing here
// names a primitive: the program dispatches the kernels of sort_composition.cpp inside the `Radix sort` region, which is
// what an unchanged TensorFrost program hands the backend. The kernel manager serves the region with the onesweep sort
// when its data flow and its kernels' digit / scatter / copy computations show it to be a radix sort over the whole
// key (shim/hip_sort_region.cpp) and runs the kernels as emitted otherwise.
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
//   params[2] = flags. How the compiler's passes cut sort.py into kernels is their decision (Compiler/Graph/Scope.cpp:5-35,
//   165-188); the flags build the same composition cut in other ways, all of which leave the result unchanged:
//       2  the two prologue copies are one kernel (values declared with keys.shape: same shape node, so they fuse)
//       4  kernels receive the shift, pass * bits evaluated on the host, instead of the pass index
//       8  group_histogram is never stored: the chunk sums and the scan in chunks unpack the packed words themselves
//      16  GetBits(keys_in, iter) is a tensor of its own, written by one more kernel, and the histogram kernel loads it
//      32  the two SortIteration calls of a host-loop iteration are separate kernels (14 kernels dispatched 3 times each,
//          as tracing `with tf.loop(iters // 2)` leaves them, instead of 7 dispatched 6 times)
//    and three that are NOT tf.sort.radix (the results are still the sort's, but the region proves less than it must):
//       1  one more dispatch inside the region (a copy into values1, which pass 0 overwrites)
//      64  the first pass's histogram reads the caller's keys instead of the region's copy of them (the same words for
//          uint keys): a kernel of an iteration sees a buffer from outside the region
//     128  the last pass's digit totals stay alive as a third output: a buffer the skipped kernels would have written
//   inputs keys[N], values[N] (uint).  outputs sorted keys, values.
#include "../sort_composition.h"
#include "registry.h"

namespace tfhost {

static void BuildRadixSortIr(Program* program, const std::vector<int64_t>& params) {
	const int key_type = params.empty() ? TFType_Uint : (int)params[0];
	const int kBits = params.size() > 1 && params[1] > 0 ? (int)params[1] : 6;
	const unsigned flags = params.size() > 2 ? (unsigned)params[2] : 0u;
	const bool extra_dispatch = flags & 1, fused_copies = flags & 2, shift_variable = flags & 4, inlined_unpack = flags & 8, digits_buffer = flags & 16,
	           kernels_per_call = flags & 32, outside_read = flags & 64, keep_totals = flags & 128;
	const unsigned variant = (shift_variable ? kSortShiftVariable : 0) | (inlined_unpack ? kSortInlinedUnpack : 0) | (digits_buffer ? kSortDigitsBuffer : 0);
	const int kHist = 1 << kBits, kGroup = kSortGroup;
	const SortRole map_role = key_type == TFType_Float ? SortRole::MapFloat : key_type == TFType_Int ? SortRole::MapInt : SortRole::Copy;
	Kernel* copy = BuildSortKernel(program, SortRole::Copy);
	Kernel* map_in = fused_copies ? BuildFusedCopyKernel(program, map_role) : BuildSortKernel(program, map_role);
	Kernel* map_out = BuildSortKernel(program, key_type == TFType_Float ? SortRole::UnmapFloat : key_type == TFType_Int ? SortRole::UnmapInt : SortRole::Copy);
	struct PassKernels {
		Kernel *digits, *histogram, *unpack, *chunk_sums, *chunk_scan, *scan_in_chunks, *totals, *scatter;
	} set[2];
	for (int k = 0; k < (kernels_per_call ? 2 : 1); k++) {
		set[k].digits = digits_buffer ? BuildDigitsKernel(program, kBits, variant) : nullptr;
		set[k].histogram = BuildSortKernel(program, SortRole::Histogram, kBits, variant);
		set[k].unpack = inlined_unpack ? nullptr : BuildSortKernel(program, SortRole::Unpack, kBits, variant);
		set[k].chunk_sums = BuildSortKernel(program, SortRole::ChunkSums, kBits, variant);
		set[k].chunk_scan = BuildSortKernel(program, SortRole::ChunkScan, kBits, variant);
		set[k].scan_in_chunks = BuildSortKernel(program, SortRole::ScanInChunks, kBits, variant);
		set[k].totals = BuildSortKernel(program, SortRole::Totals, kBits, variant);
		set[k].scatter = BuildSortKernel(program, SortRole::Scatter, kBits, variant);
	}
	if (!kernels_per_call) set[1] = set[0];
	// The host part as tracing sort.py:74-187 leaves it, the pass loop unrolled.
	HostBuilder h(program);
	const TFType key_format = (TFType)key_type;
	h.RegionBegin("Radix sort");
	V keys_in = h.Input("keys", {-1}, key_format);
	V n = h.Shape(keys_in)[0];
	V values_in = h.Input("values", {n}, TFType_Uint);
	V G = (n + h.Const(kGroup - 1)) / h.Const(kGroup), chunks = (G + h.Const(63)) / h.Const(64);
	// keys = tf.copy(keys) (+ map to uint); values = tf.copy(values)
	V keys = h.Allocate("keys", {n}, TFType_Uint), values = h.Allocate("values", {n}, TFType_Uint);
	if (fused_copies) {
		h.Dispatch(map_in, {keys, values}, {keys_in, values_in}, {n}, {n});
	} else {
		h.Dispatch(map_in, {keys}, {keys_in}, {n}, {n});
		h.Dispatch(copy, {values}, {values_in}, {n}, {n});
	}
	V keys1 = h.Allocate("keys1", {n}, TFType_Uint), values1 = h.Allocate("values1", {n}, TFType_Uint);
	if (extra_dispatch) h.Dispatch(copy, {values1}, {values_in}, {n}, {n});
	const int iters = (32 + kBits - 1) / kBits;
	V kept_totals;
	for (int pass = 0; pass < iters / 2 * 2; pass++) {
		const PassKernels& k = set[pass & 1];
		h.RegionBegin("Radix sort iteration");
		V k_in = (pass & 1) ? keys1 : keys, k_out = (pass & 1) ? keys : keys1;
		V v_in = (pass & 1) ? values1 : values, v_out = (pass & 1) ? values : values1;
		V pass_index = h.Const(shift_variable ? pass * kBits : pass);
		V packed = h.Allocate("group_histogram_packed", {G, kHist / 4}, TFType_Uint);
		if (digits_buffer) {
			V digits = h.Allocate("digits", {n}, TFType_Uint);
			h.Dispatch(k.digits, {digits}, {k_in}, {n, pass_index}, {n});
			h.Dispatch(k.histogram, {packed}, {digits}, {n, G}, {G, kHist / 4});
			h.Deallocate(digits);
		} else {
			h.Dispatch(k.histogram, {packed}, {outside_read && pass == 0 ? keys_in : k_in}, {n, G, pass_index}, {G, kHist / 4});
		}
		V hist = packed;
		if (!inlined_unpack) {
			hist = h.Allocate("group_histogram", {G, kHist}, TFType_Uint);
			h.Dispatch(k.unpack, {hist}, {packed}, {G}, {G, kHist});
			h.Deallocate(packed);
		}
		V sums = h.Allocate("chunk_scan", {chunks, kHist}, TFType_Uint);
		h.Dispatch(k.chunk_sums, {sums}, {hist}, {G, chunks}, {chunks, kHist});
		V sums_scanned = h.Allocate("chunk_scan_out", {chunks, kHist}, TFType_Uint);
		h.Dispatch(k.chunk_scan, {sums_scanned}, {sums}, {chunks}, {kHist});
		h.Deallocate(sums);
		V scan = h.Allocate("group_histogram_scan", {G, kHist}, TFType_Uint);
		h.Dispatch(k.scan_in_chunks, {scan}, {hist, sums_scanned}, {G, chunks}, {chunks, kHist});
		h.Deallocate(hist);
		h.Deallocate(sums_scanned);
		V total = h.Allocate("total_bit_histogram", {kHist}, TFType_Uint);
		h.Dispatch(k.totals, {total}, {scan}, {G}, {1});
		h.Dispatch(k.scatter, {k_out, v_out}, {k_in, v_in, scan, total}, {n, G, pass_index}, {G, kGroup});
		h.Deallocate(scan);
		if (keep_totals && pass == iters / 2 * 2 - 1)
			kept_totals = total;
		else
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
	if (keep_totals) h.Output(kept_totals);
	h.Finish();
}

static ProgramRegistrar reg_radix_sort_ir("radix_sort_ir", BuildRadixSortIr);

}  // namespace tfhost
