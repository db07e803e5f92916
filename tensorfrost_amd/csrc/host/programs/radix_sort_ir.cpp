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
		if (extra_dispatch) tf.dispatch(copy->kernel_id_, {values1}, {in[1]}, {asuint(n)}, {N}, {256});
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
