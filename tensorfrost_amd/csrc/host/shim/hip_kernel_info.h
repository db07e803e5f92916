// What the HIP kernel manager knows about a kernel when it dispatches it: everything the HIP code generator
// decided while emitting it. Nothing here refers to the compiler's tree, so the kernel manager depends only on
// TensorFrost's backend base classes (Backend/TensorMemory.h, Backend/KernelManager.h) and on this table, which the
// generator fills per kernel id (HipKernelManager::SetKernelInfo).
// (Guarded by a macro, not by `#pragma once`: the generator's side and the kernel manager's side may reach this
// header through two copies of the file.)
#ifndef TFHIP_KERNEL_INFO_H
#define TFHIP_KERNEL_INFO_H

#include <cstddef>
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace tfhip {

// An integer that is known once a dispatch supplies the kernel's variable words: a polynomial over them,
// sum of coef * prod(variables[i]).
struct DimExpr {
	std::vector<std::pair<std::vector<int>, long>> terms;
	long Eval(const uint32_t* variables) const {
		long v = 0;
		for (auto& t : terms) {
			long p = t.second;
			for (int i : t.first) p *= (long)(int)variables[i];
			v += p;
		}
		return v;
	}
};

// A whole kernel recognised as one of the lowered algorithm loops (Compiler/Implementations.cpp:243-359,
// 560-646). The kernel is still emitted; at dispatch the kernel manager evaluates extents and strides and
// hands the work to the hand-written primitive when they describe a dense row-major operand.
struct IdiomMatchInfo {
	enum Kind { None, Reduce, Scan, Matmul, ExpSum, Normalise, ExpDiff, DivideRows } kind = None;  // the last four: pieces of a row softmax, served only as a chain
	std::string op;      // Reduce: "sum" | "max" | "min"; Matmul: "" | "bias" | "bias_relu" | "mask_positive" (fused tail) | "tail" (any other element-wise tail)
	bool is_float = true;  // element type of the operands: float, or a 32-bit integer
	// Binding indices (position in read-write then read-only order) of the operands:
	// Reduce / Scan: {out, in}; Matmul: {C, A, B} and, with a fused tail, the bias / mask.
	std::vector<int> buffers;
	// Reduce / Scan: threads T, trip count K, input strides per thread and per loop step, output stride per
	// thread (Scan: also per loop step; Reduce in a 2-D kernel: then extent, input and output stride of the outer index).  Matmul: extents of the inner / outer thread index (N, M), trip count K,
	// strides of A per (outer, k), B per (k, inner), C per (outer, inner) (no C strides for "tail").
	std::vector<DimExpr> dims;
	// ExpSum: {out, X, maxima}, dims as Reduce followed by the maxima's strides per thread, per loop step [, per outer index].
	// Normalise: {Y, X, maxima, sums}, dims = extents of the inner / outer index, then (inner, outer) strides of X, Y, maxima, sums.
	// ExpDiff (E = exp(X - maxima[row])): {E, X, maxima}; DivideRows (Y = E / sums[row]): {Y, E, sums}; dims as Normalise for the three operands, result second.
	// first <= second must hold for the dispatch's host scalars (e.g. that a clamp in an address is the identity).
	std::vector<std::pair<DimExpr, DimExpr>> conditions;
};

// sort.py:89-91: groups of 128 keys; prefix_sum_grouped scans the group histograms in chunks of 64 groups (:41).
constexpr int kSortGroup = 128;
constexpr int kSortScanChunk = 64;

// The kernels tf.sort.radix lowers to, as the stand-in program builds them (sort_composition.cpp).
enum class SortRole {
	None,
	Copy,          // keys = tf.copy(keys) / values = tf.copy(values)                                   (sort.py:78-80)
	MapFloat,      // the copy fused with map_float_to_uint                                              (:54-60,82-84)
	MapInt,        // the copy fused with map_int_to_uint                                                (:68-69,86-87)
	UnmapFloat,    // map_uint_to_float after the region                                                 (:62-66,178-179)
	UnmapInt,      // map_uint_to_int after the region                                                   (:71-72,181-182)
	Histogram,     // group_histogram_packed = sum of four 8-bit counters per word over a group          (:105-112)
	Unpack,        // group_histogram[g, i]                                                              (:114-115)
	ChunkSums,     // prefix_sum_grouped: tf.sum(grouped, axis + 1)                                      (:42-43)
	ChunkScan,     // prefix_sum_grouped: tf.prefix_sum over the chunk sums                              (:43)
	ScanInChunks,  // prefix_sum_grouped: the scan inside every chunk, seeded, merged                    (:44-49)
	Totals,        // total_bit_histogram = prefix_sum of the last row                                   (:118-119)
	Scatter,       // the group-buffer scatter kernel, keys and values                                   (:133-169)
	ScatterKeys,   // the same without values (has_values == False)
};

// What a kernel does, as far as following a `Radix sort` region needs to know it (sort_features.cpp finds these in
// the kernel's tree; none of them depends on how the compiler's passes cut the program into kernels, on names, or on
// the order of the kernel's variables). Buffers are binding positions (read-write ones first, then read-only ones).
struct SortFeatures {
	// dst[i] = map(src[i]) for every thread i < extent of a one-dimensional kernel. map: 0 the word itself, 1 the
	// order-preserving map from float bits to uint (sort.py:54-60), 2 the one from int (x ^ sign bit, :68-72; it is its
	// own inverse), 3 the map from uint back to float bits (:62-66).
	struct Copy {
		int dst = -1, src = -1, map = 0;
		DimExpr extent;
	};
	std::vector<Copy> copies;
	bool copies_only = false;  // every effect of the kernel is one of `copies`
	// (load(keys, ...) >> shift) & mask occurs in the kernel: it takes a digit of the keys it reads.
	struct Digit {
		int keys = -1;
		DimExpr shift;
		uint32_t mask = 0;
	};
	std::vector<Digit> digits;
	// The scatter of one pass (sort.py:133-169): a kernel with group memory and barriers whose only global effects are
	// keys_out[d] = keys_in[e] (and values_out[d] = values_in[e]) for e = the thread's element < n, d computed from
	// the element's digit (keys_in[e] >> shift) & mask, group memory and the kernel's other read-only buffers.
	bool scatter = false;
	int keys_out = -1, values_out = -1, keys_in = -1, values_in = -1;
	DimExpr scatter_shift, scatter_n;
	uint32_t scatter_mask = 0;
};

struct HipKernelInfo {
	size_t kernel_id = 0;
	size_t tensor_count = 0;    // read-write + read-only buffers bound to the kernel
	size_t variable_count = 0;  // host scalars in its variable block (without the trailing block offset)
	std::vector<int> group_size;  // innermost first, as Node::group_size

	// How the generator mapped the kernel onto the GPU.
	std::string idiom;             // "flat", "flat:vec4", "group", "reduction:wave", "reduction:block", "primitive:<name>"
	int hip_threads = 0;           // threads of one HIP group
	int groups_per_hip_block = 1;  // IR thread-groups covered by one tile
	int hip_blocks_per_tile = 1;   // HIP groups that share one tile (row slabs of the four-wide mapping)
	int lanes_per_thread = 64;     // "reduction:wave": lanes that share one logical thread (64, 32, 16 or 8)
	int threads_per_lane_group = 1;  // "reduction:wave": logical threads a group of lanes works through, one after the other
	bool serial_load_loops = false;  // a thread walks a loop of global loads by itself (neither lanes nor waves share it)
	// "reduction:block" with one loop down the columns: several HIP groups may share a group of 64 threads, one slab of the
	// loop each. The kernel then takes two more pointers behind the tensors (per-slab results, ticket counters) and one
	// more variable word (the number of slabs); slab_trips is the loop's trip count for a dispatch.
	bool slabs = false;
	DimExpr slab_trips;
	int slab_words_per_thread = 0;
	std::string scalar_entry;      // second, one-logical-thread-per-lane entry point of a four-wide kernel ("" if none)
	int scalar_hip_threads = 0;
	int scalar_groups_per_hip_block = 1;
	// Entry point that runs several small dispatches of this kernel in one launch ("" if none): blockIdx.y picks an element
	// of its argument array, `batch_call_bytes` each: the buffer pointers, the variable words, the dispatch's HIP group count.
	std::string batch_entry;
	int batch_capacity = 0, batch_call_bytes = 0;
	size_t read_write_count = 0;  // the first so many bound buffers are written (the others only read)

	// Not emitted at all but served by a primitive of libtfhip.
	std::string primitive;
	size_t primitive_tensors = 0, primitive_variables = 0;

	IdiomMatchInfo match;          // whole-kernel idiom the dispatcher may serve with a primitive instead
	SortFeatures sort;             // what the kernel does, in the terms a `Radix sort` region is followed by
	bool has_tail_kernel = false;  // a matmul loop with an element-wise tail: the tail as a kernel of its own
	size_t tail_kernel_id = 0;
	bool has_dense_variant = false;  // the thread-serial form of a kernel whose loops are split among lanes
	size_t dense_variant_id = 0;
};

}  // namespace tfhip

#endif  // TFHIP_KERNEL_INFO_H
