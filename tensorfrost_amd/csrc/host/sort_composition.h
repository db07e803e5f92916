// The kernels tf.sort.radix lowers to (Python/TensorFrost/sort.py:38-187, the branch for a backend that is not tf.cpu),
// one builder per kernel, in the post-lowering IR form the emitter consumes.
//
// Two users: the program that stands in for an unchanged `tf.sort.radix` call (programs/radix_sort_ir.cpp), and the
// kernel manager, which follows the dispatches of a `Radix sort` region (sort.py:74,176; delivered through the region
// callback, Backend/Backend.cpp:125-133) and serves the whole region with the onesweep sort when every kernel in it is
// structurally one of these (sort_region.cpp).
#pragma once

#include <cstdint>

#include "tf_ir.h"

namespace tfhost {

// sort.py:89-91: groups of 128 keys; prefix_sum_grouped scans the group histograms in chunks of 64 groups (:41).
constexpr int kSortGroup = 128;
constexpr int kSortScanChunk = 64;

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

// Builds the kernel of `role` for digits of `bits` bits (sort.py's bits_per_pass; 6 by default) as a new kernel of `program`.
Kernel* BuildSortKernel(Program* program, SortRole role, int bits = 6);

// A hash of the kernel's IR that does not depend on node names: operations, types, constants, argument structure,
// scopes in order, buffers and variables by binding position, group size and dimensionality.
uint64_t KernelFingerprint(const Kernel* kernel);

// The role of a kernel in the composition with the default 6-bit digits, by fingerprint; None for any other kernel.
SortRole SortRoleOf(const Kernel* kernel);

}  // namespace tfhost
