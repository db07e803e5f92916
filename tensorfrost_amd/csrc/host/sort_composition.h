// The kernels tf.sort.radix lowers to (Python/TensorFrost/sort.py:38-187, the branch for a backend that is not tf.cpu),
// one builder per kernel, in the post-lowering IR form the emitter consumes.
//
// Used by the program that stands in for an unchanged `tf.sort.radix` call (programs/radix_sort_ir.cpp). The kernel
// manager, which follows the dispatches of a `Radix sort` region (sort.py:74,176; delivered through the region
// callback, Backend/Backend.cpp:125-133), does not compare kernels with these: it goes by what AnalyzeSortFeatures
// finds in whatever kernels arrive (sort_features.cpp, shim/hip_sort_region.cpp).
#pragma once

#include <cstdint>

#include "tf_ir.h"

namespace tfhost {

// Other ways the compiler's passes may cut the same composition into kernels (Compiler/Graph/Scope.cpp:5-35,165-188 and
// the fusion of element-wise values into the kernels that load them); each leaves the results unchanged.
constexpr unsigned kSortShiftVariable = 1;  // kernels receive pass * bits_per_pass, evaluated on the host, instead of the pass index
constexpr unsigned kSortInlinedUnpack = 2;  // group_histogram is never stored: chunk sums and the scan in chunks unpack the packed words themselves
constexpr unsigned kSortDigitsBuffer = 4;   // GetBits(keys_in, iter) is a tensor of its own that the histogram kernel loads

// Builds the kernel of `role` for digits of `bits` bits (sort.py's bits_per_pass; 6 by default) as a new kernel of `program`.
Kernel* BuildSortKernel(Program* program, SortRole role, int bits = 6, unsigned variant = 0);
// The two prologue copies as one kernel (key_role: Copy, MapFloat or MapInt), and the digits of a pass as a tensor.
Kernel* BuildFusedCopyKernel(Program* program, SortRole key_role);
Kernel* BuildDigitsKernel(Program* program, int bits, unsigned variant);

// A hash of the kernel's IR that does not depend on node names: operations, types, constants, argument structure,
// scopes in order, buffers and variables by binding position, group size and dimensionality.
uint64_t KernelFingerprint(const Kernel* kernel);

// Fills kernel->sort: the element-wise copies, digit extractions and the scatter form found in the kernel's tree
// (sort_features.cpp). A kernel that has none of them gets an empty record.
void AnalyzeSortFeatures(Kernel* kernel);

}  // namespace tfhost
