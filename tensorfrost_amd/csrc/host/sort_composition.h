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

// Builds the kernel of `role` for digits of `bits` bits (sort.py's bits_per_pass; 6 by default) as a new kernel of `program`.
Kernel* BuildSortKernel(Program* program, SortRole role, int bits = 6);

// A hash of the kernel's IR that does not depend on node names: operations, types, constants, argument structure,
// scopes in order, buffers and variables by binding position, group size and dimensionality.
uint64_t KernelFingerprint(const Kernel* kernel);

// The role of a kernel in the composition with the default 6-bit digits, by fingerprint; None for any other kernel.
SortRole SortRoleOf(const Kernel* kernel);

}  // namespace tfhost
