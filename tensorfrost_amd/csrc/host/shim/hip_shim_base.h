// The one tree-specific file of the HIP shim: where the backend base classes come from. In a TensorFrost checkout
// this file reads
//     #include "Backend/TensorMemory.h"
//     #include "Backend/KernelManager.h"
//     #define TFSHIM_NAMESPACE TensorFrost
//     #define TFSHIM_FLOAT32 TFTypeFloat32
// Here the base classes are this repository's restatements.
#pragma once

#include "../tf_kernel_manager.h"
#include "../tf_memory.h"

#define TFSHIM_NAMESPACE tfhost
#define TFSHIM_FLOAT32 (TFDataFormat{TFType_Float, 32})
