// TensorFrost/Backend/Backends/HIP/hip_shim_base.h -- the one tree-specific file of the HIP shim: where the backend base
// classes (TFBufferTemplate, TensorMemoryManager: Backend/TensorMemory.h:74-125; KernelManager, Kernel:
// Backend/KernelManager.h:16-30, Compiler/KernelGen.h:17-46) come from and which namespace they live in.
#pragma once
#include "Backend/TensorMemory.h"
#include "Backend/KernelManager.h"
#define TFSHIM_NAMESPACE TensorFrost
#define TFSHIM_FLOAT32 TFTypeFloat32
