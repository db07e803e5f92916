// HIP (gfx950) kernel emitter: turns one fused IR kernel into the source of one `extern "C" __global__`
// function that libtfhip compiles through hiprtc.
//
// Stands beside the reference's per-language emitters and follows their contract:
//   GenerateCPPKernel   TensorFrost/Backend/CodeGen/Langs/CPP.cpp:720-779
//   GenerateGLSLKernel  TensorFrost/Backend/CodeGen/Langs/GLSL.cpp:146-186
//   CodeGenerator       TensorFrost/Backend/CodeGen/Generators.h:63-200, Generators.cpp:240-540
// i.e. it fills kernel->generated_header_/generated_bindings_/generated_main_/full_generated_code_,
// var_names and var_types, and would be reached from GenerateKernel's language switch
// (Generators.cpp:9-23) through a new CodeGenLang::HIP arm.
#pragma once

#include <functional>
#include <string>
#include <vector>

#include "tf_ir.h"

namespace tfhost {

// Prelude shared by every generated kernel: HIP restatement of the helper functions generated C++
// kernels call (CPP.cpp:31-271) plus the ops the CPU prelude lacks (rsqrt, rcp, frac, step, modf).
std::string GetHIPHeader();

// Emits the kernel. On return kernel->hip_threads / groups_per_hip_block / idiom tell the kernel
// manager how to launch it.
void GenerateHIPKernel(Program* program, Kernel* kernel);

// Emits the kernel (which already has its kernel_id_ and kernel_name_) and whatever further kernels a dispatch of it
// may need: the thread-serial form of a kernel whose loops are split among lanes, and, for a matmul loop with an
// element-wise tail that is none of the fused forms, the tail as a kernel of its own. Also records the kernel's role in
// the tf.sort.radix composition and its whole-kernel idiom. Every further kernel is appended to the program and handed
// to `give_id`, which assigns its kernel_id_ and kernel_name_ (KernelManager::AddKernelID,
// Backend/CodeGen/Langs/CPP.cpp:565-566), before it is emitted. Returns what was emitted, `kernel` first.
std::vector<Kernel*> GenerateHIPKernelFamily(Program* program, Kernel* kernel, const std::function<void(Kernel*)>& give_id);

// What the emitter decided for a kernel, as the table entry the kernel manager dispatches by (HipKernelManager::SetKernelInfo).
HipKernelInfo MakeKernelInfo(const Kernel* kernel);

// Recognises kernels that are exactly one lowered reduction, prefix-sum or matmul loop and records the
// operand bindings, extents and strides in kernel->match (idiom_matcher.cpp).
void MatchKernelIdiom(Kernel* kernel);

// `std::format`-free float literal, same text the reference prints for constants
// (Generators.cpp:160-210): shortest of fixed / scientific with 7 digits, always with '.', 'f' suffix.
std::string FormatFloat(double value);

}  // namespace tfhost
