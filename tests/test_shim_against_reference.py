"""The HIP shim compiled against the reference's own backend headers (build container only: skipped where the
reference tree is absent).

The files a maintainer adds to a TensorFrost checkout -- tensorfrost_amd/csrc/host/shim/{HIP.h, HIP.cpp,
hip_sort_region.cpp, hip_kernel_info.h} -- are copied beside a four-line hip_shim_base.h that includes
Backend/TensorMemory.h and Backend/KernelManager.h, and every translation unit must pass the compiler's front end:
a drift between this repository's restated base classes and the reference's would show here. A second unit checks
that the C structs of include/tf_abi.h have the layout of the reference's (Backend/TensorMemory.h:19-72)."""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SHIM = ROOT / "tensorfrost_amd" / "csrc" / "host" / "shim"
REFERENCE = Path("/root/reference/TensorFrost")
SHIM_FILES = ["HIP.h", "HIP.cpp", "hip_sort_region.cpp", "hip_kernel_info.h"]

pytestmark = pytest.mark.skipif(not (REFERENCE / "Backend" / "TensorMemory.h").exists() or shutil.which("g++") is None,
                                reason="needs the reference tree and g++ (build container only)")

BASE_HEADER = """#pragma once
#include "Backend/TensorMemory.h"
#include "Backend/KernelManager.h"
#define TFSHIM_NAMESPACE TensorFrost
#define TFSHIM_FLOAT32 TFTypeFloat32
"""


def front_end(tmp_path, source):
    cmd = ["g++", "-std=c++20", "-fsyntax-only", "-Wall", f"-I{tmp_path}", f"-I{REFERENCE}", f"-I{ROOT / 'include'}", str(source)]
    return subprocess.run(cmd, capture_output=True, text=True)


def test_shim_sources_compile_against_the_reference_headers(tmp_path):
    for name in SHIM_FILES:
        shutil.copy(SHIM / name, tmp_path / name)
    (tmp_path / "hip_shim_base.h").write_text(BASE_HEADER)
    for name in [n for n in SHIM_FILES if n.endswith(".cpp")]:
        run = front_end(tmp_path, tmp_path / name)
        assert run.returncode == 0, run.stderr[-4000:]
    # the shim names nothing of this repository's own host tree
    for name in SHIM_FILES:
        text = (SHIM / name).read_text()
        assert "tfhost" not in text and "tf_ir.h" not in text and "tf_backend.h" not in text, name


def test_the_three_classes_derive_from_the_reference_base_classes(tmp_path):
    for name in SHIM_FILES:
        shutil.copy(SHIM / name, tmp_path / name)
    (tmp_path / "hip_shim_base.h").write_text(BASE_HEADER)
    unit = tmp_path / "derive.cpp"
    unit.write_text("""
#include <type_traits>
#include "HIP.h"
using namespace TensorFrost;
static_assert(std::is_base_of<TFBufferTemplate, TFHipBuffer>::value, "TFHipBuffer");
static_assert(std::is_base_of<TensorMemoryManager, HipMemoryManager>::value, "HipMemoryManager");
static_assert(std::is_base_of<KernelManager, HipKernelManager>::value, "HipKernelManager");
static_assert(!std::is_abstract<HipKernelManager>::value, "DispatchKernel is implemented");
// what the InitializeBackend arm of the patch does
TensorMemoryManager* make_memory() { return new HipMemoryManager(); }
KernelManager* make_kernels() { return new HipKernelManager(); }
""")
    run = front_end(tmp_path, unit)
    assert run.returncode == 0, run.stderr[-4000:]


def test_abi_structs_have_the_layout_of_the_reference(tmp_path):
    unit = tmp_path / "abi.cpp"
    fields = {
        "TFBuffer": ["size", "used_size", "time_since_used", "up_to_date", "read_only", "name"],
        "TFDataFormat": ["type", "size"],
        "TFTensor": ["buffer", "format", "dim", "shape"],
        "TFDispatchInfo": ["kernel_id", "read_write_count", "read_write_tensors", "read_only_count", "read_only_tensors", "variable_count", "variables",
                           "work_group_count"],
        "TFRuntime": ["alloc", "dealloc", "readback", "writeback", "dispatch", "region", "custom_data"],
    }
    lines = ['#include <cstddef>', '#include "tf_abi.h"', '#include "Backend/TensorMemory.h"']
    for struct, members in fields.items():
        lines.append(f'static_assert(sizeof(::{struct}) == sizeof(TensorFrost::{struct}), "sizeof {struct}");')
        lines.append(f'static_assert(alignof(::{struct}) == alignof(TensorFrost::{struct}), "alignof {struct}");')
        for member in members:
            lines.append(f'static_assert(offsetof(::{struct}, {member}) == offsetof(TensorFrost::{struct}, {member}), "{struct}::{member}");')
    # the enumerators carry the same values
    for ours, theirs in [("TFType_Float", "Float"), ("TFType_Uint", "Uint"), ("TFType_Int", "Int"), ("TFType_Bool", "Bool"), ("TFType_None", "None")]:
        lines.append(f'static_assert((int)::{ours} == (int)TensorFrost::TFType::{theirs}, "{ours}");')
    unit.write_text("\n".join(lines) + "\n")
    run = front_end(tmp_path, unit)
    assert run.returncode == 0, run.stderr[-4000:]
