"""The emitter's side of the drop-in boundary: reading a kernel out of the compiler's own tree.

TensorFrost hands a code generator `Program*, Kernel*` (Backend/CodeGen/Generators.cpp:9-23). Its Kernel
(Compiler/KernelGen.h:17-46) holds the kernel node, binding maps keyed by node address, a set of group memory nodes and
the kernel node's Shape arguments; its Node (Compiler/Graph/Node.h:58-96) is a child / next list with an
ArgumentManager (Compiler/Graph/Arguments.h:44-230). `KernelImporter` (csrc/host/langs/tree_import.h) turns that into
the emitter's own kernel form and `DeriveKernelGeometry` (csrc/host/kernel_geometry.cpp) finds the thread indices, their
extents and the dispatch guard, which the reference's Kernel does not name, in the tree.

Two halves:
  * where the reference tree is present (the build container), the file a maintainer adds as
    TensorFrost/Backend/CodeGen/Langs/HIP.cpp is COMPILED -- not only parsed -- against the reference's own headers,
    laid out beside the shim files as they would lie in that tree; the object must hold the importer instantiated for
    TensorFrost::Node / Kernel and define GenerateHIPKernel(Program*, Kernel*);
  * everywhere, the same importer template is run on a mirror of those classes (tests/programs/compiler_tree_mirror.h)
    filled from every kernel this repository builds -- the five benchmark configurations, the lowered idioms, the sort
    composition, the test programs and the 20 kernels the reference printed -- and the kernel that comes back must be
    emitted to the same text with the same launch decisions. Before that, each kernel's derived fields are stripped
    from a copy and must be found again.
"""
import ctypes
import json
import shutil
import subprocess
from pathlib import Path

import pytest

from conftest import TEST_PROGRAMS

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "tensorfrost_amd" / "csrc"
REFERENCE = Path("/root/reference/TensorFrost")
GOLDEN = ROOT / "tests" / "golden" / "reference_kernel_text.json"

needs_reference = pytest.mark.skipif(not (REFERENCE / "Compiler" / "KernelGen.h").exists() or shutil.which("g++") is None,
                                     reason="needs the reference tree and g++ (build container only)")


def _overlay(tmp_path):
    """The files of the patch in the places they have in a TensorFrost checkout."""
    hip = tmp_path / "Backend" / "Backends" / "HIP"
    langs = tmp_path / "Backend" / "CodeGen" / "Langs"
    hip.mkdir(parents=True)
    langs.mkdir(parents=True)
    for name in ["HIP.h", "HIP.cpp", "hip_sort_region.cpp", "hip_kernel_info.h"]:
        shutil.copy(CSRC / "host" / "shim" / name, hip / name)
    shutil.copy(CSRC / "reference_side" / "Backend" / "Backends" / "HIP" / "hip_shim_base.h", hip / "hip_shim_base.h")
    shutil.copy(CSRC / "reference_side" / "Backend" / "CodeGen" / "Langs" / "HIP.cpp", langs / "HIP.cpp")
    return langs / "HIP.cpp"


@needs_reference
def test_the_generator_arm_compiles_against_the_reference_headers(tmp_path):
    unit = _overlay(tmp_path)
    obj = tmp_path / "HIP.o"
    cmd = ["g++", "-std=c++20", "-c", f"-I{tmp_path}", f"-I{REFERENCE}", f"-I{ROOT / 'include'}", f"-I{CSRC / 'host'}", str(unit), "-o", str(obj)]
    run = subprocess.run(cmd, capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-6000:]
    symbols = subprocess.run(["nm", "-C", str(obj)], capture_output=True, text=True, check=True).stdout
    # the entry points of the patch, with the reference's own types in their signatures
    assert " T TensorFrost::GenerateHIPKernel(TensorFrost::Program*, TensorFrost::Kernel*)" in symbols
    assert " T TensorFrost::CompileHIPKernel(TensorFrost::Program*, TensorFrost::Kernel*)" in symbols
    # the importer, instantiated for the compiler's classes
    assert "tfhost::KernelImporter<TensorFrost::CompilerTree>::Import(TensorFrost::Kernel const*)" in symbols
    assert "tfhost::KernelImporter<TensorFrost::CompilerTree>::Wire(TensorFrost::Node const*)" in symbols
    # it calls the emitter and nothing of this repository's restated managers
    assert " U tfhost::GenerateHIPKernelFamily(" in symbols and " U tfhost::DeriveKernelGeometry(tfhost::Kernel*)" in symbols
    assert "tfhost::TensorMemoryManager" not in symbols and "tfhost::KernelManager" not in symbols


@needs_reference
def test_the_mirror_offers_nothing_the_reference_classes_lack(tmp_path):
    """Every member the importer template touches, asked of the reference's classes with the mirror's signatures."""
    unit = tmp_path / "members.cpp"
    unit.write_text("""
#include <type_traits>
#include "Compiler/KernelGen.h"
using namespace TensorFrost;
template <class T> using bare = std::remove_cv_t<std::remove_reference_t<T>>;
void members(const Node* n, const Kernel* k) {
    static_assert(std::is_same_v<decltype(n->child), Node*> && std::is_same_v<decltype(n->next), Node*> && std::is_same_v<decltype(n->parent), Node*>);
    static_assert(std::is_same_v<bare<decltype(n->op->name_)>, std::string>);
    static_assert(std::is_same_v<bare<decltype(n->data)>, std::vector<uint>>);
    static_assert(std::is_same_v<bare<decltype(n->group_size)>, std::vector<int>>);
    static_assert(std::is_same_v<bare<decltype(n->debug_name)>, std::string> && std::is_same_v<bare<decltype(n->var_name)>, std::string>);
    static_assert(std::is_same_v<decltype(n->format.type), TFType>);
    static_assert(std::is_same_v<decltype(n->flags.has(NodeProp::Modified)), bool>);
    static_assert(std::is_same_v<decltype(n->flags.has(NodeProp::LocalMemoryOp)), bool>);
    static_assert(std::is_same_v<decltype(n->flags.has(NodeProp::Placeholder)), bool>);
    static_assert(std::is_same_v<decltype(n->args.Get(ArgType::Input, 0)), Node*>);
    static_assert(std::is_same_v<decltype(n->args.Has(ArgType::Memory, 0)), bool>);
    static_assert(std::is_same_v<decltype(n->args.Count(ArgType::Index)), int>);
    static_assert(std::is_same_v<decltype(n->args.OutputCount()), size_t>);
    static_assert(std::is_same_v<bare<decltype(k->variables)>, std::map<Node*, size_t>>);
    static_assert(std::is_same_v<bare<decltype(k->read_write_memory)>, std::map<Node*, size_t>>);
    static_assert(std::is_same_v<bare<decltype(k->read_only_memory)>, std::map<Node*, size_t>>);
    static_assert(std::is_same_v<bare<decltype(k->group_memory)>, std::set<Node*>>);
    static_assert(std::is_same_v<bare<decltype(k->shape)>, std::map<std::pair<ArgType, int>, Node*>>);
    static_assert(std::is_same_v<decltype(k->root), Node*>);
    // the enumerators the mirror numbers
    static_assert((int)ArgType::Input == 0 && (int)ArgType::Index == 1 && (int)ArgType::Shape == 2 && (int)ArgType::Memory == 3);
    static_assert((int)NodeProp::Placeholder == 0 && (int)NodeProp::Modified == 1 && (int)NodeProp::LocalMemoryOp == 16);
    // element types carry over by value
    static_assert((int)TFType::Float == 0 && (int)TFType::Uint == 1 && (int)TFType::Int == 2 && (int)TFType::Bool == 3 && (int)TFType::None == 4);
}
""")
    run = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", f"-I{REFERENCE}", str(unit)], capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-4000:]


@pytest.fixture(scope="module")
def lib():
    import tensorfrost_amd.host  # noqa: F401  (loads libtfhost, which the test library links against)
    handle = ctypes.CDLL(str(TEST_PROGRAMS), mode=ctypes.RTLD_GLOBAL)
    handle.tftest_import_roundtrip_program.restype = ctypes.c_long
    handle.tftest_import_roundtrip_program.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t]
    handle.tftest_roundtrip_kernel_text.restype = ctypes.c_long
    handle.tftest_roundtrip_kernel_text.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    handle.tftest_import_defect.restype = ctypes.c_long
    handle.tftest_import_defect.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    return handle


# (program, parameters, least number of emitted kernels): the five benchmark configurations first
PROGRAMS = [
    ("wave_eq", [], 1),                  # config 1
    ("reductions_ir", [], 8),            # config 2: sum / max along both axes as split reductions
    ("reductions_ir", [1], 4),
    ("softmax_ir", [], 5),               # config 2: the five-kernel softmax
    ("softmax_ir", [1], 3),
    ("softmax_ir", [8], 5),
    ("softmax_ir", [8 | 16], 5),
    ("radix_sort_ir", [1], 9),           # config 3: the tf.sort.radix composition, uint / int / float keys
    ("radix_sort_ir", [2], 9),
    ("radix_sort_ir", [0], 9),
    ("nbody", [], 1),                    # config 4
    ("mlp", [], 8),                      # config 5: named primitives + element-wise kernels
    ("mlp", [2], 15),                    # config 5: every product and sum a lowered loop
    ("mlp", [1], 8),
    ("tiled_matmul_ir", [], 1),
    ("ops", [], 1),
    ("bitonic_sort", [], 1),
    ("autograd_network_forward", [], 9),
    ("split_merge", [], 2),
    ("qr_inversion", [], 10),
    ("gathered_updates", [], 1),
    ("reshape_reduction", [], 1),
    ("integer_reductions", [], 1),
    ("radix_scatter_pass", [0], 1),
    ("dense_layer", [], 1),
    ("dense_tanh", [], 1),
    ("batched_matmul", [], 1),
    ("indexing", [3], 1),
    ("indexing", [4], 1),
    ("broadcast_loops", [], 1),
    ("atomics", [], 1),
    ("group_reverse", [], 1),
    ("tile_indices", [], 1),
    ("lowered_idioms", [], 1),
]


@pytest.mark.parametrize("name,params,least", PROGRAMS, ids=[f"{n}{p}" for n, p, _ in PROGRAMS])
def test_kernels_survive_the_compiler_classes_and_back(lib, name, params, least):
    out = ctypes.create_string_buffer(1 << 16)
    arr = (ctypes.c_int64 * max(1, len(params)))(*params)
    checked = lib.tftest_import_roundtrip_program(name.encode(), arr, len(params), out, len(out))
    assert checked >= 0, out.value.decode()
    assert checked >= least, f"{name}: only {checked} kernels were checked"


def _golden_kernels():
    return json.loads(GOLDEN.read_text())["kernels"]


@pytest.mark.parametrize("verbatim", [1, 0], ids=["verbatim", "as_any_kernel"])
def test_printed_kernels_survive_the_compiler_classes_and_back(lib, verbatim):
    kernels = _golden_kernels()
    assert len(kernels) == 20
    for kernel in kernels:
        out = ctypes.create_string_buffer(1 << 16)
        status = lib.tftest_roundtrip_kernel_text("\n".join(kernel["body"]).encode(), (ctypes.c_int * 3)(*kernel["group_size"]),
                                                  "\n".join(kernel["shared"]).encode(), verbatim, out, len(out))
        assert status == 0, f"{kernel['from']}: {out.value.decode()}"


@pytest.mark.parametrize("defect,expected", [
    (0, "IR Operation not defined: dim_id"),
    (1, "Index arguments (memory indexing not finalised)"),
    (2, "neither inside the kernel nor bound to it"),
    (3, "slots of read_write_memory are not 0..n-1"),
    (4, "group extent of 256 but the kernel node says 64"),
])
def test_trees_that_are_not_in_post_lowering_form_are_refused(lib, defect, expected):
    out = ctypes.create_string_buffer(4096)
    status = lib.tftest_import_defect(defect, out, len(out))
    assert status == 0, out.value.decode()
    assert expected in out.value.decode()
