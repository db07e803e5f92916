"""Host side without a GPU: C driver surface exports, HIP emitter output, hiprtc acceptance of what it emits."""
import json
import re
from pathlib import Path

import pytest

import tensorfrost_amd.host as tf


@pytest.fixture(scope="module")
def codegen():
    tf.initialize(tf.codegen)
    yield tf
    tf.shutdown()


def test_exports_every_declared_symbol():
    lib = tf.load()
    names = tf.declared_symbols()
    assert len(names) >= 15
    assert not [n for n in names if not hasattr(lib, n)]


def test_wave_eq_emission(codegen):
    prog = tf.compile("wave_eq")
    (k,) = prog.kernels()
    src = k["source"]
    assert k["mapping"] == "flat:vec4" and k["hip_threads"] == 256
    # kernel ABI: buffers (read-write first), then one struct of 32-bit words ending in the block offset
    assert 'extern "C" __global__' in src and f"kernel_{k['kernel_id']}(" in src
    sig = src[src.index('extern "C" __global__'):]
    assert sig.index("v_new_mem") < sig.index("u_new_mem") < sig.index("const uint* __restrict__ u_mem") < sig.index("const uint* __restrict__ v_mem")
    assert "int N;" in src and "int M;" in src and "uint _kernel_block_offset;" in src
    # index contract: index_0 is the innermost (last Python axis), built from block_id and block_thread_id
    assert "int vdiv = block_id / blocks_shape_0;" in src
    assert "int index_0 = ((block_id - (vdiv * blocks_shape_0)) * 16) + block_thread_id0;" in src
    assert "int index_1 = (vdiv * 16) + block_thread_id1;" in src
    assert "bool is_inside_dispatch = (index_0 < var.M) && (index_1 < var.N);" in src
    # loads reinterpret words
    assert "asfloat(u_mem[(index_1 * var.M) + index_0])" in src
    # inside the dispatch guard the clamp of a thread index against its own extent is dropped and the
    # periodic-boundary modulus becomes one conditional subtraction
    body = src[src.index("if (is_inside_dispatch)"):src.index('extern "C" __global__')]
    assert "tf_clamp" not in body and "tf_mod" not in body and "%" not in body
    assert "((index_1 + var.N) - 1) >= var.N ? ((index_1 + var.N) - 1) - var.N : ((index_1 + var.N) - 1)" in body
    # four-wide body, emitted twice: away from the borders all six reads are 16-byte loads (the shifted taps
    # too, since no wrap can happen there); near a border centre, up, down and v rows are 16-byte loads and
    # the left/right taps stay per-element. Both outputs are 16-byte stores in either case.
    vec = src[src.index('extern "C" __global__'):]
    assert "if (is_inside_dispatch_v0 && is_inside_dispatch_v3)" in vec
    interior = vec[vec.index("if (index_0_v0 >= 4 && index_0_v3 + 4 < var.M && index_1 >= 4 && index_1 + 4 < var.N)"):]
    edge = interior[interior.index("\n      else\n"):]
    interior = interior[:interior.index("\n      else\n")]
    assert interior.count("tf_load4(") == 6 and interior.count("tf_store4(") == 2 and "?" not in interior
    assert edge.count("tf_load4(") == 4 and edge.count("tf_store4(") == 2
    assert "sinf(" in src and "asuint(" in src
    prog.destroy()


def test_execution_is_refused_on_codegen_backend(codegen):
    prog = tf.compile("wave_eq")
    with pytest.raises(tf.TFHostError, match="code generation backend|not initialized"):
        prog()
    prog.destroy()


def test_unknown_program_is_an_error(codegen):
    with pytest.raises(tf.TFHostError, match="Unknown program"):
        tf.compile("no_such_program")


def test_whole_kernel_idioms_are_recognised(codegen):
    """Kernels that are exactly one lowered reduction / prefix-sum / matmul loop carry the idiom in their mapping;
    loops with extra arithmetic (the all-pairs force loop) and element-wise kernels do not. Where the primitive does not
    serve them, reductions along the rows run a wave per row and loops down a column sliced among the waves of a group,
    each of the latter with a thread-serial twin for dispatches with enough threads."""
    prog = codegen.compile("lowered_idioms")
    assert [k["mapping"] for k in prog.kernels()] == [
        "reduction:wave+reduce", "reduction:wave+reduce", "reduction:wave+reduce", "reduction:block+reduce", "reduction:block+reduce",
        "reduction:block+reduce", "flat:vec4+scan", "flat:vec4+matmul", "flat:vec4", "flat:vec4", "flat:vec4"]
    prog.destroy()
    for name in ["nbody", "wave_eq", "ops", "atomics", "group_reverse"]:
        prog = codegen.compile(name)
        assert all("+" not in k["mapping"] for k in prog.kernels()), name
        prog.destroy()


def test_pieces_of_a_lowered_softmax_are_recognised(codegen):
    """The sum of exp(x - max) (whole rows, or 128-chunks behind the padding select) and the normalising kernel are
    marked so that the kernel manager can follow the chain; a kernel that only resembles them is not."""
    prog = codegen.compile("softmax_ir")
    assert [k["mapping"] for k in prog.kernels()] == [
        "reduction:wave+reduce", "reduction:wave+reduce", "reduction:wave+expsum", "reduction:wave+reduce", "flat:vec4+normalise"]
    prog.destroy()
    prog = codegen.compile("softmax_ir", [1])
    assert [k["mapping"].partition("+")[2] for k in prog.kernels()] == ["reduce", "expsum", "normalise"]
    prog.destroy()
    prog = codegen.compile("dense_tanh")  # element-wise kernels with loads and one division-free store
    assert all(k["mapping"].partition("+")[2] in ("", "matmul") for k in prog.kernels())
    prog.destroy()


def test_matmul_with_a_general_tail_gets_a_second_kernel_without_the_loop(codegen):
    """dense_tanh has two kernels; each is a matmul loop with an element-wise tail of its own, so each gets a twin:
    same bindings plus the product buffer bound last, no loop, the accumulator read from product[index_1 * N + index_0]."""
    prog = codegen.compile("dense_tanh")
    kernels = prog.kernels()
    assert [k["mapping"] for k in kernels] == ["flat:vec4+matmul", "reduction:wave+matmul", "flat:vec4", "flat:vec4"]
    forward, tail = kernels[0]["source"], kernels[2]["source"]
    assert "const uint* __restrict__ R_mem, const uint* __restrict__ matmul_product_mem, kernel_" in tail
    assert "matmul_product_mem" not in forward
    assert "float matmul = asfloat(matmul_product_mem[(index_1 * var.N) + index_0]);" in tail
    assert "for (int vloop" in forward and "for (int vloop" not in tail
    assert "tanhf(z)" in tail and "Z_mem[" in tail and "H_mem[" in tail
    backward_tail = kernels[3]["source"]
    assert "float matmul = asfloat(matmul_product_mem[(index_1 * var.K) + index_0]);" in backward_tail and "var.scale" in backward_tail
    # kernels whose tail is one of the fused forms stay single
    prog.destroy()
    prog = codegen.compile("dense_layer")
    assert len(prog.kernels()) == 3
    prog.destroy()


def test_int_min_constant_is_a_valid_literal(codegen):
    prog = codegen.compile("atomics")
    assert "asuint((-2147483647 - 1))" in prog.kernels()[0]["source"]
    prog.destroy()


def test_parity_of_the_innermost_index_is_a_literal_per_quad_component(codegen):
    """The Fourier features of the MLP program take sin for even and cos for odd feature indices. In the four-wide
    mapping a quad starts at a multiple of four, so index % 2 is 0, 1, 0, 1 for its components and each component
    calls one of the two functions; the one-thread-per-lane form keeps the test on the index."""
    prog = codegen.compile("mlp")
    source = next(k["source"] for k in prog.kernels() if "sinf(" in k["source"])
    assert "asuint((0 == 0) ? sinf(arg_v0) : cosf(arg_v0)), asuint((1 == 0) ? sinf(arg_v1) : cosf(arg_v1))" in source
    assert "((index_0 % 2) == 0) ? sinf(arg) : cosf(arg)" in source
    prog.destroy()


# ---- the index contract against kernel text the reference itself printed ---------------------------------------

GOLDEN_HEADER = json.loads((Path(__file__).parent / "golden" / "tiled_kernel_index_header.json").read_text())


def _run_header(lines, env):
    """Evaluates `int x = expr;` / `bool x = expr;` lines (C integer arithmetic on non-negative values) in order."""
    env = dict(env)
    for line in lines:
        m = re.fullmatch(r"(?:int|bool) (\w+) = (.*);", line.strip())
        assert m, line
        expr = m.group(2).replace("var.", "var_").replace("&&", " and ").replace("/", "//")
        env[m.group(1)] = eval(expr, {}, env)  # noqa: S307 - fixture text and emitter output, integers only
    return env


def test_index_header_is_the_one_the_reference_printed(codegen):
    """The reference's tiled matrix product is a kernel of shape [N/4, K/4] with 16x16 groups; the kernel text one of
    its runs printed (kept in its matrix_mul notebook) fixes how block_id and the thread ids become index_0 (last
    axis, block_thread_id0), index_1 and the bounds test. The emitter's kernel of the same shape must contain those
    lines verbatim, in order, and evaluate to the same indices for every thread of every group."""
    prog = codegen.compile("tile_indices")
    (k,) = prog.kernels()
    assert k["mapping"] == "group" and k["hip_threads"] == 256
    emitted = [line.strip() for line in k["source"][k["source"].index('extern "C" __global__'):].split("\n")]
    at = 0
    for line in GOLDEN_HEADER["lines"]:
        assert line in emitted[at:], f"missing or out of order: {line}"
        at = emitted.index(line, at) + 1
    assert "local_size_x = 16, local_size_y = 16, local_size_z = 1" in GOLDEN_HEADER["group_declaration"]
    first = emitted.index(GOLDEN_HEADER["lines"][0])
    last = emitted.index(GOLDEN_HEADER["lines"][-1])
    ours = [line for line in emitted[first:last + 1] if re.fullmatch(r"(?:int|bool) \w+ = .*;", line)]
    for n, kk in [(64, 64), (100, 36), (4, 260), (68, 132)]:
        nq, kq = n // 4, kk // 4
        groups = ((kq + 15) // 16) * ((nq + 15) // 16)  # work_group_count, Backend/CodeGen/Langs/CPP.cpp:503-515
        seen = set()
        for block_id in range(groups):
            for t1 in range(16):
                for t0 in range(16):
                    env = {"var_N": n, "var_K": kk, "block_id": block_id, "block_thread_id0": t0, "block_thread_id1": t1}
                    want = _run_header(GOLDEN_HEADER["lines"], env)
                    got = _run_header(ours, env)
                    for name in ("index_0", "index_1", "is_inside_dispatch", "tx", "ty", "gx", "gy"):
                        assert got[name] == want[name]
                    if want["is_inside_dispatch"]:
                        seen.add((want["index_1"], want["index_0"]))
        assert seen == {(i1, i0) for i1 in range(nq) for i0 in range(kq)}  # every element once, none outside
    prog.destroy()


def test_a_kernel_compiled_under_another_number_finds_its_code_object(codegen, tmp_path, monkeypatch):
    """Kernel numbers count up with every program a process compiles, so the same program compiled a second time carries
    other numbers in its source. The compiler is given the kernels under names made from their own text instead: the second
    compilation finds every code object (here in the process; a fresh cache directory also gets its files) and runs no
    compiler, whatever was compiled in between."""
    monkeypatch.setenv("TFHIP_CACHE_DIR", str(tmp_path))
    first = codegen.compile("nbody")
    ids_first = [k["kernel_id"] for k in first.kernels()]
    other = codegen.compile("wave_eq")
    second = codegen.compile("nbody")
    assert [k["kernel_id"] for k in second.kernels()] != ids_first
    assert second.compile_times()["kernel_compile"] < 0.05  # seconds; the compiler alone takes 0.2 s and more per kernel
    names = {p.name for p in tmp_path.glob("*.hsaco")}
    assert names, "no code object reached the cache directory"
    for prog in (first, other, second):
        prog.destroy()
    # a third time leaves the directory as it is: same hashes, nothing new
    third = codegen.compile("nbody")
    assert {p.name for p in tmp_path.glob("*.hsaco")} == names
    third.destroy()
