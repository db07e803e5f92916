"""The emitter against kernel text that the reference itself printed.

tests/golden/reference_kernel_text.json holds 20 kernels as runs of the reference printed them after all of its passes
(four notebooks; extracted by tests/golden/extract_kernel_text.py). Each one is parsed back into a kernel tree with
KernelBuilder (tests/programs/kernel_text.cpp: one node per printed operator, call, load, store, loop ...), emitted by
the HIP emitter with its range-based simplifications switched off, and the emitted body has to equal the printed body
statement for statement. That pins, against text the reference produced: the operation table and its spellings, the
statement forms (declaration, set, store, atomics, loop, if, break / continue, barrier), which values are written
out where they are used and which keep a line of their own, parenthesisation, constants, and the order of statements.

What counts as equal (the GLSL -> HIP token map):
  * spellings:  clamp min max abs sign mix smoothstep fract -> tf_clamp tf_min tf_max tf_abs tf_sign tf_lerp tf_smoothstep
    tf_frac;  sin cos exp floor pow sqrt ... -> sinf cosf expf floorf powf tf_sqrt ...;  bitfieldReverse -> reversebits;
    mod(a, b) -> fmodf(a, b);  barrier() -> group_barrier();  a / b on floats -> tf_div(a, b);  a % b -> tf_mod(a, b)
  * casts:  T(x) -> ((T)(x))
  * constants by value:  0.f, 0.3f, -6.2831854820251465f  ==  0.0f, 0.300000012f, -6.28318548f  (same float32)
  * stores write a word:  X_mem[a] = asuint(v)  ==  X_mem[a] = v  when v is a uint already
  * atomics:  atomicAdd(X_mem[a], uint(v))  ==  InterlockedAdd((T*)X_mem, a, v)
  * group arrays:  `//float t[n]` at the array's place in the tree  ==  `// float t[n] (declared as __shared__ above)`
  * the 100-character rule: the reference writes an unnamed single-use value out at its use unless the printed
    expression is 100 characters or longer (Generators.h:90-124); lengths differ between the two languages, so a
    value that only one side kept on a line of its own (named v<operation>[_n]) is substituted into its single use
    before comparing, provided nothing is assigned, stored or synchronised in between; the reference also writes an
    unnamed single-use load out at its use, the emitter keeps every load on its own line
  * v<operation>_<n>, the name of a value without one, carries each generator's own count n: such names are compared
    by the order of their declarations
Everything else -- names, types, operators, nesting, order -- has to be identical."""
import ctypes
import json
import re
import struct
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
FIXTURE = ROOT / "tests" / "golden" / "reference_kernel_text.json"
KERNELS = json.loads(FIXTURE.read_text())["kernels"]

FUNCTIONS = {  # emitted spelling -> the reference's GLSL spelling
    "tf_clamp": "clamp", "tf_min": "min", "tf_max": "max", "tf_abs": "abs", "tf_sign": "sign", "tf_lerp": "mix", "tf_smoothstep": "smoothstep",
    "tf_frac": "fract", "tf_step": "step", "tf_sqrt": "sqrt", "tf_rsqrt": "inversesqrt", "tf_rcp": "rcp", "fmodf": "mod", "reversebits": "bitfieldReverse",
    "expf": "exp", "exp2f": "exp2", "logf": "log", "log2f": "log2", "sinf": "sin", "cosf": "cos", "tanf": "tan", "asinf": "asin", "acosf": "acos",
    "atanf": "atan", "atan2f": "atan", "sinhf": "sinh", "coshf": "cosh", "tanhf": "tanh", "powf": "pow", "ceilf": "ceil", "floorf": "floor", "roundf": "round", "fmaf": "fma",
}
OPERATOR_CALLS = {"tf_div": "/", "tf_mod": "%"}
ATOMICS = {"atomicAdd": "InterlockedAdd", "atomicMin": "InterlockedMin", "atomicMax": "InterlockedMax", "atomicAnd": "InterlockedAnd", "atomicOr": "InterlockedOr", "atomicXor": "InterlockedXor"}
TYPES = ("float", "int", "uint", "bool")
OPERATIONS = ("add sub mul div mod lshift rshift and or xor eq neq lt lte gt gte notb not neg uint int float bool asuint asint asfloat asbool min max abs sign ceil floor "
              "round frac exp exp2 log log2 sqrt rsqrt rcp sin cos tan asin acos atan sinh cosh tanh pcg reversebits pcgf pow atan2 modf step clamp lerp fma smoothstep "
              "ternary const copy load").split()
AUTO_NAME = re.compile(r"^v(" + "|".join(OPERATIONS) + r")(_\d+)?$")

TOKEN = re.compile(r"\s*(?:(0[xX][0-9a-fA-F]+u?|(?:\d+\.\d*|\.\d+|\d+)(?:[eE][+-]?\d+)?[fu]?)|([A-Za-z_]\w*)|(<<|>>|<=|>=|==|!=|&&|\|\||\+=|[-+*/%<>=!~&|^?:()\[\],.;{}]))")


def tokens(text):
    out, at = [], 0
    text = text.rstrip()
    while at < len(text):
        m = TOKEN.match(text, at)
        if not m:
            raise ValueError(f"cannot tokenise {text[at:]!r}")
        out.append(("num", m.group(1)) if m.group(1) else ("id", m.group(2)) if m.group(2) else ("op", m.group(3)))
        at = m.end()
    return out


def number(text):
    if text.lower().startswith("0x"):
        return ("uint" if text.endswith("u") else "int", int(text.rstrip("u"), 16))
    if text.endswith("f") or "." in text or "e" in text.lower():
        return ("float", struct.unpack("f", struct.pack("f", float(text.rstrip("f"))))[0])
    if text.endswith("u"):
        return ("uint", int(text[:-1]))
    return ("int", int(text))


class Expr:
    """Precedence-climbing parser of the expression language both generators print; the result is a nested tuple in
    which redundant parentheses are gone and every spelling is the reference's."""
    LEVELS = [["||"], ["&&"], ["|"], ["^"], ["&"], ["==", "!="], ["<", "<=", ">", ">="], ["<<", ">>"], ["+", "-"], ["*", "/", "%"]]

    def __init__(self, toks):
        self.t, self.i = toks, 0

    def peek(self, k=0):
        return self.t[self.i + k] if self.i + k < len(self.t) else ("end", "")

    def take(self, text=None):
        tok = self.peek()
        if text is not None and tok[1] != text:
            raise ValueError(f"expected {text!r}, found {tok[1]!r}")
        self.i += 1
        return tok

    def ternary(self):
        c = self.binary(0)
        if self.peek()[1] == "?":
            self.take()
            a = self.ternary()
            self.take(":")
            return ("?:", c, a, self.ternary())
        return c

    def binary(self, level):
        if level == len(self.LEVELS):
            return self.unary()
        left = self.binary(level + 1)
        while self.peek()[0] == "op" and self.peek()[1] in self.LEVELS[level]:
            op = self.take()[1]
            left = (op, left, self.binary(level + 1))
        return left

    def unary(self):
        kind, text = self.peek()
        if kind == "op" and text in "-!~":
            self.take()
            if text == "-" and self.peek()[0] == "num":
                t, v = number(self.take()[1])
                return ("const", t, -v)
            return ("unary" + text, self.unary())
        return self.primary()

    def primary(self):
        kind, text = self.take()
        if kind == "num":
            return ("const",) + number(text)
        if kind == "op" and text == "(":
            # ((T)(x)): the emitted cast
            if self.peek()[1] == "(" and self.peek(1)[1] in TYPES and self.peek(2)[1] == ")":
                self.take()
                t = self.take()[1]
                self.take(")")
                self.take("(")
                x = self.ternary()
                self.take(")")
                self.take(")")
                return ("cast", t, x)
            if self.peek()[1] in TYPES and self.peek(1)[1] == "*" and self.peek(2)[1] == ")":  # (T*)X_mem in an atomic
                self.take(), self.take(), self.take()
                return self.primary()
            e = self.ternary()
            self.take(")")
            return e
        if kind != "id":
            raise ValueError(f"unexpected {text!r}")
        if text == "var" and self.peek()[1] == ".":
            self.take()
            return ("var", self.take()[1])
        if self.peek()[1] == "[":
            self.take()
            a = self.ternary()
            self.take("]")
            return ("index", text, a)
        if self.peek()[1] == "(":
            self.take()
            args = []
            if self.peek()[1] != ")":
                args.append(self.ternary())
                while self.peek()[1] == ",":
                    self.take()
                    args.append(self.ternary())
            self.take(")")
            if text in TYPES:
                return ("cast", text, args[0])
            if text in OPERATOR_CALLS:
                return (OPERATOR_CALLS[text], args[0], args[1])
            if text == "tf_stream_load":  # tf_stream_load(X_mem + (a)) reads X_mem[a]
                assert args[0][0] == "+" and args[0][1][0] == "name"
                return ("index", args[0][1][1], args[0][2])
            return ("call", FUNCTIONS.get(text, text)) + tuple(args)
        if text in ("true", "false"):
            return ("const", "bool", text == "true")
        return ("name", text)


def expression(text):
    p = Expr(tokens(text))
    e = p.ternary()
    if p.peek()[0] != "end":
        raise ValueError(f"trailing {p.peek()[1]!r} in {text!r}")
    return e


def statements(lines):
    """One tuple per line: ('decl', type, name, e) | ('set', name, e) | ('store', array, address, e) | ('atomic', op, buffer,
    address, e[, type, name]) | ('for', v, a, b, s) | ('if', e) | ('{',) | ('}',) | ('break',) | ('continue',) | ('barrier',) |
    ('array', type, name, size)."""
    out = []
    for raw in lines:
        line = raw.strip()
        m = re.match(r"^//\s*(float|int|uint|bool) (\w+)\[(\d+)\]", line)
        if m:
            out.append(("array", m.group(1), m.group(2), int(m.group(3))))
            continue
        line = line.split("//")[0].strip()
        if not line:
            continue
        if line in ("{", "}"):
            out.append((line,))
        elif line in ("break;", "continue;"):
            out.append((line[:-1],))
        elif line in ("barrier();", "group_barrier();"):
            out.append(("barrier",))
        elif line.startswith("for ("):
            m = re.match(r"^for \(int (\w+) = (.*); \1 < (.*); \1 \+= (.*)\)$", line)
            out.append(("for", m.group(1), expression(m.group(2)), expression(m.group(3)), expression(m.group(4))))
        elif line.startswith("if ("):
            out.append(("if", expression(line[3:])))
        else:
            assert line.endswith(";"), line
            line = line[:-1]
            decl = re.match(r"^(float|int|uint|bool) (\w+) = (.*)$", line)
            target, value = (decl.group(2), decl.group(3)) if decl else (None, line)
            atomic = re.match(r"^(?:(?:float|int|uint)\()?(atomic\w+|Interlocked\w+)\((.*?)\)?$", value)
            if atomic and (atomic.group(1) in ATOMICS or atomic.group(1).startswith(("Interlocked", "atomicAdd_"))):
                call = expression(value)
                if call[0] == "cast":
                    call = call[2]
                name, args = call[1], call[2:]
                if name in ATOMICS:  # atomicOp(X_mem[a], uint(v))
                    op, (buffer, address), v = ATOMICS[name], args[0][1:], args[1][2]
                elif name.startswith("atomicAdd_"):  # atomicAdd_X_mem(a, v)
                    op, buffer, address, v = "InterlockedAdd", name[len("atomicAdd_"):], args[0], args[1]
                else:  # InterlockedOp((T*)X_mem, a, v)
                    op, buffer, address, v = name.replace("_Prev", ""), args[0][1], args[1], args[2]
                out.append(("atomic", op, buffer, address, v) + ((decl.group(1), target) if decl else ()))
            elif decl:
                out.append(("decl", decl.group(1), target, expression(value)))
            else:
                lhs, rhs = value.split(" = ", 1)
                if "[" in lhs:
                    cell, e = expression(lhs), expression(rhs)
                    if cell[1].endswith("_mem") and e[0] == "call" and e[1] == "asuint":
                        e = e[2]
                    out.append(("store", cell[1], cell[2], e))
                else:
                    out.append(("set", lhs.strip(), expression(rhs)))
    return out


def names_in(e, acc):
    if isinstance(e, tuple):
        if e and e[0] == "name":
            acc.append(e[1])
        for x in e[1:]:
            names_in(x, acc)
    return acc


def reads_memory(e):
    return isinstance(e, tuple) and (e[:1] == ("index",) or any(reads_memory(x) for x in e[1:]))


def substitute(e, name, value):
    if not isinstance(e, tuple):
        return e
    if e[:2] == ("name", name):
        return value
    return tuple(substitute(x, name, value) for x in e)


def fold_short_lived_values(stmts):
    """The 100-character rule: a value named v<operation>[_n] that is used exactly once, in the same block, with nothing
    assigned, stored or synchronised between its line and its use, is written out at that use."""
    stmts = list(stmts)
    changed = True
    while changed:
        changed = False
        uses = {}
        for s in stmts:
            for x in s[1:]:
                for n in names_in(x, []):
                    uses[n] = uses.get(n, 0) + 1
        for i, s in enumerate(stmts):
            if s[0] != "decl" or not AUTO_NAME.match(s[2]) or uses.get(s[2], 0) != 1 :
                continue
            for j in range(i + 1, len(stmts)):
                t = stmts[j]
                if s[2] in names_in(t[1:], []):
                    stmts[j] = tuple(substitute(x, s[2], s[3]) if k else x for k, x in enumerate(t))
                    del stmts[i]
                    changed = True
                    break
                if t[0] in ("set", "store", "atomic", "barrier", "{", "}", "for", "break", "continue"):
                    break
            if changed:
                break
    return stmts


def number_unnamed_values(stmts):
    """Values without a name of their own are numbered by each generator's own count: v<operation>_<n> becomes
    v<operation>#<k>, k counting the declarations of such names in order."""
    renamed = {}
    for s in stmts:
        if s[0] == "decl" and AUTO_NAME.match(s[2]):
            renamed[s[2]] = f"{AUTO_NAME.match(s[2]).group(1)}#{len(renamed)}"

    def walk(e):
        if not isinstance(e, tuple):
            return e
        if e[:1] == ("name",) and e[1] in renamed:
            return ("name", renamed[e[1]])
        return tuple(walk(x) for x in e)

    out = []
    for s in stmts:
        if s[0] == "decl":
            out.append((s[0], s[1], renamed.get(s[2], s[2]), walk(s[3])))
        elif s[0] == "set":
            out.append((s[0], renamed.get(s[1], s[1]), walk(s[2])))
        else:
            out.append(tuple(walk(x) if k else x for k, x in enumerate(s)))
    return out


def emitted_body(source):
    """The statements of the emitted kernel that stand for the kernel's tree: the body of the one-thread function
    (kernels without group memory) or of the kernel itself behind the lines that name block_id / block_thread_id."""
    lines = source.split("\n")
    thread = next((i for i, l in enumerate(lines) if l.startswith("static __device__ __forceinline__ void kernel_0_thread(")), None)
    if thread is not None:
        end = lines.index("}", thread)
        return lines[thread + 2:end], []
    start = next(i for i, l in enumerate(lines) if l.startswith('extern "C" __global__'))
    shared = [l.strip() for l in lines[start:] if l.strip().startswith("__shared__")]
    first = next(i for i, l in enumerate(lines) if l.strip() == "{" and i > start + 1)
    last = max(i for i, l in enumerate(lines) if l == "  }")
    return lines[first + 1:last], shared


@pytest.fixture(scope="module")
def emit():
    import tensorfrost_amd.host  # noqa: F401  (loads libtfhost, which the test library links against)
    from conftest import TEST_PROGRAMS

    lib = ctypes.CDLL(str(TEST_PROGRAMS), mode=ctypes.RTLD_GLOBAL)
    fn = lib.tftest_emit_kernel_text
    fn.restype = ctypes.c_long
    fn.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]

    def run(kernel):
        out = ctypes.create_string_buffer(1 << 20)
        n = fn("\n".join(kernel["body"]).encode(), (ctypes.c_int * 3)(*kernel["group_size"]), "\n".join(kernel["shared"]).encode(), out, len(out))
        text = out.value.decode()
        if n < 0:
            raise RuntimeError(text)
        return text

    return run


def test_fixture_holds_the_kernels_of_the_four_notebooks():
    sources = [k["from"].split(",")[0] for k in KERNELS]
    assert sources.count("examples/Algorithms/matrix_mul.ipynb") == 1
    assert sources.count("examples/Algorithms/fft_group.ipynb") == 1
    assert sources.count("examples/Rendering/buddhabrot.ipynb") == 4
    assert sources.count("examples/Simulation/fluid_simulation.ipynb") == 14
    assert sum(len(k["body"]) for k in KERNELS) > 1100


def test_expression_reader_tells_different_expressions_apart():
    same = [("(a * b) + c", "a * b + c"), ("float(x) / 2.0f", "tf_div(((float)(x)), 2.0f)"), ("0.3f * t", "0.300000012f * t"), ("clamp(i, 0, n - 1)", "tf_clamp(i, 0, n - 1)"),
            ("asfloat(X_mem[i])", "asfloat(tf_stream_load(X_mem + (i)))"), ("(l < 60) ? 2 : ((l < 200) ? 1 : 0)", "l < 60 ? 2 : (l < 200 ? 1 : 0)")]
    for a, b in same:
        assert expression(a) == expression(b), (a, b)
    different = [("a * (b + c)", "(a * b) + c"), ("a - (b - c)", "(a - b) - c"), ("a / b", "b / a"), ("0.3f", "0.30000004f"), ("int(x)", "uint(x)"), ("min(a, b)", "max(a, b)"),
                 ("x >> 22", "x >> 23"), ("a < b", "a <= b"), ("-x", "x")]
    for a, b in different:
        assert expression(a) != expression(b), (a, b)


@pytest.mark.parametrize("index", range(len(KERNELS)), ids=[f"{Path(k['from'].split(',')[0]).stem}-{k['from'].rsplit(' ', 1)[1]}" for k in KERNELS])
def test_emitted_statements_equal_the_printed_ones(emit, index):
    kernel = KERNELS[index]
    body, shared = emitted_body(emit(kernel))
    want = number_unnamed_values(fold_short_lived_values(statements(kernel["body"])))
    got = number_unnamed_values(fold_short_lived_values(statements(body)))
    for k, (w, g) in enumerate(zip(want, got)):
        assert w == g, f"statement {k}:\n  printed by the reference: {w}\n  emitted:                  {g}"
    assert len(want) == len(got)
    # group arrays: same element type, name and length
    declared = sorted(re.match(r"shared (\w+) (\w+)\[(\d+)\];", s).groups() for s in kernel["shared"])
    assert sorted(re.match(r"__shared__ (\w+) (\w+)\[(\d+)\];", s).groups() for s in shared) == declared


MUTATIONS = [  # (kernel, printed text, replacement): each changes what the kernel computes
    (7, "((vx - vx_2) + vy) - vy_2", "((vx - vx_2) - vy) + vy_2"),
    (7, "clamp(index_1 + 1, 0, var.N1 - 1)", "clamp(index_1 + 1, 0, var.N1 - 2)"),
    (3, "z_re = z_re_new;\n      z_im = z_im_new;", "z_im = z_im_new;\n      z_re = z_re_new;"),
    (3, "l >= 3000", "l > 3000"),
    (1, ">> 22", ">> 21"),
    (0, "A_group_tile[(tx * 64) + k]", "A_group_tile[(k * 64) + tx]"),
]


@pytest.mark.parametrize("index,old,new", MUTATIONS)
def test_a_changed_kernel_is_told_apart(emit, index, old, new):
    kernel = dict(KERNELS[index])
    text = "\n".join(kernel["body"])
    assert text.count(old) >= 1
    kernel["body"] = text.replace(old, new, 1).split("\n")
    body, _ = emitted_body(emit(kernel))
    want = number_unnamed_values(fold_short_lived_values(statements(KERNELS[index]["body"])))
    got = number_unnamed_values(fold_short_lived_values(statements(body)))
    assert want != got


def test_emitted_kernels_compile_for_gfx950(emit):
    """Every one of the 20 kernels, as emitted from the parsed tree, builds with hiprtc (no device needed)."""
    from tensorfrost_amd._lib import load as tfhip

    compile_fn = tfhip().tfhip_module_compile
    compile_fn.restype = ctypes.c_int
    compile_fn.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    last_error = tfhip().tfhip_last_error
    last_error.restype = ctypes.c_char_p
    for k, kernel in enumerate(KERNELS):
        handle = ctypes.c_void_p()
        status = compile_fn(emit(kernel).encode(), b"kernel_0", b"", ctypes.byref(handle))
        assert status == 0, f"kernel {k} ({kernel['from']}): {last_error().decode()}"


STALE_CASES = {
    # an unnamed value that reads a modified variable may be written out at its use only if the variable cannot change on the way
    "set_between": ("""int index_0 = (block_id * 256) + block_thread_id0;
bool is_inside_dispatch = index_0 < var.N;
if (is_inside_dispatch)
{
  float x = asfloat(a_mem[index_0]);
  float vadd = x + 1.0f;
  x = 5.0f;
  out_mem[index_0] = asuint(vadd * x);
}""", r"float vadd(_\d+)? = x \+ 1\.0f;", True),
    "no_set_between": ("""int index_0 = (block_id * 256) + block_thread_id0;
bool is_inside_dispatch = index_0 < var.N;
if (is_inside_dispatch)
{
  float x = asfloat(a_mem[index_0]);
  x = 5.0f;
  float vadd = x + 1.0f;
  out_mem[index_0] = asuint(vadd * x);
}""", r"float vadd", False),
    "set_later_in_the_loop_that_holds_the_use": ("""int index_0 = (block_id * 256) + block_thread_id0;
bool is_inside_dispatch = index_0 < var.N;
if (is_inside_dispatch)
{
  float x = asfloat(a_mem[index_0]);
  float acc = 0.0f;
  float vmul = x * 2.0f;
  for (int i = 0; i < 4; i += 1)
  {
    acc = acc + vmul;
    x = x + 1.0f;
  }
  out_mem[index_0] = asuint(acc);
}""", r"float vmul(_\d+)? = x \* 2\.0f;", True),
    "value_and_use_inside_the_same_loop": ("""int index_0 = (block_id * 256) + block_thread_id0;
bool is_inside_dispatch = index_0 < var.N;
if (is_inside_dispatch)
{
  float x = asfloat(a_mem[index_0]);
  float acc = 0.0f;
  for (int i = 0; i < 4; i += 1)
  {
    float vmul = x * 2.0f;
    acc = acc + vmul;
    x = x + 1.0f;
  }
  out_mem[index_0] = asuint(acc);
}""", r"float vmul", False),
    "set_inside_a_branch_between": ("""int index_0 = (block_id * 256) + block_thread_id0;
bool is_inside_dispatch = index_0 < var.N;
if (is_inside_dispatch)
{
  float x = asfloat(a_mem[index_0]);
  float vadd = x + 1.0f;
  if (x > 0.0f)
  {
    x = 5.0f;
  }
  out_mem[index_0] = asuint(vadd * x);
}""", r"float vadd(_\d+)? = x \+ 1\.0f;", True),
}


@pytest.mark.parametrize("case", STALE_CASES)
def test_a_value_is_not_written_out_past_an_assignment_to_what_it_reads(emit, case):
    text, line, kept = STALE_CASES[case]
    body, _ = emitted_body(emit({"body": text.split("\n"), "group_size": [256, 1, 1], "shared": []}))
    emitted = "\n".join(l.strip() for l in body)
    assert (re.search(line, emitted) is not None) == kept, emitted
