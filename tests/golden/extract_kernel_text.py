"""Writes tests/golden/reference_kernel_text.json from kernel text that runs of the reference printed.

Four notebooks of the reference keep the output of `tf.get_all_generated_kernels()` (cell 1, stdout), i.e. the
kernels as its own code generator wrote them after all passes, in the GLSL dialect:
    examples/Algorithms/matrix_mul.ipynb        1 kernel   (hand-tiled matrix product: group memory, barriers)
    examples/Algorithms/fft_group.ipynb         1 kernel   (radix-2 FFT in group memory)
    examples/Rendering/buddhabrot.ipynb         4 kernels  (nested loops, break / continue, atomics, ternaries)
    examples/Simulation/fluid_simulation.ipynb 14 kernels  (stencils with clamped taps)
For every kernel this script keeps the thread-group declaration, the `shared` arrays and the statements of `main`
after the four lines that name block_id and block_thread_id0..2 (those belong to the target language, not to the
kernel's tree). The buffer declarations and helper functions printed above each `main` are boilerplate of the GLSL
generator and are left out.

Run here, where the reference tree is mounted (the notebooks are read as JSON text, nothing is imported or executed):
    python tests/golden/extract_kernel_text.py [/root/reference]
"""
import ast
import json
import re
import sys
from pathlib import Path

ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
NOTEBOOKS = [
    "examples/Algorithms/matrix_mul.ipynb",
    "examples/Algorithms/fft_group.ipynb",
    "examples/Rendering/buddhabrot.ipynb",
    "examples/Simulation/fluid_simulation.ipynb",
]
WRAPPER = ("int block_id =", "int block_thread_id0 =", "int block_thread_id1 =", "int block_thread_id2 =")

kernels = []
for rel in NOTEBOOKS:
    nb = json.loads((ref / rel).read_text())
    printed = "".join(nb["cells"][1]["outputs"][0]["text"])
    if "(('" in printed:
        # this notebook printed the kernel tuples themselves, one per line: take the string literals of each
        flat = []

        def strings(v):
            if isinstance(v, str):
                flat.append(v)
            elif isinstance(v, (tuple, list)):
                for x in v:
                    strings(x)

        for line in printed.split("\n"):
            if line.startswith("(("):
                strings(ast.literal_eval(line.strip())[0])
        printed = "\n".join(flat)
    for m in re.finditer(r"((?:shared \w+ \w+\[\d+\];\n)*)\n?layout \(local_size_x = (\d+), local_size_y = (\d+), local_size_z = (\d+)\) in;\n\nvoid main\(\) \{\n(.*?)\n\}\n", printed, flags=re.S):
        shared, gx, gy, gz, body = m.groups()
        lines = [l for l in body.split("\n") if l.strip() and not l.strip().startswith(WRAPPER)]
        kernels.append({
            "from": f"{rel}, cell 1, printed output of tf.get_all_generated_kernels(), kernel {sum(k['from'].startswith(rel) for k in kernels)}",
            "group_size": [int(gx), int(gy), int(gz)],
            "shared": [s for s in shared.split("\n") if s],
            "body": [l[2:] if l.startswith("  ") else l for l in lines],
        })

out = Path(__file__).with_name("reference_kernel_text.json")
out.write_text(json.dumps({"kernels": kernels}, indent=0) + "\n")
print(len(kernels), "kernels,", out.stat().st_size, "bytes")
for k in kernels:
    print(" ", k["from"], k["group_size"], len(k["body"]), "lines")
