"""Writes tests/golden/tiled_kernel_index_header.json from the kernel text that a run of the reference printed.

The reference keeps the output of `tf.get_all_generated_kernels()` for its tiled matrix product in
examples/Algorithms/matrix_mul.ipynb (cell 1, stdout): a 2-D kernel of shape [N/4, K/4] with 16x16 groups. The lines
of that printed kernel which turn `block_id` and the thread ids into `index_0`, `index_1` and the bounds test are the
index contract of every generated kernel (Compiler/Steps/GraphOps.cpp:1136-1186), as the reference itself computed
it. This script copies those lines, and the four that name the tile coordinates, into the fixture.

Run here, where the reference tree is mounted (it is read as JSON text, nothing is imported or executed):
    python tests/golden/extract_index_header.py [/root/reference]
"""
import json
import sys
from pathlib import Path

ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
nb = json.loads((ref / "examples/Algorithms/matrix_mul.ipynb").read_text())
printed = "".join(nb["cells"][1]["outputs"][0]["text"]).split("\n")
keep = []
for line in printed:
    s = line.strip()
    if s.startswith(("int vdiv", "int blocks_shape_", "int index_", "bool is_inside_dispatch", "int tx =", "int ty =", "int gx =", "int gy =")):
        keep.append(s)
    if s.startswith("int gy ="):
        break
group = next(line.strip() for line in printed if line.strip().startswith("layout (local_size_x"))
out = {
    "from": "examples/Algorithms/matrix_mul.ipynb, cell 1, printed output of tf.get_all_generated_kernels()",
    "kernel_shape": "[N / 4, K / 4], group_size [16, 16]",
    "group_declaration": group,
    "lines": keep,
}
Path(__file__).with_name("tiled_kernel_index_header.json").write_text(json.dumps(out, indent=1) + "\n")
print(json.dumps(out, indent=1))
