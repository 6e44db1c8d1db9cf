"""Records the row ORDER the reference's `build_codebook_abs` produces in this container.

The order is the one thing about the E8P table that nothing else pins: the reference sorts its 256
rows by squared norm with `argsort` (/root/reference/test_decode_matmul.py:84), which is not stable,
and up to 126 rows tie, so the index a row lands on depends on the torch build.  This script takes
the text of that one function (test_decode_matmul.py:73-86) out of the reference file (the module
itself cannot be imported: its line 5 imports the CUDA extension), runs it on the CPU and writes
what it returns, with the torch version, to reference_codebook_order.json.  Build container only:
it reads /root/reference, which does not exist where the GPU tests run; the tests read the JSON.

    python tests/golden/make_reference_codebook_order.py
"""
import ast
import json
import os
from itertools import product  # noqa: F401  (used by the reference's function)

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE_FILE = "/root/reference/test_decode_matmul.py"


def main():
    source = open(REFERENCE_FILE).read()
    tree = ast.parse(source)
    fn = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "build_codebook_abs")
    namespace = {"torch": torch, "product": product}
    exec(compile(ast.Module(body=[fn], type_ignores=[]), REFERENCE_FILE, "exec"), namespace)
    table = namespace["build_codebook_abs"]("cpu")
    assert table.dtype == torch.int64 and tuple(table.shape) == (256,)
    out = {
        "note": "int64[256] returned by the reference's build_codebook_abs('cpu') "
                "(test_decode_matmul.py:73-86) in the build container; the row order is specific to this torch build",
        "torch_version": torch.__version__,
        "reference_lines": [fn.lineno, fn.end_lineno],
        "codebook_abs_int64": [int(v) for v in table],
    }
    with open(os.path.join(HERE, "reference_codebook_order.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote reference_codebook_order.json, torch", torch.__version__)


if __name__ == "__main__":
    main()
