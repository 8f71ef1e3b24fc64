"""Extracts the golden index-map vectors the reference's own tests hold.

Reads the reference's test files AS TEXT (nothing is imported or executed),
finds the literal arrays passed to ``np.array(...)`` / ``torch.tensor(...)`` and
writes them to JSON next to this script:

* ``eval_vectors.json``      <- tests/test_eval.py:12-198
* ``unsqueeze_vectors.json`` <- tests/test_unsqueeze.py:17-58
* ``debugging_vectors.json`` <- tests/test_debugging.py:41-239

Usage (only where the reference checkout exists):
    python tests/golden/extract_reference_vectors.py /root/reference
"""

import ast
import json
import pathlib
import sys


def literal_arrays(path):
    tree = ast.parse(pathlib.Path(path).read_text())
    arrays = []
    for node in ast.walk(tree):
        if not isinstance(node, ast.Call) or not isinstance(node.func, ast.Attribute):
            continue
        owner = node.func.value
        if not isinstance(owner, ast.Name) or (owner.id, node.func.attr) not in (("np", "array"), ("torch", "tensor")):
            continue
        if not node.args:
            continue
        try:
            value = ast.literal_eval(node.args[0])
        except ValueError:
            continue
        arrays.append((node.lineno, value))
    arrays.sort(key=lambda item: item[0])
    return arrays


def main(reference_root):
    root = pathlib.Path(reference_root)
    here = pathlib.Path(__file__).resolve().parent
    for source, target in (
        ("tests/test_eval.py", "eval_vectors.json"),
        ("tests/test_unsqueeze.py", "unsqueeze_vectors.json"),
        ("tests/test_debugging.py", "debugging_vectors.json"),
    ):
        arrays = literal_arrays(root / source)
        payload = {"source": source, "arrays": [{"line": line, "value": value} for line, value in arrays]}
        (here / target).write_text(json.dumps(payload) + "\n")
        print(target, len(arrays), "arrays")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
