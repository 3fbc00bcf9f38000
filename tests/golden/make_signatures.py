"""Writes kernel_signatures.json: the parameter names of every public function defined in the
reference's cpm_kernels/kernels/*.py, read from the source text with ``ast`` (nothing of the
reference is imported or executed).  Run where the reference tree is present:

    python tests/golden/make_signatures.py /root/reference
"""
import ast
import glob
import json
import os
import sys


def main(ref_root: str):
    table = {}
    for path in sorted(glob.glob(os.path.join(ref_root, "cpm_kernels", "kernels", "*.py"))):
        if os.path.basename(path) in ("__init__.py", "base.py"):
            continue
        with open(path) as f:
            tree = ast.parse(f.read())
        for node in tree.body:
            if isinstance(node, ast.FunctionDef) and not node.name.startswith("_"):
                table[node.name] = [a.arg for a in node.args.args]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_signatures.json")
    with open(out, "w") as f:
        json.dump(table, f, indent=0, sort_keys=True)
    print("wrote %d signatures to %s" % (len(table), out))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
