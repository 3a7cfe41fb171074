#!/usr/bin/env python3
"""Extract the literal coordinate lists and call parameters held by the
reference's own tests into ``ref_cases.json``.

The reference test files are parsed as TEXT with ``ast`` (nothing from the
reference is imported or executed).  What is written is data only: voxel
coordinate lists plus the (shape, kernel, stride, padding, batch, channels,
subm) tuples the reference's tests call its checkers with.  The reference's
tests hold no stored outputs; expected outputs come from the oracle and from
torch's dense conv3d in this repository's tests.

Sources (relative to the reference root):
  test/test_rules.py   TestClass.*   (rule generation cases)
  test/test_conv.py    TestClass.*   (forward conv cases)
  test/test_stable.py  TestClass.*   (74-voxel stride-2 64->64 case)

Usage:  python tests/golden/extract_ref_cases.py [/root/reference]
"""
import ast
import json
import os
import sys

FILES = ["test/test_rules.py", "test/test_conv.py", "test/test_stable.py",
         "test/test_grad.py", "test/test_module.py"]


def _literal(node):
    try:
        return ast.literal_eval(node)
    except Exception:
        return None


def _tensor_literal(call):
    """torch.tensor([[...], ...], dtype=torch.int) -> list of rows, else None."""
    if not isinstance(call, ast.Call):
        return None
    # allow `.cuda()` / `.int()` suffixes
    while (isinstance(call, ast.Call) and isinstance(call.func, ast.Attribute)
           and call.func.attr in ("cuda", "int", "contiguous")):
        call = call.func.value
    if not (isinstance(call, ast.Call) and isinstance(call.func, ast.Attribute)
            and call.func.attr == "tensor" and call.args):
        return None
    val = _literal(call.args[0])
    if (isinstance(val, list) and val and isinstance(val[0], list)
            and all(isinstance(v, int) for row in val for v in row)):
        return val
    return None


def extract(path, rel):
    tree = ast.parse(open(path).read())
    cases = []
    for cls in [n for n in tree.body if isinstance(n, ast.ClassDef)]:
        for fn in [n for n in cls.body if isinstance(n, ast.FunctionDef)]:
            tensors = {}   # variable name -> coordinate list
            scalars = {}   # simple literal assignments (D = 6, kernel_size = [3,3,3] ...)
            for node in ast.walk(fn):
                if isinstance(node, ast.Assign) and len(node.targets) == 1 \
                        and isinstance(node.targets[0], ast.Name):
                    name = node.targets[0].id
                    t = _tensor_literal(node.value)
                    if t is not None:
                        tensors[name] = t
                    else:
                        lit = _literal(node.value)
                        if isinstance(lit, (int, bool, list)):
                            scalars[name] = lit
            calls = []
            for node in ast.walk(fn):
                if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) \
                        and node.func.id.startswith("assert_") and node.args \
                        and isinstance(node.args[0], ast.Name) \
                        and node.args[0].id in tensors:
                    kw = {}
                    ok = True
                    for k in node.keywords:
                        v = _literal(k.value)
                        if v is None and not isinstance(k.value, ast.Constant):
                            ok = False
                        kw[k.arg] = v
                    if ok:
                        calls.append({"line": node.lineno, "checker": node.func.id,
                                      "coords": node.args[0].id, "args": kw})
            calls.sort(key=lambda c: c["line"])
            if tensors:
                cases.append({"file": rel, "test": fn.name, "line": fn.lineno,
                              "tensors": tensors, "scalars": scalars, "calls": calls})
    return cases


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = []
    for rel in FILES:
        p = os.path.join(root, rel)
        if os.path.exists(p):
            out.extend(extract(p, rel))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_cases.json")
    with open(dst, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    ncalls = sum(len(c["calls"]) for c in out)
    print("wrote %s: %d test functions, %d checker calls" % (dst, len(out), ncalls))


if __name__ == "__main__":
    main()
