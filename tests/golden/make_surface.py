#!/usr/bin/env python3
"""
Writes tests/golden/core_surface.json and tests/golden/api_surface.json: the names a caller of the
reference can see - class -> method -> parameter names (and properties) - taken from the TEXT of the
reference's stub python/culsh/_culsh_core.pyi and of python/culsh/{rp_lsh,pstable_lsh,minhash_lsh,utils}.py
with `ast` (nothing of the reference is imported or run).  Run in the build container, where the reference
checkout is mounted; the JSON files are the fixtures, tests/test_surface.py compares this package with them.

    python tests/golden/make_surface.py [/root/reference]
"""

from __future__ import annotations

import ast
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def params(fn: ast.FunctionDef):
    a = fn.args
    names = [x.arg for x in a.posonlyargs + a.args]
    n_defaults = len(a.defaults)
    required = names[: len(names) - n_defaults] if n_defaults else list(names)
    kwonly = [x.arg for x in a.kwonlyargs]
    return {"params": [p for p in names if p not in ("self", "cls")], "kwonly": kwonly,
            "required": [p for p in required if p not in ("self", "cls")]}


def surface(path: str, public_only: bool = True):
    tree = ast.parse(open(path, encoding="utf-8").read())
    out = {"classes": {}, "functions": {}}
    for node in tree.body:
        if isinstance(node, ast.FunctionDef) and not (public_only and node.name.startswith("_")):
            out["functions"][node.name] = params(node)
        if isinstance(node, ast.ClassDef):
            methods, props, statics = {}, [], []
            for item in node.body:
                if not isinstance(item, ast.FunctionDef):
                    continue
                decos = {d.id if isinstance(d, ast.Name) else getattr(d, "attr", "") for d in item.decorator_list}
                if "property" in decos:
                    props.append(item.name)
                    continue
                if item.name.startswith("_") and item.name != "__init__":
                    continue
                methods[item.name] = params(item)
                if "staticmethod" in decos or "classmethod" in decos:
                    statics.append(item.name)
            out["classes"][node.name] = {"methods": methods, "properties": sorted(props), "static": sorted(statics)}
    return out


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    pkg = os.path.join(ref, "python", "culsh")
    core = surface(os.path.join(pkg, "_culsh_core.pyi"))
    with open(os.path.join(HERE, "core_surface.json"), "w") as f:
        json.dump({"source": "python/culsh/_culsh_core.pyi", **core}, f, indent=1, sort_keys=True)
    api = {}
    for mod in ("rp_lsh", "pstable_lsh", "minhash_lsh", "utils"):
        api[mod] = surface(os.path.join(pkg, mod + ".py"))
    init = ast.parse(open(os.path.join(pkg, "__init__.py"), encoding="utf-8").read())
    exported = []
    for node in init.body:
        if isinstance(node, ast.Assign) and any(getattr(t, "id", "") == "__all__" for t in node.targets):
            exported = [e.value for e in node.value.elts]
    with open(os.path.join(HERE, "api_surface.json"), "w") as f:
        json.dump({"source": "python/culsh/*.py", "__all__": exported, "modules": api}, f, indent=1, sort_keys=True)
    print("classes:", sorted(core["classes"]), "| exported:", exported)


if __name__ == "__main__":
    main()
