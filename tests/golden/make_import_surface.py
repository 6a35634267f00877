"""Writes tests/golden/import_surface.json: every name the reference's own modules, runners and
tests import from the modules this package mirrors (``from obkv_accel.<module> import ...`` and
``from obkv_fast import ...``), with the kind of the definition and, for functions, the parameter
names in order (for dataclasses, the field names).  The reference is read as text (``ast``),
nothing of it is imported or run.  Run here, where /root/reference exists:

    python tests/golden/make_import_surface.py
"""
import ast
import glob
import json
import os

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "import_surface.json")


def module_source(mod: str):
    for cand in (os.path.join(REF, *mod.split(".")) + ".py",):
        if os.path.exists(cand):
            return cand
    return None


def definition(tree: ast.Module, name: str):
    for node in tree.body:
        if isinstance(node, (ast.FunctionDef, ast.AsyncFunctionDef)) and node.name == name:
            a = node.args
            params = [x.arg for x in a.posonlyargs + a.args]
            kwonly = [x.arg for x in a.kwonlyargs]
            return {"kind": "function", "params": params, "kwonly": kwonly, "line": node.lineno}
        if isinstance(node, ast.ClassDef) and node.name == name:
            fields = [s.target.id for s in node.body if isinstance(s, ast.AnnAssign) and isinstance(s.target, ast.Name)]
            return {"kind": "class", "fields": fields, "line": node.lineno}
        if isinstance(node, (ast.Assign, ast.AnnAssign)):
            targets = node.targets if isinstance(node, ast.Assign) else [node.target]
            if any(isinstance(t, ast.Name) and t.id == name for t in targets):
                return {"kind": "value", "line": node.lineno}
        if isinstance(node, (ast.Try, ast.If)):        # names defined under try / if at module level
            sub = ast.Module(body=node.body + getattr(node, "orelse", []) +
                             [s for h in getattr(node, "handlers", []) for s in h.body], type_ignores=[])
            d = definition(sub, name)
            if d:
                return d
        if isinstance(node, ast.ImportFrom) and any((al.asname or al.name) == name for al in node.names):
            return {"kind": "reexport", "from": node.module, "line": node.lineno}
    return None


def main():
    files = sorted(glob.glob(os.path.join(REF, "*.py")) + glob.glob(os.path.join(REF, "obkv_accel", "*.py"))
                   + glob.glob(os.path.join(REF, "tests", "*.py")))
    surface = {}
    for path in files:
        try:
            tree = ast.parse(open(path).read())
        except SyntaxError:
            continue
        for node in ast.walk(tree):
            if not isinstance(node, ast.ImportFrom) or not node.module:
                continue
            if not (node.module.startswith("obkv_accel.") or node.module == "obkv_fast"):
                continue
            for al in node.names:
                entry = surface.setdefault(node.module, {}).setdefault(al.name, {"importers": []})
                where = f"{os.path.relpath(path, REF)}:{node.lineno}"
                if where not in entry["importers"]:
                    entry["importers"].append(where)
    for mod, names in surface.items():
        src = module_source(mod)
        tree = ast.parse(open(src).read()) if src else None
        for name, entry in names.items():
            entry["definition"] = definition(tree, name) if tree else None
    json.dump(surface, open(OUT, "w"), indent=1, sort_keys=True)
    print(f"wrote {OUT}: " + ", ".join(f"{m} ({len(n)})" for m, n in sorted(surface.items())))


if __name__ == "__main__":
    main()
