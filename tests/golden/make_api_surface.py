"""Writes tests/golden/api_surface.json: the names a backend has to supply to
plug into the reference -- the methods ``abstract_backend.py`` declares
abstract, the further methods of ``backend.py``'s ``Backend`` that its two real
backends override or that layers call, and the methods and properties of its
``Tensor`` class.  The reference's files are READ as text (parsed with ``ast``,
nothing is imported or run); only names and line numbers are kept.

    python tests/golden/make_api_surface.py [/root/reference]
"""
import ast
import json
import os
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def classes(path):
    with open(os.path.join(REF, path)) as f:
        tree = ast.parse(f.read())
    return dict((n.name, n) for n in tree.body if isinstance(n, ast.ClassDef))


def methods(cls):
    out = []
    for n in cls.body:
        if isinstance(n, ast.FunctionDef):
            decos = [d.attr if isinstance(d, ast.Attribute) else getattr(d, "id", "") for d in n.decorator_list]
            out.append({"name": n.name, "line": n.lineno, "abstract": "abstractmethod" in decos,
                        "property": "property" in decos})
    return out


abc = classes("neon/backends/abstract_backend.py")["AbstractBackend"]
api = classes("neon/backends/backend.py")
surface = {
    "source": {"abstract": "neon/backends/abstract_backend.py:40-1428 (class AbstractBackend)",
               "backend": "neon/backends/backend.py:437-1680 (class Backend)",
               "tensor": "neon/backends/backend.py:45-435 (class Tensor)"},
    "abstract_methods": sorted(m["name"] for m in methods(abc) if m["abstract"]),
    "backend_methods": sorted(m["name"] for m in methods(api["Backend"]) if not m["name"].startswith("_")),
    "tensor_methods": sorted(m["name"] for m in methods(api["Tensor"])
                             if not (m["name"].startswith("_") and not m["name"].startswith("__"))),
    "tensor_abstract": sorted(m["name"] for m in methods(api["Tensor"])
                              if any(isinstance(s, ast.Raise) for s in ast.walk(ast.Module(body=[
                                  c for c in api["Tensor"].body if isinstance(c, ast.FunctionDef) and c.name == m["name"]],
                                  type_ignores=[])))),
}
with open(os.path.join(HERE, "api_surface.json"), "w") as f:
    json.dump(surface, f, indent=1, sort_keys=True)
print("%d abstract backend methods, %d Backend methods, %d Tensor methods (%d of them raise in the base)" % (
    len(surface["abstract_methods"]), len(surface["backend_methods"]), len(surface["tensor_methods"]),
    len(surface["tensor_abstract"])))
