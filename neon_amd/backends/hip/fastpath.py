"""Loader of the CPython extension that replays repeated statements in C
(neon_amd/csrc/fastpath.c, built into neon_amd/lib/_fastpath.so by the
repository's build step).  ``NEON_HIP_FASTPATH=0`` runs without it: the same
walk, lookup and launches then happen in Python."""
import importlib.machinery
import importlib.util
import os

# (NEON_HIP_FASTPATH_LIB names another build of the extension: the sanitizer test runs one)
_PATH = os.environ.get("NEON_HIP_FASTPATH_LIB") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "lib", "_fastpath.so")
_module = None


def enabled():
    return os.environ.get("NEON_HIP_FASTPATH", "1") != "0"


def load():
    """the extension module; ImportError (naming the build step) when it has not been built"""
    global _module
    if _module is None:
        if not os.path.exists(_PATH):
            raise ImportError("%s is missing: run `python -c \"import __graft_entry__ as g; g.build()\"` "
                              "(or set NEON_HIP_FASTPATH=0 to run without it)" % _PATH)
        loader = importlib.machinery.ExtensionFileLoader("_fastpath", _PATH)
        spec = importlib.util.spec_from_loader("_fastpath", loader)
        module = importlib.util.module_from_spec(spec)
        loader.exec_module(module)
        _module = module
    return _module
