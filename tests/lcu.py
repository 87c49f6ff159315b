"""Loads the llama.cu_amd package (its directory name has a dot, so by path) for the tests."""
import importlib.util
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_PKG = os.path.join(_ROOT, "llama.cu_amd")


def package():
    if "llama_cu_amd" not in sys.modules:
        spec = importlib.util.spec_from_file_location("llama_cu_amd", os.path.join(_PKG, "__init__.py"),
                                                      submodule_search_locations=[_PKG])
        mod = importlib.util.module_from_spec(spec)
        sys.modules["llama_cu_amd"] = mod
        spec.loader.exec_module(mod)
    return sys.modules["llama_cu_amd"]
