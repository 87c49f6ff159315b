"""The shared library loads without a GPU and exports every function the C headers declare; the
Python binding lists exactly those functions; the package refuses to work without the library."""
import ctypes
import os
import re

import pytest

import lcu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = lcu.package()


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)   # comments mention function names too
    text = re.sub(r"//[^\n]*", "", text)
    return set(re.findall(r"\b(lcu_\w+)\s*\(", text))


def test_every_declared_function_is_exported():
    names = declared("llama_cu_hip.h") | declared("llama_cu_c.h")
    assert len(names) > 60
    dll = ctypes.CDLL(P.lib_path())
    missing = [n for n in sorted(names) if not hasattr(dll, n)]
    assert not missing, missing


def test_binding_lists_exactly_the_declared_functions():
    names = declared("llama_cu_hip.h") | declared("llama_cu_c.h")
    assert set(P.binding.SIGNATURES) == names


def test_reference_header_name_forwards():
    text = open(os.path.join(ROOT, "include", "llama_cu.h")).read()
    assert '#include "llama_cu_host.hpp"' in text


def test_last_error_is_a_string_before_any_call():
    assert isinstance(P.lib().lcu_last_error(), bytes)


def test_no_fallback_without_the_library(monkeypatch, tmp_path):
    monkeypatch.setattr(P.binding, "_lib", None)
    monkeypatch.setattr(P.binding, "_LIB_PATH", str(tmp_path / "libllama_cu_amd.so"))
    with pytest.raises(P.LcuError):
        P.lib()


def test_reference_public_surface_compiles_and_links(tmp_path):
    """A C++17 program that uses every public name of the reference's header with the reference's
    signatures builds against include/llama_cu.h and links against the library (g++, no HIP headers)."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = tmp_path / "public_surface"
    lib_dir = os.path.dirname(P.lib_path())
    cmd = ["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cxx", "public_surface.cpp"), "-L", lib_dir, "-lllama_cu_amd",
           "-Wl,-rpath," + lib_dir, "-Wl,--allow-shlib-undefined", "-o", str(exe)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    assert exe.exists()


def test_reference_main_program_compiles_against_the_kept_interface():
    """The reference's own main.cpp, read from the reference checkout where that exists (it is not
    copied here), is valid C++17 against include/llama_cu.h: same names, signatures and implicit
    conversions as the reference's llama_cu.h."""
    import shutil
    import subprocess
    src = "/root/reference/main.cpp"
    if shutil.which("g++") is None or not os.path.exists(src):
        pytest.skip("needs g++ and the reference checkout")
    with open(src, "rb") as f:
        res = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-x", "c++", "-I", os.path.join(ROOT, "include"), "-"],
                             stdin=f, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
