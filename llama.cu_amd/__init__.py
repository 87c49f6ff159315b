"""MI355X (gfx950) implementation of the eiz/llama.cu inference path.

The product is the shared library libllama_cu_amd.so: hand-written HIP kernels behind the C ABI of
include/llama_cu_hip.h, and a C++17 host layer with the reference's llama_cu.h interface
(include/llama_cu_host.hpp, C handles in include/llama_cu_c.h).  This package is the thin ctypes
binding the tests and bench.py use; there is no CPU fallback -- without the built library or
without a GPU every call fails.

The directory name contains a dot, so import it by path:
    spec = importlib.util.spec_from_file_location("llama_cu_amd", ".../llama.cu_amd/__init__.py",
                                                  submodule_search_locations=[".../llama.cu_amd"])
"""
from .binding import (BatchContext, DeviceBuffer, LcuError, Model, Context, Vocabulary, check, from_device, lib, lib_path, to_device)  # noqa: F401
