"""MI355X (gfx950) kernel backend for RefactorGraph's LLM-operator hot path.

The product is the C ABI in include/rg_hip.h (refactorgraph_amd/lib/librg_hip.so) and the C++
host layer that mirrors the reference's kernel plugin surface (librg_host.so).  This Python
package is the thin driver used by tests and benchmarks: it binds the C ABI with ctypes and
passes raw device pointers of torch tensors; torch is only the device allocator here.
"""
from . import abi  # noqa: F401
from .abi import lib, RgHipError  # noqa: F401
