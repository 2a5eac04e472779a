"""ctypes binding of include/rg_hip.h.  There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
# RG_HIP_LIBRARY overrides the in-tree library (e.g. to compare builds)
LIB_PATH = os.environ.get("RG_HIP_LIBRARY") or os.path.join(PKG, "lib", "librg_hip.so")
HOST_LIB_PATH = os.path.join(PKG, "lib", "librg_host.so")
HOST_TESTS_PATH = os.path.join(PKG, "lib", "rg_host_tests")

# reference DataType codes (src/00common/include/common/data_type.h:19-36 of the reference)
F32, U8, I8, U16, I16, I32, I64, FP16, F64, BF16 = 1, 2, 3, 4, 5, 6, 7, 10, 11, 16
BOOL, U32, U64 = 9, 12, 13
MMI_A_ZP_SCALAR, MMI_B_ZP_SCALAR = 1, 2

_sz, _vp, _i, _u, _f = C.c_size_t, C.c_void_p, C.c_int, C.c_uint, C.c_float

# name -> (restype, argtypes); must list every symbol include/rg_hip.h declares
SIGNATURES = {
    "rg_hip_device_count": (_i, [C.POINTER(_i)]),
    "rg_hip_set_device": (_i, [_i]),
    "rg_hip_mem_info": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "rg_hip_device_name": (_i, [C.c_char_p, _sz]),
    "rg_hip_malloc": (_i, [C.POINTER(_vp), _sz]),
    "rg_hip_free": (_i, [_vp]),
    "rg_hip_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "rg_hip_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "rg_hip_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "rg_hip_memcpy_d2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "rg_hip_sync": (_i, []),
    "rg_hip_stream_create": (_i, [C.POINTER(_vp)]),
    "rg_hip_stream_destroy": (_i, [_vp]),
    "rg_hip_stream_sync": (_i, [_vp]),
    "rg_hip_graph_begin": (_i, [_vp]),
    "rg_hip_graph_end": (_i, [_vp, C.POINTER(_vp)]),
    "rg_hip_graph_launch": (_i, [_vp, _vp]),
    "rg_hip_graph_destroy": (_i, [_vp]),
    "rg_hip_error_string": (C.c_char_p, [_i]),
    "rg_hip_rms_norm": (_i, [_vp, _vp, _vp, _sz, _sz, _f, _i, _vp]),
    "rg_hip_rms_norm_quantize_workspace": (_sz, [_sz, _sz]),
    "rg_hip_rms_norm_quantize": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _f, _vp, _sz, _vp]),
    "rg_hip_softmax": (_i, [_vp, _vp, _sz, _sz, _sz, _i, _sz, _vp]),
    "rg_hip_rope": (_i, [_vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _f, _i, _vp]),
    "rg_hip_dequantize_linear": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _i, _vp]),
    "rg_hip_dynamic_quantize_linear_workspace": (_sz, [_sz]),
    "rg_hip_dynamic_quantize_linear": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp]),
    "rg_hip_cast": (_i, [_vp, _vp, _sz, _i, _i, _vp]),
    "rg_hip_transpose": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_matmul": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _f, _sz, _sz, _sz, _sz, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_matmul_workspace": (_sz, [_i, _i, _i, _sz, _sz, _sz, _sz]),
    "rg_hip_matmul_ws": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _f, _sz, _sz, _sz, _sz, _vp, _vp, _sz, _sz, _sz, _vp, _sz, _vp]),
    "rg_hip_split": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_concat": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_expand": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_where": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "rg_hip_matmul_integer_workspace": (_sz, [_sz, _sz, _sz, _sz, _u]),
    "rg_hip_matmul_integer": (_i, [_vp, _vp, _vp, _vp, _vp, _u, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp]),
    "rg_hip_matmul_integer_dequantize": (_i, [_vp, _vp, _vp, _vp, _vp, _u, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _i,
                                              _vp, _vp]),
    "rg_hip_attention_kvcache_workspace": (_sz, [_sz, _sz, _sz, _sz, _sz, _sz]),
    "rg_hip_attention_kvcache_state_bytes": (_sz, []),
    "rg_hip_attention_kvcache": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, _sz,
                                      _f, _i, _vp, _sz, _vp, _vp]),
    "rg_hip_attention_kvcache_static_scratch_bytes": (_sz, []),
    "rg_hip_attention_kvcache_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, _sz,
                                             _f, _i, _vp]),
}


class RgHipError(RuntimeError):
    pass


_lib = None


def lib() -> C.CDLL:
    """Loads librg_hip.so (built by ``python -m refactorgraph_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RgHipError(
                f"{LIB_PATH} is missing: build it with `python -m refactorgraph_amd.build` "
                "(there is no CPU or PyTorch fallback)")
        # PyTorch carries its own copy of the HIP runtime and owns the device memory this package is
        # handed: it has to be in the process first, so that the library binds to that same copy
        # (loaded the other way round, launches fail with "no ROCm-capable device").
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status: int, what: str = "rg_hip call"):
    if status != 0:
        msg = lib().rg_hip_error_string(status)
        raise RgHipError(f"{what} failed: {msg.decode() if msg else status} ({status})")
